"""Chooses which binding of libnumml_hip.so the Python layer calls.

Two bindings export the reference module's functions (cpp/sparse_csr.cpp:307-319):

* ``compiled``: numml_amd/lib/numml_torch_cpp<ext>.so, the pybind11 torch
  extension built from csrc/torch_binding.cpp; importable as ``numml_torch_cpp``
  exactly like the reference's extension.
* ``ctypes``: numml_amd/numml_torch_cpp.py, the same functions written in Python
  over ctypes (needs nothing but the C-ABI library).

Both end in the same kernels and give identical results.  ``NUMML_AMD_BINDING``
selects one (``compiled`` | ``ctypes``); unset, the compiled extension is used
when it has been built and the ctypes mirror otherwise.  Neither has a CPU path.
"""
import glob
import importlib.util
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_compiled = None


def compiled_path():
    """Path of the built torch extension, or None when it has not been built."""
    hits = sorted(glob.glob(os.path.join(_HERE, "lib", "numml_torch_cpp*.so")))
    return hits[0] if hits else None


def load_compiled():
    """Import numml_amd/lib/numml_torch_cpp<ext>.so; raises if it is not there."""
    global _compiled
    if _compiled is None:
        path = compiled_path()
        if path is None:
            raise ImportError(
                "numml_amd: the compiled numml_torch_cpp extension has not been built "
                "(run `python -m numml_amd.build`)")
        import torch  # noqa: F401  (libtorch must be loaded before the extension)
        spec = importlib.util.spec_from_file_location("numml_torch_cpp", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _compiled = mod
    return _compiled


def _select():
    want = os.environ.get("NUMML_AMD_BINDING", "").strip().lower()
    if want not in ("", "compiled", "ctypes"):
        raise ImportError(f"NUMML_AMD_BINDING must be 'compiled' or 'ctypes', got {want!r}")
    if want == "ctypes" or (want == "" and compiled_path() is None):
        from . import numml_torch_cpp as mirror
        return mirror, "ctypes"
    return load_compiled(), "compiled"


ops, name = _select()


def backward_mode():
    """'planned', 'eager' or 'atomic': how the selected binding computes SpMV/SpMM gradients."""
    return ops.backward_mode() if name == "compiled" else ops.BACKWARD_MODE


def set_backward_mode(mode):
    """Switch the selected binding's SpMV/SpMM backward: 'planned' (transposed-structure plan from
    the second sighting of a pattern on), 'eager' (from the first) or 'atomic' (stateless)."""
    if mode not in ("planned", "eager", "atomic"):
        raise ValueError(f"backward mode must be 'planned', 'eager' or 'atomic', got {mode!r}")
    if name == "compiled":
        ops.set_backward_mode(mode)
    else:
        ops.BACKWARD_MODE = mode


def install(module_name="numml_torch_cpp"):
    """Register the compiled extension under the reference's module name.

    After this, ``import numml_torch_cpp`` (numml/sparse/_csr.py:2,
    numml/sparse/linalg.py:2) resolves to this backend, so the reference's own
    Python layer runs on it unchanged.
    """
    mod = load_compiled()
    sys.modules[module_name] = mod
    return mod
