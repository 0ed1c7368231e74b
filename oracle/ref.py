"""Loader for oracle/_ref: the reference's own CPU sources compiled in place.

TEST INFRASTRUCTURE ONLY.  ``load()`` returns the compiled extension module
(its functions take torch CPU tensors, cpp/sparse_csr.cpp:307-319) or ``None``
when it has not been built; ``call(name, *args)`` converts NumPy arguments to
tensors and results back.  The build recipe is oracle/Makefile (target
``ref``); it needs the reference tree and is therefore only run where that
tree exists.
"""
import glob
import importlib.util
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_mod = None


def load():
    global _mod
    if _mod is not None:
        return _mod
    hits = sorted(glob.glob(os.path.join(_HERE, "_ref", "numml_ref_cpu*.so")))
    if not hits:
        return None
    import torch  # noqa: F401  (libtorch must be loaded before the extension)
    spec = importlib.util.spec_from_file_location("numml_ref_cpu", hits[0])
    mod = importlib.util.module_from_spec(spec)
    try:
        spec.loader.exec_module(mod)
    except ImportError:
        return None
    _mod = mod
    return _mod


def built():
    """True when the compiled reference is present; looks at the file system only (does
    not load the library, so test collection stays free of it)."""
    return bool(glob.glob(os.path.join(_HERE, "_ref", "numml_ref_cpu*.so")))


def available():
    return load() is not None


def call(name, *args):
    """Call the reference build's ``<name>`` with NumPy arrays; returns NumPy array(s)."""
    import torch
    mod = load()
    if mod is None:
        raise RuntimeError("oracle/_ref is not built")
    targs = [torch.from_numpy(np.ascontiguousarray(a)) if isinstance(a, np.ndarray) else a
             for a in args]
    out = getattr(mod, name)(*targs)
    if isinstance(out, (list, tuple)):
        return tuple(o.numpy() for o in out)
    return out.numpy()
