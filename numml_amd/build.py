"""Builds the native parts in-tree.

    python -m numml_amd.build          # both of the below

* libnumml_hip.so: every csrc/*.hip compiled with hipcc for gfx950 and linked
  (the C ABI of include/numml_hip.h).  hipcc cross-compiles, so this runs on
  machines without a GPU.
* numml_torch_cpp<ext>.so: csrc/torch_binding.cpp, the pybind11 torch extension
  that exports the reference module's hot-path functions on top of the C ABI
  (host-only C++, compiled with g++ against the installed torch).

Objects and libraries land in numml_amd/lib/.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libnumml_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -ffp-contract=off: a*b+c is rounded twice, like the reference's CPU build
#   (x86-64 -O2 has no FMA), so that serial-order sums reproduce it bit for bit.
# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32.
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
] + os.environ.get("NM_EXTRA_HIPCC_FLAGS", "").split()


def _compile(src):
    obj = os.path.join(LIBDIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


def build_extension(verbose=True):
    """Compile csrc/torch_binding.cpp into numml_amd/lib/numml_torch_cpp<ext>.so."""
    import sysconfig

    import torch
    tdir = os.path.dirname(torch.__file__)
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(LIBDIR, "numml_torch_cpp" + ext)
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-w", "-fvisibility=hidden",
        "-Wl,-Bsymbolic",
        "-DTORCH_EXTENSION_NAME=numml_torch_cpp", "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        f"-I{os.path.join(tdir, 'include')}", f"-I{os.path.join(tdir, 'include', 'torch', 'csrc', 'api', 'include')}",
        f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include", f"-I{os.path.join(ROOT, 'include')}",
        os.path.join(CSRC, "torch_binding.cpp"), "-o", out,
        f"-L{os.path.join(tdir, 'lib')}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip",
        "-ltorch_python", f"-L{LIBDIR}", "-lnumml_hip",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{os.path.join(tdir, 'lib')}",
    ]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the torch extension failed:\n{r.stderr[-4000:]}")
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build()
    build_extension()
