"""Builds libmamba_gfx950.so (the C-ABI library of hand-written HIP kernels) in-tree with hipcc.

Usage: python -m mamba_amd.build [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmamba_gfx950.so")
ARCH = "gfx950"

# Packed-fp32 VALU instructions are switched off for every kernel of this library.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _deps():
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    hdrs.append(os.path.join(os.path.dirname(HERE), "include", "mamba_hip.h"))
    return hdrs


def _compile(src, force):
    obj = src[:-4] + ".o"
    newest = max(os.path.getmtime(p) for p in [src] + _deps())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    if r.stderr.strip():
        sys.stderr.write(r.stderr)
    return obj


EXT = os.path.join(HERE, "_torch_ext.so")
EXT_SRC = os.path.join(CSRC, "torch_ext.cpp")


def build_torch_ext(force=False):
    """Compiles csrc/torch_ext.cpp (host code only: the decode-step operators' argument handling on
    at::Tensor) into the Python extension module mamba_amd/_torch_ext.so, linked against the kernel
    library beside it.  Needs the library to exist."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    newest = max(os.path.getmtime(p) for p in (EXT_SRC, os.path.join(os.path.dirname(HERE), "include", "mamba_hip.h")))
    if not force and os.path.exists(EXT) and os.path.getmtime(EXT) >= newest:
        return EXT
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = [os.path.join(os.path.dirname(HERE), "include"), *cpp_extension.include_paths(), sysconfig.get_paths()["include"],
           "/opt/rocm/include"]
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_torch_ext",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{d}" for d in inc], EXT_SRC, "-o", EXT,
           f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python",
           f"-L{HERE}", "-l:libmamba_gfx950.so", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the torch extension failed:\n{r.stdout}\n{r.stderr}")
    return EXT


def build(force=False, jobs=None):
    """Compiles every .hip under csrc/ for gfx950, links the shared library, then builds the torch
    extension module on top of it."""
    lib = build_lib(force, jobs)
    build_torch_ext(force)
    return lib


def build_lib(force=False, jobs=None):
    """Compiles every .hip under csrc/ for gfx950 and links the shared library."""
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
