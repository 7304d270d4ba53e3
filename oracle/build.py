"""Build the two CPU oracles (test infrastructure) next to their sources.

  libpaged_kv_oracle.so  plain C (gcc), no dependencies
  libaten_oracle.so      C++ against the libtorch that ships with the installed PyTorch

Run as `python oracle/build.py`.  The reference's own files for this path cannot be
compiled without glog/gflags and vendor libraries, so there is no `_ref` build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
C_LIB = os.path.join(HERE, "libpaged_kv_oracle.so")
ATEN_LIB = os.path.join(HERE, "libaten_oracle.so")


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_c(force=True):
    src = os.path.join(HERE, "paged_kv_oracle.c")
    if not force and os.path.exists(C_LIB) and os.path.getmtime(C_LIB) >= os.path.getmtime(src):
        return C_LIB
    _run(["gcc", "-O2", "-std=c11", "-Wall", "-Wextra", "-fPIC", "-shared",
          "-ffp-contract=off", "-o", C_LIB, src, "-lm"])
    return C_LIB


def build_aten(force=True):
    src = os.path.join(HERE, "aten_oracle.cpp")
    if not force and os.path.exists(ATEN_LIB) and os.path.getmtime(ATEN_LIB) >= os.path.getmtime(src):
        return ATEN_LIB
    import torch
    from torch.utils import cpp_extension
    incs = []
    for p in cpp_extension.include_paths():
        incs += ["-isystem", p]
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
          *incs, "-o", ATEN_LIB, src, f"-L{libdir}", f"-Wl,-rpath,{libdir}",
          "-ltorch", "-ltorch_cpu", "-lc10"])
    return ATEN_LIB


def build_all(force=True):
    return build_c(force), build_aten(force)


if __name__ == "__main__":
    build_all(force="--if-stale" not in sys.argv)
