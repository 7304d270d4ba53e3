"""Build libxllm_mi355.so (HIP kernels + C ABI) for gfx950, in tree.

Run as `python -m xllm_amd.build`.  hipcc cross-compiles without a GPU.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libxllm_mi355.so")
SOURCES = ["reshape_and_cache.hip", "rope_and_cache.hip", "paged_decode_gqa.hip", "paged_decode_mla.hip", "absorbed_bmm.hip",
           "merge_and_tables.hip", "profile.hip", "hbm_probe.hip", "c_abi.hip"]
HEADERS = ["common.cuh", "launch.h", os.path.join("..", "..", "include", "xllm_mi355.h")]
# Packed-fp32 VALU forms stay off: every float op is a plain single-lane instruction.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=True, verbose=True, extra_flags=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    hdrs = [os.path.join(CSRC, h) for h in HEADERS]
    objs, jobs = [], []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(CSRC, s.replace(".hip", ".o"))
        objs.append(obj)
        if force or _stale(obj, [src] + hdrs):
            jobs.append([hipcc, *FLAGS, *extra_flags, "-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print("+", " ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)

    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(run, jobs))
    if jobs or not os.path.exists(LIB):
        run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


SHIM_LIB = os.path.join(HERE, "libxllm_mi355_torch.so")


def build_shim(force=True, verbose=True):
    """The C++ host side (torch::Tensor interface + torch op registration) over the C ABI."""
    src = os.path.join(CSRC, "shim", "ops_api.cpp")
    deps = [src, os.path.join(CSRC, "shim", "ops_api.h"), os.path.join(HERE, "..", "include", "xllm_mi355.h")]
    if not force and not _stale(SHIM_LIB, deps):
        return SHIM_LIB
    import torch
    from torch.utils import cpp_extension
    incs = []
    for p in cpp_extension.include_paths(device_type="cuda"):
        incs += ["-isystem", p]
    incs += ["-isystem", "/opt/rocm/include"]
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", *incs, "-o", SHIM_LIB, src,
           f"-L{HERE}", "-lxllm_mi355", "-Wl,-rpath,$ORIGIN", f"-L{libdir}", f"-Wl,-rpath,{libdir}",
           "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip"]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return SHIM_LIB


if __name__ == "__main__":
    build(force="--if-stale" not in sys.argv)
    build_shim(force="--if-stale" not in sys.argv)
