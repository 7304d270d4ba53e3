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


# mla_decode_w4_kernel keeps its 256 accumulators under fixed register names (a0 .. a255) that only inline assembly
# touches; the statements' clobber lists make the compiler count them but do not reserve them between statements.  The
# kernel is sound as long as the compiler has no reason to put values of its own there: all 256 accumulation registers
# in use by the kernel, nothing spilled, no scratch memory.  The build checks exactly that from the compiler's own
# resource report and, if it ever fails (another compiler, other flags, a change that raises register pressure),
# compiles the file again with the eight-wavefront kernel (XLLM_MI355_MLA_KERNEL=narrow) as the default for more than
# 64 heads, and says so.
GUARDED_SOURCE = "paged_decode_mla.hip"
GUARDED_KERNEL = "mla_decode_w4_kernel"
GUARD_FLAG = "-Rpass-analysis=kernel-resource-usage"
FALLBACK_DEFINE = "-DXLLM_MLA_DEFAULT_NARROW=1"


def resource_report(text, kernel):
    """{field: value} per instantiation of `kernel` from the remarks of -Rpass-analysis=kernel-resource-usage."""
    import re
    reports, cur = [], None
    for line in text.splitlines():
        m = re.search(r"remark:\s+Function Name:\s+(\S+)", line)
        if m:
            cur = {} if kernel in m.group(1) else None
            if cur is not None:
                reports.append(cur)
            continue
        m = re.search(r"remark:\s+([A-Za-z][A-Za-z /\[\]]*?):\s+(\S+)\s+\[-Rpass-analysis", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = m.group(2)
    return reports


def accumulators_untouched(reports):
    """The condition under which the fixed-name accumulators of mla_decode_w4_kernel are safe (see above)."""
    if not reports:
        return False, "the compiler reported no instantiation of the kernel"
    for r in reports:
        if r.get("AGPRs") != "256":
            return False, f"AGPRs = {r.get('AGPRs')} (must be 256)"
        if r.get("VGPRs Spill") != "0":
            return False, f"VGPRs Spill = {r.get('VGPRs Spill')} (must be 0)"
        if r.get("ScratchSize [bytes/lane]") != "0":
            return False, f"ScratchSize = {r.get('ScratchSize [bytes/lane]')} (must be 0)"
        if r.get("Dynamic Stack") != "False":
            return False, "dynamic stack"
    return True, "ok"


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
        if os.path.basename(cmd[-3]) != GUARDED_SOURCE:
            subprocess.run(cmd, check=True)
            return
        res = subprocess.run([*cmd, GUARD_FLAG], check=True, stderr=subprocess.PIPE, text=True)
        ok, why = accumulators_untouched(resource_report(res.stderr, GUARDED_KERNEL))
        if verbose:
            sys.stderr.write("".join(l + "\n" for l in res.stderr.splitlines() if "remark:" not in l
                                     and not l.lstrip().startswith(("|", "^")) and "__launch_bounds__" not in l))
        if ok:
            print(f"build: {GUARDED_KERNEL}: 256 accumulation registers, no spill, no scratch", flush=True)
            return
        print(f"build: WARNING: {GUARDED_KERNEL} fails its register check ({why}); compiling {GUARDED_SOURCE} again with "
              f"the eight-wavefront MLA kernel as the default", file=sys.stderr, flush=True)
        subprocess.run([*cmd, FALLBACK_DEFINE], check=True)

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
