"""ctypes binding of libxllm_mi355.so -- the same C ABI a C++/cgo/JNI caller would bind.

There is no fallback: if the library is missing, or a call returns non-zero, this module
raises.  Building is `python -m xllm_amd.build`.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# XLLM_MI355_LIBRARY names another build of the same library (A/B measurements of kernel variants)
LIB_PATH = os.environ.get("XLLM_MI355_LIBRARY") or os.path.join(_HERE, "libxllm_mi355.so")

BF16, FP16, FP32, FP8_E4M3 = 0, 1, 2, 3

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int
_f32 = ctypes.c_float
_sz = ctypes.c_size_t

# name -> (restype, argtypes); one entry per declaration in include/xllm_mi355.h
SIGNATURES = {
    "xllm_mi355_error_string": (ctypes.c_char_p, [_i32]),
    "xllm_mi355_version": (ctypes.c_char_p, []),
    "xllm_mi355_reshape_and_cache": (_i32, [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64,
                                            _i64, _i64, _i32, _i32, _p]),
    "xllm_mi355_kv_head_scales": (_i32, [_p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "xllm_mi355_paged_decode_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "xllm_mi355_paged_decode_gqa_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "xllm_mi355_paged_decode_mla_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "xllm_mi355_paged_decode_gqa": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _p, _p, _p, _i64, _i64, _i64,
                                           _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _p, _sz, _i32,
                                           _i32, _p]),
    "xllm_mi355_paged_decode_gqa_static": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _p, _p, _p, _i64, _i64, _i64,
                                                  _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i32, _i32, _p]),
    "xllm_mi355_decode_workspace_bound": (_sz, []),
    "xllm_mi355_decode_workspace_init": (_i32, [_p, _sz, _p]),
    "xllm_mi355_decode_status": (_i32, [_p, _p]),
    "xllm_mi355_debug_set": (_i32, [_i32, _i32]),
    "xllm_mi355_paged_decode_gqa_csr": (_i32, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64,
                                               _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _p, _sz, _i32,
                                               _i32, _p]),
    "xllm_mi355_paged_decode_plan_bytes": (_sz, []),
    "xllm_mi355_paged_decode_gqa_plan": (_i32, [_p, _sz, _p, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64,
                                                _i64, _i32, _p]),
    "xllm_mi355_paged_decode_gqa_planned": (_i32, [_p, _sz, _p, _p, _p, _p, _p, _p, _i64, _p, _p, _p, _p, _p, _p,
                                                   _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                                   _f32, _p, _sz, _i32, _i32, _p]),
    "xllm_mi355_write_and_decode_gqa": (_i32, [_p, _p, _p, _i64, _i64, _p, _sz, _p, _p, _p, _p, _p, _p, _i64, _p, _p,
                                               _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                               _i64, _f32, _p, _sz, _i32, _i32, _p]),
    "xllm_mi355_gather_paged_rows": (_i32, [_p, _p, _i64, _p, _p, _i64, _i64, _i64, _i64, _i64, _p]),
    "xllm_mi355_paged_decode_varlen_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "xllm_mi355_paged_decode_gqa_varlen": (_i32, [_p, _p, _p, _p, _p, _p, _p, _i64, _p, _p, _i64, _i64, _i64, _i64,
                                                  _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i32, _p,
                                                  _sz, _i32, _i32, _p]),
    "xllm_mi355_paged_decode_mla": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64,
                                           _i64, _i64, _i64, _f32, _p, _sz, _i32, _p]),
    "xllm_mi355_paged_decode_mla_plan": (_i32, [_p, _sz, _p, _i64, _p, _i64, _i64, _i64, _p]),
    "xllm_mi355_paged_decode_mla_planned": (_i32, [_p, _sz, _p, _p, _p, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64,
                                                   _i64, _i64, _i64, _f32, _p, _sz, _i32, _p]),
    "xllm_mi355_write_and_decode_mla": (_i32, [_p, _p, _i64, _p, _sz, _p, _p, _p, _p, _p, _p, _i64, _p, _i64, _i64, _i64,
                                               _i64, _i64, _i64, _i64, _f32, _p, _sz, _i32, _p]),
    "xllm_mi355_lse_merge": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "xllm_mi355_lse_combine": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i32, _i32, _p]),
    "xllm_mi355_build_block_table": (_i32, [_p, _p, _p, _p, _i64, _p, _i64, _i64, _p]),
    "xllm_mi355_decode_metadata_update": (_i32, [_p] * 15 + [_i64] * 4 + [_p]),
    "xllm_mi355_mask_block_table_padding": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "xllm_mi355_mla_absorbed_bmm": (_i32, [_p] * 3 + [_i64] * 8 + [_i32, _p]),
    "xllm_mi355_rope_and_cache": (_i32, [_p] * 10 + [_i64] * 7 + [_f32, _i32, _i64, _i64, _i32, _i32, _i32, _p]),
    "xllm_mi355_profile_enable": (_i32, [_i32]),
    "xllm_mi355_profile_collect": (_i32, [_p, _i32]),
    "xllm_mi355_stream_read": (_i32, [_p, _sz, _p, _p]),
    "xllm_mi355_stream_copy": (_i32, [_p, _p, _sz, _p]),
}

_lib = None


class XllmMi355Error(RuntimeError):
    pass


def lib():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise XllmMi355Error(
                f"{LIB_PATH} is missing: build it with `python -m xllm_amd.build` "
                "(there is no CPU or PyTorch fallback for this path)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(rc, what):
    if rc != 0:
        msg = lib().xllm_mi355_error_string(rc).decode()
        raise XllmMi355Error(f"{what} failed with code {rc}: {msg}")
