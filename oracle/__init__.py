"""ctypes bindings of the two CPU oracles.  TEST INFRASTRUCTURE: only tests, the smoke
run and the benchmark's CPU-baseline leg may import this package.

All functions take contiguous torch CPU tensors and return new CPU tensors.
"""
import ctypes
import os

import torch

from . import build as _build

_HERE = os.path.dirname(os.path.abspath(__file__))

BF16, FP16, FP32, FP8_E4M3 = 0, 1, 2, 3
_DT = {torch.bfloat16: BF16, torch.float16: FP16, torch.float32: FP32,
       torch.float8_e4m3fn: FP8_E4M3, torch.uint8: FP8_E4M3}

_c = None
_aten = None

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int
_f32 = ctypes.c_float
_f64 = ctypes.c_double


def dtype_code(t):
    return _DT[t.dtype]


def c_lib():
    """The plain-C oracle, built on first use if missing or older than its source."""
    global _c
    if _c is None:
        path = _build.build_c(force=False)
        lib = ctypes.CDLL(path)
        lib.oracle_bf16_to_f32.restype = _f32
        lib.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.oracle_f32_to_bf16.argtypes = [_f32]
        lib.oracle_fp16_to_f32.restype = _f32
        lib.oracle_fp16_to_f32.argtypes = [ctypes.c_uint16]
        lib.oracle_f32_to_fp16.restype = ctypes.c_uint16
        lib.oracle_f32_to_fp16.argtypes = [_f32]
        lib.oracle_e4m3fn_to_f32.restype = _f32
        lib.oracle_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        lib.oracle_f32_to_e4m3fn.restype = ctypes.c_uint8
        lib.oracle_f32_to_e4m3fn.argtypes = [_f32]
        lib.oracle_fp8_quantize.restype = ctypes.c_uint8
        lib.oracle_fp8_quantize.argtypes = [_f32, _f32]
        lib.oracle_reshape_and_cache.restype = _i32
        lib.oracle_reshape_and_cache.argtypes = [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64,
                                                 _i64, _i64, _i64, _i32, _i32]
        lib.oracle_kv_head_scales.restype = None
        lib.oracle_kv_head_scales.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _i32]
        lib.oracle_paged_decode_f64.restype = _i32
        lib.oracle_paged_decode_f64.argtypes = [_p, _p, _p, _p, _p, _p, _i64, _p, _p, _p, _i64, _i64,
                                                _i64, _i64, _i64, _i64, _f64, _i32, _i32, _i32]
        lib.oracle_lse_merge.restype = None
        lib.oracle_lse_merge.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _i64]
        lib.oracle_lse_combine.restype = None
        lib.oracle_lse_combine.argtypes = [_p, _p, _p, _p, _p, _p, _i64, _i64]
        lib.oracle_build_block_table.restype = None
        lib.oracle_build_block_table.argtypes = [_p, _p, _p, _p, _i64, _p, _i64, _i64]
        lib.oracle_mask_block_table_padding.restype = None
        lib.oracle_mask_block_table_padding.argtypes = [_p, _i64, _p, _p, _i64, _i64, _i64]
        lib.oracle_gather_paged_rows.restype = None
        lib.oracle_gather_paged_rows.argtypes = [_p, _p, _i64, _p, _p, _i64, _i64, _i64, _i64]
        _c = lib
    return _c


def aten_lib():
    """The ATen-op-order oracle, built on first use if missing (a minute of compilation: a stale one is
    rebuilt by the build step, not inside a test)."""
    global _aten
    if _aten is None:
        path = _build.ATEN_LIB
        if not os.path.exists(path):
            _build.build_aten()
        lib = ctypes.CDLL(path)
        lib.aten_oracle_num_threads.restype = _i32
        lib.aten_oracle_set_num_threads.argtypes = [_i32]
        lib.aten_paged_decode.restype = _i32
        lib.aten_paged_decode.argtypes = [_p, _p, _p, _p, _p, _i64, _p, _p, _p, _i64, _i64, _i64, _i64,
                                          _i64, _i64, _i64, _f32, _i32, _i32]
        lib.aten_paged_decode_csr.restype = _i32
        lib.aten_paged_decode_csr.argtypes = [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64,
                                              _i64, _i32]
        lib.aten_paged_decode_lse.restype = _i32
        lib.aten_paged_decode_lse.argtypes = [_p, _p, _p, _p, _i64, _p, _p, _i64, _i64, _i64, _i64,
                                              _i64, _i64, _f32, _i32, _i32]
        lib.aten_lse_merge.restype = _i32
        lib.aten_lse_merge.argtypes = [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i32]
        lib.aten_fp8_quantize.restype = _i32
        lib.aten_fp8_quantize.argtypes = [_p, _p, _p, _i64, _i64, _i64, _i32]
        _aten = lib
    return _aten


def _ptr(t):
    if t is None:
        return None
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle wants contiguous CPU tensors"
    return t.data_ptr()


# ------------------------------------------------------------------------------ op 1

def reshape_and_cache(key, value, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None):
    """In place on k_cache / v_cache (CPU).  key/value [T,Hkv,D] may be strided in dim 0."""
    T, Hkv, D = key.shape
    P, bs = k_cache.shape[0], k_cache.shape[1]
    assert key.stride(2) == 1 and key.stride(1) == D
    assert slot_mapping.dtype == torch.int32
    if value is not None:
        assert value.stride(2) == 1 and value.stride(1) == D
    rc = c_lib().oracle_reshape_and_cache(
        key.data_ptr(), None if value is None else value.data_ptr(), _ptr(k_cache), _ptr(v_cache),
        _ptr(slot_mapping), _ptr(k_scale), _ptr(v_scale), T, Hkv, D, bs, P,
        key.stride(0), 0 if value is None else value.stride(0), dtype_code(key), dtype_code(k_cache))
    if rc != 0:
        raise ValueError("oracle_reshape_and_cache: unsupported dtype pair")


def kv_head_scales(x):
    T, Hkv, D = x.shape
    out = torch.empty(Hkv, dtype=torch.float32)
    assert x.stride(2) == 1 and x.stride(1) == D
    c_lib().oracle_kv_head_scales(x.data_ptr(), _ptr(out), T, Hkv, D, x.stride(0), dtype_code(x))
    return out


def fp8_encode(x_f32):
    """Plain cast fp32 -> e4m3fn codes (uint8), element by element."""
    lib = c_lib()
    flat = x_f32.reshape(-1).tolist()
    return torch.tensor([lib.oracle_f32_to_e4m3fn(v) for v in flat], dtype=torch.uint8).reshape(x_f32.shape)


def fp8_decode_table():
    lib = c_lib()
    return torch.tensor([lib.oracle_e4m3fn_to_f32(c) for c in range(256)], dtype=torch.float32)


# ------------------------------------------------------------------------------ op 2

def paged_decode_f64(q, k_cache, v_cache, block_table, seq_lens, sm_scale, k_scale=None,
                     v_scale=None, dv=None, round_dequant=True):
    """Exact-arithmetic attention.  Returns (out fp32 [B,Hq,dv], lse fp32 [B,Hq])."""
    B, Hq, Dqk = q.shape
    bs, Hkv = k_cache.shape[1], k_cache.shape[2]
    if dv is None:
        dv = Dqk if v_cache is None else v_cache.shape[3]
    out = torch.empty(B, Hq, dv, dtype=torch.float32)
    lse = torch.empty(B, Hq, dtype=torch.float32)
    rc = c_lib().oracle_paged_decode_f64(
        _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(lse), _ptr(block_table),
        block_table.stride(0), _ptr(seq_lens), _ptr(k_scale), _ptr(v_scale), B, Hq, Hkv, Dqk, dv, bs,
        float(sm_scale), dtype_code(q), dtype_code(k_cache), int(round_dequant))
    if rc != 0:
        raise ValueError("oracle_paged_decode_f64 failed")
    return out, lse


def aten_paged_decode(q, k_cache, v_cache, block_table, seq_lens, sm_scale, k_scale=None,
                      v_scale=None, dv=None):
    """The reference's libtorch block-table decode.  Returns out [B,Hq,dv] in q.dtype."""
    B, Hq, Dqk = q.shape
    P, bs, Hkv = k_cache.shape[0], k_cache.shape[1], k_cache.shape[2]
    if dv is None:
        dv = Dqk if v_cache is None else v_cache.shape[3]
    out = torch.empty(B, Hq, dv, dtype=q.dtype)
    rc = aten_lib().aten_paged_decode(
        _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(block_table), block_table.stride(0),
        _ptr(seq_lens), _ptr(k_scale), _ptr(v_scale), B, Hq, Hkv, Dqk, dv, bs, P, float(sm_scale),
        dtype_code(q), dtype_code(k_cache))
    if rc != 0:
        raise ValueError("aten_paged_decode: seq_len must be positive")
    return out


def aten_paged_forward(q, k_cache, v_cache, block_table, kv_seq_lens, q_cu_seq_lens, sm_scale, causal=True):
    """Short query chunks against paged KV (layers/dcu/flash_attention.cpp:447-545, decode branch): packed
    q [T,Hq,D]; token j of the q_len tokens of sequence b attends to the first kv_len - q_len + j + 1
    tokens (causal: the chunk is the tail of the context, the bottom-right alignment that the call site's
    window arguments select) or to all kv_len.  Restated with the libtorch decode above, one query token
    at a time; tokens that attend to nothing give zeros.  The fast path itself is a closed library:
    parity with it is unpinned, the semantics are pinned against dense masked attention in the tests."""
    T = q.shape[0]
    B = kv_seq_lens.numel()
    lens = torch.zeros(T, dtype=torch.int32)
    rows = torch.zeros(T, dtype=torch.int64)
    for b in range(B):
        q0, q1 = int(q_cu_seq_lens[b]), int(q_cu_seq_lens[b + 1])
        kv = int(kv_seq_lens[b])
        for t in range(q0, q1):
            L = kv - (q1 - q0) + (t - q0) + 1 if causal else kv
            lens[t] = max(0, min(L, kv))
            rows[t] = b
    out = torch.zeros_like(q)
    live = (lens > 0).nonzero().flatten()
    if live.numel() > 0:
        out[live] = aten_paged_decode(q[live].contiguous(), k_cache, v_cache, block_table[rows[live]].contiguous(),
                                      lens[live].contiguous(), sm_scale)
    return out


def aten_paged_decode_csr(q, k_cache, v_cache, indptr, indices, last_page_len):
    B, Hq, D = q.shape
    P, bs, Hkv = k_cache.shape[0], k_cache.shape[1], k_cache.shape[2]
    out = torch.empty_like(q)
    rc = aten_lib().aten_paged_decode_csr(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(indptr),
                                          _ptr(indices), _ptr(last_page_len), B, Hq, Hkv, D, bs, P,
                                          dtype_code(q))
    if rc != 0:
        raise ValueError("aten_paged_decode_csr: empty sequence")
    return out


def aten_paged_decode_lse(q, k_cache, block_table, seq_lens, sm_scale, k_scale=None):
    B, Hq, Dqk = q.shape
    P, bs, Hkv = k_cache.shape[0], k_cache.shape[1], k_cache.shape[2]
    lse = torch.empty(B, Hq, dtype=torch.float32)
    rc = aten_lib().aten_paged_decode_lse(_ptr(q), _ptr(k_cache), _ptr(lse), _ptr(block_table),
                                          block_table.stride(0), _ptr(seq_lens), _ptr(k_scale), B, Hq,
                                          Hkv, Dqk, bs, P, float(sm_scale), dtype_code(q),
                                          dtype_code(k_cache))
    if rc != 0:
        raise ValueError("aten_paged_decode_lse failed")
    return lse


# ------------------------------------------------------------------------------ merge

def lse_merge(partial_out_f32, partial_lse):
    """C oracle.  partial_out [S,B,H,Dv] fp32, partial_lse [S,B,H] fp32."""
    S, B, H, Dv = partial_out_f32.shape
    out = torch.empty(B, H, Dv, dtype=torch.float32)
    lse = torch.empty(B, H, dtype=torch.float32)
    c_lib().oracle_lse_merge(_ptr(partial_out_f32), _ptr(partial_lse), _ptr(out), _ptr(lse), S, B, H, Dv)
    return out, lse


def lse_combine(shared_o, shared_lse, unshared_o, unshared_lse):
    """C oracle of the two-way base-2 combine.  shared_o / unshared_o [B, H, D] (any float type; computed in fp32),
    the LSEs [B, H, 1] fp32 in base 2.  Returns (out fp32 [B, H, D], merged base-2 LSE [B, H, 1])."""
    B, H, D = shared_o.shape
    so, uo = shared_o.float().contiguous(), unshared_o.float().contiguous()
    sl, ul = shared_lse.float().contiguous(), unshared_lse.float().contiguous()
    out = torch.empty(B, H, D, dtype=torch.float32)
    merged = torch.empty(B, H, 1, dtype=torch.float32)
    c_lib().oracle_lse_combine(_ptr(out), _ptr(merged), _ptr(so), _ptr(sl), _ptr(uo), _ptr(ul), B * H, D)
    return out, merged


def aten_lse_merge(partial_out, partial_lse):
    S, B, H, Dv = partial_out.shape
    out = torch.empty(B, H, Dv, dtype=partial_out.dtype)
    lse = torch.empty(B, H, dtype=torch.float32)
    aten_lib().aten_lse_merge(_ptr(partial_out), _ptr(partial_lse), _ptr(out), _ptr(lse), S, B, H, Dv,
                              dtype_code(partial_out))
    return out, lse


def aten_fp8_quantize(x, scale):
    T, Hkv, D = x.shape
    out = torch.empty(T, Hkv, D, dtype=torch.uint8)
    aten_lib().aten_fp8_quantize(_ptr(x), _ptr(out), _ptr(scale), T, Hkv, D, dtype_code(x))
    return out


def build_block_table(indptr, indices, last_page_len, table_stride, block_size):
    B = indptr.numel() - 1
    table = torch.empty(B, table_stride, dtype=torch.int32)
    seq_lens = torch.empty(B, dtype=torch.int32)
    c_lib().oracle_build_block_table(_ptr(indptr), _ptr(indices), _ptr(last_page_len), _ptr(table),
                                     table_stride, _ptr(seq_lens), B, block_size)
    return table, seq_lens


def mask_block_table_padding(block_table, kv_seq_lens, block_size):
    B, W = block_table.shape
    out = torch.empty(B, W, dtype=torch.int32)
    assert block_table.device.type == "cpu" and block_table.dtype == torch.int32 and block_table.stride(1) == 1
    c_lib().oracle_mask_block_table_padding(ctypes.c_void_p(block_table.data_ptr()), block_table.stride(0),
                                            _ptr(kv_seq_lens), _ptr(out), B, W, block_size)
    return out


def fused_qk_norm_rope(qkv, n_q, n_k, n_v, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleave,
                       position_ids):
    """Restatement of fused_qknorm_rope_kernel (xllm/core/kernels/cuda/fused_qknorm_rope.cu:79-300): fp32 between
    one load and one store -- x * rsqrt(mean(x^2) + eps) * weight, then the rotation of the leading rotary_dim dims
    by the cos | sin row of the token's position, rounded once.  Returns a new tensor.  Pinned in
    tests/test_oracle_attention.py by rotations with known answers, norm preservation, and the torch reference of
    the reference's own test (tests/core/kernels/dcu/fused_qknorm_rope_test.cpp:27-118) within its tolerance."""
    T = qkv.shape[0]
    rotary_dim = cos_sin_cache.shape[1]
    half = rotary_dim // 2
    out = qkv.clone()
    x = qkv[:, : (n_q + n_k) * head_dim].float().view(T, n_q + n_k, head_dim)
    if q_weight is not None:
        w = torch.cat([q_weight.float().view(1, 1, -1).expand(1, n_q, -1), k_weight.float().view(1, 1, -1).expand(1, n_k, -1)], 1)
        x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w
    cs = cos_sin_cache.float()[position_ids.long()]
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    rot = x[..., :rotary_dim]
    if interleave:
        e, o = rot[..., 0::2], rot[..., 1::2]
        new = torch.stack([e * cos - o * sin, e * sin + o * cos], -1).flatten(-2)
    else:
        a, b = rot[..., :half], rot[..., half:]
        new = torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
    y = torch.cat([new, x[..., rotary_dim:]], -1)
    out[:, : (n_q + n_k) * head_dim] = y.reshape(T, -1).to(qkv.dtype)
    return out


def llm_decode_metadata_update(src, dst, actual_num_tokens, padded_num_tokens, actual_batch_size,
                               actual_indices_size):
    """Restatement of llm_decode_metadata_update_kernel, rule by rule and index by index
    (xllm/core/kernels/cuda/llm_decode_metadata_update.cu:27-71).  `src` / `dst`: dicts of int32 tensors named as
    in LlmDecodeMetadataUpdateParams without the prefix; dst is modified in place.  Pinned in
    tests/test_oracle_reshape.py against the slice copies and fills of the executor's slow path
    (xllm/core/runtime/cuda_graph_executor_impl.cpp:397-453), which the kernel replaces."""
    n = max(actual_num_tokens, padded_num_tokens + 1, actual_batch_size + 1, actual_indices_size)
    for i in range(n):
        if i < actual_num_tokens:
            dst["tokens"][i] = src["tokens"][i]
            dst["positions"][i] = src["positions"][i]
            dst["new_cache_slots"][i] = src["new_cache_slots"][i]
        if actual_num_tokens <= i < padded_num_tokens:
            dst["tokens"][i] = 0
            dst["positions"][i] = 0
            dst["new_cache_slots"][i] = -1
        if i < actual_batch_size + 1:
            dst["kv_seq_lens"][i] = src["kv_seq_lens"][i]
            dst["paged_kv_indptr"][i] = src["paged_kv_indptr"][i]
        if actual_batch_size + 1 <= i < padded_num_tokens + 1:
            dst["kv_seq_lens"][i] = src["kv_seq_lens"][actual_batch_size]
            dst["paged_kv_indptr"][i] = src["paged_kv_indptr"][actual_batch_size]
        if i < actual_batch_size:
            dst["kv_seq_lens_delta"][i] = src["kv_seq_lens"][i + 1] - src["kv_seq_lens"][i]
            dst["paged_kv_last_page_len"][i] = src["paged_kv_last_page_len"][i]
        if actual_batch_size <= i < padded_num_tokens:
            dst["kv_seq_lens_delta"][i] = 0
            dst["paged_kv_last_page_len"][i] = 1
        if i < actual_indices_size:
            dst["paged_kv_indices"][i] = src["paged_kv_indices"][i]
    return dst


def gather_paged_rows(cache, block_table, cu_seq_lens, total_rows, fill=0):
    """cache [P, bs, 1, D] -> [total_rows, D]; untouched rows keep `fill`."""
    P, bs, D = cache.shape[0], cache.shape[1], cache.shape[-1]
    out = torch.full((total_rows, D), fill, dtype=cache.dtype)
    c_lib().oracle_gather_paged_rows(_ptr(cache), _ptr(block_table), block_table.stride(0), _ptr(cu_seq_lens),
                                     _ptr(out), block_table.shape[0], bs, P, D * cache.element_size())
    return out


def absorbed_bmm(x, w):
    """x [T, H, K], w [H, K, N] -> [T, H, N] the way the reference writes it
    (layers/dcu/deepseek_v2_attention.cpp:428-430, 231-238): bmm over the head-major views, here in fp32 with
    one rounding to the input dtype at the end.  Also returns the unrounded fp32 result."""
    exact = torch.bmm(x.float().transpose(0, 1), w.float()).transpose(0, 1).contiguous()
    return exact.to(x.dtype), exact
