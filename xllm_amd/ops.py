"""Host-side mirror of the reference's kernel op interface for the paged-KV decode path,
over the C ABI.  torch is used for device memory and the current stream only.

Reference interface mirrored here (paths relative to the xLLM source tree):
  ReshapePagedCacheParams / reshape_paged_cache   xllm/core/kernels/param.h:126-161, ops_api.h:31
  quant_to_paged_cache                            xllm/core/kernels/ops_api.cpp:296-310
  batch_decode (block table + seq_lens)           xllm/core/kernels/npu/npu_ops_api.h:46,
                                                  xllm/core/kernels/mlu/mlu_ops_api.h:127
  batch_decode (CSR)                              xllm/core/kernels/cuda/cuda_ops_api.h:128-144
  flash_mla::DenseDecodeParams / dense_decode     xllm/core/kernels/dcu/flash_mla_adapter.h:40-53
  merge_dcp_attention_shards                      xllm/core/layers/mlu/dcp_attention_merge.h:28-34
  build_block_table_from_paged_kv                 xllm/core/kernels/dcu/build_block_table_from_paged_kv.hip
  mask_block_table_padding                        xllm/core/layers/dcu/flash_attention.cpp:194-218
  fused_qk_norm_rope                              xllm/core/kernels/cuda/fused_qknorm_rope.cu:388-470
  LlmDecodeMetadataUpdateParams, update_llm_decode_metadata
                                                  xllm/core/kernels/cuda/llm_decode_metadata_update.h:33-56
  gather_mla_latent_cache                         xllm/core/kernels/dcu/dcu_ops_api.h:74
  absorbed MLA products (bmm with w_kc_ / w_vc_)  xllm/core/layers/dcu/deepseek_v2_attention.cpp:231-238,428-430
  FlashAttentionImpl::paged_forward (q chunks)    xllm/core/layers/dcu/flash_attention.cpp:447-545

Errors: the reference CHECK-aborts; here every violated precondition raises.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from . import capi

_DT = {torch.bfloat16: capi.BF16, torch.float16: capi.FP16, torch.float32: capi.FP32,
       torch.float8_e4m3fn: capi.FP8_E4M3, torch.uint8: capi.FP8_E4M3}


def _dtype_code(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}") from None


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _check_plan(plan):
    """The planned decode reads the plan up to its last word: refuse anything but the whole buffer."""
    need = capi.lib().xllm_mi355_paged_decode_plan_bytes()
    if plan.dtype != torch.uint8 or not plan.is_contiguous() or plan.numel() < need:
        raise ValueError(f"plan must be the contiguous uint8 buffer of update_decode_plan ({need} bytes)")


def _require_cuda(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("this path runs on the GPU only: every tensor must be a device tensor")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError("all tensors must live on the same device")
    return dev


# ------------------------------------------------------------------------------------------
# workspace: one per device, allocated once and never replaced (a launch recorded in a HIP graph keeps the
# address it was captured with), same lifetime as the reference's FlashinferWorkspace singleton
# (xllm/core/layers/cuda/flashinfer_workspace.cpp:25-41).  It serves one stream at a time: decode calls on two
# streams of one device must not overlap.

_workspaces = {}


def reserve_decode_workspace(device, nbytes=0):
    """Allocate the device's decode workspace (at least the library's bound over every supported shape, or
    nbytes if that is more).  Call it before the first decode of a process that needs more than the bound;
    a second call that would have to grow the workspace raises."""
    device = torch.device(device)
    lib = capi.lib()
    want = max(int(nbytes), int(lib.xllm_mi355_decode_workspace_bound()))
    ws = _workspaces.get(device)
    if ws is not None:
        if ws.numel() < nbytes:
            raise RuntimeError(
                f"the decode workspace of {device} holds {ws.numel()} bytes and {nbytes} are needed: it cannot grow "
                "once handed out (captured graphs hold its address); reserve_decode_workspace(device, nbytes) "
                "before the first decode call")
        return ws
    with torch.cuda.device(device):
        ws = torch.empty(want, dtype=torch.uint8, device=device)
        capi.check(lib.xllm_mi355_decode_workspace_init(ws.data_ptr(), ws.numel(), _stream(device)),
                   "xllm_mi355_decode_workspace_init")
    _workspaces[device] = ws
    return ws


def decode_workspace(device, nbytes):
    return reserve_decode_workspace(device, nbytes)


def decode_status(device):
    """0, or raises if a bounded wait inside a decode kernel gave up since the last call (the outputs of that
    launch are invalid).  Synchronises the current stream: not for use under graph capture."""
    ws = _workspaces.get(torch.device(device))
    if ws is None:
        return 0
    capi.check(capi.lib().xllm_mi355_decode_status(ws.data_ptr(), _stream(torch.device(device))),
               "xllm_mi355_decode_status")
    return 0


# ------------------------------------------------------------------------------------------
# op 1

@dataclass
class ReshapePagedCacheParams:
    """Field for field the reference struct (xllm/core/kernels/param.h:126-161).  For the fp8
    cache of this build k_cache_scale / v_cache_scale are per-KV-head [Hkv] fp32."""
    key: torch.Tensor
    k_cache: torch.Tensor
    slot_mapping: torch.Tensor
    value: Optional[torch.Tensor] = None
    v_cache: Optional[torch.Tensor] = None
    direction: bool = False
    k_cache_scale: Optional[torch.Tensor] = None
    v_cache_scale: Optional[torch.Tensor] = None


def _reshape(params, quantized):
    key, value = params.key, params.value
    k_cache, v_cache = params.k_cache, params.v_cache
    slots = params.slot_mapping
    dev = _require_cuda(key, value, k_cache, v_cache, slots, params.k_cache_scale, params.v_cache_scale)
    if params.direction:
        raise NotImplementedError("CACHE2CONTEXT is MLU-only in the reference and not part of this path")
    if key.dim() != 3 or k_cache.dim() != 4:
        raise ValueError("key must be [T, Hkv, D] and k_cache [P, bs, Hkv, D]")
    if (value is None) != (v_cache is None):
        raise ValueError("value and v_cache must be given together")
    T, Hkv, D = key.shape
    if not (key.stride(-1) == 1 and key.stride(-2) == D):
        raise ValueError("key: last two dims must be contiguous")
    if value is not None and not (value.stride(-1) == 1 and value.stride(-2) == D and value.shape == key.shape):
        raise ValueError("value: last two dims must be contiguous and the shape must match key")
    if not k_cache.is_contiguous() or (v_cache is not None and not v_cache.is_contiguous()):
        raise ValueError("caches must be contiguous")
    if tuple(k_cache.shape[2:]) != (Hkv, D):
        raise ValueError("k_cache heads / head_dim do not match key")
    if slots.dtype != torch.int32 or not slots.is_contiguous() or slots.numel() != T:
        raise ValueError("slot_mapping must be contiguous int32 [T]")
    if quantized:
        if params.k_cache_scale is None:
            raise ValueError("k_cache_scale is required for quant_to_paged_cache")
        for s in (params.k_cache_scale, params.v_cache_scale):
            if s is not None and (s.dtype != torch.float32 or s.numel() != Hkv or not s.is_contiguous()):
                raise ValueError("cache scales must be contiguous fp32 [Hkv]")
    elif k_cache.dtype != key.dtype:
        raise ValueError("key and k_cache must have the same dtype (use quant_to_paged_cache for fp8)")
    P, bs = k_cache.shape[0], k_cache.shape[1]
    rc = capi.lib().xllm_mi355_reshape_and_cache(
        key.data_ptr(), _ptr(value), k_cache.data_ptr(), _ptr(v_cache), slots.data_ptr(),
        _ptr(params.k_cache_scale) if quantized else None,
        _ptr(params.v_cache_scale) if quantized else None,
        T, Hkv, D, bs, P, key.stride(0), 0 if value is None else value.stride(0),
        _dtype_code(key), _dtype_code(k_cache), _stream(dev))
    capi.check(rc, "xllm_mi355_reshape_and_cache")


def reshape_paged_cache(params: ReshapePagedCacheParams):
    """xllm::kernel::reshape_paged_cache (ops_api.cpp:248-278): scales are ignored, dtypes equal."""
    _reshape(params, quantized=False)


def quant_to_paged_cache(params: ReshapePagedCacheParams):
    """xllm::kernel::quant_to_paged_cache (ops_api.cpp:296-310), fp8 e4m3fn with per-head scales."""
    _reshape(params, quantized=True)


def kv_head_scales(x):
    """scale[h] = max(absmax(x[:, h, :]) / 448, 1e-12) (fp8_scaled_quantize.cpp:38-42, per KV head)."""
    dev = _require_cuda(x)
    T, Hkv, D = x.shape
    if not (x.stride(-1) == 1 and x.stride(-2) == D):
        raise ValueError("x: last two dims must be contiguous")
    out = torch.empty(Hkv, dtype=torch.float32, device=dev)
    rc = capi.lib().xllm_mi355_kv_head_scales(x.data_ptr(), out.data_ptr(), T, Hkv, D, x.stride(0),
                                              _dtype_code(x), _stream(dev))
    capi.check(rc, "xllm_mi355_kv_head_scales")
    return out


# ------------------------------------------------------------------------------------------
# op 2

def _decode_common(query, k_cache, output, v_cache=None, k_scale=None, v_scale=None):
    if query.dim() != 3:
        raise ValueError("query must be [B, Hq, D]")
    if not (query.stride(-1) == 1 and query.stride(-2) == query.shape[-1]):
        raise ValueError("query: last two dims must be contiguous")
    if output.shape != query.shape or output.dtype != query.dtype:
        raise ValueError("output must have query's shape and dtype")
    if not (output.stride(-1) == 1 and output.stride(-2) == output.shape[-1]):
        raise ValueError("output: last two dims must be contiguous")
    if not k_cache.is_contiguous() or k_cache.dim() != 4:
        raise ValueError("k_cache must be contiguous [P, bs, Hkv, D]")
    if k_cache.shape[3] != query.shape[2] or query.shape[1] % k_cache.shape[2] != 0:
        raise ValueError("cache head_dim / KV heads do not match query")
    if v_cache is not None and (v_cache.shape != k_cache.shape or v_cache.dtype != k_cache.dtype
                                or not v_cache.is_contiguous()):
        raise ValueError("v_cache must match k_cache in shape and dtype, contiguous")
    if _dtype_code(k_cache) == capi.FP8_E4M3:
        for s in (k_scale, v_scale):
            if s is None or s.dtype != torch.float32 or s.numel() != k_cache.shape[2] or not s.is_contiguous():
                raise ValueError("an fp8 cache needs contiguous fp32 scales [Hkv] for K and V")
    elif k_cache.dtype != query.dtype:
        raise TypeError("the cache dtype must equal the query dtype (or be fp8)")


def update_decode_plan_info(num_qo_heads, num_kv_heads, head_dim, block_size, cache_dtype, block_table=None,
                            seq_lens=None, paged_kv_indptr=None, paged_kv_indices=None, paged_kv_last_page_len=None,
                            window_left=-1, plan=None):
    """The plan of a decode step, made once and handed to the decode calls of all layers (plan=...): the role of
    update_decode_plan_info, which the reference runs at layer 0 only (layers/cuda/flashinfer_planinfo.cpp:248-264).
    Takes the step's block table and lengths, or its CSR arrays; cache_dtype is the dtype of the KV cache.
    Returns the plan (a device buffer; pass one back in to reuse it, as a captured step must)."""
    csr = paged_kv_indptr is not None
    dev = _require_cuda(block_table, seq_lens, paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len, plan)
    lib = capi.lib()
    nbytes = int(lib.xllm_mi355_paged_decode_plan_bytes())
    if plan is None:
        plan = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    if plan.dtype != torch.uint8 or plan.numel() < nbytes or not plan.is_contiguous():
        raise ValueError(f"plan must be a contiguous uint8 buffer of {nbytes} bytes")
    if csr:
        B = paged_kv_indptr.numel() - 1
        for t, n in ((paged_kv_indptr, B + 1), (paged_kv_last_page_len, B)):
            if t.dtype != torch.int32 or t.numel() != n or not t.is_contiguous():
                raise ValueError("CSR arrays must be contiguous int32 of the documented sizes")
        if paged_kv_indices.dtype != torch.int32 or not paged_kv_indices.is_contiguous():
            raise ValueError("paged_kv_indices must be contiguous int32")
        table, stride, lens = None, 0, None
    else:
        B = seq_lens.numel()
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
            raise ValueError("block_table must be int32 [B, W] with unit column stride")
        if seq_lens.dtype != torch.int32 or not seq_lens.is_contiguous() or block_table.shape[0] != B:
            raise ValueError("seq_lens must be contiguous int32 [B], one per block_table row")
        table, stride, lens = block_table, block_table.stride(0), seq_lens
    code = capi.FP8_E4M3 if cache_dtype == torch.float8_e4m3fn else (capi.FP16 if cache_dtype == torch.float16 else capi.BF16)
    rc = lib.xllm_mi355_paged_decode_gqa_plan(
        plan.data_ptr(), plan.numel(), _ptr(table), stride, _ptr(lens), _ptr(paged_kv_indptr), _ptr(paged_kv_indices),
        _ptr(paged_kv_last_page_len), B, num_qo_heads, num_kv_heads, head_dim, block_size, int(window_left), code,
        _stream(dev))
    capi.check(rc, "xllm_mi355_paged_decode_gqa_plan")
    return plan


def batch_decode(query, k_cache, output, block_table, seq_lens, v_cache=None, output_lse=None,
                 k_cache_quant_scale=None, v_cache_quant_scale=None, scale=None, return_lse=False,
                 max_seq_len=0, window_left=-1, plan=None, new_key=None, new_value=None, slot_mapping=None):
    """Block-table paged decode.  Argument order and meaning follow mlu::batch_decode
    (mlu_ops_api.h:127) restricted to what npu::batch_decode (npu_ops_api.h:46) also has.
    query/output [B, Hq, D]; caches [P, bs, Hkv, D]; block_table [B, W] int32; seq_lens [B] int32.
    window_left >= 0: sliding window, the query attends to the last window_left + 1 tokens of its context
    (sliding_window_ of layers/dcu/flash_attention.cpp:484).
    plan: the step's plan from update_decode_plan_info (same tables, lengths, heads and window), or None.
    new_key / new_value [B, Hkv, D] with slot_mapping [B] int32: the step's K / V rows, stored into the caches by the
    same call before it attends (the reshape_paged_cache + batch_decode pair of an attention layer's decode step,
    layers/dcu/torch_attention.cpp:138-144 and :285-347, in one call; same cache bytes and output as the pair).
    Returns (output, lse or None) with lse [B, Hq, 1] fp32 natural log."""
    if v_cache is None:
        raise ValueError("GQA decode needs v_cache; the latent-KV variant is dense_decode")
    dev = _require_cuda(query, k_cache, v_cache, output, block_table, seq_lens, output_lse,
                        k_cache_quant_scale, v_cache_quant_scale, plan, new_key, new_value, slot_mapping)
    _decode_common(query, k_cache, output, v_cache, k_cache_quant_scale, v_cache_quant_scale)
    B, Hq, D = query.shape
    P, bs, Hkv, _ = k_cache.shape
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise ValueError("block_table must be int32 [B, W] with unit column stride")
    if seq_lens.dtype != torch.int32 or seq_lens.numel() != B or not seq_lens.is_contiguous():
        raise ValueError("seq_lens must be contiguous int32 [B]")
    if block_table.shape[0] != B:
        raise ValueError("block_table rows must equal the batch")
    if scale is None:
        scale = D ** -0.5
    lse = None
    if return_lse or output_lse is not None:
        lse = output_lse if output_lse is not None else torch.empty(B, Hq, 1, dtype=torch.float32, device=dev)
        if lse.dtype != torch.float32 or lse.numel() != B * Hq or not lse.is_contiguous():
            raise ValueError("output_lse must be contiguous fp32 [B, Hq, 1]")
    if max_seq_len <= 0:
        max_seq_len = block_table.shape[1] * bs
    lib = capi.lib()
    nbytes = lib.xllm_mi355_paged_decode_gqa_workspace_bytes(B, Hq, D)
    ws = decode_workspace(dev, nbytes)
    if plan is not None:
        _check_plan(plan)
    if new_key is not None or new_value is not None or slot_mapping is not None:
        if new_key is None or new_value is None or slot_mapping is None:
            raise ValueError("new_key, new_value and slot_mapping come together")
        for t in (new_key, new_value):
            if t.dtype != query.dtype or t.dim() != 3 or tuple(t.shape) != (B, Hkv, D) or t.stride(2) != 1 or \
                    t.stride(1) != D:
                raise ValueError("new_key / new_value must be [B, Hkv, D] of the query's dtype with contiguous tokens")
        if slot_mapping.dtype != torch.int32 or slot_mapping.numel() != B or not slot_mapping.is_contiguous():
            raise ValueError("slot_mapping must be contiguous int32 [B]")
        rc = lib.xllm_mi355_write_and_decode_gqa(
            new_key.data_ptr(), new_value.data_ptr(), slot_mapping.data_ptr(), new_key.stride(0), new_value.stride(0),
            _ptr(plan), 0 if plan is None else plan.numel(), query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            output.data_ptr(), _ptr(lse), block_table.data_ptr(), block_table.stride(0), seq_lens.data_ptr(), None,
            None, None, _ptr(k_cache_quant_scale), _ptr(v_cache_quant_scale), B, Hq, Hkv, D, bs, P,
            query.stride(0), output.stride(0), max_seq_len, int(window_left), float(scale), ws.data_ptr(), ws.numel(),
            _dtype_code(query), _dtype_code(k_cache), _stream(dev))
        capi.check(rc, "xllm_mi355_write_and_decode_gqa")
        return output, lse
    if plan is not None:
        rc = lib.xllm_mi355_paged_decode_gqa_planned(
            plan.data_ptr(), plan.numel(), query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(), _ptr(lse),
            block_table.data_ptr(), block_table.stride(0), seq_lens.data_ptr(), None, None, None,
            _ptr(k_cache_quant_scale), _ptr(v_cache_quant_scale), B, Hq, Hkv, D, bs, P,
            query.stride(0), output.stride(0), max_seq_len, int(window_left), float(scale), ws.data_ptr(), ws.numel(),
            _dtype_code(query), _dtype_code(k_cache), _stream(dev))
        capi.check(rc, "xllm_mi355_paged_decode_gqa_planned")
        return output, lse
    rc = lib.xllm_mi355_paged_decode_gqa(
        query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(), _ptr(lse),
        block_table.data_ptr(), block_table.stride(0), seq_lens.data_ptr(),
        _ptr(k_cache_quant_scale), _ptr(v_cache_quant_scale), B, Hq, Hkv, D, bs, P,
        query.stride(0), output.stride(0), max_seq_len, int(window_left), float(scale), ws.data_ptr(), ws.numel(),
        _dtype_code(query), _dtype_code(k_cache), _stream(dev))
    capi.check(rc, "xllm_mi355_paged_decode_gqa")
    return output, lse


def batch_decode_csr(query, k_cache, v_cache, paged_kv_indptr, paged_kv_indices,
                     paged_kv_last_page_len, window_left, sm_scale, output, output_lse=None, max_seq_len=0,
                     k_cache_quant_scale=None, v_cache_quant_scale=None, plan=None):
    """CSR paged decode: cuda::batch_decode (cuda_ops_api.h:128-144) without the FlashInfer
    uri / workspace arguments; plan plays the part of its plan_info (update_decode_plan_info; None = the launch
    derives its schedule itself); window_left as there (-1 = the whole context).  max_seq_len bounds the longest context; 0 means
    "all pages of the call could belong to one sequence"."""
    dev = _require_cuda(query, k_cache, v_cache, output, paged_kv_indptr, paged_kv_indices,
                        paged_kv_last_page_len, output_lse, k_cache_quant_scale, v_cache_quant_scale, plan)
    _decode_common(query, k_cache, output, v_cache, k_cache_quant_scale, v_cache_quant_scale)
    B, Hq, D = query.shape
    P, bs, Hkv, _ = k_cache.shape
    for t, n in ((paged_kv_indptr, B + 1), (paged_kv_last_page_len, B)):
        if t.dtype != torch.int32 or t.numel() != n or not t.is_contiguous():
            raise ValueError("CSR arrays must be contiguous int32 of the documented sizes")
    if paged_kv_indices.dtype != torch.int32 or not paged_kv_indices.is_contiguous():
        raise ValueError("paged_kv_indices must be contiguous int32")
    if max_seq_len <= 0:
        max_seq_len = max(1, paged_kv_indices.numel()) * bs
    lib = capi.lib()
    nbytes = lib.xllm_mi355_paged_decode_gqa_workspace_bytes(B, Hq, D)
    ws = decode_workspace(dev, nbytes)
    if plan is not None:
        _check_plan(plan)
        rc = lib.xllm_mi355_paged_decode_gqa_planned(
            plan.data_ptr(), plan.numel(), query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(),
            _ptr(output_lse), None, 0, None, paged_kv_indptr.data_ptr(), paged_kv_indices.data_ptr(),
            paged_kv_last_page_len.data_ptr(), _ptr(k_cache_quant_scale), _ptr(v_cache_quant_scale), B, Hq, Hkv, D,
            bs, P, query.stride(0), output.stride(0), max_seq_len, int(window_left), float(sm_scale), ws.data_ptr(),
            ws.numel(), _dtype_code(query), _dtype_code(k_cache), _stream(dev))
        capi.check(rc, "xllm_mi355_paged_decode_gqa_planned")
        return output
    rc = lib.xllm_mi355_paged_decode_gqa_csr(
        query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(), _ptr(output_lse),
        paged_kv_indptr.data_ptr(), paged_kv_indices.data_ptr(), paged_kv_last_page_len.data_ptr(),
        _ptr(k_cache_quant_scale), _ptr(v_cache_quant_scale), B, Hq, Hkv, D, bs, P,
        query.stride(0), output.stride(0), max_seq_len, int(window_left), float(sm_scale), ws.data_ptr(), ws.numel(),
        _dtype_code(query), _dtype_code(k_cache), _stream(dev))
    capi.check(rc, "xllm_mi355_paged_decode_gqa_csr")
    return output


def paged_forward(query, output, k_cache, v_cache, block_table, kv_seq_lens, q_cu_seq_lens, scale=None,
                  is_causal=True, max_seq_len=0, k_cache_quant_scale=None, v_cache_quant_scale=None,
                  max_query_len=0, window_left=-1):
    """Short query chunks (chunked prefill, speculative-decoding verification) against paged KV:
    the decode branch of FlashAttentionImpl::paged_forward (layers/dcu/flash_attention.cpp:447-545).
    query/output packed [T, Hq, D]; q_cu_seq_lens [B + 1] int32 from 0 to T; kv_seq_lens [B] int32 are
    the context lengths INCLUDING the chunk; with is_causal token j of a chunk of q_len tokens attends
    to the first kv_len - q_len + j + 1 tokens.  max_query_len (AttentionMetadata::max_query_len) bounds the
    chunk lengths; 0 = unknown.  Returns output."""
    dev = _require_cuda(query, k_cache, v_cache, output, block_table, kv_seq_lens, q_cu_seq_lens,
                        k_cache_quant_scale, v_cache_quant_scale)
    _decode_common(query, k_cache, output, v_cache, k_cache_quant_scale, v_cache_quant_scale)
    T, Hq, D = query.shape
    P, bs, Hkv, _ = k_cache.shape
    B = kv_seq_lens.numel()
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise ValueError("block_table must be int32 [B, W] with unit column stride")
    if block_table.shape[0] != B:
        raise ValueError("block_table rows must equal the batch")
    for t, n in ((kv_seq_lens, B), (q_cu_seq_lens, B + 1)):
        if t.dtype != torch.int32 or t.numel() != n or not t.is_contiguous():
            raise ValueError("kv_seq_lens [B] and q_cu_seq_lens [B + 1] must be contiguous int32")
    if scale is None:
        scale = D ** -0.5
    if max_seq_len <= 0:
        max_seq_len = block_table.shape[1] * bs
    if max_query_len > 0 and not torch.cuda.is_current_stream_capturing():
        # (a host read, so only outside capture: a chunk longer than the bound would leave its tail unwritten)
        longest = int((q_cu_seq_lens[1:] - q_cu_seq_lens[:-1]).max()) if B > 0 else 0
        if longest > max_query_len:
            raise ValueError(f"max_query_len is {max_query_len} but a chunk has {longest} query tokens")
    lib = capi.lib()
    nbytes = lib.xllm_mi355_paged_decode_varlen_workspace_bytes(max(T, B), Hq, D)
    ws = decode_workspace(dev, nbytes)
    rc = lib.xllm_mi355_paged_decode_gqa_varlen(
        query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(),
        q_cu_seq_lens.data_ptr(), kv_seq_lens.data_ptr(), block_table.data_ptr(), block_table.stride(0),
        _ptr(k_cache_quant_scale), _ptr(v_cache_quant_scale), B, T, int(max_query_len), Hq, Hkv, D, bs, P,
        query.stride(0), output.stride(0), max_seq_len, int(window_left), float(scale), 1 if is_causal else 0,
        ws.data_ptr(), ws.numel(), _dtype_code(query), _dtype_code(k_cache), _stream(dev))
    capi.check(rc, "xllm_mi355_paged_decode_gqa_varlen")
    return output


class DenseDecodeKind:
    """flash_mla::DenseDecodeKind (xllm/core/kernels/dcu/flash_mla_adapter.h:29-31)."""
    kQNopePe = 0


@dataclass
class DenseDecodeParams:
    """flash_mla::DenseDecodeParams (xllm/core/kernels/dcu/flash_mla_adapter.h:40-50), field for field."""
    q_nope: torch.Tensor       # [B, S_q, H, kv_lora_rank]
    q_pe: torch.Tensor         # [B, S_q, H, rope]
    k_cache: torch.Tensor      # [P, bs, 1, kv_lora_rank + rope]
    seqlens_k: torch.Tensor    # [B] int32
    block_table: torch.Tensor  # [B, W] int32
    head_size_v: int = 0
    softmax_scale: float = -1.0
    is_causal: bool = False
    kind: int = DenseDecodeKind.kQNopePe


def get_mla_decoding_metadata(seqlens_k, block_table, num_heads_per_head_k, block_size, plan=None):
    """The plan of an MLA decode step, made once per step for the dense_decode calls of all layers (metadata=...): the
    role of get_mla_decoding_metadata_dense_fp8, which the reference's adapter calls apart from the decode
    (flash_mla_adapter.cpp:125-130), and of the FlashInfer plan made at layer 0 (flashinfer_planinfo.cpp:248-264).
    num_heads_per_head_k = S_q * H_q as there; takes the step's lengths and block table; returns the plan (a device
    buffer; pass one back in to reuse it, as a captured step must)."""
    dev = _require_cuda(seqlens_k, block_table, plan)
    lib = capi.lib()
    nbytes = int(lib.xllm_mi355_paged_decode_plan_bytes())
    if plan is None:
        plan = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    _check_plan(plan)
    if seqlens_k.dtype != torch.int32 or not seqlens_k.is_contiguous() or seqlens_k.dim() != 1:
        raise ValueError("seqlens_k must be contiguous int32 [B]")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1 or \
            block_table.shape[0] != seqlens_k.numel():
        raise ValueError("block_table must be int32 [B, W] with unit column stride, one row per sequence")
    rc = lib.xllm_mi355_paged_decode_mla_plan(plan.data_ptr(), plan.numel(), block_table.data_ptr(),
                                              block_table.stride(0), seqlens_k.data_ptr(), seqlens_k.numel(),
                                              int(num_heads_per_head_k), int(block_size), _stream(dev))
    capi.check(rc, "xllm_mi355_paged_decode_mla_plan")
    return plan


def dense_decode(params: DenseDecodeParams, return_lse=False, max_seq_len=0, metadata=None, new_latent=None,
                 slot_mapping=None):
    """flash_mla::dense_decode (flash_mla_adapter.cpp:104-153): returns [B, S_q, H, head_size_v] (and the natural-log
    lse [B, H, S_q] fp32 when asked).  The same argument checks.  BF16 and FP16.  The S_q query tokens of a sequence
    are folded into the head count as the reference folds them (:119-123); with is_causal and S_q > 1 token j attends
    to the first seqlens_k - (S_q - 1 - j) tokens and every (sequence, token) becomes a row of its own.
    metadata: the step's plan from get_mla_decoding_metadata (same lengths and table), or None: the launch derives its
    schedule itself.  (A causal multi-token step rewrites lengths and table per token and takes no plan.)
    new_latent [B, 576] (or [B, 1, 576]) with slot_mapping [B] int32: the step's latent rows, stored into the cache by
    the same call before it attends (store_latent_cache + decode_flash_mla of the MLA layer,
    layers/dcu/deepseek_v2_attention.cpp:221-229 and :242-263, in one call; one query token per sequence)."""
    p = params
    if p.kind != DenseDecodeKind.kQNopePe:
        raise ValueError("flash_mla: only DenseDecodeKind::kQNopePe (BF16/FP16 split-q) is supported")
    dev = _require_cuda(p.q_nope, p.q_pe, p.k_cache, p.seqlens_k, p.block_table)
    if p.q_nope.dim() != 4 or p.q_pe.dim() != 4:
        raise ValueError("flash_mla: q_nope / q_pe must be 4D [B,S_q,H_q,D]")
    if p.k_cache.dim() != 4 or p.k_cache.shape[2] != 1:
        raise ValueError("flash_mla: k_cache must be 4D [blocks,page,1,D] with a single KV head")
    if p.seqlens_k.dim() != 1 or p.block_table.dim() != 2:
        raise ValueError("flash_mla: seqlens_k must be 1D [B] and block_table 2D [B,max_blocks]")
    B, Sq, H, d_latent = p.q_nope.shape
    d_rope = p.q_pe.shape[3]
    if p.q_pe.shape[:3] != p.q_nope.shape[:3]:
        raise ValueError("flash_mla: q_nope/q_pe batch, seq and head count must match")
    if p.k_cache.shape[3] != d_latent + d_rope:
        raise ValueError("flash_mla: k_cache last dim must equal q_nope.dim + q_pe.dim")
    if p.head_size_v <= 0:
        raise ValueError("flash_mla: head_size_v must be positive")
    if p.softmax_scale <= 0:
        raise ValueError("flash_mla: softmax_scale must be set by the MLA attention layer")
    if p.seqlens_k.numel() != B or p.block_table.shape[0] != B:
        raise ValueError("flash_mla: seqlens_k and block_table must have one row per sequence")
    if not p.k_cache.is_contiguous():
        raise ValueError("flash_mla: k_cache must be contiguous")
    if not (p.q_nope.dtype == p.q_pe.dtype == p.k_cache.dtype) or p.q_nope.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError("flash_mla: q_nope, q_pe and k_cache must share one dtype, BF16 or FP16")
    if p.head_size_v != d_latent:
        raise NotImplementedError("V is the latent part of the cache: head_size_v must equal kv_lora_rank")
    seqlens = (p.seqlens_k if p.seqlens_k.dtype == torch.int32 else p.seqlens_k.to(torch.int32)).contiguous()
    table = p.block_table if p.block_table.dtype == torch.int32 else p.block_table.to(torch.int32)
    if table.stride(1) != 1:
        table = table.contiguous()
    q_nope = p.q_nope.contiguous()
    q_pe = p.q_pe.contiguous()
    P, bs = p.k_cache.shape[0], p.k_cache.shape[1]
    out = torch.empty(B, Sq, H, p.head_size_v, dtype=q_nope.dtype, device=dev)
    rows, heads = B, Sq * H
    if p.is_causal and Sq > 1:
        rows, heads = B * Sq, H
        back = torch.arange(Sq - 1, -1, -1, dtype=torch.int32, device=dev)
        seqlens = (seqlens.unsqueeze(1) - back.unsqueeze(0)).clamp_min(0).reshape(rows).contiguous()
        table = table.repeat_interleave(Sq, 0).contiguous()
    lse = torch.empty(rows, heads, dtype=torch.float32, device=dev) if return_lse else None
    if max_seq_len <= 0:
        max_seq_len = table.shape[1] * bs
    lib = capi.lib()
    nbytes = lib.xllm_mi355_paged_decode_mla_workspace_bytes(rows, heads, max_seq_len)
    ws = decode_workspace(dev, nbytes)
    planned = metadata is not None and not (p.is_causal and Sq > 1)
    if planned:
        _check_plan(metadata)
    if new_latent is not None or slot_mapping is not None:
        if new_latent is None or slot_mapping is None:
            raise ValueError("new_latent and slot_mapping come together")
        if Sq != 1:
            raise ValueError("the one-call step stores one new row per sequence: S_q must be 1")
        _require_cuda(new_latent, slot_mapping)
        rows_new = new_latent.view(B, d_latent + d_rope) if new_latent.dim() == 3 else new_latent
        if rows_new.dtype != q_nope.dtype or tuple(rows_new.shape) != (B, d_latent + d_rope) or rows_new.stride(1) != 1:
            raise ValueError("new_latent must be [B, kv_lora_rank + rope dim] of the query's dtype with contiguous rows")
        if slot_mapping.dtype != torch.int32 or slot_mapping.numel() != B or not slot_mapping.is_contiguous():
            raise ValueError("slot_mapping must be contiguous int32 [B]")
        rc = lib.xllm_mi355_write_and_decode_mla(
            rows_new.data_ptr(), slot_mapping.data_ptr(), rows_new.stride(0), _ptr(metadata) if planned else None,
            metadata.numel() if planned else 0, q_nope.data_ptr(), q_pe.data_ptr(), p.k_cache.data_ptr(),
            out.data_ptr(), _ptr(lse), table.data_ptr(), table.stride(0), seqlens.data_ptr(), rows, heads, d_latent,
            d_rope, bs, P, max_seq_len, float(p.softmax_scale), ws.data_ptr(), ws.numel(), _dtype_code(q_nope),
            _stream(dev))
        capi.check(rc, "xllm_mi355_write_and_decode_mla")
    elif planned:
        rc = lib.xllm_mi355_paged_decode_mla_planned(
            metadata.data_ptr(), metadata.numel(), q_nope.data_ptr(), q_pe.data_ptr(), p.k_cache.data_ptr(),
            out.data_ptr(), _ptr(lse), table.data_ptr(), table.stride(0), seqlens.data_ptr(), rows, heads, d_latent,
            d_rope, bs, P, max_seq_len, float(p.softmax_scale), ws.data_ptr(), ws.numel(), _dtype_code(q_nope),
            _stream(dev))
        capi.check(rc, "xllm_mi355_paged_decode_mla_planned")
    else:
        rc = lib.xllm_mi355_paged_decode_mla(
            q_nope.data_ptr(), q_pe.data_ptr(), p.k_cache.data_ptr(), out.data_ptr(), _ptr(lse),
            table.data_ptr(), table.stride(0), seqlens.data_ptr(), rows, heads, d_latent, d_rope, bs, P,
            max_seq_len, float(p.softmax_scale), ws.data_ptr(), ws.numel(), _dtype_code(q_nope),
            _stream(dev))
        capi.check(rc, "xllm_mi355_paged_decode_mla")
    if return_lse:
        return out, lse.view(B, Sq, H).transpose(1, 2).contiguous()
    return out


# ------------------------------------------------------------------------------------------
# merge and table helpers

def merge_dcp_attention_shards(partial_outputs, partial_lse):
    """merge_dcp_attention_shards (dcp_attention_merge.cpp:26-65).
    partial_outputs [S, B, Q=1, H, Dv]; partial_lse [S, B, H, Q=1] -> (output [B,1,H,Dv], lse [B,H,1])."""
    dev = _require_cuda(partial_outputs, partial_lse)
    if partial_outputs.dim() != 5:
        raise ValueError("partial outputs must have shape [dcp, batch, query, heads, value]")
    if partial_lse.dim() != 4:
        raise ValueError("partial LSE must have shape [dcp, batch, heads, query]")
    S, B, Q, H, Dv = partial_outputs.shape
    if tuple(partial_lse.shape) != (S, B, H, Q):
        raise ValueError("partial outputs and LSE disagree on [dcp, batch, heads, query]")
    if Q != 1:
        raise NotImplementedError("decode path: one query token per sequence")
    po = partial_outputs.contiguous()
    pl = partial_lse.to(torch.float32).contiguous()
    out = torch.empty(B, Q, H, Dv, dtype=po.dtype, device=dev)
    lse = torch.empty(B, H, Q, dtype=torch.float32, device=dev)
    rc = capi.lib().xllm_mi355_lse_merge(po.data_ptr(), pl.data_ptr(), out.data_ptr(), lse.data_ptr(),
                                         S, B, H, Dv, _dtype_code(po), _stream(dev))
    capi.check(rc, "xllm_mi355_lse_merge")
    return out, lse


def lse_combine(output, shared_o, shared_lse, unshared_o, unshared_lse):
    """xllm::kernel::cuda::lse_combine (kernels/cuda/xattention/lse_combine.cu:99-166), same arguments: shared_o /
    unshared_o [B, H, D], the LSEs [B, H, 1] fp32 in BASE 2; output [B, H, D] (allocated like shared_o when None or
    of another shape).  Returns output."""
    dev = _require_cuda(output, shared_o, shared_lse, unshared_o, unshared_lse)
    if shared_o.dim() != 3 or unshared_o.dim() != 3:
        raise ValueError("shared_o and unshared_o must be 3D [B, H, D]")
    if shared_lse.dim() != 3 or unshared_lse.dim() != 3:
        raise ValueError("shared_lse and unshared_lse must be 3D [B, H, 1]")
    if shared_o.shape != unshared_o.shape or shared_o.dtype != unshared_o.dtype:
        raise ValueError("shared_o and unshared_o must have same shape")
    B, H, D = shared_o.shape
    for t in (shared_lse, unshared_lse):
        if t.dtype != torch.float32 or tuple(t.shape) != (B, H, 1):
            raise ValueError("the LSEs must be float32 [B, H, 1]")
    if output is None or output.shape != shared_o.shape:
        output = torch.empty_like(shared_o)
    so, uo = shared_o.contiguous(), unshared_o.contiguous()
    if not output.is_contiguous():
        raise ValueError("output must be contiguous")
    rc = capi.lib().xllm_mi355_lse_combine(
        output.data_ptr(), so.data_ptr(), shared_lse.contiguous().data_ptr(), uo.data_ptr(),
        unshared_lse.contiguous().data_ptr(), B * H, D, _dtype_code(so), _dtype_code(output), _stream(dev))
    capi.check(rc, "xllm_mi355_lse_combine")
    return output


def build_block_table_from_paged_kv(paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len,
                                    table_width, block_size):
    """CSR -> (block_table [B, table_width] int32 with -1 padding, seq_lens [B] int32)."""
    dev = _require_cuda(paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len)
    B = paged_kv_indptr.numel() - 1
    table = torch.empty(B, table_width, dtype=torch.int32, device=dev)
    seq_lens = torch.empty(B, dtype=torch.int32, device=dev)
    rc = capi.lib().xllm_mi355_build_block_table(
        paged_kv_indptr.data_ptr(), paged_kv_indices.data_ptr(), paged_kv_last_page_len.data_ptr(),
        table.data_ptr(), table_width, seq_lens.data_ptr(), B, block_size, _stream(dev))
    capi.check(rc, "xllm_mi355_build_block_table")
    return table, seq_lens


def mask_block_table_padding(block_table, kv_seq_lens, page_block_size):
    """layers/dcu/flash_attention.cpp:194-218: a copy of block_table [B, W] with -1 in the columns beyond each
    sequence's ceil(kv_seq_lens / page_block_size) pages (by position, never by page id).  int32 result."""
    dev = _require_cuda(block_table, kv_seq_lens)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise ValueError("block_table must be int32 [B, W] with unit column stride")
    B, W = block_table.shape
    if kv_seq_lens.dtype != torch.int32 or kv_seq_lens.numel() != B or not kv_seq_lens.is_contiguous():
        raise ValueError("kv_seq_lens must be contiguous int32 [B]")
    if page_block_size <= 0:
        raise ValueError("page_block_size must be positive")
    out = torch.empty(B, W, dtype=torch.int32, device=dev)
    rc = capi.lib().xllm_mi355_mask_block_table_padding(
        block_table.data_ptr(), block_table.stride(0), kv_seq_lens.data_ptr(), out.data_ptr(), out.stride(0),
        B, W, page_block_size, _stream(dev))
    capi.check(rc, "xllm_mi355_mask_block_table_padding")
    return out


def fused_qk_norm_rope(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight,
                       cos_sin_cache, interleave, position_ids, k_cache=None, v_cache=None, slot_mapping=None,
                       k_cache_scale=None, v_cache_scale=None):
    """xllm::kernel::cuda::fused_qk_norm_rope with the reference's arguments in the reference's order
    (kernels/cuda/fused_qknorm_rope.cu:388-470; caller layers/common/qwen2_attention.cpp:149-166): qkv
    [T, (Hq + Hk + Hv) * D] is normalised and rotated in place.  With k_cache / v_cache / slot_mapping the same
    launch also writes the new k and v rows into the paged cache (the reshape_paged_cache call that follows in the
    reference); fp8 caches take the per-KV-head scales."""
    dev = _require_cuda(qkv, cos_sin_cache, position_ids, q_weight, k_weight, k_cache, v_cache, slot_mapping,
                        k_cache_scale, v_cache_scale)
    if qkv.dim() != 2 or qkv.stride(1) != 1:
        raise ValueError("qkv must be [tokens, (Hq + Hk + Hv) * head_dim] with contiguous rows")
    if qkv.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError("qkv must be bf16 or fp16")
    T = qkv.shape[0]
    if qkv.shape[1] != (num_heads_q + num_heads_k + num_heads_v) * head_dim:
        raise ValueError("qkv width must be (Hq + Hk + Hv) * head_dim")
    if position_ids.dtype != torch.int64 or not position_ids.is_contiguous() or position_ids.numel() != T:
        raise ValueError("position_ids must be a contiguous int64 tensor [tokens]")
    if cos_sin_cache.dim() != 2 or not cos_sin_cache.is_contiguous():
        raise ValueError("cos_sin_cache must be [max_position, rotary_dim], contiguous")
    if (q_weight is None) != (k_weight is None):
        raise ValueError("q_weight and k_weight go together")
    for w in (q_weight, k_weight):
        if w is not None and (w.dtype != qkv.dtype or w.numel() != head_dim or not w.is_contiguous()):
            raise ValueError("q_weight / k_weight must be contiguous [head_dim] tensors of the qkv dtype")
    with_cache = k_cache is not None
    cache_code = _dtype_code(qkv)
    if with_cache:
        if v_cache is None or slot_mapping is None:
            raise ValueError("the fused cache write needs k_cache, v_cache and slot_mapping")
        if (k_cache.dim() != 4 or tuple(k_cache.shape[2:]) != (num_heads_k, head_dim) or not k_cache.is_contiguous()
                or v_cache.shape != k_cache.shape or v_cache.dtype != k_cache.dtype or not v_cache.is_contiguous()
                or num_heads_v != num_heads_k):
            raise ValueError("k_cache / v_cache must be contiguous [P, bs, num_heads_k, head_dim] of one dtype")
        if slot_mapping.dtype != torch.int32 or not slot_mapping.is_contiguous() or slot_mapping.numel() != T:
            raise ValueError("slot_mapping must be contiguous int32 [tokens]")
        cache_code = _dtype_code(k_cache)   # fp8 caches are float8_e4m3fn or uint8 tensors
        if cache_code == capi.FP8_E4M3:
            for sc in (k_cache_scale, v_cache_scale):
                if sc is None or sc.dtype != torch.float32 or sc.numel() != num_heads_k or not sc.is_contiguous():
                    raise ValueError("an fp8 cache needs contiguous fp32 scales [num_heads_k] for K and V")
        elif k_cache.dtype != qkv.dtype:
            raise TypeError("the cache dtype must equal the qkv dtype (or be fp8)")
    rc = capi.lib().xllm_mi355_rope_and_cache(
        qkv.data_ptr(), _ptr(q_weight), _ptr(k_weight), cos_sin_cache.data_ptr(), position_ids.data_ptr(),
        _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), _ptr(k_cache_scale), _ptr(v_cache_scale),
        qkv.shape[0], qkv.stride(0), num_heads_q, num_heads_k, num_heads_v, head_dim, cos_sin_cache.shape[1],
        float(eps), 1 if interleave else 0, k_cache.shape[1] if with_cache else 0,
        k_cache.shape[0] if with_cache else 0, _dtype_code(qkv), _dtype_code(cos_sin_cache),
        cache_code, _stream(dev))
    capi.check(rc, "xllm_mi355_rope_and_cache")
    return qkv


@dataclass
class LlmDecodeMetadataUpdateParams:
    """Mirror of xllm::kernel::cuda::LlmDecodeMetadataUpdateParams
    (xllm/core/kernels/cuda/llm_decode_metadata_update.h:33-53): int32 device tensors and four sizes."""
    src_tokens: torch.Tensor
    src_positions: torch.Tensor
    src_new_cache_slots: torch.Tensor
    src_kv_seq_lens: torch.Tensor          # cumulative, [actual_batch_size + 1]
    src_paged_kv_indptr: torch.Tensor
    src_paged_kv_indices: torch.Tensor
    src_paged_kv_last_page_len: torch.Tensor
    dst_tokens: torch.Tensor
    dst_positions: torch.Tensor
    dst_new_cache_slots: torch.Tensor
    dst_kv_seq_lens: torch.Tensor
    dst_kv_seq_lens_delta: torch.Tensor
    dst_paged_kv_indptr: torch.Tensor
    dst_paged_kv_indices: torch.Tensor
    dst_paged_kv_last_page_len: torch.Tensor
    actual_num_tokens: int
    padded_num_tokens: int
    actual_batch_size: int
    actual_indices_size: int


_METADATA_FIELDS = ("src_tokens", "src_positions", "src_new_cache_slots", "src_kv_seq_lens", "src_paged_kv_indptr",
                    "src_paged_kv_indices", "src_paged_kv_last_page_len", "dst_tokens", "dst_positions",
                    "dst_new_cache_slots", "dst_kv_seq_lens", "dst_kv_seq_lens_delta", "dst_paged_kv_indptr",
                    "dst_paged_kv_indices", "dst_paged_kv_last_page_len")


def update_llm_decode_metadata(params: LlmDecodeMetadataUpdateParams):
    """update_llm_decode_metadata (llm_decode_metadata_update.cu:74-104): one launch on the current stream that
    copies a decode step's metadata into the persistent buffers of a captured step and pads them."""
    tensors = [getattr(params, f) for f in _METADATA_FIELDS]
    dev = _require_cuda(*[t for t in tensors if t is not None and t.numel() > 0])
    for f, t in zip(_METADATA_FIELDS, tensors):
        if t is not None and (t.dtype != torch.int32 or not t.is_contiguous()):
            raise ValueError(f"{f} must be a contiguous int32 tensor")
    rc = capi.lib().xllm_mi355_decode_metadata_update(
        *[0 if t is None or t.numel() == 0 else t.data_ptr() for t in tensors],
        params.actual_num_tokens, params.padded_num_tokens, params.actual_batch_size, params.actual_indices_size,
        _stream(dev))
    capi.check(rc, "xllm_mi355_decode_metadata_update")


def gather_mla_latent_cache(k_cache, block_table, kv_cu_seq_lens, total_kv_len, max_seq_len=0):
    """dcu::gather_mla_latent_cache (kernels/dcu/dcu_ops_api.h:74, gather_mla_latent_cache.hip:124-190):
    k_cache [P, bs, 1, D] contiguous, block_table [B, W] int32, kv_cu_seq_lens [B + 1] int32 ->
    [total_kv_len, D] with the rows of sequence b at kv_cu_seq_lens[b] ...  max_seq_len only sizes the
    reference's launch grid and is ignored."""
    del max_seq_len
    dev = _require_cuda(k_cache, block_table, kv_cu_seq_lens)
    if k_cache.dim() != 4 or k_cache.shape[2] != 1 or not k_cache.is_contiguous():
        raise ValueError("k_cache must be contiguous [blocks, block_size, 1, dim]")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise ValueError("block_table must be int32 [B, W] with unit column stride")
    B = block_table.shape[0]
    if kv_cu_seq_lens.dtype != torch.int32 or kv_cu_seq_lens.numel() != B + 1 or not kv_cu_seq_lens.is_contiguous():
        raise ValueError("kv_cu_seq_lens must be contiguous int32 [B + 1]")
    if total_kv_len <= 0:
        raise ValueError("total_kv_len must be positive")
    P, bs, _, D = k_cache.shape
    out = torch.empty(total_kv_len, D, dtype=k_cache.dtype, device=dev)
    rc = capi.lib().xllm_mi355_gather_paged_rows(
        k_cache.data_ptr(), block_table.data_ptr(), block_table.stride(0), kv_cu_seq_lens.data_ptr(),
        out.data_ptr(), B, total_kv_len, bs, P, D * k_cache.element_size(), _stream(dev))
    capi.check(rc, "xllm_mi355_gather_paged_rows")
    return out


def absorbed_bmm(x, w, out=None):
    """The per-head product either side of the MLA decode kernel: x [T, H, K], w [H, K, N] -> [T, H, N], i.e.
    torch.bmm(x.transpose(0, 1), w).transpose(0, 1) of layers/dcu/deepseek_v2_attention.cpp:428-430 (q_nope with
    w_kc_) and :231-238 (the decode output with w_vc_).  x may be a slice of a wider tensor (unit stride in the
    last dim); w contiguous.  fp32 accumulation, one rounding to bf16."""
    dev = _require_cuda(x, w)
    if x.dim() != 3 or w.dim() != 3 or x.shape[1] != w.shape[0] or x.shape[2] != w.shape[1]:
        raise ValueError(f"shapes do not match: x {tuple(x.shape)} against w {tuple(w.shape)}")
    if x.dtype != w.dtype:
        raise TypeError("x and w must have the same dtype")
    if x.stride(2) != 1 or not w.is_contiguous():
        raise ValueError("x needs unit stride in its last dim and w must be contiguous")
    T, H, K = x.shape
    N = w.shape[2]
    if out is None:
        out = torch.empty(T, H, N, dtype=x.dtype, device=dev)
    elif out.shape != (T, H, N) or out.dtype != x.dtype or out.stride(2) != 1 or out.device != x.device:
        raise ValueError("out must be [T, H, N] of x's dtype and device with unit stride in its last dim")
    rc = capi.lib().xllm_mi355_mla_absorbed_bmm(
        x.data_ptr(), w.data_ptr(), out.data_ptr(), T, H, K, N, x.stride(0), x.stride(1), out.stride(0),
        out.stride(1), _dtype_code(x), _stream(dev))
    capi.check(rc, "xllm_mi355_mla_absorbed_bmm")
    return out
