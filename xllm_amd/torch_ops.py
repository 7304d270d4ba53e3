"""Loads the C++ host side (libxllm_mi355_torch.so): the reference's torch::Tensor op interface
over the C ABI, registered with the torch dispatcher as torch.ops.xllm_ops.*.

  torch.ops.xllm_ops.reshape_paged_cache(slot_mapping, keys, values, key_cache, value_cache)
      -- the reference's schema (xllm/core/kernels/cuda/cuda_ops_library.cpp:286-287)
  torch.ops.xllm_ops.quant_to_paged_cache(..., k_scale, v_scale)
  torch.ops.xllm_ops.batch_decode(query, k_cache, v_cache, output, block_table, seq_lens,
                                  k_scale, v_scale, max_seq_len, scale, plan=None) -> (output, lse)
  torch.ops.xllm_ops.update_decode_plan(block_table, seq_lens, num_qo_heads, num_kv_heads, head_dim, block_size,
                                        window_left, fp8_cache, plan=None) -> plan
      -- the step's plan, made once for the decode calls of all layers (the role of update_decode_plan_info,
         xllm/core/layers/cuda/flashinfer_planinfo.cpp:248-264)
  torch.ops.xllm_ops.mla_dense_decode(q_nope, q_pe, k_cache, seqlens_k, block_table,
                                      head_size_v, softmax_scale, is_causal=False) -> (out, lse)
  torch.ops.xllm_ops.merge_dcp_attention_shards(partial_outputs, partial_lse) -> (out, lse)
  torch.ops.xllm_ops.lse_combine(output, shared_o, shared_lse, unshared_o, unshared_lse) -> output   (base-2 LSEs)
  torch.ops.xllm_ops.attention_layer_forward(query, key, value, k_cache, v_cache, k_cache_scale, v_cache_scale,
        slot_mapping, block_table, kv_seq_lens, q_cu_seq_lens, max_seq_len, max_query_len, num_heads, head_size,
        num_kv_heads, scale, sliding_window, is_causal, return_lse, plan=None, layer_id=-1)
        -> (output [T, Hq * D], lse or None)
      -- AttentionImpl::forward of the reference (xllm/core/layers/dcu/attention.cpp:55-112) end to end
"""
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
SHIM_PATH = os.path.join(_HERE, "libxllm_mi355_torch.so")
_loaded = False


def load():
    global _loaded
    if not _loaded:
        if not os.path.exists(SHIM_PATH):
            raise RuntimeError(f"{SHIM_PATH} is missing: build it with `python -m xllm_amd.build`")
        torch.ops.load_library(SHIM_PATH)
        _loaded = True
    return torch.ops.xllm_ops
