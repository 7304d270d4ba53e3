// C++ host side of the MI355X paged-KV decode path: the reference's kernel op interface
// (torch::Tensor structs and free functions) over the C ABI of include/xllm_mi355.h.
//
// Names, argument order and meaning follow the reference (paths relative to the xLLM tree):
//   xllm::kernel::ReshapePagedCacheParams, reshape_paged_cache, quant_to_paged_cache
//       xllm/core/kernels/param.h:126-161, ops_api.h:31, ops_api.cpp:248-310
//   xllm::kernel::mi355::batch_decode (block table)   xllm/core/kernels/mlu/mlu_ops_api.h:127,
//                                                     xllm/core/kernels/npu/npu_ops_api.h:46
//   xllm::kernel::mi355::batch_decode_csr             xllm/core/kernels/cuda/cuda_ops_api.h:128-144
//   xllm::kernel::mi355::flash_mla::dense_decode      xllm/core/kernels/dcu/flash_mla_adapter.h:40-53
//   xllm::layer::merge_dcp_attention_shards           xllm/core/layers/mlu/dcp_attention_merge.h:28-34
// A violated precondition throws c10::Error (TORCH_CHECK) where the reference CHECK-aborts.
#pragma once

#include <torch/torch.h>

#include <optional>
#include <tuple>

namespace xllm::kernel {

struct ReshapePagedCacheParams {
  torch::Tensor key;                       // [T, Hkv, D], last two dims contiguous
  std::optional<torch::Tensor> value;      // same shape; given iff v_cache is
  torch::Tensor k_cache;                   // [P, bs, Hkv, D] contiguous
  std::optional<torch::Tensor> v_cache;
  torch::Tensor slot_mapping;              // [T] int32
  bool direction = false;                  // CACHE2CONTEXT is not part of this path
  std::optional<torch::Tensor> k_cache_scale;  // [Hkv] fp32 for the fp8 cache
  std::optional<torch::Tensor> v_cache_scale;
};

void reshape_paged_cache(ReshapePagedCacheParams& params);
void quant_to_paged_cache(ReshapePagedCacheParams& params);

namespace mi355 {

// Per-device split workspace, allocated once (at the library's bound over every supported shape, or nbytes if
// that is more) and never replaced; same lifetime as the reference's FlashinferWorkspace singleton
// (xllm/core/layers/cuda/flashinfer_workspace.cpp:25-41).  A request beyond its size throws.  It serves one
// stream at a time: decode calls on two streams of one device must not overlap.
torch::Tensor decode_workspace(const torch::Device& device, size_t nbytes);
// Throws if a bounded wait inside a decode kernel gave up since the last call (that launch's outputs are
// invalid).  Synchronises the current stream: not for use under graph capture.
void decode_status(const torch::Device& device);

void batch_decode(const torch::Tensor& query,        // [B, Hq, D]
                  const torch::Tensor& k_cache,      // [P, bs, Hkv, D]
                  torch::Tensor& output,             // [B, Hq, D]
                  const torch::Tensor& block_table,  // [B, W] int32
                  const torch::Tensor& seq_lens,     // [B] int32
                  const std::optional<torch::Tensor>& v_cache,
                  std::optional<torch::Tensor>& output_lse,  // [B, Hq, 1] fp32, natural log
                  const std::optional<torch::Tensor>& k_cache_quant_scale,
                  const std::optional<torch::Tensor>& v_cache_quant_scale,
                  int64_t max_seq_len, float scale, bool return_lse);

void batch_decode_csr(torch::Tensor query, torch::Tensor k_cache, torch::Tensor v_cache,
                      torch::Tensor paged_kv_indptr, torch::Tensor paged_kv_indices,
                      torch::Tensor paged_kv_last_page_len, double sm_scale, torch::Tensor output,
                      std::optional<torch::Tensor>& output_lse, int64_t max_seq_len);

// Short query chunks against paged KV: the decode branch of FlashAttentionImpl::paged_forward
// (xllm/core/layers/dcu/flash_attention.cpp:447-545).  query / output packed [T, Hq, D]; kv_seq_lens [B] are the
// context lengths including the chunk, q_cu_seq_lens [B + 1] the chunk boundaries, max_query_len the bound on
// the chunk lengths (AttentionMetadata::max_query_len; 0 = unknown).
void paged_forward(const torch::Tensor& query, torch::Tensor& output, const torch::Tensor& k_cache,
                   const torch::Tensor& v_cache, const torch::Tensor& block_table,
                   const torch::Tensor& kv_seq_lens, const torch::Tensor& q_cu_seq_lens, float scale,
                   bool is_causal, int64_t max_seq_len, int64_t max_query_len);

// xllm::kernel::dcu::gather_mla_latent_cache (xllm/core/kernels/dcu/dcu_ops_api.h:74), same arguments.
torch::Tensor gather_mla_latent_cache(const torch::Tensor& k_cache, const torch::Tensor& block_table,
                                      const torch::Tensor& kv_cu_seq_lens, int64_t total_kv_len,
                                      int64_t max_seq_len);

// mask_block_table_padding (xllm/core/layers/dcu/flash_attention.cpp:194-218), same arguments: a copy of
// block_table with -1 in the columns beyond each sequence's pages.
torch::Tensor mask_block_table_padding(const torch::Tensor& block_table, const torch::Tensor& kv_seq_lens,
                                       int64_t page_block_size);

// The per-head products of the absorbed MLA attention: x [T, H, K], w [H, K, N] -> [T, H, N] contiguous.
// Stands for torch::bmm(x.transpose(0, 1), w).transpose(0, 1) at xllm/core/layers/dcu/deepseek_v2_attention.cpp:428-430
// (q_nope with w_kc_) and :231-238 (the decode output with w_vc_).  x may be a slice of a wider tensor.
torch::Tensor absorbed_bmm(const torch::Tensor& x, const torch::Tensor& w);

// xllm::kernel::cuda::fused_qk_norm_rope (xllm/core/kernels/cuda/cuda_ops_api.h:235-249), same arguments.
void fused_qk_norm_rope(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                        int64_t head_dim, double eps, const torch::Tensor& q_weight, const torch::Tensor& k_weight,
                        const torch::Tensor& cos_sin_cache, bool interleaved, const torch::Tensor& position_ids);
// The same launch followed by nothing: it also stores the new k and v rows in the paged cache, which the
// reference does with reshape_paged_cache / quant_to_paged_cache right after
// (xllm/core/layers/common/qwen2_attention.cpp:149-186, xllm/core/layers/dcu/flash_attention.cpp:587-595).
void fused_qk_norm_rope_and_cache(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                                  int64_t head_dim, double eps, const torch::Tensor& q_weight,
                                  const torch::Tensor& k_weight, const torch::Tensor& cos_sin_cache, bool interleaved,
                                  const torch::Tensor& position_ids, ReshapePagedCacheParams& cache);

// xllm::kernel::cuda::LlmDecodeMetadataUpdateParams and update_llm_decode_metadata
// (xllm/core/kernels/cuda/llm_decode_metadata_update.h:33-56), field for field; the stream is the
// caller's, as there.
struct LlmDecodeMetadataUpdateParams {
  const int32_t* src_tokens;
  const int32_t* src_positions;
  const int32_t* src_new_cache_slots;
  const int32_t* src_kv_seq_lens;
  const int32_t* src_paged_kv_indptr;
  const int32_t* src_paged_kv_indices;
  const int32_t* src_paged_kv_last_page_len;
  int32_t* dst_tokens;
  int32_t* dst_positions;
  int32_t* dst_new_cache_slots;
  int32_t* dst_kv_seq_lens;
  int32_t* dst_kv_seq_lens_delta;
  int32_t* dst_paged_kv_indptr;
  int32_t* dst_paged_kv_indices;
  int32_t* dst_paged_kv_last_page_len;
  int64_t actual_num_tokens;
  int64_t padded_num_tokens;
  int64_t actual_batch_size;
  int64_t actual_indices_size;
};
void update_llm_decode_metadata(const LlmDecodeMetadataUpdateParams& params, void* stream);

namespace flash_mla {
struct DenseDecodeParams {
  torch::Tensor q_nope;       // [B, S_q, H, kv_lora_rank]
  torch::Tensor q_pe;         // [B, S_q, H, rope]
  torch::Tensor k_cache;      // [P, bs, 1, kv_lora_rank + rope]
  torch::Tensor seqlens_k;    // [B] int32
  torch::Tensor block_table;  // [B, W] int32
  int64_t head_size_v = 0;
  float softmax_scale = -1.0F;
  bool is_causal = false;
};
// Returns [B, S_q, H, head_size_v]; lse (if not null) receives [B, H, 1] fp32.
torch::Tensor dense_decode(DenseDecodeParams& params, torch::Tensor* lse = nullptr);
}  // namespace flash_mla

}  // namespace mi355
}  // namespace xllm::kernel

namespace xllm::layer {
struct DcpAttentionResult {
  torch::Tensor output;
  torch::Tensor lse;
};
// partial_outputs [S, B, Q=1, H, Dv], partial_lse [S, B, H, Q=1] (natural log).
DcpAttentionResult merge_dcp_attention_shards(const torch::Tensor& partial_outputs,
                                              const torch::Tensor& partial_lse);
}  // namespace xllm::layer
