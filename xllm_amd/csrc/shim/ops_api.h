// C++ host side of the MI355X paged-KV decode path: the reference's kernel op interface
// (torch::Tensor structs and free functions) over the C ABI of include/xllm_mi355.h.
//
// Names, argument order and meaning follow the reference (paths relative to the xLLM tree):
//   xllm::kernel::ReshapePagedCacheParams, reshape_paged_cache, quant_to_paged_cache
//       xllm/core/kernels/param.h:126-161, ops_api.h:31, ops_api.cpp:248-310
//   xllm::kernel::mi355::batch_decode (block table)   xllm/core/kernels/mlu/mlu_ops_api.h:127,
//                                                     xllm/core/kernels/npu/npu_ops_api.h:46
//   xllm::kernel::mi355::batch_decode_csr             xllm/core/kernels/cuda/cuda_ops_api.h:128-144
//   xllm::kernel::dcu::flash_mla::dense_decode        xllm/core/kernels/dcu/flash_mla_adapter.h:29-53
//   xllm::kernel::mi355::lse_combine                  xllm/core/kernels/cuda/xattention/xattention_ops_api.h:38
//   xllm::layer::merge_dcp_attention_shards           xllm/core/layers/mlu/dcp_attention_merge.h:28-34
//   xllm::layer::AttentionMetadata (decode subset), xllm::KVCache (accessors), xllm::layer::BaseAttentionImpl,
//   xllm::layer::AttentionImpl                        xllm/core/layers/common/attention_metadata.h:99-156,
//                                                     xllm/core/framework/kv_cache/kv_cache.h:29-95,
//                                                     xllm/core/layers/dcu/base_attention_impl.h:30-57,
//                                                     xllm/core/layers/dcu/attention.cpp:28-112
// A violated precondition throws c10::Error (TORCH_CHECK) where the reference CHECK-aborts.
#pragma once

#include <torch/torch.h>

#include <memory>
#include <optional>
#include <vector>
#include <string>
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

// The K / V rows of a decode step's new tokens [B, Hkv, D] and their slots [B] int32: handed to batch_decode, they
// are stored into the caches by the decode call itself (the reshape_paged_cache + batch_decode pair of
// xllm/core/layers/dcu/torch_attention.cpp:138-144 and :285-347 in one call, with the pair's cache bytes and output).
struct NewKvRows {
  torch::Tensor key, value, slot_mapping;
};

void batch_decode(const torch::Tensor& query,        // [B, Hq, D]
                  const torch::Tensor& k_cache,      // [P, bs, Hkv, D]
                  torch::Tensor& output,             // [B, Hq, D]
                  const torch::Tensor& block_table,  // [B, W] int32
                  const torch::Tensor& seq_lens,     // [B] int32
                  const std::optional<torch::Tensor>& v_cache,
                  std::optional<torch::Tensor>& output_lse,  // [B, Hq, 1] fp32, natural log
                  const std::optional<torch::Tensor>& k_cache_quant_scale,
                  const std::optional<torch::Tensor>& v_cache_quant_scale,
                  int64_t max_seq_len, int64_t window_size_left, float scale, bool return_lse,
                  const std::optional<torch::Tensor>& plan = std::nullopt, const NewKvRows* fresh = nullptr);

// The plan of a decode step, made once and taken by the decode calls of every layer (`plan` above and in
// batch_decode_csr): the part of update_decode_plan_info (xllm/core/layers/cuda/flashinfer_planinfo.cpp:248-264),
// whose result the reference hands to cuda::batch_decode as plan_info (cuda_ops_api.h:128-129).  One small launch;
// `plan` is reused when given (a captured step must reuse it), else allocated.  Either the block table with the
// lengths or the three CSR arrays; cache_dtype is the dtype of the KV cache.
torch::Tensor update_decode_plan(const std::optional<torch::Tensor>& plan,
                                 const std::optional<torch::Tensor>& block_table,
                                 const std::optional<torch::Tensor>& seq_lens,
                                 const std::optional<torch::Tensor>& paged_kv_indptr,
                                 const std::optional<torch::Tensor>& paged_kv_indices,
                                 const std::optional<torch::Tensor>& paged_kv_last_page_len,
                                 int64_t num_qo_heads, int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                 int64_t window_left, torch::ScalarType cache_dtype);

// The CSR form, with the arguments of xllm::kernel::cuda::batch_decode (cuda_ops_api.h:128-144) that are not
// FlashInfer's own (uri, plan_info, the three workspace buffers, use_tensor_core, qo_indptr), in its order;
// max_seq_len bounds the longest context (0 = unknown).
void batch_decode_csr(torch::Tensor query, torch::Tensor k_cache, torch::Tensor v_cache,
                      torch::Tensor paged_kv_indptr, torch::Tensor paged_kv_indices,
                      torch::Tensor paged_kv_last_page_len, int64_t window_left, double sm_scale,
                      torch::Tensor output, std::optional<torch::Tensor>& output_lse, int64_t max_seq_len,
                      const std::optional<torch::Tensor>& plan = std::nullopt);

// Short query chunks against paged KV: the decode branch of FlashAttentionImpl::paged_forward
// (xllm/core/layers/dcu/flash_attention.cpp:447-545).  query / output packed [T, Hq, D]; kv_seq_lens [B] are the
// context lengths including the chunk, q_cu_seq_lens [B + 1] the chunk boundaries, max_query_len the bound on
// the chunk lengths (AttentionMetadata::max_query_len; 0 = unknown).
void paged_forward(const torch::Tensor& query, torch::Tensor& output, const torch::Tensor& k_cache,
                   const torch::Tensor& v_cache, const torch::Tensor& block_table,
                   const torch::Tensor& kv_seq_lens, const torch::Tensor& q_cu_seq_lens, float scale,
                   bool is_causal, int64_t max_seq_len, int64_t max_query_len, int64_t window_left = -1,
                   const std::optional<torch::Tensor>& k_cache_quant_scale = std::nullopt,
                   const std::optional<torch::Tensor>& v_cache_quant_scale = std::nullopt);

// xllm::kernel::cuda::lse_combine (xllm/core/kernels/cuda/xattention/xattention_ops_api.h:38,
// lse_combine.cu:99-166), same arguments: the two-way combine with BASE-2 LSEs [B, H, 1] fp32.
void lse_combine(torch::Tensor output, torch::Tensor shared_o, torch::Tensor shared_lse, torch::Tensor unshared_o,
                 torch::Tensor unshared_lse);

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

}  // namespace mi355

// The reference's own namespace, types and signature (xllm/core/kernels/dcu/flash_mla_adapter.h:29-53): a caller
// such as DeepseekV2AttentionImpl::decode_flash_mla (layers/dcu/deepseek_v2_attention.cpp:242-263) compiles against
// this unchanged.
namespace dcu {
namespace flash_mla {

enum class DenseDecodeKind {
  kQNopePe,
};

// Inputs of the dense MLA decode.
//   q_nope:      [B, S_q, H_q, kv_lora_rank]
//   q_pe:        [B, S_q, H_q, qk_rope_head_dim]
//   k_cache:     [num_blocks, block_size, 1, kv_lora_rank + qk_rope_head_dim]
//   seqlens_k:   [B] int32
//   block_table: [B, max_blocks] int32
struct DenseDecodeParams {
  torch::Tensor q_nope;
  torch::Tensor q_pe;
  torch::Tensor k_cache;
  torch::Tensor seqlens_k;
  torch::Tensor block_table;
  int64_t head_size_v = 0;
  float softmax_scale = -1.0F;
  bool is_causal = false;
  DenseDecodeKind kind = DenseDecodeKind::kQNopePe;
};

// Returns [B, S_q, H_q, head_size_v].  BF16 and FP16.  S_q query tokens per sequence (multi-token speculative
// steps) are folded into the head count as the reference folds them (flash_mla_adapter.cpp:119-123); with
// is_causal and S_q > 1 token j attends to the first seqlens_k - (S_q - 1 - j) tokens.
torch::Tensor dense_decode(DenseDecodeParams& params);
// The same with the natural-log LSE, [B, H_q, S_q] fp32 (the layout of MluMlaDecodeLseTest,
// tests/core/layers/mlu/dcp_attention_merge_test.cpp:127-143, for S_q = 1: [B, H, 1]).
torch::Tensor dense_decode(DenseDecodeParams& params, torch::Tensor* lse);
// The plan of an MLA decode step, made once per step for the dense_decode calls of all layers: the role of
// get_mla_decoding_metadata_dense_fp8, which the reference's adapter calls apart from the decode
// (flash_mla_adapter.cpp:125-130: seqlens_k, num_heads_per_head_k = S_q * H_q, num_heads_k = 1; it returns
// {tile_scheduler_metadata, num_splits}), and of the FlashInfer plan made at layer 0
// (xllm/core/layers/cuda/flashinfer_planinfo.cpp:248-264).  Here the one buffer holds both; `reuse` is a buffer of an
// earlier step (a captured step must keep its address).
std::vector<torch::Tensor> get_mla_decoding_metadata(const torch::Tensor& seqlens_k, const torch::Tensor& block_table,
                                                     int64_t num_heads_per_head_k, int64_t num_heads_k,
                                                     int64_t block_size,
                                                     const std::optional<torch::Tensor>& reuse = std::nullopt);
// dense_decode from that plan (same lengths and table): bit-identical to the call without it.
torch::Tensor dense_decode(DenseDecodeParams& params, const torch::Tensor& tile_scheduler_metadata, torch::Tensor* lse);
// The decode step of the MLA layer in one call: store_latent_cache(latent_cache, slot_mapping, k_cache) followed by
// decode_flash_mla (xllm/core/layers/dcu/deepseek_v2_attention.cpp:221-229 and :242-263).  latent_cache [B, 576] (or
// [B, 1, 576]) of the query's dtype, slot_mapping [B] int32; one query token per sequence; the plan may be undefined.
// Same cache bytes and output as the two calls.
torch::Tensor store_and_dense_decode(DenseDecodeParams& params, const torch::Tensor& latent_cache,
                                     const torch::Tensor& slot_mapping,
                                     const std::optional<torch::Tensor>& tile_scheduler_metadata, torch::Tensor* lse);

}  // namespace flash_mla
}  // namespace dcu

namespace mi355 {
namespace flash_mla = ::xllm::kernel::dcu::flash_mla;
}  // namespace mi355
}  // namespace xllm::kernel

// Minimal stand-ins for the two types the layer contract takes, with the reference's member names, holding only
// what the decode path reads.
namespace xllm {
// xllm::KVCache (xllm/core/framework/kv_cache/kv_cache.h:29-95): the four accessors of the path.
class KVCache final {
 public:
  KVCache() = default;
  KVCache(torch::Tensor k_cache, torch::Tensor v_cache, std::optional<torch::Tensor> k_cache_scale = std::nullopt,
          std::optional<torch::Tensor> v_cache_scale = std::nullopt)
      : k_cache_(std::move(k_cache)), v_cache_(std::move(v_cache)), k_scale_(std::move(k_cache_scale)),
        v_scale_(std::move(v_cache_scale)) {}
  torch::Tensor get_k_cache() const { return k_cache_; }
  torch::Tensor get_v_cache() const { return v_cache_; }
  std::optional<torch::Tensor> get_k_cache_scale() const { return k_scale_; }
  std::optional<torch::Tensor> get_v_cache_scale() const { return v_scale_; }

 private:
  torch::Tensor k_cache_, v_cache_;
  std::optional<torch::Tensor> k_scale_, v_scale_;
};

namespace layer {
// xllm::layer::PlanInfo (xllm/core/layers/common/attention_metadata.h:49-53): the layer that holds it and the plan
// (here the device buffer of update_decode_plan instead of FlashInfer's integer array; no kernel uri).
struct PlanInfo {
  int32_t layer_id = -1;
  torch::Tensor plan_info;
};

// xllm::layer::AttentionMetadata (xllm/core/layers/common/attention_metadata.h:99-156), decode subset.
struct AttentionMetadata {
  torch::Tensor q_cu_seq_lens;
  torch::Tensor kv_cu_seq_lens;
  torch::Tensor kv_seq_lens;
  torch::Tensor q_seq_lens;
  torch::Tensor block_table;
  torch::Tensor slot_mapping;
  int64_t max_query_len = 1;
  int64_t max_seq_len = 0;
  int64_t total_kv_len = 0;
  std::string compute_dtype;
  bool is_prefill = false;
  bool is_chunked_prefill = false;
  bool is_dummy = false;
  bool is_causal = true;
  torch::Tensor paged_kv_indptr;
  torch::Tensor paged_kv_indices;
  torch::Tensor paged_kv_last_page_len;
  bool enable_cuda_graph = false;
  // attention_metadata.h:163; null: every layer's decode call derives its schedule itself
  std::shared_ptr<PlanInfo> plan_info;
};

namespace flashinfer {
// update_decode_plan_info (xllm/core/layers/cuda/flashinfer_planinfo.cpp:248-264): every layer calls it, layer 0
// plans.  The plan is a launch on the current stream, so a captured step re-plans on every replay and
// enable_cuda_graph needs no host-side update before a replay.
void update_decode_plan_info(std::shared_ptr<PlanInfo> plan_info, const AttentionMetadata& attn_meta,
                             c10::ScalarType key_dtype, int32_t num_qo_heads, int32_t num_kv_heads, int32_t head_dim,
                             int32_t block_size, int32_t window_size_left);
}  // namespace flashinfer

// xllm::layer::BaseAttentionImpl (xllm/core/layers/dcu/base_attention_impl.h:30-57), unchanged.
class BaseAttentionImpl {
 public:
  BaseAttentionImpl(int64_t num_heads, int64_t head_size, float scale, int64_t num_kv_heads, int64_t sliding_window)
      : num_heads_(num_heads), head_size_(head_size), scale_(scale), num_kv_heads_(num_kv_heads),
        sliding_window_(sliding_window) {}
  virtual ~BaseAttentionImpl() = default;
  virtual std::tuple<torch::Tensor, std::optional<torch::Tensor>> forward(const AttentionMetadata& attn_metadata,
                                                                          torch::Tensor& query, torch::Tensor& key,
                                                                          torch::Tensor& value, torch::Tensor& output,
                                                                          KVCache& kv_cache) = 0;

 protected:
  int64_t num_heads_;
  int64_t head_size_;
  float scale_;
  int64_t num_kv_heads_;
  int64_t sliding_window_;
  bool decode_use_tensor_core_ = false;
};

// The MI355X implementation behind that interface: the write-then-attend step of FlashAttentionImpl::forward
// (xllm/core/layers/dcu/flash_attention.cpp:547-660) for decode and for chunked prefill with chunks of up to 16
// tokens, on this library's kernels.  The quantising store is chosen where the cache carries scales
// (xllm/core/layers/mlu/attention.cpp:109-117).  Prefill is not part of this path and throws.
// return_lse: also return the natural-log LSE [tokens, num_heads] fp32 (decode only).
class Mi355AttentionImpl final : public BaseAttentionImpl {
 public:
  Mi355AttentionImpl(int64_t num_heads, int64_t head_size, float scale, int64_t num_kv_heads, int64_t sliding_window,
                     bool return_lse = false)
      : BaseAttentionImpl(num_heads, head_size, scale, num_kv_heads, sliding_window), return_lse_(return_lse) {}
  std::tuple<torch::Tensor, std::optional<torch::Tensor>> forward(const AttentionMetadata& attn_metadata,
                                                                  torch::Tensor& query, torch::Tensor& key,
                                                                  torch::Tensor& value, torch::Tensor& output,
                                                                  KVCache& kv_cache) override;

 private:
  bool return_lse_;
};

// xllm::layer::AttentionImpl (xllm/core/layers/dcu/attention.cpp:28-112): picks the implementation, allocates
// output = empty_like(query) and forwards.
class AttentionImpl final {
 public:
  AttentionImpl(int64_t num_heads, int64_t head_size, float scale, int64_t num_kv_heads, int64_t sliding_window,
                bool return_lse = false)
      : attention_impl_(std::make_shared<Mi355AttentionImpl>(num_heads, head_size, scale, num_kv_heads, sliding_window,
                                                             return_lse)) {}
  std::tuple<torch::Tensor, std::optional<torch::Tensor>> forward(const AttentionMetadata& attn_metadata,
                                                                  torch::Tensor& query, torch::Tensor& key,
                                                                  torch::Tensor& value, KVCache& kv_cache) {
    torch::Tensor output = torch::empty_like(query);
    return attention_impl_->forward(attn_metadata, query, key, value, output, kv_cache);
  }

 private:
  std::shared_ptr<BaseAttentionImpl> attention_impl_;
};
}  // namespace layer
}  // namespace xllm

namespace xllm::layer {
struct DcpAttentionResult {
  torch::Tensor output;
  torch::Tensor lse;
};
// partial_outputs [S, B, Q=1, H, Dv], partial_lse [S, B, H, Q=1] (natural log).
DcpAttentionResult merge_dcp_attention_shards(const torch::Tensor& partial_outputs,
                                              const torch::Tensor& partial_lse);
}  // namespace xllm::layer
