// Internal host-side launchers behind the C ABI of include/xllm_mi355.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/xllm_mi355.h"

namespace xllm_mi355 {

int reshape_and_cache(const void* key, const void* value, void* k_cache, void* v_cache,
                      const int32_t* slot_mapping, const float* k_scale, const float* v_scale,
                      int64_t n_tokens, int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                      int64_t num_blocks, int64_t k_token_stride, int64_t v_token_stride,
                      int in_dtype, int cache_dtype, hipStream_t stream);

int kv_head_scales(const void* x, float* scales, int64_t n_tokens, int64_t n_kv_heads,
                   int64_t head_dim, int64_t token_stride, int in_dtype, hipStream_t stream);

// Addressing of one decode call: block table + seq_lens, or CSR.
struct PageAddressing {
  const int32_t* block_table = nullptr;  // [B, table_stride]
  int64_t table_stride = 0;
  const int32_t* seq_lens = nullptr;     // [B]
  const int32_t* indptr = nullptr;       // CSR when non-null: [B+1]
  const int32_t* indices = nullptr;
  const int32_t* last_page_len = nullptr;
};

// Workspace bytes of the GQA decode (item prefix + two partial slots per persistent workgroup).
size_t gqa_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t head_dim);
// Workspace bytes of the MLA decode for an upper bound of the context length.
size_t mla_workspace_bytes(int64_t batch, int64_t n_heads, int64_t max_seq_len);

int paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache, void* out, float* lse,
                     const PageAddressing& addr, const float* k_scale, const float* v_scale,
                     int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                     int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                     int64_t out_token_stride, int64_t max_seq_len, float sm_scale, void* workspace,
                     size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream);

int paged_decode_mla(const void* q_nope, const void* q_pe, const void* k_cache, void* out, float* lse,
                     const PageAddressing& addr, int64_t batch, int64_t n_heads, int64_t d_latent,
                     int64_t d_rope, int64_t block_size, int64_t num_blocks, int64_t max_seq_len,
                     float sm_scale, void* workspace, size_t workspace_bytes, int dtype,
                     hipStream_t stream);

int lse_merge(const void* partial_out, const float* partial_lse, void* out, float* lse,
              int64_t n_shards, int64_t batch, int64_t n_heads, int64_t v_head_dim, int dtype,
              hipStream_t stream);

int build_block_table(const int32_t* indptr, const int32_t* indices, const int32_t* last_page_len,
                      int32_t* block_table, int64_t table_stride, int32_t* seq_lens, int64_t batch,
                      int64_t block_size, hipStream_t stream);

// Opt-in timing of the dominant kernel (profile.hip).  profile_begin returns true when a
// start event was recorded; the caller then must call profile_end after its launch.
bool profile_begin(hipStream_t stream);
void profile_end(hipStream_t stream);

}  // namespace xllm_mi355
