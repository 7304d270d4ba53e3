// Internal host-side launchers behind the C ABI of include/xllm_mi355.h.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

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
  const int32_t* table_rows = nullptr;   // [B] block-table row of each entry, or null for row b (block-table form only)
  // packed query chunks (block-table form, head dim 128 on the matrix-core kernel only): entry b is a sequence
  // with cu_q[b + 1] - cu_q[b] <= chunk_blocks * (16 / group) query tokens; q / out hold n_tokens rows
  const int32_t* cu_q = nullptr;         // [B + 1]
  int64_t n_tokens = 0;
  int chunk_blocks = 0;
  int causal = 0;
  const int32_t* indptr = nullptr;       // CSR when non-null: [B+1]
  const int32_t* indices = nullptr;
  const int32_t* last_page_len = nullptr;
  // sliding window: the query at position L - 1 attends to positions >= L - 1 - window_left; negative: all
  int64_t window_left = -1;
  // the step's plan (paged_decode_gqa_plan with the same shape, lengths and tables), or null
  const void* plan = nullptr;
};

// Layout of a decode workspace, the same for every decode entry point and independent of the batch, so that
// a launch recorded in a HIP graph keeps meaning the same addresses whatever later calls ask for:
//   [0, kWsHeaderBytes)                 header: word 0 = status flags (kStatus*); from byte kWsCountersOff on,
//                                       one arrival counter per persistent worker (zero between launches)
//   [kWsHeaderBytes, kWsPartialsOff)    item prefix of up to kWsMaxBatch sequences per launch
//   [kWsPartialsOff, ...)               two fp32 partial slots per persistent worker
// (xllm_mi355_decode_workspace_init clears the header.)
constexpr size_t kWsCountersOff = 256;
constexpr int kWsMaxWorkers = 4096;
constexpr size_t kWsHeaderBytes = kWsCountersOff + static_cast<size_t>(kWsMaxWorkers) * 4;
constexpr int kWsMaxBatch = 2048;
constexpr size_t kWsPartialsOff = kWsHeaderBytes + (static_cast<size_t>(kWsMaxBatch + 1) * 4 + 255) / 256 * 256;
constexpr int kStatusWaitGaveUp = 1;  // a bounded wait of one wavefront on another ran out: the launch's output is invalid
constexpr int kStatusPlanMismatch = 2;  // a decode launch was given a plan made for another shape (it wrote no output) or for other lengths

// A plan of a decode step (ints), made once per step and read by the decode launches of every layer.  Word 0: the
// signature of what it was made for | from kPlanPrefixOff the item prefix [batch + 1] of the schedule and, for the GQA
// kernel, the cut between its pools | from kPlanChunksOff 64 page-table entries per team (group of workers of the GQA
// kernel, workgroup team of the MLA kernel): the chunk of the context's table that holds the page of the team's first
// tokens; the tail repeats the context's last page | from kPlanLensOff the context lengths [batch] the plan was made
// with: a planned call compares them with its own, so that a plan that was not made again for a new step is reported
// (kStatusPlanMismatch) instead of followed silently.
constexpr int kPlanPrefixOff = 64;
constexpr int kPlanChunksOff = kPlanPrefixOff + (kWsMaxBatch + 2 + 63) / 64 * 64;
constexpr int kPlanMaxTeams = 4096;
constexpr int kPlanLensOff = kPlanChunksOff + kPlanMaxTeams * 64;
constexpr size_t kPlanBytes = (static_cast<size_t>(kPlanLensOff) + static_cast<size_t>(kWsMaxBatch)) * 4;

// Bound of the polls of one wavefront on another (test hook: xllm_mi355_debug_set_wait_spins).
int wait_spin_limit();

// Workspace bytes of the GQA decode (header + item prefix + two partial slots per persistent worker).
size_t gqa_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t head_dim);
// Workspace bytes of the MLA decode.
size_t mla_workspace_bytes(int64_t batch, int64_t n_heads, int64_t max_seq_len);
// Bytes that serve every GQA call, MLA calls with up to 1024 heads and varlen calls of up to 65536 query tokens.
size_t decode_workspace_bound();
// Clears the header of a workspace (a fill kernel: legal under graph capture).
int decode_workspace_init(void* workspace, size_t workspace_bytes, hipStream_t stream);

// The K / V rows of the step's new tokens, [batch, Hkv, D] of the query's dtype with token strides in elements, and
// their slots [batch]: the decode call writes them to the caches before it attends, as reshape_and_cache would
// (slots outside [0, num_blocks * block_size) are skipped; with fp8 pages the rows are quantised with the call's
// scales).  Sequence b's slot must be the place of its token seq_len - 1 in its table.
struct NewKvRows {
  const void* key = nullptr;
  const void* value = nullptr;
  const int32_t* slots = nullptr;
  int64_t k_token_stride = 0, v_token_stride = 0;
};

int paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache, void* out, float* lse,
                     const PageAddressing& addr, const float* k_scale, const float* v_scale,
                     int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                     int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                     int64_t out_token_stride, int64_t max_seq_len, float sm_scale, void* workspace,
                     size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream,
                     const NewKvRows* fresh = nullptr);

// The plan of a decode step (item prefix, pool cut, first page-table chunk of every group of workers), made
// once and handed to the decode calls of all layers through PageAddressing::plan.
size_t gqa_plan_bytes();
int paged_decode_gqa_plan(void* plan, size_t plan_bytes, const PageAddressing& addr, int64_t batch, int64_t n_q_heads,
                          int64_t n_kv_heads, int64_t head_dim, int64_t block_size, int cache_dtype,
                          hipStream_t stream);

// The plan of an MLA decode step (the same buffer as the GQA plan, for the kernel that serves more than 64 heads).
int paged_decode_mla_plan(void* plan, size_t plan_bytes, const PageAddressing& addr, int64_t batch, int64_t n_heads,
                          int64_t block_size, hipStream_t stream);

// The latent rows of the step's new tokens, [batch] rows of 576 values of the query's dtype (row stride in elements),
// and their slots [batch]: the MLA decode call stores them into the cache before it attends, as reshape_and_cache
// without a value tensor would.  Sequence b's slot must be the place of its token seq_len - 1 in its table.
struct NewLatentRows {
  const void* rows = nullptr;
  const int32_t* slots = nullptr;
  int64_t row_stride = 0;
};

int paged_decode_mla(const void* q_nope, const void* q_pe, const void* k_cache, void* out, float* lse,
                     const PageAddressing& addr, int64_t batch, int64_t n_heads, int64_t d_latent,
                     int64_t d_rope, int64_t block_size, int64_t num_blocks, int64_t max_seq_len,
                     float sm_scale, void* workspace, size_t workspace_bytes, int dtype,
                     hipStream_t stream, const NewLatentRows* fresh = nullptr);

// Several query tokens per sequence (packed q, cu_seqlens_q) through the decode kernels: token j of a
// sequence with q_len tokens attends to the first kv_len - q_len + j + 1 tokens (causal) or to all kv_len.
// The first varlen_extra_bytes(n_tokens) of the workspace hold the per-token lengths and table rows.
size_t varlen_extra_bytes(int64_t n_tokens);
int paged_decode_gqa_varlen(const void* q, const void* k_cache, const void* v_cache, void* out,
                            const int32_t* cu_seqlens_q, const int32_t* kv_seq_lens,
                            const int32_t* block_table, int64_t table_stride, const float* k_scale,
                            const float* v_scale, int64_t batch, int64_t n_tokens, int64_t max_q_len,
                            int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                            int64_t num_blocks, int64_t q_token_stride, int64_t out_token_stride,
                            int64_t max_seq_len, int64_t window_left, float sm_scale, int causal, void* workspace,
                            size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream);

int lse_merge(const void* partial_out, const float* partial_lse, void* out, float* lse,
              int64_t n_shards, int64_t batch, int64_t n_heads, int64_t v_head_dim, int dtype,
              hipStream_t stream);

int lse_combine(void* out, const void* shared_o, const float* shared_lse, const void* unshared_o,
                const float* unshared_lse, int64_t rows, int64_t head_dim, int in_dtype, int out_dtype,
                hipStream_t stream);

int build_block_table(const int32_t* indptr, const int32_t* indices, const int32_t* last_page_len,
                      int32_t* block_table, int64_t table_stride, int32_t* seq_lens, int64_t batch,
                      int64_t block_size, hipStream_t stream);

int mask_block_table_padding(const int32_t* block_table, int64_t table_stride, const int32_t* kv_seq_lens,
                             int32_t* out, int64_t out_stride, int64_t batch, int64_t width, int64_t block_size,
                             hipStream_t stream);

int gather_paged_rows(const void* cache, const int32_t* block_table, int64_t table_stride,
                      const int32_t* cu_seq_lens, void* out, int64_t batch, int64_t total_rows,
                      int64_t block_size, int64_t num_blocks, int64_t row_bytes, hipStream_t stream);

// y[t, h, :] = x[t, h, :] . w[h, :, :]: the absorbed MLA products (strides in elements)
int absorbed_bmm(const void* x, const void* w, void* y, int64_t n_tokens, int64_t n_heads, int64_t k, int64_t n,
                 int64_t x_token_stride, int64_t x_head_stride, int64_t y_token_stride, int64_t y_head_stride,
                 int dtype, hipStream_t stream);

int rope_and_cache(void* qkv, const void* q_weight, const void* k_weight, const void* cos_sin_cache,
                   const int64_t* position_ids, void* k_cache, void* v_cache, const int32_t* slot_mapping,
                   const float* k_scale, const float* v_scale, int64_t n_tokens, int64_t token_stride,
                   int64_t n_heads_q, int64_t n_heads_k, int64_t n_heads_v, int64_t head_dim, int64_t rotary_dim,
                   float eps, int interleave, int64_t block_size, int64_t num_blocks, int dtype, int cos_sin_dtype,
                   int cache_dtype, hipStream_t stream);

int decode_metadata_update(const int32_t* src_tokens, const int32_t* src_positions, const int32_t* src_new_cache_slots,
                           const int32_t* src_kv_seq_lens, const int32_t* src_paged_kv_indptr,
                           const int32_t* src_paged_kv_indices, const int32_t* src_paged_kv_last_page_len,
                           int32_t* dst_tokens, int32_t* dst_positions, int32_t* dst_new_cache_slots,
                           int32_t* dst_kv_seq_lens, int32_t* dst_kv_seq_lens_delta, int32_t* dst_paged_kv_indptr,
                           int32_t* dst_paged_kv_indices, int32_t* dst_paged_kv_last_page_len,
                           int64_t actual_num_tokens, int64_t padded_num_tokens, int64_t actual_batch_size,
                           int64_t actual_indices_size, hipStream_t stream);

// Kernel attributes (dynamic LDS size) are set per device.  Returns true the first time it is called with
// `seen` on the current device (devices 0..63; beyond that always true: setting them again is harmless).
inline bool first_use_on_current_device(std::atomic<uint64_t>& seen) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) return true;
  const uint64_t bit = 1ull << dev;
  if ((seen.load(std::memory_order_acquire) & bit) != 0) return false;
  seen.fetch_or(bit, std::memory_order_acq_rel);
  return true;
}

// Compute units of the current device, looked up once per device (a process may drive several GPUs, and they need
// not be alike).  256 if the runtime cannot say.
inline int device_cu_count() {
  static std::atomic<int> cached[64];  // zero-initialised; 0 = not looked up yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  const bool slot = dev >= 0 && dev < 64;
  if (slot) {
    const int n = cached[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
  }
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  if (slot) cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

// Opt-in timing of the dominant kernel (profile.hip).  While it is enabled, launch_timed hands the launch
// a pair of HIP events that the runtime fills with the kernel's own start and end (the time stamps of
// the dispatch, the ones a profiler reports): events recorded on the stream before and after the launch
// would also count the 2-3 us each that their own packets take, 5 % of a 100 us kernel.
bool profile_events(hipEvent_t* start, hipEvent_t* stop);
void profile_commit();
// A launch that a caller of xllm_mi355_profile_collect counts on did not take place (its work was done by the
// launch before): recorded as an entry of 0 ms.
void profile_skip();

template <typename Kernel, typename... Args>
inline void launch_timed(Kernel kernel, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream, Args... args) {
  hipEvent_t start, stop;
  if (profile_events(&start, &stop)) {
    hipExtLaunchKernelGGL(kernel, grid, block, static_cast<uint32_t>(lds_bytes), stream, start, stop, 0, args...);
    profile_commit();
  } else {
    kernel<<<grid, block, lds_bytes, stream>>>(args...);
  }
}

}  // namespace xllm_mi355
