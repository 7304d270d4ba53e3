// extern "C" surface of libxllm_mi355.so: plain pointers and sizes in, enqueue only.
#include "launch.h"

#include <mutex>

using namespace xllm_mi355;

namespace xllm_mi355 {
namespace {
constexpr int kDefaultWaitSpins = 1 << 22;
std::atomic<int> g_wait_spins{kDefaultWaitSpins};
}  // namespace
int wait_spin_limit() { return g_wait_spins.load(std::memory_order_relaxed); }
void set_mla_kernel_knob(int first_letter);  // paged_decode_mla.hip
void set_fold_merge(int on);                 // paged_decode_gqa.hip
void set_stream_stores(int v);               // paged_decode_gqa.hip
void set_mla_fold(int on);                   // paged_decode_mla.hip
}  // namespace xllm_mi355

// Scratch of xllm_mi355_paged_decode_gqa_static: a decode workspace that lives in the code object, one copy
// per GPU that loads the library, held until the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; kernels and fills take the per-device address kept in static_scratch().
constexpr size_t kStaticScratchBytes = XLLM_MI355_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
// The device address of `scratch` on the current device, looked up once per device.
int static_scratch(void** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kMaxDevices) return XLLM_MI355_EINVAL;
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 255) != 0) return XLLM_MI355_EWORKSPACE;
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return XLLM_MI355_OK;
}
}  // namespace

extern "C" {

const char* xllm_mi355_version(void) { return "0.1.0"; }

const char* xllm_mi355_error_string(int code) {
  switch (code) {
    case XLLM_MI355_OK: return "ok";
    case XLLM_MI355_EINVAL: return "invalid argument (null pointer, non-positive size or bad stride)";
    case XLLM_MI355_EDTYPE: return "dtype combination not implemented";
    case XLLM_MI355_ESHAPE: return "head dim, group size or block size not implemented";
    case XLLM_MI355_EWORKSPACE: return "split-K workspace missing, misaligned or too small";
    case XLLM_MI355_EALIGN: return "pointer or stride not 16-byte aligned";
    case XLLM_MI355_ESTALLED: return "a bounded wait inside a decode kernel gave up: the outputs of that launch are invalid";
    case XLLM_MI355_EPLAN: return "a decode launch was given a plan made for another shape or for other sequence lengths: its output is invalid";
    case XLLM_MI355_ESCRATCH: return "the problem needs more scratch than the static scratch of the no-allocation entry point holds";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}

int xllm_mi355_reshape_and_cache(const void* key, const void* value, void* k_cache, void* v_cache,
                                 const int32_t* slot_mapping, const float* k_scale,
                                 const float* v_scale, int64_t n_tokens, int64_t n_kv_heads,
                                 int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                 int64_t k_token_stride, int64_t v_token_stride, int in_dtype,
                                 int cache_dtype, void* stream) {
  return reshape_and_cache(key, value, k_cache, v_cache, slot_mapping, k_scale, v_scale, n_tokens,
                           n_kv_heads, head_dim, block_size, num_blocks, k_token_stride,
                           v_token_stride, in_dtype, cache_dtype, static_cast<hipStream_t>(stream));
}

int xllm_mi355_kv_head_scales(const void* x, float* scales, int64_t n_tokens, int64_t n_kv_heads,
                              int64_t head_dim, int64_t token_stride, int in_dtype, void* stream) {
  return kv_head_scales(x, scales, n_tokens, n_kv_heads, head_dim, token_stride, in_dtype,
                        static_cast<hipStream_t>(stream));
}

size_t xllm_mi355_paged_decode_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t v_head_dim,
                                               int64_t max_seq_len) {
  if (batch <= 0 || n_q_heads <= 0 || v_head_dim <= 0) return 0;
  // (kept for callers written against the first version of this header, which asked for both variants here: a width
  // of 512 meant the MLA latent; new code asks xllm_mi355_paged_decode_mla_workspace_bytes for that)
  if (v_head_dim == 512) return mla_workspace_bytes(batch, n_q_heads, max_seq_len);
  return gqa_workspace_bytes(batch, n_q_heads, v_head_dim);
}

size_t xllm_mi355_paged_decode_gqa_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t head_dim) {
  if (batch <= 0 || n_q_heads <= 0 || head_dim <= 0) return 0;
  return gqa_workspace_bytes(batch, n_q_heads, head_dim);
}

size_t xllm_mi355_paged_decode_mla_workspace_bytes(int64_t batch, int64_t n_heads, int64_t max_seq_len) {
  if (batch <= 0 || n_heads <= 0) return 0;
  return mla_workspace_bytes(batch, n_heads, max_seq_len);
}

size_t xllm_mi355_decode_workspace_bound(void) { return decode_workspace_bound(); }

int xllm_mi355_decode_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
  return decode_workspace_init(workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int xllm_mi355_decode_status(void* workspace, void* stream) {
  if (workspace == nullptr) {
    const int rc = static_scratch(&workspace);
    if (rc != 0) return rc;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  int status = 0;
  hipError_t e = hipMemcpyAsync(&status, workspace, sizeof(int), hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  if (e != hipSuccess) return static_cast<int>(e);
  if (status == 0) return XLLM_MI355_OK;
  // the launch that gave up may also have left arrival counters behind: the whole header starts over
  const int rc = decode_workspace_init(workspace, kWsHeaderBytes, s);
  if (rc != 0) return rc;
  e = hipStreamSynchronize(s);
  if (e != hipSuccess) return static_cast<int>(e);
  return (status & kStatusWaitGaveUp) != 0 ? XLLM_MI355_ESTALLED : XLLM_MI355_EPLAN;
}

int xllm_mi355_debug_set(int what, int value) {
  switch (what) {
    case XLLM_MI355_DEBUG_WAIT_SPINS:
      g_wait_spins.store(value < 0 ? kDefaultWaitSpins : value, std::memory_order_relaxed);
      return XLLM_MI355_OK;
    case XLLM_MI355_DEBUG_MLA_KERNEL:
      set_mla_kernel_knob(value);
      return XLLM_MI355_OK;
    case XLLM_MI355_DEBUG_GQA_FOLD:
      set_fold_merge(value);
      return XLLM_MI355_OK;
    case XLLM_MI355_DEBUG_GQA_STREAM_STORES:
      set_stream_stores(value);
      return XLLM_MI355_OK;
    case XLLM_MI355_DEBUG_MLA_FOLD:
      set_mla_fold(value);
      return XLLM_MI355_OK;
    default: return XLLM_MI355_EINVAL;
  }
}

int xllm_mi355_paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache, void* out,
                                float* lse, const int32_t* block_table, int64_t table_stride,
                                const int32_t* seq_lens, const float* k_scale, const float* v_scale,
                                int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                                int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                                int64_t out_token_stride, int64_t max_seq_len, int64_t window_left, float sm_scale,
                                void* workspace, size_t workspace_bytes, int q_dtype, int cache_dtype,
                                void* stream) {
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = seq_lens;
  addr.window_left = window_left;
  return paged_decode_gqa(q, k_cache, v_cache, out, lse, addr, k_scale, v_scale, batch, n_q_heads,
                          n_kv_heads, head_dim, block_size, num_blocks, q_token_stride,
                          out_token_stride, max_seq_len, sm_scale, workspace, workspace_bytes, q_dtype,
                          cache_dtype, static_cast<hipStream_t>(stream));
}

int xllm_mi355_paged_decode_gqa_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       float* lse, const int32_t* block_table, int64_t table_stride,
                                       const int32_t* seq_lens, const float* k_scale, const float* v_scale,
                                       int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                                       int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                                       int64_t out_token_stride, int64_t max_seq_len, int64_t window_left,
                                       float sm_scale, int q_dtype, int cache_dtype, void* stream) {
  if (batch > kWsMaxBatch) return XLLM_MI355_ESCRATCH;  // (a longer batch would be decoded in slices that share the scratch)
  void* ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc != 0) return rc;
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = seq_lens;
  addr.window_left = window_left;
  rc = paged_decode_gqa(q, k_cache, v_cache, out, lse, addr, k_scale, v_scale, batch, n_q_heads, n_kv_heads,
                        head_dim, block_size, num_blocks, q_token_stride, out_token_stride, max_seq_len, sm_scale,
                        ws, kStaticScratchBytes, q_dtype, cache_dtype, static_cast<hipStream_t>(stream));
  return rc == XLLM_MI355_EWORKSPACE ? XLLM_MI355_ESCRATCH : rc;
}

int xllm_mi355_paged_decode_gqa_csr(const void* q, const void* k_cache, const void* v_cache, void* out,
                                    float* lse, const int32_t* paged_kv_indptr,
                                    const int32_t* paged_kv_indices,
                                    const int32_t* paged_kv_last_page_len, const float* k_scale,
                                    const float* v_scale, int64_t batch, int64_t n_q_heads,
                                    int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                                    int64_t num_blocks, int64_t q_token_stride,
                                    int64_t out_token_stride, int64_t max_seq_len, int64_t window_left,
                                    float sm_scale, void* workspace, size_t workspace_bytes, int q_dtype,
                                    int cache_dtype, void* stream) {
  if (paged_kv_indptr == nullptr) return XLLM_MI355_EINVAL;
  PageAddressing addr;
  addr.window_left = window_left;
  addr.indptr = paged_kv_indptr;
  addr.indices = paged_kv_indices;
  addr.last_page_len = paged_kv_last_page_len;
  return paged_decode_gqa(q, k_cache, v_cache, out, lse, addr, k_scale, v_scale, batch, n_q_heads,
                          n_kv_heads, head_dim, block_size, num_blocks, q_token_stride,
                          out_token_stride, max_seq_len, sm_scale, workspace, workspace_bytes, q_dtype,
                          cache_dtype, static_cast<hipStream_t>(stream));
}

size_t xllm_mi355_paged_decode_plan_bytes(void) { return gqa_plan_bytes(); }

int xllm_mi355_paged_decode_gqa_plan(void* plan, size_t plan_bytes, const int32_t* block_table,
                                     int64_t table_stride, const int32_t* seq_lens,
                                     const int32_t* paged_kv_indptr, const int32_t* paged_kv_indices,
                                     const int32_t* paged_kv_last_page_len, int64_t batch, int64_t n_q_heads,
                                     int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                                     int64_t window_left, int cache_dtype, void* stream) {
  PageAddressing addr;
  addr.window_left = window_left;
  if (paged_kv_indptr != nullptr) {
    addr.indptr = paged_kv_indptr;
    addr.indices = paged_kv_indices;
    addr.last_page_len = paged_kv_last_page_len;
  } else {
    addr.block_table = block_table;
    addr.table_stride = table_stride;
    addr.seq_lens = seq_lens;
  }
  return paged_decode_gqa_plan(plan, plan_bytes, addr, batch, n_q_heads, n_kv_heads, head_dim, block_size,
                               cache_dtype, static_cast<hipStream_t>(stream));
}

int xllm_mi355_write_and_decode_gqa(const void* key, const void* value, const int32_t* slot_mapping,
                                    int64_t k_token_stride, int64_t v_token_stride, const void* plan, size_t plan_bytes,
                                    const void* q, void* k_cache, void* v_cache, void* out, float* lse,
                                    const int32_t* block_table, int64_t table_stride, const int32_t* seq_lens,
                                    const int32_t* paged_kv_indptr, const int32_t* paged_kv_indices,
                                    const int32_t* paged_kv_last_page_len, const float* k_scale, const float* v_scale,
                                    int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                                    int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                                    int64_t out_token_stride, int64_t max_seq_len, int64_t window_left, float sm_scale,
                                    void* workspace, size_t workspace_bytes, int q_dtype, int cache_dtype,
                                    void* stream) {
  if (key == nullptr || value == nullptr || slot_mapping == nullptr) return XLLM_MI355_EINVAL;
  if (k_token_stride < n_kv_heads * head_dim || v_token_stride < n_kv_heads * head_dim) return XLLM_MI355_EINVAL;
  if (plan != nullptr && plan_bytes < gqa_plan_bytes()) return XLLM_MI355_EWORKSPACE;
  PageAddressing addr;
  addr.window_left = window_left;
  addr.plan = plan;
  if (paged_kv_indptr != nullptr) {
    addr.indptr = paged_kv_indptr;
    addr.indices = paged_kv_indices;
    addr.last_page_len = paged_kv_last_page_len;
  } else {
    addr.block_table = block_table;
    addr.table_stride = table_stride;
    addr.seq_lens = seq_lens;
  }
  NewKvRows fresh;
  fresh.key = key;
  fresh.value = value;
  fresh.slots = slot_mapping;
  fresh.k_token_stride = k_token_stride;
  fresh.v_token_stride = v_token_stride;
  return paged_decode_gqa(q, k_cache, v_cache, out, lse, addr, k_scale, v_scale, batch, n_q_heads, n_kv_heads,
                          head_dim, block_size, num_blocks, q_token_stride, out_token_stride, max_seq_len, sm_scale,
                          workspace, workspace_bytes, q_dtype, cache_dtype, static_cast<hipStream_t>(stream), &fresh);
}

int xllm_mi355_paged_decode_gqa_planned(const void* plan, size_t plan_bytes, const void* q, const void* k_cache,
                                        const void* v_cache, void* out, float* lse,
                                        const int32_t* block_table, int64_t table_stride,
                                        const int32_t* seq_lens, const int32_t* paged_kv_indptr,
                                        const int32_t* paged_kv_indices,
                                        const int32_t* paged_kv_last_page_len, const float* k_scale,
                                        const float* v_scale, int64_t batch, int64_t n_q_heads,
                                        int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                                        int64_t num_blocks, int64_t q_token_stride, int64_t out_token_stride,
                                        int64_t max_seq_len, int64_t window_left, float sm_scale,
                                        void* workspace, size_t workspace_bytes, int q_dtype, int cache_dtype,
                                        void* stream) {
  if (plan == nullptr) return XLLM_MI355_EINVAL;
  // (the kernels read the plan up to its last word before they look at its signature)
  if (plan_bytes < gqa_plan_bytes()) return XLLM_MI355_EWORKSPACE;
  PageAddressing addr;
  addr.window_left = window_left;
  addr.plan = plan;
  if (paged_kv_indptr != nullptr) {
    addr.indptr = paged_kv_indptr;
    addr.indices = paged_kv_indices;
    addr.last_page_len = paged_kv_last_page_len;
  } else {
    addr.block_table = block_table;
    addr.table_stride = table_stride;
    addr.seq_lens = seq_lens;
  }
  return paged_decode_gqa(q, k_cache, v_cache, out, lse, addr, k_scale, v_scale, batch, n_q_heads, n_kv_heads,
                          head_dim, block_size, num_blocks, q_token_stride, out_token_stride, max_seq_len, sm_scale,
                          workspace, workspace_bytes, q_dtype, cache_dtype, static_cast<hipStream_t>(stream));
}

int xllm_mi355_gather_paged_rows(const void* cache, const int32_t* block_table, int64_t table_stride,
                                 const int32_t* cu_seq_lens, void* out, int64_t batch, int64_t total_rows,
                                 int64_t block_size, int64_t num_blocks, int64_t row_bytes, void* stream) {
  return gather_paged_rows(cache, block_table, table_stride, cu_seq_lens, out, batch, total_rows, block_size,
                           num_blocks, row_bytes, static_cast<hipStream_t>(stream));
}

int xllm_mi355_mask_block_table_padding(const int32_t* block_table, int64_t table_stride, const int32_t* kv_seq_lens,
                                        int32_t* out, int64_t out_stride, int64_t batch, int64_t width,
                                        int64_t block_size, void* stream) {
  return mask_block_table_padding(block_table, table_stride, kv_seq_lens, out, out_stride, batch, width, block_size,
                                  static_cast<hipStream_t>(stream));
}

int xllm_mi355_mla_absorbed_bmm(const void* x, const void* w, void* y, int64_t n_tokens, int64_t n_heads,
                                int64_t k, int64_t n, int64_t x_token_stride, int64_t x_head_stride,
                                int64_t y_token_stride, int64_t y_head_stride, int dtype, void* stream) {
  return absorbed_bmm(x, w, y, n_tokens, n_heads, k, n, x_token_stride, x_head_stride, y_token_stride,
                      y_head_stride, dtype, static_cast<hipStream_t>(stream));
}

size_t xllm_mi355_paged_decode_varlen_workspace_bytes(int64_t n_tokens, int64_t n_q_heads, int64_t head_dim) {
  if (n_tokens <= 0 || n_q_heads <= 0 || head_dim <= 0) return 0;
  return gqa_workspace_bytes(n_tokens, n_q_heads, head_dim) + varlen_extra_bytes(n_tokens) + 256;
}

int xllm_mi355_paged_decode_gqa_varlen(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       const int32_t* cu_seqlens_q, const int32_t* kv_seq_lens,
                                       const int32_t* block_table, int64_t table_stride,
                                       const float* k_scale, const float* v_scale, int64_t batch,
                                       int64_t n_tokens, int64_t max_q_len, int64_t n_q_heads, int64_t n_kv_heads,
                                       int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                       int64_t q_token_stride, int64_t out_token_stride,
                                       int64_t max_seq_len, int64_t window_left, float sm_scale, int causal,
                                       void* workspace, size_t workspace_bytes, int q_dtype, int cache_dtype,
                                       void* stream) {
  return paged_decode_gqa_varlen(q, k_cache, v_cache, out, cu_seqlens_q, kv_seq_lens, block_table,
                                 table_stride, k_scale, v_scale, batch, n_tokens, max_q_len, n_q_heads, n_kv_heads,
                                 head_dim, block_size, num_blocks, q_token_stride, out_token_stride,
                                 max_seq_len, window_left, sm_scale, causal, workspace, workspace_bytes, q_dtype,
                                 cache_dtype, static_cast<hipStream_t>(stream));
}

int xllm_mi355_paged_decode_mla(const void* q_nope, const void* q_pe, const void* k_cache, void* out,
                                float* lse, const int32_t* block_table, int64_t table_stride,
                                const int32_t* seq_lens, int64_t batch, int64_t n_heads,
                                int64_t d_latent, int64_t d_rope, int64_t block_size,
                                int64_t num_blocks, int64_t max_seq_len, float sm_scale,
                                void* workspace, size_t workspace_bytes, int dtype, void* stream) {
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = seq_lens;
  return paged_decode_mla(q_nope, q_pe, k_cache, out, lse, addr, batch, n_heads, d_latent, d_rope,
                          block_size, num_blocks, max_seq_len, sm_scale, workspace, workspace_bytes,
                          dtype, static_cast<hipStream_t>(stream));
}

int xllm_mi355_paged_decode_mla_plan(void* plan, size_t plan_bytes, const int32_t* block_table, int64_t table_stride,
                                     const int32_t* seq_lens, int64_t batch, int64_t n_heads, int64_t block_size,
                                     void* stream) {
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = seq_lens;
  return paged_decode_mla_plan(plan, plan_bytes, addr, batch, n_heads, block_size, static_cast<hipStream_t>(stream));
}

int xllm_mi355_write_and_decode_mla(const void* new_latent, const int32_t* slot_mapping, int64_t latent_row_stride,
                                    const void* plan, size_t plan_bytes, const void* q_nope, const void* q_pe,
                                    void* k_cache, void* out, float* lse, const int32_t* block_table,
                                    int64_t table_stride, const int32_t* seq_lens, int64_t batch, int64_t n_heads,
                                    int64_t d_latent, int64_t d_rope, int64_t block_size, int64_t num_blocks,
                                    int64_t max_seq_len, float sm_scale, void* workspace, size_t workspace_bytes,
                                    int dtype, void* stream) {
  if (new_latent == nullptr || slot_mapping == nullptr || latent_row_stride < d_latent + d_rope) return XLLM_MI355_EINVAL;
  if (plan != nullptr && plan_bytes < gqa_plan_bytes()) return XLLM_MI355_EWORKSPACE;
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = seq_lens;
  addr.plan = plan;
  NewLatentRows fresh;
  fresh.rows = new_latent;
  fresh.slots = slot_mapping;
  fresh.row_stride = latent_row_stride;
  return paged_decode_mla(q_nope, q_pe, k_cache, out, lse, addr, batch, n_heads, d_latent, d_rope, block_size,
                          num_blocks, max_seq_len, sm_scale, workspace, workspace_bytes, dtype,
                          static_cast<hipStream_t>(stream), &fresh);
}

int xllm_mi355_paged_decode_mla_planned(const void* plan, size_t plan_bytes, const void* q_nope, const void* q_pe,
                                        const void* k_cache, void* out, float* lse, const int32_t* block_table,
                                        int64_t table_stride, const int32_t* seq_lens, int64_t batch, int64_t n_heads,
                                        int64_t d_latent, int64_t d_rope, int64_t block_size, int64_t num_blocks,
                                        int64_t max_seq_len, float sm_scale, void* workspace, size_t workspace_bytes,
                                        int dtype, void* stream) {
  if (plan == nullptr) return XLLM_MI355_EINVAL;
  // (the kernel reads the plan up to its last word before it looks at its signature)
  if (plan_bytes < gqa_plan_bytes()) return XLLM_MI355_EWORKSPACE;
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = seq_lens;
  addr.plan = plan;
  return paged_decode_mla(q_nope, q_pe, k_cache, out, lse, addr, batch, n_heads, d_latent, d_rope, block_size,
                          num_blocks, max_seq_len, sm_scale, workspace, workspace_bytes, dtype,
                          static_cast<hipStream_t>(stream));
}

int xllm_mi355_lse_merge(const void* partial_out, const float* partial_lse, void* out, float* lse,
                         int64_t n_shards, int64_t batch, int64_t n_heads, int64_t v_head_dim,
                         int dtype, void* stream) {
  return lse_merge(partial_out, partial_lse, out, lse, n_shards, batch, n_heads, v_head_dim, dtype,
                   static_cast<hipStream_t>(stream));
}

int xllm_mi355_lse_combine(void* out, const void* shared_o, const float* shared_lse, const void* unshared_o,
                           const float* unshared_lse, int64_t rows, int64_t head_dim, int in_dtype, int out_dtype,
                           void* stream) {
  return lse_combine(out, shared_o, shared_lse, unshared_o, unshared_lse, rows, head_dim, in_dtype, out_dtype,
                     static_cast<hipStream_t>(stream));
}

int xllm_mi355_rope_and_cache(void* qkv, const void* q_weight, const void* k_weight, const void* cos_sin_cache,
                              const int64_t* position_ids, void* k_cache, void* v_cache,
                              const int32_t* slot_mapping, const float* k_scale, const float* v_scale,
                              int64_t n_tokens, int64_t token_stride, int64_t n_heads_q, int64_t n_heads_k,
                              int64_t n_heads_v, int64_t head_dim, int64_t rotary_dim, float eps, int interleave,
                              int64_t block_size, int64_t num_blocks, int dtype, int cos_sin_dtype, int cache_dtype,
                              void* stream) {
  return rope_and_cache(qkv, q_weight, k_weight, cos_sin_cache, position_ids, k_cache, v_cache, slot_mapping, k_scale,
                        v_scale, n_tokens, token_stride, n_heads_q, n_heads_k, n_heads_v, head_dim, rotary_dim, eps,
                        interleave, block_size, num_blocks, dtype, cos_sin_dtype, cache_dtype,
                        static_cast<hipStream_t>(stream));
}

int xllm_mi355_decode_metadata_update(const int32_t* src_tokens, const int32_t* src_positions,
                                      const int32_t* src_new_cache_slots, const int32_t* src_kv_seq_lens,
                                      const int32_t* src_paged_kv_indptr, const int32_t* src_paged_kv_indices,
                                      const int32_t* src_paged_kv_last_page_len, int32_t* dst_tokens,
                                      int32_t* dst_positions, int32_t* dst_new_cache_slots, int32_t* dst_kv_seq_lens,
                                      int32_t* dst_kv_seq_lens_delta, int32_t* dst_paged_kv_indptr,
                                      int32_t* dst_paged_kv_indices, int32_t* dst_paged_kv_last_page_len,
                                      int64_t actual_num_tokens, int64_t padded_num_tokens, int64_t actual_batch_size,
                                      int64_t actual_indices_size, void* stream) {
  return decode_metadata_update(src_tokens, src_positions, src_new_cache_slots, src_kv_seq_lens, src_paged_kv_indptr,
                                src_paged_kv_indices, src_paged_kv_last_page_len, dst_tokens, dst_positions,
                                dst_new_cache_slots, dst_kv_seq_lens, dst_kv_seq_lens_delta, dst_paged_kv_indptr,
                                dst_paged_kv_indices, dst_paged_kv_last_page_len, actual_num_tokens, padded_num_tokens,
                                actual_batch_size, actual_indices_size, static_cast<hipStream_t>(stream));
}

int xllm_mi355_build_block_table(const int32_t* paged_kv_indptr, const int32_t* paged_kv_indices,
                                 const int32_t* paged_kv_last_page_len, int32_t* block_table,
                                 int64_t table_stride, int32_t* seq_lens, int64_t batch,
                                 int64_t block_size, void* stream) {
  return build_block_table(paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len, block_table,
                           table_stride, seq_lens, batch, block_size, static_cast<hipStream_t>(stream));
}

}  // extern "C"
