// Small data-movement kernels either side of the decode kernels:
//   lse_merge          -- log-sum-exp merge of S partial attention results
//                         (xllm/core/layers/mlu/dcp_attention_merge.cpp:26-65)
//   build_block_table  -- CSR page lists -> padded [B, stride] table, -1 fill
//                         (xllm/core/kernels/dcu/build_block_table_from_paged_kv.hip:44-149)
//   gather_paged_rows  -- rows of paged sequences -> one packed [total_rows, row_bytes] buffer, sequence after
//                         sequence (xllm/core/kernels/dcu/gather_mla_latent_cache.hip:32-75: the latent rows
//                         of the context for prefill with context)
//   decode_metadata_update -- a step's metadata into the persistent buffers of a captured step, padded
//                         (xllm/core/kernels/cuda/llm_decode_metadata_update.cu:27-71)
//   expand_varlen      -- per query token of a packed batch: attended length and block-table row, so that
//                         short query chunks run through the decode kernels
//                         (xllm/core/layers/dcu/flash_attention.cpp:447-545, the hg_prefix_decode_varlen_fwd branch)
#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

// One workgroup per (batch, head).  natural-log LSE in and out, fp32 arithmetic in the
// order of the reference: max over shards, weights exp(lse - max) with non-finite
// shards weighted 0, weighted sum, division by the weight sum.
template <int DT>
__global__ __launch_bounds__(128) void lse_merge_kernel(const char* partial_out,
                                                        const float* partial_lse, char* out,
                                                        float* lse, int n_shards, int64_t bh, int dv) {
  constexpr int ES = DT == XLLM_MI355_FP32 ? 4 : 2;
  const int64_t i = blockIdx.x;
  float mx = -INFINITY;
  for (int s = 0; s < n_shards; ++s) mx = fmaxf(mx, partial_lse[s * bh + i]);
  const float safe_max = isfinite(mx) ? mx : 0.0f;
  float wsum = 0.0f;
  for (int s = 0; s < n_shards; ++s) {
    const float v = partial_lse[s * bh + i];
    wsum += isfinite(v) ? expf(v - safe_max) : 0.0f;
  }
  for (int d = threadIdx.x; d < dv; d += 128) {
    float o = 0.0f;
    for (int s = 0; s < n_shards; ++s) {
      const float v = partial_lse[s * bh + i];
      const float w = isfinite(v) ? expf(v - safe_max) : 0.0f;
      const char* p = partial_out + ((s * bh + i) * dv + d) * ES;
      float x;
      if constexpr (DT == XLLM_MI355_FP32) x = *reinterpret_cast<const float*>(p);
      else if constexpr (DT == XLLM_MI355_BF16) x = BF16::to_f32(*reinterpret_cast<const uint16_t*>(p));
      else x = FP16::to_f32(*reinterpret_cast<const uint16_t*>(p));
      o += x * w;
    }
    const float val = wsum > 0.0f ? o / wsum : 0.0f;
    char* q = out + (i * dv + d) * ES;
    if constexpr (DT == XLLM_MI355_FP32) *reinterpret_cast<float*>(q) = val;
    else if constexpr (DT == XLLM_MI355_BF16) *reinterpret_cast<uint16_t*>(q) = BF16::from_f32(val);
    else *reinterpret_cast<uint16_t*>(q) = FP16::from_f32(val);
  }
  if (lse != nullptr && threadIdx.x == 0) lse[i] = wsum > 0.0f ? safe_max + logf(wsum) : -INFINITY;
}

// Two-way combine with base-2 LSEs, one workgroup per (batch, head) row, the arithmetic of the reference kernel
// in its order (xllm/core/kernels/cuda/xattention/lse_combine.cu:41-85): maximum, exp2 of both against it, merged
// LSE = max + log2(sum), weights exp2(lse - merged), weighted sum, one rounding to the output type.
template <int IN, int OUT>
__global__ __launch_bounds__(128) void lse_combine_kernel(char* out, const char* shared_o, const float* shared_lse,
                                                          const char* unshared_o, const float* unshared_lse, int d_total) {
  const int64_t idx = blockIdx.x;
  const float a = shared_lse[idx], b = unshared_lse[idx];
  const float lse_max = fmaxf(a, b);
  const float ea = exp2f(a - lse_max), eb = exp2f(b - lse_max);
  const float lse_new = lse_max + log2f(ea + eb);
  const float wa = exp2f(a - lse_new), wb = exp2f(b - lse_new);
  auto load = [](const char* p, int64_t i) -> float {
    if constexpr (IN == XLLM_MI355_FP32) return reinterpret_cast<const float*>(p)[i];
    else if constexpr (IN == XLLM_MI355_BF16) return BF16::to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
    else return FP16::to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  };
  for (int d = threadIdx.x; d < d_total; d += 128) {
    const int64_t i = idx * d_total + d;
    const float v = wa * load(shared_o, i) + wb * load(unshared_o, i);
    if constexpr (OUT == XLLM_MI355_FP32) reinterpret_cast<float*>(out)[i] = v;
    else if constexpr (OUT == XLLM_MI355_BF16) reinterpret_cast<uint16_t*>(out)[i] = BF16::from_f32(v);
    else reinterpret_cast<uint16_t*>(out)[i] = FP16::from_f32(v);
  }
}

__global__ __launch_bounds__(256) void build_block_table_kernel(const int32_t* indptr,
                                                                const int32_t* indices,
                                                                const int32_t* last_page_len,
                                                                int32_t* table, int64_t stride,
                                                                int32_t* seq_lens, int block_size) {
  const int b = blockIdx.x;
  const int p0 = indptr[b];
  const int n = indptr[b + 1] - p0;
  for (int64_t j = threadIdx.x; j < stride; j += 256)
    table[b * stride + j] = j < n ? indices[p0 + j] : -1;
  if (seq_lens != nullptr && threadIdx.x == 0)
    seq_lens[b] = n > 0 ? (n - 1) * block_size + last_page_len[b] : 0;
}

// out[b, j] = table[b, j] for the columns a sequence of kv_seq_lens[b] tokens uses, -1 beyond them
// (never by page id: page 0 is a valid page).  In place when out == table.
__global__ __launch_bounds__(256) void mask_block_table_padding_kernel(const int32_t* table, int64_t stride,
                                                                       const int32_t* kv_seq_lens, int32_t* out,
                                                                       int64_t out_stride, int width, int block_size) {
  const int b = blockIdx.x;
  const int64_t len = kv_seq_lens[b];
  const int64_t pages = len > 0 ? (len + block_size - 1) / block_size : 0;
  for (int j = threadIdx.x; j < width; j += 256) out[b * out_stride + j] = j < pages ? table[b * stride + j] : -1;
}

struct MetadataUpdate {
  const int32_t *tokens, *positions, *slots, *kv_cu, *indptr, *indices, *last_page_len;
  int32_t *d_tokens, *d_positions, *d_slots, *d_kv_cu, *d_kv_delta, *d_indptr, *d_indices, *d_last_page_len;
  int64_t n_tokens, n_padded, batch, n_indices;
};
// One thread per index of the longest array.  Integer copies and fills, nothing else: the rules of the
// reference kernel index by index.
__global__ __launch_bounds__(256) void decode_metadata_update_kernel(MetadataUpdate u, int64_t n) {
  const int64_t step = static_cast<int64_t>(gridDim.x) * 256;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += step) {
    if (i < u.n_tokens) {
      u.d_tokens[i] = u.tokens[i];
      u.d_positions[i] = u.positions[i];
      u.d_slots[i] = u.slots[i];
    } else if (i < u.n_padded) {
      u.d_tokens[i] = 0;
      u.d_positions[i] = 0;
      u.d_slots[i] = -1;
    }
    if (i < u.batch + 1) {
      u.d_kv_cu[i] = u.kv_cu[i];
      u.d_indptr[i] = u.indptr[i];
    } else if (i < u.n_padded + 1) {
      u.d_kv_cu[i] = u.kv_cu[u.batch];
      u.d_indptr[i] = u.indptr[u.batch];
    }
    if (i < u.batch) {
      u.d_kv_delta[i] = u.kv_cu[i + 1] - u.kv_cu[i];
      u.d_last_page_len[i] = u.last_page_len[i];
    } else if (i < u.n_padded) {
      u.d_kv_delta[i] = 0;
      u.d_last_page_len[i] = 1;
    }
    if (i < u.n_indices) u.d_indices[i] = u.indices[i];
  }
}

// One thread per query token.  Token t belongs to the sequence b with cu[b] <= t < cu[b + 1]; with q_len
// tokens in that sequence, token j of them attends to kv_len - q_len + j + 1 tokens when causal (the chunk
// is the tail of the context), to kv_len otherwise.  Tokens outside cu[0] .. cu[B] get length 0.
__global__ __launch_bounds__(256) void expand_varlen_kernel(const int32_t* cu_seqlens_q,
                                                            const int32_t* kv_seq_lens,
                                                            int32_t* tok_lens, int32_t* tok_rows,
                                                            int n_tokens, int batch, int causal) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= n_tokens) return;
  int lo = 0, hi = batch;  // largest b in [0, batch) with cu[b] <= t (cu[0] is 0 for well-formed input)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_seqlens_q[mid] <= t) lo = mid; else hi = mid;
  }
  const int b = lo;
  const int q0 = cu_seqlens_q[b], q1 = cu_seqlens_q[b + 1];
  int L = 0;
  if (t >= q0 && t < q1) {
    const int kv = kv_seq_lens[b];
    L = causal != 0 ? kv - (q1 - q0) + (t - q0) + 1 : kv;
    L = L < 0 ? 0 : (L > kv ? kv : L);
  }
  tok_lens[t] = L;
  tok_rows[t] = b;
}

// One workgroup per kGatherRows output rows.  Their first threads find the sequence of their row (cu[b] <= row <
// cu[b + 1]) and its source row in the paged cache; then the 256 threads copy the rows in pieces of VB bytes
// (16 when the row length allows it), consecutive threads taking consecutive pieces of a row.  Rows whose
// page id is negative or beyond the cache are left untouched, as in the reference kernel (which skips
// negative ids; an id beyond the cache would be an out-of-bounds read there).
// The search is a chain of dependent reads, so the row offsets go to LDS first when they fit (one trip to memory for
// all of them instead of log2(batch) in a row), and a thread asks for kGatherDepth pieces before it stores the first: the
// launch is a stream of rows that are read once and written once, with non-temporal loads and stores.
constexpr int kGatherCuLds = 2048;   // row offsets kept in LDS
constexpr int kGatherRows = 64;      // output rows per workgroup
constexpr int kGatherDepth = 8;      // pieces a thread asks for before it stores the first
template <int VB>
__global__ __launch_bounds__(256) void gather_paged_rows_kernel(const char* cache, const int32_t* block_table,
                                                                int64_t table_stride, const int32_t* cu_seq_lens,
                                                                char* out, int batch, int64_t total_rows,
                                                                int block_size, int num_blocks, int row_bytes) {
  __shared__ int64_t src_row[kGatherRows];
  extern __shared__ int cu_l[];   // [batch + 1] when batch <= kGatherCuLds
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kGatherRows;
  const bool in_lds = batch <= kGatherCuLds;
  if (in_lds) {
    for (int i = threadIdx.x; i <= batch; i += 256) cu_l[i] = cu_seq_lens[i];
    __syncthreads();
  }
  if (threadIdx.x < kGatherRows) {
    const int64_t row = row0 + threadIdx.x;
    int64_t src = -1;
    if (row < total_rows) {
      int lo = 0, hi = batch;  // largest b in [0, batch) with cu[b] <= row
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if ((in_lds ? cu_l[mid] : cu_seq_lens[mid]) <= row) lo = mid; else hi = mid;
      }
      const int64_t first = in_lds ? cu_l[lo] : cu_seq_lens[lo], next = in_lds ? cu_l[lo + 1] : cu_seq_lens[lo + 1];
      const int64_t tok = row - first;
      if (tok >= 0 && row < next && tok / block_size < table_stride) {
        const int page = block_table[lo * table_stride + tok / block_size];
        if (page >= 0 && page < num_blocks) src = static_cast<int64_t>(page) * block_size + tok % block_size;
      }
    }
    src_row[threadIdx.x] = src;
  }
  __syncthreads();
  const int pieces = row_bytes / VB;
  const int n = kGatherRows * pieces;
  if constexpr (VB == 16) {
    for (int i0 = threadIdx.x; i0 < n; i0 += kGatherDepth * 256) {
      u32x4 v[kGatherDepth];
      char* to[kGatherDepth];
#pragma unroll
      for (int u = 0; u < kGatherDepth; ++u) {
        const int i = i0 + u * 256;
        to[u] = nullptr;
        if (i < n) {
          const int r = i / pieces, c = i - r * pieces;
          const int64_t src = src_row[r];
          if (src >= 0) {
            v[u] = ldg16_stream(cache + src * row_bytes + static_cast<int64_t>(c) * 16);
            to[u] = out + (row0 + r) * row_bytes + static_cast<int64_t>(c) * 16;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kGatherDepth; ++u)
        if (to[u] != nullptr) __builtin_nontemporal_store(v[u], reinterpret_cast<u32x4*>(to[u]));
    }
  } else {
    for (int i = threadIdx.x; i < n; i += 256) {
      const int r = i / pieces, c = i - r * pieces;
      const int64_t src = src_row[r];
      if (src < 0) continue;
      const char* from = cache + src * row_bytes + static_cast<int64_t>(c) * VB;
      char* to = out + (row0 + r) * row_bytes + static_cast<int64_t>(c) * VB;
      if constexpr (VB == 4) *reinterpret_cast<uint32_t*>(to) = *reinterpret_cast<const uint32_t*>(from);
      else *to = *from;
    }
  }
}

}  // namespace

int gather_paged_rows(const void* cache, const int32_t* block_table, int64_t table_stride,
                      const int32_t* cu_seq_lens, void* out, int64_t batch, int64_t total_rows,
                      int64_t block_size, int64_t num_blocks, int64_t row_bytes, hipStream_t stream) {
  if (batch == 0 || total_rows == 0) return XLLM_MI355_OK;
  if (cache == nullptr || block_table == nullptr || cu_seq_lens == nullptr || out == nullptr) return XLLM_MI355_EINVAL;
  if (batch < 0 || total_rows < 0 || batch > 0x7fffffffLL || table_stride <= 0 || block_size <= 0 ||
      block_size > 0x7fffffffLL || num_blocks <= 0 || num_blocks > 0x7fffffffLL || row_bytes <= 0 ||
      row_bytes > 0x7fffffffLL / kGatherRows)
    return XLLM_MI355_EINVAL;
  const int64_t n_groups = (total_rows + kGatherRows - 1) / kGatherRows;
  if (n_groups > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  const dim3 grid(static_cast<unsigned>(n_groups));
  const char* c = static_cast<const char*>(cache);
  char* o = static_cast<char*>(out);
  const bool a16 = ((reinterpret_cast<uintptr_t>(cache) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  const bool a4 = ((reinterpret_cast<uintptr_t>(cache) | reinterpret_cast<uintptr_t>(out)) & 3) == 0;
  const int b = static_cast<int>(batch), bs = static_cast<int>(block_size), nb = static_cast<int>(num_blocks),
            rb = static_cast<int>(row_bytes);
  const size_t lds = batch <= kGatherCuLds ? (static_cast<size_t>(batch) + 1) * 4 : 0;
  if (row_bytes % 16 == 0 && a16)
    gather_paged_rows_kernel<16><<<grid, 256, lds, stream>>>(c, block_table, table_stride, cu_seq_lens, o, b, total_rows, bs, nb, rb);
  else if (row_bytes % 4 == 0 && a4)
    gather_paged_rows_kernel<4><<<grid, 256, lds, stream>>>(c, block_table, table_stride, cu_seq_lens, o, b, total_rows, bs, nb, rb);
  else
    gather_paged_rows_kernel<1><<<grid, 256, lds, stream>>>(c, block_table, table_stride, cu_seq_lens, o, b, total_rows, bs, nb, rb);
  return static_cast<int>(hipGetLastError());
}

namespace {
__global__ __launch_bounds__(256) void clear_words_kernel(int* p, int n) {
  for (int i = threadIdx.x; i < n; i += 256) p[i] = 0;
}
}  // namespace

int decode_workspace_init(void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 || workspace_bytes < kWsHeaderBytes)
    return XLLM_MI355_EWORKSPACE;
  clear_words_kernel<<<dim3(1), 256, 0, stream>>>(static_cast<int*>(workspace), static_cast<int>(kWsHeaderBytes / 4));
  return static_cast<int>(hipGetLastError());
}

size_t decode_workspace_bound() {
  size_t need = gqa_workspace_bytes(1, 1, 256);
  for (int64_t heads = 128; heads <= 1024; heads += 128) {
    const size_t m = mla_workspace_bytes(1, heads, 0);
    need = m > need ? m : need;
  }
  return need + varlen_extra_bytes(65536) + 256;
}

size_t varlen_extra_bytes(int64_t n_tokens) {
  return n_tokens <= 0 ? 0 : (static_cast<size_t>(n_tokens) * 2 * 4 + 255) / 256 * 256;
}

int paged_decode_gqa_varlen(const void* q, const void* k_cache, const void* v_cache, void* out,
                            const int32_t* cu_seqlens_q, const int32_t* kv_seq_lens,
                            const int32_t* block_table, int64_t table_stride, const float* k_scale,
                            const float* v_scale, int64_t batch, int64_t n_tokens, int64_t max_q_len,
                            int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                            int64_t num_blocks, int64_t q_token_stride, int64_t out_token_stride,
                            int64_t max_seq_len, int64_t window_left, float sm_scale, int causal, void* workspace,
                            size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream) {
  if (batch == 0 || n_tokens == 0) return XLLM_MI355_OK;
  if (cu_seqlens_q == nullptr || kv_seq_lens == nullptr || block_table == nullptr || table_stride <= 0)
    return XLLM_MI355_EINVAL;
  if (batch < 0 || n_tokens < 0 || batch > 0x7fffffffLL || n_tokens > 0x7fffffffLL || n_q_heads <= 0 ||
      n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0)
    return XLLM_MI355_EINVAL;
  // The (token, head) pairs of a chunk share the 16 columns of the matrix-core kernel, 16 / group tokens per
  // pass over the pages; the kernel cuts a chunk longer than the caller's bound.
  const int64_t group = n_q_heads / n_kv_heads;
  bool pow2 = false;
  for (int s = 4; s < 31; ++s) pow2 |= (1LL << s) == block_size;
  const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 7) == 0 && ((out_token_stride * 2) & 7) == 0;
  // tokens per column block, column blocks per KV head; with one token per block (group 16) and several
  // blocks an entry per token is cheaper, its repeated page reads being served partly by L2
  const int64_t per = group <= 16 ? 16 / group : 0;
  const int64_t blocks = per > 0 && max_q_len > 0 ? (max_q_len + per - 1) / per : 0;
  // (with a sliding window every token has its own first position: the per-token path below serves that)
  if (window_left < 0 && blocks >= 1 && blocks <= 16 && (per >= 2 || blocks == 1) && head_dim == 128 && pow2 && out_aligned) {
    PageAddressing addr;
    addr.chunk_blocks = static_cast<int>(blocks);
    addr.block_table = block_table;
    addr.table_stride = table_stride;
    addr.seq_lens = kv_seq_lens;
    addr.cu_q = cu_seqlens_q;
    addr.n_tokens = n_tokens;
    addr.causal = causal;
    return paged_decode_gqa(q, k_cache, v_cache, out, nullptr, addr, k_scale, v_scale, batch, n_q_heads,
                            n_kv_heads, head_dim, block_size, num_blocks, q_token_stride, out_token_stride,
                            max_seq_len, sm_scale, workspace, workspace_bytes, q_dtype, cache_dtype, stream);
  }
  // Otherwise every query token becomes a decode entry of its own; their lengths and table rows take the
  // last bytes of the workspace (the header, prefix and partials keep their places at its start).
  const size_t extra = varlen_extra_bytes(n_tokens);
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 || workspace_bytes < extra)
    return XLLM_MI355_EWORKSPACE;
  const size_t usable = (workspace_bytes - extra) / 256 * 256;
  int32_t* tok_lens = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + usable);
  int32_t* tok_rows = tok_lens + n_tokens;
  const unsigned grid = static_cast<unsigned>((n_tokens + 255) / 256);
  expand_varlen_kernel<<<dim3(grid), 256, 0, stream>>>(cu_seqlens_q, kv_seq_lens, tok_lens, tok_rows,
                                                       static_cast<int>(n_tokens), static_cast<int>(batch), causal);
  const int rc = static_cast<int>(hipGetLastError());
  if (rc != 0) return rc;
  PageAddressing addr;
  addr.block_table = block_table;
  addr.table_stride = table_stride;
  addr.seq_lens = tok_lens;
  addr.table_rows = tok_rows;
  addr.window_left = window_left;   // token j sits at position tok_lens[j] - 1 of its own attended range
  return paged_decode_gqa(q, k_cache, v_cache, out, nullptr, addr, k_scale, v_scale, n_tokens, n_q_heads,
                          n_kv_heads, head_dim, block_size, num_blocks, q_token_stride, out_token_stride,
                          max_seq_len, sm_scale, workspace, usable, q_dtype, cache_dtype, stream);
}

int lse_merge(const void* partial_out, const float* partial_lse, void* out, float* lse,
              int64_t n_shards, int64_t batch, int64_t n_heads, int64_t v_head_dim, int dtype,
              hipStream_t stream) {
  if (batch == 0 || n_heads == 0) return XLLM_MI355_OK;
  if (partial_out == nullptr || partial_lse == nullptr || out == nullptr) return XLLM_MI355_EINVAL;
  if (n_shards <= 0 || batch < 0 || n_heads < 0 || v_head_dim <= 0) return XLLM_MI355_EINVAL;
  const int64_t bh = batch * n_heads;
  if (bh > 0x7fffffffLL || n_shards > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  dim3 grid(static_cast<unsigned>(bh));
  const char* po = static_cast<const char*>(partial_out);
  char* o = static_cast<char*>(out);
  const int s = static_cast<int>(n_shards), dv = static_cast<int>(v_head_dim);
  switch (dtype) {
    case XLLM_MI355_BF16:
      lse_merge_kernel<XLLM_MI355_BF16><<<grid, 128, 0, stream>>>(po, partial_lse, o, lse, s, bh, dv);
      break;
    case XLLM_MI355_FP16:
      lse_merge_kernel<XLLM_MI355_FP16><<<grid, 128, 0, stream>>>(po, partial_lse, o, lse, s, bh, dv);
      break;
    case XLLM_MI355_FP32:
      lse_merge_kernel<XLLM_MI355_FP32><<<grid, 128, 0, stream>>>(po, partial_lse, o, lse, s, bh, dv);
      break;
    default: return XLLM_MI355_EDTYPE;
  }
  return static_cast<int>(hipGetLastError());
}

int lse_combine(void* out, const void* shared_o, const float* shared_lse, const void* unshared_o,
                const float* unshared_lse, int64_t rows, int64_t head_dim, int in_dtype, int out_dtype,
                hipStream_t stream) {
  if (rows == 0 || head_dim == 0) return XLLM_MI355_OK;
  if (out == nullptr || shared_o == nullptr || shared_lse == nullptr || unshared_o == nullptr || unshared_lse == nullptr)
    return XLLM_MI355_EINVAL;
  if (rows < 0 || rows > 0x7fffffffLL || head_dim < 0 || head_dim > 0x7fffffffLL) return XLLM_MI355_EINVAL;
  const dim3 grid(static_cast<unsigned>(rows));
  char* o = static_cast<char*>(out);
  const char* s = static_cast<const char*>(shared_o);
  const char* u = static_cast<const char*>(unshared_o);
  const int d = static_cast<int>(head_dim);
#define XLLM_COMBINE(IN, OUT) lse_combine_kernel<IN, OUT><<<grid, 128, 0, stream>>>(o, s, shared_lse, u, unshared_lse, d)
#define XLLM_COMBINE_OUT(IN)                                                    \
  switch (out_dtype) {                                                          \
    case XLLM_MI355_BF16: XLLM_COMBINE(IN, XLLM_MI355_BF16); break;             \
    case XLLM_MI355_FP16: XLLM_COMBINE(IN, XLLM_MI355_FP16); break;             \
    case XLLM_MI355_FP32: XLLM_COMBINE(IN, XLLM_MI355_FP32); break;             \
    default: return XLLM_MI355_EDTYPE;                                          \
  }
  switch (in_dtype) {
    case XLLM_MI355_BF16: XLLM_COMBINE_OUT(XLLM_MI355_BF16); break;
    case XLLM_MI355_FP16: XLLM_COMBINE_OUT(XLLM_MI355_FP16); break;
    case XLLM_MI355_FP32: XLLM_COMBINE_OUT(XLLM_MI355_FP32); break;
    default: return XLLM_MI355_EDTYPE;
  }
#undef XLLM_COMBINE_OUT
#undef XLLM_COMBINE
  return static_cast<int>(hipGetLastError());
}

int mask_block_table_padding(const int32_t* block_table, int64_t table_stride, const int32_t* kv_seq_lens,
                             int32_t* out, int64_t out_stride, int64_t batch, int64_t width, int64_t block_size,
                             hipStream_t stream) {
  if (batch == 0 || width == 0) return XLLM_MI355_OK;
  if (block_table == nullptr || kv_seq_lens == nullptr || out == nullptr) return XLLM_MI355_EINVAL;
  if (batch < 0 || batch > 0x7fffffffLL || width < 0 || width > 0x7fffffffLL || table_stride < width ||
      out_stride < width || block_size <= 0 || block_size > 0x7fffffffLL)
    return XLLM_MI355_EINVAL;
  mask_block_table_padding_kernel<<<dim3(static_cast<unsigned>(batch)), 256, 0, stream>>>(
      block_table, table_stride, kv_seq_lens, out, out_stride, static_cast<int>(width), static_cast<int>(block_size));
  return static_cast<int>(hipGetLastError());
}

int build_block_table(const int32_t* indptr, const int32_t* indices, const int32_t* last_page_len,
                      int32_t* block_table, int64_t table_stride, int32_t* seq_lens, int64_t batch,
                      int64_t block_size, hipStream_t stream) {
  if (batch == 0) return XLLM_MI355_OK;
  if (indptr == nullptr || indices == nullptr || block_table == nullptr) return XLLM_MI355_EINVAL;
  if (seq_lens != nullptr && last_page_len == nullptr) return XLLM_MI355_EINVAL;
  if (batch < 0 || batch > 0x7fffffffLL || table_stride <= 0 || block_size <= 0) return XLLM_MI355_EINVAL;
  build_block_table_kernel<<<dim3(static_cast<unsigned>(batch)), 256, 0, stream>>>(
      indptr, indices, last_page_len, block_table, table_stride, seq_lens, static_cast<int>(block_size));
  return static_cast<int>(hipGetLastError());
}

int decode_metadata_update(const int32_t* src_tokens, const int32_t* src_positions, const int32_t* src_new_cache_slots,
                           const int32_t* src_kv_seq_lens, const int32_t* src_paged_kv_indptr,
                           const int32_t* src_paged_kv_indices, const int32_t* src_paged_kv_last_page_len,
                           int32_t* dst_tokens, int32_t* dst_positions, int32_t* dst_new_cache_slots,
                           int32_t* dst_kv_seq_lens, int32_t* dst_kv_seq_lens_delta, int32_t* dst_paged_kv_indptr,
                           int32_t* dst_paged_kv_indices, int32_t* dst_paged_kv_last_page_len,
                           int64_t actual_num_tokens, int64_t padded_num_tokens, int64_t actual_batch_size,
                           int64_t actual_indices_size, hipStream_t stream) {
  if (actual_num_tokens < 0 || padded_num_tokens < 0 || actual_batch_size < 0 || actual_indices_size < 0)
    return XLLM_MI355_EINVAL;
  // the largest index any rule touches (llm_decode_metadata_update.cu:76-91)
  int64_t n = actual_num_tokens;
  if (padded_num_tokens + 1 > n) n = padded_num_tokens + 1;
  if (actual_batch_size + 1 > n) n = actual_batch_size + 1;
  if (actual_indices_size > n) n = actual_indices_size;
  const bool tokens_on = actual_num_tokens > 0 || padded_num_tokens > 0;
  if (tokens_on && (dst_tokens == nullptr || dst_positions == nullptr || dst_new_cache_slots == nullptr ||
                    dst_kv_seq_lens_delta == nullptr || dst_paged_kv_last_page_len == nullptr))
    return XLLM_MI355_EINVAL;
  if (actual_num_tokens > 0 && (src_tokens == nullptr || src_positions == nullptr || src_new_cache_slots == nullptr))
    return XLLM_MI355_EINVAL;
  if (src_kv_seq_lens == nullptr || src_paged_kv_indptr == nullptr || dst_kv_seq_lens == nullptr ||
      dst_paged_kv_indptr == nullptr)
    return XLLM_MI355_EINVAL;
  if (actual_batch_size > 0 && src_paged_kv_last_page_len == nullptr) return XLLM_MI355_EINVAL;
  if (actual_indices_size > 0 && (src_paged_kv_indices == nullptr || dst_paged_kv_indices == nullptr))
    return XLLM_MI355_EINVAL;
  const MetadataUpdate u = {src_tokens, src_positions, src_new_cache_slots, src_kv_seq_lens, src_paged_kv_indptr,
                            src_paged_kv_indices, src_paged_kv_last_page_len, dst_tokens, dst_positions,
                            dst_new_cache_slots, dst_kv_seq_lens, dst_kv_seq_lens_delta, dst_paged_kv_indptr,
                            dst_paged_kv_indices, dst_paged_kv_last_page_len, actual_num_tokens, padded_num_tokens,
                            actual_batch_size, actual_indices_size};
  const int64_t blocks = (n + 255) / 256;
  decode_metadata_update_kernel<<<dim3(static_cast<unsigned>(blocks < 4096 ? blocks : 4096)), 256, 0, stream>>>(u, n);
  return static_cast<int>(hipGetLastError());
}

}  // namespace xllm_mi355
