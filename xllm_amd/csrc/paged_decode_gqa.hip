// Paged decode attention, GQA, for gfx950.
//
// Work decomposition: one 256-thread workgroup per (sequence, KV-head block, split),
// a split being `chunk_tokens` consecutive context tokens.  Inside the workgroup each
// of the 4 wavefronts walks its own interleaved share of the split's pages:
//   * a token's [D] row of one KV head is read by LPT adjacent lanes with one 16-byte
//     load each (64/LPT tokens per load instruction), K and V alike, so every load
//     instruction covers whole contiguous rows of the [P, bs, Hkv, D] pages;
//   * q.k is v_dot2 on packed 16-bit pairs into fp32, reduced over the LPT lanes by
//     DPP row operations; all G query heads of the KV head reuse the same K registers;
//   * each row of LPT lanes keeps its own running (max, sum, acc) -- no cross-row
//     traffic inside the loop; rows and wavefronts are merged once through LDS;
//   * fp8 pages are converted to the 16-bit pair type in registers (exact), the
//     per-head scales are folded into the score scale (K) and the output (V).
// The page walk reads slot ids (page * bs + row) staged in LDS once per split, so the
// loop has no division and never touches table columns past ceil(L / bs).
// Splits write normalised fp32 partials + log2-domain LSE to the workspace and a small
// merge kernel combines them; a sequence with one split writes its output directly.
//
// Arithmetic follows the block-table oracle of the reference,
// xllm/core/kernels/npu/attention.cpp:26-78 (head h reads KV head h / group, explicit
// scale, non-causal softmax over the first L tokens of the listed pages).
#include <cstdlib>

#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

struct GqaArgs {
  const char* q;
  const char* k_cache;
  const char* v_cache;
  char* out;
  float* lse;
  const int32_t* block_table;
  const int32_t* seq_lens;
  const int32_t* indptr;
  const int32_t* indices;
  const int32_t* last_page_len;
  const float* k_scale;
  const float* v_scale;
  float* ws_out;
  float* ws_lse;
  int64_t table_stride;
  int64_t q_stride_bytes;
  int64_t out_stride_bytes;
  int64_t row_bytes;  // Hkv * D * sizeof(cache element)
  int n_q_heads;
  int n_kv_heads;
  int group;
  int block_size;
  int bs_shift;  // log2(block_size) or -1
  int num_blocks;
  int chunk_tokens;
  int max_splits;
  float scale_log2;  // sm_scale * log2(e)
};

__device__ __forceinline__ void sequence_of(const GqaArgs& a, int b, const int32_t*& pages, int& L) {
  if (a.indptr != nullptr) {
    const int p0 = a.indptr[b];
    const int np = a.indptr[b + 1] - p0;
    pages = a.indices + p0;
    L = np > 0 ? (np - 1) * a.block_size + a.last_page_len[b] : 0;
  } else {
    pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
    L = a.seq_lens[b];
  }
}

// QT: BF16 or FP16 (query, output and non-fp8 cache element).  FP8: cache holds e4m3fn.
// D: head dim.  LPT: lanes per token row.  G: query heads per workgroup.  U: token rows
// per lane and step.
template <typename QT, bool FP8, int D, int LPT, int G, int U>
__global__ __launch_bounds__(kThreads) void gqa_decode_kernel(GqaArgs a) {
  constexpr int TPP = kWave / LPT;       // token rows per load instruction
  constexpr int EPL = FP8 ? 16 : 8;      // cache elements per 16-byte load
  constexpr int VEC = D / LPT;           // cache elements per lane and token
  constexpr int NLD = VEC / EPL;         // 16-byte loads per lane and token
  constexpr int STEP = U * TPP;          // tokens per wavefront step
  constexpr int NP = kWaves * TPP;       // partial softmax states per workgroup
  constexpr int PSTRIDE = D + 2;         // acc[D], max, sum
  static_assert(NLD >= 1 && NLD * EPL * LPT == D, "lane mapping must tile the head dim");

  extern __shared__ __align__(16) char smem[];
  int* slots = reinterpret_cast<int*>(smem);
  float* part = reinterpret_cast<float*>(smem + static_cast<size_t>(a.chunk_tokens) * 4);

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int c = lane % LPT;  // 16-byte column of the row
  const int r = lane / LPT;  // token row within a load
  const int split = blockIdx.x;
  const int b = blockIdx.z;
  const int hb_per_kv = (a.group + G - 1) / G;
  const int kvh = blockIdx.y / hb_per_kv;
  const int h0 = kvh * a.group + (blockIdx.y % hb_per_kv) * G;
  const int nh = min(G, (kvh + 1) * a.group - h0);

  const int32_t* pages;
  int L;
  sequence_of(a, b, pages, L);
  if (L <= 0) {
    if (split == 0) {
      for (int i = tid; i < nh * D; i += kThreads) {
        const int h = i / D, d = i % D;
        reinterpret_cast<uint16_t*>(a.out + b * a.out_stride_bytes)[(h0 + h) * D + d] = 0;
      }
      if (a.lse != nullptr && tid < nh) a.lse[b * a.n_q_heads + h0 + tid] = -INFINITY;
    }
    return;
  }
  const int n_splits = (L + a.chunk_tokens - 1) / a.chunk_tokens;
  if (split >= n_splits) return;
  const int t0 = split * a.chunk_tokens;
  const int t1 = min(L, t0 + a.chunk_tokens);
  const int n_steps = (t1 - t0 + STEP - 1) / STEP;

  // slot id of every token of the split (tail entries repeat the last valid token)
  for (int i = tid; i < n_steps * STEP; i += kThreads) {
    const int tok = min(t0 + i, L - 1);
    int pg, off;
    if (a.bs_shift >= 0) {
      pg = tok >> a.bs_shift;
      off = tok & (a.block_size - 1);
    } else {
      pg = tok / a.block_size;
      off = tok - pg * a.block_size;
    }
    int page = pages[pg];
    page = max(0, min(page, a.num_blocks - 1));  // a corrupt table must not fault the GPU
    slots[i] = page * a.block_size + off;
  }

  // query registers: for each head the 16-bit pairs matching this lane's cache columns
  u32 qreg[G][NLD][EPL / 2];
#pragma unroll
  for (int h = 0; h < G; ++h) {
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
      if (h < nh) {
        const char* qp = a.q + b * a.q_stride_bytes +
                         (static_cast<int64_t>(h0 + h) * D + (j * LPT + c) * EPL) * 2;
#pragma unroll
        for (int e = 0; e < EPL / 8; ++e) {
          const u32x4 x = ldg16(qp + e * 16);
          qreg[h][j][e * 4 + 0] = x[0];
          qreg[h][j][e * 4 + 1] = x[1];
          qreg[h][j][e * 4 + 2] = x[2];
          qreg[h][j][e * 4 + 3] = x[3];
        }
      } else {
#pragma unroll
        for (int e = 0; e < EPL / 2; ++e) qreg[h][j][e] = 0u;
      }
    }
  }

  float score_scale = a.scale_log2;
  if constexpr (FP8) score_scale *= a.k_scale[kvh];

  float m[G], l[G], acc[G][NLD * EPL];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = kNegBig;
    l[h] = 0.0f;
#pragma unroll
    for (int e = 0; e < NLD * EPL; ++e) acc[h][e] = 0.0f;
  }

  constexpr int CES = FP8 ? 1 : 2;
  const int64_t lane_off = static_cast<int64_t>(kvh) * D * CES + c * 16;
  const char* kbase = a.k_cache + lane_off;
  const char* vbase = a.v_cache + lane_off;

  struct Tile {
    u32x4 k[U][NLD];
    u32x4 v[U][NLD];
  };

  __syncthreads();  // slots ready

  auto load_tile = [&](Tile& t, int step) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int slot = slots[step * STEP + u * TPP + r];
      const int64_t off = static_cast<int64_t>(slot) * a.row_bytes;
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
        t.k[u][j] = ldg16(kbase + off + j * (LPT * 16));
        t.v[u][j] = ldg16(vbase + off + j * (LPT * 16));
      }
    }
  };

  auto compute_tile = [&](const Tile& t, int step) {
    float s[U][G];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      u32 kp[NLD][EPL / 2];
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          if constexpr (FP8) {
            kp[j][2 * w] = QT::template from_fp8x2<false>(t.k[u][j][w]);
            kp[j][2 * w + 1] = QT::template from_fp8x2<true>(t.k[u][j][w]);
          } else {
            kp[j][w] = t.k[u][j][w];
          }
        }
      }
      const bool valid = t0 + step * STEP + u * TPP + r < t1;
#pragma unroll
      for (int h = 0; h < G; ++h) {
        float d = 0.0f;
#pragma unroll
        for (int j = 0; j < NLD; ++j)
#pragma unroll
          for (int e = 0; e < EPL / 2; ++e) d = QT::dot2(kp[j][e], qreg[h][j][e], d);
        d = group_sum<LPT>(d);
        s[u][h] = valid ? d * score_scale : -INFINITY;
      }
    }
    // online softmax of this lane row's U tokens
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float mx = s[0][h];
#pragma unroll
      for (int u = 1; u < U; ++u) mx = fmaxf(mx, s[u][h]);
      const float m_new = fmaxf(m[h], mx);
      const float alpha = fast_exp2(m[h] - m_new);
      m[h] = m_new;
      float sum = 0.0f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        s[u][h] = fast_exp2(s[u][h] - m_new);
        sum += s[u][h];
      }
      l[h] = l[h] * alpha + sum;
#pragma unroll
      for (int e = 0; e < NLD * EPL; ++e) acc[h][e] *= alpha;
    }
    // acc += p . v
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int j = 0; j < NLD; ++j) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const u32 x = t.v[u][j][w];
          if constexpr (FP8) {
            const f32x2 f01 = fp8x2_to_f32<false>(x);
            const f32x2 f23 = fp8x2_to_f32<true>(x);
#pragma unroll
            for (int h = 0; h < G; ++h) {
              acc[h][j * EPL + 4 * w + 0] += s[u][h] * f01[0];
              acc[h][j * EPL + 4 * w + 1] += s[u][h] * f01[1];
              acc[h][j * EPL + 4 * w + 2] += s[u][h] * f23[0];
              acc[h][j * EPL + 4 * w + 3] += s[u][h] * f23[1];
            }
          } else {
            const float v0 = QT::lo(x);
            const float v1 = QT::hi(x);
#pragma unroll
            for (int h = 0; h < G; ++h) {
              acc[h][j * EPL + 2 * w + 0] += s[u][h] * v0;
              acc[h][j * EPL + 2 * w + 1] += s[u][h] * v1;
            }
          }
        }
      }
    }
  };

  // steps are dealt round-robin to the wavefronts; two register tiles alternate so that
  // the loads of the next step are in flight while the current one is reduced
  Tile ta, tb;
  int step = wave;
  if (step < n_steps) load_tile(ta, step);
  while (step < n_steps) {
    const int next = step + kWaves;
    if (next < n_steps) load_tile(tb, next);
    compute_tile(ta, step);
    if (next >= n_steps) break;
    const int next2 = next + kWaves;
    if (next2 < n_steps) load_tile(ta, next2);
    compute_tile(tb, next);
    step = next2;
  }

  // one head at a time: every lane row publishes its state, the workgroup folds the NP states
  float out_scale = 1.0f;
  if constexpr (FP8) out_scale = a.v_scale[kvh];
  const int pi = wave * TPP + r;
#pragma unroll
  for (int h = 0; h < G; ++h) {
    if (h > 0) __syncthreads();  // the previous head's states have been consumed
    {
      float* p = part + pi * PSTRIDE;
#pragma unroll
      for (int j = 0; j < NLD; ++j)
#pragma unroll
        for (int e = 0; e < EPL; ++e) p[(j * LPT + c) * EPL + e] = acc[h][j * EPL + e];
      if (c == 0) {
        p[D] = m[h];
        p[D + 1] = l[h];
      }
    }
    __syncthreads();
    if (h < nh) {
      for (int d = tid; d < D; d += kThreads) {
        float mx = kNegBig;
#pragma unroll
        for (int p = 0; p < NP; ++p) mx = fmaxf(mx, part[p * PSTRIDE + D]);
        float lsum = 0.0f, o = 0.0f;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
          const float* pp = part + p * PSTRIDE;
          const float w = fast_exp2(pp[D] - mx);
          lsum += w * pp[D + 1];
          o += w * pp[d];
        }
        const float val = o / lsum * out_scale;
        const int hq = h0 + h;
        if (n_splits == 1) {
          reinterpret_cast<uint16_t*>(a.out + b * a.out_stride_bytes)[hq * D + d] = QT::from_f32(val);
          if (a.lse != nullptr && d == 0) a.lse[b * a.n_q_heads + hq] = (mx + fast_log2(lsum)) * kLn2;
        } else {
          const int64_t wi = (static_cast<int64_t>(b) * a.n_q_heads + hq) * a.max_splits + split;
          a.ws_out[wi * D + d] = val;
          if (d == 0) a.ws_lse[wi] = mx + fast_log2(lsum);
        }
      }
    }
  }
}

// Merge of split partials: one workgroup per (sequence, query head).
template <typename QT>
__global__ __launch_bounds__(128) void merge_splits_kernel(const float* ws_out, const float* ws_lse,
                                                           char* out, float* lse, GqaArgs a, int dv) {
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int32_t* pages;
  int L;
  sequence_of(a, b, pages, L);
  const int n_splits = (L + a.chunk_tokens - 1) / a.chunk_tokens;
  if (n_splits <= 1) return;  // written directly by the decode kernel
  const int64_t w0 = (static_cast<int64_t>(b) * a.n_q_heads + hq) * a.max_splits;
  float mx = kNegBig;
  for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, ws_lse[w0 + s]);
  float wsum = 0.0f;
  for (int s = 0; s < n_splits; ++s) wsum += fast_exp2(ws_lse[w0 + s] - mx);
  const float inv = 1.0f / wsum;
  for (int d = threadIdx.x; d < dv; d += 128) {
    float o = 0.0f;
    for (int s = 0; s < n_splits; ++s)
      o += fast_exp2(ws_lse[w0 + s] - mx) * ws_out[(w0 + s) * dv + d];
    reinterpret_cast<uint16_t*>(out + b * a.out_stride_bytes)[hq * dv + d] = QT::from_f32(o * inv);
  }
  if (lse != nullptr && threadIdx.x == 0) lse[b * a.n_q_heads + hq] = (mx + fast_log2(wsum)) * kLn2;
}

template <typename QT, bool FP8, int D, int LPT, int G, int U>
int launch_gqa(const GqaArgs& a, int64_t batch, int n_head_blocks, hipStream_t stream) {
  constexpr int NP = kWaves * (kWave / LPT);
  const size_t smem = static_cast<size_t>(a.chunk_tokens) * 4 + static_cast<size_t>(NP) * (D + 2) * 4;
  auto kern = gqa_decode_kernel<QT, FP8, D, LPT, G, U>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  dim3 grid(static_cast<unsigned>(a.max_splits), static_cast<unsigned>(n_head_blocks),
            static_cast<unsigned>(batch));
  kern<<<grid, kThreads, smem, stream>>>(a);
  return static_cast<int>(hipGetLastError());
}

template <typename QT, bool FP8, int D, int LPT, int U>
int dispatch_group(const GqaArgs& a, int64_t batch, int g_block, hipStream_t stream) {
  const int hb = a.n_kv_heads * ((a.group + g_block - 1) / g_block);
  switch (g_block) {
    case 1: return launch_gqa<QT, FP8, D, LPT, 1, U>(a, batch, hb, stream);
    case 2: return launch_gqa<QT, FP8, D, LPT, 2, U>(a, batch, hb, stream);
    case 4: return launch_gqa<QT, FP8, D, LPT, 4, U>(a, batch, hb, stream);
    default: return launch_gqa<QT, FP8, D, LPT, 8, U>(a, batch, hb, stream);
  }
}

template <typename QT, bool FP8>
int dispatch_dim(const GqaArgs& a, int64_t batch, int head_dim, int g_block, hipStream_t stream) {
  // lanes per token row: 16-byte loads, one per lane (two for bf16 D=256)
  if constexpr (FP8) {
    switch (head_dim) {
      case 64: return dispatch_group<QT, true, 64, 4, 1>(a, batch, g_block, stream);
      case 128: return dispatch_group<QT, true, 128, 8, 2>(a, batch, g_block, stream);
      case 256: return dispatch_group<QT, true, 256, 16, 4>(a, batch, g_block, stream);
      default: return XLLM_MI355_ESHAPE;
    }
  } else {
    switch (head_dim) {
      case 64: return dispatch_group<QT, false, 64, 8, 2>(a, batch, g_block, stream);
      case 128: return dispatch_group<QT, false, 128, 16, 4>(a, batch, g_block, stream);
      case 256: return dispatch_group<QT, false, 256, 32, 4>(a, batch, g_block, stream);
      default: return XLLM_MI355_ESHAPE;
    }
  }
}

int group_block(int group) {
  if (group <= 1) return 1;
  if (group <= 2) return 2;
  if (group <= 4) return 4;
  return 8;
}

}  // namespace

SplitPlan plan_splits(int64_t batch, int64_t n_head_blocks, int64_t max_seq_len) {
  // Enough workgroups to fill the 256 CUs a few times over (each workgroup pays a fixed
  // prologue and merge, so fewer and longer splits win once the chip is full); splits are
  // never shorter than 256 tokens nor longer than 8192 (their slot list lives in LDS).
  static const int64_t kTargetWorkgroups = [] {
    const char* e = getenv("XLLM_MI355_TARGET_WGS");  // tuning knob
    const long v = e ? atol(e) : 0;
    return static_cast<int64_t>(v > 0 ? v : 1024);
  }();
  constexpr int64_t kMinChunk = 256, kMaxChunk = 8192;
  if (max_seq_len < 1) max_seq_len = 1;
  const int64_t units = batch * n_head_blocks > 0 ? batch * n_head_blocks : 1;
  int64_t splits = (kTargetWorkgroups + units - 1) / units;
  const int64_t max_by_len = (max_seq_len + kMinChunk - 1) / kMinChunk;
  if (splits > max_by_len) splits = max_by_len;
  if (splits < 1) splits = 1;
  int64_t chunk = (max_seq_len + splits - 1) / splits;
  chunk = (chunk + kMinChunk - 1) / kMinChunk * kMinChunk;
  if (chunk > kMaxChunk) chunk = kMaxChunk;
  SplitPlan p;
  p.chunk_tokens = static_cast<int>(chunk);
  p.max_splits = static_cast<int>((max_seq_len + chunk - 1) / chunk);
  return p;
}

SplitPlan plan_mla_splits(int64_t batch, int64_t n_head_blocks, int64_t max_seq_len) {
  // One MLA workgroup owns a CU (its two LDS tiles fill it) and every split costs a
  // [heads, 512] fp32 partial, so: about two workgroups per CU, splits of at least 512 tokens.
  static const int64_t kTarget = [] {
    const char* e = getenv("XLLM_MI355_MLA_TARGET_WGS");  // tuning knob
    const long v = e ? atol(e) : 0;
    return static_cast<int64_t>(v > 0 ? v : 512);
  }();
  constexpr int64_t kMinChunk = 512, kTileTokens = 64;
  if (max_seq_len < 1) max_seq_len = 1;
  const int64_t units = batch * n_head_blocks > 0 ? batch * n_head_blocks : 1;
  int64_t splits = (kTarget + units - 1) / units;
  const int64_t max_by_len = (max_seq_len + kMinChunk - 1) / kMinChunk;
  if (splits > max_by_len) splits = max_by_len;
  if (splits < 1) splits = 1;
  int64_t chunk = (max_seq_len + splits - 1) / splits;
  chunk = (chunk + kTileTokens - 1) / kTileTokens * kTileTokens;
  SplitPlan p;
  p.chunk_tokens = static_cast<int>(chunk);
  p.max_splits = static_cast<int>((max_seq_len + chunk - 1) / chunk);
  return p;
}

size_t split_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t v_head_dim, int max_splits) {
  if (max_splits <= 1) return 0;
  return static_cast<size_t>(batch) * n_q_heads * max_splits * (v_head_dim + 1) * sizeof(float);
}

int merge_splits(const float* ws_out, const float* ws_lse, void* out, float* lse,
                 const PageAddressing& addr, int64_t batch, int64_t n_heads, int64_t v_head_dim,
                 int64_t block_size, int64_t out_token_stride, int chunk_tokens, int max_splits,
                 int out_dtype, hipStream_t stream) {
  GqaArgs a = {};
  a.block_table = addr.block_table;
  a.seq_lens = addr.seq_lens;
  a.indptr = addr.indptr;
  a.indices = addr.indices;
  a.last_page_len = addr.last_page_len;
  a.table_stride = addr.table_stride;
  a.out_stride_bytes = out_token_stride * 2;
  a.n_q_heads = static_cast<int>(n_heads);
  a.block_size = static_cast<int>(block_size);
  a.chunk_tokens = chunk_tokens;
  a.max_splits = max_splits;
  dim3 grid(static_cast<unsigned>(n_heads), static_cast<unsigned>(batch));
  if (out_dtype == XLLM_MI355_BF16)
    merge_splits_kernel<BF16><<<grid, 128, 0, stream>>>(ws_out, ws_lse, static_cast<char*>(out), lse, a,
                                                        static_cast<int>(v_head_dim));
  else
    merge_splits_kernel<FP16><<<grid, 128, 0, stream>>>(ws_out, ws_lse, static_cast<char*>(out), lse, a,
                                                        static_cast<int>(v_head_dim));
  return static_cast<int>(hipGetLastError());
}

int paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache, void* out, float* lse,
                     const PageAddressing& addr, const float* k_scale, const float* v_scale,
                     int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                     int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                     int64_t out_token_stride, int64_t max_seq_len, float sm_scale, void* workspace,
                     size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream) {
  if (batch == 0) return XLLM_MI355_OK;
  if (q == nullptr || k_cache == nullptr || v_cache == nullptr || out == nullptr) return XLLM_MI355_EINVAL;
  const bool csr = addr.indptr != nullptr;
  if (csr ? (addr.indices == nullptr || addr.last_page_len == nullptr)
          : (addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0))
    return XLLM_MI355_EINVAL;
  if (batch < 0 || batch > 65535 || n_q_heads <= 0 || n_kv_heads <= 0 || block_size <= 0 ||
      num_blocks <= 0 || n_q_heads % n_kv_heads != 0 || n_q_heads > 65535)
    return XLLM_MI355_EINVAL;
  if (num_blocks * block_size > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  if (q_dtype != XLLM_MI355_BF16 && q_dtype != XLLM_MI355_FP16) return XLLM_MI355_EDTYPE;
  const bool fp8 = cache_dtype == XLLM_MI355_FP8_E4M3;
  if (!fp8 && cache_dtype != q_dtype) return XLLM_MI355_EDTYPE;
  if (fp8 && (k_scale == nullptr || v_scale == nullptr)) return XLLM_MI355_EINVAL;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return XLLM_MI355_ESHAPE;
  if (q_token_stride < n_q_heads * head_dim || out_token_stride < n_q_heads * head_dim)
    return XLLM_MI355_EINVAL;
  auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || (q_token_stride * 2) % 16 != 0)
    return XLLM_MI355_EALIGN;
  if (max_seq_len <= 0) {
    if (csr) return XLLM_MI355_EINVAL;  // CSR carries no host-visible bound
    max_seq_len = addr.table_stride * block_size;
  }

  const int group = static_cast<int>(n_q_heads / n_kv_heads);
  const int g_block = group_block(group);
  const int hb = static_cast<int>(n_kv_heads) * ((group + g_block - 1) / g_block);
  if (hb > 65535) return XLLM_MI355_ESHAPE;
  SplitPlan plan = plan_splits(batch, hb, max_seq_len);
  // fewer, longer splits if the caller's workspace is small
  while (plan.max_splits > 1 &&
         split_workspace_bytes(batch, n_q_heads, head_dim, plan.max_splits) > workspace_bytes) {
    if (plan.chunk_tokens >= 8192) return XLLM_MI355_EWORKSPACE;
    plan.chunk_tokens *= 2;
    if (plan.chunk_tokens > 8192) plan.chunk_tokens = 8192;
    plan.max_splits = static_cast<int>((max_seq_len + plan.chunk_tokens - 1) / plan.chunk_tokens);
  }
  if (plan.max_splits > 1 && (workspace == nullptr || !aligned16(workspace))) return XLLM_MI355_EWORKSPACE;

  GqaArgs a = {};
  a.q = static_cast<const char*>(q);
  a.k_cache = static_cast<const char*>(k_cache);
  a.v_cache = static_cast<const char*>(v_cache);
  a.out = static_cast<char*>(out);
  a.lse = lse;
  a.block_table = addr.block_table;
  a.seq_lens = addr.seq_lens;
  a.indptr = addr.indptr;
  a.indices = addr.indices;
  a.last_page_len = addr.last_page_len;
  a.k_scale = k_scale;
  a.v_scale = v_scale;
  a.table_stride = addr.table_stride;
  a.q_stride_bytes = q_token_stride * 2;
  a.out_stride_bytes = out_token_stride * 2;
  a.row_bytes = n_kv_heads * head_dim * (fp8 ? 1 : 2);
  a.n_q_heads = static_cast<int>(n_q_heads);
  a.n_kv_heads = static_cast<int>(n_kv_heads);
  a.group = group;
  a.block_size = static_cast<int>(block_size);
  a.bs_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1LL << s) == block_size) a.bs_shift = s;
  a.num_blocks = static_cast<int>(num_blocks);
  a.chunk_tokens = plan.chunk_tokens;
  a.max_splits = plan.max_splits;
  a.scale_log2 = sm_scale * kLog2e;
  if (plan.max_splits > 1) {
    a.ws_out = static_cast<float*>(workspace);
    a.ws_lse = a.ws_out + static_cast<size_t>(batch) * n_q_heads * plan.max_splits * head_dim;
  }

  int rc;
  const bool timed = profile_begin(stream);
  if (q_dtype == XLLM_MI355_BF16)
    rc = fp8 ? dispatch_dim<BF16, true>(a, batch, static_cast<int>(head_dim), g_block, stream)
             : dispatch_dim<BF16, false>(a, batch, static_cast<int>(head_dim), g_block, stream);
  else
    rc = fp8 ? dispatch_dim<FP16, true>(a, batch, static_cast<int>(head_dim), g_block, stream)
             : dispatch_dim<FP16, false>(a, batch, static_cast<int>(head_dim), g_block, stream);
  if (timed) profile_end(stream);
  if (rc != 0 || plan.max_splits <= 1) return rc;
  return merge_splits(a.ws_out, a.ws_lse, out, lse, addr, batch, n_q_heads, head_dim, block_size,
                      out_token_stride, plan.chunk_tokens, plan.max_splits, q_dtype, stream);
}

}  // namespace xllm_mi355
