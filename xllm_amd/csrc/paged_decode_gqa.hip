// Paged decode attention, GQA, for gfx950.
//
// Scheduling.  The context of every (sequence, KV-head block) is cut into items of 64
// tokens; the items of the whole batch form one flat list ordered (sequence, head block,
// item).  A fixed grid of persistent 256-thread workgroups (as many as fit on the chip at
// once) splits that list into equal contiguous ranges, so every workgroup streams the same
// number of KV bytes whatever the mix of context lengths, and a workgroup keeps its online
// softmax state in registers for as long as it stays inside one (sequence, head block).
// A run of items that covers a whole context writes the output directly; a run that
// covers part of one (only the first and the last run of a workgroup can) writes a
// normalised fp32 partial + log2-domain LSE, and a small merge kernel folds those.
// The item counts are prefix-summed inside every workgroup (no extra launch, no host read).
//
// Inner loop, per wavefront (the 4 wavefronts of a workgroup take steps round-robin):
//   * a token's [D] row of one KV head is read by LPT adjacent lanes with one 16-byte
//     load each (64/LPT tokens per load instruction), K and V alike, so every load
//     instruction covers whole contiguous rows of the [P, bs, Hkv, D] pages; two register
//     tiles alternate so the next step's loads fly while the current step is reduced;
//   * q.k is v_dot2 on packed 16-bit pairs into fp32, reduced over the LPT lanes by DPP
//     row operations; all G query heads of the KV head reuse the same K registers;
//   * p.v is v_dot2 as well: V words of two consecutive token rows are byte-permuted into
//     (token, token+1) pairs and dotted with the packed pair of probabilities;
//   * each row of LPT lanes keeps its own running (max, sum, acc); the accumulator is
//     rescaled only on steps where some maximum moved; rows and wavefronts are merged
//     through LDS once per run;
//   * fp8 pages are converted to 16-bit pairs in registers (exact), the per-head scales are
//     folded into the score scale (K) and the output (V).
// The page walk reads slot ids (page * bs + row) staged in LDS per 2048 tokens, so the
// loop has no division and never touches table columns past ceil(L / bs).
//
// Arithmetic follows the block-table oracle of the reference,
// xllm/core/kernels/npu/attention.cpp:26-78 (head h reads KV head h / group, explicit
// scale, non-causal softmax over the first L tokens of the listed pages).
#include <cstdlib>
#include <type_traits>

#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kItem = 64;      // tokens per schedulable item
constexpr int kSub = 2048;     // tokens whose slot ids are staged in LDS at a time
constexpr int kMaxBatch = 2048;  // sequences per launch (their item prefix lives in LDS)

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
  int* ws_prefix;  // [batch + 1] item prefix, written by workgroup 0 for the merge kernel
  float* ws_out;   // [2 * n_workgroups][G][D]
  float* ws_lse;   // [2 * n_workgroups][G]
  int64_t table_stride;
  int64_t q_stride_bytes;
  int64_t out_stride_bytes;
  int64_t row_bytes;  // Hkv * D * sizeof(cache element)
  int batch;
  int n_q_heads;
  int n_kv_heads;
  int group;
  int g_block;        // query heads per head block (the kernel's G)
  int block_size;
  int bs_shift;       // log2(block_size) or -1
  int num_blocks;
  int n_workgroups;   // grid size of the decode kernel
  float scale_log2;   // sm_scale * log2(e)
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

__device__ __forceinline__ int items_of(int L) { return L > 0 ? (L + kItem - 1) / kItem : 0; }

// First flat item of workgroup w when `total` items are dealt to `n` workgroups.
__device__ __forceinline__ int64_t range_start(int64_t w, int64_t total, int64_t n) { return w * total / n; }

// The workgroup whose range holds flat item `id`.
__device__ __forceinline__ int workgroup_of(int64_t id, int64_t total, int64_t n) {
  int64_t w = id * n / total;
  while (w + 1 < n && range_start(w + 1, total, n) <= id) ++w;
  return static_cast<int>(w);
}

// Exclusive prefix sum of the per-sequence item counts into prefix[0..batch] (LDS).
// Every thread sums a contiguous slice, then adds the totals of the slices before it.
__device__ __forceinline__ void item_prefix(const GqaArgs& a, int* prefix, int* tmp) {
  const int tid = threadIdx.x;
  const int per = (a.batch + kThreads - 1) / kThreads;
  const int lo = min(a.batch, tid * per), hi = min(a.batch, lo + per);
  int local = 0;
  for (int b = lo; b < hi; ++b) {
    const int32_t* pages;
    int L;
    sequence_of(a, b, pages, L);
    local += items_of(L);
  }
  tmp[tid] = local;
  __syncthreads();
  int excl = 0;
  for (int j = 0; j < tid; ++j) excl += tmp[j];
  for (int b = lo; b < hi; ++b) {
    const int32_t* pages;
    int L;
    sequence_of(a, b, pages, L);
    prefix[b] = excl;
    excl += items_of(L);
  }
  if (lo < hi && hi == a.batch) prefix[a.batch] = excl;  // the last non-empty slice holds the total
  __syncthreads();
}

// End-of-run fold: NP per-lane-row states (D accumulators, maximum, sum; stride D + 2 floats) of
// one head lie in LDS; thread tid produces dimension tid of the head's normalised output and
// the head's LSE.  A whole context goes to the caller's output, a piece of one to the partial
// slot pidx.  Every thread computes (threads past D repeat a dimension) and the stores hang off
// flat, un-nested conditions: a divergent branch nested at the tail of another one has been
// seen to leave the register allocator's copies for the code after it under the narrowed
// execution mask.
template <typename QT, int D, int NP>
__device__ __forceinline__ void fold_states(const GqaArgs& a, const float* part, int tid, bool head_on,
                                            bool complete, int b, int hq, int64_t pidx, float out_scale) {
  static_assert(D <= kThreads, "one thread per output dimension");
  constexpr int PSTRIDE = D + 2;
  const int d = tid & (D - 1);
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
  const float lse2 = mx + fast_log2(lsum);
  const bool wr = head_on && tid < D;
  const bool wl = head_on && tid == 0;
  if (wr && complete) reinterpret_cast<uint16_t*>(a.out + b * a.out_stride_bytes)[hq * D + d] = QT::from_f32(val);
  if (wr && !complete) a.ws_out[pidx * D + d] = val;
  if (wl && complete && a.lse != nullptr) a.lse[b * a.n_q_heads + hq] = lse2 * kLn2;
  if (wl && !complete) a.ws_lse[pidx] = lse2;
}

// QT: BF16 or FP16 (query, output and non-fp8 cache element).  FP8: cache holds e4m3fn.
// D: head dim.  LPT: lanes per token row.  G: query heads per workgroup.  U: token rows
// per lane and step (even).
template <typename QT, bool FP8, int D, int LPT, int G, int U>
__global__ __launch_bounds__(kThreads) void gqa_decode_kernel(GqaArgs a) {
  constexpr int TPP = kWave / LPT;       // token rows per load instruction
  constexpr int EPL = FP8 ? 16 : 8;      // cache elements per 16-byte load
  constexpr int VEC = D / LPT;           // cache elements per lane and token
  constexpr int NLD = VEC / EPL;         // 16-byte loads per lane and token
  constexpr int STEP = U * TPP;          // tokens per wavefront step
  constexpr int NP = kWaves * TPP;       // partial softmax states per workgroup
  constexpr int PSTRIDE = D + 2;         // acc[D], max, sum
  constexpr int CES = FP8 ? 1 : 2;
  static_assert(NLD >= 1 && NLD * EPL * LPT == D, "lane mapping must tile the head dim");
  static_assert(U % 2 == 0 && kItem % STEP == 0 && kSub % kItem == 0, "step must tile an item");

  extern __shared__ __align__(16) char smem[];
  int* slots = reinterpret_cast<int*>(smem);                       // [kSub]
  float* part = reinterpret_cast<float*>(smem + kSub * 4);         // [NP][PSTRIDE]
  int* tmp = reinterpret_cast<int*>(smem + kSub * 4 + NP * PSTRIDE * 4);  // [kThreads]
  int* prefix = tmp + kThreads;                                    // [batch + 1]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int c = lane % LPT;  // 16-byte column of the row
  const int r = lane / LPT;  // token row within a load
  const int hb_per_kv = (a.group + G - 1) / G;
  const int n_hb = a.n_kv_heads * hb_per_kv;

  item_prefix(a, prefix, tmp);
  const int64_t total = static_cast<int64_t>(prefix[a.batch]) * n_hb;
  if (blockIdx.x == 0) {
    for (int i = tid; i <= a.batch; i += kThreads) a.ws_prefix[i] = prefix[i];
  }
  if (total == 0) return;
  const int64_t n_wg = gridDim.x;
  int64_t cur = range_start(blockIdx.x, total, n_wg);
  const int64_t end = range_start(blockIdx.x + 1, total, n_wg);
  bool first_run = true;

  struct Tile {
    u32x4 k[U][NLD];
    u32x4 v[U][NLD];
  };

  while (cur < end) {
    // ---- locate the run: sequence b (binary search in the prefix), head block, first item
    int lo = 0, hi = a.batch;  // prefix[lo] * n_hb <= cur < prefix[hi] * n_hb
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (static_cast<int64_t>(prefix[mid]) * n_hb <= cur) lo = mid; else hi = mid;
    }
    const int b = lo;
    const int n_items = prefix[b + 1] - prefix[b];
    const int64_t rem = cur - static_cast<int64_t>(prefix[b]) * n_hb;
    const int hbk = static_cast<int>(rem / n_items);
    const int item0 = static_cast<int>(rem - static_cast<int64_t>(hbk) * n_items);
    const int run_items = static_cast<int>(min<int64_t>(n_items - item0, end - cur));
    const bool complete = item0 == 0 && run_items == n_items;
    cur += run_items;

    const int32_t* pages;
    int L;
    sequence_of(a, b, pages, L);
    const int kvh = hbk / hb_per_kv;
    const int h0 = kvh * a.group + (hbk % hb_per_kv) * G;
    const int nh = min(G, (kvh + 1) * a.group - h0);
    const int run_t0 = item0 * kItem;
    const int run_t1 = min(L, (item0 + run_items) * kItem);

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
    const int64_t lane_off = static_cast<int64_t>(kvh) * D * CES + c * 16;
    const char* kbase = a.k_cache + lane_off;
    const char* vbase = a.v_cache + lane_off;

    for (int t0 = run_t0; t0 < run_t1; t0 += kSub) {
      const int t1 = min(run_t1, t0 + kSub);
      const int n_steps = (t1 - t0 + STEP - 1) / STEP;
      const bool ragged = (t1 - t0) % STEP != 0;  // only the last step of a context can be

      __syncthreads();  // the previous slot list (and the merge buffer) are no longer read
      for (int i = tid; i < n_steps * STEP; i += kThreads) {
        const int tok = min(t0 + i, L - 1);  // tail entries repeat the last valid token
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
      __syncthreads();

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

      auto compute_tile = [&](const Tile& t, int step, auto masked) {
        constexpr bool MASKED = decltype(masked)::value;
        // ---- scores: raw q.k per (token row u, head h), summed over the LPT lanes
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
#pragma unroll
          for (int h = 0; h < G; ++h) {
            float d = 0.0f;
#pragma unroll
            for (int j = 0; j < NLD; ++j)
#pragma unroll
              for (int e = 0; e < EPL / 2; ++e) d = QT::dot2(kp[j][e], qreg[h][j][e], d);
            s[u][h] = group_sum<LPT>(d);
          }
          if constexpr (MASKED) {
            if (t0 + step * STEP + u * TPP + r >= t1) {
#pragma unroll
              for (int h = 0; h < G; ++h) s[u][h] = -INFINITY;
            }
          }
        }
        // ---- online softmax of this lane row's U tokens, in the log2 domain:
        // p = exp2(s * c - m) with m the running maximum of s * c (c > 0)
        bool moved = false;
        float alpha[G];
        u32 pp[U / 2][G];
#pragma unroll
        for (int h = 0; h < G; ++h) {
          float mx = s[0][h];
#pragma unroll
          for (int u = 1; u < U; ++u) mx = fmaxf(mx, s[u][h]);
          const float m_new = fmaxf(m[h], mx * score_scale);
          alpha[h] = fast_exp2(m[h] - m_new);
          moved |= m_new != m[h];
          m[h] = m_new;
          float sum = 0.0f;
#pragma unroll
          for (int u = 0; u < U; ++u) {
            s[u][h] = fast_exp2(__builtin_fmaf(s[u][h], score_scale, -m_new));
            sum += s[u][h];
          }
          l[h] = __builtin_fmaf(l[h], alpha[h], sum);
#pragma unroll
          for (int up = 0; up < U / 2; ++up) pp[up][h] = QT::pack(s[2 * up][h], s[2 * up + 1][h]);
        }
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {  // rare once the maxima have settled
#pragma unroll
          for (int h = 0; h < G; ++h)
#pragma unroll
            for (int e = 0; e < NLD * EPL; ++e) acc[h][e] *= alpha[h];
        }
        // ---- acc += p . v on (token, token + 1) pairs
#pragma unroll
        for (int up = 0; up < U / 2; ++up) {
#pragma unroll
          for (int j = 0; j < NLD; ++j) {
            u32 v0[EPL / 2], v1[EPL / 2];  // pairs of consecutive dims of rows 2up and 2up+1
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              if constexpr (FP8) {
                v0[2 * w] = QT::template from_fp8x2<false>(t.v[2 * up][j][w]);
                v0[2 * w + 1] = QT::template from_fp8x2<true>(t.v[2 * up][j][w]);
                v1[2 * w] = QT::template from_fp8x2<false>(t.v[2 * up + 1][j][w]);
                v1[2 * w + 1] = QT::template from_fp8x2<true>(t.v[2 * up + 1][j][w]);
              } else {
                v0[w] = t.v[2 * up][j][w];
                v1[w] = t.v[2 * up + 1][j][w];
              }
            }
#pragma unroll
            for (int w = 0; w < EPL / 2; ++w) {
              const u32 even = __builtin_amdgcn_perm(v1[w], v0[w], 0x05040100u);  // dim 2w of both rows
              const u32 odd = __builtin_amdgcn_perm(v1[w], v0[w], 0x07060302u);   // dim 2w+1
#pragma unroll
              for (int h = 0; h < G; ++h) {
                acc[h][j * EPL + 2 * w] = QT::dot2(even, pp[up][h], acc[h][j * EPL + 2 * w]);
                acc[h][j * EPL + 2 * w + 1] = QT::dot2(odd, pp[up][h], acc[h][j * EPL + 2 * w + 1]);
              }
            }
          }
        }
      };

      auto compute = [&](const Tile& t, int step) {
        if (ragged && step == n_steps - 1) compute_tile(t, step, std::true_type{});
        else compute_tile(t, step, std::false_type{});
      };

      // Steps are dealt round-robin to the wavefronts; three register tiles rotate so that the
      // loads of the next two steps are in flight while the current one is reduced.  Every
      // iteration issues its prefetch unconditionally (past the end it re-reads the last
      // step), so the number of loads in flight at each use is a compile-time constant and
      // the compiler can wait for exactly the tile it needs instead of draining the queue.
      int step = wave;
      if (step < n_steps) {
        const int last = n_steps - 1;
        Tile ta, tb, tc;
        load_tile(ta, step);
        load_tile(tb, min(step + kWaves, last));
        while (true) {
          load_tile(tc, min(step + 2 * kWaves, last));
          compute(ta, step);
          step += kWaves;
          if (step >= n_steps) break;
          load_tile(ta, min(step + 2 * kWaves, last));
          compute(tb, step);
          step += kWaves;
          if (step >= n_steps) break;
          load_tile(tb, min(step + 2 * kWaves, last));
          compute(tc, step);
          step += kWaves;
          if (step >= n_steps) break;
        }
      }
    }

    // ---- end of the run: one head at a time every lane row publishes its state and the
    // workgroup folds the NP states into the output or into a partial
    float out_scale = 1.0f;
    if constexpr (FP8) out_scale = a.v_scale[kvh];
    const int pi = wave * TPP + r;
    const int64_t pslot = static_cast<int64_t>(blockIdx.x) * 2 + (first_run ? 0 : 1);
#pragma unroll
    for (int h = 0; h < G; ++h) {
      __syncthreads();  // the slot list / the previous head's states have been consumed
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
      fold_states<QT, D, NP>(a, part, tid, h < nh, complete, b, h0 + h, pslot * G + h, out_scale);
    }
    first_run = false;
  }
}

// Merge of the partials of contexts that span several workgroups; also writes the output
// of empty sequences.  One workgroup per (query head, sequence).
template <typename QT>
__global__ __launch_bounds__(128) void merge_partials_kernel(GqaArgs a, int dv) {
  const int hq = blockIdx.x;
  const int b = blockIdx.y;
  const int G = a.g_block;
  const int32_t* pages;
  int L;
  sequence_of(a, b, pages, L);
  uint16_t* out = reinterpret_cast<uint16_t*>(a.out + b * a.out_stride_bytes) + hq * dv;
  if (L <= 0) {
    for (int d = threadIdx.x; d < dv; d += 128) out[d] = 0;
    if (a.lse != nullptr && threadIdx.x == 0) a.lse[b * a.n_q_heads + hq] = -INFINITY;
    return;
  }
  const int hb_per_kv = (a.group + G - 1) / G;
  const int n_hb = a.n_kv_heads * hb_per_kv;
  const int kvh = hq / a.group;
  const int hbk = kvh * hb_per_kv + (hq - kvh * a.group) / G;
  const int h = (hq - kvh * a.group) % G;
  const int64_t total = static_cast<int64_t>(a.ws_prefix[a.batch]) * n_hb;
  const int n_items = a.ws_prefix[b + 1] - a.ws_prefix[b];
  const int64_t first = static_cast<int64_t>(a.ws_prefix[b]) * n_hb + static_cast<int64_t>(hbk) * n_items;
  const int64_t last = first + n_items - 1;
  const int64_t n_wg = a.n_workgroups;
  const int w_first = workgroup_of(first, total, n_wg);
  const int w_last = workgroup_of(last, total, n_wg);
  if (w_first == w_last) return;  // one workgroup saw the whole context and wrote the output
  // the first workgroup holds this context as its last run (slot 1) unless its range starts
  // exactly here; every later one holds it as its first run (slot 0)
  const int slot_first = range_start(w_first, total, n_wg) < first ? 1 : 0;
  auto pslot = [&](int w) { return static_cast<int64_t>(w) * 2 + (w == w_first ? slot_first : 0); };
  // with fewer items than workgroups some ranges in between are empty and own no partial
  auto has_items = [&](int w) { return range_start(w, total, n_wg) < range_start(w + 1, total, n_wg); };
  float mx = kNegBig;
  for (int w = w_first; w <= w_last; ++w)
    if (has_items(w)) mx = fmaxf(mx, a.ws_lse[pslot(w) * G + h]);
  float wsum = 0.0f;
  for (int w = w_first; w <= w_last; ++w)
    if (has_items(w)) wsum += fast_exp2(a.ws_lse[pslot(w) * G + h] - mx);
  const float inv = 1.0f / wsum;
  for (int d = threadIdx.x; d < dv; d += 128) {
    float o = 0.0f;
    for (int w = w_first; w <= w_last; ++w) {
      if (!has_items(w)) continue;
      const int64_t ps = pslot(w) * G + h;
      o += fast_exp2(a.ws_lse[ps] - mx) * a.ws_out[ps * dv + d];
    }
    out[d] = QT::from_f32(o * inv);
  }
  if (a.lse != nullptr && threadIdx.x == 0) a.lse[b * a.n_q_heads + hq] = (mx + fast_log2(wsum)) * kLn2;
}

int device_cu_count() {
  static const int n = [] {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) return 256;
    return p.multiProcessorCount > 0 ? p.multiProcessorCount : 256;
  }();
  return n;
}

template <typename QT, bool FP8, int D, int LPT, int G, int U>
int launch_gqa(GqaArgs& a, size_t workspace_bytes, hipStream_t stream, bool plan_only, size_t* need) {
  constexpr int NP = kWaves * (kWave / LPT);
  auto kern = gqa_decode_kernel<QT, FP8, D, LPT, G, U>;
  const size_t smem = kSub * 4 + static_cast<size_t>(NP) * (D + 2) * 4 + kThreads * 4 +
                      (static_cast<size_t>(a.batch) + 1) * 4;
  static const int per_cu = [&] {
    const char* e = getenv("XLLM_MI355_GQA_WGS_PER_CU");  // tuning knob
    if (e != nullptr && atoi(e) > 0) return atoi(e);
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(kern), kThreads,
                                                     kSub * 4 + NP * (D + 2) * 4 + kThreads * 4 + 1028) != hipSuccess || n < 1)
      n = 2;
    return n;
  }();
  a.n_workgroups = device_cu_count() * per_cu;
  const size_t prefix_bytes = ((static_cast<size_t>(a.batch) + 1) * 4 + 255) / 256 * 256;
  const size_t part_floats = static_cast<size_t>(a.n_workgroups) * 2 * G * (D + 1);
  *need = prefix_bytes + part_floats * 4;
  if (plan_only) return XLLM_MI355_OK;
  if (*need > workspace_bytes) return XLLM_MI355_EWORKSPACE;
  a.ws_out = reinterpret_cast<float*>(reinterpret_cast<char*>(a.ws_prefix) + prefix_bytes);
  a.ws_lse = a.ws_out + static_cast<size_t>(a.n_workgroups) * 2 * G * D;
  const bool timed = profile_begin(stream);
  kern<<<dim3(static_cast<unsigned>(a.n_workgroups)), kThreads, smem, stream>>>(a);
  if (timed) profile_end(stream);
  return static_cast<int>(hipGetLastError());
}

template <typename QT, bool FP8, int D, int LPT, int U>
int dispatch_group(GqaArgs& a, size_t wsb, hipStream_t s, bool plan_only, size_t* need) {
  switch (a.g_block) {
    case 1: return launch_gqa<QT, FP8, D, LPT, 1, U>(a, wsb, s, plan_only, need);
    case 2: return launch_gqa<QT, FP8, D, LPT, 2, U>(a, wsb, s, plan_only, need);
    case 4: return launch_gqa<QT, FP8, D, LPT, 4, U>(a, wsb, s, plan_only, need);
    default: return launch_gqa<QT, FP8, D, LPT, 8, (U > 2 ? U / 2 : U)>(a, wsb, s, plan_only, need);
  }
}

template <typename QT, bool FP8>
int dispatch_dim(GqaArgs& a, int head_dim, size_t wsb, hipStream_t s, bool plan_only, size_t* need) {
  // lanes per token row: one 16-byte load per lane and row
  if constexpr (FP8) {
    switch (head_dim) {
      case 64: return dispatch_group<QT, true, 64, 4, 2>(a, wsb, s, plan_only, need);
      case 128: return dispatch_group<QT, true, 128, 8, 2>(a, wsb, s, plan_only, need);
      case 256: return dispatch_group<QT, true, 256, 16, 4>(a, wsb, s, plan_only, need);
      default: return XLLM_MI355_ESHAPE;
    }
  } else {
    switch (head_dim) {
      case 64: return dispatch_group<QT, false, 64, 8, 2>(a, wsb, s, plan_only, need);
      case 128: return dispatch_group<QT, false, 128, 16, 4>(a, wsb, s, plan_only, need);
      case 256: return dispatch_group<QT, false, 256, 32, 4>(a, wsb, s, plan_only, need);
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

size_t gqa_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t head_dim) {
  // Upper bound over every kernel variant: at most 8 workgroups per CU, 8 heads per block.
  (void)n_q_heads;
  const size_t b = static_cast<size_t>(batch < kMaxBatch ? batch : kMaxBatch);
  const size_t prefix_bytes = ((b + 1) * 4 + 255) / 256 * 256;
  return prefix_bytes + static_cast<size_t>(device_cu_count()) * 8 * 2 * 8 * (head_dim + 1) * 4;
}

int paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache, void* out, float* lse,
                     const PageAddressing& addr, const float* k_scale, const float* v_scale,
                     int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                     int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                     int64_t out_token_stride, int64_t max_seq_len, float sm_scale, void* workspace,
                     size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream) {
  (void)max_seq_len;  // the schedule is computed on the device from the actual lengths
  if (batch == 0) return XLLM_MI355_OK;
  if (q == nullptr || k_cache == nullptr || v_cache == nullptr || out == nullptr) return XLLM_MI355_EINVAL;
  const bool csr = addr.indptr != nullptr;
  if (csr ? (addr.indices == nullptr || addr.last_page_len == nullptr)
          : (addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0))
    return XLLM_MI355_EINVAL;
  if (batch < 0 || n_q_heads <= 0 || n_kv_heads <= 0 || block_size <= 0 || num_blocks <= 0 ||
      n_q_heads % n_kv_heads != 0 || n_q_heads > 65535 || !(sm_scale > 0.0f))
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
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return XLLM_MI355_EWORKSPACE;

  const int group = static_cast<int>(n_q_heads / n_kv_heads);
  // Batches beyond the LDS prefix capacity are decoded in slices; each slice is an
  // independent launch pair on the same stream and workspace.
  for (int64_t b0 = 0; b0 < batch; b0 += kMaxBatch) {
    const int64_t nb = batch - b0 < kMaxBatch ? batch - b0 : kMaxBatch;
    GqaArgs a = {};
    a.q = static_cast<const char*>(q) + b0 * q_token_stride * 2;
    a.k_cache = static_cast<const char*>(k_cache);
    a.v_cache = static_cast<const char*>(v_cache);
    a.out = static_cast<char*>(out) + b0 * out_token_stride * 2;
    a.lse = lse == nullptr ? nullptr : lse + b0 * n_q_heads;
    a.block_table = csr ? nullptr : addr.block_table + b0 * addr.table_stride;
    a.seq_lens = csr ? nullptr : addr.seq_lens + b0;
    a.indptr = csr ? addr.indptr + b0 : nullptr;
    a.indices = addr.indices;
    a.last_page_len = csr ? addr.last_page_len + b0 : nullptr;
    a.k_scale = k_scale;
    a.v_scale = v_scale;
    a.ws_prefix = static_cast<int*>(workspace);
    a.table_stride = addr.table_stride;
    a.q_stride_bytes = q_token_stride * 2;
    a.out_stride_bytes = out_token_stride * 2;
    a.row_bytes = n_kv_heads * head_dim * (fp8 ? 1 : 2);
    a.batch = static_cast<int>(nb);
    a.n_q_heads = static_cast<int>(n_q_heads);
    a.n_kv_heads = static_cast<int>(n_kv_heads);
    a.group = group;
    a.g_block = group_block(group);
    a.block_size = static_cast<int>(block_size);
    a.bs_shift = -1;
    for (int s = 0; s < 31; ++s)
      if ((1LL << s) == block_size) a.bs_shift = s;
    a.num_blocks = static_cast<int>(num_blocks);
    a.scale_log2 = sm_scale * kLog2e;

    size_t need = 0;
    int rc;
    if (q_dtype == XLLM_MI355_BF16)
      rc = fp8 ? dispatch_dim<BF16, true>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need)
               : dispatch_dim<BF16, false>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need);
    else
      rc = fp8 ? dispatch_dim<FP16, true>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need)
               : dispatch_dim<FP16, false>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need);
    if (rc != 0) return rc;
    dim3 grid(static_cast<unsigned>(n_q_heads), static_cast<unsigned>(nb));
    if (q_dtype == XLLM_MI355_BF16)
      merge_partials_kernel<BF16><<<grid, 128, 0, stream>>>(a, static_cast<int>(head_dim));
    else
      merge_partials_kernel<FP16><<<grid, 128, 0, stream>>>(a, static_cast<int>(head_dim));
    rc = static_cast<int>(hipGetLastError());
    if (rc != 0) return rc;
  }
  return XLLM_MI355_OK;
}

}  // namespace xllm_mi355
