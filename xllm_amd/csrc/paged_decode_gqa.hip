// Paged decode attention, GQA, for gfx950.
//
// Scheduling (both kernels of this file).  The context of every (sequence, KV-head block) is cut
// into items; the items of the whole batch form one flat list ordered (sequence, head block,
// item).  A fixed set of persistent workers splits that list into equal contiguous ranges, so
// every worker streams the same number of KV bytes whatever the mix of context lengths, and a
// worker keeps its online softmax state in registers for as long as it stays inside one
// (sequence, head block).  A run of items that covers a whole context writes the output
// directly; a run that covers part of one (only the first and the last run of a worker can)
// writes a normalised fp32 partial + log2-domain LSE, and a small merge kernel folds those.
// The item counts are prefix-summed inside every workgroup (no extra launch, no host read).
//
// gqa_mfma_kernel (head_dim 128, or 64 with 16-bit pages; block size a power of two >= 16): worker = a loading
// and a computing wavefront, item = 16 tokens (32 for rows of 128 bytes: fp8 pages, head_dim 64); rows travel global memory -> LDS directly into a
// private ring per worker and both products run on the matrix cores.  Its own comment below has the
// details.
//
// gqa_decode_kernel (every other shape): worker = workgroup, item = 64 tokens, the 4 wavefronts
// of a workgroup take steps round-robin:
//   * a token's [D] row of one KV head is read by LPT adjacent lanes with one 16-byte
//     load each (64/LPT tokens per load instruction), K and V alike, so every load
//     instruction covers whole contiguous rows of the [P, bs, Hkv, D] pages; three register
//     tiles rotate so the next steps' loads fly while the current step is reduced;
//   * q.k is v_dot2 on packed 16-bit pairs into fp32, reduced over the LPT lanes by DPP
//     row operations; all G query heads of the KV head reuse the same K registers;
//   * p.v is v_dot2 as well: V words of two consecutive token rows are byte-permuted into
//     (token, token+1) pairs and dotted with the packed pair of probabilities;
//   * each row of LPT lanes keeps its own running (max, sum, acc); the accumulator is
//     rescaled only on steps where some maximum moved; rows and wavefronts are merged
//     through LDS once per run;
//   * fp8 pages are converted to 16-bit pairs in registers (exact), the per-head scales are
//     folded into the score scale (K) and the output (V);
//   * the page walk reads slot ids (page * bs + row) staged in LDS per 2048 tokens, so the
//     loop has no division and never touches table columns past ceil(L / bs).
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
constexpr int kMaxBatch = kWsMaxBatch;  // sequences per launch (their item prefix lives in LDS)

struct GqaArgs {
  const char* q;
  const char* k_cache;
  const char* v_cache;
  char* k_cache_w;   // the same caches, writable (write-then-attend only)
  char* v_cache_w;
  char* out;
  float* lse;
  const int32_t* block_table;
  const int32_t* table_rows;  // block-table row of each batch entry, or null for row b (several query tokens of a sequence)
  const int32_t* cu_q;        // packed query chunks (matrix-core kernel only): [batch + 1] token offsets, or null
  int n_tokens;               // rows of q / out in that case
  int chunk_blocks;           // column blocks per KV head in that case: ceil(longest chunk * group / 16)
  int causal;                 // query token j of a chunk of n attends to the first L - n + j + 1 tokens
  const int32_t* seq_lens;
  const int32_t* indptr;
  const int32_t* indices;
  const int32_t* last_page_len;
  const float* k_scale;
  const float* v_scale;
  int* ws_status;  // status flags of the workspace (kStatus*), only ever OR-ed into
  unsigned* ws_arrivals;  // one counter per worker (zero between launches): pieces of the context that starts in its range
  int fold_merge;  // the matrix-core kernel merges a context's partials itself (last piece to arrive) and writes empty rows
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
  int n_workgroups;   // workers of the decode kernel (workgroups; wavefront pairs of the matrix-core kernel)
  // Matrix-core kernel: this many workers of a workgroup (1, 2 or 4) walk the same stages of adjacent head blocks
  // side by side, so that the rows they ask for at the same time are neighbours in memory (a token's rows of all KV
  // heads are contiguous in a page), or the same rows (head blocks of one KV head).  A plain streaming kernel reads 128-byte pieces that lie 1 KB apart at 5.8 TB/s
  // when the neighbouring pieces are fetched at other times by other workgroups, at 6.7 TB/s when two wavefronts of a
  // workgroup fetch adjacent pieces together (the rate of 256-byte pieces) and at 7.0 TB/s with four.  The flat list
  // then holds (sequence, group of head blocks, stage) and is dealt to groups of workers.  The workers of a group
  // start together and are left to themselves: made to wait for each other (stage i only after all have issued stage
  // i - 1, or i - 3, or i - 9) they were 1-2 % slower than free, which is 2-5 % faster than apart.
  int head_lock;
  // Matrix-core kernel: the flat list is cut in two, in the ratio pool_even : pool_odd, and the first part dealt to
  // the workgroups whose index is even modulo 8, the second to the others.  A tuned default, not a fact the results
  // rest on: on the full MI355X (256 CUs, workgroup i dispatched to XCD i % 8) the workgroups on the odd XCDs were
  // seen to stream their rows 8-11 % slower with equal shares, and 9 : 8 ends the decode kernels 1.7-2.7 % earlier; a
  // device that dispatches otherwise only loses that gain (the merge walks whatever cut the decode kernel used).  The
  // host sets it only for a device of 256 CUs; 0 : 0 = one list.
  int pool_even, pool_odd;
  // Matrix-core kernel: a plan of the step, made once by gqa_plan_kernel for all layers (see kPlan*), or null: the
  // item prefix, the cut between the pools and, for every group of workers, the 64 page-table entries its first
  // stage needs.  With it the kernel's start is one trip to memory (prefix, lengths and pages together), then rows,
  // instead of three in a row (lengths -> prefix -> pages of the range's first context) before the first row moves.
  const int* plan;
  int plan_sig;       // what the plan must have been made for (plan_signature), checked against the plan's own word
  // Matrix-core kernel: output rows and partial rows leave with non-temporal stores (written through, no line kept in
  // L2).  With ordinary stores a launch that ends many runs (many sequences, many heads) has workers that are held up
  // after a run's stores and at their exit: on 256 sequences x 64 heads the last worker leaves at 487-491 us instead
  // of 502-507 us and the launch takes 2 % less; all stores have to be non-temporal for that (only those in the
  // middle of a range, or only those at its end, changed nothing).  Launches with few run ends lose 1-1.5 % (64
  // sequences x 32 heads: 91.1 -> 92.3 us, and the merge kernel, which then finds no partial in L2, 5.2 -> 5.5 us), so
  // the host turns it on from 8192 output rows (sequences x heads) per launch.
  int stream_stores;
  // Write-then-attend in one launch: the step's new K / V rows [batch, Hkv, D] of the query's 16-bit type (token strides
  // in bytes) and their slots, or null.  The worker that reaches the last stage of (sequence, KV head) puts the new
  // row where the stage expects it in LDS (quantised for fp8 pages, over whatever the loader fetched from the slot
  // that is not written yet) and writes the same bytes to the cache: what reshape_and_cache would have written before
  // the launch.  Slots outside [0, n_slots) are skipped, as there.
  const char* new_k;
  const char* new_v;
  const int32_t* new_slots;
  int64_t new_k_stride_bytes, new_v_stride_bytes;
  int64_t n_slots;
  int wait_spins;     // bound of the polls of one wavefront of a pair on the other
  int window_left;    // sliding window: the query (position L - 1) attends to positions >= L - 1 - window_left; < 0: all
  float scale_log2;   // sm_scale * log2(e)
};

__device__ __forceinline__ void sequence_of(const GqaArgs& a, int b, const int32_t*& pages, int& L) {
  if (a.indptr != nullptr) {
    const int p0 = a.indptr[b];
    const int np = a.indptr[b + 1] - p0;
    pages = a.indices + p0;
    L = np > 0 ? (np - 1) * a.block_size + a.last_page_len[b] : 0;
  } else {
    pages = a.block_table + static_cast<int64_t>(a.table_rows != nullptr ? a.table_rows[b] : b) * a.table_stride;
    L = a.seq_lens[b];
  }
}

// First token a query at position L - 1 attends to (0 without a sliding window).
__device__ __forceinline__ int first_token(const GqaArgs& a, int L) {
  return a.window_left < 0 ? 0 : max(0, L - 1 - a.window_left);
}
// Items of a context: those that hold a token of the attended range [first_token, L).
template <int ITEM>
__device__ __forceinline__ int items_of(const GqaArgs& a, int L) {
  return L > 0 ? (L + ITEM - 1) / ITEM - first_token(a, L) / ITEM : 0;
}

// First flat item of workgroup w when `total` items are dealt to `n` workgroups.
// (a 64-bit division is a long instruction sequence on this GPU, and these sit on the dependent chains at the start
// of the decode and merge kernels: 32 bits whenever the products fit, which they do unless a batch holds more than a
// million items)
__device__ __forceinline__ int64_t range_start(int64_t w, int64_t total, int64_t n) {
  if (total * n < (1LL << 31)) return static_cast<uint32_t>(w) * static_cast<uint32_t>(total) / static_cast<uint32_t>(n);
  return w * total / n;
}

// With fewer items than workers only the first `total` workers take part (one item each): no range in the middle of
// the list is ever empty, and the merge need not ask which ones are.
__device__ __forceinline__ int64_t used_workers(int64_t n, int64_t total) { return total < n ? total : n; }

// The workgroup whose range holds flat item `id`.
__device__ __forceinline__ int workgroup_of(int64_t id, int64_t total, int64_t n) {
  int64_t w = total * n < (1LL << 31) ? static_cast<int64_t>(static_cast<uint32_t>(id) * static_cast<uint32_t>(n) / static_cast<uint32_t>(total))
                                      : id * n / total;
  while (w + 1 < n && range_start(w + 1, total, n) <= id) ++w;
  return static_cast<int>(w);
}

// The two pools of GqaArgs::pool_even / pool_odd.  Groups of workers ("teams", `per` of them in a workgroup) are
// numbered pool by pool: index q of pool `par` (0: even XCDs, 1: odd XCDs) <-> team of_pool(par, q).
struct Pools {
  int64_t total, cut;  // the flat list and where the second pool's part begins
  int half, per_shift; // teams per pool; log2 of the teams per workgroup (1, 2 or 4 of them)
  __device__ __forceinline__ int64_t size(int par) const { return par ? total - cut : cut; }
  __device__ __forceinline__ int64_t base(int par) const { return par ? cut : 0; }
  __device__ __forceinline__ int of_pool(int par, int q) const {
    const int r = q >> per_shift, o = q - (r << per_shift);
    return (((r >> 2) * 8 + (r & 3) * 2 + par) << per_shift) + o;
  }
  __device__ __forceinline__ void of_team(int team, int& par, int& q) const {
    const int g = team >> per_shift, o = team - (g << per_shift), xcd = g & 7;
    par = xcd & 1;
    q = (((g >> 3) * 4 + (xcd >> 1)) << per_shift) + o;
  }
};
__device__ __forceinline__ int64_t pool_cut(const GqaArgs& a, int64_t total) {
  return total * a.pool_even / (a.pool_even + a.pool_odd);
}
// (the merge kernel takes the cut that the decode kernel left behind the item prefix: no division there)
__device__ __forceinline__ Pools make_pools(const GqaArgs& a, int64_t total, int64_t cut) {
  Pools p;
  p.total = total;
  p.cut = cut;
  p.per_shift = a.head_lock == 4 ? 0 : a.head_lock == 2 ? 1 : 2;   // (kWaves = 4 workers in a workgroup)
  p.half = a.n_workgroups / a.head_lock / 2;
  return p;
}

// The range [cur, end) of the flat list that group of workers `team` of `n_teams` takes; false: none.
__device__ __forceinline__ bool team_range(const GqaArgs& a, int64_t total, int64_t cut, int64_t team, int64_t n_teams,
                                           int64_t& cur, int64_t& end) {
  if (a.pool_even != 0) {   // the list in two parts: one for the teams on even XCDs, one for those on odd XCDs
    const Pools pools = make_pools(a, total, cut);
    int par, q;
    pools.of_team(static_cast<int>(team), par, q);
    const int64_t n_use = used_workers(pools.half, pools.size(par));
    if (q >= n_use) return false;
    cur = pools.base(par) + range_start(q, pools.size(par), n_use);
    end = pools.base(par) + range_start(q + 1, pools.size(par), n_use);
  } else {
    const int64_t n_use = used_workers(n_teams, total);
    if (team >= n_use) return false;
    cur = range_start(team, total, n_use);
    end = range_start(team + 1, total, n_use);
  }
  return cur < end;
}

// Exclusive prefix sum of the per-sequence item counts into prefix[0..batch] (LDS).
// Every thread sums a contiguous slice, then adds the totals of the slices before it.  Threads past
// kThreads (the matrix-core kernel has a wavefront of them) only take part in the barriers.
template <int ITEM>
__device__ __forceinline__ void item_prefix(const GqaArgs& a, int* prefix, int* tmp, int* lens = nullptr) {
  const int tid = threadIdx.x;
  const bool on = tid < kThreads;
  const int per = (a.batch + kThreads - 1) / kThreads;
  const int lo = on ? min(a.batch, tid * per) : a.batch, hi = min(a.batch, lo + per);
  int local = 0, last_len = 0;
  for (int b = lo; b < hi; ++b) {
    const int32_t* pages;
    int L;
    sequence_of(a, b, pages, L);
    local += items_of<ITEM>(a, L);
    last_len = L;
  }
  // scan inside the wavefront, then over the wavefronts' totals (a thread that summed the counts of all threads before
  // it one by one took 2.5 us at 256 sequences, and every worker waits for the prefix)
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  int incl = local;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int t = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += t;
  }
  if (on && lane == kWave - 1) tmp[wave] = incl;
  if (lens != nullptr && per == 1 && lo < hi) lens[lo] = last_len;  // (kept for the workers: saves them a load each)
  __syncthreads();
  if (lo < hi) {  // (threads without a slice have nothing to place: most of them at decode batch sizes)
    int excl = incl - local;
    for (int w = 0; w < wave; ++w) excl += tmp[w];
    if (per == 1) {  // the slice is one sequence: its count is still in `local`
      prefix[lo] = excl;
      excl += local;
    } else {
      for (int b = lo; b < hi; ++b) {
        const int32_t* pages;
        int L;
        sequence_of(a, b, pages, L);
        prefix[b] = excl;
        excl += items_of<ITEM>(a, L);
      }
    }
    if (hi == a.batch) prefix[a.batch] = excl;  // the last non-empty slice holds the total
  }
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

  item_prefix<kItem>(a, prefix, tmp);
  const int64_t total = static_cast<int64_t>(prefix[a.batch]) * n_hb;
  if (blockIdx.x == 0) {
    for (int i = tid; i <= a.batch; i += kThreads) a.ws_prefix[i] = prefix[i];
  }
  if (total == 0) return;
  const int64_t n_wg = used_workers(gridDim.x, total);
  if (blockIdx.x >= n_wg) return;
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
    const int win_lo = first_token(a, L);   // tokens before it lie outside the sliding window
    const int item_lo = win_lo / kItem;     // first item of the context that is scheduled
    const int run_t0 = (item_lo + item0) * kItem;
    const int run_t1 = min(L, (item_lo + item0 + run_items) * kItem);

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
            t.k[u][j] = ldg16_stream(kbase + off + j * (LPT * 16));
            t.v[u][j] = ldg16_stream(vbase + off + j * (LPT * 16));
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
            if (t0 + step * STEP + u * TPP + r >= t1 || t0 + step * STEP + u * TPP + r < win_lo) {
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
        if ((ragged && step == n_steps - 1) || t0 + step * STEP < win_lo) compute_tile(t, step, std::true_type{});
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

// ---------------------------------------------------------------------------------------------
// Matrix-core variant, described for D = 128 with 16-bit pages (fp8 pages and D = 64 differ in the
// number of tokens per stage and are noted where they do).
//
// A worker is a PAIR of wavefronts that share a SIMD: wavefront w of the workgroup loads, wavefront
// kWaves + w computes.  A wavefront cannot issue more than one load-to-LDS instruction per 90 ns or
// so (0.75-0.85 us for the 8 of a stage) and does nothing else while it issues; in one wavefront the
// 0.3-0.5 us of arithmetic per stage came on top of that, which is more than the memory system leaves
// a wavefront per stage (1.15 us at 7.1 TB/s over 1024 workers).  The two meet in two LDS counters:
// stages whose loads have completed (the computing wavefront cannot wait on loads it did not issue)
// and stages whose ring slot has been given back.  A worker owns a contiguous range of the flat item
// list, keeps its own softmax state, and never meets the other workers of its workgroup after the
// common item prefix sum, so there is no barrier anywhere in the streaming loop.
//
// Data path.  A stage is 16 tokens of one KV head (32 for fp8 pages): K rows, then V rows, 8 KB.
// Stages travel from global memory straight into the worker's private LDS ring
// (global_load_lds_dwordx4, 16 adjacent lanes per 256-byte row so every instruction reads whole
// contiguous rows), NS stages deep, NS - 1 in flight while one is consumed.  Within a row the
// 16-byte chunks are XOR-swizzled so that both operand reads below touch every LDS bank once.
//   S^T[tok, head] = K[tok, 128] . Q^T[128, head]   v_mfma_f32_16x16x32: A = K rows read from LDS
//                                                   (16 bytes per lane), B = Q^T resident in registers
//   O^T[dim, head] += V^T[dim, tok] . P^T[tok, head] v_mfma_f32_16x16x16: A = V^T through the
//                                                   transposing LDS read, B = P^T taken from the
//                                                   S^T accumulator registers as they are
// fp8 pages are converted to 16-bit after the LDS read (exact); their V^T comes through the 8-bit
// transposing read (within 16 lanes, result lane i element j = input lane 2j + i/8, element
// i%8) and P.V runs on the 16x16x32 MFMA over both score blocks of the stage.
// Up to 16 query heads of the KV head ride in the MFMA columns (heads past the group are zero
// columns), so a lane owns one head: its running maximum and sum are plain per-lane scalars.
// The maximum only moves when a score exceeds it by more than kSlack (log2 units).
//
// Nothing in the loading wavefront waits on a register load from global memory: such a wait would also
// wait for every younger stage in flight (the counter is in order).  Page-table entries (64 at a
// time: the current chunk, the next one, and the first one of the next context), the Q rows of
// the next context and the stages all take the LDS path and are covered by one explicit wait per
// stage; sequence lengths and fp8 scales come through the scalar cache.  Loads that write
// registers are never issued from inline assembly: the register allocator does not know they
// are pending and may hand their destination to something else.
constexpr float kSlack = 8.0f;
constexpr int kStageBytes = 8192;  // K rows then V rows: 16 tokens of 16-bit pages, 32 of fp8 pages
constexpr int kMfmaHeads = 16;                        // head columns of one MFMA

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef __attribute__((address_space(3))) volatile int lds_vint;  // a word of LDS that other wavefronts write
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) u32x2 lds_u32x2;

// 16 (4) bytes per lane from global memory straight into LDS at lds_addr + lane * 16 (4);
// lds_addr is wave-uniform and travels in M0.
__device__ __forceinline__ void dma16(const void* gptr, u32 lds_addr) {
  const u32 base = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(base), "v"(gptr) : "memory");
}
__device__ __forceinline__ void dma4(const void* gptr, u32 lds_addr) {
  const u32 base = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(base), "v"(gptr) : "memory");
}
// Same as dma16 with a wave-uniform 64-bit base in SGPRs plus a 32-bit per-lane byte offset, and marked
// non-temporal: the rows of the cache are read once per launch, and streaming them past the caches
// instead of through them is worth 15 % of read bandwidth on this GPU (7.0-7.1 TB/s against 6.1-6.25 TB/s
// for a plain load of the same pattern).
__device__ __forceinline__ void dma16_row(uint64_t base, u32 lane_off, u32 lds_addr) {
  const u32 m0 = __builtin_amdgcn_readfirstlane(lds_addr);
  const u32 lo = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(base)));
  const u32 hi = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(base >> 32)));
  const uint64_t sb = (static_cast<uint64_t>(hi) << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m0), "v"(lane_off), "s"(sb) : "memory");
}
// Wait until at most 8 * stages of the wavefront's vector memory operations are outstanding.
__device__ __forceinline__ void wait_younger_stages(int stages) {
  if (stages <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if (stages == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (stages == 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
}
// One dword through the scalar cache (wave-uniform address); does not touch the vector memory counter.
__device__ __forceinline__ int sload32(const int32_t* p) {
  const uint64_t x = reinterpret_cast<uint64_t>(p);
  // (the builtin returns a signed int: each half goes through u32 so the low one is not sign-extended)
  const u32 lo = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(x)));
  const u32 hi = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(x >> 32)));
  const uint64_t u = (static_cast<uint64_t>(hi) << 32) | lo;
  int v;
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(u) : "memory");
  return v;
}
__device__ __forceinline__ void sequence_of_scalar(const GqaArgs& a, int b, const int32_t*& pages, int& L) {
  if (a.indptr != nullptr) {
    const int p0 = sload32(a.indptr + b);
    const int np = sload32(a.indptr + b + 1) - p0;
    pages = a.indices + p0;
    L = np > 0 ? (np - 1) * a.block_size + sload32(a.last_page_len + b) : 0;
  } else {
    pages = a.block_table + static_cast<int64_t>(a.table_rows != nullptr ? sload32(a.table_rows + b) : b) * a.table_stride;
    L = sload32(a.seq_lens + b);
  }
}
__device__ __forceinline__ float quad_rows_max(float x) {  // over lanes l, l ^ 16, l ^ 32, l ^ 48
  auto t = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
  x = fmaxf(as_f32(t[0]), as_f32(t[1]));
  auto u = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
  return fmaxf(as_f32(u[0]), as_f32(u[1]));
}
__device__ __forceinline__ float quad_rows_sum(float x) {
  auto t = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
  x = as_f32(t[0]) + as_f32(t[1]);
  auto u = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
  return as_f32(u[0]) + as_f32(u[1]);
}

// Position of a stage in the flat list (sequence, head block, stage of 16 tokens).
struct CtxCursor {
  int b, hbk, st, n_st;
  int st0;  // first scheduled stage of the context (stages before it lie outside the sliding window)
  int kvh;  // KV head of the head block: hbk / (head blocks per KV head)
  int L;
  const int32_t* pages;
  // packed query chunks: the sequence's chunk (first query token, number of tokens), and the part of it that
  // the column block hbk % chunk_blocks holds: its first token, its number of tokens, and the index of its
  // first token inside the chunk
  int Q0, QN, q0, qn, jb;
  int QF;  // the chunk's full length (QN is cut to what the column blocks hold): the causal offset counts from it
};
// Field by field, and the chunk fields only where they are in use: a whole-struct copy with fields that
// were never written goes through scratch memory, whose loads count on the same counter as the stages
// in flight.
template <bool VL>
__device__ __forceinline__ void copy_cursor(CtxCursor& d, const CtxCursor& s) {
  d.b = s.b;
  d.hbk = s.hbk;
  d.kvh = s.kvh;
  d.st = s.st;
  d.st0 = s.st0;
  d.n_st = s.n_st;
  d.L = s.L;
  d.pages = s.pages;
  if constexpr (VL) {
    d.Q0 = s.Q0;
    d.QN = s.QN;
    d.QF = s.QF;
    d.q0 = s.q0;
    d.qn = s.qn;
    d.jb = s.jb;
  }
}

constexpr int kMfmaThreads = 2 * kThreads;   // kWaves loading wavefronts and kWaves computing wavefronts

template <typename QT, bool VL, bool COHERENT = false>
__device__ __forceinline__ void merge_context(const GqaArgs& a, int dv, int hbk, int b, int tid, int nthreads,
                                              int p0, int p1, int pt, int cut = 0);
// Words of the partials that workers exchange inside one launch: relaxed atomics at device scope, which go to
// the level of the memory system that all CUs share (the L2 of an XCD is not coherent with the other seven; a
// fence that makes it so writes back and invalidates the whole L2, 60 us per launch when 1024 workers do it).
__device__ __forceinline__ void store_shared(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int NS, int D = 128>
struct MfmaLayout {
  // LDS: ring [waves][NS][stage] | Q rows [waves][16][kQRow B] | page-table chunks [waves][3][64] |
  //      scan scratch [kThreads] | progress counters [waves][2] | context lengths [kThreads] |
  //      stage prefix [batch + 1]
  static constexpr int kRingBytes = kWaves * NS * kStageBytes;
  static constexpr int kQRow = D * 2 > 256 ? D * 2 : 256;
  static constexpr int kQOff = kRingBytes;
  static constexpr int kPageOff = kQOff + kWaves * kMfmaHeads * kQRow;
  static constexpr int kTmpOff = kPageOff + kWaves * 3 * kWave * 4;
  static constexpr int kSyncOff = kTmpOff + kThreads * 4;
  static constexpr int kLensOff = kSyncOff + 2 * kWaves * 4;   // context lengths of up to kThreads sequences
  static constexpr int kPrefixOff = kLensOff + kThreads * 4;
};

// VL (packed query chunks): a batch entry is a sequence with cu_q[b + 1] - cu_q[b] query tokens.  The 16 MFMA
// columns hold (token j, head h) pairs, column j * group + h, all against the same pages: 16 / group tokens
// per column block, chunk_blocks column blocks per KV head, so a chunk costs the page traffic of
// ceil(tokens * group / 16) single tokens; column j is masked beyond its own length.
// D = 64 (16-bit pages only): rows of 128 bytes, so a stage holds 32 tokens and is multiplied as two blocks
// of 16 like an fp8 stage, with 2 k-steps per score block and 4 dim blocks.
// D = 64 with fp8 pages: rows of 64 bytes, a stage holds 64 tokens and is multiplied as two halves of 32, each like
// an fp8 stage of head dim 128 (2 k-steps per score block, 4 dim blocks).
// D = 256 (16-bit pages only): rows of 512 bytes, a stage holds 8 tokens.  They take the first 8 rows of a
// 16-token score block whose other rows repeat them under a mask (the matrix pipe has time to spare: a stage
// is 8 KB of HBM traffic whatever the head dim), with 8 k-steps per score block and 16 dim blocks.
template <typename QT, bool FP8, int NS, bool VL, int D>
__global__ __launch_bounds__(kMfmaThreads) void gqa_mfma_kernel(GqaArgs a) {
  static_assert(NS >= 2 && NS <= 4, "wait_younger_stages covers up to three stages in flight");
  static_assert(D == 128 || D == 64 || D == 256, "head dims of the matrix-core loop");
  using Lay = MfmaLayout<NS, D>;
  constexpr int G = kMfmaHeads;
  constexpr int KS = D / 32;               // k-steps of a score block
  constexpr int MB = D / 16;               // dim blocks of the output
  constexpr int QLPR = D * 2 / 16;         // 16-byte chunks of a Q row
  constexpr int QRPI = kWave / QLPR;       // Q rows per load instruction
  constexpr int RB = FP8 ? D : 2 * D;      // bytes of one token row of one KV head
  constexpr int T = kStageBytes / 2 / RB;  // tokens per stage
  constexpr int LPR = RB / 16;             // lanes (16-byte chunks) per row in a load instruction
  constexpr int RPI = kWave / LPR;         // rows per load instruction

  extern __shared__ __align__(16) char smem[];
  int* tmp = reinterpret_cast<int*>(smem + Lay::kTmpOff);
  int* prefix = reinterpret_cast<int*>(smem + Lay::kPrefixOff);
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15;   // MFMA column (head) / row (token, dim); 16-byte chunk of a row in the loads
  const int g = lane >> 4;     // MFMA k-group; token row of a load instruction
  const int dc = lane % LPR;   // chunk and row of the lane in a load instruction of a K / V tile
  const int dr = lane / LPR;
  // chunk swizzles within a row: K by the row number; V by twice its low two bits (16-bit pages,
  // whose transposing read takes 4 rows x 32 bytes per 16 lanes) or by its low three bits (fp8)
  auto swz_k = [](int row) { return row & (LPR - 1); };
  constexpr int SW8 = LPR < 8 ? LPR - 1 : 7;   // fp8 rows: chunk swizzle by the low bits of the row, as many as the row has chunks
  auto swz_v = [](int row) { return FP8 ? (row & SW8) : ((row & 3) << 1); };
  const int hb_per_kv = VL ? a.chunk_blocks : (a.group + G - 1) / G;
  const int n_hb = a.n_kv_heads * hb_per_kv;
  const int HL = a.head_lock;          // workers that walk the same stages of adjacent head blocks (see GqaArgs)
  const int n_hbl = n_hb / HL;         // groups of head blocks in the flat list
  // packed query chunks: the part of the sequence's chunk that column block cu.hbk holds
  auto chunk_part = [&](CtxCursor& cu) {
    if constexpr (VL) {
      const int per = G / a.group;
      cu.jb = (cu.hbk % hb_per_kv) * per;
      cu.qn = max(0, min(cu.QN - cu.jb, per));
      cu.q0 = cu.Q0 + cu.jb;
    }
  };
  // ... after loading the chunk of sequence cu.b, its size clamped to what the column blocks hold
  auto chunk_of = [&](CtxCursor& cu) {
    if constexpr (VL) {
      cu.Q0 = sload32(a.cu_q + cu.b);
      cu.QF = max(0, sload32(a.cu_q + cu.b + 1) - cu.Q0);
      cu.QN = min(cu.QF, hb_per_kv * (G / a.group));
      chunk_part(cu);
    }
  };
  // byte offset of column c's row in q (VL: token q0 + c / group, clamped into the buffer; head kvh * group + c % group)
  auto q_row_offset = [&](const CtxCursor& cu, int kvh, int c) -> int64_t {
    const int j = c / a.group;
    const int tok = max(0, min(cu.q0 + j, a.n_tokens - 1));
    return tok * a.q_stride_bytes + (static_cast<int64_t>(kvh * a.group + (c - j * a.group)) * D) * 2;
  };

  // progress of pair w: sync[2 w] stages that have landed, sync[2 w + 1] stages whose slots are free again
  lds_vint* sync = (lds_vint*)(smem + Lay::kSyncOff);
  if (tid < 2 * kWaves) sync[tid] = 0;
  // With a plain block table and at most kThreads sequences the context lengths stay in LDS: a worker
  // then finds a sequence without a trip to memory (one of the four in a row before its first row moves).
  int* lens = reinterpret_cast<int*>(smem + Lay::kLensOff);
  const bool lens_in_lds = a.indptr == nullptr && a.table_rows == nullptr && a.batch <= kThreads;
  const bool loader = wave < kWaves;   // wavefronts 0 .. kWaves - 1 load, wavefront kWaves + w computes what w loads
  const int pair = wave & (kWaves - 1);
  const int64_t worker = static_cast<int64_t>(blockIdx.x) * kWaves + pair;   // owns the partial slots 2 worker, 2 worker + 1
  const int64_t n_workers = static_cast<int64_t>(gridDim.x) * kWaves / HL;   // groups of HL workers share a range
  const int64_t team = worker / HL;
  const int member = pair % HL;        // head block member + HL * (group of head blocks)
  const u32 lds_base = static_cast<u32>(reinterpret_cast<uintptr_t>(smem));
  const u32 page_lds = __builtin_amdgcn_readfirstlane(lds_base + Lay::kPageOff + pair * 3 * kWave * 4);
  const bool planned = !VL && a.plan != nullptr;
  if (planned) {
    // one trip to memory: the pages of the first stage straight into the worker's chunk buffer, the plan's prefix
    // and the lengths into LDS (a plan made for another shape says so in its first word: nothing is written then)
    if (loader) dma4(a.plan + kPlanChunksOff + team * kWave + lane, page_lds);
    const int sig = a.plan[0];
    for (int i = tid; i <= a.batch + 1; i += kMfmaThreads) prefix[i] = a.plan[kPlanPrefixOff + i];
    if (lens_in_lds)
      for (int i = tid; i < a.batch; i += kMfmaThreads) lens[i] = a.seq_lens[i];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (sig != a.plan_sig) {
      if (tid == 0) atomicOr(a.ws_status, kStatusPlanMismatch);
      return;
    }
    __syncthreads();
  } else {
    item_prefix<T>(a, prefix, tmp, lens_in_lds ? lens : nullptr);
  }
  const int64_t total = static_cast<int64_t>(prefix[a.batch]) * n_hbl;
  const int64_t cut = a.pool_even == 0 ? 0 : planned ? prefix[a.batch + 1] : pool_cut(a, total);
  if (blockIdx.x == 0 && !planned) {   // (with a plan the merge kernel reads the plan's)
    for (int i = tid; i <= a.batch; i += kMfmaThreads) a.ws_prefix[i] = prefix[i];
    if (tid == 0 && a.pool_even != 0) a.ws_prefix[a.batch + 1] = static_cast<int>(cut);
  }
  auto sequence_at = [&](int b, const int32_t*& pages, int& L) {
    if (lens_in_lds) {
      pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
      L = __builtin_amdgcn_readfirstlane(lens[b]);
    } else {
      sequence_of_scalar(a, b, pages, L);
    }
  };
  if constexpr (!VL) {
    if (a.fold_merge != 0) {  // rows of empty sequences (no item, so no worker ever meets them)
      for (int b = blockIdx.x; b < a.batch; b += gridDim.x)
        if (prefix[b + 1] == prefix[b])
          for (int hbk = 0; hbk < n_hb; ++hbk) merge_context<QT, false>(a, D, hbk, b, tid, kMfmaThreads, 0, 0, 0);
    }
  }
  if (total == 0) return;
  // ---- from here on the pairs are independent: no workgroup barrier below this line
  int64_t cur, end;
  if (!team_range(a, total, cut, team, n_workers, cur, end)) return;
  const int n_stages = static_cast<int>(end - cur);
  lds_vint* landed = sync + 2 * pair;
  lds_vint* freed = landed + 1;

  const u32 ring_lds = __builtin_amdgcn_readfirstlane(lds_base + pair * NS * kStageBytes);
  const char* ring = smem + pair * NS * kStageBytes;
  const char* pagebuf = smem + Lay::kPageOff + pair * 3 * kWave * 4;
  const u32 q_lds = __builtin_amdgcn_readfirstlane(lds_base + Lay::kQOff + pair * G * Lay::kQRow);
  const char* qbuf = smem + Lay::kQOff + pair * G * Lay::kQRow;

  auto locate = [&](int64_t f, CtxCursor& cu) {
    int lo = 0;
    if (a.batch <= 8 * kWave) {
      // the prefix does not decrease, so the sequences that start at or before f are a leading run: count
      // them, one comparison per lane and independent LDS reads, instead of a chain of dependent ones
      int n_le = 0;
      for (int b0 = 0; b0 < a.batch; b0 += kWave) {
        const int b = b0 + lane;
        const bool le = b < a.batch && static_cast<int64_t>(prefix[b]) * n_hbl <= f;
        n_le += __builtin_popcountll(__builtin_amdgcn_ballot_w64(le));
      }
      lo = n_le - 1;
    } else {
      int hi = a.batch;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (static_cast<int64_t>(prefix[mid]) * n_hbl <= f) lo = mid; else hi = mid;
      }
    }
    cu.b = __builtin_amdgcn_readfirstlane(lo);
    cu.n_st = __builtin_amdgcn_readfirstlane(prefix[cu.b + 1] - prefix[cu.b]);
    const int64_t rem = f - static_cast<int64_t>(prefix[cu.b]) * n_hbl;
    const int hbl = __builtin_amdgcn_readfirstlane(static_cast<int>(rem / cu.n_st));
    cu.st = __builtin_amdgcn_readfirstlane(static_cast<int>(rem - static_cast<int64_t>(hbl) * cu.n_st));
    cu.hbk = hbl * HL + member;
    cu.kvh = cu.hbk / hb_per_kv;
    sequence_at(cu.b, cu.pages, cu.L);
    cu.st0 = first_token(a, cu.L) / T;
    chunk_of(cu);
  };
  auto next_context = [&](CtxCursor& cu) {  // the caller never steps past the last context of the batch
    cu.st = 0;
    cu.hbk += HL;
    if (cu.hbk < n_hb) {
      cu.kvh = cu.hbk / hb_per_kv;
      chunk_part(cu);
      return;
    }
    cu.hbk = member;
    cu.kvh = member / hb_per_kv;
    do {
      ++cu.b;
      cu.n_st = __builtin_amdgcn_readfirstlane(prefix[cu.b + 1] - prefix[cu.b]);
    } while (cu.n_st == 0);
    sequence_at(cu.b, cu.pages, cu.L);
    cu.st0 = first_token(a, cu.L) / T;
    chunk_of(cu);
  };
  // 64 entries of the context's page table, from page 64 ck on (the tail repeats the last page),
  // into the chunk buffer at byte offset off
  auto issue_chunk = [&](const CtxCursor& cu, int ck, u32 off) {
    const int n_pages = (cu.L + a.block_size - 1) >> a.bs_shift;
    // (never in front of the table, and never entry 0 of a context that has no pages, which in the CSR form may lie
    // past the end of the index array: with a plan made for other lengths a context may have no pages here; any
    // readable word will do then, page ids are clamped)
    const int32_t* src = cu.pages + max(0, min(ck * kWave + lane, n_pages - 1));
    if (n_pages <= 0 && a.indptr != nullptr) src = a.indptr;
    dma4(src, page_lds + off);
  };

  // byte offset of the lane's 16 bytes from the first row of a stage: row 4i + g, chunk swizzled
  u32 lane_k[4], lane_v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = RPI * i + dr;  // its sub-block of 16 tokens has its own base address
    lane_k[i] = static_cast<u32>((row & 15) * a.row_bytes) + ((dc ^ swz_k(row)) * 16);
    lane_v[i] = static_cast<u32>((row & 15) * a.row_bytes) + ((dc ^ swz_v(row)) * 16);
  }
  // per-lane constants of the operand reads
  const int q_read = c16 * (D * 2);  // Q rows (16-bit): + ((chunk ^ (c16 % QLPR)) * 16)
  // 16-bit pages.  K: row c16, + ((chunk ^ c16) * 16).  V: lane c16 of a 16-lane group addresses 4 dims
  // (8 bytes) of token row 4g + c16/4; + (v_y ^ (mb << 5)) selects dims 16 mb ..
  // (a stage of 8 tokens: rows 8 .. 15 of the score block and of the V^T operand repeat rows 0 .. 7)
  constexpr int TR = T < 16 ? T : 16;      // distinct token rows of a 16-row block
  const int k_row = c16 & (TR - 1);
  const int k_read = k_row * RB;
  const int v_read = T * RB + ((4 * g + (c16 >> 2)) & (TR - 1)) * RB + ((c16 & 3) >> 1) * 16 + (c16 & 1) * 8;
  const int v_y = (c16 >> 2) << 5;
  // fp8 pages.  K: rows c16 and 16 + c16, 8 bytes of chunk kk*2 + g/2.  V: lane c16 of a 16-lane group
  // addresses 8 dims (8 bytes) of the token in k-slot c16/2 of the group: tokens 4g .. 4g+3, then
  // 16 + 4g .. 16 + 4g+3 -- the order in which the two score blocks leave the P^T registers
  // (a 16-token stage, rows of 256 bytes, has one score block: the k-slots of the second repeat the first's tokens
  // and meet zeros in P^T)
  const int v8_row = T >= 32 ? ((c16 >> 1) < 4 ? 0 : 12) + 4 * g + (c16 >> 1) : 4 * g + ((c16 >> 1) & 3);
  const int v8_read = T * RB + v8_row * RB + (c16 & 1) * 8;
  const int v8_y = (v8_row & SW8) << 4;

  if (loader) {
  // ---- the loading wavefront: issues stage p of the worker's range; pc is the context of that stage
  CtxCursor pc;
  locate(cur, pc);
  CtxCursor pn;                              // the context after pc (valid while has_c)
  copy_cursor<VL>(pn, pc);
  int p = 0;
  u32 off_a = 0, off_b = kWave * 4, off_c = 2 * kWave * 4;  // chunk buffers: current, next of pc, first of pn
  int ck_a = 0;
  int t_b = 0, t_c = 0;                      // value of p when the buffer's load was issued
  bool has_b = false, has_c = false;
  int p_ctx_first = 0, p_prev_len = 0;

  // A chunk or Q load issued while p was t has landed once stage t has: this wavefront has waited for
  // that before it issues stage t + NS - 1; otherwise everything in flight is awaited (short contexts
  // only).
  auto ensure_landed = [&](bool issued, int t) {
    if (!(issued && t + NS - 1 <= p)) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  auto begin_context = [&](bool first) {
    if (first) {
      ck_a = (((pc.st0 + pc.st) * T) >> a.bs_shift) >> 6;
      if (!planned) issue_chunk(pc, ck_a, off_a);   // (a plan brought that chunk in with the prefix)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
      const u32 t = off_a;
      off_a = off_c;
      off_c = t;
      ck_a = ((pc.st0 * T) >> a.bs_shift) >> 6;   // the chunk that was fetched ahead: the one of the first stage
      ensure_landed(has_c, t_c);
    }
    has_b = has_c = false;
    p_ctx_first = p;
    if (pc.n_st - pc.st < n_stages - p) {  // the range goes on into another context
      copy_cursor<VL>(pn, pc);
      next_context(pn);
      issue_chunk(pn, ((pn.st0 * T) >> a.bs_shift) >> 6, off_c);
      t_c = p;
      has_c = true;
    }
    const int n_pages = (pc.L + a.block_size - 1) >> a.bs_shift;
    if ((ck_a + 1) * kWave < n_pages) {
      issue_chunk(pc, ck_a + 1, off_b);
      t_b = p;
      has_b = true;
    }
    if (first || p_prev_len >= NS) {
      // Q rows of the context's heads travel ahead of its first stage, swizzled like K rows (rows
      // past the group repeat the last head; the computing wavefront zeroes them).  The single buffer
      // is free: that wavefront copied the previous context's rows to registers when it began that
      // context, at least NS stages ago, and has released the slot of that stage since.  After a shorter
      // context it loads Q itself.
      const int kvh = pc.kvh;
      if constexpr (VL) {
        const int nhp = pc.qn * a.group;
#pragma unroll
        for (int i = 0; i < G / QRPI; ++i) {
          const int row = QRPI * i + lane / QLPR;
          dma16(a.q + q_row_offset(pc, kvh, max(0, min(row, nhp - 1))) + (((lane % QLPR) ^ (row % QLPR)) * 16), q_lds + i * 1024);
        }
      } else {
        const int h0p = kvh * a.group + (pc.hbk % hb_per_kv) * G;
        const int nhp = min(G, (kvh + 1) * a.group - h0p);
        const char* qb = a.q + pc.b * a.q_stride_bytes;
#pragma unroll
        for (int i = 0; i < G / QRPI; ++i) {
          const int row = QRPI * i + lane / QLPR;
          dma16(qb + (static_cast<int64_t>(h0p + min(row, nhp - 1)) * D) * 2 + (((lane % QLPR) ^ (row % QLPR)) * 16), q_lds + i * 1024);
        }
      }
    }
  };
  auto issue_stage = [&]() {
    if (p == 0) {
      begin_context(true);
    } else if (pc.st == pc.n_st) {
      p_prev_len = p - p_ctx_first;
      copy_cursor<VL>(pc, pn);
      begin_context(false);
    }
    const int tok0 = (pc.st0 + pc.st) * T;
    // last valid row of the stage (never negative: under a plan made for longer contexts a stage may lie past the end
    // of its context, and its rows then repeat the stage's first row, which is inside the page)
    const int lim = max(0, pc.L - tok0 - 1);
    // block size >= 16: a sub-block of 16 tokens lies in one page
    constexpr int NSUB = T >= 16 ? T / 16 : 1;
    uint64_t kb[NSUB], vb[NSUB];
#pragma unroll
    for (int sub = 0; sub < NSUB; ++sub) {
      if (sub == 0 || sub * 16 <= lim) {
        const int tok = tok0 + sub * 16;
        const int pi = tok >> a.bs_shift;
        if ((pi >> 6) != ck_a) {
          const u32 t = off_a;
          off_a = off_b;
          off_b = t;
          ck_a = pi >> 6;
          ensure_landed(has_b, t_b);
          has_b = false;
          const int n_pages = (pc.L + a.block_size - 1) >> a.bs_shift;
          if ((ck_a + 1) * kWave < n_pages) {
            issue_chunk(pc, ck_a + 1, off_b);
            t_b = p;
            has_b = true;
          }
        }
        int page = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const int*>(pagebuf + off_a + (pi & 63) * 4));
        page = max(0, min(page, a.num_blocks - 1));  // a corrupt table must not fault the GPU
        const int slot0 = page * a.block_size + (tok & (a.block_size - 1));
        const uint64_t row0 = static_cast<uint64_t>(slot0) * static_cast<uint64_t>(a.row_bytes) +
                              static_cast<uint64_t>(pc.kvh) * RB;
        kb[sub] = reinterpret_cast<uint64_t>(a.k_cache) + row0;
        vb[sub] = reinterpret_cast<uint64_t>(a.v_cache) + row0;
      } else {  // past the end of the context: its rows repeat the last valid one
        kb[sub] = kb[sub - 1];
        vb[sub] = vb[sub - 1];
      }
    }
    const u32 dst = ring_lds + (p % NS) * kStageBytes;
    if (lim >= T - 1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dma16_row(kb[(RPI * i) >> 4], lane_k[i], dst + i * 1024);
        dma16_row(vb[(RPI * i) >> 4], lane_v[i], dst + T * RB + i * 1024);
      }
    } else {  // ragged end of a context: rows past it repeat the last valid row
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = RPI * i + dr;
        const int sub = min(RPI * i, lim) >> 4;  // sub-block of the rows this instruction reads
        const u32 ro = static_cast<u32>((min(row, lim) & 15) * a.row_bytes);
        uint64_t kbs = kb[0], vbs = vb[0];
#pragma unroll
        for (int s2 = 1; s2 < NSUB; ++s2) {
          if (sub >= s2) {
            kbs = kb[s2];
            vbs = vb[s2];
          }
        }
        dma16_row(kbs, ro + ((dc ^ swz_k(row)) * 16), dst + i * 1024);
        dma16_row(vbs, ro + ((dc ^ swz_v(row)) * 16), dst + T * RB + i * 1024);
      }
    }
    ++p;
    ++pc.st;
  };

  // Stage i goes out once stage i - (NS - 1) has landed -- said to the computing wavefront, which cannot
  // wait for loads that another wavefront issued -- and the slot of stage i - NS has been given back.
  // NS - 1 stages are in flight while the other wavefront computes on the oldest one.
  int published = 0, released = 0;
  for (int i = 0; i < n_stages; ++i) {
    while (published < i - (NS - 2)) {
      wait_younger_stages(i - 1 - published);
      ++published;
      *landed = published;
    }
    for (int spin = 0; i - released >= NS; ++spin) {
      released = __builtin_amdgcn_readfirstlane(*freed);
      if (i - released < NS) break;
      if (spin >= a.wait_spins) {  // (never in a correct run: the computing wavefront gives every slot back)
        if (lane == 0) atomicOr(a.ws_status, kStatusWaitGaveUp);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stages in flight land before the LDS is handed back
        return;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    issue_stage();
  }
  while (published < n_stages) {
    wait_younger_stages(n_stages - 1 - published);
    ++published;
    *landed = published;
  }
  return;
  }  // loader

  // ---- the computing wavefront
  CtxCursor cc;
  locate(cur, cc);
  bool run_start = true;
  bool first_run = true;
  bool complete = false;
  int h0 = 0, nh = 0;
  int Lc = 0;                 // tokens the lane's column attends to (the context length unless VL and causal)
  int Lo = 0;                 // first token it attends to (0 without a sliding window)
  int64_t out_off = 0;        // VL: byte offset of the lane's output row
  int c_ctx_first = 0, c_prev_len = 0;
  int n_pend = 0, pend_b0 = 0, pend_h0 = 0, pend_b1 = 0, pend_h1 = 0;  // pieces of contexts this worker left as partials
  u32x4 q[KS];
  f32x4 o[MB];
  float m = kNegBig, l = 0.0f;
  float score_scale = a.scale_log2, out_scale = 1.0f;
  // write-then-attend: the lane's 16 bytes of the new K and V rows as the cache holds them (chunk dc of the row; with
  // fp8 pages the codes of 16 values), fetched when a run begins that reaches its context's end; the slot, or -1
  const bool fused = !VL && a.new_k != nullptr;
  u32x4 new_k = {0u, 0u, 0u, 0u}, new_v = {0u, 0u, 0u, 0u};
  int64_t new_slot = -1;

  int arrived = 0;
  for (int s = 0; s < n_stages; ++s) {
    for (int spin = 0; arrived <= s; ++spin) {
      arrived = __builtin_amdgcn_readfirstlane(*landed);
      if (arrived > s) break;
      if (spin >= a.wait_spins) {  // (never in a correct run: the loading wavefront announces every stage)
        if (lane == 0) atomicOr(a.ws_status, kStatusWaitGaveUp);
        return;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    asm volatile("" ::: "memory");  // no read of the stage moves above the poll

    if (run_start) {  // first stage of a run: the (sequence, head block) changes
      run_start = false;
      const int kvh = cc.kvh;
      if constexpr (VL) {
        nh = cc.qn * a.group;
        const int col = max(0, min(c16, nh - 1));
        const int j = col / a.group;
        Lc = a.causal != 0 ? cc.L - (cc.QF - 1 - (cc.jb + j)) : cc.L;
        const int tok = max(0, min(cc.q0 + j, a.n_tokens - 1));
        out_off = tok * a.out_stride_bytes + (static_cast<int64_t>(kvh * a.group + (col - j * a.group)) * D) * 2;
      } else {
        h0 = kvh * a.group + (cc.hbk % hb_per_kv) * G;
        nh = min(G, (kvh + 1) * a.group - h0);
        Lc = cc.L;
      }
      Lo = first_token(a, cc.L);
      complete = cc.st == 0 && cc.n_st <= n_stages - s;
      if (s == 0 || c_prev_len >= NS) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)  // the rows landed before this stage's tiles did
          q[kk] = *reinterpret_cast<const u32x4*>(qbuf + q_read + (((kk * 4 + g) ^ (c16 % QLPR)) * 16));
      } else {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
          if constexpr (VL)
            q[kk] = ldg16(a.q + q_row_offset(cc, kvh, max(0, min(c16, nh - 1))) + (kk * 32 + g * 8) * 2);
          else
            q[kk] = ldg16(a.q + cc.b * a.q_stride_bytes +
                          (static_cast<int64_t>(h0 + min(c16, nh - 1)) * D + kk * 32 + g * 8) * 2);
        }
        // The wait for these loads (it also drains the stages in flight) must stay on this path:
        // left to the first use after the join it would run on every stage.
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) asm volatile("" : "+v"(q[kk]));
      }
      if (c16 >= nh) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) q[kk] = u32x4{0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) o[mb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      m = kNegBig;
      l = 0.0f;
      c_ctx_first = s;
      float k_scale_h = 1.0f;
      if constexpr (FP8) {  // per-KV-head scales, through the scalar cache like the lengths
        k_scale_h = as_f32(sload32(reinterpret_cast<const int32_t*>(a.k_scale) + kvh));
        score_scale = a.scale_log2 * k_scale_h;
        out_scale = as_f32(sload32(reinterpret_cast<const int32_t*>(a.v_scale) + kvh));
      }
      if constexpr (!VL) {
        new_slot = -1;
        if (fused && cc.n_st - cc.st <= n_stages - s) {   // this run holds the context's last stage: the new token's
          const int64_t slot = sload32(a.new_slots + cc.b);
          if (slot >= 0 && slot < a.n_slots) {
            new_slot = slot;
            const char* kp = a.new_k + cc.b * a.new_k_stride_bytes + static_cast<int64_t>(kvh) * D * 2;
            const char* vp = a.new_v + cc.b * a.new_v_stride_bytes + static_cast<int64_t>(kvh) * D * 2;
            if constexpr (!FP8) {
              new_k = ldg16(kp + dc * 16);
              new_v = ldg16(vp + dc * 16);
            } else {
              // 16 codes from 32 bytes of input, with the arithmetic of reshape_and_cache
              const u32x4 k0 = ldg16(kp + dc * 32), k1 = ldg16(kp + dc * 32 + 16);
              const u32x4 v0 = ldg16(vp + dc * 32), v1 = ldg16(vp + dc * 32 + 16);
              const float ik = 1.0f / k_scale_h, iv = 1.0f / out_scale;
              auto codes = [](u32 w, float inv) {
                return fp8_quantize(QT::lo(w), inv) | (fp8_quantize(QT::hi(w), inv) << 8);
              };
#pragma unroll
              for (int i = 0; i < 2; ++i) {
                new_k[i] = codes(k0[2 * i], ik) | (codes(k0[2 * i + 1], ik) << 16);
                new_k[2 + i] = codes(k1[2 * i], ik) | (codes(k1[2 * i + 1], ik) << 16);
                new_v[i] = codes(v0[2 * i], iv) | (codes(v0[2 * i + 1], iv) << 16);
                new_v[2 + i] = codes(v1[2 * i], iv) | (codes(v1[2 * i + 1], iv) << 16);
              }
            }
          }
        }
      }
    }

    const char* st = ring + (s % NS) * kStageBytes;
    if constexpr (!VL) {
      if (new_slot >= 0 && cc.st == cc.n_st - 1) {
        // The context's last stage: the new token is row r of it, and the rows behind it repeat it (the loader fetched
        // them from the slot, which holds whatever it held before).  Every row from r on gets the new row, chunk by chunk
        // where the operand reads expect it; row r also goes to the cache.
        const int r = cc.L - 1 - (cc.st0 + cc.st) * T;
        char* stw = const_cast<char*>(st);
        for (int row = r + dr; row < T; row += RPI) {
          *(lds_u32x4*)(stw + row * RB + ((dc ^ swz_k(row)) * 16)) = new_k;
          *(lds_u32x4*)(stw + T * RB + row * RB + ((dc ^ swz_v(row)) * 16)) = new_v;
        }
        if (dr == 0) {
          const int64_t off = new_slot * a.row_bytes + static_cast<int64_t>(cc.kvh) * RB + dc * 16;
          stg16(a.k_cache_w + off, new_k);
          stg16(a.v_cache_w + off, new_v);
        }
        new_slot = -1;
      }
    }
    if constexpr (!FP8 && T <= 16) {
      // ---- all operand reads of the stage first: the latency of the V^T reads passes behind the score
      // MFMAs and the softmax (the scheduler would otherwise place them next to their use)
      u32x4 kr[KS];
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) kr[kk] = *reinterpret_cast<const u32x4*>(st + k_read + (((kk * 4 + g) ^ k_row) * 16));
      s16x4 vt[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        vt[mb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + v_read + (v_y ^ (mb << 5))));
      __builtin_amdgcn_sched_barrier(0);
      // ---- scores of the stage's tokens: lane (head c16, tokens 4g .. 4g+3); two chains of KS / 2 MFMAs
      f32x4 sc = Mfma<QT>::k32(kr[0], q[0], f32x4{0.0f, 0.0f, 0.0f, 0.0f});
      f32x4 sc1 = Mfma<QT>::k32(kr[1], q[1], f32x4{0.0f, 0.0f, 0.0f, 0.0f});
#pragma unroll
      for (int kk = 2; kk < KS; kk += 2) {
        sc = Mfma<QT>::k32(kr[kk], q[kk], sc);
        sc1 = Mfma<QT>::k32(kr[kk + 1], q[kk + 1], sc1);
      }
      sc += sc1;
      const int tok0 = (cc.st0 + cc.st) * T + 4 * g;
      float sv[4];
      bool over = false;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool in_stage = T >= 16 || 4 * g + r < T;   // (rows past a short stage repeat its tokens)
        sv[r] = in_stage && tok0 + r < Lc && tok0 + r >= Lo ? sc[r] * score_scale : -INFINITY;
        over |= sv[r] > m + kSlack;
      }
      if (__builtin_amdgcn_ballot_w64(over) != 0) {  // rare once the maxima have settled
        const float mx = quad_rows_max(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
        if (mx > m + kSlack) {
          const float alpha = fast_exp2(m - mx);
          m = mx;
          l *= alpha;
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) o[mb] *= alpha;
        }
      }
      float pr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pr[r] = fast_exp2(sv[r] - m);
        l += pr[r];
      }
      const u32x2 pb = {QT::pack(pr[0], pr[1]), QT::pack(pr[2], pr[3])};
      // ---- O^T += V^T . P^T: lane c16 of a 16-lane group supplies the address of 4 dims of token
      // row 4g + c16/4 and receives the 4 tokens of dim column 16 mb + c16
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) o[mb] = Mfma<QT>::k16(vt[mb], pb, o[mb]);
    } else if constexpr (!FP8) {
      // ---- 16-bit pages with 32 tokens per stage (head dim 64): two score blocks of 16 tokens,
      // lane (head c16, tokens 16 tb + 4g ..), then all 32 tokens in one P.V MFMA per dim block
      u32x4 kr[2][KS];
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) {
        const int tok = tb * 16 + c16;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)
          kr[tb][kk] = *reinterpret_cast<const u32x4*>(st + tok * RB + (((kk * 4 + g) ^ (tok & (LPR - 1))) * 16));
      }
      s16x4 vlo[MB], vhi[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        vlo[mb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + v_read + (v_y ^ (mb << 5))));
        vhi[mb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(st + v_read + 16 * RB + (v_y ^ (mb << 5))));
      }
      __builtin_amdgcn_sched_barrier(0);
      float sv[8];
      bool over = false;
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) {
        f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) sc = Mfma<QT>::k32(kr[tb][kk], q[kk], sc);
        const int tok0 = (cc.st0 + cc.st) * T + tb * 16 + 4 * g;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sv[tb * 4 + r] = tok0 + r < Lc && tok0 + r >= Lo ? sc[r] * score_scale : -INFINITY;
          over |= sv[tb * 4 + r] > m + kSlack;
        }
      }
      if (__builtin_amdgcn_ballot_w64(over) != 0) {  // rare once the maxima have settled
        float mx = sv[0];
#pragma unroll
        for (int r = 1; r < 8; ++r) mx = fmaxf(mx, sv[r]);
        mx = quad_rows_max(mx);
        if (mx > m + kSlack) {
          const float alpha = fast_exp2(m - mx);
          m = mx;
          l *= alpha;
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) o[mb] *= alpha;
        }
      }
      float pr[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        pr[r] = fast_exp2(sv[r] - m);
        l += pr[r];
      }
      // k-slot 8g + j of the P.V MFMA <-> token 4g + j of block 0 (j < 4), of block 1 (j >= 4)
      const u32x4 pb = {QT::pack(pr[0], pr[1]), QT::pack(pr[2], pr[3]), QT::pack(pr[4], pr[5]), QT::pack(pr[6], pr[7])};
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const u32x2 lo = __builtin_bit_cast(u32x2, vlo[mb]), hi = __builtin_bit_cast(u32x2, vhi[mb]);
        o[mb] = Mfma<QT>::k32(u32x4{lo[0], lo[1], hi[0], hi[1]}, pb, o[mb]);
      }
    } else {
      // ---- fp8 pages: the stage's tokens in halves of 32 (one half at head dim 128, two at head dim 64; the 16 tokens
      // of a stage at head dim 256 are the first score block of one half whose second block is masked)
      constexpr int NTB = T >= 32 ? 2 : 1;
#pragma unroll
      for (int hf = 0; hf < (T >= 32 ? T / 32 : 1); ++hf) {
      const char* sth = st + hf * 32 * RB;
      // scores of the half's 32 tokens, two blocks of 16: lane (head c16, tokens 16 tb + 4g ..)
      float sv[8];
      bool over = false;
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) {
        if (tb >= NTB) {
#pragma unroll
          for (int r = 0; r < 4; ++r) sv[tb * 4 + r] = -INFINITY;
          continue;
        }
        f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
        const int tok = tb * 16 + c16;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
          const u32x2 k8 = *reinterpret_cast<const u32x2*>(
              sth + tok * RB + (((kk * 2 + (g >> 1)) ^ (tok & (LPR - 1))) * 16) + (g & 1) * 8);
          const u32x4 kr = {QT::template from_fp8x2<false>(k8[0]), QT::template from_fp8x2<true>(k8[0]),
                            QT::template from_fp8x2<false>(k8[1]), QT::template from_fp8x2<true>(k8[1])};
          sc = Mfma<QT>::k32(kr, q[kk], sc);
        }
        const int tok0 = (cc.st0 + cc.st) * T + hf * 32 + tb * 16 + 4 * g;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sv[tb * 4 + r] = tok0 + r < Lc && tok0 + r >= Lo ? sc[r] * score_scale : -INFINITY;
          over |= sv[tb * 4 + r] > m + kSlack;
        }
      }
      if (__builtin_amdgcn_ballot_w64(over) != 0) {  // rare once the maxima have settled
        float mx = sv[0];
#pragma unroll
        for (int r = 1; r < 8; ++r) mx = fmaxf(mx, sv[r]);
        mx = quad_rows_max(mx);
        if (mx > m + kSlack) {
          const float alpha = fast_exp2(m - mx);
          m = mx;
          l *= alpha;
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) o[mb] *= alpha;
        }
      }
      float pr[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        pr[r] = fast_exp2(sv[r] - m);
        l += pr[r];
      }
      const u32x4 pb = {QT::pack(pr[0], pr[1]), QT::pack(pr[2], pr[3]), QT::pack(pr[4], pr[5]), QT::pack(pr[6], pr[7])};
      // ---- O^T += V^T . P^T over the 32 tokens: the 8-bit transposing read hands lane c16 the
      // eight tokens of its group's k-slots for dim column 16 mb + c16
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const i32x2 v8 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(sth + v8_read + (v8_y ^ (mb << 4))));
        const u32x4 vt = {QT::template from_fp8x2<false>(static_cast<u32>(v8[0])),
                          QT::template from_fp8x2<true>(static_cast<u32>(v8[0])),
                          QT::template from_fp8x2<false>(static_cast<u32>(v8[1])),
                          QT::template from_fp8x2<true>(static_cast<u32>(v8[1]))};
        o[mb] = Mfma<QT>::k32(vt, pb, o[mb]);
      }
      }  // halves
    }

    // ---- end of a run: last stage of the context or of the worker's range
    const bool ctx_end = cc.st == cc.n_st - 1;
    if (ctx_end || s == n_stages - 1) {
      const float lsum = quad_rows_sum(l);
      // (VL: a column that attends to nothing -- a chunk longer than its context -- gives zeros)
      const float inv = VL && !(lsum > 0.0f) ? 0.0f : out_scale / lsum;
      const float lse2 = m + fast_log2(lsum);
      const bool head_on = c16 < nh;
      const int hq = h0 + c16;
      const int64_t pidx = (worker * 2 + (first_run ? 0 : 1)) * G + c16;
      if (head_on && complete) {
        char* op = VL ? a.out + out_off + 4 * g * 2
                      : a.out + cc.b * a.out_stride_bytes + (static_cast<int64_t>(hq) * D + 4 * g) * 2;
        if (a.stream_stores != 0) {
          // (behind an offset the compiler cannot see through, store by store: it otherwise folds the stores of the two
          // branches into one sequence and drops the hint)
          int zero = 0;
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const u32x2 w = {QT::pack(o[mb][0] * inv, o[mb][1] * inv), QT::pack(o[mb][2] * inv, o[mb][3] * inv)};
            asm volatile("" : "+s"(zero));
            __builtin_nontemporal_store(w, reinterpret_cast<u32x2*>(op + zero + mb * 32));
          }
        } else {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const u32x2 w = {QT::pack(o[mb][0] * inv, o[mb][1] * inv), QT::pack(o[mb][2] * inv, o[mb][3] * inv)};
            *reinterpret_cast<u32x2*>(op + mb * 32) = w;
          }
        }
      }
      const bool shared = !VL && a.fold_merge != 0;  // another worker of this launch reads the partial
      if (head_on && !complete && !shared) {
        float* wp = a.ws_out + pidx * D + 4 * g;
        if (a.stream_stores != 0) {
          int zero = 0;
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const f32x4 w = {o[mb][0] * inv, o[mb][1] * inv, o[mb][2] * inv, o[mb][3] * inv};
            asm volatile("" : "+s"(zero));
            __builtin_nontemporal_store(w, reinterpret_cast<f32x4*>(wp + zero + mb * 16));
          }
        } else {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const f32x4 w = {o[mb][0] * inv, o[mb][1] * inv, o[mb][2] * inv, o[mb][3] * inv};
            *reinterpret_cast<f32x4*>(wp + mb * 16) = w;
          }
        }
      }
      if (head_on && !complete && shared) {
        float* wp = a.ws_out + pidx * D + 4 * g;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int r = 0; r < 4; ++r) store_shared(wp + mb * 16 + r, o[mb][r] * inv);
      }
      if (!VL && head_on && g == 0 && complete && a.lse != nullptr) a.lse[cc.b * a.n_q_heads + hq] = lse2 * kLn2;
      if (head_on && g == 0 && !complete && !shared) a.ws_lse[pidx] = lse2;
      if (head_on && g == 0 && !complete && shared) store_shared(a.ws_lse + pidx, lse2);
      if constexpr (!VL) {
        if (!complete) {  // (only the first and the last run of a range can be pieces)
          if (n_pend == 0) {
            pend_b0 = cc.b;
            pend_h0 = cc.hbk;
          } else {
            pend_b1 = cc.b;
            pend_h1 = cc.hbk;
          }
          ++n_pend;
        }
      }
      first_run = false;
    }
    // The operand reads of the stage have returned (the MFMAs that take them have been issued) and LDS
    // serves a wavefront's instructions in order: the slot may be written again.
    asm volatile("" ::: "memory");  // no read of the stage moves below the store
    *freed = s + 1;
    ++cc.st;
    if (ctx_end && s + 1 < n_stages) {
      c_prev_len = s + 1 - c_ctx_first;
      next_context(cc);
      run_start = true;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // ---- the pieces this worker wrote as partials: the worker that brings a context's last piece merges them.
  // One counter per context that spans workers, kept with the worker in whose range it starts (at most one
  // such context per worker); atomicInc wraps it back to zero with the last arrival.  The partials were
  // stored with store_shared and those stores have completed (the wait above), so the worker that sees the
  // last arrival finds all of them with load_shared.
  if constexpr (!VL) {
    if (a.fold_merge != 0 && n_pend > 0) {
      for (int i = 0; i < n_pend; ++i) {
        const int b = i == 0 ? pend_b0 : pend_b1, hbk = i == 0 ? pend_h0 : pend_h1;
        const int p0 = prefix[b], p1 = prefix[b + 1];
        const int n_items = p1 - p0;
        const int64_t first = static_cast<int64_t>(p0) * n_hb + static_cast<int64_t>(hbk) * n_items;
        const int64_t last = first + n_items - 1;
        const int64_t n_use = used_workers(n_workers, total);
        const int w_first = workgroup_of(first, total, n_use), w_last = workgroup_of(last, total, n_use);
        const int pieces = w_last - w_first + 1;  // (no range in between is empty)
        unsigned old = 0;
        if (lane == 0) old = atomicInc(a.ws_arrivals + w_first, static_cast<unsigned>(pieces - 1));
        old = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(old)));
        if (static_cast<int>(old) == pieces - 1)
          merge_context<QT, false, true>(a, D, hbk, b, lane, kWave, p0, p1, prefix[a.batch]);
      }
    }
  }
}

// Merge of the partials of contexts that span several workers (workgroups of the dot-product
// kernel, wavefronts of the matrix-core kernel); also writes the output of empty sequences.
// One workgroup per (head block, sequence); a thread owns four consecutive dims of one head, so
// a partial's rows (contiguous over the heads of the block) are read with 16-byte loads.  The
// kernel is a chain of dependent round trips to memory, so it keeps them to two: the item
// prefix, then the LSEs and accumulators of four consecutive workers at a time, all loads of a
// group issued together.
// VL: the columns of a partial are (query token, head) pairs of the sequence's chunk (see gqa_mfma_kernel).
// The merge of one (head block hbk, sequence b) by `nthreads` threads (this one is `tid`); p0, p1, pt = item
// prefix of the sequence, of the next one, and the batch total; cut = where the second pool's part of the list
// begins (GqaArgs::pool_even).  COHERENT: the partials were written by
// other workers of the same launch (store_shared) and are read the same way.
template <typename QT, bool VL, bool COHERENT>
__device__ __forceinline__ void merge_context(const GqaArgs& a, int dv, int hbk, int b, int tid, int nthreads,
                                              int p0, int p1, int pt, int cut) {
  const int G = a.g_block;
  const int hb_per_kv = VL ? a.chunk_blocks : (a.group + G - 1) / G;
  const int n_hb = a.n_kv_heads * hb_per_kv;
  const int kvh = hbk / hb_per_kv;
  const int h0 = kvh * a.group + (hbk - kvh * hb_per_kv) * G;
  int q0 = 0, qn = 0;
  if constexpr (VL) {  // the part of the chunk in this column block, as in the decode kernel
    const int per = G / a.group;
    const int jb = (hbk - kvh * hb_per_kv) * per;
    const int QN = max(0, min(a.cu_q[b + 1] - a.cu_q[b], hb_per_kv * per));
    q0 = a.cu_q[b] + jb;
    qn = max(0, min(QN - jb, per));
  }
  const int nh = VL ? qn * a.group : min(G, (kvh + 1) * a.group - h0);
  const int dv4 = dv >> 2;         // 16-byte groups per head row
  const int n_vec = nh * dv4;      // per partial
  char* out_row = a.out + b * a.out_stride_bytes;
  const bool wide = ((reinterpret_cast<uintptr_t>(a.out) | static_cast<uintptr_t>(a.out_stride_bytes)) & 7) == 0;
  auto store4 = [&](int h, int d, float x0, float x1, float x2, float x3) {
    uint16_t* o = reinterpret_cast<uint16_t*>(out_row) + static_cast<int64_t>(h0 + h) * dv + d;
    if constexpr (VL) {
      const int j = h / a.group;
      const int tok = max(0, min(q0 + j, a.n_tokens - 1));
      o = reinterpret_cast<uint16_t*>(a.out + tok * a.out_stride_bytes) +
          static_cast<int64_t>(kvh * a.group + (h - j * a.group)) * dv + d;
    }
    if (wide) {
      const u32x2 w = {QT::pack(x0, x1), QT::pack(x2, x3)};
      *reinterpret_cast<u32x2*>(o) = w;
    } else {
      o[0] = QT::from_f32(x0);
      o[1] = QT::from_f32(x1);
      o[2] = QT::from_f32(x2);
      o[3] = QT::from_f32(x3);
    }
  };
  const int n_items = p1 - p0;
  if (n_items <= 0) {  // empty sequence
    for (int v = tid; v < n_vec; v += nthreads) {
      store4(v / dv4, (v % dv4) * 4, 0.0f, 0.0f, 0.0f, 0.0f);
      if (!VL && a.lse != nullptr && v % dv4 == 0) a.lse[b * a.n_q_heads + h0 + v / dv4] = -INFINITY;
    }
    return;
  }
  // (head_lock workers share a range of the list of (sequence, group of head blocks, item); member `hbk % head_lock`
  // of every such group of workers holds this head block's partials)
  const int HL = a.head_lock;
  const int n_hbl = n_hb / HL, member = hbk % HL;
  const int64_t total = static_cast<int64_t>(pt) * n_hbl;
  const int64_t first = static_cast<int64_t>(p0) * n_hbl + static_cast<int64_t>(hbk / HL) * n_items;
  const int64_t last = first + n_items - 1;
  // The pieces of the context lie with consecutive teams of a list: of the whole list, or with the two pools of
  // GqaArgs::pool_even of one or both of its parts (two segments then).  A segment: teams wf .. wl of a list of `tot`
  // items dealt to `n` teams.
  const bool pooled = a.pool_even != 0;
  Pools pools = {};
  if (pooled) pools = make_pools(a, total, cut);
  const bool in0 = !pooled || first < pools.cut;         // pieces in the whole list / in the first pool's part
  const bool in1 = pooled && last >= pools.cut;          // pieces in the second pool's part
  const int64_t tot0 = pooled ? pools.cut : total, n0 = used_workers(pooled ? pools.half : a.n_workgroups / HL, tot0);
  const int64_t tot1 = total - pools.cut, n1 = used_workers(pools.half, tot1);
  const int64_t lo1 = first >= pools.cut ? first : pools.cut, hi0 = in1 ? pools.cut - 1 : last;
  // (one copy of the arithmetic for both segments: two trips through a loop that is not unrolled, the second one
  // for the few contexts that lie across the cut)
  int wf0 = 0, wl0 = -1, sf0 = 0, wf1 = 0, wl1 = -1, sf1 = 0;
#pragma nounroll
  for (int sg = 0; sg < 2; ++sg) {
    if (!(sg ? in1 : in0)) continue;
    const int64_t base = sg ? pools.cut : 0, tot = sg ? tot1 : tot0, n = sg ? n1 : n0;
    const int wf = workgroup_of((sg ? lo1 : first) - base, tot, n);
    const int wl = workgroup_of((sg ? last : hi0) - base, tot, n);
    // the first team of a segment holds this context as its last run (slot 1) unless its range starts inside the
    // context; every later one holds it as its first run (slot 0)
    const int sf = base + range_start(wf, tot, n) < first ? 1 : 0;
    if (sg) {
      wf1 = wf;
      wl1 = wl;
      sf1 = sf;
    } else {
      wf0 = wf;
      wl0 = wl;
      sf0 = sf;
    }
  }
  const int cnt0 = wl0 - wf0 + 1, cnt = cnt0 + (wl1 - wf1 + 1);   // teams of the first segment, of both
  if (cnt == 1) return;  // one team saw the whole context and wrote the output
  for (int v = tid; v < n_vec; v += nthreads) {
    const int h = v / dv4, d = (v - h * dv4) * 4;
    float M = kNegBig, W = 0.0f;
    f32x4 O = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j0 = 0; j0 < cnt; j0 += 4) {
      float lse[4];
      f32x4 x[4];
      bool on[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int j = min(j0 + k, cnt - 1);
        const bool second = j >= cnt0;
        const int w = second ? wf1 + (j - cnt0) : wf0 + j;
        on[k] = j0 + k < cnt;
        const int team = pooled ? pools.of_pool(second ? 1 : 0, w) : w;
        const int slot = j == 0 ? (in0 ? sf0 : sf1) : (j == cnt0 ? sf1 : 0);
        const int64_t ps = ((static_cast<int64_t>(team) * HL + member) * 2 + slot) * G + h;
        if constexpr (COHERENT) {
          const float* xp = a.ws_out + ps * dv + d;
          lse[k] = on[k] ? load_shared(a.ws_lse + ps) : kNegBig;
          x[k] = on[k] ? f32x4{load_shared(xp), load_shared(xp + 1), load_shared(xp + 2), load_shared(xp + 3)}
                       : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        } else {
          lse[k] = on[k] ? a.ws_lse[ps] : kNegBig;
          x[k] = on[k] ? *reinterpret_cast<const f32x4*>(a.ws_out + ps * dv + d) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
      }
      const float m_new = fmaxf(fmaxf(M, fmaxf(lse[0], lse[1])), fmaxf(lse[2], lse[3]));
      const float keep = fast_exp2(M - m_new);
      W *= keep;
      O *= keep;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float e = on[k] ? fast_exp2(lse[k] - m_new) : 0.0f;
        W += e;
        O += e * x[k];
      }
      M = m_new;
    }
    const float inv = VL && !(W > 0.0f) ? 0.0f : 1.0f / W;
    store4(h, d, O[0] * inv, O[1] * inv, O[2] * inv, O[3] * inv);
    if (!VL && a.lse != nullptr && d == 0) a.lse[b * a.n_q_heads + h0 + h] = (M + fast_log2(W)) * kLn2;
  }
}

// The plan of a step for gqa_mfma_kernel (GqaArgs::plan): one wavefront per group of workers finds the start of the
// group's range as the decode kernel would and copies the 64 page-table entries around the first stage's page.
// T: tokens per stage of the decode kernel the plan is for.
template <int T>
__global__ __launch_bounds__(kThreads) void gqa_plan_kernel(GqaArgs a, int* plan, int n_teams) {
  extern __shared__ __align__(16) char smem[];
  int* tmp = reinterpret_cast<int*>(smem);
  int* prefix = tmp + kThreads;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  item_prefix<T>(a, prefix, tmp);
  const int hb_per_kv = (a.group + kMfmaHeads - 1) / kMfmaHeads;
  const int n_hbl = a.n_kv_heads * hb_per_kv / a.head_lock;
  const int64_t total = static_cast<int64_t>(prefix[a.batch]) * n_hbl;
  const int64_t cut = a.pool_even == 0 ? 0 : pool_cut(a, total);
  if (blockIdx.x == 0) {
    for (int i = tid; i <= a.batch; i += kThreads) plan[kPlanPrefixOff + i] = prefix[i];
    for (int i = tid; i < a.batch; i += kThreads) {
      const int32_t* pages;
      int L;
      sequence_of(a, i, pages, L);
      plan[kPlanLensOff + i] = L;
    }
    if (tid == 0) plan[kPlanPrefixOff + a.batch + 1] = static_cast<int>(cut);
    if (tid == 0) plan[0] = a.plan_sig;
  }
  const int team = blockIdx.x * kWaves + wave;
  int64_t cur, end;
  if (team >= n_teams || !team_range(a, total, cut, team, n_teams, cur, end)) return;
  int lo = 0, hi = a.batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(prefix[mid]) * n_hbl <= cur) lo = mid; else hi = mid;
  }
  const int n_st = prefix[lo + 1] - prefix[lo];
  const int st = static_cast<int>((cur - static_cast<int64_t>(prefix[lo]) * n_hbl) % n_st);
  const int32_t* pages;
  int L;
  sequence_of(a, lo, pages, L);
  const int st0 = first_token(a, L) / T;
  const int ck = (((st0 + st) * T) >> a.bs_shift) >> 6;
  const int n_pages = (L + a.block_size - 1) >> a.bs_shift;
  plan[kPlanChunksOff + team * kWave + lane] = pages[max(0, min(ck * kWave + lane, n_pages - 1))];
}

template <typename QT, bool VL>
__global__ __launch_bounds__(kThreads) void merge_partials_kernel(GqaArgs a, int dv) {
  const int b = blockIdx.y;
  if (a.plan != nullptr && a.plan[0] != a.plan_sig) return;   // the decode kernel wrote nothing and raised the flag
  if (!VL && a.plan != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
    // a plan made with other lengths (the step before, say): the decode kernel followed its ranges, the output is
    // invalid, and the caller hears of it through the status word
    const int32_t* pages;
    int L;
    sequence_of(a, b, pages, L);
    if (L != a.plan[kPlanLensOff + b]) atomicOr(a.ws_status, kStatusPlanMismatch);
  }
  merge_context<QT, VL>(a, dv, blockIdx.x, b, threadIdx.x, kThreads, a.ws_prefix[b], a.ws_prefix[b + 1],
                        a.ws_prefix[a.batch], a.pool_even != 0 ? a.ws_prefix[a.batch + 1] : 0);
}

template <typename QT, bool FP8, int D, int LPT, int G, int U>
int launch_gqa(GqaArgs& a, size_t workspace_bytes, hipStream_t stream, bool plan_only, size_t* need) {
  constexpr int NP = kWaves * (kWave / LPT);
  auto kern = gqa_decode_kernel<QT, FP8, D, LPT, G, U>;
  const size_t smem = kSub * 4 + static_cast<size_t>(NP) * (D + 2) * 4 + kThreads * 4 +
                      (static_cast<size_t>(a.batch) + 1) * 4;
  // workgroups of this kernel that a CU of the current device holds, asked once per device
  static std::atomic<int> per_cu_of[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) dev = 0;
  int per_cu = per_cu_of[dev].load(std::memory_order_relaxed);
  if (per_cu <= 0) {
    const char* e = getenv("XLLM_MI355_GQA_WGS_PER_CU");  // tuning knob
    if (e != nullptr && atoi(e) > 0) {
      per_cu = atoi(e);
    } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), kThreads,
                                                            kSub * 4 + NP * (D + 2) * 4 + kThreads * 4 + 1028) != hipSuccess ||
               per_cu < 1) {
      per_cu = 2;
    }
    per_cu_of[dev].store(per_cu, std::memory_order_relaxed);
  }
  a.n_workgroups = device_cu_count() * per_cu;
  a.plan = nullptr;   // (plans are for the matrix-core kernel)
  const size_t part_floats = static_cast<size_t>(a.n_workgroups) * 2 * G * (D + 1);
  *need = kWsPartialsOff + part_floats * 4;
  if (plan_only) return XLLM_MI355_OK;
  if (*need > workspace_bytes) return XLLM_MI355_EWORKSPACE;
  a.ws_out = reinterpret_cast<float*>(reinterpret_cast<char*>(a.ws_status) + kWsPartialsOff);
  a.ws_lse = a.ws_out + static_cast<size_t>(a.n_workgroups) * 2 * G * D;
  launch_timed(kern, dim3(static_cast<unsigned>(a.n_workgroups)), dim3(kThreads), smem, stream, a);
  return static_cast<int>(hipGetLastError());
}

constexpr int kMfmaStages = 4;

// Tuning knob XLLM_MI355_GQA_XCD_POOLS: the share of the teams on even XCDs in eighths of the share of those on odd
// XCDs (default 9, see GqaArgs::pool_even; 0 = one list for all teams).
int xcd_pools_knob() {
  static const int v = [] {
    const char* e = getenv("XLLM_MI355_GQA_XCD_POOLS");
    const int x = e ? atoi(e) : -1;
    return x >= 0 && x <= 16 ? x : 9;
  }();
  return v;
}

// Tuning knob XLLM_MI355_GQA_HEAD_LOCK (1, 2 or 4; default 4): see GqaArgs::head_lock.
int head_lock_knob() {
  static const int v = [] {
    const char* e = getenv("XLLM_MI355_GQA_HEAD_LOCK");
    const int x = e ? atoi(e) : 0;
    return x == 1 || x == 2 || x == 4 ? x : 4;
  }();
  return v;
}

// Tuning knob XLLM_MI355_GQA_STREAM_STORES, read once per process: 0 / 1 force GqaArgs::stream_stores off / on;
// anything else leaves the choice to the number of output rows of the launch.  set_stream_stores (test hook)
// overrides it: 0, 1, or negative for the choice per launch.
std::atomic<int> g_stream_stores{-2};
int stream_stores_knob() {
  int v = g_stream_stores.load(std::memory_order_relaxed);
  if (v == -2) {
    const char* e = getenv("XLLM_MI355_GQA_STREAM_STORES");
    v = e != nullptr && (e[0] == '0' || e[0] == '1') ? e[0] - '0' : -1;
    g_stream_stores.store(v, std::memory_order_relaxed);
  }
  return v;
}

// Whether the matrix-core kernel merges the partials itself: the worker that brings a context's last piece
// reads the others' partials and writes the output, and no merge kernel is launched.  Off by default: the
// exchange inside one launch has to go through the memory level that all XCDs share (store_shared /
// load_shared), and its chain of three round trips at the tail of the launch costs more (about 12 us on the
// 64-sequence configuration) than the separate merge launch it saves (4.5 us).  "1" in XLLM_MI355_GQA_FOLD, read
// once per process, or set_fold_merge (test hook) turn it on.
std::atomic<int> g_fold_merge{-1};
bool fold_merge_enabled() {
  int v = g_fold_merge.load(std::memory_order_relaxed);
  if (v < 0) {
    const char* e = getenv("XLLM_MI355_GQA_FOLD");  // tuning knob
    v = e != nullptr && e[0] == '1' ? 1 : 0;
    g_fold_merge.store(v, std::memory_order_relaxed);
  }
  return v != 0;
}

// What a plan is made for: everything that the list and its ranges depend on besides the lengths themselves.
int plan_signature(const GqaArgs& a, int stage_tokens) {
  uint32_t h = 2166136261u;
  const int v[] = {a.batch, a.n_kv_heads, a.group, stage_tokens, a.head_lock, a.pool_even, a.pool_odd, a.n_workgroups,
                   a.window_left, a.bs_shift, a.indptr != nullptr ? 1 : 0};
  for (int x : v) h = (h ^ static_cast<uint32_t>(x)) * 16777619u;
  return static_cast<int>(h | 1u);
}

// The shape of the matrix-core kernel's launch: workers, workers side by side, pools.
void configure_mfma(GqaArgs& a, bool fp8, int head_dim, bool varlen) {
  a.g_block = kMfmaHeads;
  const int n_wg = device_cu_count();  // the ring fills a CU's LDS: one workgroup each
  a.n_workgroups = n_wg * kWaves;      // independent workers = wavefronts
  a.fold_merge = !varlen && a.n_workgroups <= kWsMaxWorkers && fold_merge_enabled() ? 1 : 0;
  // Adjacent head blocks side by side: adjacent KV heads when a KV head has one head block; with several (more than
  // 16 query heads per KV head, or packed query chunks of more than 16 / group tokens) the blocks of one KV head, which
  // read the same rows, so that all but the first find them in L2.  (The in-kernel merge keeps its own bookkeeping
  // per worker.)
  a.head_lock = 1;
  if (a.fold_merge == 0) {
    const int hb_per_kv = varlen ? a.chunk_blocks : (a.group + kMfmaHeads - 1) / kMfmaHeads;
    const int n_hb = a.n_kv_heads * hb_per_kv;
    const int want = head_lock_knob();
    for (int hl = kWaves; hl > 1; hl >>= 1)
      if (hl <= want && n_hb % hl == 0 && kWaves % hl == 0) {
        a.head_lock = hl;
        break;
      }
  }
  // (the pools need whole groups of eight workgroups, one per XCD; the in-kernel merge walks one list; fp8 rows of
  // 64 bytes keep the computing wavefronts busy enough that the XCDs end together with equal ranges: 134 us against
  // 139 us with the cut)
  const int64_t out_rows = static_cast<int64_t>(varlen ? a.n_tokens : a.batch) * a.n_q_heads;
  a.stream_stores = stream_stores_knob() >= 0 ? stream_stores_knob() : (out_rows >= 8192 ? 1 : 0);
  a.pool_even = a.pool_odd = 0;
  // The cut is a tuned default for the full MI355X (256 CUs in 8 XCDs, workgroups dealt to the XCDs round robin), not
  // a property of the algorithm: any other CU count (a partitioned or CU-masked device) gets one list.
  if (a.fold_merge == 0 && n_wg == 256 && xcd_pools_knob() != 0 && !(fp8 && head_dim == 64)) {
    a.pool_even = xcd_pools_knob();
    a.pool_odd = 8;
  }
}
constexpr int stage_tokens(bool fp8, int head_dim) { return kStageBytes / 2 / (fp8 ? head_dim : 2 * head_dim); }

template <typename QT, bool FP8, bool VL = false, int D = 128>
int launch_gqa_mfma(GqaArgs& a, size_t workspace_bytes, hipStream_t stream, bool plan_only, size_t* need) {
  // (head dim 256: the Q rows of the four pairs take 32 KB of the LDS, which leaves room for three stages each)
  constexpr int NS = D == 256 ? kMfmaStages - 1 : kMfmaStages;
  using Lay = MfmaLayout<NS, D>;
  static_assert(Lay::kPrefixOff + (kMaxBatch + 2) * 4 <= 160 * 1024, "LDS of a CU");
  auto kern = gqa_mfma_kernel<QT, FP8, NS, VL, D>;
  static std::atomic<uint64_t> configured{0};
  if (first_use_on_current_device(configured)) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize,
                                             Lay::kPrefixOff + (kMaxBatch + 2) * 4);
    if (e != hipSuccess) return static_cast<int>(e);
  }
  configure_mfma(a, FP8, D, VL);
  const int n_wg = a.n_workgroups / kWaves;
  const size_t part_floats = static_cast<size_t>(a.n_workgroups) * 2 * kMfmaHeads * (D + 1);
  *need = kWsPartialsOff + part_floats * 4;
  if (plan_only) return XLLM_MI355_OK;
  if (*need > workspace_bytes) return XLLM_MI355_EWORKSPACE;
  a.ws_out = reinterpret_cast<float*>(reinterpret_cast<char*>(a.ws_status) + kWsPartialsOff);
  a.ws_lse = a.ws_out + static_cast<size_t>(a.n_workgroups) * 2 * kMfmaHeads * D;
  a.ws_arrivals = reinterpret_cast<unsigned*>(reinterpret_cast<char*>(a.ws_status) + kWsCountersOff);
  if (VL || a.fold_merge != 0 || a.n_workgroups / a.head_lock > kPlanMaxTeams) a.plan = nullptr;
  if (a.plan != nullptr) {   // the merge kernel reads the plan's prefix and cut
    a.plan_sig = plan_signature(a, stage_tokens(FP8, D));
    a.ws_prefix = const_cast<int*>(a.plan) + kPlanPrefixOff;
  }
  const size_t smem = Lay::kPrefixOff + (static_cast<size_t>(a.batch) + 2) * 4;
  launch_timed(kern, dim3(static_cast<unsigned>(n_wg)), dim3(kMfmaThreads), smem, stream, a);
  return static_cast<int>(hipGetLastError());
}

// Which kernel serves head_dim 128 (or 64 with 16-bit pages) and a power-of-two block size: the
// matrix-core one ("mfma", default) or the dot-product one ("rows").
bool use_mfma_kernel() {
  static const bool v = [] {
    const char* e = getenv("XLLM_MI355_GQA_KERNEL");  // tuning knob
    return !(e != nullptr && e[0] == 'r');
  }();
  return v;
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

// Whether the matrix-core kernel serves a one-query-token call (its epilogue stores 8 output bytes at a time; its
// stages are whole parts of a page of a power-of-two size from 16 tokens on).
bool mfma_serves(const GqaArgs& a, bool fp8, int head_dim) {
  (void)fp8;
  const bool out_aligned = (reinterpret_cast<uintptr_t>(a.out) & 7) == 0 && (a.out_stride_bytes & 7) == 0;
  const bool dim_ok = head_dim == 64 || head_dim == 128 || head_dim == 256;
  return dim_ok && a.bs_shift >= 4 && out_aligned && use_mfma_kernel();
}

template <typename QT, bool FP8>
int dispatch_dim(GqaArgs& a, int head_dim, size_t wsb, hipStream_t s, bool plan_only, size_t* need) {
  // lanes per token row: one 16-byte load per lane and row
  const bool mfma = mfma_serves(a, FP8, head_dim);
  if constexpr (FP8) {
    if (head_dim == 128 && mfma) return launch_gqa_mfma<QT, true>(a, wsb, s, plan_only, need);
    if (head_dim == 64 && mfma) return launch_gqa_mfma<QT, true, false, 64>(a, wsb, s, plan_only, need);
    if (head_dim == 256 && mfma) return launch_gqa_mfma<QT, true, false, 256>(a, wsb, s, plan_only, need);
    switch (head_dim) {
      case 64: return dispatch_group<QT, true, 64, 4, 2>(a, wsb, s, plan_only, need);
      case 128: return dispatch_group<QT, true, 128, 8, 2>(a, wsb, s, plan_only, need);
      case 256: return dispatch_group<QT, true, 256, 16, 4>(a, wsb, s, plan_only, need);
      default: return XLLM_MI355_ESHAPE;
    }
  } else {
    if (head_dim == 128 && mfma) return launch_gqa_mfma<QT, false>(a, wsb, s, plan_only, need);
    if (head_dim == 64 && mfma) return launch_gqa_mfma<QT, false, false, 64>(a, wsb, s, plan_only, need);
    if (head_dim == 256 && mfma) return launch_gqa_mfma<QT, false, false, 256>(a, wsb, s, plan_only, need);
    switch (head_dim) {
      case 64: return dispatch_group<QT, false, 64, 8, 2>(a, wsb, s, plan_only, need);
      case 128: return dispatch_group<QT, false, 128, 16, 4>(a, wsb, s, plan_only, need);
      case 256: return dispatch_group<QT, false, 256, 32, 4>(a, wsb, s, plan_only, need);
      default: return XLLM_MI355_ESHAPE;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// fp32 query, fp32 pages, fp32 output: the caches that reshape_and_cache stores for fp32 models (the reference's
// own cases {4,1,16,1,64,f32} and {1,4,16,4,128,f32}, tests/core/kernels/dcu/reshape_paged_cache_test.cpp:135-158)
// can be attended too, as the reference's libtorch decode attends any dtype (kernels/npu/attention.cpp:26-78).  A
// compatibility path, not a tuned one: one workgroup per (query head, sequence), no split over workgroups, no
// workspace; a wavefront takes every fourth token, a lane D / 64 dims of it; a score is a sum over the wavefront's
// lanes; the four wavefronts' states meet in LDS at the end.
template <int D>
__global__ __launch_bounds__(256) void gqa_decode_f32_kernel(GqaArgs a) {
  constexpr int E = D / 64;   // dims per lane
  __shared__ float part[4][D + 2];
  const int h = blockIdx.x, b = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kvh = h / a.group;
  const int32_t* pages;
  int L;
  sequence_of(a, b, pages, L);
  float* out = reinterpret_cast<float*>(a.out + b * a.out_stride_bytes) + static_cast<int64_t>(h) * D;
  if (L <= 0) {
    for (int d = threadIdx.x; d < D; d += 256) out[d] = 0.0f;
    if (a.lse != nullptr && threadIdx.x == 0) a.lse[b * a.n_q_heads + h] = -INFINITY;
    return;
  }
  const float* q = reinterpret_cast<const float*>(a.q + b * a.q_stride_bytes) + static_cast<int64_t>(h) * D + lane * E;
  float qv[E], o[E];
#pragma unroll
  for (int i = 0; i < E; ++i) {
    qv[i] = q[i] * a.scale_log2;
    o[i] = 0.0f;
  }
  float m = kNegBig, l = 0.0f;
  const int64_t head_off = static_cast<int64_t>(kvh) * D + lane * E;
  for (int t = first_token(a, L) + wave; t < L; t += 4) {
    int page = pages[t / a.block_size];
    page = max(0, min(page, a.num_blocks - 1));   // a corrupt table must not fault the GPU
    const int64_t row = (static_cast<int64_t>(page) * a.block_size + t % a.block_size) * (a.row_bytes / 4) + head_off;
    const float* k = reinterpret_cast<const float*>(a.k_cache) + row;
    const float* v = reinterpret_cast<const float*>(a.v_cache) + row;
    float kv[E], vv[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
      kv[i] = k[i];
      vv[i] = v[i];
    }
    float sc = 0.0f;
#pragma unroll
    for (int i = 0; i < E; ++i) sc += qv[i] * kv[i];
    sc = group_sum<32>(sc);
    sc += __shfl_xor(sc, 32, kWave);
    const float m_new = fmaxf(m, sc);
    const float keep = fast_exp2(m - m_new), p = fast_exp2(sc - m_new);
    l = l * keep + p;
#pragma unroll
    for (int i = 0; i < E; ++i) o[i] = o[i] * keep + p * vv[i];
    m = m_new;
  }
#pragma unroll
  for (int i = 0; i < E; ++i) part[wave][lane * E + i] = o[i];
  if (lane == 0) {
    part[wave][D] = m;
    part[wave][D + 1] = l;
  }
  __syncthreads();
  float M = kNegBig;
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, part[w][D]);
  float W = 0.0f;
#pragma unroll
  for (int w = 0; w < 4; ++w) W += part[w][D + 1] * fast_exp2(part[w][D] - M);   // (a wavefront without tokens: 0 * 1)
  for (int d = threadIdx.x; d < D; d += 256) {
    float x = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) x += part[w][d] * fast_exp2(part[w][D] - M);
    out[d] = x / W;
  }
  if (a.lse != nullptr && threadIdx.x == 0) a.lse[b * a.n_q_heads + h] = (M + fast_log2(W)) * kLn2;
}

int group_block(int group) {
  if (group <= 1) return 1;
  if (group <= 2) return 2;
  if (group <= 4) return 4;
  return 8;
}

}  // namespace

void set_fold_merge(int on) { g_fold_merge.store(on != 0 ? 1 : 0, std::memory_order_relaxed); }
void set_stream_stores(int v) { g_stream_stores.store(v < 0 ? -1 : (v != 0 ? 1 : 0), std::memory_order_relaxed); }

size_t gqa_plan_bytes() { return kPlanBytes; }

int paged_decode_gqa_plan(void* plan, size_t plan_bytes, const PageAddressing& addr, int64_t batch, int64_t n_q_heads,
                          int64_t n_kv_heads, int64_t head_dim, int64_t block_size, int cache_dtype,
                          hipStream_t stream) {
  if (batch == 0) return XLLM_MI355_OK;
  if (plan == nullptr || (reinterpret_cast<uintptr_t>(plan) & 255) != 0 || plan_bytes < kPlanBytes)
    return XLLM_MI355_EWORKSPACE;
  const bool csr = addr.indptr != nullptr;
  if (csr ? (addr.indices == nullptr || addr.last_page_len == nullptr)
          : (addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0))
    return XLLM_MI355_EINVAL;
  if (batch < 0 || n_q_heads <= 0 || n_kv_heads <= 0 || block_size <= 0 || n_q_heads % n_kv_heads != 0 ||
      n_q_heads > 65535)
    return XLLM_MI355_EINVAL;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return XLLM_MI355_ESHAPE;
  const bool fp8 = cache_dtype == XLLM_MI355_FP8_E4M3;
  GqaArgs a = {};
  a.block_table = csr ? nullptr : addr.block_table;
  a.seq_lens = csr ? nullptr : addr.seq_lens;
  a.indptr = csr ? addr.indptr : nullptr;
  a.indices = addr.indices;
  a.last_page_len = csr ? addr.last_page_len : nullptr;
  a.table_stride = addr.table_stride;
  a.window_left = addr.window_left < 0 ? -1 : static_cast<int>(addr.window_left < 0x7fffffffLL ? addr.window_left : 0x7fffffffLL);
  a.batch = static_cast<int>(batch);
  a.n_q_heads = static_cast<int>(n_q_heads);
  a.n_kv_heads = static_cast<int>(n_kv_heads);
  a.group = static_cast<int>(n_q_heads / n_kv_heads);
  a.block_size = static_cast<int>(block_size);
  a.bs_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1LL << s) == block_size) a.bs_shift = s;
  // Shapes that the matrix-core kernel does not serve, and batches decoded in slices, take no plan: the planned
  // entry point decodes them like the plain one.
  if (batch > kMaxBatch || a.bs_shift < 4 || !use_mfma_kernel()) return XLLM_MI355_OK;
  configure_mfma(a, fp8, static_cast<int>(head_dim), false);
  const int n_teams = a.n_workgroups / a.head_lock;
  if (a.fold_merge != 0 || n_teams > kPlanMaxTeams) return XLLM_MI355_OK;
  const int T = stage_tokens(fp8, static_cast<int>(head_dim));
  a.plan_sig = plan_signature(a, T);
  const dim3 grid(static_cast<unsigned>((n_teams + kWaves - 1) / kWaves));
  const size_t smem = (static_cast<size_t>(kThreads) + a.batch + 1) * 4;
  int* words = static_cast<int*>(plan);
  switch (T) {
    case 8: launch_timed(gqa_plan_kernel<8>, grid, dim3(kThreads), smem, stream, a, words, n_teams); break;
    case 16: launch_timed(gqa_plan_kernel<16>, grid, dim3(kThreads), smem, stream, a, words, n_teams); break;
    case 32: launch_timed(gqa_plan_kernel<32>, grid, dim3(kThreads), smem, stream, a, words, n_teams); break;
    case 64: launch_timed(gqa_plan_kernel<64>, grid, dim3(kThreads), smem, stream, a, words, n_teams); break;
    default: return XLLM_MI355_ESHAPE;
  }
  return static_cast<int>(hipGetLastError());
}

size_t gqa_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t head_dim) {
  // Upper bound over every kernel variant, independent of the batch: at most 8 workgroups per CU, 8 heads
  // per block (the matrix-core kernel: 4 workers per CU, 16 heads).
  (void)batch;
  (void)n_q_heads;
  return kWsPartialsOff + static_cast<size_t>(device_cu_count()) * 8 * 2 * 8 * (head_dim + 1) * 4;
}

int paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache, void* out, float* lse,
                     const PageAddressing& addr, const float* k_scale, const float* v_scale,
                     int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                     int64_t block_size, int64_t num_blocks, int64_t q_token_stride,
                     int64_t out_token_stride, int64_t max_seq_len, float sm_scale, void* workspace,
                     size_t workspace_bytes, int q_dtype, int cache_dtype, hipStream_t stream, const NewKvRows* fresh) {
  (void)max_seq_len;  // the schedule is computed on the device from the actual lengths
  if (batch == 0) return XLLM_MI355_OK;
  if (q == nullptr || k_cache == nullptr || v_cache == nullptr || out == nullptr) return XLLM_MI355_EINVAL;
  if (fresh != nullptr && (fresh->key == nullptr || fresh->value == nullptr || fresh->slots == nullptr ||
                           addr.cu_q != nullptr))
    return XLLM_MI355_EINVAL;
  const bool csr = addr.indptr != nullptr;
  if (csr ? (addr.indices == nullptr || addr.last_page_len == nullptr)
          : (addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0))
    return XLLM_MI355_EINVAL;
  if (batch < 0 || n_q_heads <= 0 || n_kv_heads <= 0 || block_size <= 0 || num_blocks <= 0 ||
      n_q_heads % n_kv_heads != 0 || n_q_heads > 65535 || !(sm_scale > 0.0f))
    return XLLM_MI355_EINVAL;
  if (num_blocks * block_size > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  if (q_dtype != XLLM_MI355_BF16 && q_dtype != XLLM_MI355_FP16 && q_dtype != XLLM_MI355_FP32) return XLLM_MI355_EDTYPE;
  const bool fp8 = cache_dtype == XLLM_MI355_FP8_E4M3;
  if (!fp8 && cache_dtype != q_dtype) return XLLM_MI355_EDTYPE;
  if (fp8 && q_dtype == XLLM_MI355_FP32) return XLLM_MI355_EDTYPE;
  if (fp8 && (k_scale == nullptr || v_scale == nullptr)) return XLLM_MI355_EINVAL;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return XLLM_MI355_ESHAPE;
  if (q_token_stride < n_q_heads * head_dim || out_token_stride < n_q_heads * head_dim)
    return XLLM_MI355_EINVAL;
  if (q_dtype == XLLM_MI355_FP32) {   // fp32 query over fp32 pages: the compatibility kernel, no workspace
    if (addr.cu_q != nullptr || addr.table_rows != nullptr) return XLLM_MI355_EDTYPE;
    if (((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(k_cache) |
          reinterpret_cast<uintptr_t>(v_cache)) & 15) != 0 || (q_token_stride * 4) % 16 != 0 || (out_token_stride * 4) % 16 != 0)
      return XLLM_MI355_EALIGN;
    if (batch > 65535) return XLLM_MI355_ESHAPE;
    if (fresh != nullptr) {
      const int rc = reshape_and_cache(fresh->key, fresh->value, const_cast<void*>(k_cache), const_cast<void*>(v_cache),
                                       fresh->slots, k_scale, v_scale, batch, n_kv_heads, head_dim, block_size, num_blocks,
                                       fresh->k_token_stride, fresh->v_token_stride, q_dtype, cache_dtype, stream);
      if (rc != 0) return rc;
    }
    GqaArgs a = {};
    a.q = static_cast<const char*>(q);
    a.k_cache = static_cast<const char*>(k_cache);
    a.v_cache = static_cast<const char*>(v_cache);
    a.out = static_cast<char*>(out);
    a.lse = lse;
    a.block_table = csr ? nullptr : addr.block_table;
    a.seq_lens = csr ? nullptr : addr.seq_lens;
    a.indptr = csr ? addr.indptr : nullptr;
    a.indices = addr.indices;
    a.last_page_len = csr ? addr.last_page_len : nullptr;
    a.table_stride = addr.table_stride;
    a.window_left = addr.window_left < 0 ? -1 : static_cast<int>(addr.window_left < 0x7fffffffLL ? addr.window_left : 0x7fffffffLL);
    a.q_stride_bytes = q_token_stride * 4;
    a.out_stride_bytes = out_token_stride * 4;
    a.row_bytes = n_kv_heads * head_dim * 4;
    a.batch = static_cast<int>(batch);
    a.n_q_heads = static_cast<int>(n_q_heads);
    a.n_kv_heads = static_cast<int>(n_kv_heads);
    a.group = static_cast<int>(n_q_heads / n_kv_heads);
    a.block_size = static_cast<int>(block_size);
    a.num_blocks = static_cast<int>(num_blocks);
    a.scale_log2 = sm_scale * kLog2e;
    const dim3 grid(static_cast<unsigned>(n_q_heads), static_cast<unsigned>(batch));
    switch (head_dim) {
      case 64: launch_timed(gqa_decode_f32_kernel<64>, grid, dim3(256), 0, stream, a); break;
      case 128: launch_timed(gqa_decode_f32_kernel<128>, grid, dim3(256), 0, stream, a); break;
      default: launch_timed(gqa_decode_f32_kernel<256>, grid, dim3(256), 0, stream, a); break;
    }
    profile_skip();   // (no merge launch)
    return static_cast<int>(hipGetLastError());
  }
  auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || (q_token_stride * 2) % 16 != 0)
    return XLLM_MI355_EALIGN;
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return XLLM_MI355_EWORKSPACE;
  if (addr.plan != nullptr && (reinterpret_cast<uintptr_t>(addr.plan) & 255) != 0) return XLLM_MI355_EWORKSPACE;

  const int group = static_cast<int>(n_q_heads / n_kv_heads);
  const bool packed = addr.cu_q != nullptr;  // several query tokens per sequence in the MFMA columns
  if (packed) {
    const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 7) == 0 && ((out_token_stride * 2) & 7) == 0;
    bool pow2 = false;
    for (int s = 4; s < 31; ++s) pow2 |= (1LL << s) == block_size;
    if (csr || lse != nullptr || head_dim != 128 || !pow2 || !out_aligned || group > kMfmaHeads ||
        addr.n_tokens <= 0 || addr.n_tokens > 0x7fffffffLL || addr.chunk_blocks <= 0 || addr.chunk_blocks > kMfmaHeads ||
        addr.window_left >= 0)
      return XLLM_MI355_EINVAL;
  }
  // The step's new rows: inside the matrix-core kernel when it serves the call and a lane can take 16 bytes of a row
  // at a time; otherwise the write is a launch of its own before the decode, with the same result.
  bool fused = false;
  if (fresh != nullptr) {
    GqaArgs probe = {};
    probe.out = static_cast<char*>(out);
    probe.out_stride_bytes = out_token_stride * 2;
    probe.bs_shift = -1;
    for (int s = 0; s < 31; ++s)
      if ((1LL << s) == block_size) probe.bs_shift = s;
    fused = mfma_serves(probe, fp8, static_cast<int>(head_dim)) && aligned16(fresh->key) && aligned16(fresh->value) &&
            (fresh->k_token_stride * 2) % 16 == 0 && (fresh->v_token_stride * 2) % 16 == 0 &&
            fresh->k_token_stride >= n_kv_heads * head_dim && fresh->v_token_stride >= n_kv_heads * head_dim;
    if (!fused) {
      const int rc = reshape_and_cache(fresh->key, fresh->value, const_cast<void*>(k_cache), const_cast<void*>(v_cache),
                                       fresh->slots, k_scale, v_scale, batch, n_kv_heads, head_dim, block_size, num_blocks,
                                       fresh->k_token_stride, fresh->v_token_stride, q_dtype, cache_dtype, stream);
      if (rc != 0) return rc;
    }
  }
  // Batches beyond the LDS prefix capacity are decoded in slices; each slice is an
  // independent launch pair on the same stream and workspace.
  for (int64_t b0 = 0; b0 < batch; b0 += kMaxBatch) {
    const int64_t nb = batch - b0 < kMaxBatch ? batch - b0 : kMaxBatch;
    GqaArgs a = {};
    a.head_lock = 1;
    a.q = static_cast<const char*>(q) + (packed ? 0 : b0 * q_token_stride * 2);
    a.k_cache = static_cast<const char*>(k_cache);
    a.v_cache = static_cast<const char*>(v_cache);
    a.out = static_cast<char*>(out) + (packed ? 0 : b0 * out_token_stride * 2);
    a.lse = lse == nullptr ? nullptr : lse + b0 * n_q_heads;
    a.block_table = csr ? nullptr : (addr.table_rows != nullptr ? addr.block_table : addr.block_table + b0 * addr.table_stride);
    a.table_rows = csr || addr.table_rows == nullptr ? nullptr : addr.table_rows + b0;
    a.seq_lens = csr ? nullptr : addr.seq_lens + b0;
    a.cu_q = packed ? addr.cu_q + b0 : nullptr;
    a.n_tokens = static_cast<int>(addr.n_tokens);
    a.chunk_blocks = addr.chunk_blocks;
    a.causal = addr.causal;
    a.indptr = csr ? addr.indptr + b0 : nullptr;
    a.indices = addr.indices;
    a.last_page_len = csr ? addr.last_page_len + b0 : nullptr;
    a.k_scale = k_scale;
    a.v_scale = v_scale;
    if (fused) {
      a.k_cache_w = const_cast<char*>(a.k_cache);
      a.v_cache_w = const_cast<char*>(a.v_cache);
      a.new_k = static_cast<const char*>(fresh->key) + b0 * fresh->k_token_stride * 2;
      a.new_v = static_cast<const char*>(fresh->value) + b0 * fresh->v_token_stride * 2;
      a.new_slots = fresh->slots + b0;
      a.new_k_stride_bytes = fresh->k_token_stride * 2;
      a.new_v_stride_bytes = fresh->v_token_stride * 2;
      a.n_slots = num_blocks * block_size;
    }
    a.ws_status = static_cast<int*>(workspace);
    a.ws_prefix = reinterpret_cast<int*>(static_cast<char*>(workspace) + kWsHeaderBytes);
    a.plan = !packed && batch <= kMaxBatch ? static_cast<const int*>(addr.plan) : nullptr;
    a.wait_spins = wait_spin_limit();
    a.window_left = addr.window_left < 0 ? -1 : static_cast<int>(addr.window_left < 0x7fffffffLL ? addr.window_left : 0x7fffffffLL);
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
    if (packed) {
      if (q_dtype == XLLM_MI355_BF16)
        rc = fp8 ? launch_gqa_mfma<BF16, true, true>(a, workspace_bytes, stream, false, &need)
                 : launch_gqa_mfma<BF16, false, true>(a, workspace_bytes, stream, false, &need);
      else
        rc = fp8 ? launch_gqa_mfma<FP16, true, true>(a, workspace_bytes, stream, false, &need)
                 : launch_gqa_mfma<FP16, false, true>(a, workspace_bytes, stream, false, &need);
      if (rc != 0) return rc;
      dim3 grid(static_cast<unsigned>(n_kv_heads * addr.chunk_blocks), static_cast<unsigned>(nb));
      if (q_dtype == XLLM_MI355_BF16)
        launch_timed(merge_partials_kernel<BF16, true>, grid, dim3(kThreads), 0, stream, a, static_cast<int>(head_dim));
      else
        launch_timed(merge_partials_kernel<FP16, true>, grid, dim3(kThreads), 0, stream, a, static_cast<int>(head_dim));
      rc = static_cast<int>(hipGetLastError());
      if (rc != 0) return rc;
      continue;
    }
    if (q_dtype == XLLM_MI355_BF16)
      rc = fp8 ? dispatch_dim<BF16, true>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need)
               : dispatch_dim<BF16, false>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need);
    else
      rc = fp8 ? dispatch_dim<FP16, true>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need)
               : dispatch_dim<FP16, false>(a, static_cast<int>(head_dim), workspace_bytes, stream, false, &need);
    if (rc != 0) return rc;
    if (a.fold_merge != 0) {  // the decode kernel merged
      profile_skip();
      continue;
    }
    const int hb_per_kv = (group + a.g_block - 1) / a.g_block;
    dim3 grid(static_cast<unsigned>(n_kv_heads * hb_per_kv), static_cast<unsigned>(nb));
    if (q_dtype == XLLM_MI355_BF16)
      launch_timed(merge_partials_kernel<BF16, false>, grid, dim3(kThreads), 0, stream, a, static_cast<int>(head_dim));
    else
      launch_timed(merge_partials_kernel<FP16, false>, grid, dim3(kThreads), 0, stream, a, static_cast<int>(head_dim));
    rc = static_cast<int>(hipGetLastError());
    if (rc != 0) return rc;
  }
  return XLLM_MI355_OK;
}

}  // namespace xllm_mi355
