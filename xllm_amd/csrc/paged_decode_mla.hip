// Paged decode attention, MLA latent-KV variant, for gfx950.
//
// Four decode kernels live here, each with shapes that no other serves (paged_decode_mla at the end of the file picks):
//   mla_decode_w4_kernel   more than 64 heads, block size a power of two >= 16: the full-model shape (128 heads).  One
//                          workgroup holds O^T of 128 heads in its accumulation registers.  The default there.
//   mla_decode_ds_kernel   the same shapes with 16 heads per MFMA block and O^T by dim block in ordinary registers:
//                          what the build switches those shapes to when the compiler's resource report shows that the
//                          fixed accumulation registers of mla_decode_w4_kernel are not left alone (build.py), and
//                          XLLM_MI355_MLA_KERNEL=narrow by hand.
//   mla_decode16_kernel    up to 64 heads (the heads of a tensor-parallel shard: 16 per MFMA block), same block sizes.
//                          (With more heads only under XLLM_MI355_MLA_KERNEL=heads, for comparison.)
//   mla_decode_kernel      every other block size (below 16, or not a power of two): whole 64-token tiles gathered row
//                          by row.  Described first, below; the others say where they differ.
// mla_merge_tiles_kernel folds the partial pieces of mla_decode_w4_kernel, mla_merge_kernel those of the others.
//
// All query heads share ONE latent KV head of 576 dims (512 latent + 64 rope); V is the
// first 512 dims of the same rows.  With up to 128 heads per sequence the two products are
// dense contractions, so they run on MFMA (v_mfma_f32_32x32x16_bf16):
//   S^T[tok, head]  = K[tok, 576] . Q^T[576, head]       A = K rows from the LDS tile
//                                                        B = Q^T, resident in registers
//   O^T[dim, head] += V^T[dim, tok] . P^T[tok, head]     A = V^T, read from the SAME LDS tile
//                                                            with the transposing LDS load
//                                                        B = P^T, taken from the S^T
//                                                            accumulator registers
// so every 64-token tile is staged in LDS once (rows padded to 1168 bytes: 16 consecutive
// rows then cover all banks for the 16-byte operand reads) and serves both products.
//
// Tiles travel from global memory straight into LDS (global_load_lds_dwordx4), double
// buffered, with the next tile in flight during the whole current tile.
//
// Workgroup = 256 threads = 64 heads: wavefront (hb, t) owns heads 32hb..32hb+31; for
// Q.K it takes token block t (32 tokens) over all 576 dims, for P.V it takes dims
// 256t..256t+255 over all 64 tokens.  The two wavefronts of a head block swap their
// bf16 P^T block and its row maxima through LDS once per tile.  Two barriers per tile:
// (A) tile landed / previous P.V done, (B) exchange visible.  The accumulators are
// rescaled only on tiles where a running maximum moved.
//
// Scheduling: the 64-token tiles of the whole batch form one flat list; a fixed grid of
// persistent workgroups, one per CU, grouped in teams of ceil(H/64) that share a tile
// range (team members get block ids 8 apart, i.e. the same XCD, so the second reader of a
// tile hits that XCD's L2), splits the list into equal contiguous ranges.  A run that
// covers a whole context writes the output, a partial run writes a normalised fp32 partial
// + log2-domain LSE and a small merge kernel folds those.
//
// Semantics: xllm/core/kernels/dcu/flash_mla_adapter.h:40-53 (shapes, single KV head),
// tests/core/layers/mlu/dcp_attention_merge_test.cpp:77-144 (V = K[..., :512], natural-log LSE).
#include <cstdlib>

#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

constexpr int kDL = 512;            // latent dims (= V dims)
constexpr int kDR = 64;             // rope dims
constexpr int kDK = kDL + kDR;      // QK dims
constexpr int kTile = 64;           // tokens per LDS tile (= one schedulable item)
constexpr int kRowBytes = kDK * 2;  // 1152
constexpr int kLdsRow = kRowBytes + 16;
constexpr int kTileBytes = kTile * kLdsRow;  // 74752
constexpr int kMlaThreads = 256;
constexpr int kHeadsPerWg = 64;
constexpr int kKSteps = kDK / 16;   // 36 k-steps of the 32x32x16 MFMA
constexpr float kSlack = 8.0f;    // log2 head room of the running maximum
constexpr int kMaxBatchMla = 1024;  // sequences per launch (their tile prefix lives in LDS)
// LDS map: two tiles | P^T exchange [4 waves][8 regs][64 lanes] | row-max exchange [4][32] | prefix
constexpr int kXchPOff = 2 * kTileBytes;
constexpr int kXchMOff = kXchPOff + 4 * 8 * 64 * 4;
constexpr int kPrefixOff = kXchMOff + 4 * 32 * 4;

typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) u32x2 lds_u32x2;
typedef __attribute__((address_space(3))) float lds_f32;
typedef __attribute__((address_space(3))) volatile int lds_vint;  // a word of LDS that other wavefronts write
struct MlaArgs {
  const char* q_nope;
  const char* q_pe;
  const char* k_cache;
  char* out;
  float* lse;
  const int32_t* block_table;
  const int32_t* seq_lens;
  int* ws_prefix;  // [batch + 1]
  float* ws_out;   // [2 * n_teams][slot_heads][512]: partial rows, head by head, or as the tiles of the accumulators
                   // (mla_decode_w4_kernel with mla_merge_tiles_kernel)
  float* ws_lse;   // [2 * n_teams][H]
  int64_t table_stride;
  int batch;
  int n_heads;
  int slot_heads;  // n_heads rounded up to 16
  // mla_decode_w4_kernel and mla_merge_tiles_kernel: the schedule counts every context that holds tokens as its
  // sub-tiles plus this many, in front of them (the start of a run costs a workgroup about as much as six sub-tiles; a
  // range that holds the start of a context receives that many fewer).  0: the schedule counts sub-tiles only
  int run_cost;
  int n_hb;        // head blocks of 64 = workgroups per team
  int n_teams;
  int block_size;
  int bs_shift;
  int num_blocks;
  float scale_log2;
  // mla_decode_w4_kernel merges the pieces of a context itself and no merge kernel follows (see the fold at the end of
  // that kernel): ws_written holds one counter per (team, head block of 128), zero between launches, that counts the
  // pieces of the context that starts in that team's range as they reach memory
  // mla_decode_w4_kernel: the plan of the step (mla_plan_kernel: kPlan*), or null
  const int* plan;
  int plan_sig;     // what the plan must have been made for, checked against the plan's own first word
  int fold;
  unsigned* ws_written;
  int* ws_status;   // status flags of the workspace (kStatus*), only ever OR-ed into
  int wait_spins;   // bound of the folding workgroup's polls on ws_written
  // mla_decode_w4_kernel, store-then-attend in one launch: the step's new latent rows [batch] of 576 values (row stride
  // in bytes) and their slots, or null.  The workgroup whose run holds a context's last token writes that row to the
  // cache at the start of the run, before it fetches the first tile: what reshape_and_cache would have written before
  // the launch.  Slots outside [0, n_slots) are skipped, as there.
  const char* new_rows;
  const int32_t* new_slots;
  int64_t new_row_stride_bytes;
  int64_t n_slots;
  char* k_cache_w;
};

__device__ __forceinline__ int tiles_of(int L) { return L > 0 ? (L + kTile - 1) / kTile : 0; }
// (32-bit divisions whenever the products fit: a 64-bit one is a long instruction sequence, and these sit on the
// dependent chains at the start of the decode and merge kernels)
__device__ __forceinline__ int64_t team_start(int64_t t, int64_t total, int64_t n) {
  if (total * n < (1LL << 31)) return static_cast<uint32_t>(t) * static_cast<uint32_t>(total) / static_cast<uint32_t>(n);
  return t * total / n;
}
__device__ __forceinline__ int team_of(int64_t id, int64_t total, int64_t n) {
  int64_t t = total * n < (1LL << 31) ? static_cast<int64_t>(static_cast<uint32_t>(id) * static_cast<uint32_t>(n) / static_cast<uint32_t>(total))
                                      : id * n / total;
  while (t + 1 < n && team_start(t + 1, total, n) <= id) ++t;
  return static_cast<int>(t);
}

__device__ __forceinline__ float half_swap_max(float x) {  // over lanes l and l ^ 32
  auto t = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
  return fmaxf(as_f32(t[0]), as_f32(t[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
  auto t = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
  return as_f32(t[0]) + as_f32(t[1]);
}

// 16 bytes per active lane from global memory straight into LDS at lds_addr + lane * 16
// (lds_addr is wave-uniform; it travels in M0).  Every tile load of this file is marked non-temporal:
// a launch reads each latent row once, and streaming reads that bypass the caches move faster on this GPU.
__device__ __forceinline__ void dma16(const void* gptr, u32 lds_addr) {
  const u32 base = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(base), "v"(gptr) : "memory");
}
// Same with a wave-uniform 64-bit row base in SGPRs plus a 32-bit per-lane byte offset.
__device__ __forceinline__ void dma16_row(uint64_t row_base, u32 lane_off, u32 lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(lane_off), "s"(row_base)
               : "memory");
}
__device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <typename QT>
__global__ __launch_bounds__(kMlaThreads) void mla_decode_kernel(MlaArgs a) {
  extern __shared__ __align__(16) char smem[];
  u32* xch_p = reinterpret_cast<u32*>(smem + kXchPOff);
  float* xch_m = reinterpret_cast<float*>(smem + kXchMOff);
  int* prefix = reinterpret_cast<int*>(smem + kPrefixOff);
  int* tmp = reinterpret_cast<int*>(smem + kXchPOff);  // prologue only

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int hb32 = wave >> 1;   // 32-head block of the wavefront
  const int tblk = wave & 1;    // its token block for Q.K and its dim half for P.V
  const int c32 = lane & 31;    // MFMA row / column index owned by the lane
  const int g = lane >> 5;      // MFMA k-group of the lane
  const int H = a.n_heads;

  // block id -> (team, head block): members of a team are 8 ids apart (same XCD)
  const int xcd = blockIdx.x & 7;
  const int y = blockIdx.x >> 3;
  const int hb64 = y % a.n_hb;
  const int team = (y / a.n_hb) * 8 + xcd;
  const int head = hb64 * kHeadsPerWg + hb32 * 32 + c32;
  const bool head_ok = head < H;
  const bool wave_ok = hb64 * kHeadsPerWg + hb32 * 32 < H;

  // ---- tile prefix over the batch (every workgroup computes it; no extra launch)
  {
    const int per = (a.batch + kMlaThreads - 1) / kMlaThreads;
    const int lo = min(a.batch, tid * per), hi = min(a.batch, lo + per);
    int local = 0;
    for (int b = lo; b < hi; ++b) local += tiles_of(a.seq_lens[b]);
    tmp[tid] = local;
    __syncthreads();
    if (lo < hi) {  // (threads without a slice have nothing to place: most of them at decode batch sizes)
      int excl = 0;
      for (int j = 0; j < tid; ++j) excl += tmp[j];
      if (per == 1) {  // the slice is one sequence: its count is still in `local`
        prefix[lo] = excl;
        excl += local;
      } else {
        for (int b = lo; b < hi; ++b) {
          prefix[b] = excl;
          excl += tiles_of(a.seq_lens[b]);
        }
      }
      if (hi == a.batch) prefix[a.batch] = excl;
    }
    __syncthreads();
  }
  const int64_t total = prefix[a.batch];
  if (blockIdx.x == 0)
    for (int i = tid; i <= a.batch; i += kMlaThreads) a.ws_prefix[i] = prefix[i];
  if (total == 0) return;
  int64_t cur = team_start(team, total, a.n_teams);
  const int64_t end = team_start(team + 1, total, a.n_teams);
  bool first_run = true;

  const u32 lds_base = static_cast<u32>(reinterpret_cast<uintptr_t>(smem));

  while (cur < end) {
    int lo = 0, hi = a.batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (prefix[mid] <= cur) lo = mid; else hi = mid;
    }
    const int b = lo;
    const int n_tiles_seq = prefix[b + 1] - prefix[b];
    const int tile0 = static_cast<int>(cur - prefix[b]);
    const int run_tiles = static_cast<int>(min<int64_t>(n_tiles_seq - tile0, end - cur));
    const bool complete = tile0 == 0 && run_tiles == n_tiles_seq;
    cur += run_tiles;
    const int32_t* pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
    const int L = a.seq_lens[b];

    // Q^T operand: lane (head c32, k-group g) keeps dims ks*16 + g*8 .. +8 of every k-step
    u32x4 q[kKSteps];
    {
      const char* qn = a.q_nope + (static_cast<int64_t>(b) * H + head) * kDL * 2;
      const char* qp = a.q_pe + (static_cast<int64_t>(b) * H + head) * kDR * 2;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        u32x4 x = {0u, 0u, 0u, 0u};
        if (head_ok)
          x = ks < kDL / 16 ? ldg16(qn + (ks * 16 + g * 8) * 2) : ldg16(qp + ((ks - kDL / 16) * 16 + g * 8) * 2);
        q[ks] = x;
      }
    }
    f32x16 o[8];  // O^T blocks: dims tblk*256 + mb*32 + (8*(r/4) + 4g + r%4), head c32
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[i][r] = 0.0f;
    float m = kNegBig, l = 0.0f;

    // Tile rows go from global memory straight into LDS (no staging registers): one
    // 64-lane load moves the 1024 latent bytes of a row, a second one with 8 lanes the 128
    // rope bytes.  Each wavefront moves 16 rows; lane i < 16 first looks up the slot of row i.
    // The loads are issued from inline assembly so that the compiler's own wait insertion
    // does not see them: they are awaited explicitly (dma_wait) one tile later.
    // slot (page * bs + row) of row wave*16 + (lane & 15) of a tile; looked up one tile before
    // the tile is issued, so the table load's latency never sits in front of the tile loads
    auto lookup_page = [&](int tile, int& row_off) {
      const int tok = min((tile0 + tile) * kTile + wave * 16 + (lane & 15), L - 1);
      int pg, off;
      if (a.bs_shift >= 0) {
        pg = tok >> a.bs_shift;
        off = tok & (a.block_size - 1);
      } else {
        pg = tok / a.block_size;
        off = tok - pg * a.block_size;
      }
      row_off = off;
      return pages[pg];  // raw: nothing may depend on the loaded value before the tile is issued
    };
    auto issue_tile = [&](int page, int off, int buf) {
      asm volatile("" : "+v"(page));  // the wait for the table load belongs here, one tile later
      page = max(0, min(page, a.num_blocks - 1));  // a corrupt table must not fault the GPU
      const int slot = page * a.block_size + off;
      const u32 lds_tile =
          __builtin_amdgcn_readfirstlane(lds_base + buf * kTileBytes + wave * 16 * kLdsRow);
      const uint64_t cache = reinterpret_cast<uint64_t>(a.k_cache);
      const u32 lane_off = lane * 16;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint64_t row = cache + static_cast<uint64_t>(static_cast<u32>(__builtin_amdgcn_readlane(slot, i))) * kRowBytes;
        dma16_row(row, lane_off, lds_tile + i * kLdsRow);
        if (lane < kDR * 2 / 16) dma16_row(row + kDL * 2, lane_off, lds_tile + i * kLdsRow + kDL * 2);
      }
    };

    // make the compiler wait for the Q loads here, not after the first tile prefetch
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      u32x4 x = __builtin_bit_cast(u32x4, q[ks]);
      asm volatile("" : "+v"(x));
      q[ks] = x;
    }
    __syncthreads();  // the previous run no longer reads the tiles or the exchange buffers
    int off_next = 0;
    int page_next = lookup_page(0, off_next);
    issue_tile(page_next, off_next, 0);
    page_next = lookup_page(1, off_next);

    for (int tile = 0; tile < run_tiles; ++tile) {
      const int buf = tile & 1;
      const char* kb = smem + buf * kTileBytes;
      dma_wait();
      __syncthreads();  // (A) this tile has landed in LDS; every wavefront is past the previous P.V
      if (tile + 1 < run_tiles) {
        issue_tile(page_next, off_next, buf ^ 1);  // in flight during the whole tile
        page_next = lookup_page(tile + 2, off_next);
      }

      u32 pk_own[8];
      float m_own = kNegBig, sum_own = 0.0f;
      if (wave_ok) {
        // ---- S^T block of this wavefront: tokens tblk*32 + (8*(r/4) + 4g + r%4), head c32
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.0f;
        const char* ka = kb + (tblk * 32 + c32) * kLdsRow + g * 16;
        __builtin_amdgcn_sched_barrier(0);  // the pipeline below covers the Q.K reads only
#pragma unroll
        for (int ks = 0; ks < kKSteps; ks += 2) {
          const u32x4 x0 = *reinterpret_cast<const u32x4*>(ka + ks * 32);
          const u32x4 x1 = *reinterpret_cast<const u32x4*>(ka + ks * 32 + 32);
          s = Mfma<QT>::w32(x0, q[ks], s);
          s = Mfma<QT>::w32(x1, q[ks + 1], s);
        }
        // pipeline the LDS operand reads four MFMAs ahead of their use
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < kKSteps - 4; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_barrier(0);
        const int tok_base = (tile0 + tile) * kTile + tblk * 32 + g * 4;
        if ((tile0 + tile + 1) * kTile > L) {  // only the last tile of a context is ragged
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (tok_base + 8 * (r >> 2) + (r & 3) >= L) s[r] = -INFINITY;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) m_own = fmaxf(m_own, s[r]);
        m_own = half_swap_max(m_own) * a.scale_log2;  // row maximum of this token block (scale > 0)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          s[r] = fast_exp2(__builtin_fmaf(s[r], a.scale_log2, -m_own));
          sum_own += s[r];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) pk_own[i] = QT::pack(s[2 * i], s[2 * i + 1]);
#pragma unroll
        for (int i = 0; i < 8; ++i) xch_p[(wave * 8 + i) * 64 + lane] = pk_own[i];
        if (g == 0) xch_m[wave * 32 + c32] = m_own;
      }
      __syncthreads();  // (B) P^T blocks and maxima of this tile are visible
      float m_other = kNegBig;
      u32 theirs_raw[8];
      if (wave_ok) {
        m_other = xch_m[(wave ^ 1) * 32 + c32];
#pragma unroll
        for (int i = 0; i < 8; ++i) theirs_raw[i] = xch_p[((wave ^ 1) * 8 + i) * 64 + lane];
      }

      if (wave_ok) {
        // The reference maximum m only follows the tile maxima when they exceed it by more than
        // kSlack (log2 units): probabilities then stay below 2^kSlack, well inside bf16 / fp32
        // range, and the 128 accumulators are rescaled a handful of times per context.
        const float m_tile = fmaxf(m_own, m_other);
        const float m_new = m_tile > m + kSlack ? m_tile : m;
        const float alpha = fast_exp2(m - m_new);
        const float f_own = fast_exp2(m_own - m_new);
        const float f_other = fast_exp2(m_other - m_new);
        m = m_new;
        l = l * alpha + sum_own * f_own;  // this wavefront's share of the normaliser
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
          for (int i = 0; i < 8; ++i) o[i] *= alpha;
        }
        // B operands per k-step: k-slot g*8 + j <-> rows 16*kk + 4g + j (j < 4), + 8 more (j >= 4)
        // of the own token block (pb_own) and of the partner's (pb_other)
        u32x4 pb_own[2], pb_other[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          u32x4 mine, theirs;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const u32 w = pk_own[4 * kk + i];
            mine[i] = QT::pack(QT::lo(w) * f_own, QT::hi(w) * f_own);
            const u32 t = theirs_raw[4 * kk + i];
            theirs[i] = QT::pack(QT::lo(t) * f_other, QT::hi(t) * f_other);
          }
          pb_own[kk] = mine;
          pb_other[kk] = theirs;
        }
        // ---- O^T += V^T . P^T over the 64 tokens, dims tblk*256 .. +256.  The transposing
        // LDS load works on groups of 16 lanes: lane p of a group supplies the address of 4
        // dims of token row p/4 and receives the 4 tokens of dim column p.
        const int p16 = lane & 15;
        const char* vb = kb + (g * 4 + (p16 >> 2)) * kLdsRow +
                         (tblk * 256 + ((lane >> 4) & 1) * 16 + (p16 & 3) * 4) * 2;
        const char* vb_own = vb + tblk * 32 * kLdsRow;
        const char* vb_other = vb + (tblk ^ 1) * 32 * kLdsRow;
        __builtin_amdgcn_sched_barrier(0);  // the pipeline below covers the P.V reads only
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {  // own token block: k-steps 0, 1; the partner's: 2, 3
#pragma unroll
          for (int mb = 0; mb < 8; ++mb) {  // 8 independent accumulators per k-step
            const char* rows = (ks < 2 ? vb_own : vb_other) + (16 * (ks & 1)) * kLdsRow + mb * 64;
            const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(rows));
            const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(rows + 8 * kLdsRow));
            const s16x8 v = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
            o[mb] = Mfma<QT>::w32(__builtin_bit_cast(u32x4, v), ks < 2 ? pb_own[ks & 1] : pb_other[ks & 1], o[mb]);
          }
        }
        // pipeline the transposing reads (two per MFMA) four MFMAs ahead of their use
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < 28; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- end of the run: the two wavefronts of a head block add their normaliser shares
    __syncthreads();
    const float l_wave = half_swap_sum(l);
    if (wave_ok && g == 0) xch_m[wave * 32 + c32] = l_wave;
    __syncthreads();
    if (head_ok) {
      const float lsum = xch_m[wave * 32 + c32] + xch_m[(wave ^ 1) * 32 + c32];
      const float inv = 1.0f / lsum;
      if (complete) {
        char* op = a.out + ((static_cast<int64_t>(b) * H + head) * kDL + tblk * 256) * 2;
#pragma unroll
        for (int mb = 0; mb < 8; ++mb)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            u32x2 w;
            w[0] = QT::pack(o[mb][4 * qd] * inv, o[mb][4 * qd + 1] * inv);
            w[1] = QT::pack(o[mb][4 * qd + 2] * inv, o[mb][4 * qd + 3] * inv);
            *reinterpret_cast<u32x2*>(op + (mb * 32 + 8 * qd + 4 * g) * 2) = w;
          }
        if (a.lse != nullptr && g == 0 && tblk == 0) a.lse[b * H + head] = (m + fast_log2(lsum)) * kLn2;
      } else {
        const int64_t ps = (static_cast<int64_t>(team) * 2 + (first_run ? 0 : 1)) * H + head;
        float* wp = a.ws_out + ps * kDL + tblk * 256;
#pragma unroll
        for (int mb = 0; mb < 8; ++mb)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            f32x4 w = {o[mb][4 * qd] * inv, o[mb][4 * qd + 1] * inv, o[mb][4 * qd + 2] * inv,
                       o[mb][4 * qd + 3] * inv};
            *reinterpret_cast<f32x4*>(wp + mb * 32 + 8 * qd + 4 * g) = w;
          }
        if (g == 0 && tblk == 0) a.ws_lse[ps] = m + fast_log2(lsum);
      }
    }
    first_run = false;
  }
}

// ---------------------------------------------------------------------------------------------
// Main kernel: 16 heads per wavefront, nothing exchanged between wavefronts, and a four-deep ring
// of 32-token sub-tiles.
//
// Workgroup = 512 threads = 8 wavefronts = 128 heads: wavefront w owns heads 16w..16w+15 for all
// 32 tokens of every sub-tile and all 512 output dims, with v_mfma_f32_16x16x32_bf16 for BOTH
// products:
//   S^T[tok, head] = K[tok, 576] . Q^T[576, head]    2 token blocks x 18 k-steps, A = K rows from the
//                                                    LDS sub-tile, B = Q^T in 72 VGPRs
//   O^T[dim, head] += V^T[dim, tok] . P^T[tok, head]  32 dim blocks over the 32 tokens, A = V^T through the
//                                                    transposing LDS read, B = P^T taken from the S^T
//                                                    accumulator registers
// so a lane owns one head, its softmax state is a pair of per-lane scalars and a wavefront writes
// its own heads at the end of a run.  One barrier per sub-tile (sub-tile landed / oldest ring
// slot released).  With at most 256 registers per wavefront two wavefronts share a SIMD, so
// one's softmax overlaps the other's MFMAs.
//
// Three sub-tiles are in flight while one is consumed: with a single tile of prefetch the loop ran
// at the latency of a tile fetch.  As in the GQA matrix-core kernel nothing in the loop waits on a
// register load (the in-order counter would drain the ring): page-table entries come through the
// LDS path in chunks of 64, fetched by wavefront 0 at least 32 sub-tiles ahead.
//
// A sub-tile in LDS is two areas.  The latent parts of its rows are 1056 bytes apart and the 16-byte
// chunks of a row are XOR-ed with bit 2 of the row number: the 16-byte operand reads (8 consecutive
// rows per cycle) and the transposing reads (4 rows x 32 bytes per cycle) then both touch every LDS
// bank once.  The rope parts sit behind them, 128 bytes per row, chunk XOR-ed with the low 3 bits of
// the row number.  Keeping them apart lets ONE load instruction bring the rope bytes of 4 rows (32
// lanes x 16 bytes, the lane picks row and chunk through its global offset) instead of one
// 8-lane instruction per row: a wavefront issues 5 loads per sub-tile instead of 8 (an 8-lane
// load costs its wavefront as much issue time as a 64-lane one).  With 128 heads that time is
// covered by the other wavefront of the SIMD and the layout changes nothing; with the few heads
// of a tensor-parallel shard the computing wavefronts also issue loads and it is on their path.
constexpr int kRow16 = kDL * 2 + 32;
constexpr int kSubTok = 32;                      // tokens per sub-tile
constexpr int kRing16 = 4;                       // ring slots
constexpr int kRope16Off = kSubTok * kRow16;     // rope area of a sub-tile
constexpr int kSubBytes = kRope16Off + kSubTok * kDR * 2;  // 37888
constexpr int kLoadsPerSub16 = 5;                // per wavefront
constexpr int kThreads16 = 512;
constexpr int kHeadsPerWg16 = 128;
constexpr int kPage16Off = kRing16 * kSubBytes;  // LDS: ring | page-table chunks [2][64] | prefix
constexpr int kPrefix16Off = kPage16Off + 2 * kWave * 4;
constexpr int kKSteps32 = kDK / 32;              // 18 k-steps of the 16x16x32 MFMA
constexpr int kAhead = 4;                        // LDS operand reads in flight ahead of the MFMAs

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
// 4 bytes per lane from global memory straight into LDS at lds_addr + lane * 4
__device__ __forceinline__ void dma4(const void* gptr, u32 lds_addr) {
  const u32 base = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(base), "v"(gptr) : "memory");
}
// Wait until at most kLoadsPerSub16 * subs of the wavefront's vector memory operations are outstanding.
__device__ __forceinline__ void wait_younger_subs(int subs) {
  static_assert(kLoadsPerSub16 == 5, "the immediates below are multiples of the loads per sub-tile");
  if (subs <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if (subs == 1) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
}

//
// SPLIT (at most 64 heads per GPU, the head counts of tensor-parallel shards): with 16 heads per
// wavefront only H / 16 wavefronts would compute and the loop would run at the pace of one
// wavefront's chain of reads and MFMAs, well below what HBM delivers.  The two 16-token blocks of
// every sub-tile then go to different wavefronts: wavefront (head block w % 4, token block w / 4)
// keeps its own maximum, sum and O^T, and at the end of a run the token-block-1 wavefronts hand
// theirs to their partners through the (then idle) ring, merged like two partials.
template <typename QT, bool SPLIT>
__global__ __launch_bounds__(kThreads16) void mla_decode16_kernel(MlaArgs a) {
  extern __shared__ __align__(16) char smem[];
  int* prefix = reinterpret_cast<int*>(smem + kPrefix16Off);
  const int* pagebuf = reinterpret_cast<const int*>(smem + kPage16Off);
  int* tmp = reinterpret_cast<int*>(smem);  // prologue only

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15;    // MFMA row / column index owned by the lane
  const int g = lane >> 4;      // MFMA k-group of the lane
  const int H = a.n_heads;

  // block id -> (team, head block): members of a team are 8 ids apart (same XCD)
  const int xcd = blockIdx.x & 7;
  const int y = blockIdx.x >> 3;
  const int hb128 = y % a.n_hb;
  const int team = (y / a.n_hb) * 8 + xcd;
  const int hblk = SPLIT ? (wave & 3) : wave;  // 16-head block of the wavefront
  const int tb = SPLIT ? (wave >> 2) : 0;      // SPLIT: its 16-token block of every sub-tile
  const int head = hb128 * kHeadsPerWg16 + hblk * 16 + c16;
  const bool head_ok = head < H;
  const bool wave_ok = hb128 * kHeadsPerWg16 + hblk * 16 < H;

  // ---- tile prefix over the batch (every workgroup computes it; no extra launch)
  {
    const int per = (a.batch + kThreads16 - 1) / kThreads16;
    const int lo = min(a.batch, tid * per), hi = min(a.batch, lo + per);
    int local = 0;
    for (int b = lo; b < hi; ++b) local += tiles_of(a.seq_lens[b]);
    tmp[tid] = local;
    __syncthreads();
    if (lo < hi) {  // (threads without a slice have nothing to place: most of them at decode batch sizes)
      int excl = 0;
      for (int j = 0; j < tid; ++j) excl += tmp[j];
      if (per == 1) {  // the slice is one sequence: its count is still in `local`
        prefix[lo] = excl;
        excl += local;
      } else {
        for (int b = lo; b < hi; ++b) {
          prefix[b] = excl;
          excl += tiles_of(a.seq_lens[b]);
        }
      }
      if (hi == a.batch) prefix[a.batch] = excl;
    }
    __syncthreads();
  }
  const int64_t total = prefix[a.batch];
  if (blockIdx.x == 0)
    for (int i = tid; i <= a.batch; i += kThreads16) a.ws_prefix[i] = prefix[i];
  if (total == 0) return;
  int64_t cur = team_start(team, total, a.n_teams);
  const int64_t end = team_start(team + 1, total, a.n_teams);
  bool first_run = true;

  const u32 lds_base = static_cast<u32>(reinterpret_cast<uintptr_t>(smem));
  const u32 page_lds = __builtin_amdgcn_readfirstlane(lds_base + kPage16Off);
  // per-lane constants of the operand reads (byte offsets inside a sub-tile)
  //   K: row c16 (+ 16 for the second token block), 16-byte chunk kk*4 + g XOR-ed with bit 2 of the row: + kk * 64
  const int k_row0 = c16 * kRow16 + ((g ^ ((c16 >> 2) & 1)) * 16);
  //   V: lane c16 of a 16-lane group addresses 4 dims (8 bytes) of token row 4g + c16/4 (+ 16),
  //      chunk 2 mb + (c16 & 3) / 2 XOR-ed with bit 2 of the row (= g & 1): + mb * 32
  const int v_row0 = (4 * g + (c16 >> 2)) * kRow16 + ((((c16 & 3) >> 1) ^ (g & 1)) * 16) + (c16 & 1) * 8;
  // tile loads: this wavefront moves rows wave*4 .. +3 of a sub-tile; bit 2 of those rows is wave & 1
  const u32 lane_off = (lane ^ (wave & 1)) * 16;
  // The kernel runs at the register limit, and a per-lane constant more costs the operand reads of
  // the loop a buffer of their pipeline: the few per-lane offsets of the rope area are therefore
  // recomputed where they are used, from this copy of the lane number that the compiler cannot
  // trace back to the thread index (it would otherwise hoist them into registers of their own).
  auto lane_again = [&]() {
    u32 x = lane_off;
    asm volatile("" : "+v"(x));
    return static_cast<int>(x >> 4) ^ (wave & 1);
  };

  while (cur < end) {
    int lo = 0, hi = a.batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (prefix[mid] <= cur) lo = mid; else hi = mid;
    }
    const int b = __builtin_amdgcn_readfirstlane(lo);
    const int n_tiles_seq = prefix[b + 1] - prefix[b];
    const int tile0 = static_cast<int>(cur - prefix[b]);
    const int run_tiles = static_cast<int>(min<int64_t>(n_tiles_seq - tile0, end - cur));
    const bool complete = tile0 == 0 && run_tiles == n_tiles_seq;
    cur += run_tiles;
    const int32_t* pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
    const int L = __builtin_amdgcn_readfirstlane(a.seq_lens[b]);
    const int t_begin = tile0 * kTile;
    const int t_end = min(L, (tile0 + run_tiles) * kTile);
    const int n_sub = (t_end - t_begin + kSubTok - 1) / kSubTok;
    const int n_pages = (L + a.block_size - 1) >> a.bs_shift;

    // Q^T operand: lane (head c16, k-group g) keeps dims kk*32 + g*8 .. +8 of every k-step
    u32x4 q[kKSteps32];
    {
      const char* qn = a.q_nope + (static_cast<int64_t>(b) * H + head) * kDL * 2;
      const char* qp = a.q_pe + (static_cast<int64_t>(b) * H + head) * kDR * 2;
#pragma unroll
      for (int kk = 0; kk < kKSteps32; ++kk) {
        u32x4 x = {0u, 0u, 0u, 0u};
        if (head_ok)
          x = kk < kDL / 32 ? ldg16(qn + (kk * 32 + g * 8) * 2) : ldg16(qp + ((kk - kDL / 32) * 32 + g * 8) * 2);
        q[kk] = x;
      }
    }
    f32x4 o[32];  // O^T blocks: dims mb*16 + 4g + r, head c16
#pragma unroll
    for (int i = 0; i < 32; ++i) o[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = kNegBig, l = 0.0f;

    // 64 entries of the page table from page 64 ck on (the tail repeats the last page) -> chunk buffer ck & 1
    auto issue_chunk = [&](int ck) {
      dma4(pages + min(ck * kWave + lane, n_pages - 1), page_lds + (ck & 1) * kWave * 4);
    };
    int ck_cur = (t_begin >> a.bs_shift) >> 6;  // chunk of the sub-tile being issued
    // Rows go from global memory straight into LDS: one 64-lane load per row moves its 1024 latent
    // bytes, a fifth load with 32 lanes the 128 rope bytes of all 4 rows.
    auto issue_sub = [&](int sub) {
      const int tok0 = t_begin + sub * kSubTok + wave * 4;  // block_size >= 16: the 4 rows share a page
      const u32 slot = lds_base + (sub & (kRing16 - 1)) * kSubBytes;
      const u32 dst = __builtin_amdgcn_readfirstlane(slot + wave * 4 * kRow16);
      const u32 dst_rope = __builtin_amdgcn_readfirstlane(slot + kRope16Off + wave * 4 * (kDR * 2));
      const uint64_t cache = reinterpret_cast<uint64_t>(a.k_cache);
      const int tb = min(tok0, L - 1);  // rows past the end of the context repeat the last valid row
      const int ck = (tb >> a.bs_shift) >> 6;
      if (ck != ck_cur) {  // first sub-tile of a chunk: wavefront 0 fetches the one after it
        ck_cur = ck;
        if (wave == 0 && (ck + 1) * kWave < n_pages) issue_chunk(ck + 1);
      }
      int page = __builtin_amdgcn_readfirstlane(pagebuf[(ck & 1) * kWave + ((tb >> a.bs_shift) & 63)]);
      page = max(0, min(page, a.num_blocks - 1));  // a corrupt table must not fault the GPU
      const uint64_t row = cache + static_cast<uint64_t>(page * a.block_size + (tb & (a.block_size - 1))) * kRowBytes;
      const u32 lo = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(row)));
      const u32 hi = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(row >> 32)));
      const uint64_t sb = (static_cast<uint64_t>(hi) << 32) | lo;
      const int last = __builtin_amdgcn_readfirstlane(L - 1 - tb);  // valid rows after the first: >= 0
#pragma unroll
      for (int i = 0; i < 4; ++i) dma16_row(sb + static_cast<uint64_t>(min(i, last)) * kRowBytes, lane_off, dst + i * kRow16);
      // rope load: lane (row r = lane / 8 of the 4, position p = lane % 8) lands at rope row wave*4 + r,
      // position p, and so fetches chunk p ^ (low 3 bits of that row)
      const int ln = lane_again();
      const int rope_r = (ln >> 3) & 3;
      const u32 rope_off = min(rope_r, last) * kRowBytes + kDL * 2 + (((ln & 7) ^ ((wave & 1) * 4 + rope_r)) * 16);
      if (lane < 4 * kDR * 2 / 16) dma16_row(sb, rope_off, dst_rope);
    };

    // make the compiler wait for the Q loads here, not inside the loop
#pragma unroll
    for (int kk = 0; kk < kKSteps32; ++kk) asm volatile("" : "+v"(q[kk]));
    __syncthreads();  // the previous run no longer reads the ring or the chunks
    if (wave == 0) {
      issue_chunk(ck_cur);
      if ((ck_cur + 1) * kWave < n_pages) issue_chunk(ck_cur + 1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    for (int sub = 0; sub < kRing16 - 1 && sub < n_sub; ++sub) issue_sub(sub);

    for (int sub = 0; sub < n_sub; ++sub) {
      wait_younger_subs(min(kRing16 - 2, n_sub - 1 - sub));
      __syncthreads();  // this sub-tile has landed in LDS; every wavefront is past the previous one
      // Every wavefront issues its rows of sub-tile sub + 3 (into the slot released just now) before it
      // computes.  (With 8 loads per wavefront it paid to let the second wavefront of each SIMD issue after
      // its arithmetic; with 5 it no longer does.)
      if (sub + kRing16 - 1 < n_sub) issue_sub(sub + kRing16 - 1);
      const char* kb = smem + (sub & (kRing16 - 1)) * kSubBytes;
      if (wave_ok) {
        // rope k-steps: row c16 of the rope area, chunk (kk - 16) * 4 + g XOR-ed with the low 3 bits of the row
        const int ln = lane_again();
        const char* kr = kb + kRope16Off + (ln & 15) * (kDR * 2);
        const int kr_x = (ln >> 4) ^ (ln & 7);
        if constexpr (SPLIT) {
          // ---- S^T of the wavefront's 16 tokens: lane (head c16, tokens 16 tb + 4g + r)
          f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f};
          const char* ka = kb + k_row0 + tb * 16 * kRow16;
          __builtin_amdgcn_sched_barrier(0);  // the pipeline below covers the Q.K reads only
#pragma unroll
          for (int kk = 0; kk < kKSteps32; ++kk) {
            const char* k0 = kk < kDL / 32 ? ka + kk * 64 : kr + tb * 16 * (kDR * 2) + (kk == kDL / 32 ? kr_x : kr_x ^ 4) * 16;
            const u32x4 x0 = *reinterpret_cast<const u32x4*>(k0);
            s0 = Mfma<QT>::k32(x0, q[kk], s0);
          }
          __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
          for (int i = 0; i < kKSteps32 - kAhead; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
          __builtin_amdgcn_sched_barrier(0);
          float sv[4];
          const int tok_base = t_begin + sub * kSubTok + tb * 16 + 4 * g;
          bool over = false;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            sv[r] = tok_base + r < L ? s0[r] * a.scale_log2 : -INFINITY;
            over |= sv[r] > m + kSlack;
          }
          if (__builtin_amdgcn_ballot_w64(over) != 0) {  // rare once the maxima have settled
            const float mx = quad_rows_max(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])));
            if (mx > m + kSlack) {
              const float alpha = fast_exp2(m - mx);
              m = mx;
              l *= alpha;
#pragma unroll
              for (int i = 0; i < 32; ++i) o[i] *= alpha;
            }
          }
          float p[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            p[r] = fast_exp2(sv[r] - m);
            l += p[r];
          }
          const u32x2 pb = {QT::pack(p[0], p[1]), QT::pack(p[2], p[3])};
          // ---- O^T += V^T . P^T over the 16 tokens: k-slot 4g + j of the MFMA <-> token 4g + j of the block
          const char* va = kb + v_row0 + tb * 16 * kRow16;
          __builtin_amdgcn_sched_barrier(0);  // the pipeline below covers the P.V reads only
#pragma unroll
          for (int mb = 0; mb < 32; ++mb) {
            const s16x4 v4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + mb * 32));
            o[mb] = Mfma<QT>::k16(v4, pb, o[mb]);
          }
          __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
          for (int i = 0; i < 32 - kAhead; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
          __builtin_amdgcn_sched_barrier(0);
        } else {
          // ---- S^T of the sub-tile, two blocks of 16 tokens: lane (head c16, tokens 16 tb + 4g + r)
          f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
          const char* ka = kb + k_row0;
          __builtin_amdgcn_sched_barrier(0);  // the pipeline below covers the Q.K reads only
#pragma unroll
          for (int kk = 0; kk < kKSteps32; ++kk) {
            const char* k0 = kk < kDL / 32 ? ka + kk * 64 : kr + (kk == kDL / 32 ? kr_x : kr_x ^ 4) * 16;
            const u32x4 x0 = *reinterpret_cast<const u32x4*>(k0);
            const u32x4 x1 = *reinterpret_cast<const u32x4*>(k0 + 16 * (kk < kDL / 32 ? kRow16 : kDR * 2));
            s0 = Mfma<QT>::k32(x0, q[kk], s0);
            s1 = Mfma<QT>::k32(x1, q[kk], s1);
          }
          // pipeline the LDS operand reads kAhead MFMAs ahead of their use
          __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
          for (int i = 0; i < 2 * kKSteps32 - kAhead; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
          __builtin_amdgcn_sched_barrier(0);
          float sv[8];
          const int tok_base = t_begin + sub * kSubTok + 4 * g;
          bool over = false;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            sv[r] = tok_base + r < L ? s0[r] * a.scale_log2 : -INFINITY;
            sv[4 + r] = tok_base + 16 + r < L ? s1[r] * a.scale_log2 : -INFINITY;
          }
#pragma unroll
          for (int r = 0; r < 8; ++r) over |= sv[r] > m + kSlack;
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
              for (int i = 0; i < 32; ++i) o[i] *= alpha;
            }
          }
          float p[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            p[r] = fast_exp2(sv[r] - m);
            l += p[r];
          }
          // k-slot g*8 + j of the P.V MFMA <-> token 4g + j of block 0 (j < 4), of block 1 (j >= 4)
          const u32x4 pb = {QT::pack(p[0], p[1]), QT::pack(p[2], p[3]), QT::pack(p[4], p[5]), QT::pack(p[6], p[7])};
          // ---- O^T += V^T . P^T over the 32 tokens and all 512 dims.  The transposing LDS load works on
          // groups of 16 lanes: lane p of a group supplies the address of 4 dims of token row p/4 and
          // receives the 4 tokens of dim column p.
          const char* va = kb + v_row0;
          __builtin_amdgcn_sched_barrier(0);  // the pipeline below covers the P.V reads only
#pragma unroll
          for (int mb = 0; mb < 32; ++mb) {
            const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + mb * 32));
            const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + 16 * kRow16 + mb * 32));
            const s16x8 v = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
            o[mb] = Mfma<QT>::k32(__builtin_bit_cast(u32x4, v), pb, o[mb]);
          }
          // pipeline the transposing reads (two per MFMA) kAhead MFMAs ahead of their use
          __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
          for (int i = 0; i < 32 - kAhead; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, kAhead, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    if constexpr (SPLIT) {
      // the token-block-1 wavefronts hand their state to their partners: [head block][value][lane] floats
      // in the ring, which nobody reads or writes between the last sub-tile and the next run
      constexpr int kState = 32 * 4 + 2;
      float* xch = reinterpret_cast<float*>(smem) + hblk * kState * kWave + lane;
      static_assert(4 * kState * kWave * 4 <= kRing16 * kSubBytes, "the exchange fits the ring");
      __syncthreads();
      if (tb == 1 && wave_ok) {
#pragma unroll
        for (int i = 0; i < 32; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) xch[(i * 4 + r) * kWave] = o[i][r];
        xch[128 * kWave] = m;
        xch[129 * kWave] = l;
      }
      __syncthreads();
      if (tb == 0 && wave_ok) {
        const float m1 = xch[128 * kWave], l1 = xch[129 * kWave];
        const float mm = fmaxf(m, m1);
        const float a0 = fast_exp2(m - mm), a1 = fast_exp2(m1 - mm);
#pragma unroll
        for (int i = 0; i < 32; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[i][r] = o[i][r] * a0 + xch[(i * 4 + r) * kWave] * a1;
        l = l * a0 + l1 * a1;
        m = mm;
      }
    }
    // ---- end of the run: every wavefront (SPLIT: of token block 0) writes its own heads
    const bool writer = head_ok && tb == 0;
    const float lsum = quad_rows_sum(l);
    const float inv = 1.0f / lsum;
    const float lse2 = m + fast_log2(lsum);
    const int64_t ps = (static_cast<int64_t>(team) * 2 + (first_run ? 0 : 1)) * H + head;
    if (writer && complete) {
      char* op = a.out + ((static_cast<int64_t>(b) * H + head) * kDL + 4 * g) * 2;
#pragma unroll
      for (int mb = 0; mb < 32; ++mb) {
        const u32x2 w = {QT::pack(o[mb][0] * inv, o[mb][1] * inv), QT::pack(o[mb][2] * inv, o[mb][3] * inv)};
        *reinterpret_cast<u32x2*>(op + mb * 32) = w;
      }
    }
    if (writer && !complete) {
      float* wp = a.ws_out + ps * kDL + 4 * g;
#pragma unroll
      for (int mb = 0; mb < 32; ++mb) {
        const f32x4 w = {o[mb][0] * inv, o[mb][1] * inv, o[mb][2] * inv, o[mb][3] * inv};
        *reinterpret_cast<f32x4*>(wp + mb * 16) = w;
      }
    }
    if (writer && g == 0 && complete && a.lse != nullptr) a.lse[b * H + head] = lse2 * kLn2;
    if (writer && g == 0 && !complete) a.ws_lse[ps] = lse2;
    first_run = false;
  }
}

// ---------------------------------------------------------------------------------------------
// The kernel for more than 64 heads: scores by head block, P.V by DIM block, the two out of phase on a SIMD.
//
// In mla_decode16_kernel every wavefront reads the whole K tile AND the whole V tile from LDS for its 16 heads:
// 68 KB per wavefront and sub-tile, 544 KB per workgroup, against an LDS that delivers 128 bytes per cycle and
// a matrix pipe that needs 2176 cycles for the same sub-tile: the loop runs at the pace of the LDS.  Here the
// second product is cut the other way.  Wavefront w still computes S^T for heads 16w .. 16w+15 (Q^T stays in 72
// registers, K operands from LDS as before) and their softmax, and leaves its P^T block (32 tokens x 16 heads,
// 1 KB, already in the B-operand layout) in LDS.  After the barrier every wavefront multiplies ALL 8 P^T blocks
// with ITS 64 output dims: O^T[dims 64w .. 64w+63, all 128 heads] in the same 128 accumulator registers.  Its
// A operands are 4 KB of V^T instead of 32 KB, its B operands the 8 KB of P^T: 49 KB per wavefront and sub-tile
// instead of 68, 392 KB per workgroup instead of 544.
//
// One barrier per sub-tile.  Between barrier t and barrier t + 1 a wavefront has two independent jobs: P.V of
// sub-tile t (its V^T operands are already in registers, P^T of t is complete) and the scores + softmax of
// sub-tile t + 1 (into the other P^T buffer).  Wavefronts 0-3 take them in this order, wavefronts 4-7 in the
// other: a SIMD holds one of each, so while one keeps the matrix pipe busy with P.V (light on LDS) the other
// streams K operands from LDS for its scores (light on the matrix pipe), and their tile loads go out at different
// times.  A wavefront reads the V^T operands of a sub-tile right after it is done with its scores, so after the
// next barrier nobody needs the sub-tile any more and its ring slot is refilled at once: three slots keep two
// sub-tiles in flight.
//
// The running maximum and sum of a head stay with the wavefront that owns its scores; when a maximum moves
// (rare, the maxima carry kSlack of head room) the owner leaves the factor in LDS and raises a flag, and every
// wavefront rescales that head block's accumulators before it adds the sub-tile.  At the end of a run the
// owners publish 1 / sum and every wavefront writes its dims.
// LDS: ring [3 sub-tiles] | P^T [2][8 blocks] | factors [2][128] | flags [3] | page chunks [2][64] | prefix.
constexpr int kDsRing = 3;
constexpr int kDsPOff = kDsRing * kSubBytes;               // P^T blocks: [2][8][64 lanes][16 bytes]
constexpr int kDsFacOff = kDsPOff + 2 * 8 * 1024;          // [2][128] rescale factors of a sub-tile; [128] 1 / sum at the end
constexpr int kDsFlagOff = kDsFacOff + 2 * kHeadsPerWg16 * 4;  // [3] head blocks whose maximum moved, by sub-tile % 3
constexpr int kDsPageOff = kDsFlagOff + 16;
constexpr int kDsStashOff = kDsPageOff + 2 * kWave * 4;   // V^T operands of wavefronts 4-7 between two windows: [4][4 KB]
constexpr int kDsPrefixOff = kDsStashOff + 4 * 4096;
constexpr int kDsMaxBatch = kMaxBatchMla;
constexpr int kDsLdsBytes = kDsPrefixOff + (kDsMaxBatch + 1) * 4;
static_assert(kDsLdsBytes <= 160 * 1024, "LDS of a CU");

template <typename QT>
__global__ __launch_bounds__(kThreads16) void mla_decode_ds_kernel(MlaArgs a) {
  extern __shared__ __align__(16) char smem[];
  int* prefix = reinterpret_cast<int*>(smem + kDsPrefixOff);
  const int* pagebuf = reinterpret_cast<const int*>(smem + kDsPageOff);
  float* fac = reinterpret_cast<float*>(smem + kDsFacOff);
  int* flags = reinterpret_cast<int*>(smem + kDsFlagOff);
  int* tmp = reinterpret_cast<int*>(smem);  // prologue only

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15;    // MFMA row / column index owned by the lane
  const int g = lane >> 4;      // MFMA k-group of the lane
  const int H = a.n_heads;
  const bool pv_first = wave < 4;  // order of the two jobs between barriers (the SIMD's other wavefront has the other)

  // block id -> (team, head block of 128): members of a team are 8 ids apart (same XCD)
  const int xcd = blockIdx.x & 7;
  const int y = blockIdx.x >> 3;
  const int hb128 = y % a.n_hb;
  const int team = (y / a.n_hb) * 8 + xcd;
  const int head0 = hb128 * kHeadsPerWg16;
  const int n16 = min(8, (H - head0 + 15) >> 4);       // 16-head blocks of this workgroup that hold heads
  const int head = head0 + wave * 16 + c16;            // the head whose scores this lane owns
  const bool head_ok = head < H;
  const bool wave_ok = wave < n16;

  // ---- tile prefix over the batch (every workgroup computes it; no extra launch)
  {
    const int per = (a.batch + kThreads16 - 1) / kThreads16;
    const int lo = min(a.batch, tid * per), hi = min(a.batch, lo + per);
    int local = 0;
    for (int b = lo; b < hi; ++b) local += tiles_of(a.seq_lens[b]);
    tmp[tid] = local;
    __syncthreads();
    if (lo < hi) {
      int excl = 0;
      for (int j = 0; j < tid; ++j) excl += tmp[j];
      if (per == 1) {
        prefix[lo] = excl;
        excl += local;
      } else {
        for (int b = lo; b < hi; ++b) {
          prefix[b] = excl;
          excl += tiles_of(a.seq_lens[b]);
        }
      }
      if (hi == a.batch) prefix[a.batch] = excl;
    }
    __syncthreads();
  }
  const int64_t total = prefix[a.batch];
  if (blockIdx.x == 0)
    for (int i = tid; i <= a.batch; i += kThreads16) a.ws_prefix[i] = prefix[i];
  if (total == 0) return;
  int64_t cur = team_start(team, total, a.n_teams);
  const int64_t end = team_start(team + 1, total, a.n_teams);
  bool first_run = true;
  if (!wave_ok) {  // a head block without heads: its P^T blocks stay zero, P.V multiplies all eight
    *reinterpret_cast<u32x4*>(smem + kDsPOff + wave * 1024 + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(smem + kDsPOff + (8 + wave) * 1024 + lane * 16) = u32x4{0u, 0u, 0u, 0u};
  }

  const u32 lds_base = static_cast<u32>(reinterpret_cast<uintptr_t>(smem));
  const u32 page_lds = __builtin_amdgcn_readfirstlane(lds_base + kDsPageOff);
  // per-lane constants of the operand reads (byte offsets inside a sub-tile), as in mla_decode16_kernel
  const int k_row0 = c16 * kRow16 + ((g ^ ((c16 >> 2) & 1)) * 16);
  const int v_row0 = (4 * g + (c16 >> 2)) * kRow16 + ((((c16 & 3) >> 1) ^ (g & 1)) * 16) + (c16 & 1) * 8 + wave * (4 * 32);
  const u32 lane_off = (lane ^ (wave & 1)) * 16;
  auto lane_again = [&]() {
    u32 x = lane_off;
    asm volatile("" : "+v"(x));
    return static_cast<int>(x >> 4) ^ (wave & 1);
  };

  while (cur < end) {
    int lo = 0, hi = a.batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (prefix[mid] <= cur) lo = mid; else hi = mid;
    }
    const int b = __builtin_amdgcn_readfirstlane(lo);
    const int n_tiles_seq = prefix[b + 1] - prefix[b];
    const int tile0 = static_cast<int>(cur - prefix[b]);
    const int run_tiles = static_cast<int>(min<int64_t>(n_tiles_seq - tile0, end - cur));
    const bool complete = tile0 == 0 && run_tiles == n_tiles_seq;
    cur += run_tiles;
    const int32_t* pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
    const int L = __builtin_amdgcn_readfirstlane(a.seq_lens[b]);
    const int t_begin = tile0 * kTile;
    const int t_end = min(L, (tile0 + run_tiles) * kTile);
    const int n_sub = (t_end - t_begin + kSubTok - 1) / kSubTok;
    const int n_pages = (L + a.block_size - 1) >> a.bs_shift;

    auto issue_chunk = [&](int ck) {
      dma4(pages + min(ck * kWave + lane, n_pages - 1), page_lds + (ck & 1) * kWave * 4);
    };
    int ck_cur = (t_begin >> a.bs_shift) >> 6;
    __syncthreads();  // the previous run no longer reads the ring, the chunks, the factors or the flags
    // the page-table chunks of the run's first sub-tiles travel while the Q rows do
    if (wave == 0) {
      issue_chunk(ck_cur);
      if ((ck_cur + 1) * kWave < n_pages) issue_chunk(ck_cur + 1);
    }
    if (tid < 3) flags[tid] = 0;

    // Q^T operand: lane (head c16, k-group g) keeps dims kk*32 + g*8 .. +8 of every k-step
    u32x4 q[kKSteps32];
    {
      const char* qn = a.q_nope + (static_cast<int64_t>(b) * H + head) * kDL * 2;
      const char* qp = a.q_pe + (static_cast<int64_t>(b) * H + head) * kDR * 2;
#pragma unroll
      for (int kk = 0; kk < kKSteps32; ++kk) {
        u32x4 x = {0u, 0u, 0u, 0u};
        if (head_ok)
          x = kk < kDL / 32 ? ldg16(qn + (kk * 32 + g * 8) * 2) : ldg16(qp + ((kk - kDL / 32) * 32 + g * 8) * 2);
        q[kk] = x;
      }
    }
    // O^T blocks of the wavefront's 64 dims: o[db][hb] = dims 64 wave + 16 db + 4g + r, head 16 hb + c16
    f32x4 o[4][8];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int hb = 0; hb < 8; ++hb) o[db][hb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = 0.0f, l = 0.0f;   // reference maximum (set by the run's first sub-tile) and sum of the lane's head

    auto issue_sub = [&](int sub) {
      const int tok0 = t_begin + sub * kSubTok + wave * 4;
      const u32 slot = lds_base + (sub % kDsRing) * kSubBytes;
      const u32 dst = __builtin_amdgcn_readfirstlane(slot + wave * 4 * kRow16);
      const u32 dst_rope = __builtin_amdgcn_readfirstlane(slot + kRope16Off + wave * 4 * (kDR * 2));
      const uint64_t cache = reinterpret_cast<uint64_t>(a.k_cache);
      const int tb = min(tok0, L - 1);
      const int ck = (tb >> a.bs_shift) >> 6;
      if (ck != ck_cur) {
        ck_cur = ck;
        if (wave == 0 && (ck + 1) * kWave < n_pages) issue_chunk(ck + 1);
      }
      int page = __builtin_amdgcn_readfirstlane(pagebuf[(ck & 1) * kWave + ((tb >> a.bs_shift) & 63)]);
      page = max(0, min(page, a.num_blocks - 1));
      const uint64_t row = cache + static_cast<uint64_t>(page * a.block_size + (tb & (a.block_size - 1))) * kRowBytes;
      const u32 rlo = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(row)));
      const u32 rhi = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(row >> 32)));
      const uint64_t sb = (static_cast<uint64_t>(rhi) << 32) | rlo;
      const int last = __builtin_amdgcn_readfirstlane(L - 1 - tb);
#pragma unroll
      for (int i = 0; i < 4; ++i) dma16_row(sb + static_cast<uint64_t>(min(i, last)) * kRowBytes, lane_off, dst + i * kRow16);
      const int ln = lane_again();
      const int rope_r = (ln >> 3) & 3;
      const u32 rope_off = min(rope_r, last) * kRowBytes + kDL * 2 + (((ln & 7) ^ ((wave & 1) * 4 + rope_r)) * 16);
      if (lane < 4 * kDR * 2 / 16) dma16_row(sb, rope_off, dst_rope);
    };

    // ---- scores and softmax of sub-tile `sub` for the wavefront's 16 heads; P^T block, factor and flag to LDS
    auto scores = [&](int sub) {
      if (!wave_ok) return;
      const char* kb = smem + (sub % kDsRing) * kSubBytes;
      const int ln = lane_again();
      const char* kr = kb + kRope16Off + (ln & 15) * (kDR * 2);
      const int kr_x = (ln >> 4) ^ (ln & 7);
      f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
      const char* ka = kb + k_row0;
      // K operands kDsAhead k-steps ahead of the MFMAs that take them, in an order the scheduler may not change:
      // left to itself it puts every read right in front of its MFMA, and a k-step then costs a whole LDS round
      // trip (about 120 cycles against the 32 of its two MFMAs).
      constexpr int kDsAhead = 2;
      auto k_addr = [&](int kk) -> const char* {
        return kk < kDL / 32 ? ka + kk * 64 : kr + (kk == kDL / 32 ? kr_x : kr_x ^ 4) * 16;
      };
      u32x4 xa[kDsAhead], xb[kDsAhead];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < kDsAhead; ++i) {
        xa[i] = *reinterpret_cast<const u32x4*>(k_addr(i));
        xb[i] = *reinterpret_cast<const u32x4*>(k_addr(i) + 16 * (i < kDL / 32 ? kRow16 : kDR * 2));
      }
#pragma unroll
      for (int kk = 0; kk < kKSteps32; ++kk) {
        __builtin_amdgcn_sched_barrier(0);
        s0 = Mfma<QT>::k32(xa[kk % kDsAhead], q[kk], s0);
        s1 = Mfma<QT>::k32(xb[kk % kDsAhead], q[kk], s1);
        if (kk + kDsAhead < kKSteps32) {
          const int kn = kk + kDsAhead;
          xa[kk % kDsAhead] = *reinterpret_cast<const u32x4*>(k_addr(kn));
          xb[kk % kDsAhead] = *reinterpret_cast<const u32x4*>(k_addr(kn) + 16 * (kn < kDL / 32 ? kRow16 : kDR * 2));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // exponents = scaled score - maximum in one fused multiply-add each; tokens past the end of the context are
      // masked only in the sub-tile that has any (wave-uniform), and the test for a moved maximum is one compare
      // of the block's top exponent
      float sv[8];
      const bool first = sub == 0;   // nothing accumulated yet: the maximum is set, whatever the scores
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sv[r] = __builtin_fmaf(s0[r], a.scale_log2, -m);
        sv[4 + r] = __builtin_fmaf(s1[r], a.scale_log2, -m);
      }
      if (t_begin + (sub + 1) * kSubTok > L) {
        const int tok_base = t_begin + sub * kSubTok + 4 * g;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (tok_base + r >= L) sv[r] = -INFINITY;
          if (tok_base + 16 + r >= L) sv[4 + r] = -INFINITY;
        }
      }
      const float top = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
      if (__builtin_amdgcn_ballot_w64(top > kSlack || first) != 0) {  // rare once the maxima have settled
        const float rise = quad_rows_max(top);   // the head's highest score of the sub-tile, above its maximum
        float alpha = 1.0f;
        if (rise > kSlack || first) {
          alpha = first ? 1.0f : fast_exp2(-rise);
          m += rise;
          l *= alpha;
#pragma unroll
          for (int r = 0; r < 8; ++r) sv[r] -= rise;
        }
        // the factor of every head of the block (1 where the maximum stayed), and the block's flag (the lane's
        // position is recomputed here: kept in registers of their own for this rare path, the addresses get spilled,
        // and a reload from scratch waits for every tile load in flight)
        const int lnx = lane_again();
        if ((lnx >> 4) == 0) fac[(sub & 1) * kHeadsPerWg16 + wave * 16 + (lnx & 15)] = alpha;
        if (lnx == 0) {
          int bit;
          asm volatile("s_lshl_b32 %0, 1, %1" : "=s"(bit) : "s"(wave));
          atomicOr(flags + sub % 3, bit);
        }
      }
      float p[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        p[r] = fast_exp2(sv[r]);
        l += p[r];
      }
      // k-slot g*8 + j of the P.V MFMA <-> token 4g + j of block 0 (j < 4), of block 1 (j >= 4): the lane's
      // eight probabilities are its 16 bytes of the B operand
      const u32x4 pb = {QT::pack(p[0], p[1]), QT::pack(p[2], p[3]), QT::pack(p[4], p[5]), QT::pack(p[6], p[7])};
      *reinterpret_cast<u32x4*>(smem + kDsPOff + ((sub & 1) * 8 + wave) * 1024 + lane * 16) = pb;
    };
    // ---- the V^T operands of sub-tile `sub` for the wavefront's dims, into registers
    auto read_vt = [&](int sub, u32x4 (&vt)[4]) {
      const char* va = smem + (sub % kDsRing) * kSubBytes + v_row0;
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + db * 32));
        const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + 16 * kRow16 + db * 32));
        const s16x8 v = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        vt[db] = __builtin_bit_cast(u32x4, v);
      }
    };
    // ---- O^T[64 dims of the wavefront, all heads] += V^T . P^T of sub-tile `sub` (its P^T blocks are complete)
    auto pv = [&](int sub, const u32x4 (&vt)[4]) {
      // (read as LDS on purpose: a generic volatile pointer becomes a flat load, whose wait drains the tile loads in flight)
      const int moved = __builtin_amdgcn_readfirstlane(*((lds_vint*)(smem + kDsFlagOff) + sub % 3));
      if (moved != 0) {
#pragma unroll
        for (int hb = 0; hb < 8; ++hb) {
          if ((moved >> hb) & 1) {
            const float f = fac[(sub & 1) * kHeadsPerWg16 + hb * 16 + c16];
#pragma unroll
            for (int db = 0; db < 4; ++db) o[db][hb] *= f;
          }
        }
      }
      // all P^T blocks first: their reads return in order, so the MFMAs of a block start as soon as it is there
      // while the later blocks are still on their way (a read per block in front of its MFMAs would put the LDS
      // latency on the path eight times).  Blocks without heads hold zeros.
      const char* pbase = smem + kDsPOff + (sub & 1) * 8 * 1024 + lane * 16;
      u32x4 pb[8];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int hb = 0; hb < 8; ++hb) pb[hb] = *reinterpret_cast<const u32x4*>(pbase + hb * 1024);
#pragma unroll
      for (int hb = 0; hb < 8; ++hb)
#pragma unroll
        for (int db = 0; db < 4; ++db) o[db][hb] = Mfma<QT>::k32(vt[db], pb[hb], o[db][hb]);
      // kPvAhead block reads ahead of the MFMAs that use them (registers allow three blocks in flight)
      constexpr int kPvAhead = 3;
      __builtin_amdgcn_sched_group_barrier(0x100, kPvAhead, 0);
#pragma unroll
      for (int i = 0; i < 8 - kPvAhead; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * kPvAhead, 0);
      __builtin_amdgcn_sched_barrier(0);
    };

    // the chunk loads and the Q loads have landed (one wait for both latencies)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int kk = 0; kk < kKSteps32; ++kk) asm volatile("" : "+v"(q[kk]));
    __syncthreads();
    for (int sub = 0; sub < kDsRing && sub < n_sub; ++sub) issue_sub(sub);
    // sub-tile 0 before the loop
    wait_younger_subs(min(kDsRing - 1, n_sub - 1));
    __syncthreads();
    scores(0);
    if (pv_first) {
      // ---- wavefronts 0-3: P.V of `sub`, then the scores of sub + 1; the V^T operands wait in registers
      u32x4 vt[4];  // V^T operands of the sub-tile whose P.V comes next: dims 64 wave + 16 db .., its 32 tokens
      read_vt(0, vt);
      for (int sub = 0; sub < n_sub; ++sub) {
        // the wavefront's rows of sub-tile sub + 1 have landed (sub + 2 may still be in flight)
        wait_younger_subs(min(kDsRing - 2, n_sub - 2 - sub));
        __syncthreads();  // P^T of `sub` is complete; sub + 1 has landed; nobody reads sub-tile `sub` in LDS any more
        if (tid == 0) flags[(sub + 2) % 3] = 0;   // (last read before this barrier, next raised after the next one)
        if (sub + kDsRing < n_sub) issue_sub(sub + kDsRing);
        pv(sub, vt);
        if (sub + 1 < n_sub) {
          scores(sub + 1);
          read_vt(sub + 1, vt);
        }
      }
    } else {
      // ---- wavefronts 4-7: the scores of sub + 1, then P.V of `sub`.  They park the V^T operands (read while the
      // sub-tile is still in the ring) in a private piece of LDS instead of holding 16 registers across the scores.
      char* stash = smem + kDsStashOff + (wave & 3) * 4096 + lane * 16;
      {
        u32x4 vt[4];
        read_vt(0, vt);
#pragma unroll
        for (int db = 0; db < 4; ++db) *reinterpret_cast<u32x4*>(stash + db * 1024) = vt[db];
      }
      for (int sub = 0; sub < n_sub; ++sub) {
        wait_younger_subs(min(kDsRing - 2, n_sub - 2 - sub));
        __syncthreads();
        const bool more = sub + 1 < n_sub;
        if (more) scores(sub + 1);
        if (sub + kDsRing < n_sub) issue_sub(sub + kDsRing);
        u32x4 vt[4];
#pragma unroll
        for (int db = 0; db < 4; ++db) vt[db] = *reinterpret_cast<const u32x4*>(stash + db * 1024);
        pv(sub, vt);
        if (more) {
          read_vt(sub + 1, vt);
#pragma unroll
          for (int db = 0; db < 4; ++db) *reinterpret_cast<u32x4*>(stash + db * 1024) = vt[db];
        }
      }
    }

    // ---- end of the run: the owners publish 1 / sum per head, every wavefront writes its dims of every head
    const float lsum = quad_rows_sum(l);
    const float lse2 = m + fast_log2(lsum);
    const int64_t ps_base = (static_cast<int64_t>(team) * 2 + (first_run ? 0 : 1)) * H;
    __syncthreads();  // the last sub-tile's factors have been read
    if (wave_ok && g == 0) fac[wave * 16 + c16] = 1.0f / lsum;
    if (wave_ok && head_ok && g == 0) {
      if (complete && a.lse != nullptr) a.lse[b * H + head] = lse2 * kLn2;
      if (!complete) a.ws_lse[ps_base + head] = lse2;
    }
    __syncthreads();
#pragma unroll
    for (int hb = 0; hb < 8; ++hb) {
      const int hd = head0 + hb * 16 + c16;
      if (hb < n16 && hd < H) {
        const float inv = fac[hb * 16 + c16];
        if (complete) {
          char* op = a.out + ((static_cast<int64_t>(b) * H + hd) * kDL + wave * 64 + 4 * g) * 2;
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            const u32x2 w = {QT::pack(o[db][hb][0] * inv, o[db][hb][1] * inv), QT::pack(o[db][hb][2] * inv, o[db][hb][3] * inv)};
            *reinterpret_cast<u32x2*>(op + db * 32) = w;
          }
        } else {
          float* wp = a.ws_out + (ps_base + hd) * kDL + wave * 64 + 4 * g;
#pragma unroll
          for (int db = 0; db < 4; ++db) {
            const f32x4 w = {o[db][hb][0] * inv, o[db][hb][1] * inv, o[db][hb][2] * inv, o[db][hb][3] * inv};
            *reinterpret_cast<f32x4*>(wp + db * 16) = w;
          }
        }
      }
    }
    first_run = false;
  }
}

// ---------------------------------------------------------------------------------------------
// Four wavefronts of 512 registers: the same cut (scores by head block, P.V by dim block), 32 heads per wavefront.
//
// With 16 heads per wavefront every K operand read from LDS (1 KB) feeds ONE 16-cycle MFMA and the eight
// wavefronts read the K tile eight times: 288 KB of the 392 KB a sub-tile moves through an LDS that delivers 128
// bytes per cycle - 3060 cycles against the 2176 of the matrix pipe.  A wavefront that keeps Q^T of 32 heads
// (144 registers) feeds two MFMAs per read, but 144 + 128 accumulators do not fit the 256 registers a wavefront
// has when two share a SIMD.  Here a SIMD holds ONE wavefront with 512 registers: Q^T of its 32 heads, and the
// accumulators of ITS 128 output dims for all 128 heads (256 registers).  The K tile is read four times, a
// sub-tile moves 208 KB through LDS (1630 cycles).
//
// Nothing runs beside the wavefront on its SIMD, so the overlap is written into its one instruction stream:
// between two barriers it computes the scores of sub-tile t + 1 (72 MFMAs, K operands read a few k-steps ahead),
// then P.V of sub-tile t (64 MFMAs) with the softmax arithmetic of sub-tile t + 1 in the shadow of those MFMAs,
// leaves its two P^T blocks in LDS and reads its V^T operands of t + 1.  The sums and maxima of a head stay
// with the wavefront that owns its scores; a moved maximum goes through LDS as in mla_decode_ds_kernel.
// LDS: ring [3 sub-tiles] | P^T [2][8 blocks] | factors [2][128] | flags [3] | page chunks [2][64] | prefix.
// The 256 accumulation registers of mla_decode_w4_kernel hold O^T and nothing else, under fixed names: block
// (db, hb) = a[32 hb + 4 db .. + 3].  They are only touched by the inline assembly below, which names them as
// clobbers so that the compiler counts them and keeps its own values out of them; left to the register
// allocator, a file that is full to the last register is reshuffled at every branch (hundreds of copies and
// spills per sub-tile).  The compiler does not know these are MFMAs: callers leave the wait states themselves.
#define XLLM_W4_MFMA(OP, R0, R1, R2, R3, A, B)                                                        \
  asm volatile(OP " a[" #R0 ":" #R3 "], %0, %1, a[" #R0 ":" #R3 "]" ::"v"(A), "v"(B) : "a" #R0, "a" #R1, "a" #R2, "a" #R3)
#define XLLM_W4_SET(R0, R1, R2, R3, X)                                                                \
  asm volatile("v_accvgpr_write_b32 a" #R0 ", %0\n\tv_accvgpr_write_b32 a" #R1 ", %1\n\t"             \
               "v_accvgpr_write_b32 a" #R2 ", %2\n\tv_accvgpr_write_b32 a" #R3 ", %3" ::"v"((X)[0]),  \
               "v"((X)[1]), "v"((X)[2]), "v"((X)[3])                                                  \
               : "a" #R0, "a" #R1, "a" #R2, "a" #R3)
#define XLLM_W4_GET(R0, R1, R2, R3, X)                                                                \
  asm volatile("v_accvgpr_read_b32 %0, a" #R0 "\n\tv_accvgpr_read_b32 %1, a" #R1 "\n\t"               \
               "v_accvgpr_read_b32 %2, a" #R2 "\n\tv_accvgpr_read_b32 %3, a" #R3                      \
               : "=v"((X)[0]), "=v"((X)[1]), "=v"((X)[2]), "=v"((X)[3]))
#define XLLM_W4_ROW0(F) F(0, 0, 0, 1, 2, 3) F(1, 0, 4, 5, 6, 7) F(2, 0, 8, 9, 10, 11) F(3, 0, 12, 13, 14, 15) F(4, 0, 16, 17, 18, 19) F(5, 0, 20, 21, 22, 23) F(6, 0, 24, 25, 26, 27) F(7, 0, 28, 29, 30, 31)
#define XLLM_W4_ROW1(F) F(0, 1, 32, 33, 34, 35) F(1, 1, 36, 37, 38, 39) F(2, 1, 40, 41, 42, 43) F(3, 1, 44, 45, 46, 47) F(4, 1, 48, 49, 50, 51) F(5, 1, 52, 53, 54, 55) F(6, 1, 56, 57, 58, 59) F(7, 1, 60, 61, 62, 63)
#define XLLM_W4_ROW2(F) F(0, 2, 64, 65, 66, 67) F(1, 2, 68, 69, 70, 71) F(2, 2, 72, 73, 74, 75) F(3, 2, 76, 77, 78, 79) F(4, 2, 80, 81, 82, 83) F(5, 2, 84, 85, 86, 87) F(6, 2, 88, 89, 90, 91) F(7, 2, 92, 93, 94, 95)
#define XLLM_W4_ROW3(F) F(0, 3, 96, 97, 98, 99) F(1, 3, 100, 101, 102, 103) F(2, 3, 104, 105, 106, 107) F(3, 3, 108, 109, 110, 111) F(4, 3, 112, 113, 114, 115) F(5, 3, 116, 117, 118, 119) F(6, 3, 120, 121, 122, 123) F(7, 3, 124, 125, 126, 127)
#define XLLM_W4_ROW4(F) F(0, 4, 128, 129, 130, 131) F(1, 4, 132, 133, 134, 135) F(2, 4, 136, 137, 138, 139) F(3, 4, 140, 141, 142, 143) F(4, 4, 144, 145, 146, 147) F(5, 4, 148, 149, 150, 151) F(6, 4, 152, 153, 154, 155) F(7, 4, 156, 157, 158, 159)
#define XLLM_W4_ROW5(F) F(0, 5, 160, 161, 162, 163) F(1, 5, 164, 165, 166, 167) F(2, 5, 168, 169, 170, 171) F(3, 5, 172, 173, 174, 175) F(4, 5, 176, 177, 178, 179) F(5, 5, 180, 181, 182, 183) F(6, 5, 184, 185, 186, 187) F(7, 5, 188, 189, 190, 191)
#define XLLM_W4_ROW6(F) F(0, 6, 192, 193, 194, 195) F(1, 6, 196, 197, 198, 199) F(2, 6, 200, 201, 202, 203) F(3, 6, 204, 205, 206, 207) F(4, 6, 208, 209, 210, 211) F(5, 6, 212, 213, 214, 215) F(6, 6, 216, 217, 218, 219) F(7, 6, 220, 221, 222, 223)
#define XLLM_W4_ROW7(F) F(0, 7, 224, 225, 226, 227) F(1, 7, 228, 229, 230, 231) F(2, 7, 232, 233, 234, 235) F(3, 7, 236, 237, 238, 239) F(4, 7, 240, 241, 242, 243) F(5, 7, 244, 245, 246, 247) F(6, 7, 248, 249, 250, 251) F(7, 7, 252, 253, 254, 255)
#define XLLM_W4_ALL(F) XLLM_W4_ROW0(F) XLLM_W4_ROW1(F) XLLM_W4_ROW2(F) XLLM_W4_ROW3(F) XLLM_W4_ROW4(F) XLLM_W4_ROW5(F) XLLM_W4_ROW6(F) XLLM_W4_ROW7(F)
constexpr int kW4Threads = 256;

// ---- pieces of a context that spans several teams, and their merge (tiles of mla_decode_w4_kernel) ----------------
// mla_decode_w4_kernel deals the list to min(teams, items) teams, so that no range in the middle of the list is empty:
// the pieces of a context lie with consecutive teams, one piece each.
__device__ __forceinline__ int64_t w4_teams_in_use(const MlaArgs& a, int64_t total) {
  return total < a.n_teams ? total : static_cast<int64_t>(a.n_teams);
}
struct MlaPieces {
  int t_first, t_last;   // teams t_first .. t_last hold the context's pieces
  int slot_first;        // slot of the first team's piece (1 when its range starts in front of the context, with an earlier run)
  int count;             // t_last - t_first + 1
};
// front, stop: the context's share of what the schedule divides, [prefix[b], prefix[b + 1]): run_cost, then its tiles.
// False: the context has no tiles.
__device__ __forceinline__ bool mla_locate_pieces(const MlaArgs& a, int64_t front, int64_t stop, int64_t total, MlaPieces& p) {
  const int64_t first = front + a.run_cost, last = stop - 1;
  if (last < first) return false;
  const int64_t n = w4_teams_in_use(a, total);
  p.t_first = team_of(first, total, n);
  p.t_last = team_of(last, total, n);
  // (a range that starts in front of the context holds the last tile of an earlier one)
  p.slot_first = team_start(p.t_first, total, n) < front ? 1 : 0;
  p.count = p.t_last - p.t_first + 1;
  return true;
}

typedef __attribute__((address_space(3))) const u32x4 lds_cu32x4;
// A 16-byte load / store that other workgroups of the same launch are the counterpart of: at the scope of the whole
// GPU (the L2 of an XCD is not coherent with the other seven inside a launch; these go to the level that all share).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t coherent_window(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);
}
constexpr int kAuxDeviceScope = 16;   // the cache-policy bit that the compiler sets for device-scope atomics (sc1)
__device__ __forceinline__ void coherent_store16(__amdgpu_buffer_rsrc_t w, u32 byte_off, u32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, w, byte_off, 0, kAuxDeviceScope);
}

// One piece joins the running merge of a head's rows: maximum M, weight sum W, O[db] = the lane's four values of dim block
// db.  Piece by piece in the order of the teams, with every product and sum spelled out, so that the result is the same
// bits whoever merges and however the loads are grouped.  x: the lane's 16-bit values of the piece, pairs of dim blocks.
template <typename QT>
__device__ __forceinline__ void mla_merge_piece(float lse, bool on, const u32x4 (&x)[4], float& M, float& W, f32x4 (&O)[8]) {
  const float l = on ? lse : kNegBig;
  const float m_new = fmaxf(M, l);
  const float keep = fast_exp2(M - m_new);
  const float e = on ? fast_exp2(l - m_new) : 0.0f;
  W = __builtin_fmaf(W, keep, e);
#pragma unroll
  for (int dp = 0; dp < 4; ++dp) {
    const u32x4 v = x[dp];
    const float lo[4] = {QT::lo(v[0]), QT::hi(v[0]), QT::lo(v[1]), QT::hi(v[1])};
    const float hi[4] = {QT::lo(v[2]), QT::hi(v[2]), QT::lo(v[3]), QT::hi(v[3])};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      O[2 * dp][r] = __builtin_fmaf(e, lo[r], O[2 * dp][r] * keep);
      O[2 * dp + 1][r] = __builtin_fmaf(e, hi[r], O[2 * dp + 1][r] * keep);
    }
  }
  M = m_new;
}
// The rows of head hd of context b from a finished merge: dims 128 w + 16 db + 4 g .. + 3 (out points at the first).
template <typename QT>
__device__ __forceinline__ void mla_merge_store(const MlaArgs& a, char* out, int b, int hd, bool lse_lane, float M, float W,
                                                const f32x4 (&O)[8]) {
  const float inv = 1.0f / W;
#pragma unroll
  for (int db = 0; db < 8; ++db)
    *reinterpret_cast<u32x2*>(out + db * 32) = u32x2{QT::pack(O[db][0] * inv, O[db][1] * inv), QT::pack(O[db][2] * inv, O[db][3] * inv)};
  if (a.lse != nullptr && lse_lane) a.lse[b * a.n_heads + hd] = (M + fast_log2(W)) * kLn2;
}

// The merge of one (block of 16 heads hb, context b) by 256 threads laid out like the four wavefronts that wrote the
// tiles: wavefront w, lane (head c16, k-group g) owns dims 128 w + 16 db + 4 g .. + 3 of head 16 hb + c16 for the
// eight dim blocks db, and every load instruction reads 1 KB in one piece.  Four teams at a time, their 32 loads per
// lane issued together.
template <typename QT>
__device__ __forceinline__ void mla_merge_tiles(const MlaArgs& a, const MlaPieces& p, int hb, int b, int w, int lane) {
  const int H = a.n_heads;
  const int c16 = lane & 15, g = lane >> 4;
  const int hd = hb * 16 + c16;
  const bool head_ok = hd < H;
  char* out = a.out + ((static_cast<int64_t>(b) * H + hd) * kDL + w * 128 + 4 * g) * 2;
  const int64_t slot_bytes = static_cast<int64_t>(a.slot_heads) * kDL * 2;
  const char* tiles = reinterpret_cast<const char*>(a.ws_out) + (hb * 4 + w) * 4096 + lane * 16;
  float M = kNegBig, W = 0.0f;
  f32x4 O[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) O[db] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  for (int tb = p.t_first; tb <= p.t_last; tb += 4) {
    float lse[4];
    u32x4 x[4][4];   // pairs of dim blocks, 16-bit values
    bool on[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int t = tb + k;
      on[k] = t <= p.t_last && head_ok;
      const int64_t slot = static_cast<int64_t>(t) * 2 + (t == p.t_first ? p.slot_first : 0);
      lse[k] = on[k] ? a.ws_lse[slot * H + hd] : kNegBig;
#pragma unroll
      for (int dp = 0; dp < 4; ++dp)
        x[k][dp] = on[k] ? *reinterpret_cast<const u32x4*>(tiles + slot * slot_bytes + dp * 1024) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (on[k]) mla_merge_piece<QT>(lse[k], true, x[k], M, W, O);   // (on[k] is uniform over the head's lanes)
  }
  if (!head_ok) return;
  mla_merge_store<QT>(a, out, b, hd, w == 0 && g == 0, M, W, O);
}

// The same merge inside mla_decode_w4_kernel, by one wavefront (w of the workgroup's four, each on its own: no barrier in
// here) for the head blocks hb_first, hb_first + hb_step, ... < n16 of the workgroup's 128 heads (block 0 = heads
// 16 hb_base ..).  The pieces were written by other workgroups of the same launch, so they are fetched at the scope of
// the whole GPU, and straight into LDS (no register is in flight): a stream of (head block, piece) units of 4 KB per
// wavefront, four units to a step, the next step's 20 loads in flight while the current one is merged.  region: this
// wavefront's 2 x 17 KB of LDS (4 units + their LSEs, twice).
template <typename QT>
__device__ __forceinline__ void mla_fold_stream(const MlaArgs& a, const MlaPieces& p, int b,
                                                int hb_base, int hb_first, int hb_step, int n16, int w, int lane,
                                                const char* region, u32 region_lds) {
  const int P = p.count;
  const int m = hb_first < n16 ? (n16 - hb_first + hb_step - 1) / hb_step : 0;
  if (m <= 0 || P <= 0) return;
  const int H = a.n_heads;
  const int U = m * P, S = (U + 3) >> 2;
  constexpr int kBuf = 4 * 4096 + 1024;
  const int64_t slot_bytes = static_cast<int64_t>(a.slot_heads) * kDL * 2;
  const int c16 = lane & 15, g = lane >> 4;
  // (the lane's offsets, opaque to the compiler: it would otherwise carry them from the top of the kernel)
  u32 lane16 = static_cast<u32>(lane) * 16u;
  asm volatile("" : "+v"(lane16));
  auto slot_of = [&](int i) -> int64_t { return static_cast<int64_t>(p.t_first + i) * 2 + (i == 0 ? p.slot_first : 0); };
  auto uniform64 = [](uint64_t x) -> uint64_t {
    const u32 lo = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(x)));
    const u32 hi = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(x >> 32)));
    return (static_cast<uint64_t>(hi) << 32) | lo;
  };
  int iu = 0, ihh = 0, ii = 0;   // the unit the next load belongs to: index, head block of the share, piece
  auto issue = [&](int s) {
    const u32 buf = region_lds + static_cast<u32>(s & 1) * kBuf;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      // (past the last unit: that one's again, so that every step is 20 loads and the waits below can count)
      const int hb = hb_base + hb_first + ihh * hb_step;
      const int64_t slot = slot_of(ii);
      const uint64_t src = uniform64(reinterpret_cast<uint64_t>(a.ws_out) + static_cast<uint64_t>(slot * slot_bytes) +
                                     static_cast<uint64_t>((hb * 4 + w) * 4096));
      const u32 dst = __builtin_amdgcn_readfirstlane(buf + k * 4096);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                   "global_load_lds_dwordx4 %1, %2 sc1\n\t"
                   "global_load_lds_dwordx4 %1, %2 offset:1024 sc1\n\t"
                   "global_load_lds_dwordx4 %1, %2 offset:2048 sc1\n\t"
                   "global_load_lds_dwordx4 %1, %2 offset:3072 sc1" ::"s"(dst), "v"(lane16), "s"(src) : "memory");
      const int hd = min(hb * 16 + c16, H - 1);
      const uint64_t lsrc = uniform64(reinterpret_cast<uint64_t>(a.ws_lse) + static_cast<uint64_t>(slot * H) * 4);
      const u32 ldst = __builtin_amdgcn_readfirstlane(buf + 4 * 4096 + k * 256);
      const u32 loff = static_cast<u32>(hd) * 4u;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2 sc1" ::"s"(ldst), "v"(loff), "s"(lsrc) : "memory");
      if (iu + 1 < U) {
        ++iu;
        if (++ii == P) {
          ii = 0;
          ++ihh;
        }
      }
    }
  };
  float M = kNegBig, W = 0.0f;
  f32x4 O[8];
  int hh = 0, i = 0;
  issue(0);
  for (int s = 0; s < S; ++s) {
    if (s + 1 < S) {
      issue(s + 1);
      asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const char* buf = region + (s & 1) * kBuf;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (4 * s + k < U) {
        if (i == 0) {
          M = kNegBig;
          W = 0.0f;
#pragma unroll
          for (int db = 0; db < 8; ++db) O[db] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        const int hb = hb_base + hb_first + hh * hb_step;
        const int hd = hb * 16 + c16;
        const float lse = *(const lds_f32*)(buf + 4 * 4096 + k * 256 + lane * 4);
        u32x4 x[4];
#pragma unroll
        for (int dp = 0; dp < 4; ++dp) x[dp] = *(lds_cu32x4*)(buf + k * 4096 + dp * 1024 + lane * 16);
        mla_merge_piece<QT>(lse, true, x, M, W, O);
        if (++i == P) {
          i = 0;
          ++hh;
          if (hd < H) {
            char* out = a.out + ((static_cast<int64_t>(b) * H + hd) * kDL + w * 128 + 4 * g) * 2;
            mla_merge_store<QT>(a, out, b, hd, w == 0 && g == 0, M, W, O);
          }
        }
      }
    }
    asm volatile("" ::: "memory");   // (the reads of this step's buffer stay in front of the loads that refill it)
  }
}

// Output rows of a context without tokens: zeros, LSE -inf (same layout of the 256 threads).
template <typename QT>
__device__ __forceinline__ void mla_write_empty(const MlaArgs& a, int hb, int b, int w, int lane) {
  const int c16 = lane & 15, g = lane >> 4;
  const int hd = hb * 16 + c16;
  if (hd >= a.n_heads) return;
  char* out = a.out + ((static_cast<int64_t>(b) * a.n_heads + hd) * kDL + w * 128 + 4 * g) * 2;
#pragma unroll
  for (int db = 0; db < 8; ++db) *reinterpret_cast<u32x2*>(out + db * 32) = u32x2{0u, 0u};
  if (a.lse != nullptr && w == 0 && g == 0) a.lse[b * a.n_heads + hd] = -INFINITY;
}
// At the start of a run the Q rows of the 128 heads pass through the ring and the P^T area on their way into the
// registers: latent parts at a pitch of 1040 bytes (16 lanes that read 16 bytes of 16 rows hit 64 different banks),
// then the rope parts.  The small arrays sit behind them.
// What the schedule of mla_decode_w4_kernel divides: sub-tiles.  The loop runs sub-tile by sub-tile, so a range may
// end at any of them, and the workgroups' shares differ by one sub-tile at most instead of one 64-token tile.
constexpr int kW4Item = 32;
constexpr int kW4QRow = kDL * 2 + 16;
constexpr int kW4QRopeOff = kHeadsPerWg16 * kW4QRow;
constexpr int kW4QEnd = kW4QRopeOff + kHeadsPerWg16 * kDR * 2;
constexpr int kW4FacOff = kW4QEnd > kDsPOff + 2 * 8 * 1024 ? kW4QEnd : kDsPOff + 2 * 8 * 1024;   // as kDsFacOff
constexpr int kW4FlagOff = kW4FacOff + 2 * kHeadsPerWg16 * 4;
constexpr int kW4PageOff = kW4FlagOff + 16;
constexpr int kW4PrefixOff = kW4PageOff + 2 * kWave * 4;
constexpr int kW4LdsBytes = kW4PrefixOff + (kMaxBatchMla + 1) * 4 + kMaxBatchMla * 4;   // prefix, then (with a plan) the lengths
constexpr int kW4Loads = 9;   // loads a wavefront sends for a sub-tile: 8 rows and their rope parts
// The fold at the end of a run (mla_fold_stream): every wavefront streams pieces through 2 x 17 KB of the LDS that the
// ring and the Q rows no longer need; the second counter of a context (how many merging workgroups have seen the first
// one full) lies kFoldSeenOff words behind the first.
constexpr int kFoldRegion = 2 * (4 * 4096 + 1024);
constexpr int kFoldSeenOff = kWsMaxWorkers / 2;
static_assert(4 * kFoldRegion <= kW4FacOff, "the fold's LDS lies in front of the factors, flags and the prefix");
static_assert(kW4LdsBytes <= 160 * 1024, "LDS of a CU");

// The prefix over the batch of what mla_decode_w4_kernel's schedule divides (sub-tiles, and run_cost more at the front of
// every context that holds tokens) into prefix[0 .. batch] (LDS), by 256 threads; tmp: 4 words of LDS.
__device__ __forceinline__ void w4_item_prefix(const MlaArgs& a, int* prefix, int* tmp) {
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int per = (a.batch + kW4Threads - 1) / kW4Threads;
  const int lo = min(a.batch, tid * per), hi = min(a.batch, lo + per);
  int local = 0;
  auto span_of = [&](int len) { return len > 0 ? (len + kW4Item - 1) / kW4Item + a.run_cost : 0; };
  for (int b = lo; b < hi; ++b) local += span_of(a.seq_lens[b]);
  // (scan inside the wavefront, then over the wavefronts' totals)
  int incl = local;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int t = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += t;
  }
  if (lane == kWave - 1) tmp[wave] = incl;
  __syncthreads();
  if (lo < hi) {
    int excl = incl - local;
    for (int w = 0; w < wave; ++w) excl += tmp[w];
    if (per == 1) {
      prefix[lo] = excl;
      excl += local;
    } else {
      for (int b = lo; b < hi; ++b) {
        prefix[b] = excl;
        excl += span_of(a.seq_lens[b]);
      }
    }
    if (hi == a.batch) prefix[a.batch] = excl;
  }
  __syncthreads();
}

// The plan of a step for mla_decode_w4_kernel (MlaArgs::plan): the prefix, the lengths it was made with, and for every
// team the 64 page-table entries around the page of its range's first tokens, found as the decode kernel finds them.
// One wavefront per team.
__global__ __launch_bounds__(kW4Threads) void mla_plan_kernel(MlaArgs a, int* plan) {
  extern __shared__ __align__(16) char smem[];
  int* tmp = reinterpret_cast<int*>(smem);
  int* prefix = tmp + 8;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  w4_item_prefix(a, prefix, tmp);
  if (blockIdx.x == 0) {
    for (int i = tid; i <= a.batch; i += kW4Threads) plan[kPlanPrefixOff + i] = prefix[i];
    for (int i = tid; i < a.batch; i += kW4Threads) plan[kPlanLensOff + i] = a.seq_lens[i];
    if (tid == 0) plan[0] = a.plan_sig;
  }
  const int64_t total = prefix[a.batch];
  const int64_t n_use = w4_teams_in_use(a, total);
  const int team = blockIdx.x * (kW4Threads / kWave) + wave;
  if (team >= n_use) return;
  const int64_t cur = team_start(team, total, n_use);
  int lo = 0, hi = a.batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= cur) lo = mid; else hi = mid;
  }
  const int L = a.seq_lens[lo];
  const int tile0 = max(0, static_cast<int>(cur - prefix[lo]) - a.run_cost);
  const int ck = ((tile0 * kW4Item) >> a.bs_shift) >> 6;
  const int n_pages = max(1, (L + a.block_size - 1) >> a.bs_shift);
  const int32_t* pages = a.block_table + static_cast<int64_t>(lo) * a.table_stride;
  plan[kPlanChunksOff + team * kWave + lane] = pages[max(0, min(ck * kWave + lane, n_pages - 1))];
}

template <typename QT>
__global__ __launch_bounds__(kW4Threads) void mla_decode_w4_kernel(MlaArgs a) {
  extern __shared__ __align__(16) char smem[];
  int* prefix = reinterpret_cast<int*>(smem + kW4PrefixOff);
  const int* pagebuf = reinterpret_cast<const int*>(smem + kW4PageOff);
  float* fac = reinterpret_cast<float*>(smem + kW4FacOff);
  int* flags = reinterpret_cast<int*>(smem + kW4FlagOff);
  int* tmp = reinterpret_cast<int*>(smem);  // prologue only

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // heads 32 wave .., dims 128 wave ..
  const int c16 = lane & 15;    // MFMA row / column index owned by the lane
  const int g = lane >> 4;      // MFMA k-group of the lane
  const int H = a.n_heads;

  // block id -> (team, head block of 128): members of a team are 8 ids apart (same XCD: they read the same pages),
  // and so are consecutive teams: those that share a context read its Q rows from HBM once, then from their L2
  // (one XCD after the other they fetch them four times over, 38 MB instead of 9 at the start of a launch of 64
  // contexts)
  const int xcd = blockIdx.x & 7;
  const int y = blockIdx.x >> 3;
  const int hb128 = y % a.n_hb;
  const int team = xcd * (a.n_teams >> 3) + y / a.n_hb;
  const int head0 = hb128 * kHeadsPerWg16;
  const int n16 = min(8, (H - head0 + 15) >> 4);       // 16-head blocks of this workgroup that hold heads

  const u32 lds_base = static_cast<u32>(reinterpret_cast<uintptr_t>(smem));
  const u32 page_lds = __builtin_amdgcn_readfirstlane(lds_base + kW4PageOff);
  // ---- prefix over the batch of what the schedule divides: tiles, and run_cost more at the front of every context.
  // Every workgroup computes it (no extra launch), or takes it from the step's plan: then one trip to memory brings
  // the prefix, the lengths and the page-table entries of the team's first tokens together, where a launch on its own
  // makes three in a row (lengths -> prefix -> the length and the pages of the context its range starts in).
  const bool planned = a.plan != nullptr;
  int* lens_l = prefix + kMaxBatchMla + 1;   // (with a plan) the context lengths
  if (planned) {
    if (wave == 0) {   // (into both chunk buffers: which one the first run reads depends on where it starts)
      dma4(a.plan + kPlanChunksOff + team * kWave + lane, page_lds);
      dma4(a.plan + kPlanChunksOff + team * kWave + lane, page_lds + kWave * 4);
    }
    const int sig = a.plan[0];
    for (int i = tid; i <= a.batch; i += kW4Threads) prefix[i] = a.plan[kPlanPrefixOff + i];
    bool stale = false;
    for (int i = tid; i < a.batch; i += kW4Threads) {
      const int len = a.plan[kPlanLensOff + i];
      lens_l[i] = len;
      if (blockIdx.x == 0) stale |= len != a.seq_lens[i];   // (one workgroup checks for all)
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (sig != a.plan_sig) {   // a plan for another shape: nothing is written
      if (tid == 0) atomicOr(a.ws_status, kStatusPlanMismatch);
      return;
    }
    // a plan made with other lengths (the step before, say): the launch follows it, and its output is invalid
    if (stale) atomicOr(a.ws_status, kStatusPlanMismatch);
    __syncthreads();
  } else {
    w4_item_prefix(a, prefix, tmp);
  }
  const int64_t total = prefix[a.batch];
  if (blockIdx.x == 0 && !planned)   // (the merge kernel of a planned call reads the plan's)
    for (int i = tid; i <= a.batch; i += kW4Threads) a.ws_prefix[i] = prefix[i];
  if (a.fold != 0) {   // no merge kernel follows: the rows of sequences without tokens, which no run ever meets
    for (int b = team; b < a.batch; b += a.n_teams)
      if (prefix[b + 1] == prefix[b])
        for (int hb = 0; hb < n16; ++hb) mla_write_empty<QT>(a, hb128 * 8 + hb, b, wave, lane);
  }
  if (total == 0) return;
  // (min(teams, items) teams take part: no range in the middle of the list is empty)
  const int64_t n_use = w4_teams_in_use(a, total);
  if (team >= n_use) return;
  int64_t cur = team_start(team, total, n_use);
  const int64_t end = team_start(team + 1, total, n_use);
  bool first_run = true;
  bool plan_chunk = planned;   // the chunk buffers hold the plan's entries for the range's first tokens
  // fold: the counter of a piece this workgroup has stored and not yet announced (its stores are known to have landed
  // after the next run's wait for its Q rows, or at the end of the kernel), or -1
  int pending = -1;
  auto announce = [&](int counter) {
    __hip_atomic_fetch_add(a.ws_written + counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  // per-lane constants of the operand reads (byte offsets inside a sub-tile), as in mla_decode16_kernel
  const int k_row0 = c16 * kRow16 + ((g ^ ((c16 >> 2) & 1)) * 16);
  const int v_row0 = (4 * g + (c16 >> 2)) * kRow16 + ((((c16 & 3) >> 1) ^ (g & 1)) * 16) + (c16 & 1) * 8 + wave * (8 * 32);
  const u32 lane_off = lane * 16;
  auto lane_again = [&]() {
    u32 x = lane_off;
    asm volatile("" : "+v"(x));
    return static_cast<int>(x >> 4);
  };

  while (cur < end) {
    int lo = 0, hi = a.batch;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (prefix[mid] <= cur) lo = mid; else hi = mid;
    }
    const int b = __builtin_amdgcn_readfirstlane(lo);
    const int n_tiles_seq = prefix[b + 1] - prefix[b] - a.run_cost;
    const int64_t piece_end = min<int64_t>(prefix[b + 1], end);
    const int tile0 = max(0, static_cast<int>(cur - prefix[b]) - a.run_cost);
    const int run_tiles = max(0, static_cast<int>(piece_end - prefix[b]) - a.run_cost) - tile0;
    const bool complete = tile0 == 0 && run_tiles == n_tiles_seq;
    cur = piece_end;
    if (run_tiles <= 0) {   // (the range ends inside the allowance in front of this context's tiles)
      plan_chunk = false;
      continue;
    }
    const int32_t* pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
    const int L = __builtin_amdgcn_readfirstlane(planned ? lens_l[b] : a.seq_lens[b]);
    const int t_begin = tile0 * kW4Item;
    const int t_end = min(L, (tile0 + run_tiles) * kW4Item);
    const int n_sub = (t_end - t_begin + kSubTok - 1) / kSubTok;
    const int n_pages = (L + a.block_size - 1) >> a.bs_shift;

    auto issue_chunk = [&](int ck) {
      dma4(pages + min(ck * kWave + lane, n_pages - 1), page_lds + (ck & 1) * kWave * 4);
    };
    int ck_cur = (t_begin >> a.bs_shift) >> 6;
    __syncthreads();  // the previous run no longer reads the ring, the chunks, the factors or the flags
    // Store-then-attend: this run holds the context's last token, whose row the step has not stored yet.  Wavefront 0
    // fetches it now, with the loads of the run's prologue, and stores it behind their common wait; the barrier in
    // front of the run's first tile loads comes after the store has completed, so the loads of the last sub-tile find
    // the row in the cache like any other.  (Every workgroup of a team does so for itself, with the same bytes: what it
    // reads later is what it wrote.)
    u32x4 new_latent = {0u, 0u, 0u, 0u}, new_rope = {0u, 0u, 0u, 0u};
    int64_t new_slot = -1;
    const bool stores_row = a.new_rows != nullptr && t_end == L && wave == 0;
    if (stores_row) {   // (slot and row travel together: the slot is looked at when the row is stored)
      new_slot = a.new_slots[b];
      const int ln = lane_again();
      const char* nrow = a.new_rows + static_cast<int64_t>(b) * a.new_row_stride_bytes;
      new_latent = ldg16(nrow + ln * 16);
      if (ln < kDR * 2 / 16) new_rope = ldg16(nrow + kDL * 2 + ln * 16);
    }
    // the page-table chunks of the run's first sub-tiles travel while the Q rows do
    if (wave == 0) {
      if (!plan_chunk) issue_chunk(ck_cur);   // (the plan brought the first run's chunk in with the prefix)
      if ((ck_cur + 1) * kWave < n_pages) issue_chunk(ck_cur + 1);
    }
    plan_chunk = false;
    // (the lane's coordinates, opaque to the compiler: what it can compute from them before the first run it keeps in
    // scratch memory through the loop, and a reload here waits for the chunk loads just issued)
    const int lane_p = lane_again();
    const int c16p = lane_p & 15, gp = lane_p >> 4;
    if (wave == 0 && lane_p < 3) flags[lane_p] = 0;

    // Q^T operands of the two 16-head blocks: lane (head c16, k-group g) keeps dims kk*32 + g*8 .. +8 of every k-step.
    // The rows of the wavefront's 32 heads travel through LDS, 36 loads of 1 KB (whole rows) and then 72 LDS reads per
    // lane.  Gathered from memory by the lanes of that layout the same bytes take 72 loads that touch 16 rows each,
    // and the four wavefronts keep the CU's address unit busy with them for 10 000 cycles.
    u32x4 q[2][kKSteps32];
    {
      const int head_w = head0 + wave * 32;
#pragma unroll 4
      for (int i = 0; i < 32; ++i) {   // (rows of heads beyond the last one: that one's again; their results go nowhere)
        const int head = min(head_w + i, H - 1);
        const uint64_t row = reinterpret_cast<uint64_t>(a.q_nope) + (static_cast<uint64_t>(b) * H + head) * (kDL * 2);
        const u32 dst = __builtin_amdgcn_readfirstlane(lds_base + (wave * 32 + i) * kW4QRow);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane_off), "s"(row) : "memory");
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {    // rope parts, eight heads per load: lane -> head 8 i + lane / 8, piece lane % 8
        const int head = min(head_w + 8 * i + (lane_p >> 3), H - 1);
        const char* src = a.q_pe + (static_cast<int64_t>(b) * H + head) * (kDR * 2) + (lane_p & 7) * 16;
        const u32 dst = __builtin_amdgcn_readfirstlane(lds_base + kW4QRopeOff + (wave * 32 + 8 * i) * (kDR * 2));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src) : "memory");
      }
    }
    // O^T blocks of the wavefront's 128 dims in the accumulation registers: block (db, hb) = dims 128 wave + 16 db
    // + 4g + r, head 16 hb + c16
    {
      const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#define XLLM_W4_ZERO(DB, HB, R0, R1, R2, R3) XLLM_W4_SET(R0, R1, R2, R3, zero);
      XLLM_W4_ALL(XLLM_W4_ZERO)
#undef XLLM_W4_ZERO
    }
    // reference maxima (set by the run's first sub-tile) and sums of heads 32 wave + 16 j + c16 (the lane's tokens)
    float m[2] = {0.0f, 0.0f}, l[2] = {0.0f, 0.0f};

    // ---- the wavefront sends rows 8 wave .. 8 wave + 7 of sub-tile `sub` and their rope parts: nine loads, which
    // the loop spreads over the P.V MFMAs (a wavefront that sends them in one go waits for the address unit to take
    // them, its own and those of the other three wavefronts: about 700 cycles with the matrix pipe idle)
    struct Send {
      uint64_t sb;     // first row of the eight in the cache
      int last;        // rows of the context after that one
      u32 dst, dst_rope;
    };
    // (filled field by field: a struct that is copied as a whole goes through scratch memory, whose loads count
    // on the same counter as the tile loads in flight)
    // in two steps, so that the trip to LDS for the page id passes behind other work: the read ...
    auto issue_prepare_read = [&](int sub) -> int {
      const int tb = min(t_begin + sub * kSubTok + wave * 8, L - 1);   // block_size >= 16: the 8 rows share a page
      const int ck = (tb >> a.bs_shift) >> 6;
      if (ck != ck_cur) {
        ck_cur = ck;
        if (wave == 0 && (ck + 1) * kWave < n_pages) issue_chunk(ck + 1);
      }
      return pagebuf[(ck & 1) * kWave + ((tb >> a.bs_shift) & 63)];
    };
    // ... and the addresses
    auto issue_prepare_finish = [&](int sub, int page_read, Send& sd) {
      const int tb = min(t_begin + sub * kSubTok + wave * 8, L - 1);
      const u32 slot = lds_base + (sub % kDsRing) * kSubBytes;
      sd.dst = __builtin_amdgcn_readfirstlane(slot + wave * 8 * kRow16);
      sd.dst_rope = __builtin_amdgcn_readfirstlane(slot + kRope16Off + wave * 8 * (kDR * 2));
      const uint64_t cache = reinterpret_cast<uint64_t>(a.k_cache);
      int page = __builtin_amdgcn_readfirstlane(page_read);
      page = max(0, min(page, a.num_blocks - 1));
      const uint64_t row = cache + static_cast<uint64_t>(page * a.block_size + (tb & (a.block_size - 1))) * kRowBytes;
      const u32 rlo = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(row)));
      const u32 rhi = static_cast<u32>(__builtin_amdgcn_readfirstlane(static_cast<u32>(row >> 32)));
      sd.sb = (static_cast<uint64_t>(rhi) << 32) | rlo;
      sd.last = __builtin_amdgcn_readfirstlane(L - 1 - tb);
    };
    auto issue_prepare = [&](int sub, Send& sd) { issue_prepare_finish(sub, issue_prepare_read(sub), sd); };
    // (the row's distance from the first one rides in the per-lane offset: one vector add instead of five
    // scalar instructions for a 64-bit base)
    auto issue_row = [&](const Send& sd, int i) {
      dma16_row(sd.sb, (i < 4 ? lane_off : lane_off ^ 16u) + static_cast<u32>(min(i, sd.last)) * kRowBytes, sd.dst + i * kRow16);
    };
    auto issue_rope = [&](const Send& sd) {
      const int ln = lane_again();
      const int rope_r = ln >> 3;   // row of the eight; its rope chunks are XOR-ed with the low 3 bits of the row
      const u32 rope_off = min(rope_r, sd.last) * kRowBytes + kDL * 2 + (((ln & 7) ^ rope_r) * 16);
      dma16_row(sd.sb, rope_off, sd.dst_rope);
    };
    auto issue_sub = [&](int sub) {
      Send sd;
      issue_prepare(sub, sd);
#pragma unroll
      for (int i = 0; i < 8; ++i) issue_row(sd, i);
      issue_rope(sd);
    };
    // all but the youngest `subs` sub-tiles this wavefront has sent are in LDS
    auto wait_sent = [&](int subs) {
      static_assert(kW4Loads == 9, "the immediates below are multiples of the loads per sub-tile");
      if (subs <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else if (subs == 1) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
    };

    // ---- S^T of sub-tile `sub` for the wavefront's 32 heads: s[j][tb] = tokens 16 tb + 4g + r, head 16 j + c16
    constexpr int kAheadW = 3;
    // the K operands of the first kAheadW k-steps of sub-tile `sub` (its rows have landed): sent for before the first
    // half of P.V, so that the scores start on operands that are there
    auto scores_begin = [&](int sub, u32x4 (&xa)[kAheadW], u32x4 (&xb)[kAheadW]) {
      const char* ka = smem + (sub % kDsRing) * kSubBytes + k_row0;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < kAheadW; ++i) {   // (kAheadW <= 16: latent k-steps)
        xa[i] = *reinterpret_cast<const u32x4*>(ka + i * 64);
        xb[i] = *reinterpret_cast<const u32x4*>(ka + i * 64 + 16 * kRow16);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    auto scores = [&](int sub, f32x4 (&s)[2][2], u32x4 (&xa)[kAheadW], u32x4 (&xb)[kAheadW]) {
      const char* kb = smem + (sub % kDsRing) * kSubBytes;
      const int ln = lane_again();
      const char* kr = kb + kRope16Off + (ln & 15) * (kDR * 2);
      const int kr_x = (ln >> 4) ^ (ln & 7);
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) s[j][tb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      const char* ka = kb + k_row0;
      // K operands kAheadW k-steps ahead of the MFMAs that take them, in an order the scheduler may not change
      auto k_addr = [&](int kk) -> const char* {
        return kk < kDL / 32 ? ka + kk * 64 : kr + (kk == kDL / 32 ? kr_x : kr_x ^ 4) * 16;
      };
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < kKSteps32; ++kk) {
        __builtin_amdgcn_sched_barrier(0);
        Mfma<QT>::k32_v(xa[kk % kAheadW], q[0][kk], s[0][0]);
        Mfma<QT>::k32_v(xa[kk % kAheadW], q[1][kk], s[1][0]);
        Mfma<QT>::k32_v(xb[kk % kAheadW], q[0][kk], s[0][1]);
        Mfma<QT>::k32_v(xb[kk % kAheadW], q[1][kk], s[1][1]);
        if (kk + kAheadW < kKSteps32) {
          const int kn = kk + kAheadW;
          xa[kk % kAheadW] = *reinterpret_cast<const u32x4*>(k_addr(kn));
          xb[kk % kAheadW] = *reinterpret_cast<const u32x4*>(k_addr(kn) + 16 * (kn < kDL / 32 ? kRow16 : kDR * 2));
        }
      }
      mfma_result_nops();
      __builtin_amdgcn_sched_barrier(0);
    };
    // ---- exponents sv = scaled score - maximum of sub-tile `sub`; masks (last sub-tile of a context only), moved
    // maxima (rare), their factors and flag
    auto exponents_rest = [&](int sub, float (&sv)[2][8]) {
      const bool first = sub == 0;   // nothing accumulated yet: the maxima are set, whatever the scores
      bool over = first;
      float top[2];
      if (t_begin + (sub + 1) * kSubTok > L) {   // (wave-uniform) tokens past the end of the context
        const int tok_base = t_begin + sub * kSubTok + 4 * g;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if (tok_base + r >= L) sv[j][r] = -INFINITY;
            if (tok_base + 16 + r >= L) sv[j][4 + r] = -INFINITY;
          }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        top[j] = fmaxf(fmaxf(fmaxf(sv[j][0], sv[j][1]), fmaxf(sv[j][2], sv[j][3])),
                       fmaxf(fmaxf(sv[j][4], sv[j][5]), fmaxf(sv[j][6], sv[j][7])));
        over |= top[j] > kSlack;
      }
      if (__builtin_amdgcn_ballot_w64(over) != 0) {  // rare once the maxima have settled
        const int lnx = lane_again();
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const float rise = quad_rows_max(top[j]);   // the head's highest score of the sub-tile, above its maximum
          float alpha = 1.0f;
          if (rise > kSlack || first) {
            alpha = first ? 1.0f : fast_exp2(-rise);
            m[j] += rise;
            l[j] *= alpha;
#pragma unroll
            for (int r = 0; r < 8; ++r) sv[j][r] -= rise;
          }
          // the factor of every head of the block (1 where the maximum stayed)
          if ((lnx >> 4) == 0) fac[(sub & 1) * kHeadsPerWg16 + wave * 32 + j * 16 + (lnx & 15)] = alpha;
        }
        if (lnx == 0) {
          int bits;
          asm volatile("s_lshl_b32 %0, 3, %1" : "=s"(bits) : "s"(wave * 2));
          atomicOr(flags + sub % 3, bits);
        }
      }
    };
    auto exponents = [&](int sub, const f32x4 (&s)[2][2], float (&sv)[2][8]) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sv[j][r] = __builtin_fmaf(s[j][0][r], a.scale_log2, -m[j]);
          sv[j][4 + r] = __builtin_fmaf(s[j][1][r], a.scale_log2, -m[j]);
        }
      }
      exponents_rest(sub, sv);
    };
    // ---- probabilities of sub-tile `sub` from its exponents; the wavefront's two P^T blocks to LDS
    auto probabilities = [&](int sub, const float (&sv)[2][8]) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        float p[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          p[r] = fast_exp2(sv[j][r]);
          l[j] += p[r];
        }
        // k-slot g*8 + i of the P.V MFMA <-> token 4g + i of block 0 (i < 4), of block 1 (i >= 4): the lane's
        // eight probabilities are its 16 bytes of the B operand
        const u32x4 pb = {QT::pack(p[0], p[1]), QT::pack(p[2], p[3]), QT::pack(p[4], p[5]), QT::pack(p[6], p[7])};
        *reinterpret_cast<u32x4*>(smem + kDsPOff + ((sub & 1) * 8 + wave * 2 + j) * 1024 + lane * 16) = pb;
      }
    };
    // ---- the V^T operands of sub-tile `sub` for the wavefront's dims, into registers
    auto read_vt = [&](int sub, u32x4 (&vt)[8], int db0 = 0, int db1 = 8) {
      const char* va = smem + (sub % kDsRing) * kSubBytes + v_row0;
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        if (db < db0 || db >= db1) continue;
        const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + db * 32));
        const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(va + 16 * kRow16 + db * 32));
        const s16x8 v = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        vt[db] = __builtin_bit_cast(u32x4, v);
      }
    };
    // ---- the accumulators follow the maxima that moved in sub-tile `sub`
    auto rescale = [&](int sub, int moved) {
      if (moved != 0) {
        mfma_result_nops();
#define XLLM_W4_SCALE(DB, HB, R0, R1, R2, R3) \
  {                                           \
    f32x4 t;                                  \
    XLLM_W4_GET(R0, R1, R2, R3, t);           \
    t *= f;                                   \
    XLLM_W4_SET(R0, R1, R2, R3, t);           \
  }
#define XLLM_W4_SCALE_ROW(HB, ROW)                                            \
  if ((moved >> HB) & 1) {                                                    \
    const float f = fac[(sub & 1) * kHeadsPerWg16 + HB * 16 + c16];           \
    ROW(XLLM_W4_SCALE)                                                        \
  }
        XLLM_W4_SCALE_ROW(0, XLLM_W4_ROW0)
        XLLM_W4_SCALE_ROW(1, XLLM_W4_ROW1)
        XLLM_W4_SCALE_ROW(2, XLLM_W4_ROW2)
        XLLM_W4_SCALE_ROW(3, XLLM_W4_ROW3)
        XLLM_W4_SCALE_ROW(4, XLLM_W4_ROW4)
        XLLM_W4_SCALE_ROW(5, XLLM_W4_ROW5)
        XLLM_W4_SCALE_ROW(6, XLLM_W4_ROW6)
        XLLM_W4_SCALE_ROW(7, XLLM_W4_ROW7)
#undef XLLM_W4_SCALE_ROW
#undef XLLM_W4_SCALE
        asm volatile("s_nop 7" ::: "memory");
      }
    };
    // ---- O^T[128 dims of the wavefront, all heads] += V^T . P^T of sub-tile `sub` (its P^T blocks are complete)
    // (the first two P^T blocks are on their way when it is called: pv_begin)
    auto pv_begin = [&](int sub, u32x4 (&pb)[2]) -> int {
      const char* pbase = smem + kDsPOff + (sub & 1) * 8 * 1024 + lane * 16;
      __builtin_amdgcn_sched_barrier(0);
      pb[0] = *reinterpret_cast<const u32x4*>(pbase);
      pb[1] = *reinterpret_cast<const u32x4*>(pbase + 1024);
      __builtin_amdgcn_sched_barrier(0);
      // the head blocks whose maxima moved in this sub-tile: read behind the two blocks, so that one trip to LDS
      // covers all three (read as LDS on purpose: a generic volatile pointer becomes a flat load, whose wait drains
      // the tile loads in flight)
      return __builtin_amdgcn_readfirstlane(*((lds_vint*)(smem + kW4FlagOff) + sub % 3));
    };
    // Rows FIRST .. LAST - 1 (head blocks) of one half of the wavefront's dims (HALF 0: dim blocks 0-3, with the
    // tile loads of a later sub-tile, one per row; HALF 1: dim blocks 4-7).  MODE says what rides in the shadow of
    // the MFMAs of half 1, a few vector instructions behind each of them (a wavefront issues an MFMA every 16
    // cycles and has 12 of them for other instructions): 1 = exponents and block maxima of the scores in `sc`
    // (rows 0-2), 2 = exponentials, sums and the two P^T blocks (rows 3-7), 0 = nothing.
    auto pv_rows = [&](auto half_tag, auto mode_tag, auto first_tag, auto last_tag, auto sends_tag, int sub,
                       const u32x4 (&vt)[8], const Send& sd, u32x4 (&pb)[2], const f32x4 (&sc)[2][2], float (&sv)[2][8],
                       float (&top)[2], bool prep = false, int page_read = 0, Send* sd_next = nullptr) {
      constexpr int HALF = decltype(half_tag)::value, MODE = decltype(mode_tag)::value;
      constexpr int FIRST = decltype(first_tag)::value, LAST = decltype(last_tag)::value;
      constexpr bool sends = decltype(sends_tag)::value;
      const char* pbase = smem + kDsPOff + (sub & 1) * 8 * 1024 + lane * 16;
      auto hook = [&](auto n_tag) {
        constexpr int n = decltype(n_tag)::value;   // MFMA number within the half: 4 * row + dim block
        if constexpr (HALF == 0 && n == 22) {   // the addresses of the loads that the next sub-tile's P.V sends (scalar work)
          if (prep) issue_prepare_finish(sub + 1 + kDsRing, page_read, *sd_next);
        }
        if constexpr (MODE == 1 && n >= 2 && n < 10) {
          constexpr int k = n - 2, v0 = 2 * k, v1 = 2 * k + 1, j = v0 >> 3, r0 = v0 & 7, r1 = v1 & 7;
          sv[j][r0] = __builtin_fmaf(sc[j][r0 >> 2][r0 & 3], a.scale_log2, -m[j]);
          sv[j][r1] = __builtin_fmaf(sc[j][r1 >> 2][r1 & 3], a.scale_log2, -m[j]);
          const float t = fmaxf(sv[j][r0], sv[j][r1]);
          top[j] = (k & 3) == 0 ? t : fmaxf(top[j], t);
        }
        if constexpr (MODE == 2 && n >= 12 && n < 28) {
          constexpr int v = n - 12, j = v >> 3, r = v & 7;
          sv[j][r] = fast_exp2(sv[j][r]);
          l[j] += sv[j][r];
        }
        if constexpr (MODE == 2 && (n == 21 || n == 29)) {
          // k-slot g*8 + i of the P.V MFMA <-> token 4g + i of block 0 (i < 4), of block 1 (i >= 4): the lane's
          // eight probabilities are its 16 bytes of the B operand
          constexpr int j = n == 21 ? 0 : 1;
          const u32x4 w = {QT::pack(sv[j][0], sv[j][1]), QT::pack(sv[j][2], sv[j][3]), QT::pack(sv[j][4], sv[j][5]),
                           QT::pack(sv[j][6], sv[j][7])};
          *reinterpret_cast<u32x4*>(smem + kDsPOff + (((sub + 1) & 1) * 8 + wave * 2 + j) * 1024 + lane * 16) = w;
        }
        __builtin_amdgcn_sched_barrier(0);
      };
#define XLLM_W4_PV_BF16(DB, HB, R0, R1, R2, R3)                                                 \
  if constexpr ((DB >> 2) == HALF) {                                                            \
    XLLM_W4_MFMA("v_mfma_f32_16x16x32_bf16", R0, R1, R2, R3, vt[DB], pb[HB & 1]);               \
    hook(std::integral_constant<int, HB * 4 + (DB & 3)>{});                                     \
  }
#define XLLM_W4_PV_F16(DB, HB, R0, R1, R2, R3)                                                  \
  if constexpr ((DB >> 2) == HALF) {                                                            \
    XLLM_W4_MFMA("v_mfma_f32_16x16x32_f16", R0, R1, R2, R3, vt[DB], pb[HB & 1]);                \
    hook(std::integral_constant<int, HB * 4 + (DB & 3)>{});                                     \
  }
#define XLLM_W4_PV_ROW(HB, ROW)                                                                 \
  if constexpr (HB >= FIRST && HB < LAST) {                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                          \
    if constexpr (QT::kIsBf16) { ROW(XLLM_W4_PV_BF16) } else { ROW(XLLM_W4_PV_F16) }            \
    if (HB + 2 < 8) pb[HB & 1] = *reinterpret_cast<const u32x4*>(pbase + (HB + 2) * 1024);      \
    if constexpr (sends) { /* the loads of a later sub-tile, one per row (spread over both halves they cost more: the */ \
      issue_row(sd, HB);   /* second half is dense with the softmax arithmetic) */              \
      if (HB == 3) issue_rope(sd);                                                              \
    }                                                                                           \
  }
      XLLM_W4_PV_ROW(0, XLLM_W4_ROW0)
      XLLM_W4_PV_ROW(1, XLLM_W4_ROW1)
      XLLM_W4_PV_ROW(2, XLLM_W4_ROW2)
      XLLM_W4_PV_ROW(3, XLLM_W4_ROW3)
      XLLM_W4_PV_ROW(4, XLLM_W4_ROW4)
      XLLM_W4_PV_ROW(5, XLLM_W4_ROW5)
      XLLM_W4_PV_ROW(6, XLLM_W4_ROW6)
      XLLM_W4_PV_ROW(7, XLLM_W4_ROW7)
#undef XLLM_W4_PV_ROW
#undef XLLM_W4_PV_F16
#undef XLLM_W4_PV_BF16
      __builtin_amdgcn_sched_barrier(0);
    };
    // the first two P^T blocks of `sub` again, for the second half of its P.V
    auto pv_again = [&](int sub, u32x4 (&pb)[2]) {
      const char* pbase = smem + kDsPOff + (sub & 1) * 8 * 1024 + lane * 16;
      pb[0] = *reinterpret_cast<const u32x4*>(pbase);
      pb[1] = *reinterpret_cast<const u32x4*>(pbase + 1024);
    };

    // the chunk loads and the Q rows have landed (one wait for both latencies); the wavefront reads the rows it sent
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (stores_row && new_slot >= 0 && new_slot < a.n_slots) {   // (wavefront 0 of a run that ends its context)
      const int ln = lane_again();
      char* dst = a.k_cache_w + new_slot * kRowBytes;
      stg16(dst + ln * 16, new_latent);
      if (ln < kDR * 2 / 16) stg16(dst + kDL * 2 + ln * 16, new_rope);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const char* qrow = smem + (wave * 32 + j * 16 + c16p) * kW4QRow + gp * 16;
      const char* qrope = smem + kW4QRopeOff + (wave * 32 + j * 16 + c16p) * (kDR * 2) + gp * 16;
#pragma unroll
      for (int kk = 0; kk < kKSteps32; ++kk)
        q[j][kk] = kk < kDL / 32 ? *reinterpret_cast<const u32x4*>(qrow + kk * 64)
                                 : *reinterpret_cast<const u32x4*>(qrope + (kk - kDL / 32) * 64);
    }
    if (stores_row) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the step's row is in the cache
    __syncthreads();   // (the ring is free for the first sub-tiles)
    if (pending >= 0) {   // every wavefront's stores of the piece before have landed (the wait above), and all are past it
      if (tid == 0) announce(pending);
      pending = -1;
    }
    for (int sub = 0; sub < kDsRing && sub < n_sub; ++sub) issue_sub(sub);
    wait_sent(min(kDsRing - 1, n_sub - 1));
    __syncthreads();
    u32x4 vt[8];  // V^T operands of the sub-tile whose P.V comes next: dims 128 wave + 16 db .., its 32 tokens
    {
      f32x4 s[2][2];
      float sv[2][8];
      u32x4 xa[kAheadW], xb[kAheadW];
      scores_begin(0, xa, xb);
      scores(0, s, xa, xb);
      exponents(0, s, sv);
      probabilities(0, sv);
      read_vt(0, vt);
    }
    bool sends = kDsRing < n_sub;
    Send sd;
    sd.sb = 0;
    sd.last = 0;
    sd.dst = sd.dst_rope = 0;
    if (sends) issue_prepare(kDsRing, sd);
    for (int sub = 0; sub < n_sub; ++sub) {
      const bool more = sub + 1 < n_sub;
      // the wavefront's rows of sub-tile sub + 1 have landed (sub + 2 may still be in flight)
      wait_sent(min(kDsRing - 2, n_sub - 2 - sub));
      __syncthreads();  // P^T of `sub` is complete; sub + 1 has landed; nobody reads sub-tile `sub` in LDS any more
      if (tid == 0) flags[(sub + 2) % 3] = 0;   // (last read before this barrier, next raised after the next one)
      using I0 = std::integral_constant<int, 0>;
      using I1 = std::integral_constant<int, 1>;
      using I2 = std::integral_constant<int, 2>;
      using I3 = std::integral_constant<int, 3>;
      using I8 = std::integral_constant<int, 8>;
      u32x4 pb[2];
      f32x4 sc[2][2];
      float sv[2][8];
      float top[2] = {0.0f, 0.0f};
      // the page id behind the addresses of the loads that the NEXT sub-tile's P.V sends, and the first K operands of
      // the scores: their trips to LDS pass behind the first half of P.V
      const bool sends_next = more && sub + 1 + kDsRing < n_sub;
      int page_read = 0;
      if (sends_next) page_read = issue_prepare_read(sub + 1 + kDsRing);
      Send sd_next;
      sd_next.sb = 0;
      sd_next.last = 0;
      sd_next.dst = sd_next.dst_rope = 0;
      const int moved = pv_begin(sub, pb);
      rescale(sub, moved);
      // ---- first half of P.V of `sub` (dim blocks 0-3), with the loads of sub + 3
      if (sends) pv_rows(I0{}, I0{}, I0{}, I8{}, std::true_type{}, sub, vt, sd, pb, sc, sv, top, sends_next, page_read, &sd_next);
      else pv_rows(I0{}, I0{}, I0{}, I8{}, std::false_type{}, sub, vt, sd, pb, sc, sv, top, sends_next, page_read, &sd_next);
      if (more) {
        u32x4 xa[kAheadW], xb[kAheadW];
        scores_begin(sub + 1, xa, xb);
        scores(sub + 1, sc, xa, xb);
        // ---- second half of P.V of `sub` (dim blocks 4-7) with the softmax of sub + 1 in the shadow of its MFMAs
        pv_again(sub, pb);
        pv_rows(I1{}, I1{}, I0{}, I3{}, std::false_type{}, sub, vt, sd, pb, sc, sv, top);
        const bool plain = t_begin + (sub + 2) * kSubTok <= L && !(top[0] > kSlack || top[1] > kSlack);
        if (__builtin_amdgcn_ballot_w64(!plain) == 0) {
          pv_rows(I1{}, I2{}, I3{}, I8{}, std::false_type{}, sub, vt, sd, pb, sc, sv, top);
        } else {   // a maximum moves, or the sub-tile is the ragged end of a context: one thing after the other
          pv_rows(I1{}, I0{}, I3{}, I8{}, std::false_type{}, sub, vt, sd, pb, sc, sv, top);
          exponents_rest(sub + 1, sv);
          probabilities(sub + 1, sv);
        }
        read_vt(sub + 1, vt);
      } else {   // (the last sub-tile of a run sends nothing: sub + 3 is past its end)
        pv_again(sub, pb);
        pv_rows(I1{}, I0{}, I0{}, I8{}, std::false_type{}, sub, vt, sd, pb, sc, sv, top);
      }
      sends = sends_next;
      sd.sb = sd_next.sb;
      sd.last = sd_next.last;
      sd.dst = sd_next.dst;
      sd.dst_rope = sd_next.dst_rope;
    }

    // ---- end of the run: the owners publish 1 / sum per head, every wavefront writes its dims of every head
    const float lsum0 = quad_rows_sum(l[0]), lsum1 = quad_rows_sum(l[1]);
    const int64_t slot_id = static_cast<int64_t>(team) * 2 + (first_run ? 0 : 1);
    const int64_t ps_base = slot_id * H;
    // fold: a piece goes to memory at the scope of the whole GPU, for the workgroups of this launch that merge it
    const bool shared = a.fold != 0 && !complete;
    // The lane's coordinates once more, opaque to the compiler.  Address arithmetic of the epilogue that can be done
    // before the loop is done there otherwise, and carried through the loop in scratch memory: every reload then waits
    // for all the stores issued before it (one counter covers loads and stores), a round trip to memory per row.
    const int ln = lane_again();
    const int c16e = ln & 15, ge = ln >> 4;
    mfma_result_nops();
    __syncthreads();  // the last sub-tile's factors have been read
    if (ge == 0) {
      fac[wave * 32 + c16e] = 1.0f / lsum0;
      fac[wave * 32 + 16 + c16e] = 1.0f / lsum1;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int hd = head0 + wave * 32 + j * 16 + c16e;
        if (hd < H) {
          const float lse2 = m[j] + fast_log2(j == 0 ? lsum0 : lsum1);
          if (complete && a.lse != nullptr) a.lse[b * H + hd] = lse2 * kLn2;
          if (!complete && !shared) a.ws_lse[ps_base + hd] = lse2;
          if (shared) __hip_atomic_store(a.ws_lse + ps_base + hd, lse2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    __syncthreads();
    // Output rows of a whole context go out head by head (MODE 0).  Partial rows go out as the tiles they are in the
    // registers, [16-head block][wavefront][pair of dim blocks][lane][2 x 4 values]: every store instruction then
    // writes 1 KB in one piece (MODE 1; MODE 2: the same at the scope of the whole GPU).  Head by head it writes sixteen
    // pieces of 64 bytes, and the burst of partial rows that ends a launch takes twice as long to issue (it is bound by
    // the number of write requests, not by their bytes).  A partial row is normalised (a convex combination of V rows,
    // like the output), so it is stored in the output's own 16-bit type: half the stores here, half the bytes for the
    // merge, whose time is reading them; the LSEs stay fp32.
#define XLLM_W4_OUT(DB, HB, R0, R1, R2, R3)                                                          \
  {                                                                                                  \
    f32x4 t;                                                                                         \
    XLLM_W4_GET(R0, R1, R2, R3, t);                                                                  \
    t *= inv;                                                                                        \
    const u32x2 w = {QT::pack(t[0], t[1]), QT::pack(t[2], t[3])};                                    \
    if (MODE == 0) {                                                                                 \
      *reinterpret_cast<u32x2*>(dst + DB * 32) = w;                                                  \
    } else if ((DB & 1) == 0) {                                                                      \
      held = w;                                                                                      \
    } else if (MODE == 1) {                                                                          \
      *reinterpret_cast<u32x4*>(dst + (DB >> 1) * 1024) = u32x4{held[0], held[1], w[0], w[1]};       \
    } else {                                                                                         \
      coherent_store16(window, voff + (HB * 4 + wave) * 4096 + (DB >> 1) * 1024,                     \
                       u32x4{held[0], held[1], w[0], w[1]});                                         \
    }                                                                                                \
  }
#define XLLM_W4_OUT_ROW(HB, ROW)                                                                     \
  {                                                                                                  \
    const int hd = head0 + HB * 16 + c16e;                                                           \
    if (HB < n16 && hd < H) {                                                                        \
      const float inv = fac[HB * 16 + c16e];                                                         \
      u32x2 held = {0u, 0u};                                                                         \
      char* dst = MODE == 0 ? a.out + ((static_cast<int64_t>(b) * H + hd) * kDL + wave * 128 + 4 * ge) * 2 \
                            : tiles + (HB * 4 + wave) * 4096;                                        \
      ROW(XLLM_W4_OUT)                                                                               \
    }                                                                                                \
  }
#define XLLM_W4_OUT_ROWS                                                                             \
  XLLM_W4_OUT_ROW(0, XLLM_W4_ROW0)                                                                   \
  XLLM_W4_OUT_ROW(1, XLLM_W4_ROW1)                                                                   \
  XLLM_W4_OUT_ROW(2, XLLM_W4_ROW2)                                                                   \
  XLLM_W4_OUT_ROW(3, XLLM_W4_ROW3)                                                                   \
  XLLM_W4_OUT_ROW(4, XLLM_W4_ROW4)                                                                   \
  XLLM_W4_OUT_ROW(5, XLLM_W4_ROW5)                                                                   \
  XLLM_W4_OUT_ROW(6, XLLM_W4_ROW6)                                                                   \
  XLLM_W4_OUT_ROW(7, XLLM_W4_ROW7)
    // (16-head blocks of this workgroup's 128 heads: block hb128 * 8 + HB of the slot)
    const int64_t tile_base = (slot_id * a.slot_heads + head0) * (kDL * 2) + ln * 16;
    char* tiles = reinterpret_cast<char*>(a.ws_out) + tile_base;
    const u32 voff = static_cast<u32>(tile_base);
    const __amdgpu_buffer_rsrc_t window = coherent_window(a.ws_out);
    if (complete) {
      constexpr int MODE = 0;
      XLLM_W4_OUT_ROWS
    } else if (!shared) {
      constexpr int MODE = 1;
      XLLM_W4_OUT_ROWS
    } else {
      constexpr int MODE = 2;
      XLLM_W4_OUT_ROWS
    }
#undef XLLM_W4_OUT_ROWS
#undef XLLM_W4_OUT_ROW
#undef XLLM_W4_OUT
    if (shared) {
      // The pieces of the context lie with teams t_first .. t_last; one counter per context (kept with its first team)
      // counts them as they reach memory.  The workgroups whose piece ends their range (all but the one that holds the
      // context's end, which has another run to go) wait for the count and merge the head blocks between them, team j
      // of the nf taking blocks j, j + nf, ...: nobody waits before it has announced everything it wrote itself, so
      // every wait ends.  The last of the nf to have seen the full count clears it for the next launch.
      MlaPieces pc;
      mla_locate_pieces(a, prefix[b], prefix[b + 1], total, pc);
      const int counter = pc.t_first * a.n_hb + hb128;
      const int nf = pc.t_last - pc.t_first;
      const int jf = team - pc.t_first;
      if (team == pc.t_last) {
        pending = counter;   // announced once its stores have landed: after the next run's wait, or at the kernel's end
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();   // every wavefront's stores have landed
        if (tid == 0) {
          if (pending >= 0) announce(pending);
          announce(counter);
          const unsigned need = static_cast<unsigned>(pc.count);
          bool ok = a.wait_spins > 0;
          for (int spins = a.wait_spins; ok; --spins) {
            if (__hip_atomic_load(a.ws_written + counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= need) break;
            if (spins <= 1) ok = false;
            __builtin_amdgcn_s_sleep(16);
          }
          if (!ok) atomicOr(a.ws_status, kStatusWaitGaveUp);
          flags[3] = ok ? 1 : 0;
        }
        pending = -1;
        __syncthreads();
        if (flags[3] != 0) {
          mla_fold_stream<QT>(a, pc, b, hb128 * 8, jf, nf, n16, wave, lane_again(),
                              smem + wave * kFoldRegion, lds_base + wave * kFoldRegion);
          __syncthreads();   // every wavefront has read what it needs of the pieces
          if (tid == 0) {
            const unsigned seen = atomicInc(a.ws_written + kFoldSeenOff + counter, static_cast<unsigned>(nf - 1));
            if (seen == static_cast<unsigned>(nf - 1))
              __hip_atomic_store(a.ws_written + counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
    }
    first_run = false;
  }
  if (pending >= 0) {   // a piece stored by this workgroup's last run that it does not merge itself
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) announce(pending);
  }
}

// Merge of the partials of contexts that span several teams; also writes the output of
// empty sequences.  One workgroup per (head, sequence).
template <typename QT>
__global__ __launch_bounds__(128) void mla_merge_kernel(MlaArgs a) {
  // One workgroup per (head, sequence); thread t owns dims 4t .. 4t+3, read from the fp32 partials
  // with 16-byte loads.  Two dependent round trips to memory: the tile prefix, then the LSEs and
  // accumulators of four consecutive teams at a time, all loads of a group issued together.
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int H = a.n_heads;
  const int d = threadIdx.x * 4;
  const int64_t first = a.ws_prefix[b];
  const int64_t last = static_cast<int64_t>(a.ws_prefix[b + 1]) - 1;
  const int64_t total = a.ws_prefix[a.batch];
  uint16_t* out = reinterpret_cast<uint16_t*>(a.out) + (static_cast<int64_t>(b) * H + h) * kDL + d;
  if (last < first) {  // empty sequence
    *reinterpret_cast<u32x2*>(out) = u32x2{0u, 0u};
    if (a.lse != nullptr && threadIdx.x == 0) a.lse[b * H + h] = -INFINITY;
    return;
  }
  const int64_t n = a.n_teams;
  const int t_first = team_of(first, total, n);
  const int t_last = team_of(last, total, n);
  if (t_first == t_last) return;  // one team saw the whole context and wrote the output
  // team_start(t) = t * q + floor(t * r / n) with total = q * n + r: stepped without a division
  const bool fits32 = total * n < (1LL << 31);
  const int64_t q = fits32 ? static_cast<int64_t>(static_cast<uint32_t>(total) / static_cast<uint32_t>(n)) : total / n, r = total - q * n;
  int64_t acc = fits32 ? static_cast<int64_t>(static_cast<uint32_t>(t_first) * static_cast<uint32_t>(r) % static_cast<uint32_t>(n))
                       : (static_cast<int64_t>(t_first) * r) % n;
  // the first team holds this context as its last run (slot 1) unless its range starts exactly
  // here; every later one holds it as its first run (slot 0)
  const int slot_first = team_start(t_first, total, n) < first ? 1 : 0;
  float M = kNegBig, W = 0.0f;
  f32x4 O = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int tb = t_first; tb <= t_last; tb += 4) {
    float lse[4];
    f32x4 x[4];
    bool on[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int t = tb + k;
      acc += r;
      const int64_t step = q + (acc >= n ? 1 : 0);
      acc -= acc >= n ? n : 0;
      // with fewer tiles than teams some ranges in between are empty and own no partial
      on[k] = t <= t_last && step > 0;
      const int64_t ps = (static_cast<int64_t>(t) * 2 + (t == t_first ? slot_first : 0)) * H + h;
      lse[k] = on[k] ? a.ws_lse[ps] : kNegBig;
      x[k] = on[k] ? *reinterpret_cast<const f32x4*>(a.ws_out + ps * kDL + d) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
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
  const float inv = 1.0f / W;
  *reinterpret_cast<u32x2*>(out) = u32x2{QT::pack(O[0] * inv, O[1] * inv), QT::pack(O[2] * inv, O[3] * inv)};
  if (a.lse != nullptr && threadIdx.x == 0) a.lse[b * H + h] = (M + fast_log2(W)) * kLn2;
}

// The merge of mla_decode_w4_kernel's partial rows as a launch of its own (when the decode kernel does not fold them
// itself): one workgroup per (block of 16 heads, sequence); also writes the output of empty sequences.
template <typename QT>
__global__ __launch_bounds__(256) void mla_merge_tiles_kernel(MlaArgs a) {
  const int hb = blockIdx.x;
  const int b = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  if (a.plan != nullptr && a.plan[0] != a.plan_sig) return;   // the decode kernel wrote nothing and raised the flag
  MlaPieces p;
  if (!mla_locate_pieces(a, a.ws_prefix[b], a.ws_prefix[b + 1], a.ws_prefix[a.batch], p)) {  // empty sequence
    mla_write_empty<QT>(a, hb, b, w, lane);
    return;
  }
  if (p.t_first == p.t_last) return;  // one team saw the whole context and wrote the output
  mla_merge_tiles<QT>(a, p, hb, b, w, lane);
}

// Teams: as many as there are CUs for the team size, a multiple of 8 (one per XCD slot).
int mla_teams(int n_hb) {
  static const int knob = [] {
    const char* e = getenv("XLLM_MI355_MLA_WGS");  // tuning knob: workgroups in flight
    const int v = e ? atoi(e) : 0;
    return v > 0 ? v : 0;
  }();
  const int wgs = knob > 0 ? knob : device_cu_count();
  int teams = wgs / n_hb / 8 * 8;
  return teams < 8 ? 8 : teams;
}

// Tuning knob XLLM_MI355_MLA_KERNEL, read once per process (first letter: 'p' pairs, 'h' heads, 'n' narrow); a test may
// override it through set_mla_kernel_knob.
std::atomic<int> g_mla_knob{-1};
int mla_kernel_knob() {
  int v = g_mla_knob.load(std::memory_order_relaxed);
  if (v < 0) {
    const char* e = getenv("XLLM_MI355_MLA_KERNEL");
    v = e != nullptr ? static_cast<unsigned char>(e[0]) : 0;
    g_mla_knob.store(v, std::memory_order_relaxed);
  }
  return v;
}

// Whether mla_decode_w4_kernel merges the pieces of a context itself instead of leaving them to mla_merge_tiles_kernel.
// Off by default.  The merge moves the same bytes either way (every piece, 128 KB of 16-bit rows per workgroup and run,
// written once and read once: 41 MB on 64 contexts over 256 workgroups), and that is what it costs: the merging
// workgroups of one launch read them at 4.8 TB/s between them (6.3 us per workgroup after 2.3 us of waiting for the
// count), whether they ask for them at the scope of the GPU or of the workgroup, where the second launch takes 11.5 us:
// decode + merge 182.6 us as two launches, 183.5 us as one, a step 189 us against 191 us.  What the one launch adds is
// a wait of workgroups on each other, which needs all of them resident at once; a device that runs fewer at a time
// reports XLLM_MI355_ESTALLED instead of an output.  "1" in XLLM_MI355_MLA_FOLD, read once per process, or set_mla_fold
// (test hook) turn it on.  Same bits either way.
std::atomic<int> g_mla_fold{-1};
bool mla_fold_enabled() {
  int v = g_mla_fold.load(std::memory_order_relaxed);
  if (v < 0) {
    const char* e = getenv("XLLM_MI355_MLA_FOLD");  // tuning knob
    v = e != nullptr && e[0] == '1' ? 1 : 0;
    g_mla_fold.store(v, std::memory_order_relaxed);
  }
  return v != 0;
}

}  // namespace

void set_mla_fold(int on) { g_mla_fold.store(on < 0 ? -1 : (on != 0 ? 1 : 0), std::memory_order_relaxed); }
void set_mla_kernel_knob(int first_letter) { g_mla_knob.store(first_letter < 0 ? 0 : first_letter, std::memory_order_relaxed); }

namespace {
// Tiles that the schedule of mla_decode_w4_kernel charges for the start of a run (tuning knob XLLM_MI355_MLA_RUN_COST).
int w4_run_cost() {
  static const int run_cost = [] {
    const char* e = getenv("XLLM_MI355_MLA_RUN_COST");
    const int v = e ? atoi(e) : -1;
    return v >= 0 && v <= 64 ? v : 3;
  }();
  return run_cost * (kTile / kW4Item);
}
// Whether mla_decode_w4_kernel serves a call (more than 64 heads, block size a power of two >= 16, no knob that asks
// for another kernel); a plan is made for it and for no other.
bool w4_serves(int64_t n_heads, int64_t block_size) {
  const int knob = mla_kernel_knob();
  const bool pairs = knob == 'p' || block_size < 16 || (block_size & (block_size - 1)) != 0;
  const bool by_dims = !pairs && knob != 'h' && n_heads > 64;
#ifdef XLLM_MLA_DEFAULT_NARROW
  return by_dims && knob == 'w';
#else
  return by_dims && knob != 'n';
#endif
}
// What a plan is made for: everything that the schedule depends on besides the lengths themselves.
int mla_plan_signature(const MlaArgs& a) {
  uint32_t h = 2166136261u;
  const int v[] = {a.batch, a.n_heads, a.n_teams, a.n_hb, a.run_cost, a.bs_shift, 0x6d6c61};
  for (int x : v) h = (h ^ static_cast<uint32_t>(x)) * 16777619u;
  return static_cast<int>(h | 1u);
}
}  // namespace

int paged_decode_mla_plan(void* plan, size_t plan_bytes, const PageAddressing& addr, int64_t batch, int64_t n_heads,
                          int64_t block_size, hipStream_t stream) {
  if (batch == 0) return XLLM_MI355_OK;
  if (plan == nullptr || (reinterpret_cast<uintptr_t>(plan) & 255) != 0 || plan_bytes < kPlanBytes)
    return XLLM_MI355_EWORKSPACE;
  if (addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0) return XLLM_MI355_EINVAL;
  if (batch < 0 || n_heads <= 0 || n_heads > 65535 || block_size <= 0) return XLLM_MI355_EINVAL;
  // Shapes that mla_decode_w4_kernel does not serve, and batches decoded in slices, take no plan: the planned entry
  // point decodes them like the plain one.
  const int64_t max_batch = kDsMaxBatch < kMaxBatchMla ? kDsMaxBatch : kMaxBatchMla;
  if (!w4_serves(n_heads, block_size) || batch > max_batch) return XLLM_MI355_OK;
  MlaArgs a = {};
  a.block_table = addr.block_table;
  a.seq_lens = addr.seq_lens;
  a.table_stride = addr.table_stride;
  a.batch = static_cast<int>(batch);
  a.n_heads = static_cast<int>(n_heads);
  a.n_hb = static_cast<int>((n_heads + kHeadsPerWg16 - 1) / kHeadsPerWg16);
  a.n_teams = mla_teams(a.n_hb);
  if (a.n_teams > kPlanMaxTeams) return XLLM_MI355_OK;
  a.block_size = static_cast<int>(block_size);
  a.bs_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1LL << s) == block_size) a.bs_shift = s;
  a.run_cost = w4_run_cost();
  a.plan_sig = mla_plan_signature(a);
  const int per_wg = kW4Threads / kWave;
  const dim3 grid(static_cast<unsigned>((a.n_teams + per_wg - 1) / per_wg));
  const size_t smem = (static_cast<size_t>(a.batch) + 1 + 8) * 4;
  launch_timed(mla_plan_kernel, grid, dim3(kW4Threads), smem, stream, a, static_cast<int*>(plan));
  return static_cast<int>(hipGetLastError());
}

size_t mla_workspace_bytes(int64_t batch, int64_t n_heads, int64_t max_seq_len) {
  (void)batch;  // (the layout does not depend on it)
  (void)max_seq_len;
  // the kernel with 128 heads per workgroup has the fewer workgroups per team, hence the more teams
  const int n_hb = static_cast<int>((n_heads + kHeadsPerWg16 - 1) / kHeadsPerWg16);
  // (slots of whole 16-head blocks: the kernel with 128 heads per workgroup writes its partial rows as tiles)
  const size_t slot_heads = static_cast<size_t>((n_heads + 15) / 16 * 16);
  return kWsPartialsOff + static_cast<size_t>(mla_teams(n_hb)) * 2 * (slot_heads * kDL + n_heads) * 4;
}

int paged_decode_mla(const void* q_nope, const void* q_pe, const void* k_cache, void* out, float* lse,
                     const PageAddressing& addr, int64_t batch, int64_t n_heads, int64_t d_latent,
                     int64_t d_rope, int64_t block_size, int64_t num_blocks, int64_t max_seq_len,
                     float sm_scale, void* workspace, size_t workspace_bytes, int dtype,
                     hipStream_t stream, const NewLatentRows* fresh) {
  (void)max_seq_len;  // the schedule is computed on the device from the actual lengths
  if (batch == 0) return XLLM_MI355_OK;
  if (q_nope == nullptr || q_pe == nullptr || k_cache == nullptr || out == nullptr ||
      addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0)
    return XLLM_MI355_EINVAL;
  if (fresh != nullptr && (fresh->rows == nullptr || fresh->slots == nullptr || fresh->row_stride < kDK))
    return XLLM_MI355_EINVAL;
  if (batch < 0 || n_heads <= 0 || n_heads > 65535 || block_size <= 0 || num_blocks <= 0 ||
      !(sm_scale > 0.0f))
    return XLLM_MI355_EINVAL;
  if (d_latent != kDL || d_rope != kDR) return XLLM_MI355_ESHAPE;
  if (dtype != XLLM_MI355_BF16 && dtype != XLLM_MI355_FP16) return XLLM_MI355_EDTYPE;
  const bool f16 = dtype == XLLM_MI355_FP16;
  if (num_blocks * block_size > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!aligned16(q_nope) || !aligned16(q_pe) || !aligned16(k_cache) || !aligned16(out))
    return XLLM_MI355_EALIGN;
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 ||
      workspace_bytes < mla_workspace_bytes(batch, n_heads, 0))
    return XLLM_MI355_EWORKSPACE;
  if (addr.plan != nullptr && (reinterpret_cast<uintptr_t>(addr.plan) & 255) != 0) return XLLM_MI355_EWORKSPACE;

  // "pairs" selects the kernel with the per-tile exchange (also taken for block sizes below 16 or not a power
  // of two: the other kernels look pages up per group of 4 tokens inside chunks of 64 pages)
  const int knob = mla_kernel_knob();
  const bool pairs = knob == 'p' || block_size < 16 || (block_size & (block_size - 1)) != 0;
  // more than 64 heads: scores by head block, P.V by dim block ("heads" keeps P.V by head block, for comparison)
  const bool by_dims = !pairs && knob != 'h' && n_heads > 64;
  const int64_t max_batch = by_dims ? (kDsMaxBatch < kMaxBatchMla ? kDsMaxBatch : kMaxBatchMla) : kMaxBatchMla;
  const int n_hb = static_cast<int>(pairs ? (n_heads + kHeadsPerWg - 1) / kHeadsPerWg
                                          : (n_heads + kHeadsPerWg16 - 1) / kHeadsPerWg16);
  static std::atomic<uint64_t> configured{0};
  const size_t smem = pairs ? kPrefixOff + (kMaxBatchMla + 1) * 4 : kPrefix16Off + (kMaxBatchMla + 1) * 4;
  if (first_use_on_current_device(configured)) {
    hipError_t e = hipSuccess;
    const int lds_pairs = static_cast<int>(kPrefixOff + (kMaxBatchMla + 1) * 4);
    const int lds_16 = static_cast<int>(kPrefix16Off + (kMaxBatchMla + 1) * 4);
    const void* pairs_kernels[] = {reinterpret_cast<const void*>(mla_decode_kernel<BF16>),
                                   reinterpret_cast<const void*>(mla_decode_kernel<FP16>)};
    const void* kernels_16[] = {reinterpret_cast<const void*>(mla_decode16_kernel<BF16, false>),
                                reinterpret_cast<const void*>(mla_decode16_kernel<BF16, true>),
                                reinterpret_cast<const void*>(mla_decode16_kernel<FP16, false>),
                                reinterpret_cast<const void*>(mla_decode16_kernel<FP16, true>)};
    for (const void* k : pairs_kernels)
      if (e == hipSuccess) e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds_pairs);
    for (const void* k : kernels_16)
      if (e == hipSuccess) e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds_16);
    const void* kernels_ds[] = {reinterpret_cast<const void*>(mla_decode_ds_kernel<BF16>),
                                reinterpret_cast<const void*>(mla_decode_ds_kernel<FP16>)};
    for (const void* k : kernels_ds)
      if (e == hipSuccess) e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kDsLdsBytes);
    const void* kernels_w4[] = {reinterpret_cast<const void*>(mla_decode_w4_kernel<BF16>),
                                reinterpret_cast<const void*>(mla_decode_w4_kernel<FP16>)};
    for (const void* k : kernels_w4)
      if (e == hipSuccess) e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kW4LdsBytes);
    if (e != hipSuccess) return static_cast<int>(e);
  }
  // The step's new rows: inside mla_decode_w4_kernel where it serves the call and the rows can be fetched 16 bytes at
  // a time; otherwise the store is a launch of its own before the decode, with the same result.
  const bool w4_call = w4_serves(n_heads, block_size);
  const bool fused = fresh != nullptr && w4_call && aligned16(fresh->rows) && (fresh->row_stride * 2) % 16 == 0;
  if (fresh != nullptr && !fused) {
    const int rc = reshape_and_cache(fresh->rows, nullptr, const_cast<void*>(k_cache), nullptr, fresh->slots, nullptr,
                                     nullptr, batch, 1, kDK, block_size, num_blocks, fresh->row_stride, 0, dtype, dtype,
                                     stream);
    if (rc != 0) return rc;
  }
  for (int64_t b0 = 0; b0 < batch; b0 += max_batch) {
    const int64_t nb = batch - b0 < max_batch ? batch - b0 : max_batch;
    MlaArgs a = {};
    if (fused) {
      a.new_rows = static_cast<const char*>(fresh->rows) + b0 * fresh->row_stride * 2;
      a.new_slots = fresh->slots + b0;
      a.new_row_stride_bytes = fresh->row_stride * 2;
      a.n_slots = num_blocks * block_size;
      a.k_cache_w = static_cast<char*>(const_cast<void*>(k_cache));
    }
    a.q_nope = static_cast<const char*>(q_nope) + b0 * n_heads * kDL * 2;
    a.q_pe = static_cast<const char*>(q_pe) + b0 * n_heads * kDR * 2;
    a.k_cache = static_cast<const char*>(k_cache);
    a.out = static_cast<char*>(out) + b0 * n_heads * kDL * 2;
    a.lse = lse == nullptr ? nullptr : lse + b0 * n_heads;
    a.block_table = addr.block_table + b0 * addr.table_stride;
    a.seq_lens = addr.seq_lens + b0;
    a.table_stride = addr.table_stride;
    a.batch = static_cast<int>(nb);
    a.n_heads = static_cast<int>(n_heads);
    a.n_hb = n_hb;
    a.n_teams = mla_teams(a.n_hb);
    a.block_size = static_cast<int>(block_size);
    a.bs_shift = -1;
    for (int s = 0; s < 31; ++s)
      if ((1LL << s) == block_size) a.bs_shift = s;
    a.num_blocks = static_cast<int>(num_blocks);
    a.scale_log2 = sm_scale * kLog2e;
    a.ws_prefix = reinterpret_cast<int*>(static_cast<char*>(workspace) + kWsHeaderBytes);
    a.ws_out = reinterpret_cast<float*>(static_cast<char*>(workspace) + kWsPartialsOff);
    a.slot_heads = static_cast<int>((n_heads + 15) / 16 * 16);
    a.ws_lse = a.ws_out + static_cast<size_t>(a.n_teams) * 2 * a.slot_heads * kDL;
    // (XLLM_MLA_DEFAULT_NARROW: the build found that the compiler did not leave the fixed-name accumulators of
    // mla_decode_w4_kernel alone and made the eight-wavefront kernel the default; 'w' still asks for the other)
    const bool w4 = w4_call;
    a.run_cost = w4 ? w4_run_cost() : 0;
    // the step's plan: for the kernel it was made for, and not for a batch decoded in slices
    a.plan = w4 && batch <= max_batch && a.n_teams <= kPlanMaxTeams ? static_cast<const int*>(addr.plan) : nullptr;
    if (a.plan != nullptr) {
      a.plan_sig = mla_plan_signature(a);
      a.ws_prefix = const_cast<int*>(a.plan) + kPlanPrefixOff;   // (what the merge kernel reads)
    }
    // (two counters per context, kept with its first team, in the header of the workspace)
    a.fold = w4 && a.n_teams * a.n_hb <= kFoldSeenOff && mla_fold_enabled() ? 1 : 0;
    a.ws_status = static_cast<int*>(workspace);
    a.ws_written = reinterpret_cast<unsigned*>(static_cast<char*>(workspace) + kWsCountersOff);
    a.wait_spins = wait_spin_limit();

    const dim3 grid(static_cast<unsigned>(a.n_teams * a.n_hb));
    if (pairs) {
      if (f16) launch_timed(mla_decode_kernel<FP16>, grid, dim3(kMlaThreads), smem, stream, a);
      else launch_timed(mla_decode_kernel<BF16>, grid, dim3(kMlaThreads), smem, stream, a);
    } else if (w4) {  // ('n'arrow: the kernel with 16 heads per scoring wavefront, 3 % slower on 128 heads)
      if (f16) launch_timed(mla_decode_w4_kernel<FP16>, grid, dim3(kW4Threads), kW4LdsBytes, stream, a);
      else launch_timed(mla_decode_w4_kernel<BF16>, grid, dim3(kW4Threads), kW4LdsBytes, stream, a);
    } else if (by_dims) {
      if (f16) launch_timed(mla_decode_ds_kernel<FP16>, grid, dim3(kThreads16), kDsLdsBytes, stream, a);
      else launch_timed(mla_decode_ds_kernel<BF16>, grid, dim3(kThreads16), kDsLdsBytes, stream, a);
    } else if (n_heads <= 64) {  // head counts of tensor-parallel shards: two wavefronts per 16 heads
      if (f16) launch_timed(mla_decode16_kernel<FP16, true>, grid, dim3(kThreads16), smem, stream, a);
      else launch_timed(mla_decode16_kernel<BF16, true>, grid, dim3(kThreads16), smem, stream, a);
    } else {
      if (f16) launch_timed(mla_decode16_kernel<FP16, false>, grid, dim3(kThreads16), smem, stream, a);
      else launch_timed(mla_decode16_kernel<BF16, false>, grid, dim3(kThreads16), smem, stream, a);
    }
    int rc = static_cast<int>(hipGetLastError());
    if (rc != 0) return rc;
    const dim3 mgrid(static_cast<unsigned>(n_heads), static_cast<unsigned>(nb));
    if (a.fold != 0) {   // the decode kernel merged
      profile_skip();
    } else if (w4) {   // (its partial rows are tiles)
      const dim3 tgrid(static_cast<unsigned>(a.slot_heads / 16), static_cast<unsigned>(nb));
      if (f16) launch_timed(mla_merge_tiles_kernel<FP16>, tgrid, dim3(256), 0, stream, a);
      else launch_timed(mla_merge_tiles_kernel<BF16>, tgrid, dim3(256), 0, stream, a);
    } else {
      if (f16) launch_timed(mla_merge_kernel<FP16>, mgrid, dim3(128), 0, stream, a);
      else launch_timed(mla_merge_kernel<BF16>, mgrid, dim3(128), 0, stream, a);
    }
    rc = static_cast<int>(hipGetLastError());
    if (rc != 0) return rc;
  }
  return XLLM_MI355_OK;
}

}  // namespace xllm_mi355
