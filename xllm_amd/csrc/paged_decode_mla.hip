// Paged decode attention, MLA latent-KV variant, for gfx950.
//
// All query heads share ONE latent KV head of 576 dims (512 latent + 64 rope); V is the
// first 512 dims of the same rows.  With 16..128 heads per sequence the two products are
// dense contractions, so they run on MFMA (v_mfma_f32_16x16x32_bf16):
//   S^T[tok, head]  = K[tok, 576] . Q^T[576, head]       A = K tile from LDS (16-byte rows)
//                                                        B = Q^T, resident in registers
//   O^T[dim, head] += V^T[dim, tok] . P^T[tok, head]     A = V^T read from the SAME LDS tile
//                                                            with the transposing LDS load
//                                                        B = P^T, taken straight from the
//                                                            S^T accumulator registers
// so each 64-token page is staged in LDS once (rows padded to 1168 bytes, which spreads
// 16 consecutive rows over all banks for the 16-byte operand reads) and serves both
// products; softmax state lives in the lanes that own a head column, and the rescale of
// the 128 output accumulators is skipped while the running maximum does not move.
// One 256-thread workgroup covers 64 heads (16 per wavefront) of one (sequence, split);
// tiles are double-buffered in LDS with the next tile's global loads in flight during
// the MFMAs.  Splits write normalised fp32 partials that merge_splits folds.
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
constexpr int kTile = 64;           // tokens per LDS tile
constexpr int kRowBytes = kDK * 2;  // 1152
constexpr int kLdsRow = kRowBytes + 16;
constexpr int kTileBytes = kTile * kLdsRow;  // 74752
constexpr int kMlaThreads = 256;
constexpr int kMlaWaves = kMlaThreads / kWave;
constexpr int kHeadsPerWg = 16 * kMlaWaves;  // 64
constexpr int kChunksPerRow = kRowBytes / 16;                                 // 72
constexpr int kLoadsPerThread = kTile * kChunksPerRow / kMlaThreads;          // 18
constexpr int kKSteps = kDK / 32;   // 18
constexpr int kMBlocks = kDL / 16;  // 32

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

struct MlaArgs {
  const char* q_nope;
  const char* q_pe;
  const char* k_cache;
  char* out;
  float* lse;
  const int32_t* block_table;
  const int32_t* seq_lens;
  float* ws_out;
  float* ws_lse;
  int64_t table_stride;
  int n_heads;
  int block_size;
  int bs_shift;
  int num_blocks;
  int chunk_tokens;
  int max_splits;
  float scale_log2;
};

struct SplitPlan {
  int chunk_tokens;  // tokens of one split (multiple of the tile)
  int max_splits;    // ceil(max_seq_len / chunk_tokens)
};

SplitPlan plan_mla_splits(int64_t batch, int64_t n_head_blocks, int64_t max_seq_len) {
  // One MLA workgroup owns a CU (its two LDS tiles fill it) and every split costs a
  // [heads, 512] fp32 partial, so: about two workgroups per CU, splits of at least 512 tokens.
  static const int64_t kTarget = [] {
    const char* e = getenv("XLLM_MI355_MLA_TARGET_WGS");  // tuning knob
    const long v = e ? atol(e) : 0;
    return static_cast<int64_t>(v > 0 ? v : 512);
  }();
  constexpr int64_t kMinChunk = 512;
  if (max_seq_len < 1) max_seq_len = 1;
  const int64_t units = batch * n_head_blocks > 0 ? batch * n_head_blocks : 1;
  int64_t splits = (kTarget + units - 1) / units;
  const int64_t max_by_len = (max_seq_len + kMinChunk - 1) / kMinChunk;
  if (splits > max_by_len) splits = max_by_len;
  if (splits < 1) splits = 1;
  int64_t chunk = (max_seq_len + splits - 1) / splits;
  chunk = (chunk + kTile - 1) / kTile * kTile;
  SplitPlan p;
  p.chunk_tokens = static_cast<int>(chunk);
  p.max_splits = static_cast<int>((max_seq_len + chunk - 1) / chunk);
  return p;
}

size_t split_workspace_bytes(int64_t batch, int64_t n_heads, int max_splits) {
  if (max_splits <= 1) return 0;
  return static_cast<size_t>(batch) * n_heads * max_splits * (kDL + 1) * sizeof(float);
}

// Merge of split partials: one workgroup per (head, sequence).
__global__ __launch_bounds__(128) void mla_merge_kernel(const float* ws_out, const float* ws_lse,
                                                        char* out, float* lse, const int32_t* seq_lens,
                                                        int n_heads, int chunk_tokens, int max_splits) {
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int L = seq_lens[b];
  const int n_splits = (L + chunk_tokens - 1) / chunk_tokens;
  if (n_splits <= 1) return;  // written directly by the decode kernel
  const int64_t w0 = (static_cast<int64_t>(b) * n_heads + h) * max_splits;
  float mx = kNegBig;
  for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, ws_lse[w0 + s]);
  float wsum = 0.0f;
  for (int s = 0; s < n_splits; ++s) wsum += fast_exp2(ws_lse[w0 + s] - mx);
  const float inv = 1.0f / wsum;
  uint16_t* o = reinterpret_cast<uint16_t*>(out) + (static_cast<int64_t>(b) * n_heads + h) * kDL;
  for (int d = threadIdx.x; d < kDL; d += 128) {
    float acc = 0.0f;
    for (int s = 0; s < n_splits; ++s) acc += fast_exp2(ws_lse[w0 + s] - mx) * ws_out[(w0 + s) * kDL + d];
    o[d] = BF16::from_f32(acc * inv);
  }
  if (lse != nullptr && threadIdx.x == 0) lse[b * n_heads + h] = (mx + fast_log2(wsum)) * kLn2;
}

__device__ __forceinline__ float xlane_max(float x) {  // over lanes l, l^16, l^32, l^48
  auto r = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
  x = fmaxf(as_f32(r[0]), as_f32(r[1]));
  auto t = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
  return fmaxf(as_f32(t[0]), as_f32(t[1]));
}

__device__ __forceinline__ float xlane_sum(float x) {
  auto r = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
  x = as_f32(r[0]) + as_f32(r[1]);
  auto t = __builtin_amdgcn_permlane32_swap(as_u32(x), as_u32(x), false, false);
  return as_f32(t[0]) + as_f32(t[1]);
}

__global__ __launch_bounds__(kMlaThreads) void mla_decode_kernel(MlaArgs a) {
  extern __shared__ __align__(16) char smem[];  // two tiles of [64][1168] bytes

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int c16 = lane & 15;  // MFMA row / column index owned by the lane
  const int g = lane >> 4;    // MFMA k-group of the lane
  const int split = blockIdx.x;
  const int b = blockIdx.z;
  const int head_base = blockIdx.y * kHeadsPerWg;
  const int head = head_base + wave * 16 + c16;
  const bool head_ok = head < a.n_heads;
  const bool wave_ok = head_base + wave * 16 < a.n_heads;
  const int H = a.n_heads;

  const int32_t* pages = a.block_table + static_cast<int64_t>(b) * a.table_stride;
  const int L = a.seq_lens[b];
  if (L <= 0) {
    if (split == 0 && head_ok) {
      u32x2* o = reinterpret_cast<u32x2*>(a.out + (static_cast<int64_t>(b) * H + head) * kDL * 2);
      for (int i = g; i < kDL / 4; i += 4) o[i] = u32x2{0u, 0u};
      if (a.lse != nullptr && g == 0) a.lse[b * H + head] = -INFINITY;
    }
    return;
  }
  const int n_splits = (L + a.chunk_tokens - 1) / a.chunk_tokens;
  if (split >= n_splits) return;
  const int t0 = split * a.chunk_tokens;
  const int t1 = min(L, t0 + a.chunk_tokens);
  const int n_tiles = (t1 - t0 + kTile - 1) / kTile;

  // Q^T operand: lane (head c16, k-group g) keeps dims ks*32 + g*8 .. +8 of every k-step
  bf16x8 q[kKSteps];
  {
    const char* qn = a.q_nope + (static_cast<int64_t>(b) * H + head) * kDL * 2;
    const char* qp = a.q_pe + (static_cast<int64_t>(b) * H + head) * kDR * 2;
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      u32x4 x = {0u, 0u, 0u, 0u};
      if (head_ok) x = ks < kDL / 32 ? ldg16(qn + (ks * 32 + g * 8) * 2) : ldg16(qp + ((ks - kDL / 32) * 32 + g * 8) * 2);
      q[ks] = __builtin_bit_cast(bf16x8, x);
    }
  }

  f32x4 o[kMBlocks];
#pragma unroll
  for (int i = 0; i < kMBlocks; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = kNegBig, l = 0.0f;

  u32x4 stage[kLoadsPerThread];
  auto load_tile = [&](int tile) {
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) {
      const int c = i * kMlaThreads + tid;
      const int row = c / kChunksPerRow;
      const int col = c - row * kChunksPerRow;
      const int tok = min(t0 + tile * kTile + row, L - 1);
      int pg, off;
      if (a.bs_shift >= 0) {
        pg = tok >> a.bs_shift;
        off = tok & (a.block_size - 1);
      } else {
        pg = tok / a.block_size;
        off = tok - pg * a.block_size;
      }
      int page = pages[pg];
      page = max(0, min(page, a.num_blocks - 1));
      const int64_t slot = static_cast<int64_t>(page) * a.block_size + off;
      stage[i] = ldg16(a.k_cache + slot * kRowBytes + col * 16);
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kLoadsPerThread; ++i) {
      const int c = i * kMlaThreads + tid;
      const int row = c / kChunksPerRow;
      const int col = c - row * kChunksPerRow;
      *reinterpret_cast<u32x4*>(smem + buf * kTileBytes + row * kLdsRow + col * 16) = stage[i];
    }
  };

  auto compute = [&](int buf, int tile) {
    const char* kb = smem + buf * kTileBytes;
    // ---- S^T = K . Q^T : 4 token blocks of 16, 18 k-steps
    f32x4 s[4];
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) s[tb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
#pragma unroll
      for (int tb = 0; tb < 4; ++tb) {
        const u32x4 x = *reinterpret_cast<const u32x4*>(kb + (tb * 16 + c16) * kLdsRow + (ks * 32 + g * 8) * 2);
        s[tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x), q[ks], s[tb], 0, 0, 0);
      }
    }
    // ---- online softmax; the lane owns head c16 and tokens tb*16 + g*4 + i
    const int tok_base = t0 + tile * kTile + g * 4;
    float mx = kNegBig;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = tok_base + tb * 16 + i < t1 ? s[tb][i] * a.scale_log2 : -INFINITY;
        s[tb][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = xlane_max(mx);
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2(m - m_new);
    m = m_new;
    float sum = 0.0f;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        s[tb][i] = fast_exp2(s[tb][i] - m_new);
        sum += s[tb][i];
      }
    l = l * alpha + sum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int i = 0; i < kMBlocks; ++i) o[i] *= alpha;
    }
    // P^T operands: k-step kk uses token blocks 2kk and 2kk+1, k-slot g*8+i <-> token block
    // (2kk + i/4), row g*4 + i%4 -- the V^T operand below is gathered in the same order
    bf16x8 pb[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      u32x4 x;
      x[0] = BF16::pack(s[2 * kk][0], s[2 * kk][1]);
      x[1] = BF16::pack(s[2 * kk][2], s[2 * kk][3]);
      x[2] = BF16::pack(s[2 * kk + 1][0], s[2 * kk + 1][1]);
      x[3] = BF16::pack(s[2 * kk + 1][2], s[2 * kk + 1][3]);
      pb[kk] = __builtin_bit_cast(bf16x8, x);
    }
    // ---- O^T += V^T . P^T : the transposing LDS load hands lane c16 the 4 tokens g*4..+4
    // of dim column mb*16 + c16; each lane supplies the address of 4 dims of one token row
    const char* vb = kb + (g * 4 + (c16 >> 2)) * kLdsRow + (c16 & 3) * 8;
#pragma unroll
    for (int mb = 0; mb < kMBlocks; ++mb) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s16x4*)(vb + (2 * kk) * 16 * kLdsRow + mb * 32));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_s16x4*)(vb + (2 * kk + 1) * 16 * kLdsRow + mb * 32));
        typedef __attribute__((ext_vector_type(8))) short s16x8;
        const s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        o[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v), pb[kk], o[mb], 0, 0, 0);
      }
    }
  };

  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int tile = 0; tile < n_tiles; ++tile) {
    const int buf = tile & 1;
    const bool more = tile + 1 < n_tiles;
    if (more) load_tile(tile + 1);
    if (wave_ok) compute(buf, tile);
    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  if (!head_ok) return;
  l = xlane_sum(l);
  const float inv = 1.0f / l;
  if (n_splits == 1) {
    char* op = a.out + (static_cast<int64_t>(b) * H + head) * kDL * 2;
#pragma unroll
    for (int mb = 0; mb < kMBlocks; ++mb) {
      u32x2 w;
      w[0] = BF16::pack(o[mb][0] * inv, o[mb][1] * inv);
      w[1] = BF16::pack(o[mb][2] * inv, o[mb][3] * inv);
      *reinterpret_cast<u32x2*>(op + (mb * 16 + g * 4) * 2) = w;
    }
    if (a.lse != nullptr && g == 0) a.lse[b * H + head] = (m + fast_log2(l)) * kLn2;
  } else {
    const int64_t wi = (static_cast<int64_t>(b) * H + head) * a.max_splits + split;
    float* wp = a.ws_out + wi * kDL;
#pragma unroll
    for (int mb = 0; mb < kMBlocks; ++mb)
      *reinterpret_cast<f32x4*>(wp + mb * 16 + g * 4) = o[mb] * inv;
    if (g == 0) a.ws_lse[wi] = m + fast_log2(l);
  }
}

}  // namespace

int paged_decode_mla(const void* q_nope, const void* q_pe, const void* k_cache, void* out, float* lse,
                     const PageAddressing& addr, int64_t batch, int64_t n_heads, int64_t d_latent,
                     int64_t d_rope, int64_t block_size, int64_t num_blocks, int64_t max_seq_len,
                     float sm_scale, void* workspace, size_t workspace_bytes, int dtype,
                     hipStream_t stream) {
  if (batch == 0) return XLLM_MI355_OK;
  if (q_nope == nullptr || q_pe == nullptr || k_cache == nullptr || out == nullptr ||
      addr.block_table == nullptr || addr.seq_lens == nullptr || addr.table_stride <= 0)
    return XLLM_MI355_EINVAL;
  if (batch < 0 || batch > 65535 || n_heads <= 0 || n_heads > 65535 || block_size <= 0 ||
      num_blocks <= 0)
    return XLLM_MI355_EINVAL;
  if (d_latent != kDL || d_rope != kDR) return XLLM_MI355_ESHAPE;
  if (dtype != XLLM_MI355_BF16) return XLLM_MI355_EDTYPE;
  if (num_blocks * block_size > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (!aligned16(q_nope) || !aligned16(q_pe) || !aligned16(k_cache) || !aligned16(out))
    return XLLM_MI355_EALIGN;
  if (max_seq_len <= 0) max_seq_len = addr.table_stride * block_size;

  const int head_blocks = static_cast<int>((n_heads + kHeadsPerWg - 1) / kHeadsPerWg);
  SplitPlan plan = plan_mla_splits(batch, head_blocks, max_seq_len);
  while (plan.max_splits > 1 &&
         split_workspace_bytes(batch, n_heads, plan.max_splits) > workspace_bytes) {
    if (plan.chunk_tokens >= (1 << 20)) return XLLM_MI355_EWORKSPACE;
    plan.chunk_tokens *= 2;
    plan.max_splits = static_cast<int>((max_seq_len + plan.chunk_tokens - 1) / plan.chunk_tokens);
  }
  if (plan.max_splits > 1 && (workspace == nullptr || !aligned16(workspace))) return XLLM_MI355_EWORKSPACE;

  MlaArgs a = {};
  a.q_nope = static_cast<const char*>(q_nope);
  a.q_pe = static_cast<const char*>(q_pe);
  a.k_cache = static_cast<const char*>(k_cache);
  a.out = static_cast<char*>(out);
  a.lse = lse;
  a.block_table = addr.block_table;
  a.seq_lens = addr.seq_lens;
  a.table_stride = addr.table_stride;
  a.n_heads = static_cast<int>(n_heads);
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
    a.ws_lse = a.ws_out + static_cast<size_t>(batch) * n_heads * plan.max_splits * kDL;
  }

  const size_t smem = 2 * static_cast<size_t>(kTileBytes);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mla_decode_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (e != hipSuccess) return static_cast<int>(e);
    attr_set = true;
  }
  dim3 grid(static_cast<unsigned>(plan.max_splits), static_cast<unsigned>(head_blocks),
            static_cast<unsigned>(batch));
  const bool timed = profile_begin(stream);
  mla_decode_kernel<<<grid, kMlaThreads, smem, stream>>>(a);
  if (timed) profile_end(stream);
  int rc = static_cast<int>(hipGetLastError());
  if (rc != 0 || plan.max_splits <= 1) return rc;
  mla_merge_kernel<<<dim3(static_cast<unsigned>(n_heads), static_cast<unsigned>(batch)), 128, 0, stream>>>(
      a.ws_out, a.ws_lse, static_cast<char*>(out), lse, addr.seq_lens, static_cast<int>(n_heads),
      plan.chunk_tokens, plan.max_splits);
  return static_cast<int>(hipGetLastError());
}

size_t mla_workspace_bytes(int64_t batch, int64_t n_heads, int64_t max_seq_len) {
  if (max_seq_len <= 0) return 0;
  const SplitPlan plan = plan_mla_splits(batch, (n_heads + kHeadsPerWg - 1) / kHeadsPerWg, max_seq_len);
  return split_workspace_bytes(batch, n_heads, plan.max_splits);
}

}  // namespace xllm_mi355
