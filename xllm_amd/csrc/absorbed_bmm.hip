// The two per-head matrix products either side of the MLA decode kernel, for gfx950:
//   y[t, h, :] = x[t, h, :] . w[h, :, :]        x [T, H, K], w [H, K, N] contiguous, y [T, H, N]
// They replace the torch::bmm calls of the reference's absorbed MLA attention
//   q_nope_absorbed = bmm(q_nope.transpose(0, 1), w_kc_).transpose(0, 1)
//       (xllm/core/layers/dcu/deepseek_v2_attention.cpp:428-430; K = 128, N = 512 for DeepSeek-V3)
//   attn_bmm = bmm(attn_latent.transpose(0, 1), w_vc_).transpose(0, 1)
//       (deepseek_v2_attention.cpp:231-238; K = 512, N = 128)
// with w_kc_ / w_vc_ in the layouts the reference prepares at load time (deepseek_v2_attention.cpp:479-485).
//
// At decode sizes the product is bound by reading the weights once (16.8 MB per matrix for 128 heads
// against 1 GFLOP), so the kernel is laid out for streaming: one workgroup per (head, 64 or 128 output
// columns, 64 to 256 tokens), the weight block staged through LDS 128 contraction rows at a time, and
// x read straight from global memory (the 8 workgroups of a head share it through L2).
//
// Matrix-core mapping (v_mfma_f32_16x16x32_bf16, fp32 accumulation), per wavefront = 16 tokens:
//   A = w^T block: row n, contraction k.  w is stored with n contiguous, so the 8 k-values a lane
//       needs are 8 rows apart: two transposing LDS reads (4 rows x 16 columns per 16 lanes each).
//   B = x^T: column t, the lane's 8 k-values are 16 contiguous bytes of x.
//   C = y^T: lane (t, g) holds columns 4g .. 4g+3 of its token; the block leaves through LDS as
//       128-byte rows.
#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {
namespace {

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int kBmmThreads = 256;
constexpr int kBmmCols = 64;                // output columns per workgroup (128 for many tokens)
constexpr int kBmmChunk = 128;              // contraction rows in LDS at a time

struct BmmArgs {
  const char* x;
  const char* w;
  char* y;
  int64_t x_token_stride, x_head_stride;  // bytes
  int64_t y_token_stride, y_head_stride;  // bytes
  int n_tokens, n_heads, k, n;
};

// TW = token blocks of 16 per wavefront: 16 * 4 * TW tokens per workgroup share one pass over the weights.
// NB = output columns per workgroup: x is read once per NB columns and w once per 64 TW tokens, so with
// many tokens the wider block halves what the workgroups of a head pull through L2.
template <int TW, int NB>
__global__ __launch_bounds__(kBmmThreads) void absorbed_bmm_kernel(BmmArgs a) {
  constexpr int kBmmRow = NB * 2 + 16;      // LDS row stride: 16 bytes of padding spread the rows over the banks
  constexpr int kRowThreads = NB * 2 / 16;  // threads that stage one row
  constexpr int kPassRows = kBmmThreads / kRowThreads;
  constexpr int kPasses = kBmmChunk / kPassRows;
  __shared__ __align__(16) char tile[kBmmChunk * kBmmRow];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int c16 = lane & 15;
  const int g = lane >> 4;
  const int n_blocks = a.n / NB;
  const int h = blockIdx.x / n_blocks;
  const int n0 = (blockIdx.x % n_blocks) * NB;
  const int t0 = (blockIdx.y * 4 + wave) * 16 * TW;  // first token of the wavefront

  const char* xp = a.x + (t0 + c16) * a.x_token_stride + h * a.x_head_stride + g * 16;
  const int64_t w_row = static_cast<int64_t>(a.n) * 2;
  // staging: thread -> 16 bytes of row tid / kRowThreads (+ kPassRows per pass)
  const char* wp = a.w + (static_cast<int64_t>(h) * a.k + tid / kRowThreads) * w_row + n0 * 2 + (tid % kRowThreads) * 16;
  char* stage = tile + (tid / kRowThreads) * kBmmRow + (tid % kRowThreads) * 16;
  // transposing read: lane p of a 16-lane group addresses 4 columns of row p / 4 and receives rows 0..3 of column p
  const char* rd = tile + (8 * g + (c16 >> 2)) * kBmmRow + (c16 & 3) * 8;

  f32x4 acc[TW][NB / 16];
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < NB / 16; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  // the weight rows of a chunk are in flight while the chunk before it is multiplied
  u32x4 wv[kPasses];
#pragma unroll
  for (int p = 0; p < kPasses; ++p) wv[p] = ldg16_stream(wp + p * kPassRows * w_row);
  for (int k0 = 0; k0 < a.k; k0 += kBmmChunk) {
    u32x4 xv[TW][kBmmChunk / 32];
#pragma unroll
    for (int i = 0; i < TW; ++i)
#pragma unroll
      for (int ks = 0; ks < kBmmChunk / 32; ++ks)
        xv[i][ks] = t0 + i * 16 + c16 < a.n_tokens ? ldg16(xp + i * 16 * a.x_token_stride + (k0 + ks * 32) * 2)
                                                   : u32x4{0u, 0u, 0u, 0u};
    __syncthreads();  // the previous chunk is no longer read
#pragma unroll
    for (int p = 0; p < kPasses; ++p) *reinterpret_cast<u32x4*>(stage + p * kPassRows * kBmmRow) = wv[p];
    __syncthreads();
    if (k0 + kBmmChunk < a.k) {
#pragma unroll
      for (int p = 0; p < kPasses; ++p) wv[p] = ldg16_stream(wp + (k0 + kBmmChunk + p * kPassRows) * w_row);
    }
#pragma unroll
    for (int ks = 0; ks < kBmmChunk / 32; ++ks) {
#pragma unroll
      for (int j = 0; j < NB / 16; ++j) {
        const char* r = rd + ks * 32 * kBmmRow + j * 32;
        const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(r));
        const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(r + 4 * kBmmRow));
        const s16x8 v = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
#pragma unroll
        for (int i = 0; i < TW; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v),
                                                              __builtin_bit_cast(bf16x8, xv[i][ks]), acc[i][j], 0, 0, 0);
      }
    }
  }
  // Output through LDS so that a token's NB columns leave as one row of 2 NB bytes: the accumulator layout
  // (4 columns of one token per lane) would store 8 bytes per lane, 16 tokens apart.
  __syncthreads();  // every wavefront is done with the weight rows
  static_assert(4 * 16 * kBmmRow <= kBmmChunk * kBmmRow, "one 16-token block per wavefront fits the tile");
  char* mine = tile + wave * 16 * kBmmRow;
#pragma unroll
  for (int i = 0; i < TW; ++i) {
#pragma unroll
    for (int j = 0; j < NB / 16; ++j) {
      const u32x2 o = {BF16::pack(acc[i][j][0], acc[i][j][1]), BF16::pack(acc[i][j][2], acc[i][j][3])};
      *reinterpret_cast<u32x2*>(mine + c16 * kBmmRow + (j * 16 + 4 * g) * 2) = o;
    }
#pragma unroll
    for (int part = 0; part < 16 / (kWave / kRowThreads); ++part) {
      const int row = part * (kWave / kRowThreads) + lane / kRowThreads;
      const int t = t0 + i * 16 + row;
      const u32x4 v = *reinterpret_cast<const u32x4*>(mine + row * kBmmRow + (lane % kRowThreads) * 16);
      if (t < a.n_tokens)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(a.y + t * a.y_token_stride + h * a.y_head_stride + n0 * 2 +
                                                                (lane % kRowThreads) * 16));
    }
  }
}

}  // namespace

int absorbed_bmm(const void* x, const void* w, void* y, int64_t n_tokens, int64_t n_heads, int64_t k, int64_t n,
                 int64_t x_token_stride, int64_t x_head_stride, int64_t y_token_stride, int64_t y_head_stride,
                 int dtype, hipStream_t stream) {
  if (n_tokens == 0) return XLLM_MI355_OK;
  if (x == nullptr || w == nullptr || y == nullptr) return XLLM_MI355_EINVAL;
  if (n_tokens < 0 || n_heads <= 0 || k <= 0 || n <= 0) return XLLM_MI355_EINVAL;
  if (dtype != XLLM_MI355_BF16) return XLLM_MI355_EDTYPE;
  if (k % kBmmChunk != 0 || n % kBmmCols != 0) return XLLM_MI355_ESHAPE;
  if (x_head_stride < k || y_head_stride < n || x_token_stride < k || y_token_stride < n) return XLLM_MI355_EINVAL;
  const uintptr_t ptrs = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(y);
  if ((ptrs & 15) != 0 || ((x_token_stride | x_head_stride | y_token_stride | y_head_stride) * 2) % 16 != 0)
    return XLLM_MI355_EALIGN;
  // tokens per workgroup: more of them share one pass over the weights, fewer leave wavefronts idle
  const int tw = n_tokens <= 64 ? 1 : n_tokens <= 128 ? 2 : 4;
  const int nb = tw == 4 && n % 128 == 0 ? 128 : kBmmCols;
  const int64_t gx = n_heads * (n / nb), gy = (n_tokens + 64 * tw - 1) / (64 * tw);
  if (gx > 0x7fffffffLL || gy > 65535 || k > 0x7fffffffLL / 4 || n > 0x7fffffffLL / 4) return XLLM_MI355_ESHAPE;
  BmmArgs a = {};
  a.x = static_cast<const char*>(x);
  a.w = static_cast<const char*>(w);
  a.y = static_cast<char*>(y);
  a.x_token_stride = x_token_stride * 2;
  a.x_head_stride = x_head_stride * 2;
  a.y_token_stride = y_token_stride * 2;
  a.y_head_stride = y_head_stride * 2;
  a.n_tokens = static_cast<int>(n_tokens);
  a.n_heads = static_cast<int>(n_heads);
  a.k = static_cast<int>(k);
  a.n = static_cast<int>(n);
  const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy));
  if (tw == 1) absorbed_bmm_kernel<1, 64><<<grid, kBmmThreads, 0, stream>>>(a);
  else if (tw == 2) absorbed_bmm_kernel<2, 64><<<grid, kBmmThreads, 0, stream>>>(a);
  else if (nb == 64) absorbed_bmm_kernel<4, 64><<<grid, kBmmThreads, 0, stream>>>(a);
  else absorbed_bmm_kernel<4, 128><<<grid, kBmmThreads, 0, stream>>>(a);
  return static_cast<int>(hipGetLastError());
}

}  // namespace xllm_mi355
