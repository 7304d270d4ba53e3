// reshape_and_cache for gfx950: scatter new K/V token rows into the paged cache.
//
// One workgroup row per token; each thread moves one 16-byte vector of the token's
// [Hkv * D] row (K vectors first, then V), so a 2 KiB Llama-3 row pair is one
// 256-thread workgroup of coalesced 16-byte loads and stores.  With an fp8 cache the
// thread quantises its 16 bytes in registers (per-KV-head scale, clamp, RNE) and
// stores the packed codes.  Rows that are not 16-byte friendly take an element-wise
// kernel with the same arithmetic.
//
// Semantics follow xllm/core/kernels/cuda/reshape_paged_cache.cu:23-63 (negative slot =
// skip, independent K/V token strides) and, for fp8, kernels/cuda/fp8_quant.cu:92-103.
#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

struct ReshapeArgs {
  const char* key;
  const char* value;
  char* k_cache;
  char* v_cache;
  const int32_t* slots;
  const float* k_scale;
  const float* v_scale;
  int64_t k_stride_bytes;
  int64_t v_stride_bytes;
  int64_t n_slots;     // num_blocks * block_size
  int64_t n_tokens;
  int row_elems;       // Hkv * D
  int head_dim;
  int n_vec;           // 16-byte input vectors per row
};

// IN: 0 bf16, 1 fp16, 2 fp32.  FP8: quantise, else byte copy.  TPW: tokens per workgroup row.  With one token a
// thread has 16 bytes in flight, which is right for the few tokens of a decode step (the launch is then a chain of two
// trips to memory, slot id then row) and leaves a prefill chunk bound by latency: from kStreamTokens tokens on a
// thread takes the same vector of TPW = 4 consecutive tokens, asks for all four before it stores the first, and the
// rows come and go with non-temporal accesses (a row is read once and written once).
constexpr int kStreamTokens = 2048;
template <int IN, bool FP8, int TPW>
__global__ __launch_bounds__(256) void reshape_vec_kernel(ReshapeArgs a) {
  int w = blockIdx.y * 256 + threadIdx.x;
  const bool is_v = w >= a.n_vec;
  if (is_v) w -= a.n_vec;
  if (w >= a.n_vec) return;
  const char* src = is_v ? a.value : a.key;
  char* cache = is_v ? a.v_cache : a.k_cache;
  if (src == nullptr || cache == nullptr) return;
  const int64_t stride = is_v ? a.v_stride_bytes : a.k_stride_bytes;
  int64_t slot[TPW];
  u32x4 x[TPW];
#pragma unroll
  for (int u = 0; u < TPW; ++u) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TPW + u;
    slot[u] = t < a.n_tokens ? a.slots[t] : -1;   // (looked at below, behind the row loads)
  }
  // (a row is asked for whether or not its slot turns out to be one to write: the two loads then travel together
  // instead of one after the other)
#pragma unroll
  for (int u = 0; u < TPW; ++u) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * TPW + u;
    const char* p = src + t * stride + static_cast<int64_t>(w) * 16;
    x[u] = u32x4{0u, 0u, 0u, 0u};
    if (t < a.n_tokens) x[u] = TPW > 1 ? ldg16_stream(p) : ldg16(p);
  }
  constexpr int EPV = IN == 2 ? 4 : 8;  // elements per 16-byte input vector
  float inv_scale = 0.0f;
  if constexpr (FP8) inv_scale = 1.0f / (is_v ? a.v_scale : a.k_scale)[w * EPV / a.head_dim];
#pragma unroll
  for (int u = 0; u < TPW; ++u) {
    if (slot[u] < 0 || slot[u] >= a.n_slots) continue;
    if constexpr (!FP8) {
      constexpr int ES = IN == 2 ? 4 : 2;
      char* dst = cache + slot[u] * (static_cast<int64_t>(a.row_elems) * ES) + static_cast<int64_t>(w) * 16;
      if constexpr (TPW > 1) __builtin_nontemporal_store(x[u], reinterpret_cast<u32x4*>(dst));
      else stg16(dst, x[u]);
    } else {
      char* dst = cache + slot[u] * static_cast<int64_t>(a.row_elems) + w * EPV;
      if constexpr (IN == 2) {
        u32 c = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) c |= fp8_quantize(as_f32(x[u][i]), inv_scale) << (8 * i);
        *reinterpret_cast<u32*>(dst) = c;
      } else {
        u32x2 c = {0u, 0u};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float lo, hi;
          if constexpr (IN == 0) { lo = BF16::lo(x[u][i]); hi = BF16::hi(x[u][i]); }
          else { lo = FP16::lo(x[u][i]); hi = FP16::hi(x[u][i]); }
          const u32 two = fp8_quantize(lo, inv_scale) | (fp8_quantize(hi, inv_scale) << 8);
          c[i >> 1] |= two << (16 * (i & 1));
        }
        *reinterpret_cast<u32x2*>(dst) = c;
      }
    }
  }
}

// Element-wise path for rows that are not a multiple of 16 bytes or not 16-byte aligned.
template <int IN, bool FP8>
__global__ __launch_bounds__(256) void reshape_elem_kernel(ReshapeArgs a) {
  const int64_t t = blockIdx.x;
  const int64_t slot = a.slots[t];
  if (slot < 0 || slot >= a.n_slots) return;
  constexpr int ES = IN == 2 ? 4 : 2;
  for (int pass = 0; pass < 2; ++pass) {
    const char* src = pass ? a.value : a.key;
    char* cache = pass ? a.v_cache : a.k_cache;
    if (src == nullptr || cache == nullptr) continue;
    const int64_t stride = pass ? a.v_stride_bytes : a.k_stride_bytes;
    const float* scale = pass ? a.v_scale : a.k_scale;
    for (int e = threadIdx.x; e < a.row_elems; e += 256) {
      const char* p = src + t * stride + static_cast<int64_t>(e) * ES;
      if constexpr (!FP8) {
        char* d = cache + (slot * a.row_elems + e) * ES;
        if constexpr (ES == 4) *reinterpret_cast<u32*>(d) = *reinterpret_cast<const u32*>(p);
        else *reinterpret_cast<uint16_t*>(d) = *reinterpret_cast<const uint16_t*>(p);
      } else {
        float x;
        if constexpr (IN == 2) x = *reinterpret_cast<const float*>(p);
        else if constexpr (IN == 0) x = BF16::to_f32(*reinterpret_cast<const uint16_t*>(p));
        else x = FP16::to_f32(*reinterpret_cast<const uint16_t*>(p));
        const float inv_scale = 1.0f / scale[e / a.head_dim];
        reinterpret_cast<uint8_t*>(cache)[slot * a.row_elems + e] =
            static_cast<uint8_t>(fp8_quantize(x, inv_scale));
      }
    }
  }
}

// Per-KV-head dynamic scale max(|x|) / 448 (floor 1e-12), the quantity the reference's
// fp8_scaled_quantize derives when no scale is given (kernels/cuda/fp8_scaled_quantize.cpp:38-42).
// scales[] is first cleared, then every workgroup folds a chunk of tokens of one head and
// publishes its candidate with an integer atomic maximum on the float's bits (all candidates are
// positive, so the bit patterns order like the values); dividing before or after the maximum gives
// the same float.
constexpr int kScaleChunk = 512;  // tokens per workgroup

__global__ void clear_scales_kernel(float* scales, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) scales[i] = 0.0f;
}

template <int IN>
__global__ __launch_bounds__(256) void kv_head_scales_kernel(const char* x, float* scales,
                                                             int64_t n_tokens, int head_dim,
                                                             int64_t stride_bytes, int vec_ok) {
  constexpr int ES = IN == 2 ? 4 : 2;
  const int h = blockIdx.y;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kScaleChunk;
  const int64_t t1 = min(n_tokens, t0 + kScaleChunk);
  const char* base = x + static_cast<int64_t>(h) * head_dim * ES;
  float amax = 0.0f;
  auto fold = [&](u32 w) {
    if constexpr (IN == 2) {
      amax = fmaxf(amax, fabsf(as_f32(w)));
    } else if constexpr (IN == 0) {
      amax = fmaxf(amax, fmaxf(fabsf(BF16::lo(w)), fabsf(BF16::hi(w))));
    } else {
      amax = fmaxf(amax, fmaxf(fabsf(FP16::lo(w)), fabsf(FP16::hi(w))));
    }
  };
  const int vpr = head_dim * ES / 16;  // 16-byte vectors per head row
  if (vec_ok && vpr <= 256) {
    const int v = threadIdx.x % vpr, tr = threadIdx.x / vpr, tpp = 256 / vpr;
    if (tr < tpp) {
      for (int64_t t = t0 + tr; t < t1; t += tpp) {
        const u32x4 w = ldg16(base + t * stride_bytes + v * 16);
        fold(w[0]);
        fold(w[1]);
        fold(w[2]);
        fold(w[3]);
      }
    }
  } else {
    for (int64_t t = t0; t < t1; ++t) {
      for (int d = threadIdx.x; d < head_dim; d += 256) {
        const char* p = base + t * stride_bytes + static_cast<int64_t>(d) * ES;
        float val;
        if constexpr (IN == 2) val = *reinterpret_cast<const float*>(p);
        else if constexpr (IN == 0) val = BF16::to_f32(*reinterpret_cast<const uint16_t*>(p));
        else val = FP16::to_f32(*reinterpret_cast<const uint16_t*>(p));
        amax = fmaxf(amax, fabsf(val));
      }
    }
  }
  __shared__ float red[256];
  red[threadIdx.x] = amax;
  __syncthreads();
  for (int st = 128; st > 0; st >>= 1) {
    if (threadIdx.x < st) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + st]);
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float cand = fmaxf(red[0] / 448.0f, 1e-12f);
    atomicMax(reinterpret_cast<unsigned int*>(scales + h), __float_as_uint(cand));
  }
}

template <int IN>
int launch_reshape(const ReshapeArgs& a, int64_t n_tokens, bool fp8, bool vec_ok, hipStream_t stream) {
  if (vec_ok) {
    const int n_work = a.n_vec * (a.value != nullptr ? 2 : 1);
    const unsigned gy = static_cast<unsigned>((n_work + 255) / 256);
    if (n_tokens >= kStreamTokens) {
      dim3 grid(static_cast<unsigned>((n_tokens + 3) / 4), gy);
      if (fp8) reshape_vec_kernel<IN, true, 4><<<grid, 256, 0, stream>>>(a);
      else reshape_vec_kernel<IN, false, 4><<<grid, 256, 0, stream>>>(a);
    } else {
      dim3 grid(static_cast<unsigned>(n_tokens), gy);
      if (fp8) reshape_vec_kernel<IN, true, 1><<<grid, 256, 0, stream>>>(a);
      else reshape_vec_kernel<IN, false, 1><<<grid, 256, 0, stream>>>(a);
    }
  } else {
    dim3 grid(static_cast<unsigned>(n_tokens));
    if (fp8) reshape_elem_kernel<IN, true><<<grid, 256, 0, stream>>>(a);
    else reshape_elem_kernel<IN, false><<<grid, 256, 0, stream>>>(a);
  }
  return static_cast<int>(hipGetLastError());
}

}  // namespace

int reshape_and_cache(const void* key, const void* value, void* k_cache, void* v_cache,
                      const int32_t* slot_mapping, const float* k_scale, const float* v_scale,
                      int64_t n_tokens, int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                      int64_t num_blocks, int64_t k_token_stride, int64_t v_token_stride,
                      int in_dtype, int cache_dtype, hipStream_t stream) {
  if (n_tokens == 0) return XLLM_MI355_OK;
  if (key == nullptr || k_cache == nullptr || slot_mapping == nullptr) return XLLM_MI355_EINVAL;
  if ((value == nullptr) != (v_cache == nullptr)) return XLLM_MI355_EINVAL;
  if (n_tokens < 0 || n_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 || num_blocks <= 0)
    return XLLM_MI355_EINVAL;
  if (in_dtype != XLLM_MI355_BF16 && in_dtype != XLLM_MI355_FP16 && in_dtype != XLLM_MI355_FP32)
    return XLLM_MI355_EDTYPE;
  const bool fp8 = cache_dtype == XLLM_MI355_FP8_E4M3;
  if (!fp8 && cache_dtype != in_dtype) return XLLM_MI355_EDTYPE;
  if (fp8 && (k_scale == nullptr || (value != nullptr && v_scale == nullptr))) return XLLM_MI355_EINVAL;
  const int64_t row = n_kv_heads * head_dim;
  if (k_token_stride < row || (value != nullptr && v_token_stride < row)) return XLLM_MI355_EINVAL;
  if (row > (1 << 24) || n_tokens > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  const int es = in_dtype == XLLM_MI355_FP32 ? 4 : 2;
  const int ces = fp8 ? 1 : es;

  ReshapeArgs a;
  a.key = static_cast<const char*>(key);
  a.value = static_cast<const char*>(value);
  a.k_cache = static_cast<char*>(k_cache);
  a.v_cache = static_cast<char*>(v_cache);
  a.slots = slot_mapping;
  a.k_scale = k_scale;
  a.v_scale = v_scale;
  a.k_stride_bytes = k_token_stride * es;
  a.v_stride_bytes = v_token_stride * es;
  a.n_slots = num_blocks * block_size;
  a.n_tokens = n_tokens;
  a.row_elems = static_cast<int>(row);
  a.head_dim = static_cast<int>(head_dim);
  a.n_vec = static_cast<int>(row * es / 16);

  auto aligned = [](const void* p, int64_t n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; };
  const int out_vec = 16 / es * ces;  // bytes each thread stores
  bool vec_ok = (head_dim * es) % 16 == 0 && aligned(key, 16) && a.k_stride_bytes % 16 == 0 &&
                aligned(k_cache, out_vec) && (row * ces) % out_vec == 0;
  if (value != nullptr)
    vec_ok = vec_ok && aligned(value, 16) && a.v_stride_bytes % 16 == 0 && aligned(v_cache, out_vec);
  if (a.n_vec * 2 > 65535 * 256) vec_ok = false;

  switch (in_dtype) {
    case XLLM_MI355_BF16: return launch_reshape<0>(a, n_tokens, fp8, vec_ok, stream);
    case XLLM_MI355_FP16: return launch_reshape<1>(a, n_tokens, fp8, vec_ok, stream);
    default: return launch_reshape<2>(a, n_tokens, fp8, vec_ok, stream);
  }
}

int kv_head_scales(const void* x, float* scales, int64_t n_tokens, int64_t n_kv_heads,
                   int64_t head_dim, int64_t token_stride, int in_dtype, hipStream_t stream) {
  if (x == nullptr || scales == nullptr || n_tokens <= 0 || n_kv_heads <= 0 || head_dim <= 0)
    return XLLM_MI355_EINVAL;
  if (token_stride < n_kv_heads * head_dim || n_kv_heads > 65535 || head_dim > (1 << 20))
    return XLLM_MI355_EINVAL;
  const char* p = static_cast<const char*>(x);
  const int es = in_dtype == XLLM_MI355_FP32 ? 4 : 2;
  const int vec_ok = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (token_stride * es) % 16 == 0 &&
                     (head_dim * es) % 16 == 0;
  clear_scales_kernel<<<dim3(static_cast<unsigned>((n_kv_heads + 255) / 256)), 256, 0, stream>>>(
      scales, static_cast<int>(n_kv_heads));
  dim3 grid(static_cast<unsigned>((n_tokens + kScaleChunk - 1) / kScaleChunk), static_cast<unsigned>(n_kv_heads));
  switch (in_dtype) {
    case XLLM_MI355_BF16:
      kv_head_scales_kernel<0><<<grid, 256, 0, stream>>>(p, scales, n_tokens, (int)head_dim, token_stride * 2, vec_ok);
      break;
    case XLLM_MI355_FP16:
      kv_head_scales_kernel<1><<<grid, 256, 0, stream>>>(p, scales, n_tokens, (int)head_dim, token_stride * 2, vec_ok);
      break;
    case XLLM_MI355_FP32:
      kv_head_scales_kernel<2><<<grid, 256, 0, stream>>>(p, scales, n_tokens, (int)head_dim, token_stride * 4, vec_ok);
      break;
    default: return XLLM_MI355_EDTYPE;
  }
  return static_cast<int>(hipGetLastError());
}

}  // namespace xllm_mi355
