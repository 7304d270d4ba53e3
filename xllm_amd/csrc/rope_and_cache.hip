// Per-head RMS norm + rotary embedding of the q and k heads of a fused qkv buffer, in place, and -- in the
// same launch, when a paged cache is given -- the cache write of the new k and v rows.
//
// Replaces xllm::kernel::cuda::fused_qk_norm_rope (xllm/core/kernels/cuda/fused_qknorm_rope.cu:79-300,
// caller xllm/core/layers/common/qwen2_attention.cpp:144-186) and, with the cache arguments, the
// reshape_paged_cache call that follows it (xllm/core/kernels/cuda/reshape_paged_cache.cu:23-63): at decode
// both are launch bound, one launch does the work of two.
//
// Arithmetic of the reference kernel: everything in fp32 between one load and one store --
//   y = x * rsqrt(mean(x^2) + eps) * weight          (weights of the qkv dtype, one set for q, one for k)
//   rotary_dim leading dims rotated by the cos | sin row of the token's position, either
//     interleaved  (y[2i], y[2i+1]) -> (y[2i] c_i - y[2i+1] s_i, y[2i] s_i + y[2i+1] c_i)
//     or split     (y[i], y[i+h])   -> (y[i] c_i - y[i+h] s_i,  y[i+h] c_i + y[i] s_i),  h = rotary_dim / 2
//   rounded once to the qkv dtype.
// The cache receives the rounded k (the bits that were just stored in place) and the untouched v, quantised
// with the per-head scales when the cache is fp8 -- exactly what reshape_and_cache would write from the
// buffer afterwards.
//
// Mapping: 32 lanes per (token, head), two heads per wavefront; a lane owns head_dim / 32 consecutive
// dims (2, 4 or 8: one 4-, 8- or 16-byte load).  Sum of squares by DPP within the 32 lanes; the partner of
// the split form is (rotary_dim / 2) / (head_dim / 32) lanes away.
#include "common.cuh"
#include "launch.h"

namespace xllm_mi355 {

namespace {

struct RopeArgs {
  char* qkv;
  const char* q_weight;
  const char* k_weight;
  const char* cos_sin;
  const int64_t* positions;
  char* k_cache;
  char* v_cache;
  const int32_t* slots;
  const float* k_scale;
  const float* v_scale;
  int64_t token_stride_bytes;
  int64_t n_units;   // tokens * heads handled per token
  int64_t n_slots;   // P * block_size
  float eps;
  int n_q, n_k, n_v;
  int rotary_dim;
  int heads_per_token;  // n_q + n_k (+ n_v with a cache)
  int norm;             // 0: no RMS norm (weights absent)
};

// cos / sin caches come in fp32 or in a 16-bit type.  N consecutive entries from index i on, with one
// vector load (two for 8 fp32 entries): i is a multiple of N and the rows of the cache start at multiples
// of 2 N entries, so the load is aligned whenever the cache itself is 16-byte aligned.  Entry by entry
// these loads were most of the kernel's memory instructions.
template <int CT, int N>
__device__ __forceinline__ void cache_vec(const char* p, int64_t i, float (&out)[N]) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8, "entries per lane");
  if constexpr (CT == XLLM_MI355_FP32) {
    const float* f = reinterpret_cast<const float*>(p) + i;
    if constexpr (N == 1) {
      out[0] = f[0];
    } else if constexpr (N == 2) {
      const f32x2 v = *reinterpret_cast<const f32x2*>(f);
      out[0] = v[0];
      out[1] = v[1];
    } else {
#pragma unroll
      for (int k = 0; k < N / 4; ++k) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(f + 4 * k);
#pragma unroll
        for (int j = 0; j < 4; ++j) out[4 * k + j] = v[j];
      }
    }
  } else {
    uint16_t h[N];
    const uint16_t* q = reinterpret_cast<const uint16_t*>(p) + i;
    if constexpr (N == 1) h[0] = q[0];
    else if constexpr (N == 2) *reinterpret_cast<u32*>(h) = *reinterpret_cast<const u32*>(q);
    else if constexpr (N == 4) *reinterpret_cast<u32x2*>(h) = *reinterpret_cast<const u32x2*>(q);
    else *reinterpret_cast<u32x4*>(h) = *reinterpret_cast<const u32x4*>(q);
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = CT == XLLM_MI355_BF16 ? BF16::to_f32(h[j]) : FP16::to_f32(h[j]);
  }
}

__device__ __forceinline__ float lane_xor(float x, int mask, int lane) {
  return as_f32(static_cast<u32>(__builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, static_cast<int>(as_u32(x)))));
}

// U = (token, head) units per 32-lane group.  With one unit a lane has 4 to 16 bytes in flight, which at
// prefill sizes leaves the launch bound by memory latency; with four consecutive units (adjacent heads of a
// token: adjacent rows) the loads of all four are issued before the first is used.  SAME: the heads of a token are a
// multiple of U, so the units of a group belong to one token: its position, its slot and its cos | sin entries are
// fetched once for the group instead of once per unit (they were 3 of a unit's 4 loads and two thirds of its bytes).
template <typename QT, int D, int CT, bool INTERLEAVE, bool FP8, int U, bool SAME = false>
__global__ __launch_bounds__(256) void rope_and_cache_kernel(RopeArgs a) {
  constexpr int E = D / 32;  // dims per lane
  const int lane = threadIdx.x & 63;
  const int sub = lane & 31;
  const int64_t unit0 = ((static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) >> 5) * U;
  const int half = a.rotary_dim >> 1;
  const int rotary_lanes = a.rotary_dim / E;
  const bool rotated = sub < rotary_lanes;

  bool on[U], is_q[U], is_v[U];  // (lanes past the end keep running: the exchanges below are wave wide)
  int64_t token[U];
  int head[U];
  char* row[U];
  uint16_t raw[U][E];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t unit = unit0 + u;
    on[u] = unit < a.n_units;
    token[u] = on[u] ? unit / a.heads_per_token : 0;
    head[u] = on[u] ? static_cast<int>(unit - token[u] * a.heads_per_token) : 0;
    is_q[u] = head[u] < a.n_q;
    is_v[u] = head[u] >= a.n_q + a.n_k;
    row[u] = a.qkv + token[u] * a.token_stride_bytes + (static_cast<int64_t>(head[u]) * D + sub * E) * 2;
    if constexpr (E == 2) *reinterpret_cast<u32*>(raw[u]) = *reinterpret_cast<const u32*>(row[u]);
    else if constexpr (E == 4) *reinterpret_cast<u32x2*>(raw[u]) = *reinterpret_cast<const u32x2*>(row[u]);
    else *reinterpret_cast<u32x4*>(raw[u]) = *reinterpret_cast<const u32x4*>(row[u]);
  }
  int64_t cs[U];
  int64_t slot[U];
  if constexpr (SAME) {
    const int64_t cs0 = (on[0] ? a.positions[token[0]] : 0) * a.rotary_dim;
    const int64_t slot0 = a.k_cache != nullptr && on[0] ? a.slots[token[0]] : -1;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      cs[u] = cs0;
      slot[u] = on[u] && !is_q[u] ? slot0 : -1;
    }
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      cs[u] = (on[u] ? a.positions[token[u]] : 0) * a.rotary_dim;
      slot[u] = a.k_cache != nullptr && on[u] && !is_q[u] ? a.slots[token[u]] : -1;
    }
  }
  // cos | sin of the lane's dims: c[u][i], sn[u][i] belong to pair i of the interleaved form, to dim i of the split form
  constexpr int NC = INTERLEAVE ? E / 2 : E;
  constexpr int UC = SAME ? 1 : U;   // (one set for the group when its units share a token: a set per unit costs the
                                     // registers that decide how many wavefronts a SIMD holds)
  float c[UC][NC], sn[UC][NC];
  // the lane's dims lie on one side of the split form (rotary_dim / 2 is a multiple of E)
  const int j0 = INTERLEAVE ? (sub * E) / 2 : (sub * E < half ? sub * E : sub * E - half);
  // (lanes and units that are not rotated never look at their entries: the rotation below is under the same conditions)
#pragma unroll
  for (int u = 0; u < UC; ++u) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      c[u][i] = 1.0f;
      sn[u][i] = 0.0f;
    }
    // (SAME: the row of the token's position exists whatever the units' kinds)
    if (rotated && (SAME || !is_v[u])) {
      cache_vec<CT, NC>(a.cos_sin, cs[u] + j0, c[u]);
      cache_vec<CT, NC>(a.cos_sin, cs[u] + half + j0, sn[u]);
    }
  }

  // the lane's norm weights, once for the group (the q set and the k set)
  float wq[E], wk[E];
  if (a.norm != 0) {
    const uint16_t* q = reinterpret_cast<const uint16_t*>(a.q_weight) + sub * E;
    const uint16_t* k = reinterpret_cast<const uint16_t*>(a.k_weight) + sub * E;
    uint16_t hq[E], hk[E];
    if constexpr (E == 2) {
      *reinterpret_cast<u32*>(hq) = *reinterpret_cast<const u32*>(q);
      *reinterpret_cast<u32*>(hk) = *reinterpret_cast<const u32*>(k);
    } else if constexpr (E == 4) {
      *reinterpret_cast<u32x2*>(hq) = *reinterpret_cast<const u32x2*>(q);
      *reinterpret_cast<u32x2*>(hk) = *reinterpret_cast<const u32x2*>(k);
    } else {
      *reinterpret_cast<u32x4*>(hq) = *reinterpret_cast<const u32x4*>(q);
      *reinterpret_cast<u32x4*>(hk) = *reinterpret_cast<const u32x4*>(k);
    }
#pragma unroll
    for (int i = 0; i < E; ++i) {
      wq[i] = QT::to_f32(hq[i]);
      wk[i] = QT::to_f32(hk[i]);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float x[E];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < E; ++i) {
      x[i] = QT::to_f32(raw[u][i]);
      ss += x[i] * x[i];
    }
    ss = group_sum<32>(ss);
    if (!is_v[u] && a.norm != 0) {
      const float r = __builtin_amdgcn_rsqf(ss / static_cast<float>(D) + a.eps);
#pragma unroll
      for (int i = 0; i < E; ++i) x[i] *= r * (is_q[u] ? wq[i] : wk[i]);
    }
    // rotary embedding of the leading rotary_dim dims
    const int uc = SAME ? 0 : u;
    if constexpr (INTERLEAVE) {
      if (!is_v[u] && rotated) {
#pragma unroll
        for (int i = 0; i < E / 2; ++i) {
          // (the fused multiply-adds spelled out: left to the compiler, the instantiations for decode and prefill sizes
          // rounded differently in the last bit)
          const float e = x[2 * i], o = x[2 * i + 1];
          x[2 * i] = __builtin_fmaf(e, c[uc][i], -(o * sn[uc][i]));
          x[2 * i + 1] = __builtin_fmaf(e, sn[uc][i], o * c[uc][i]);
        }
      }
    } else {
      const int pair = half / E;  // lanes between a dim and its partner
      float other[E];
#pragma unroll
      for (int i = 0; i < E; ++i) other[i] = lane_xor(x[i], pair, lane);
      if (!is_v[u] && rotated) {
#pragma unroll
        for (int i = 0; i < E; ++i) {
          const int d = sub * E + i;
          x[i] = __builtin_fmaf(x[i], c[uc][i], (d < half ? -other[i] : other[i]) * sn[uc][i]);
        }
      }
    }
    if (!on[u]) continue;

    if (!is_v[u]) {
#pragma unroll
      for (int i = 0; i < E; ++i) raw[u][i] = QT::from_f32(x[i]);
      if constexpr (E == 2) *reinterpret_cast<u32*>(row[u]) = *reinterpret_cast<const u32*>(raw[u]);
      else if constexpr (E == 4) *reinterpret_cast<u32x2*>(row[u]) = *reinterpret_cast<const u32x2*>(raw[u]);
      else *reinterpret_cast<u32x4*>(row[u]) = *reinterpret_cast<const u32x4*>(raw[u]);
    }
    if (a.k_cache == nullptr || is_q[u]) continue;

    // cache write of the k head (the bits just stored) or the v head (as loaded)
    if (slot[u] < 0 || slot[u] >= a.n_slots) continue;
    const int kvh = is_v[u] ? head[u] - a.n_q - a.n_k : head[u] - a.n_q;
    const int n_kv = is_v[u] ? a.n_v : a.n_k;
    const int64_t e0 = (slot[u] * n_kv + kvh) * D + sub * E;
    char* dst = (is_v[u] ? a.v_cache : a.k_cache);
    if constexpr (FP8) {
      const float inv = 1.0f / (is_v[u] ? a.v_scale : a.k_scale)[kvh];
      uint8_t code[E];
#pragma unroll
      for (int i = 0; i < E; ++i) code[i] = static_cast<uint8_t>(fp8_quantize(QT::to_f32(raw[u][i]), inv));
      if constexpr (E == 2) *reinterpret_cast<uint16_t*>(dst + e0) = *reinterpret_cast<const uint16_t*>(code);
      else if constexpr (E == 4) *reinterpret_cast<u32*>(dst + e0) = *reinterpret_cast<const u32*>(code);
      else *reinterpret_cast<u32x2*>(dst + e0) = *reinterpret_cast<const u32x2*>(code);
    } else {
      if constexpr (E == 2) *reinterpret_cast<u32*>(dst + e0 * 2) = *reinterpret_cast<const u32*>(raw[u]);
      else if constexpr (E == 4) *reinterpret_cast<u32x2*>(dst + e0 * 2) = *reinterpret_cast<const u32x2*>(raw[u]);
      else *reinterpret_cast<u32x4*>(dst + e0 * 2) = *reinterpret_cast<const u32x4*>(raw[u]);
    }
  }
}

template <typename QT, int D, int CT, int U>
int launch_rope_units(const RopeArgs& a, bool interleave, bool fp8, hipStream_t stream) {
  const int64_t threads = (a.n_units + U - 1) / U * 32;
  const dim3 grid(static_cast<unsigned>((threads + 255) / 256));
  // (the units of a group belong to one token when a token's heads are a multiple of the group's units)
  const bool same = U > 1 && a.heads_per_token % U == 0;
#define XLLM_ROPE_LAUNCH(IL, F8)                                                                      \
  do {                                                                                                \
    if (same) rope_and_cache_kernel<QT, D, CT, IL, F8, U, (U > 1)><<<grid, 256, 0, stream>>>(a);      \
    else rope_and_cache_kernel<QT, D, CT, IL, F8, U, false><<<grid, 256, 0, stream>>>(a);             \
  } while (0)
  if (interleave) {
    if (fp8) XLLM_ROPE_LAUNCH(true, true);
    else XLLM_ROPE_LAUNCH(true, false);
  } else {
    if (fp8) XLLM_ROPE_LAUNCH(false, true);
    else XLLM_ROPE_LAUNCH(false, false);
  }
#undef XLLM_ROPE_LAUNCH
  return static_cast<int>(hipGetLastError());
}

template <typename QT, int D, int CT>
int launch_rope(const RopeArgs& a, bool interleave, bool fp8, hipStream_t stream) {
  // one unit per group while that still gives every CU several workgroups (decode), four beyond (eight, with the
  // registers they take, measured slower: 57.7 us against 50.3 us on 8192 tokens of 48 heads; sixteen lanes of 16 bytes
  // per unit instead of 32 of 8 at head dim 128: the same 47.3 us)
  if (a.n_units * 32 / 256 < 8192) return launch_rope_units<QT, D, CT, 1>(a, interleave, fp8, stream);
  return launch_rope_units<QT, D, CT, 4>(a, interleave, fp8, stream);
}

template <typename QT, int D>
int dispatch_cache_type(const RopeArgs& a, int cos_sin_dtype, bool interleave, bool fp8, hipStream_t stream) {
  switch (cos_sin_dtype) {
    case XLLM_MI355_FP32: return launch_rope<QT, D, XLLM_MI355_FP32>(a, interleave, fp8, stream);
    case XLLM_MI355_BF16: return launch_rope<QT, D, XLLM_MI355_BF16>(a, interleave, fp8, stream);
    case XLLM_MI355_FP16: return launch_rope<QT, D, XLLM_MI355_FP16>(a, interleave, fp8, stream);
    default: return XLLM_MI355_EDTYPE;
  }
}

template <typename QT>
int dispatch_head_dim(const RopeArgs& a, int64_t head_dim, int cos_sin_dtype, bool interleave, bool fp8,
                      hipStream_t stream) {
  switch (head_dim) {
    case 64: return dispatch_cache_type<QT, 64>(a, cos_sin_dtype, interleave, fp8, stream);
    case 128: return dispatch_cache_type<QT, 128>(a, cos_sin_dtype, interleave, fp8, stream);
    case 256: return dispatch_cache_type<QT, 256>(a, cos_sin_dtype, interleave, fp8, stream);
    default: return XLLM_MI355_ESHAPE;
  }
}

}  // namespace

int rope_and_cache(void* qkv, const void* q_weight, const void* k_weight, const void* cos_sin_cache,
                   const int64_t* position_ids, void* k_cache, void* v_cache, const int32_t* slot_mapping,
                   const float* k_scale, const float* v_scale, int64_t n_tokens, int64_t token_stride,
                   int64_t n_heads_q, int64_t n_heads_k, int64_t n_heads_v, int64_t head_dim, int64_t rotary_dim,
                   float eps, int interleave, int64_t block_size, int64_t num_blocks, int dtype, int cos_sin_dtype,
                   int cache_dtype, hipStream_t stream) {
  if (n_tokens == 0) return XLLM_MI355_OK;
  if (qkv == nullptr || cos_sin_cache == nullptr || position_ids == nullptr) return XLLM_MI355_EINVAL;
  if ((q_weight == nullptr) != (k_weight == nullptr)) return XLLM_MI355_EINVAL;
  if (n_tokens < 0 || n_heads_q <= 0 || n_heads_k <= 0 || n_heads_v < 0) return XLLM_MI355_EINVAL;
  if (dtype != XLLM_MI355_BF16 && dtype != XLLM_MI355_FP16) return XLLM_MI355_EDTYPE;
  const int64_t dims_per_lane = head_dim / 32;
  // the reference's conditions (fused_qknorm_rope.cu:150-153, 420-440): an even number of dims per lane,
  // the rotated lanes a power of two so that a dim's partner is a fixed number of lanes away
  if (rotary_dim <= 0 || rotary_dim > head_dim || rotary_dim % (2 * dims_per_lane) != 0) return XLLM_MI355_ESHAPE;
  const int64_t rotary_lanes = rotary_dim / (dims_per_lane > 0 ? dims_per_lane : 1);
  if (interleave == 0 && (rotary_lanes & (rotary_lanes - 1)) != 0) return XLLM_MI355_ESHAPE;
  if (token_stride < (n_heads_q + n_heads_k + n_heads_v) * head_dim) return XLLM_MI355_EINVAL;
  if (((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(cos_sin_cache)) & 15) != 0 || (token_stride * 2) % 16 != 0)
    return XLLM_MI355_EALIGN;
  // (a lane reads its head_dim / 32 norm weights with one vector load)
  if (q_weight != nullptr &&
      ((reinterpret_cast<uintptr_t>(q_weight) | reinterpret_cast<uintptr_t>(k_weight)) & 15) != 0)
    return XLLM_MI355_EALIGN;
  const bool with_cache = k_cache != nullptr;
  const bool fp8 = with_cache && cache_dtype == XLLM_MI355_FP8_E4M3;
  if (with_cache) {
    if (v_cache == nullptr || slot_mapping == nullptr || n_heads_v != n_heads_k || block_size <= 0 || num_blocks <= 0)
      return XLLM_MI355_EINVAL;
    if (!fp8 && cache_dtype != dtype) return XLLM_MI355_EDTYPE;
    if (fp8 && (k_scale == nullptr || v_scale == nullptr)) return XLLM_MI355_EINVAL;
    if (((reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15) != 0) return XLLM_MI355_EALIGN;
  }
  RopeArgs a = {};
  a.qkv = static_cast<char*>(qkv);
  a.q_weight = static_cast<const char*>(q_weight);
  a.k_weight = static_cast<const char*>(k_weight);
  a.cos_sin = static_cast<const char*>(cos_sin_cache);
  a.positions = position_ids;
  a.k_cache = static_cast<char*>(k_cache);
  a.v_cache = static_cast<char*>(v_cache);
  a.slots = slot_mapping;
  a.k_scale = k_scale;
  a.v_scale = v_scale;
  a.token_stride_bytes = token_stride * 2;
  a.n_slots = with_cache ? num_blocks * block_size : 0;
  a.eps = eps;
  a.n_q = static_cast<int>(n_heads_q);
  a.n_k = static_cast<int>(n_heads_k);
  a.n_v = static_cast<int>(n_heads_v);
  a.rotary_dim = static_cast<int>(rotary_dim);
  a.heads_per_token = static_cast<int>(n_heads_q + n_heads_k + (with_cache ? n_heads_v : 0));
  a.n_units = n_tokens * a.heads_per_token;
  a.norm = q_weight != nullptr ? 1 : 0;
  if (a.n_units * 32 / 256 > 0x7fffffffLL) return XLLM_MI355_ESHAPE;
  return dtype == XLLM_MI355_BF16
             ? dispatch_head_dim<BF16>(a, head_dim, cos_sin_dtype, interleave != 0, fp8, stream)
             : dispatch_head_dim<FP16>(a, head_dim, cos_sin_dtype, interleave != 0, fp8, stream);
}

}  // namespace xllm_mi355
