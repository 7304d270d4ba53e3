// Shared device helpers of the gfx950 paged-KV decode kernels: element traits for the
// 16-bit query/cache types, fp8 e4m3fn conversions, DPP lane reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xllm_mi355 {

typedef uint32_t u32;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// "No score yet" marker of a running maximum.  Finite on purpose: exp2(-inf - kNegBig)
// is 0 and exp2(kNegBig - kNegBig) is 1, so a fully masked group needs no branch.
constexpr float kNegBig = -3.0e38f;

__device__ __forceinline__ u32 as_u32(float f) { return __builtin_bit_cast(u32, f); }
__device__ __forceinline__ float as_f32(u32 u) { return __builtin_bit_cast(float, u); }

// ---- 16-bit element traits -------------------------------------------------------------

struct BF16 {
  static constexpr bool kIsBf16 = true;
  // a.lo*b.lo + a.hi*b.hi + c with fp32 accumulation (v_dot2c_f32_bf16)
  static __device__ __forceinline__ float dot2(u32 a, u32 b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a),
                                           __builtin_bit_cast(bf16x2, b), c, false);
  }
  static __device__ __forceinline__ float lo(u32 a) { return as_f32(a << 16); }
  static __device__ __forceinline__ float hi(u32 a) { return as_f32(a & 0xffff0000u); }
  // round-to-nearest-even pack (v_cvt_pk_bf16_f32)
  static __device__ __forceinline__ u32 pack(float a, float b) {
    bf16x2 p = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(u32, p);
  }
  static __device__ __forceinline__ uint16_t from_f32(float a) {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(a));
  }
  static __device__ __forceinline__ float to_f32(uint16_t a) { return as_f32(static_cast<u32>(a) << 16); }
  // two e4m3fn codes (half-word `HI` of w) -> packed pair, exact
  template <bool HI>
  static __device__ __forceinline__ u32 from_fp8x2(u32 w) {
    return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, HI));
  }
};

struct FP16 {
  static constexpr bool kIsBf16 = false;
  static __device__ __forceinline__ float dot2(u32 a, u32 b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  }
  static __device__ __forceinline__ float lo(u32 a) {
    return static_cast<float>(__builtin_bit_cast(f16x2, a)[0]);
  }
  static __device__ __forceinline__ float hi(u32 a) {
    return static_cast<float>(__builtin_bit_cast(f16x2, a)[1]);
  }
  static __device__ __forceinline__ u32 pack(float a, float b) {
    f16x2 p = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
    return __builtin_bit_cast(u32, p);
  }
  static __device__ __forceinline__ uint16_t from_f32(float a) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(a));
  }
  static __device__ __forceinline__ float to_f32(uint16_t a) {
    return static_cast<float>(__builtin_bit_cast(_Float16, a));
  }
  template <bool HI>
  static __device__ __forceinline__ u32 from_fp8x2(u32 w) {
    return __builtin_bit_cast(u32, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, HI));
  }
};

// two e4m3fn codes (half-word `HI` of w) -> two fp32 (v_cvt_pk_f32_fp8)
template <bool HI>
__device__ __forceinline__ f32x2 fp8x2_to_f32(u32 w) {
  return __builtin_amdgcn_cvt_pk_f32_fp8(w, HI);
}

// fp32 -> e4m3fn code, round to nearest even, for |x| <= 448 (the caller clamps).
// Integer arithmetic only, so that the cache bytes do not depend on any hardware
// conversion mode: subnormal targets (|x| < 2^-6, quantum 2^-9) are rounded by the
// fp32 adder against 2^14, normal targets by the carry of 0x7ffff + odd bit.
__device__ __forceinline__ u32 f32_to_e4m3fn_rne(float x) {
  const u32 u = as_u32(x);
  const u32 sign = (u >> 24) & 0x80u;
  const u32 a = u & 0x7fffffffu;
  u32 r;
  if (a < 0x3c800000u) {
    r = as_u32(as_f32(a) + 16384.0f) - 0x46800000u;
  } else {
    r = a - 0x3c000000u;
    r = (r + 0x7ffffu + ((r >> 20) & 1u)) >> 20;
  }
  return sign | r;
}

// The reference's scaled fp8 conversion: clamp(x * inv_scale, +-448) then the cast.
// fminf/fmaxf return the non-NaN operand, so NaN quantises to +448 as in the reference.
__device__ __forceinline__ u32 fp8_quantize(float x, float inv_scale) {
  const float y = x * inv_scale;
  const float r = fmaxf(-448.0f, fminf(y, 448.0f));
  return f32_to_e4m3fn_rne(r);
}

// ---- DPP lane exchange ---------------------------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
  return as_f32(static_cast<u32>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(as_u32(x)), CTRL, 0xf, 0xf, false)));
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <- lane 7-i of its half row
constexpr int kDppMirror = 0x140;     // lane i <- lane 15-i of its row

// Sum over each aligned group of N lanes (N = 4, 8, 16, 32), result in every lane of the group.
template <int N>
__device__ __forceinline__ float group_sum(float x) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16 || N == 32, "group size");
  if constexpr (N >= 2) x += dpp<kDppXor1>(x);
  if constexpr (N >= 4) x += dpp<kDppXor2>(x);
  if constexpr (N >= 8) x += dpp<kDppHalfMirror>(x);
  if constexpr (N >= 16) x += dpp<kDppMirror>(x);
  if constexpr (N >= 32) {
    // v_permlane16_swap exchanges the odd rows of its first operand with the even rows
    // of its second: with both equal to x the two results add up to the sum of each row pair.
    auto r = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
    x = as_f32(r[0]) + as_f32(r[1]);
  }
  return x;
}

template <int N>
__device__ __forceinline__ float group_max(float x) {
  if constexpr (N >= 2) x = fmaxf(x, dpp<kDppXor1>(x));
  if constexpr (N >= 4) x = fmaxf(x, dpp<kDppXor2>(x));
  if constexpr (N >= 8) x = fmaxf(x, dpp<kDppHalfMirror>(x));
  if constexpr (N >= 16) x = fmaxf(x, dpp<kDppMirror>(x));
  if constexpr (N >= 32) {
    auto r = __builtin_amdgcn_permlane16_swap(as_u32(x), as_u32(x), false, false);
    x = fmaxf(as_f32(r[0]), as_f32(r[1]));
  }
  return x;
}

// ---- MFMA by element type --------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <typename QT>
struct Mfma;
// wait states between an MFMA written as inline assembly and the first instruction that reads its result
__device__ __forceinline__ void mfma_result_nops() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
template <>
struct Mfma<BF16> {
  // v_mfma_f32_16x16x32_bf16: 8 elements of A and of B per lane
  static __device__ __forceinline__ f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  // The same with the accumulator in ordinary vector registers, whatever form the compiler picks for its own
  // MFMAs (in a kernel with one wavefront per SIMD it puts every accumulator of the builtin into the 256
  // accumulation registers, which a kernel may need in full for other products).  The compiler does not know
  // this is an MFMA: the caller leaves kMfmaResultNops wait states before other instructions read the result.
  static __device__ __forceinline__ void k32_v(u32x4 a, u32x4 b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  // v_mfma_f32_16x16x16_bf16: 4 elements per lane
  static __device__ __forceinline__ f32x4 k16(s16x4 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
  // v_mfma_f32_32x32x16_bf16: 8 elements per lane, 16 accumulators
  static __device__ __forceinline__ f32x16 w32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<FP16> {
  static __device__ __forceinline__ f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void k32_v(u32x4 a, u32x4 b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ f32x4 k16(s16x4 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 w32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// 16-byte global load / store
__device__ __forceinline__ u32x4 ldg16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void stg16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
// The same for data that a launch reads once (rows of the paged caches): marked non-temporal, which on
// this GPU streams at 5.7-6.4 TB/s where a plain load of the same pattern reaches 5.0-5.7 TB/s.
__device__ __forceinline__ u32x4 ldg16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

}  // namespace xllm_mi355
