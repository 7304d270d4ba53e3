/*
 * paged_kv_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain-C CPU restatement of the reference's paged-KV decode path, used only as
 * the checker in tests, in the smoke run and as a timed CPU baseline.  Nothing
 * the library ships may call into this file.
 *
 * Each function names the reference lines it follows (paths relative to the
 * xLLM source tree).  Byte- and index-exact parts (scatter, fp8 encode, block
 * table build) are restated exactly; the attention itself is restated as the
 * textbook fp64 softmax attention (the pattern of decode_attention_reference,
 * tests/core/kernels/npu/npu_xllm_ops_test.cpp:109-125) so that it can pin the
 * ATen-op-order oracle in aten_oracle.cpp, which is the one that follows
 * xllm/core/kernels/npu/attention.cpp:26-78 call for call.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   fp8 encode/decode   all 256 codes round-trip; exhaustive 65536 bf16 patterns
 *                       and random fp32 against torch's float8_e4m3fn cast;
 *                       special cases 0, -0, +-448, 2^-9, 2^-10 ties, NaN.
 *   reshape_and_cache   closed form (a permutation copy): the reference tests'
 *                       five shape cases and the 130-token/128-block case.
 *   decode (fp64)       invariants L=1, equal K rows, equal V rows, page
 *                       permutation, head mapping; logsumexp closed form.
 *   lse_merge           the three known answers of DcpAttentionMergeTest and
 *                       merge(split) == unsplit.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { DT_BF16 = 0, DT_FP16 = 1, DT_FP32 = 2, DT_FP8_E4M3 = 3 };

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- scalar format conversions ------------------------------------------------ */

float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even, NaN kept quiet. */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float oracle_fp16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * (1.0f / 16777216.0f);
    return bits_f32(f32_bits(v) | sign);
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> fp16, round to nearest even (overflow -> inf). */
uint16_t oracle_f32_to_fp16(float f) {
  uint32_t u = f32_bits(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (65520 rounds up below) */
  if (a < 0x38800000u) { /* below 2^-14: subnormal half */
    /* add 0.5f so that the fp32 adder performs the RNE at 2^-24 granularity */
    float t = bits_f32(a) + 0.5f;
    return (uint16_t)(sign | (f32_bits(t) - 0x3f000000u));
  }
  uint32_t r = a - 0x38000000u; /* rebias 127 -> 15 */
  r += 0xfffu + ((r >> 13) & 1u);
  r >>= 13;
  if (r >= 0x7c00u) r = 0x7c00u;
  return (uint16_t)(sign | r);
}

/*
 * e4m3fn (OCP, 1-4-3, bias 7, no inf, 0x7f/0xff = NaN, max 448), decode.
 */
float oracle_e4m3fn_to_f32(uint8_t c) {
  uint32_t sign = (uint32_t)(c & 0x80u) << 24;
  uint32_t exp = (c >> 3) & 0xfu;
  uint32_t man = c & 0x7u;
  if (exp == 0xfu && man == 0x7u) return bits_f32(sign | 0x7fc00000u);
  if (exp == 0) {
    float v = (float)man * (1.0f / 512.0f); /* man * 2^-9 */
    return bits_f32(f32_bits(v) | sign);
  }
  return bits_f32(sign | ((exp + 120u) << 23) | (man << 20));
}

/*
 * fp32 -> e4m3fn, round to nearest even; magnitudes that round above 448 and
 * NaN give the NaN code 0x7f (what a plain cast does; the quantiser below clamps
 * first, so it never reaches that branch).
 */
uint8_t oracle_f32_to_e4m3fn(float f) {
  uint32_t u = f32_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  /* 464 is the midpoint of 448 (even code 0x7e) and the NaN code's would-be value 480:
     the tie goes to 448, anything above it has no finite code. */
  if (a > 0x43e80000u) return (uint8_t)(sign | 0x7fu);
  if (a < 0x3c800000u) { /* < 2^-6: subnormal target, quantum 2^-9 */
    /* adding 2^14 (ulp = 2^-9) makes the fp32 adder round to the quantum, RNE */
    float t = bits_f32(a) + 16384.0f;
    return (uint8_t)(sign | (uint8_t)(f32_bits(t) - 0x46800000u));
  }
  uint32_t r = a - 0x3c000000u; /* rebias 127 -> 7 */
  r += 0x7ffffu + ((r >> 20) & 1u);
  return (uint8_t)(sign | (uint8_t)(r >> 20));
}

/*
 * The reference's scaled fp8 conversion with saturation,
 * scaled_fp8_conversion<true, e4m3fn> (kernels/cuda/fp8_quant_utils.cuh:111-130)
 * called with inv_scale = 1.0f / scale (kernels/cuda/fp8_quant.cu:92-103):
 *   x = val * inv_scale; r = fmaxf(-448, fminf(x, 448)); cast r.
 * fminf/fmaxf return the non-NaN operand, so a NaN input quantises to +448.
 */
uint8_t oracle_fp8_quantize(float val, float inv_scale) {
  float x = val * inv_scale;
  float r = fmaxf(-448.0f, fminf(x, 448.0f));
  return oracle_f32_to_e4m3fn(r);
}

static float load_as_f32(const void* p, int64_t i, int dt) {
  switch (dt) {
    case DT_BF16: return oracle_bf16_to_f32(((const uint16_t*)p)[i]);
    case DT_FP16: return oracle_fp16_to_f32(((const uint16_t*)p)[i]);
    case DT_FP32: return ((const float*)p)[i];
    default: return oracle_e4m3fn_to_f32(((const uint8_t*)p)[i]);
  }
}

static int esize(int dt) { return dt == DT_FP32 ? 4 : (dt == DT_FP8_E4M3 ? 1 : 2); }

/* ---- op 1: reshape_and_cache ------------------------------------------------------ */

/*
 * Follows reshape_paged_cache_kernel (kernels/cuda/reshape_paged_cache.cu:23-63) and
 * reference_reshape_paged_cache (tests/core/kernels/dcu/reshape_paged_cache_test.cpp:34-51):
 * token t goes to page slot/bs, row slot%bs; negative slots are skipped; K and V
 * have independent token strides.  value/v_cache may be NULL (MLA latent store,
 * layers/dcu/deepseek_v2_attention.cpp:221-229).  With an fp8 cache each element is
 * quantised with the per-KV-head scale by oracle_fp8_quantize.
 * Returns 0, or -1 on an unsupported dtype pair.
 */
int oracle_reshape_and_cache(const void* key, const void* value, void* k_cache, void* v_cache,
                             const int32_t* slot_mapping, const float* k_scale,
                             const float* v_scale, int64_t n_tokens, int64_t n_kv_heads,
                             int64_t head_dim, int64_t block_size, int64_t num_blocks,
                             int64_t k_token_stride, int64_t v_token_stride, int in_dtype,
                             int cache_dtype) {
  const int64_t row = n_kv_heads * head_dim;
  if (cache_dtype != in_dtype && cache_dtype != DT_FP8_E4M3) return -1;
  if (in_dtype == DT_FP8_E4M3) return -1;
  for (int64_t t = 0; t < n_tokens; ++t) {
    const int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_blocks * block_size) continue;
    const int64_t block_idx = slot / block_size;
    const int64_t block_off = slot % block_size;
    const int64_t dst = (block_idx * block_size + block_off) * row;
    for (int pass = 0; pass < 2; ++pass) {
      const void* src = pass == 0 ? key : value;
      void* cache = pass == 0 ? k_cache : v_cache;
      const float* scale = pass == 0 ? k_scale : v_scale;
      const int64_t stride = pass == 0 ? k_token_stride : v_token_stride;
      if (src == NULL || cache == NULL) continue;
      if (cache_dtype == in_dtype) {
        const int es = esize(in_dtype);
        memcpy((char*)cache + dst * es, (const char*)src + t * stride * es, (size_t)(row * es));
      } else {
        for (int64_t h = 0; h < n_kv_heads; ++h) {
          const float inv_scale = 1.0f / scale[h];
          for (int64_t d = 0; d < head_dim; ++d) {
            const float x = load_as_f32(src, t * stride + h * head_dim + d, in_dtype);
            ((uint8_t*)cache)[dst + h * head_dim + d] = oracle_fp8_quantize(x, inv_scale);
          }
        }
      }
    }
  }
  return 0;
}

/*
 * scale[h] = max(absmax / 448, 1e-12) in fp32: the dynamic branch of
 * fp8_scaled_quantize (kernels/cuda/fp8_scaled_quantize.cpp:38-42) per KV head.
 */
void oracle_kv_head_scales(const void* x, float* scales, int64_t n_tokens, int64_t n_kv_heads,
                           int64_t head_dim, int64_t token_stride, int in_dtype) {
  for (int64_t h = 0; h < n_kv_heads; ++h) {
    float amax = 0.0f;
    for (int64_t t = 0; t < n_tokens; ++t)
      for (int64_t d = 0; d < head_dim; ++d) {
        const float a = fabsf(load_as_f32(x, t * token_stride + h * head_dim + d, in_dtype));
        if (a > amax) amax = a;
      }
    const float s = amax / 448.0f;
    scales[h] = s < 1e-12f ? 1e-12f : s;
  }
}

/* ---- op 2: paged decode attention, exact-arithmetic form ------------------------------ */

/*
 * Textbook softmax attention over block-table-addressed pages, accumulated in
 * fp64.  Addressing follows ascend950_paged_attention
 * (kernels/npu/attention.cpp:26-78): sequence b reads ceil(L/bs) table entries,
 * token t lives at page table[b][t/bs], row t%bs; query head h reads KV head
 * h / (Hq/Hkv) (expand_kv_heads, kernels/npu/utils.cpp:108-121).
 * v_cache == NULL means V = first dv dims of K (MLA,
 * tests/core/layers/mlu/dcp_attention_merge_test.cpp:77-144).
 * fp8 caches are dequantised as float(code) * scale[h], rounded to the query
 * dtype (the int8 precedent of layers/mlu/attention.cpp:171-222) when
 * round_dequant != 0.
 * out: [B, Hq, dv] fp32; lse: [B, Hq] fp32 natural log (may be NULL).
 */
int oracle_paged_decode_f64(const void* q, const void* k_cache, const void* v_cache, float* out,
                            float* lse, const int32_t* block_table, int64_t table_stride,
                            const int32_t* seq_lens, const float* k_scale, const float* v_scale,
                            int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t dqk,
                            int64_t dv, int64_t block_size, double sm_scale, int q_dtype,
                            int cache_dtype, int round_dequant) {
  if (n_q_heads % n_kv_heads != 0) return -1;
  const int64_t group = n_q_heads / n_kv_heads;
  const int64_t krow = n_kv_heads * dqk;
  const int64_t vrow = v_cache ? n_kv_heads * dv : krow;
  const void* vsrc = v_cache ? v_cache : k_cache;
  const int64_t vdim = v_cache ? dv : dqk;
  for (int64_t b = 0; b < batch; ++b) {
    const int64_t L = seq_lens[b];
    double* s = (double*)malloc(sizeof(double) * (size_t)(L > 0 ? L : 1));
    double* acc = (double*)malloc(sizeof(double) * (size_t)dv);
    for (int64_t h = 0; h < n_q_heads; ++h) {
      const int64_t kvh = h / group;
      float* o = out + (b * n_q_heads + h) * dv;
      if (L <= 0) {
        for (int64_t d = 0; d < dv; ++d) o[d] = 0.0f;
        if (lse) lse[b * n_q_heads + h] = -INFINITY;
        continue;
      }
      double m = -INFINITY;
      for (int64_t t = 0; t < L; ++t) {
        const int64_t page = block_table[b * table_stride + t / block_size];
        const int64_t base = (page * block_size + t % block_size) * krow + kvh * dqk;
        double dot = 0.0;
        for (int64_t d = 0; d < dqk; ++d) {
          float kf = load_as_f32(k_cache, base + d, cache_dtype);
          if (cache_dtype == DT_FP8_E4M3) {
            kf = kf * k_scale[kvh];
            if (round_dequant)
              kf = q_dtype == DT_FP16 ? oracle_fp16_to_f32(oracle_f32_to_fp16(kf))
                                      : oracle_bf16_to_f32(oracle_f32_to_bf16(kf));
          }
          dot += (double)load_as_f32(q, (b * n_q_heads + h) * dqk + d, q_dtype) * (double)kf;
        }
        s[t] = dot * sm_scale;
        if (s[t] > m) m = s[t];
      }
      double l = 0.0;
      for (int64_t d = 0; d < dv; ++d) acc[d] = 0.0;
      for (int64_t t = 0; t < L; ++t) {
        const double p = exp(s[t] - m);
        l += p;
        const int64_t page = block_table[b * table_stride + t / block_size];
        const int64_t base = (page * block_size + t % block_size) * vrow + kvh * vdim;
        for (int64_t d = 0; d < dv; ++d) {
          float vf = load_as_f32(vsrc, base + d, cache_dtype);
          if (cache_dtype == DT_FP8_E4M3) {
            vf = vf * (v_cache ? v_scale[kvh] : k_scale[kvh]);
            if (round_dequant)
              vf = q_dtype == DT_FP16 ? oracle_fp16_to_f32(oracle_f32_to_fp16(vf))
                                      : oracle_bf16_to_f32(oracle_f32_to_bf16(vf));
          }
          acc[d] += p * (double)vf;
        }
      }
      for (int64_t d = 0; d < dv; ++d) o[d] = (float)(acc[d] / l);
      if (lse) lse[b * n_q_heads + h] = (float)(m + log(l));
    }
    free(s);
    free(acc);
  }
  return 0;
}

/* ---- LSE merge ------------------------------------------------------------------ */

/*
 * Follows merge_dcp_attention_shards (layers/mlu/dcp_attention_merge.cpp:26-65) in
 * fp32, step for step: max over shards; non-finite max -> 0; weights = exp(lse -
 * max) for finite lse else 0; out = sum w o / sum w (0 when sum w == 0); lse = max
 * + log(sum w) (-inf when sum w == 0).
 * partial_out [S, B, H, Dv] fp32, partial_lse [S, B, H], out [B, H, Dv], lse [B, H].
 */
void oracle_lse_merge(const float* partial_out, const float* partial_lse, float* out, float* lse,
                      int64_t n_shards, int64_t batch, int64_t n_heads, int64_t dv) {
  const int64_t bh = batch * n_heads;
  for (int64_t i = 0; i < bh; ++i) {
    float mx = -INFINITY;
    for (int64_t s = 0; s < n_shards; ++s) {
      const float v = partial_lse[s * bh + i];
      if (v > mx) mx = v;
    }
    const float safe_max = isfinite(mx) ? mx : 0.0f;
    float wsum = 0.0f;
    for (int64_t d = 0; d < dv; ++d) out[i * dv + d] = 0.0f;
    for (int64_t s = 0; s < n_shards; ++s) {
      const float v = partial_lse[s * bh + i];
      const float w = isfinite(v) ? expf(v - safe_max) : 0.0f;
      wsum += w;
      for (int64_t d = 0; d < dv; ++d) out[i * dv + d] += partial_out[(s * bh + i) * dv + d] * w;
    }
    if (wsum > 0.0f) {
      for (int64_t d = 0; d < dv; ++d) out[i * dv + d] /= wsum;
      if (lse) lse[i] = safe_max + logf(wsum);
    } else {
      for (int64_t d = 0; d < dv; ++d) out[i * dv + d] = 0.0f;
      if (lse) lse[i] = -INFINITY;
    }
  }
}

/*
 * Follows lse_combine_kernel (kernels/cuda/xattention/lse_combine.cu:41-85) in fp32, step for step, with the
 * LSEs in base 2: max; exp2 of both against it; merged = max + log2(sum); weights exp2(lse - merged);
 * out = w_shared * shared_o + w_unshared * unshared_o.  All arrays fp32: shared_o / unshared_o / out [rows, d],
 * the LSEs [rows].  The reference writes no merged LSE; `merged` (may be null) receives it for the tests.
 */
void oracle_lse_combine(float* out, float* merged, const float* shared_o, const float* shared_lse,
                        const float* unshared_o, const float* unshared_lse, int64_t rows, int64_t d) {
  for (int64_t i = 0; i < rows; ++i) {
    const float a = shared_lse[i], b = unshared_lse[i];
    const float lse_max = fmaxf(a, b);
    const float ea = exp2f(a - lse_max), eb = exp2f(b - lse_max);
    const float lse_new = lse_max + log2f(ea + eb);
    const float wa = exp2f(a - lse_new), wb = exp2f(b - lse_new);
    for (int64_t k = 0; k < d; ++k) out[i * d + k] = wa * shared_o[i * d + k] + wb * unshared_o[i * d + k];
    if (merged) merged[i] = lse_new;
  }
}

/* ---- CSR -> block table ------------------------------------------------------------ */

/*
 * Follows build_block_table_kernel (kernels/dcu/build_block_table_from_paged_kv.hip:44-149):
 * -1 fill, then row b receives its pages.  seq_lens[b] = (pages-1)*bs + last_page_len[b].
 */
void oracle_build_block_table(const int32_t* indptr, const int32_t* indices,
                              const int32_t* last_page_len, int32_t* block_table,
                              int64_t table_stride, int32_t* seq_lens, int64_t batch,
                              int64_t block_size) {
  for (int64_t b = 0; b < batch; ++b) {
    const int64_t n = indptr[b + 1] - indptr[b];
    for (int64_t j = 0; j < table_stride; ++j)
      block_table[b * table_stride + j] = j < n ? indices[indptr[b] + j] : -1;
    if (seq_lens) seq_lens[b] = n > 0 ? (int32_t)((n - 1) * block_size + last_page_len[b]) : 0;
  }
}

/*
 * mask_block_table_padding (layers/dcu/flash_attention.cpp:194-218): page_counts = (len + bs - 1) / bs;
 * columns j >= page_counts[b] become -1, the others keep their value.
 */
void oracle_mask_block_table_padding(const int32_t* block_table, int64_t table_stride,
                                     const int32_t* kv_seq_lens, int32_t* out, int64_t batch,
                                     int64_t width, int64_t block_size) {
  for (int64_t b = 0; b < batch; ++b) {
    const int64_t pages = ((int64_t)kv_seq_lens[b] + block_size - 1) / block_size;
    for (int64_t j = 0; j < width; ++j)
      out[b * width + j] = j >= pages ? -1 : block_table[b * table_stride + j];
  }
}

/*
 * Rows of paged sequences -> packed buffer (kernels/dcu/gather_mla_latent_cache.hip:32-75): for every sequence b
 * and token t < cu[b+1] - cu[b], out row cu[b] + t = cache row block_table[b, t / bs] * bs + t % bs; rows with a
 * negative page id are skipped (the reference's `physical_block < 0` return), and so are ids beyond the cache.
 */
void oracle_gather_paged_rows(const uint8_t* cache, const int32_t* block_table, int64_t table_stride,
                              const int32_t* cu_seq_lens, uint8_t* out, int64_t batch, int64_t block_size,
                              int64_t num_blocks, int64_t row_bytes) {
  for (int64_t b = 0; b < batch; ++b) {
    const int64_t n = (int64_t)cu_seq_lens[b + 1] - cu_seq_lens[b];
    for (int64_t t = 0; t < n; ++t) {
      const int64_t page = block_table[b * table_stride + t / block_size];
      if (page < 0 || page >= num_blocks) continue;
      const uint8_t* from = cache + (page * block_size + t % block_size) * row_bytes;
      uint8_t* to = out + ((int64_t)cu_seq_lens[b] + t) * row_bytes;
      for (int64_t i = 0; i < row_bytes; ++i) to[i] = from[i];
    }
  }
}
