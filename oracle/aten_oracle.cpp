// aten_oracle.cpp -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// CPU restatement of the reference's libtorch implementations of the paged-KV
// decode path.  Each function issues the same ATen operators in the same order
// as the reference lines it names (paths relative to the xLLM source tree), on
// CPU tensors that wrap the caller's host buffers.  Only tests, the smoke run and
// the benchmark's CPU-baseline leg may load this library; nothing the product
// ships links to it.
//
// The C ABI below takes HOST pointers.  dtype codes: 0 bf16, 1 fp16, 2 fp32, 3 fp8 e4m3fn.
//
// How each function is pinned (tests/test_oracle_*.py): against the exact fp64
// softmax attention of paged_kv_oracle.c on seeded inputs (expected gap is the
// bf16 rounding of ATen's CPU SDPA, checked to be below 2e-3 max-abs), against the
// attention invariants (L = 1, equal rows, page permutation, head mapping), and
// against the known answers of DcpAttentionMergeTest for the merge.
#include <torch/torch.h>

#include <cmath>
#include <cstdint>
#include <limits>
#include <optional>
#include <vector>

namespace {

torch::ScalarType to_scalar_type(int dt) {
  switch (dt) {
    case 0: return torch::kBFloat16;
    case 1: return torch::kFloat16;
    case 2: return torch::kFloat32;
    default: return torch::kFloat8_e4m3fn;
  }
}

torch::Tensor wrap(const void* p, std::vector<int64_t> sizes, torch::ScalarType st) {
  return torch::from_blob(const_cast<void*>(p), sizes, torch::TensorOptions().dtype(st));
}

// expand_kv_heads, xllm/core/kernels/npu/utils.cpp:108-121.
torch::Tensor expand_kv_heads(const torch::Tensor& tensor, int64_t num_heads, int64_t num_kv_heads) {
  if (num_heads == num_kv_heads) return tensor;
  TORCH_CHECK(num_heads % num_kv_heads == 0, "num_heads must be divisible by num_kv_heads");
  const int64_t expansion_factor = num_heads / num_kv_heads;
  return tensor.unsqueeze(2)
      .expand({tensor.size(0), num_kv_heads, expansion_factor, tensor.size(2)})
      .reshape({tensor.size(0), num_heads, tensor.size(2)});
}

// fp8 pages -> query dtype: float(code) * scale[h], then cast.  The reference has
// no fp8 KV read path; this is the rule of its int8 path, which dequantises the
// paged K/V to the query dtype before ordinary attention
// (xllm/core/layers/mlu/attention.cpp:171-222) with fp32 scales
// (xllm/core/kernels/mlu/mlu_ops_api.h:67-71).
torch::Tensor dequant_pages(const torch::Tensor& pages /*[n,bs,Hkv,D] fp8*/, const torch::Tensor& scale /*[Hkv]*/,
                            torch::ScalarType out_type) {
  return (pages.to(torch::kFloat32) * scale.view({1, 1, -1, 1})).to(out_type);
}

}  // namespace

extern "C" {

int aten_oracle_num_threads() { return at::get_num_threads(); }
void aten_oracle_set_num_threads(int n) { at::set_num_threads(n); }

// Block-table paged decode.  Follows ascend950_paged_attention,
// xllm/core/kernels/npu/attention.cpp:26-78, line for line: per sequence
// narrow(block_table row) -> int64 -> index_select pages -> reshape -> narrow(L)
// -> expand_kv_heads -> scaled_dot_product_attention(scale) -> copy_ into output.
// v_cache == nullptr: V is the first dv dims of the K pages (MLA; the boundary of
// xllm/core/kernels/dcu/flash_mla_adapter.h:40-53 with semantics pinned by
// tests/core/layers/mlu/dcp_attention_merge_test.cpp:77-144).
// out: [B, Hq, dv] in q_dtype.
int aten_paged_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                      const int32_t* block_table, int64_t table_stride, const int32_t* seq_lens,
                      const float* k_scale, const float* v_scale, int64_t batch, int64_t n_q_heads,
                      int64_t n_kv_heads, int64_t dqk, int64_t dv, int64_t block_size,
                      int64_t num_blocks, float scale, int q_dtype, int cache_dtype) {
  torch::NoGradGuard no_grad;
  const auto qt = to_scalar_type(q_dtype);
  const auto ct = to_scalar_type(cache_dtype);
  const torch::Tensor query = wrap(q, {batch, n_q_heads, dqk}, qt);
  const torch::Tensor kc = wrap(k_cache, {num_blocks, block_size, n_kv_heads, dqk}, ct);
  torch::Tensor vc;
  if (v_cache != nullptr) vc = wrap(v_cache, {num_blocks, block_size, n_kv_heads, dv}, ct);
  const torch::Tensor table = wrap(block_table, {batch, table_stride}, torch::kInt32);
  const torch::Tensor seq_lens_cpu = wrap(seq_lens, {batch}, torch::kInt32);
  torch::Tensor output = wrap(out, {batch, n_q_heads, dv}, qt);
  torch::Tensor ks, vs;
  if (cache_dtype == 3) {
    ks = wrap(k_scale, {n_kv_heads}, torch::kFloat32);
    if (v_cache != nullptr) vs = wrap(v_scale, {n_kv_heads}, torch::kFloat32);
  }

  for (int64_t batch_index = 0; batch_index < batch; ++batch_index) {
    const int64_t seq_len = seq_lens_cpu[batch_index].item<int64_t>();
    if (seq_len <= 0) return -1;  // the reference CHECK_GT(seq_len, 0)
    const int64_t n_blocks = (seq_len + block_size - 1) / block_size;
    torch::Tensor block_indices = table[batch_index].narrow(0, 0, n_blocks);
    block_indices = block_indices.to(torch::kInt64);

    torch::Tensor kpages = kc.index_select(0, block_indices);
    if (cache_dtype == 3) kpages = dequant_pages(kpages, ks, qt);
    torch::Tensor key = kpages.reshape({n_blocks * block_size, n_kv_heads, dqk}).narrow(0, 0, seq_len);
    torch::Tensor value;
    if (v_cache != nullptr) {
      torch::Tensor vpages = vc.index_select(0, block_indices);
      if (cache_dtype == 3) vpages = dequant_pages(vpages, vs, qt);
      value = vpages.reshape({n_blocks * block_size, n_kv_heads, dv}).narrow(0, 0, seq_len);
    } else {
      value = key.narrow(2, 0, dv);
    }
    key = expand_kv_heads(key, n_q_heads, n_kv_heads);
    value = expand_kv_heads(value, n_q_heads, n_kv_heads);

    const torch::Tensor query_4d = query[batch_index].unsqueeze(0).unsqueeze(2);
    const torch::Tensor key_4d = key.permute({1, 0, 2}).unsqueeze(0);
    const torch::Tensor value_4d = value.permute({1, 0, 2}).unsqueeze(0);
    const torch::Tensor sequence_output =
        torch::scaled_dot_product_attention(query_4d, key_4d, value_4d,
                                            /*attn_mask=*/std::nullopt,
                                            /*dropout_p=*/0.0,
                                            /*is_causal=*/false,
                                            /*scale=*/static_cast<double>(scale))
            .squeeze(0)
            .squeeze(1);
    output[batch_index].copy_(sequence_output);
  }
  return 0;
}

// CSR paged decode.  Follows the decode branch of TorchAttentionImpl::forward,
// xllm/core/layers/dcu/torch_attention.cpp:285-347 with expand_kv_for_mqa (:40-65)
// and compute_attention (:67-110): per sequence narrow each page (the last one to
// last_page_len), cat, expand KV heads, SDPA with NO scale argument (ATen's default
// 1/sqrt(D)).  Pages with an index >= num_blocks are skipped as in the reference.
int aten_paged_decode_csr(const void* q, const void* k_cache, const void* v_cache, void* out,
                          const int32_t* indptr, const int32_t* indices, const int32_t* last_page_len,
                          int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t head_dim,
                          int64_t block_size, int64_t num_blocks, int q_dtype) {
  torch::NoGradGuard no_grad;
  const auto qt = to_scalar_type(q_dtype);
  const torch::Tensor query = wrap(q, {batch, n_q_heads, head_dim}, qt);
  const torch::Tensor kc = wrap(k_cache, {num_blocks, block_size, n_kv_heads, head_dim}, qt);
  const torch::Tensor vc = wrap(v_cache, {num_blocks, block_size, n_kv_heads, head_dim}, qt);
  torch::Tensor output = wrap(out, {batch, n_q_heads, head_dim}, qt);
  const int64_t expansion_factor = n_q_heads / n_kv_heads;

  for (int64_t i = 0; i < batch; ++i) {
    std::vector<torch::Tensor> kv_pages_k, kv_pages_v;
    const int64_t page_start = indptr[i];
    const int64_t page_end = indptr[i + 1];
    for (int64_t p = page_start; p < page_end; ++p) {
      const int64_t page_idx = indices[p];
      if (page_idx < num_blocks) {
        const int64_t n = (p == page_end - 1) ? last_page_len[i] : block_size;
        kv_pages_k.push_back(kc[page_idx].narrow(0, 0, n));
        kv_pages_v.push_back(vc[page_idx].narrow(0, 0, n));
      }
    }
    if (kv_pages_k.empty()) return -1;  // the reference falls back to the new token's K/V here
    torch::Tensor full_k = torch::cat(kv_pages_k, 0);
    torch::Tensor full_v = torch::cat(kv_pages_v, 0);
    if (n_kv_heads != n_q_heads) {
      const int64_t seq_len = full_k.size(0);
      full_k = full_k.unsqueeze(2)
                   .expand({seq_len, n_kv_heads, expansion_factor, head_dim})
                   .reshape({seq_len, n_q_heads, head_dim});
      full_v = full_v.unsqueeze(2)
                   .expand({seq_len, n_kv_heads, expansion_factor, head_dim})
                   .reshape({seq_len, n_q_heads, head_dim});
    }
    torch::Tensor q_seq = query.slice(0, i, i + 1);
    torch::Tensor query_4d = q_seq.unsqueeze(0).permute({0, 2, 1, 3});
    torch::Tensor key_4d = full_k.unsqueeze(0).permute({0, 2, 1, 3});
    torch::Tensor value_4d = full_v.unsqueeze(0).permute({0, 2, 1, 3});
    torch::Tensor attn_output = at::scaled_dot_product_attention(query_4d, key_4d, value_4d,
                                                                 std::nullopt,
                                                                 /*dropout_p=*/0.0,
                                                                 /*is_causal=*/false);
    output.slice(0, i, i + 1).copy_(attn_output.permute({0, 2, 1, 3}).squeeze(0));
  }
  return 0;
}

// LSE of a paged decode in fp32: logsumexp(q . k^T * scale, -1), the expected value
// of MluMlaDecodeLseTest (tests/core/layers/mlu/dcp_attention_merge_test.cpp:127-143).
// lse: [B, Hq] fp32.
int aten_paged_decode_lse(const void* q, const void* k_cache, float* lse, const int32_t* block_table,
                          int64_t table_stride, const int32_t* seq_lens, const float* k_scale,
                          int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t dqk,
                          int64_t block_size, int64_t num_blocks, float scale, int q_dtype,
                          int cache_dtype) {
  torch::NoGradGuard no_grad;
  const auto qt = to_scalar_type(q_dtype);
  const auto ct = to_scalar_type(cache_dtype);
  const torch::Tensor query = wrap(q, {batch, n_q_heads, dqk}, qt);
  const torch::Tensor kc = wrap(k_cache, {num_blocks, block_size, n_kv_heads, dqk}, ct);
  const torch::Tensor table = wrap(block_table, {batch, table_stride}, torch::kInt32);
  torch::Tensor out = wrap(lse, {batch, n_q_heads}, torch::kFloat32);
  torch::Tensor ks;
  if (cache_dtype == 3) ks = wrap(k_scale, {n_kv_heads}, torch::kFloat32);
  for (int64_t b = 0; b < batch; ++b) {
    const int64_t seq_len = seq_lens[b];
    if (seq_len <= 0) return -1;
    const int64_t n_blocks = (seq_len + block_size - 1) / block_size;
    torch::Tensor block_indices = table[b].narrow(0, 0, n_blocks).to(torch::kInt64);
    torch::Tensor kpages = kc.index_select(0, block_indices);
    if (cache_dtype == 3) kpages = dequant_pages(kpages, ks, qt);
    torch::Tensor keys_float = expand_kv_heads(
        kpages.reshape({n_blocks * block_size, n_kv_heads, dqk}).narrow(0, 0, seq_len),
        n_q_heads, n_kv_heads).to(torch::kFloat32);                 // [L, Hq, D]
    torch::Tensor query_float = query[b].to(torch::kFloat32);       // [Hq, D]
    torch::Tensor scores = torch::einsum("hd,lhd->hl", {query_float, keys_float}) * scale;
    out[b].copy_(torch::logsumexp(scores, /*dim=*/-1));
  }
  return 0;
}

// merge_dcp_attention_shards, xllm/core/layers/mlu/dcp_attention_merge.cpp:26-65, with
// the [dcp, batch, query, heads, value] / [dcp, batch, heads, query] shapes of the
// reference at query = 1.  partial_out [S,B,H,Dv] of dtype, partial_lse [S,B,H] fp32.
int aten_lse_merge(const void* partial_out, const float* partial_lse, void* out, float* lse_out,
                   int64_t n_shards, int64_t batch, int64_t n_heads, int64_t dv, int dtype) {
  torch::NoGradGuard no_grad;
  const auto st = to_scalar_type(dtype);
  const torch::Tensor partial_outputs = wrap(partial_out, {n_shards, batch, 1, n_heads, dv}, st);
  const torch::Tensor partial_lse_t = wrap(partial_lse, {n_shards, batch, n_heads, 1}, torch::kFloat32);

  torch::Tensor lse = partial_lse_t.to(torch::kFloat32);
  torch::Tensor max_lse = std::get<0>(lse.max(/*dim=*/0, /*keepdim=*/true));
  torch::Tensor has_finite_shard = torch::isfinite(max_lse);
  torch::Tensor safe_max_lse = torch::where(has_finite_shard, max_lse, torch::zeros_like(max_lse));
  torch::Tensor weights =
      torch::where(torch::isfinite(lse), torch::exp(lse - safe_max_lse), torch::zeros_like(lse));
  torch::Tensor weight_sum = weights.sum(/*dim=*/0);
  torch::Tensor safe_weight_sum =
      torch::where(weight_sum > 0, weight_sum, torch::ones_like(weight_sum));
  torch::Tensor weighted_output =
      (partial_outputs.to(torch::kFloat32) * weights.unsqueeze(/*dim=*/2)).sum(/*dim=*/0);
  torch::Tensor has_output = (weight_sum > 0).unsqueeze(/*dim=*/1);
  torch::Tensor output = torch::where(has_output,
                                      weighted_output / safe_weight_sum.unsqueeze(/*dim=*/1),
                                      torch::zeros_like(weighted_output));
  const float negative_infinity = -std::numeric_limits<float>::infinity();
  torch::Tensor merged_lse =
      torch::where(weight_sum > 0, safe_max_lse.squeeze(/*dim=*/0) + torch::log(safe_weight_sum),
                   torch::full_like(weight_sum, negative_infinity));
  wrap(out, {batch, 1, n_heads, dv}, st).copy_(output.to(st));
  if (lse_out != nullptr) wrap(lse_out, {batch, n_heads, 1}, torch::kFloat32).copy_(merged_lse);
  return 0;
}

// fp8 store convention in ATen form: (float(x) * (1.0f / scale[h])) clamped to +-448,
// cast to float8_e4m3fn (xllm/core/kernels/cuda/fp8_quant.cu:92-103).  Used only to
// cross-check the C oracle's encoder on finite inputs; for NaN the reference's
// fminf/fmaxf give +448 while at::clamp propagates NaN.
int aten_fp8_quantize(const void* x, uint8_t* out, const float* scale, int64_t n_tokens,
                      int64_t n_kv_heads, int64_t head_dim, int in_dtype) {
  torch::NoGradGuard no_grad;
  const torch::Tensor xt = wrap(x, {n_tokens, n_kv_heads, head_dim}, to_scalar_type(in_dtype));
  const torch::Tensor st = wrap(scale, {n_kv_heads}, torch::kFloat32);
  const torch::Tensor inv = torch::reciprocal(st).view({1, -1, 1});
  const torch::Tensor q = (xt.to(torch::kFloat32) * inv).clamp(-448.0, 448.0).to(torch::kFloat8_e4m3fn);
  wrap(out, {n_tokens, n_kv_heads, head_dim}, torch::kFloat8_e4m3fn).copy_(q);
  return 0;
}

}  // extern "C"
