// See ops_api.h.  Host code only: it unpacks torch::Tensor arguments, checks what the
// reference checks, fetches the current HIP stream from PyTorch and calls the C ABI.
#include "ops_api.h"

#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <mutex>
#include <unordered_map>

#include "../../../include/xllm_mi355.h"

namespace {

int dtype_code(const torch::Tensor& t) {
  switch (t.scalar_type()) {
    case torch::kBFloat16: return XLLM_MI355_BF16;
    case torch::kFloat16: return XLLM_MI355_FP16;
    case torch::kFloat32: return XLLM_MI355_FP32;
    case torch::kFloat8_e4m3fn:
    case torch::kUInt8: return XLLM_MI355_FP8_E4M3;
    default: TORCH_CHECK(false, "unsupported dtype ", t.scalar_type()); return -1;
  }
}

void* current_stream(const torch::Tensor& t) {
  return c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void check_rc(int rc, const char* what) {
  TORCH_CHECK(rc == 0, what, " failed with code ", rc, ": ", xllm_mi355_error_string(rc));
}

const void* ptr_or_null(const std::optional<torch::Tensor>& t) {
  return t.has_value() && t->defined() ? t->data_ptr() : nullptr;
}

void reshape_impl(xllm::kernel::ReshapePagedCacheParams& p, bool quantized) {
  TORCH_CHECK(!p.direction, "CACHE2CONTEXT is not part of the decode path");
  const torch::Tensor& key = p.key;
  TORCH_CHECK(key.is_cuda() && key.dim() == 3, "key must be a device tensor [T, Hkv, D]");
  TORCH_CHECK(key.stride(-1) == 1 && key.stride(-2) == key.size(-1), "key: last two dims must be contiguous");
  const bool has_v = p.value.has_value() && p.value->defined();
  TORCH_CHECK(has_v == (p.v_cache.has_value() && p.v_cache->defined()), "value and v_cache go together");
  if (has_v) {
    TORCH_CHECK(p.value->stride(-1) == 1 && p.value->stride(-2) == p.value->size(-1) &&
                    p.value->sizes() == key.sizes(),
                "value: last two dims must be contiguous and the shape must match key");
  }
  TORCH_CHECK(p.k_cache.is_cuda() && p.k_cache.dim() == 4 && p.k_cache.is_contiguous(),
              "k_cache must be a contiguous device tensor [P, bs, Hkv, D]");
  TORCH_CHECK(p.k_cache.size(2) == key.size(1) && p.k_cache.size(3) == key.size(2),
              "k_cache heads / head_dim do not match key");
  if (has_v) {
    TORCH_CHECK(p.v_cache->is_cuda() && p.v_cache->is_contiguous() && p.v_cache->sizes() == p.k_cache.sizes() &&
                    p.v_cache->scalar_type() == p.k_cache.scalar_type() && p.value->scalar_type() == key.scalar_type(),
                "v_cache must match k_cache in shape and dtype (contiguous), value must match key in dtype");
  }
  TORCH_CHECK(p.slot_mapping.is_cuda(), "slot_mapping must be a device tensor");
  TORCH_CHECK(p.slot_mapping.scalar_type() == torch::kInt32 && p.slot_mapping.is_contiguous() &&
                  p.slot_mapping.numel() == key.size(0),
              "slot_mapping must be contiguous int32 [T]");
  if (quantized) {
    TORCH_CHECK(p.k_cache_scale.has_value() && p.k_cache_scale->defined(),
                "k_cache_scale is required for quant_to_paged_cache");
    TORCH_CHECK(!has_v || (p.v_cache_scale.has_value() && p.v_cache_scale->defined()),
                "v_cache_scale is required with a v_cache");
    for (const std::optional<torch::Tensor>* s : {&p.k_cache_scale, &p.v_cache_scale}) {
      if (!s->has_value() || !(*s)->defined()) continue;
      TORCH_CHECK((*s)->is_cuda() && (*s)->scalar_type() == torch::kFloat32 && (*s)->is_contiguous() &&
                      (*s)->numel() == key.size(1),
                  "cache scales must be contiguous fp32 device tensors [Hkv]");
    }
    TORCH_CHECK(p.k_cache.scalar_type() == torch::kFloat8_e4m3fn || p.k_cache.scalar_type() == torch::kUInt8,
                "quant_to_paged_cache writes an fp8 e4m3fn (or uint8) cache");
  } else {
    TORCH_CHECK(p.k_cache.scalar_type() == key.scalar_type(), "key and k_cache must have the same dtype");
  }
  const int rc = xllm_mi355_reshape_and_cache(
      key.data_ptr(), has_v ? p.value->data_ptr() : nullptr, p.k_cache.data_ptr(),
      has_v ? p.v_cache->data_ptr() : nullptr, p.slot_mapping.data_ptr<int32_t>(),
      quantized ? static_cast<const float*>(ptr_or_null(p.k_cache_scale)) : nullptr,
      quantized ? static_cast<const float*>(ptr_or_null(p.v_cache_scale)) : nullptr, key.size(0), key.size(1),
      key.size(2), p.k_cache.size(1), p.k_cache.size(0), key.stride(0), has_v ? p.value->stride(0) : 0,
      dtype_code(key), dtype_code(p.k_cache), current_stream(key));
  check_rc(rc, "xllm_mi355_reshape_and_cache");
}

// What every GQA decode entry needs of its operands before their pointers reach a kernel.
void check_decode_operands(const torch::Tensor& query, const torch::Tensor& output, const torch::Tensor& k_cache,
                           const torch::Tensor& v_cache, const std::optional<torch::Tensor>& k_scale,
                           const std::optional<torch::Tensor>& v_scale) {
  TORCH_CHECK(query.is_cuda() && query.dim() == 3, "query must be a device tensor [B, Hq, D]");
  TORCH_CHECK(query.stride(-1) == 1 && query.stride(-2) == query.size(-1), "query: last two dims must be contiguous");
  TORCH_CHECK(output.is_cuda() && output.sizes() == query.sizes() && output.scalar_type() == query.scalar_type(),
              "output must be a device tensor of query's shape and dtype");
  TORCH_CHECK(output.stride(-1) == 1 && output.stride(-2) == output.size(-1), "output: last two dims must be contiguous");
  TORCH_CHECK(k_cache.is_cuda() && k_cache.dim() == 4 && k_cache.is_contiguous(),
              "k_cache must be a contiguous device tensor [P, bs, Hkv, D]");
  TORCH_CHECK(v_cache.is_cuda() && v_cache.is_contiguous() && v_cache.sizes() == k_cache.sizes() &&
                  v_cache.scalar_type() == k_cache.scalar_type(),
              "v_cache must match k_cache in shape and dtype, contiguous");
  TORCH_CHECK(k_cache.size(3) == query.size(2) && k_cache.size(2) > 0 && query.size(1) % k_cache.size(2) == 0,
              "cache head_dim / KV heads do not match query");
  const bool fp8 = k_cache.scalar_type() == torch::kFloat8_e4m3fn || k_cache.scalar_type() == torch::kUInt8;
  if (fp8) {
    for (const std::optional<torch::Tensor>* s : {&k_scale, &v_scale})
      TORCH_CHECK(s->has_value() && (*s)->defined() && (*s)->is_cuda() && (*s)->scalar_type() == torch::kFloat32 &&
                      (*s)->is_contiguous() && (*s)->numel() == k_cache.size(2),
                  "an fp8 cache needs contiguous fp32 device scales [Hkv] for K and V");
  } else {
    TORCH_CHECK(k_cache.scalar_type() == query.scalar_type(), "cache dtype must equal the query dtype (or be fp8)");
  }
}

}  // namespace

namespace xllm::kernel {

void reshape_paged_cache(ReshapePagedCacheParams& params) { reshape_impl(params, false); }
void quant_to_paged_cache(ReshapePagedCacheParams& params) { reshape_impl(params, true); }

namespace mi355 {

torch::Tensor decode_workspace(const torch::Device& device, size_t nbytes) {
  static std::mutex mu;
  static std::unordered_map<int, torch::Tensor> ws;
  std::lock_guard<std::mutex> lock(mu);
  torch::Tensor& t = ws[device.index()];
  if (!t.defined()) {
    // once per device, at the library's bound over every supported shape, and never replaced: a launch
    // recorded in a HIP graph keeps the address it was captured with
    const size_t want = std::max<size_t>(nbytes, xllm_mi355_decode_workspace_bound());
    t = torch::empty({static_cast<int64_t>(want)}, torch::TensorOptions().dtype(torch::kUInt8).device(device));
    check_rc(xllm_mi355_decode_workspace_init(t.data_ptr(), want, c10::hip::getCurrentHIPStream(device.index()).stream()),
             "xllm_mi355_decode_workspace_init");
  }
  TORCH_CHECK(static_cast<size_t>(t.numel()) >= nbytes, "the decode workspace of device ", device.index(), " holds ",
              t.numel(), " bytes and ", nbytes,
              " are needed: it cannot grow once handed out (captured graphs hold its address); call "
              "decode_workspace(device, nbytes) with the largest need before the first decode call");
  return t;
}

void decode_status(const torch::Device& device) {
  torch::Tensor ws = decode_workspace(device, 0);
  check_rc(xllm_mi355_decode_status(ws.data_ptr(), c10::hip::getCurrentHIPStream(device.index()).stream()),
           "xllm_mi355_decode_status");
}

void batch_decode(const torch::Tensor& query, const torch::Tensor& k_cache, torch::Tensor& output,
                  const torch::Tensor& block_table, const torch::Tensor& seq_lens,
                  const std::optional<torch::Tensor>& v_cache, std::optional<torch::Tensor>& output_lse,
                  const std::optional<torch::Tensor>& k_cache_quant_scale,
                  const std::optional<torch::Tensor>& v_cache_quant_scale, int64_t max_seq_len,
                  int64_t window_size_left, float scale, bool return_lse, const std::optional<torch::Tensor>& plan,
                  const NewKvRows* fresh) {
  TORCH_CHECK(v_cache.has_value() && v_cache->defined(), "GQA decode needs v_cache");
  check_decode_operands(query, output, k_cache, *v_cache, k_cache_quant_scale, v_cache_quant_scale);
  TORCH_CHECK(block_table.scalar_type() == torch::kInt32 && block_table.dim() == 2 && block_table.stride(1) == 1 &&
                  block_table.size(0) == query.size(0),
              "block_table must be int32 [B, W]");
  TORCH_CHECK(seq_lens.scalar_type() == torch::kInt32 && seq_lens.is_contiguous() && seq_lens.numel() == query.size(0),
              "seq_lens must be contiguous int32 [B]");
  const int64_t B = query.size(0), Hq = query.size(1), D = query.size(2);
  if (return_lse && !(output_lse.has_value() && output_lse->defined()))
    output_lse = torch::empty({B, Hq, 1}, query.options().dtype(torch::kFloat32));
  float* lse = nullptr;
  if (output_lse.has_value() && output_lse->defined()) {
    TORCH_CHECK(output_lse->scalar_type() == torch::kFloat32 && output_lse->is_contiguous() &&
                    output_lse->numel() == B * Hq,
                "output_lse must be contiguous fp32 [B, Hq, 1]");
    lse = output_lse->data_ptr<float>();
  }
  if (max_seq_len <= 0) max_seq_len = block_table.size(1) * k_cache.size(1);
  const size_t nbytes = xllm_mi355_paged_decode_gqa_workspace_bytes(B, Hq, D);
  torch::Tensor ws = decode_workspace(query.device(), nbytes);
  const bool planned = plan.has_value() && plan->defined();
  if (planned)
    TORCH_CHECK(plan->is_cuda() && plan->is_contiguous() && plan->scalar_type() == torch::kUInt8 &&
                    static_cast<size_t>(plan->numel()) >= xllm_mi355_paged_decode_plan_bytes(),
                "plan must be the buffer of update_decode_plan (uint8, xllm_mi355_paged_decode_plan_bytes() bytes)");
  if (fresh != nullptr) {
    for (const torch::Tensor* t : {&fresh->key, &fresh->value})
      TORCH_CHECK(t->is_cuda() && t->dim() == 3 && t->size(0) == B && t->size(1) == k_cache.size(2) && t->size(2) == D &&
                      t->stride(2) == 1 && t->stride(1) == D && t->scalar_type() == query.scalar_type(),
                  "the step's key / value must be device tensors [B, Hkv, D] of the query's dtype, tokens contiguous");
    TORCH_CHECK(fresh->slot_mapping.is_cuda() && fresh->slot_mapping.scalar_type() == torch::kInt32 &&
                    fresh->slot_mapping.is_contiguous() && fresh->slot_mapping.numel() == B,
                "slot_mapping must be contiguous int32 [B]");
    const int rc = xllm_mi355_write_and_decode_gqa(
        fresh->key.data_ptr(), fresh->value.data_ptr(), fresh->slot_mapping.data_ptr<int32_t>(), fresh->key.stride(0),
        fresh->value.stride(0), planned ? plan->data_ptr() : nullptr, planned ? static_cast<size_t>(plan->numel()) : 0,
        query.data_ptr(), k_cache.data_ptr(), v_cache->data_ptr(), output.data_ptr(), lse,
        block_table.data_ptr<int32_t>(), block_table.stride(0), seq_lens.data_ptr<int32_t>(), nullptr, nullptr, nullptr,
        static_cast<const float*>(ptr_or_null(k_cache_quant_scale)),
        static_cast<const float*>(ptr_or_null(v_cache_quant_scale)), B, Hq, k_cache.size(2), D, k_cache.size(1),
        k_cache.size(0), query.stride(0), output.stride(0), max_seq_len, window_size_left, scale, ws.data_ptr(),
        static_cast<size_t>(ws.numel()), dtype_code(query), dtype_code(k_cache), current_stream(query));
    check_rc(rc, "xllm_mi355_write_and_decode_gqa");
    return;
  }
  if (planned) {
    const int rc = xllm_mi355_paged_decode_gqa_planned(
        plan->data_ptr(), static_cast<size_t>(plan->numel()), query.data_ptr(), k_cache.data_ptr(), v_cache->data_ptr(), output.data_ptr(), lse,
        block_table.data_ptr<int32_t>(), block_table.stride(0), seq_lens.data_ptr<int32_t>(), nullptr, nullptr, nullptr,
        static_cast<const float*>(ptr_or_null(k_cache_quant_scale)),
        static_cast<const float*>(ptr_or_null(v_cache_quant_scale)), B, Hq, k_cache.size(2), D, k_cache.size(1),
        k_cache.size(0), query.stride(0), output.stride(0), max_seq_len, window_size_left, scale, ws.data_ptr(),
        static_cast<size_t>(ws.numel()), dtype_code(query), dtype_code(k_cache), current_stream(query));
    check_rc(rc, "xllm_mi355_paged_decode_gqa_planned");
    return;
  }
  const int rc = xllm_mi355_paged_decode_gqa(
      query.data_ptr(), k_cache.data_ptr(), v_cache->data_ptr(), output.data_ptr(), lse,
      block_table.data_ptr<int32_t>(), block_table.stride(0), seq_lens.data_ptr<int32_t>(),
      static_cast<const float*>(ptr_or_null(k_cache_quant_scale)),
      static_cast<const float*>(ptr_or_null(v_cache_quant_scale)), B, Hq, k_cache.size(2), D, k_cache.size(1),
      k_cache.size(0), query.stride(0), output.stride(0), max_seq_len, window_size_left, scale, ws.data_ptr(),
      static_cast<size_t>(ws.numel()), dtype_code(query), dtype_code(k_cache), current_stream(query));
  check_rc(rc, "xllm_mi355_paged_decode_gqa");
}

void batch_decode_csr(torch::Tensor query, torch::Tensor k_cache, torch::Tensor v_cache,
                      torch::Tensor paged_kv_indptr, torch::Tensor paged_kv_indices,
                      torch::Tensor paged_kv_last_page_len, int64_t window_left, double sm_scale,
                      torch::Tensor output, std::optional<torch::Tensor>& output_lse, int64_t max_seq_len,
                      const std::optional<torch::Tensor>& plan) {
  check_decode_operands(query, output, k_cache, v_cache, std::nullopt, std::nullopt);
  const int64_t B = query.size(0), Hq = query.size(1), D = query.size(2);
  for (const torch::Tensor* t : {&paged_kv_indptr, &paged_kv_indices, &paged_kv_last_page_len})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kInt32 && t->is_contiguous(),
                "CSR arrays must be contiguous int32 device tensors");
  TORCH_CHECK(paged_kv_indptr.numel() == B + 1 && paged_kv_last_page_len.numel() == B, "CSR sizes");
  float* lse = nullptr;
  if (output_lse.has_value() && output_lse->defined()) {
    TORCH_CHECK(output_lse->is_cuda() && output_lse->scalar_type() == torch::kFloat32 && output_lse->is_contiguous() &&
                    output_lse->numel() == B * Hq,
                "output_lse must be contiguous fp32 [B, Hq, 1]");
    lse = output_lse->data_ptr<float>();
  }
  if (max_seq_len <= 0) max_seq_len = std::max<int64_t>(1, paged_kv_indices.numel()) * k_cache.size(1);
  const size_t nbytes = xllm_mi355_paged_decode_gqa_workspace_bytes(B, Hq, D);
  torch::Tensor ws = decode_workspace(query.device(), nbytes);
  if (plan.has_value() && plan->defined()) {
    TORCH_CHECK(plan->is_cuda() && plan->is_contiguous() && plan->scalar_type() == torch::kUInt8 &&
                    static_cast<size_t>(plan->numel()) >= xllm_mi355_paged_decode_plan_bytes(),
                "plan must be the buffer of update_decode_plan (uint8, xllm_mi355_paged_decode_plan_bytes() bytes)");
    const int rc = xllm_mi355_paged_decode_gqa_planned(
        plan->data_ptr(), static_cast<size_t>(plan->numel()), query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(), lse, nullptr, 0,
        nullptr, paged_kv_indptr.data_ptr<int32_t>(), paged_kv_indices.data_ptr<int32_t>(),
        paged_kv_last_page_len.data_ptr<int32_t>(), nullptr, nullptr, B, Hq, k_cache.size(2), D, k_cache.size(1),
        k_cache.size(0), query.stride(0), output.stride(0), max_seq_len, window_left, static_cast<float>(sm_scale),
        ws.data_ptr(), static_cast<size_t>(ws.numel()), dtype_code(query), dtype_code(k_cache), current_stream(query));
    check_rc(rc, "xllm_mi355_paged_decode_gqa_planned");
    return;
  }
  const int rc = xllm_mi355_paged_decode_gqa_csr(
      query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(), lse,
      paged_kv_indptr.data_ptr<int32_t>(), paged_kv_indices.data_ptr<int32_t>(),
      paged_kv_last_page_len.data_ptr<int32_t>(), nullptr, nullptr, B, Hq, k_cache.size(2), D, k_cache.size(1),
      k_cache.size(0), query.stride(0), output.stride(0), max_seq_len, window_left, static_cast<float>(sm_scale),
      ws.data_ptr(), static_cast<size_t>(ws.numel()), dtype_code(query), dtype_code(k_cache),
      current_stream(query));
  check_rc(rc, "xllm_mi355_paged_decode_gqa_csr");
}

torch::Tensor update_decode_plan(const std::optional<torch::Tensor>& plan,
                                 const std::optional<torch::Tensor>& block_table,
                                 const std::optional<torch::Tensor>& seq_lens,
                                 const std::optional<torch::Tensor>& paged_kv_indptr,
                                 const std::optional<torch::Tensor>& paged_kv_indices,
                                 const std::optional<torch::Tensor>& paged_kv_last_page_len,
                                 int64_t num_qo_heads, int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                 int64_t window_left, torch::ScalarType cache_dtype) {
  auto defined = [](const std::optional<torch::Tensor>& t) { return t.has_value() && t->defined(); };
  auto int32_device = [](const torch::Tensor& t) {
    return t.is_cuda() && t.scalar_type() == torch::kInt32;
  };
  const bool csr = defined(paged_kv_indptr);
  const torch::Tensor& anchor = csr ? *paged_kv_indptr : *seq_lens;
  const int64_t nbytes = static_cast<int64_t>(xllm_mi355_paged_decode_plan_bytes());
  torch::Tensor buf = defined(plan) ? *plan : torch::empty({nbytes}, anchor.options().dtype(torch::kUInt8));
  TORCH_CHECK(buf.is_cuda() && buf.is_contiguous() && static_cast<int64_t>(buf.nbytes()) >= nbytes,
              "plan must be a contiguous device buffer of xllm_mi355_paged_decode_plan_bytes() bytes");
  int64_t B = 0;
  const int32_t *table = nullptr, *lens = nullptr, *indptr = nullptr, *indices = nullptr, *last = nullptr;
  int64_t stride = 0;
  if (csr) {
    TORCH_CHECK(defined(paged_kv_indices) && defined(paged_kv_last_page_len), "the CSR form needs all three arrays");
    for (const torch::Tensor* t : {&*paged_kv_indptr, &*paged_kv_indices, &*paged_kv_last_page_len})
      TORCH_CHECK(int32_device(*t) && t->is_contiguous(), "CSR arrays must be contiguous int32 device tensors");
    B = paged_kv_last_page_len->numel();
    TORCH_CHECK(paged_kv_indptr->numel() == B + 1, "CSR sizes");
    indptr = paged_kv_indptr->data_ptr<int32_t>();
    indices = paged_kv_indices->data_ptr<int32_t>();
    last = paged_kv_last_page_len->data_ptr<int32_t>();
  } else {
    TORCH_CHECK(defined(block_table) && defined(seq_lens), "the block-table form needs the table and the lengths");
    TORCH_CHECK(int32_device(*block_table) && block_table->dim() == 2 && block_table->stride(1) == 1 &&
                    int32_device(*seq_lens) && seq_lens->is_contiguous() && block_table->size(0) == seq_lens->numel(),
                "block_table must be int32 [B, W], seq_lens contiguous int32 [B]");
    B = seq_lens->numel();
    table = block_table->data_ptr<int32_t>();
    stride = block_table->stride(0);
    lens = seq_lens->data_ptr<int32_t>();
  }
  const int code = cache_dtype == torch::kFloat8_e4m3fn ? XLLM_MI355_FP8_E4M3
                   : cache_dtype == torch::kFloat16     ? XLLM_MI355_FP16
                                                        : XLLM_MI355_BF16;
  const int rc = xllm_mi355_paged_decode_gqa_plan(buf.data_ptr(), static_cast<size_t>(buf.nbytes()), table, stride, lens,
                                                  indptr, indices, last, B, num_qo_heads, num_kv_heads, head_dim,
                                                  block_size, window_left, code, current_stream(anchor));
  check_rc(rc, "xllm_mi355_paged_decode_gqa_plan");
  return buf;
}

void paged_forward(const torch::Tensor& query, torch::Tensor& output, const torch::Tensor& k_cache,
                   const torch::Tensor& v_cache, const torch::Tensor& block_table,
                   const torch::Tensor& kv_seq_lens, const torch::Tensor& q_cu_seq_lens, float scale,
                   bool is_causal, int64_t max_seq_len, int64_t max_query_len, int64_t window_left,
                   const std::optional<torch::Tensor>& k_cache_quant_scale,
                   const std::optional<torch::Tensor>& v_cache_quant_scale) {
  check_decode_operands(query, output, k_cache, v_cache, k_cache_quant_scale, v_cache_quant_scale);
  const int64_t T = query.size(0), Hq = query.size(1), D = query.size(2), B = kv_seq_lens.numel();
  TORCH_CHECK(block_table.scalar_type() == torch::kInt32 && block_table.dim() == 2 && block_table.stride(1) == 1 &&
                  block_table.size(0) == B,
              "block_table must be int32 [B, W]");
  TORCH_CHECK(kv_seq_lens.scalar_type() == torch::kInt32 && kv_seq_lens.is_contiguous() &&
                  q_cu_seq_lens.scalar_type() == torch::kInt32 && q_cu_seq_lens.is_contiguous() &&
                  q_cu_seq_lens.numel() == B + 1,
              "kv_seq_lens [B] and q_cu_seq_lens [B + 1] must be contiguous int32");
  if (max_seq_len <= 0) max_seq_len = block_table.size(1) * k_cache.size(1);
  const size_t nbytes = xllm_mi355_paged_decode_varlen_workspace_bytes(std::max(T, B), Hq, D);
  torch::Tensor ws = decode_workspace(query.device(), nbytes);
  const int rc = xllm_mi355_paged_decode_gqa_varlen(
      query.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), output.data_ptr(),
      q_cu_seq_lens.data_ptr<int32_t>(), kv_seq_lens.data_ptr<int32_t>(), block_table.data_ptr<int32_t>(),
      block_table.stride(0), static_cast<const float*>(ptr_or_null(k_cache_quant_scale)),
      static_cast<const float*>(ptr_or_null(v_cache_quant_scale)), B, T, max_query_len, Hq, k_cache.size(2), D,
      k_cache.size(1), k_cache.size(0),
      query.stride(0), output.stride(0), max_seq_len, window_left, scale, is_causal ? 1 : 0, ws.data_ptr(),
      static_cast<size_t>(ws.numel()), dtype_code(query), dtype_code(k_cache), current_stream(query));
  check_rc(rc, "xllm_mi355_paged_decode_gqa_varlen");
}

torch::Tensor mask_block_table_padding(const torch::Tensor& block_table, const torch::Tensor& kv_seq_lens,
                                       int64_t page_block_size) {
  // the checks of xllm/core/layers/dcu/flash_attention.cpp:200-202
  TORCH_CHECK(block_table.defined(), "block_table must be defined");
  TORCH_CHECK(kv_seq_lens.defined(), "kv_seq_lens must be defined");
  TORCH_CHECK(page_block_size > 0, "page_block_size must be positive");
  TORCH_CHECK(block_table.is_cuda() && kv_seq_lens.is_cuda(), "tensors must be on the device");
  TORCH_CHECK(block_table.dim() == 2 && kv_seq_lens.numel() == block_table.size(0),
              "block_table must be [batch, max_blocks] and kv_seq_lens [batch]");
  torch::Tensor table = block_table.scalar_type() == torch::kInt32 ? block_table : block_table.to(torch::kInt32);
  if (table.stride(1) != 1) table = table.contiguous();
  torch::Tensor lens = (kv_seq_lens.scalar_type() == torch::kInt32 ? kv_seq_lens : kv_seq_lens.to(torch::kInt32)).contiguous();
  torch::Tensor out = torch::empty({table.size(0), table.size(1)}, table.options());
  const int rc = xllm_mi355_mask_block_table_padding(table.data_ptr<int32_t>(), table.stride(0), lens.data_ptr<int32_t>(),
                                                     out.data_ptr<int32_t>(), out.stride(0), table.size(0),
                                                     table.size(1), page_block_size, current_stream(table));
  check_rc(rc, "xllm_mi355_mask_block_table_padding");
  return out;
}

torch::Tensor absorbed_bmm(const torch::Tensor& x, const torch::Tensor& w) {
  // the conditions torch::bmm puts on its operands, on the head-major views of
  // xllm/core/layers/dcu/deepseek_v2_attention.cpp:428-430, 231-238
  TORCH_CHECK(x.defined() && w.defined(), "absorbed_bmm requires x and w");
  TORCH_CHECK(x.is_cuda() && w.is_cuda(), "tensors must be on the device");
  TORCH_CHECK(x.dim() == 3 && w.dim() == 3, "x must be [tokens, heads, k] and w [heads, k, n]");
  TORCH_CHECK(x.size(1) == w.size(0) && x.size(2) == w.size(1), "x [tokens, heads, k] does not match w [heads, k, n]");
  TORCH_CHECK(x.scalar_type() == w.scalar_type(), "x and w must have the same dtype");
  const torch::Tensor xs = x.stride(2) == 1 ? x : x.contiguous();
  const torch::Tensor ws = w.contiguous();
  torch::Tensor out = torch::empty({x.size(0), x.size(1), w.size(2)}, x.options());
  const int rc = xllm_mi355_mla_absorbed_bmm(xs.data_ptr(), ws.data_ptr(), out.data_ptr(), xs.size(0), xs.size(1),
                                             xs.size(2), ws.size(2), xs.stride(0), xs.stride(1), out.stride(0),
                                             out.stride(1), dtype_code(xs), current_stream(xs));
  check_rc(rc, "xllm_mi355_mla_absorbed_bmm");
  return out;
}

torch::Tensor gather_mla_latent_cache(const torch::Tensor& k_cache, const torch::Tensor& block_table,
                                      const torch::Tensor& kv_cu_seq_lens, int64_t total_kv_len,
                                      int64_t max_seq_len) {
  // the checks of xllm/core/kernels/dcu/gather_mla_latent_cache.hip:124-150
  TORCH_CHECK(k_cache.defined() && block_table.defined() && kv_cu_seq_lens.defined(),
              "gather_mla_latent_cache requires k_cache, block_table and kv_cu_seq_lens");
  TORCH_CHECK(k_cache.is_cuda() && block_table.is_cuda() && kv_cu_seq_lens.is_cuda(), "tensors must be on the device");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.size(2) == 1, "k_cache must be [blocks, block_size, 1, dim]");
  TORCH_CHECK(block_table.dim() == 2, "block_table must be [batch, max_blocks]");
  TORCH_CHECK(kv_cu_seq_lens.dim() == 1 && kv_cu_seq_lens.size(0) == block_table.size(0) + 1,
              "kv_cu_seq_lens must be [batch + 1]");
  TORCH_CHECK(total_kv_len > 0 && max_seq_len > 0, "total_kv_len and max_seq_len must be positive");
  TORCH_CHECK(k_cache.is_contiguous(), "k_cache must be contiguous");
  torch::Tensor table = (block_table.scalar_type() == torch::kInt32 ? block_table : block_table.to(torch::kInt32)).contiguous();
  torch::Tensor cu = (kv_cu_seq_lens.scalar_type() == torch::kInt32 ? kv_cu_seq_lens : kv_cu_seq_lens.to(torch::kInt32)).contiguous();
  torch::Tensor out = torch::empty({total_kv_len, k_cache.size(3)}, k_cache.options());
  const int rc = xllm_mi355_gather_paged_rows(k_cache.data_ptr(), table.data_ptr<int32_t>(), table.stride(0),
                                              cu.data_ptr<int32_t>(), out.data_ptr(), table.size(0), total_kv_len,
                                              k_cache.size(1), k_cache.size(0),
                                              k_cache.size(3) * static_cast<int64_t>(k_cache.element_size()),
                                              current_stream(k_cache));
  check_rc(rc, "xllm_mi355_gather_paged_rows");
  return out;
}

namespace {
void rope_launch(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v, int64_t head_dim,
                 double eps, const torch::Tensor& q_weight, const torch::Tensor& k_weight,
                 const torch::Tensor& cos_sin_cache, bool interleaved, const torch::Tensor& position_ids,
                 ReshapePagedCacheParams* cache) {
  // the checks of xllm/core/kernels/cuda/fused_qknorm_rope.cu:402-447
  TORCH_CHECK(qkv.is_cuda() && qkv.is_contiguous(), "qkv must be a contiguous device tensor");
  TORCH_CHECK(position_ids.is_cuda() && position_ids.is_contiguous(), "position_ids must be a contiguous device tensor");
  TORCH_CHECK(q_weight.is_cuda() && q_weight.is_contiguous() && k_weight.is_cuda() && k_weight.is_contiguous(),
              "q_weight and k_weight must be contiguous device tensors");
  TORCH_CHECK(cos_sin_cache.is_cuda() && cos_sin_cache.is_contiguous(), "cos_sin_cache must be a contiguous device tensor");
  TORCH_CHECK(position_ids.scalar_type() == torch::kInt64, "position_ids must be int64");
  TORCH_CHECK(qkv.dim() == 2 && position_ids.dim() == 1 && q_weight.dim() == 1 && k_weight.dim() == 1 &&
                  cos_sin_cache.dim() == 2,
              "qkv [T, (Hq + Hk + Hv) * D], position_ids [T], weights [D], cos_sin_cache [max_position, rotary_dim]");
  TORCH_CHECK(q_weight.size(0) == head_dim && k_weight.size(0) == head_dim, "weights must be [head_dim]");
  TORCH_CHECK(cos_sin_cache.size(1) % 2 == 0 && cos_sin_cache.size(1) <= head_dim, "rotary_dim must be even and <= head_dim");
  TORCH_CHECK(qkv.scalar_type() == q_weight.scalar_type() && qkv.scalar_type() == k_weight.scalar_type(),
              "qkv, q_weight and k_weight must have the same dtype");
  TORCH_CHECK(position_ids.size(0) == qkv.size(0), "one position per token");
  TORCH_CHECK(qkv.size(1) == (num_heads_q + num_heads_k + num_heads_v) * head_dim, "qkv width");
  void* kc = nullptr;
  void* vc = nullptr;
  const int32_t* slots = nullptr;
  const float* ks = nullptr;
  const float* vs = nullptr;
  int64_t bs = 0, blocks = 0;
  int cache_dtype = dtype_code(qkv);
  torch::Tensor slot32;
  if (cache != nullptr) {
    TORCH_CHECK(cache->v_cache.has_value() && cache->v_cache->defined() && cache->k_cache.defined(),
                "the fused cache write needs k_cache and v_cache");
    TORCH_CHECK(cache->k_cache.is_cuda() && cache->v_cache->is_cuda() && cache->slot_mapping.is_cuda(),
                "caches and slot_mapping must be device tensors");
    TORCH_CHECK(cache->k_cache.is_contiguous() && cache->v_cache->is_contiguous(), "caches must be contiguous");
    TORCH_CHECK(cache->k_cache.dim() == 4 && cache->k_cache.size(2) == num_heads_k && cache->k_cache.size(3) == head_dim &&
                    cache->v_cache->sizes() == cache->k_cache.sizes() &&
                    cache->v_cache->scalar_type() == cache->k_cache.scalar_type() && num_heads_v == num_heads_k,
                "caches must be [P, bs, num_heads_k, head_dim], v_cache like k_cache");
    TORCH_CHECK(cache->slot_mapping.numel() == qkv.size(0), "one slot per token");
    const bool fp8 = cache->k_cache.scalar_type() == torch::kFloat8_e4m3fn || cache->k_cache.scalar_type() == torch::kUInt8;
    if (fp8) {
      for (const std::optional<torch::Tensor>* s : {&cache->k_cache_scale, &cache->v_cache_scale})
        TORCH_CHECK(s->has_value() && (*s)->defined() && (*s)->is_cuda() && (*s)->scalar_type() == torch::kFloat32 &&
                        (*s)->is_contiguous() && (*s)->numel() == num_heads_k,
                    "an fp8 cache needs contiguous fp32 device scales [num_heads_k]");
    } else {
      TORCH_CHECK(cache->k_cache.scalar_type() == qkv.scalar_type(), "cache dtype must equal the qkv dtype (or be fp8)");
    }
    slot32 = (cache->slot_mapping.scalar_type() == torch::kInt32 ? cache->slot_mapping
                                                                   : cache->slot_mapping.to(torch::kInt32)).contiguous();
    kc = cache->k_cache.data_ptr();
    vc = cache->v_cache->data_ptr();
    slots = slot32.data_ptr<int32_t>();
    bs = cache->k_cache.size(1);
    blocks = cache->k_cache.size(0);
    cache_dtype = dtype_code(cache->k_cache);
    if (cache->k_cache_scale.has_value()) ks = cache->k_cache_scale->data_ptr<float>();
    if (cache->v_cache_scale.has_value()) vs = cache->v_cache_scale->data_ptr<float>();
  }
  const int rc = xllm_mi355_rope_and_cache(
      qkv.data_ptr(), q_weight.data_ptr(), k_weight.data_ptr(), cos_sin_cache.data_ptr(), position_ids.data_ptr<int64_t>(),
      kc, vc, slots, ks, vs, qkv.size(0), qkv.stride(0), num_heads_q, num_heads_k, num_heads_v, head_dim,
      cos_sin_cache.size(1), static_cast<float>(eps), interleaved ? 1 : 0, bs, blocks, dtype_code(qkv),
      dtype_code(cos_sin_cache), cache_dtype, current_stream(qkv));
  check_rc(rc, "xllm_mi355_rope_and_cache");
}
}  // namespace

void fused_qk_norm_rope(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                        int64_t head_dim, double eps, const torch::Tensor& q_weight, const torch::Tensor& k_weight,
                        const torch::Tensor& cos_sin_cache, bool interleaved, const torch::Tensor& position_ids) {
  rope_launch(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleaved,
              position_ids, nullptr);
}

void fused_qk_norm_rope_and_cache(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                                  int64_t head_dim, double eps, const torch::Tensor& q_weight,
                                  const torch::Tensor& k_weight, const torch::Tensor& cos_sin_cache, bool interleaved,
                                  const torch::Tensor& position_ids, ReshapePagedCacheParams& cache) {
  rope_launch(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleaved,
              position_ids, &cache);
}

void update_llm_decode_metadata(const LlmDecodeMetadataUpdateParams& p, void* stream) {
  const int rc = xllm_mi355_decode_metadata_update(
      p.src_tokens, p.src_positions, p.src_new_cache_slots, p.src_kv_seq_lens, p.src_paged_kv_indptr,
      p.src_paged_kv_indices, p.src_paged_kv_last_page_len, p.dst_tokens, p.dst_positions, p.dst_new_cache_slots,
      p.dst_kv_seq_lens, p.dst_kv_seq_lens_delta, p.dst_paged_kv_indptr, p.dst_paged_kv_indices,
      p.dst_paged_kv_last_page_len, p.actual_num_tokens, p.padded_num_tokens, p.actual_batch_size,
      p.actual_indices_size, stream);
  check_rc(rc, "xllm_mi355_decode_metadata_update");
}

void lse_combine(torch::Tensor output, torch::Tensor shared_o, torch::Tensor shared_lse, torch::Tensor unshared_o,
                 torch::Tensor unshared_lse) {
  // the checks of xllm/core/kernels/cuda/xattention/lse_combine.cu:104-131
  TORCH_CHECK(shared_o.dim() == 3, "shared_o must be 3D [B, H, D]");
  TORCH_CHECK(unshared_o.dim() == 3, "unshared_o must be 3D [B, H, D]");
  TORCH_CHECK(shared_lse.dim() == 3, "shared_lse must be 3D [B, H, 1]");
  TORCH_CHECK(unshared_lse.dim() == 3, "unshared_lse must be 3D [B, H, 1]");
  const int64_t B = shared_o.size(0), H = shared_o.size(1), D = shared_o.size(2);
  TORCH_CHECK(shared_o.sizes() == unshared_o.sizes() && shared_o.scalar_type() == unshared_o.scalar_type(),
              "shared_o and unshared_o must have same shape");
  TORCH_CHECK(shared_lse.scalar_type() == torch::kFloat32, "shared_lse must be float32");
  TORCH_CHECK(unshared_lse.scalar_type() == torch::kFloat32, "unshared_lse must be float32");
  for (const torch::Tensor* t : {&shared_lse, &unshared_lse})
    TORCH_CHECK(t->size(0) == B && t->size(1) == H && t->size(2) == 1, "lse shape mismatch, expected [B, H, 1]");
  TORCH_CHECK(shared_o.is_cuda() && unshared_o.is_cuda() && shared_lse.is_cuda() && unshared_lse.is_cuda(),
              "tensors must be on the device");
  // (like the reference, a missing or misshapen output is replaced by a local tensor the caller never sees)
  if (!output.defined() || output.sizes() != shared_o.sizes()) output = torch::empty_like(shared_o);
  TORCH_CHECK(output.is_cuda() && output.is_contiguous(), "output must be a contiguous device tensor");
  const torch::Tensor so = shared_o.contiguous(), uo = unshared_o.contiguous();
  const torch::Tensor sl = shared_lse.contiguous(), ul = unshared_lse.contiguous();
  const int rc = xllm_mi355_lse_combine(output.data_ptr(), so.data_ptr(), sl.data_ptr<float>(), uo.data_ptr(),
                                        ul.data_ptr<float>(), B * H, D, dtype_code(so), dtype_code(output),
                                        current_stream(so));
  check_rc(rc, "xllm_mi355_lse_combine");
}

}  // namespace mi355

namespace dcu {
namespace flash_mla {

namespace {
// check_dense_decode_inputs, xllm/core/kernels/dcu/flash_mla_adapter.cpp:55-100 (the page size is not pinned to
// 64 here: the kernels take any block size)
void check_dense_decode_inputs(const DenseDecodeParams& p) {
  TORCH_CHECK(p.q_nope.defined(), "flash_mla: q_nope must be defined");
  TORCH_CHECK(p.q_pe.defined(), "flash_mla: q_pe must be defined");
  TORCH_CHECK(p.k_cache.defined(), "flash_mla: k_cache must be defined");
  TORCH_CHECK(p.seqlens_k.defined(), "flash_mla: seqlens_k must be defined");
  TORCH_CHECK(p.block_table.defined(), "flash_mla: block_table must be defined");
  const torch::Device dev = p.k_cache.device();
  TORCH_CHECK(dev.is_cuda(), "flash_mla: k_cache must be on the device");
  TORCH_CHECK(p.q_nope.device() == dev, "flash_mla: q_nope must be on the device of k_cache");
  TORCH_CHECK(p.q_pe.device() == dev, "flash_mla: q_pe must be on the device of k_cache");
  TORCH_CHECK(p.seqlens_k.device() == dev, "flash_mla: seqlens_k must be on the device of k_cache");
  TORCH_CHECK(p.block_table.device() == dev, "flash_mla: block_table must be on the device of k_cache");
  TORCH_CHECK(p.q_nope.dim() == 4, "flash_mla: q_nope must be 4D [B,S_q,H_q,D]");
  TORCH_CHECK(p.q_pe.dim() == 4, "flash_mla: q_pe must be 4D [B,S_q,H_q,D]");
  TORCH_CHECK(p.k_cache.dim() == 4, "flash_mla: k_cache must be 4D [blocks,page,1,D]");
  TORCH_CHECK(p.k_cache.size(2) == 1, "flash_mla: MLA expects a single KV head (num_heads_k == 1)");
  TORCH_CHECK(p.seqlens_k.dim() == 1, "flash_mla: seqlens_k must be 1D [B]");
  TORCH_CHECK(p.block_table.dim() == 2, "flash_mla: block_table must be 2D [B,max_blocks]");
  TORCH_CHECK(p.k_cache.size(3) == p.q_nope.size(3) + p.q_pe.size(3),
              "flash_mla: k_cache last dim must equal q_nope.dim + q_pe.dim");
  TORCH_CHECK(p.q_nope.size(0) == p.q_pe.size(0), "flash_mla: q_nope/q_pe batch must match");
  TORCH_CHECK(p.q_nope.size(1) == p.q_pe.size(1), "flash_mla: q_nope/q_pe seq must match");
  TORCH_CHECK(p.q_nope.size(2) == p.q_pe.size(2), "flash_mla: q_nope/q_pe head count must match");
  TORCH_CHECK(p.head_size_v > 0, "flash_mla: head_size_v must be positive");
  // what the kernels behind this adapter add
  TORCH_CHECK(p.seqlens_k.numel() == p.q_nope.size(0) && p.block_table.size(0) == p.q_nope.size(0),
              "flash_mla: seqlens_k and block_table must have one row per sequence");
  TORCH_CHECK(p.k_cache.is_contiguous(), "flash_mla: k_cache must be contiguous");
  TORCH_CHECK(p.q_nope.scalar_type() == p.q_pe.scalar_type() && p.q_nope.scalar_type() == p.k_cache.scalar_type(),
              "flash_mla: q_nope, q_pe and k_cache must have the same dtype");
  TORCH_CHECK(p.q_nope.scalar_type() == torch::kBFloat16 || p.q_nope.scalar_type() == torch::kFloat16,
              "flash_mla: BF16 / FP16 only");
  TORCH_CHECK(p.head_size_v == p.q_nope.size(3), "flash_mla: V is the latent part of the cache (head_size_v == q_nope.dim)");
}
}  // namespace

namespace {
struct NewLatent {
  torch::Tensor rows, slots;
};
torch::Tensor dense_decode_impl(DenseDecodeParams& p, const torch::Tensor* plan, torch::Tensor* lse_out,
                                const NewLatent* fresh = nullptr);
}
torch::Tensor store_and_dense_decode(DenseDecodeParams& p, const torch::Tensor& latent_cache,
                                     const torch::Tensor& slot_mapping,
                                     const std::optional<torch::Tensor>& tile_scheduler_metadata, torch::Tensor* lse_out) {
  const bool planned = tile_scheduler_metadata.has_value() && tile_scheduler_metadata->defined();
  if (planned)
    TORCH_CHECK(tile_scheduler_metadata->is_cuda() && tile_scheduler_metadata->is_contiguous() &&
                    tile_scheduler_metadata->scalar_type() == torch::kUInt8 &&
                    static_cast<size_t>(tile_scheduler_metadata->numel()) >= xllm_mi355_paged_decode_plan_bytes(),
                "flash_mla: tile_scheduler_metadata must be the buffer of get_mla_decoding_metadata");
  TORCH_CHECK(latent_cache.defined() && latent_cache.is_cuda() && (latent_cache.dim() == 2 || latent_cache.dim() == 3),
              "flash_mla: latent_cache must be a device tensor [B, D] or [B, 1, D]");
  const NewLatent fresh{latent_cache.dim() == 3 ? latent_cache.view({latent_cache.size(0), -1}) : latent_cache, slot_mapping};
  return dense_decode_impl(p, planned ? &*tile_scheduler_metadata : nullptr, lse_out, &fresh);
}
torch::Tensor dense_decode(DenseDecodeParams& p, torch::Tensor* lse_out) { return dense_decode_impl(p, nullptr, lse_out); }
torch::Tensor dense_decode(DenseDecodeParams& p, const torch::Tensor& tile_scheduler_metadata, torch::Tensor* lse_out) {
  TORCH_CHECK(tile_scheduler_metadata.defined() && tile_scheduler_metadata.is_cuda() &&
                  tile_scheduler_metadata.is_contiguous() && tile_scheduler_metadata.scalar_type() == torch::kUInt8 &&
                  static_cast<size_t>(tile_scheduler_metadata.numel()) >= xllm_mi355_paged_decode_plan_bytes(),
              "flash_mla: tile_scheduler_metadata must be the buffer of get_mla_decoding_metadata");
  return dense_decode_impl(p, &tile_scheduler_metadata, lse_out);
}

std::vector<torch::Tensor> get_mla_decoding_metadata(const torch::Tensor& seqlens_k, const torch::Tensor& block_table,
                                                     int64_t num_heads_per_head_k, int64_t num_heads_k,
                                                     int64_t block_size, const std::optional<torch::Tensor>& reuse) {
  TORCH_CHECK(num_heads_k == 1, "flash_mla: the latent cache has one KV head");
  TORCH_CHECK(seqlens_k.is_cuda() && seqlens_k.dim() == 1 && seqlens_k.scalar_type() == torch::kInt32 &&
                  seqlens_k.is_contiguous(),
              "flash_mla: seqlens_k must be contiguous int32 [B] on the device");
  TORCH_CHECK(block_table.is_cuda() && block_table.dim() == 2 && block_table.scalar_type() == torch::kInt32 &&
                  block_table.stride(1) == 1 && block_table.size(0) == seqlens_k.numel(),
              "flash_mla: block_table must be int32 [B, max_blocks] with unit column stride");
  const int64_t nbytes = static_cast<int64_t>(xllm_mi355_paged_decode_plan_bytes());
  torch::Tensor buf = reuse.has_value() && reuse->defined()
                          ? *reuse
                          : torch::empty({nbytes}, seqlens_k.options().dtype(torch::kUInt8));
  TORCH_CHECK(buf.is_cuda() && buf.is_contiguous() && buf.scalar_type() == torch::kUInt8 && buf.numel() >= nbytes,
              "flash_mla: the plan must be a contiguous uint8 device buffer of xllm_mi355_paged_decode_plan_bytes() bytes");
  const int rc = xllm_mi355_paged_decode_mla_plan(buf.data_ptr(), static_cast<size_t>(buf.numel()),
                                                  block_table.data_ptr<int32_t>(), block_table.stride(0),
                                                  seqlens_k.data_ptr<int32_t>(), seqlens_k.numel(), num_heads_per_head_k,
                                                  block_size, current_stream(seqlens_k));
  check_rc(rc, "xllm_mi355_paged_decode_mla_plan");
  // (the reference returns {tile_scheduler_metadata, num_splits}; the splits live in the same buffer here)
  return {buf, torch::empty({0}, seqlens_k.options())};
}

namespace {
torch::Tensor dense_decode_impl(DenseDecodeParams& p, const torch::Tensor* plan, torch::Tensor* lse_out,
                                const NewLatent* fresh) {
  TORCH_CHECK(p.kind == DenseDecodeKind::kQNopePe,
              "flash_mla: only DenseDecodeKind::kQNopePe (BF16/FP16 split-q) is supported");
  check_dense_decode_inputs(p);
  torch::Tensor seqlens = p.seqlens_k.scalar_type() == torch::kInt32 ? p.seqlens_k : p.seqlens_k.to(torch::kInt32);
  torch::Tensor table = p.block_table.scalar_type() == torch::kInt32 ? p.block_table : p.block_table.to(torch::kInt32);
  seqlens = seqlens.contiguous();
  if (table.stride(1) != 1) table = table.contiguous();
  TORCH_CHECK(p.softmax_scale > 0.0F, "flash_mla: softmax_scale must be set by the MLA attention layer");
  const torch::Tensor q_nope = p.q_nope.contiguous(), q_pe = p.q_pe.contiguous();
  const int64_t B = q_nope.size(0), Sq = q_nope.size(1), H = q_nope.size(2);
  torch::Tensor out = torch::empty({B, Sq, H, p.head_size_v}, q_nope.options());
  // The reference folds the S_q query tokens of a sequence into the head count (flash_mla_adapter.cpp:119-123):
  // q [B, S_q * H, D] against the same pages.  With a causal mask token j sees S_q - 1 - j tokens less than the
  // last one, so every (sequence, token) becomes a row of its own: [B * S_q, H, D] with its own length and the
  // table row of its sequence.
  const bool per_token = p.is_causal && Sq > 1;
  int64_t rows = B, heads = Sq * H;
  if (per_token) {
    rows = B * Sq;
    heads = H;
    const torch::Tensor back = torch::arange(Sq - 1, -1, -1, seqlens.options());            // S_q - 1 - j
    seqlens = (seqlens.unsqueeze(1) - back.unsqueeze(0)).clamp_min(0).reshape({rows}).contiguous();
    table = table.repeat_interleave(Sq, 0).contiguous();
  }
  torch::Tensor lse_rows;  // [rows, heads]
  float* lse = nullptr;
  if (lse_out != nullptr) {
    lse_rows = torch::empty({rows, heads}, q_nope.options().dtype(torch::kFloat32));
    lse = lse_rows.data_ptr<float>();
  }
  const int64_t max_seq_len = table.size(1) * p.k_cache.size(1);
  const size_t nbytes = xllm_mi355_paged_decode_mla_workspace_bytes(rows, heads, max_seq_len);
  torch::Tensor ws = mi355::decode_workspace(q_nope.device(), nbytes);
  if (fresh != nullptr) {
    TORCH_CHECK(Sq == 1, "flash_mla: the one-call step stores one new row per sequence (S_q == 1)");
    TORCH_CHECK(fresh->rows.size(0) == B && fresh->rows.size(1) == p.k_cache.size(3) && fresh->rows.stride(1) == 1 &&
                    fresh->rows.scalar_type() == q_nope.scalar_type(),
                "flash_mla: latent_cache must hold one row of the cache's width per sequence, in the query's dtype");
    TORCH_CHECK(fresh->slots.is_cuda() && fresh->slots.scalar_type() == torch::kInt32 && fresh->slots.is_contiguous() &&
                    fresh->slots.numel() == B,
                "flash_mla: slot_mapping must be contiguous int32 [B]");
    const int rc = xllm_mi355_write_and_decode_mla(
        fresh->rows.data_ptr(), fresh->slots.data_ptr<int32_t>(), fresh->rows.stride(0),
        plan != nullptr ? plan->data_ptr() : nullptr, plan != nullptr ? static_cast<size_t>(plan->numel()) : 0,
        q_nope.data_ptr(), q_pe.data_ptr(), p.k_cache.data_ptr(), out.data_ptr(), lse, table.data_ptr<int32_t>(),
        table.stride(0), seqlens.data_ptr<int32_t>(), rows, heads, q_nope.size(3), q_pe.size(3), p.k_cache.size(1),
        p.k_cache.size(0), max_seq_len, p.softmax_scale, ws.data_ptr(), static_cast<size_t>(ws.numel()),
        dtype_code(q_nope), current_stream(q_nope));
    check_rc(rc, "xllm_mi355_write_and_decode_mla");
  } else if (plan != nullptr && !per_token) {   // (a causal multi-token step rewrites lengths and table per token: no plan)
    const int rc = xllm_mi355_paged_decode_mla_planned(
        plan->data_ptr(), static_cast<size_t>(plan->numel()), q_nope.data_ptr(), q_pe.data_ptr(), p.k_cache.data_ptr(),
        out.data_ptr(), lse, table.data_ptr<int32_t>(), table.stride(0), seqlens.data_ptr<int32_t>(), rows, heads,
        q_nope.size(3), q_pe.size(3), p.k_cache.size(1), p.k_cache.size(0), max_seq_len, p.softmax_scale, ws.data_ptr(),
        static_cast<size_t>(ws.numel()), dtype_code(q_nope), current_stream(q_nope));
    check_rc(rc, "xllm_mi355_paged_decode_mla_planned");
  } else {
    const int rc = xllm_mi355_paged_decode_mla(
        q_nope.data_ptr(), q_pe.data_ptr(), p.k_cache.data_ptr(), out.data_ptr(), lse, table.data_ptr<int32_t>(),
        table.stride(0), seqlens.data_ptr<int32_t>(), rows, heads, q_nope.size(3), q_pe.size(3), p.k_cache.size(1),
        p.k_cache.size(0), max_seq_len, p.softmax_scale, ws.data_ptr(), static_cast<size_t>(ws.numel()),
        dtype_code(q_nope), current_stream(q_nope));
    check_rc(rc, "xllm_mi355_paged_decode_mla");
  }
  if (lse_out != nullptr) *lse_out = lse_rows.view({B, Sq, H}).transpose(1, 2).contiguous();  // [B, H, S_q]
  return out;
}
}  // namespace

torch::Tensor dense_decode(DenseDecodeParams& params) { return dense_decode(params, nullptr); }

}  // namespace flash_mla
}  // namespace dcu
}  // namespace xllm::kernel

namespace xllm::layer {

DcpAttentionResult merge_dcp_attention_shards(const torch::Tensor& partial_outputs,
                                              const torch::Tensor& partial_lse) {
  TORCH_CHECK(partial_outputs.dim() == 5, "partial outputs must have shape [dcp, batch, query, heads, value]");
  TORCH_CHECK(partial_lse.dim() == 4, "partial LSE must have shape [dcp, batch, heads, query]");
  const int64_t S = partial_outputs.size(0), B = partial_outputs.size(1), Q = partial_outputs.size(2),
                H = partial_outputs.size(3), Dv = partial_outputs.size(4);
  TORCH_CHECK(partial_lse.size(0) == S && partial_lse.size(1) == B && partial_lse.size(3) == Q &&
                  partial_lse.size(2) == H,
              "partial outputs and LSE disagree");
  TORCH_CHECK(Q == 1, "decode path: one query token per sequence");
  torch::Tensor po = partial_outputs.contiguous();
  torch::Tensor pl = partial_lse.to(torch::kFloat32).contiguous();
  torch::Tensor out = torch::empty({B, Q, H, Dv}, po.options());
  torch::Tensor lse = torch::empty({B, H, Q}, pl.options());
  const int rc = xllm_mi355_lse_merge(po.data_ptr(), pl.data_ptr<float>(), out.data_ptr(), lse.data_ptr<float>(), S, B,
                                      H, Dv, dtype_code(po), current_stream(po));
  check_rc(rc, "xllm_mi355_lse_merge");
  return {out, lse};
}

// The decode and short-chunk branches of FlashAttentionImpl::forward / paged_forward
// (xllm/core/layers/dcu/flash_attention.cpp:547-660, 447-545) on this library's kernels.
std::tuple<torch::Tensor, std::optional<torch::Tensor>> Mi355AttentionImpl::forward(
    const AttentionMetadata& attn_metadata, torch::Tensor& query, torch::Tensor& key, torch::Tensor& value,
    torch::Tensor& output, KVCache& kv_cache) {
  std::optional<torch::Tensor> output_lse = std::nullopt;
  if (attn_metadata.max_seq_len == 0) {
    output = output.view({-1, num_heads_ * head_size_});
    return std::make_tuple(output, output_lse);
  }
  query = query.view({-1, num_heads_, head_size_});
  key = key.view({-1, num_kv_heads_, head_size_});
  value = value.view({-1, num_kv_heads_, head_size_});
  output = output.view({-1, num_heads_, head_size_});

  torch::Tensor k_cache = kv_cache.get_k_cache();
  torch::Tensor v_cache = kv_cache.get_v_cache();
  const std::optional<torch::Tensor> k_scale = kv_cache.get_k_cache_scale();
  const std::optional<torch::Tensor> v_scale = kv_cache.get_v_cache_scale();
  const bool quantized = k_scale.has_value() && k_scale->defined();

  // store the step's K / V rows; the quantising store where the cache carries scales
  // (xllm/core/layers/mlu/attention.cpp:109-117).  A plain decode step stores them inside its decode call below.
  const bool has_cache = k_cache.defined() && k_cache.dim() >= 2;
  const bool decode_step = !attn_metadata.is_chunked_prefill && !attn_metadata.is_prefill;
  const bool one_call = has_cache && decode_step && key.size(0) == query.size(0) && key.stride(1) == head_size_ &&
                        value.stride(1) == head_size_ && attn_metadata.slot_mapping.scalar_type() == torch::kInt32 &&
                        attn_metadata.slot_mapping.is_contiguous() &&
                        (quantized || k_cache.scalar_type() == key.scalar_type());
  if (has_cache && !one_call) {
    xllm::kernel::ReshapePagedCacheParams params;
    params.key = key;
    params.value = value;
    params.k_cache = k_cache;
    params.v_cache = v_cache;
    params.slot_mapping = attn_metadata.slot_mapping;
    if (quantized) {
      params.k_cache_scale = k_scale;
      params.v_cache_scale = v_scale;
      xllm::kernel::quant_to_paged_cache(params);
    } else {
      xllm::kernel::reshape_paged_cache(params);
    }
  }

  TORCH_CHECK(!attn_metadata.is_prefill || attn_metadata.is_chunked_prefill,
              "prefill is not part of the paged decode path");
  // window_left: a positive sliding window, otherwise the whole context (flash_attention.cpp:484)
  const int64_t window_left = sliding_window_ > 0 ? sliding_window_ : -1;
  torch::Tensor kv_seq_lens = attn_metadata.kv_seq_lens.scalar_type() == torch::kInt32
                                  ? attn_metadata.kv_seq_lens
                                  : attn_metadata.kv_seq_lens.to(torch::kInt32);
  kv_seq_lens = kv_seq_lens.contiguous();
  torch::Tensor block_table = attn_metadata.block_table.scalar_type() == torch::kInt32
                                  ? attn_metadata.block_table
                                  : attn_metadata.block_table.to(torch::kInt32);
  if (attn_metadata.is_chunked_prefill) {
    constexpr int64_t kDecodeMaxQueryLen = 16;  // kHgPrefixDecodeMaxQueryLen, flash_attention.cpp:504
    TORCH_CHECK(attn_metadata.max_query_len <= kDecodeMaxQueryLen,
                "query chunks of more than 16 tokens belong to the prefill kernel, which is not part of this path");
    const torch::Tensor cu = attn_metadata.q_cu_seq_lens.to(torch::kInt32).contiguous();
    xllm::kernel::mi355::paged_forward(query, output, k_cache, v_cache, block_table, kv_seq_lens, cu, scale_,
                                       attn_metadata.is_causal, attn_metadata.max_seq_len,
                                       attn_metadata.max_query_len, window_left, k_scale, v_scale);
  } else {
    // decode: one query token per sequence, a token attends to its whole context whatever is_causal says.
    // With a PlanInfo in the metadata, layer 0 plans the step and every layer decodes from that plan
    // (xllm/core/layers/cuda/flashinfer_attention.cpp:305-323 and the plan_info argument of its batch_decode call).
    std::optional<torch::Tensor> plan = std::nullopt;
    if (attn_metadata.plan_info != nullptr) {
      AttentionMetadata planned_meta = attn_metadata;
      planned_meta.block_table = block_table;
      planned_meta.kv_seq_lens = kv_seq_lens;
      flashinfer::update_decode_plan_info(attn_metadata.plan_info, planned_meta, k_cache.scalar_type(),
                                          static_cast<int32_t>(num_heads_), static_cast<int32_t>(num_kv_heads_),
                                          static_cast<int32_t>(head_size_), static_cast<int32_t>(k_cache.size(1)),
                                          static_cast<int32_t>(window_left));
      TORCH_CHECK(attn_metadata.plan_info->plan_info.defined(), "no layer 0 has planned this step");
      plan = attn_metadata.plan_info->plan_info;
    }
    const xllm::kernel::mi355::NewKvRows fresh{key, value, attn_metadata.slot_mapping};
    xllm::kernel::mi355::batch_decode(query, k_cache, output, block_table, kv_seq_lens, v_cache, output_lse, k_scale,
                                      v_scale, attn_metadata.max_seq_len, window_left, scale_, return_lse_, plan,
                                      one_call ? &fresh : nullptr);
  }
  output = output.view({-1, num_heads_ * head_size_});
  return std::make_tuple(output, output_lse);
}

namespace flashinfer {
void update_decode_plan_info(std::shared_ptr<PlanInfo> plan_info, const AttentionMetadata& attn_meta,
                             c10::ScalarType key_dtype, int32_t num_qo_heads, int32_t num_kv_heads, int32_t head_dim,
                             int32_t block_size, int32_t window_size_left) {
  TORCH_CHECK(plan_info != nullptr && plan_info->layer_id != -1, "Need to set layer_id to PlanInfo.");
  if (plan_info->layer_id != 0) return;
  std::optional<torch::Tensor> old = std::nullopt;
  if (plan_info->plan_info.defined()) old = plan_info->plan_info;
  plan_info->plan_info = xllm::kernel::mi355::update_decode_plan(
      old, attn_meta.block_table, attn_meta.kv_seq_lens, std::nullopt, std::nullopt, std::nullopt, num_qo_heads,
      num_kv_heads, head_dim, block_size, window_size_left, key_dtype);
}
}  // namespace flashinfer

}  // namespace xllm::layer

// torch dispatcher registration: the schema of xllm_ops::reshape_paged_cache is the reference's
// (xllm/core/kernels/cuda/cuda_ops_library.cpp:286-287); the decode ops are this build's.
namespace {

torch::Tensor op_reshape_paged_cache(torch::Tensor slot_mapping, torch::Tensor keys, torch::Tensor values,
                                     torch::Tensor key_cache, torch::Tensor value_cache) {
  xllm::kernel::ReshapePagedCacheParams p;
  p.key = keys;
  p.value = values;
  p.k_cache = key_cache;
  p.v_cache = value_cache;
  p.slot_mapping = slot_mapping;
  xllm::kernel::reshape_paged_cache(p);
  return key_cache;
}

torch::Tensor op_quant_to_paged_cache(torch::Tensor slot_mapping, torch::Tensor keys, torch::Tensor values,
                                      torch::Tensor key_cache, torch::Tensor value_cache,
                                      torch::Tensor k_scale, torch::Tensor v_scale) {
  xllm::kernel::ReshapePagedCacheParams p;
  p.key = keys;
  p.value = values;
  p.k_cache = key_cache;
  p.v_cache = value_cache;
  p.slot_mapping = slot_mapping;
  p.k_cache_scale = k_scale;
  p.v_cache_scale = v_scale;
  xllm::kernel::quant_to_paged_cache(p);
  return key_cache;
}

std::tuple<torch::Tensor, torch::Tensor> op_batch_decode(torch::Tensor query, torch::Tensor k_cache,
                                                         torch::Tensor v_cache, torch::Tensor output,
                                                         torch::Tensor block_table, torch::Tensor seq_lens,
                                                         std::optional<torch::Tensor> k_scale,
                                                         std::optional<torch::Tensor> v_scale, int64_t max_seq_len,
                                                         double scale, std::optional<torch::Tensor> plan) {
  std::optional<torch::Tensor> lse;
  xllm::kernel::mi355::batch_decode(query, k_cache, output, block_table, seq_lens, v_cache, lse, k_scale, v_scale,
                                    max_seq_len, /*window_size_left=*/-1, static_cast<float>(scale), /*return_lse=*/true,
                                    plan);
  return {output, lse.value()};
}

torch::Tensor op_update_decode_plan(torch::Tensor block_table, torch::Tensor seq_lens, int64_t num_qo_heads,
                                    int64_t num_kv_heads, int64_t head_dim, int64_t block_size, int64_t window_left,
                                    bool fp8_cache, std::optional<torch::Tensor> plan) {
  return xllm::kernel::mi355::update_decode_plan(plan, block_table, seq_lens, std::nullopt, std::nullopt, std::nullopt,
                                                 num_qo_heads, num_kv_heads, head_dim, block_size, window_left,
                                                 fp8_cache ? torch::kFloat8_e4m3fn : torch::kBFloat16);
}

torch::Tensor op_lse_combine(torch::Tensor output, torch::Tensor shared_o, torch::Tensor shared_lse,
                             torch::Tensor unshared_o, torch::Tensor unshared_lse) {
  xllm::kernel::mi355::lse_combine(output, shared_o, shared_lse, unshared_o, unshared_lse);
  return output;
}

// The layer contract end to end: AttentionMetadata + KVCache + AttentionImpl::forward built from plain arguments
// (xllm/core/layers/dcu/attention.cpp:55-112).  q_cu_seq_lens undefined: decode, one token per sequence.
std::tuple<torch::Tensor, std::optional<torch::Tensor>> op_attention_layer_forward(
    torch::Tensor query, torch::Tensor key, torch::Tensor value, torch::Tensor k_cache, torch::Tensor v_cache,
    std::optional<torch::Tensor> k_cache_scale, std::optional<torch::Tensor> v_cache_scale, torch::Tensor slot_mapping,
    torch::Tensor block_table, torch::Tensor kv_seq_lens, std::optional<torch::Tensor> q_cu_seq_lens, int64_t max_seq_len,
    int64_t max_query_len, int64_t num_heads, int64_t head_size, int64_t num_kv_heads, double scale,
    int64_t sliding_window, bool is_causal, bool return_lse, std::optional<torch::Tensor> plan, int64_t layer_id) {
  xllm::layer::AttentionMetadata meta;
  if (layer_id >= 0) {  // the step's PlanInfo as this layer sees it: layer 0 fills `plan`, the others read it
    TORCH_CHECK(plan.has_value() && plan->defined(), "a layer with a layer_id needs the step's plan buffer");
    meta.plan_info = std::make_shared<xllm::layer::PlanInfo>();
    meta.plan_info->layer_id = static_cast<int32_t>(layer_id);
    meta.plan_info->plan_info = *plan;
  }
  meta.kv_seq_lens = kv_seq_lens;
  meta.block_table = block_table;
  meta.slot_mapping = slot_mapping;
  meta.max_seq_len = max_seq_len;
  meta.max_query_len = max_query_len;
  meta.is_causal = is_causal;
  if (q_cu_seq_lens.has_value() && q_cu_seq_lens->defined()) {
    meta.q_cu_seq_lens = *q_cu_seq_lens;
    meta.is_prefill = true;
    meta.is_chunked_prefill = true;
  }
  xllm::KVCache cache(k_cache, v_cache, k_cache_scale, v_cache_scale);
  xllm::layer::AttentionImpl attn(num_heads, head_size, static_cast<float>(scale), num_kv_heads, sliding_window, return_lse);
  return attn.forward(meta, query, key, value, cache);
}

std::tuple<torch::Tensor, torch::Tensor> op_mla_dense_decode(torch::Tensor q_nope, torch::Tensor q_pe,
                                                             torch::Tensor k_cache, torch::Tensor seqlens_k,
                                                             torch::Tensor block_table, int64_t head_size_v,
                                                             double softmax_scale, bool is_causal,
                                                             std::optional<torch::Tensor> plan,
                                                             std::optional<torch::Tensor> latent_cache,
                                                             std::optional<torch::Tensor> slot_mapping) {
  xllm::kernel::dcu::flash_mla::DenseDecodeParams p;
  p.q_nope = q_nope;
  p.q_pe = q_pe;
  p.k_cache = k_cache;
  p.seqlens_k = seqlens_k;
  p.block_table = block_table;
  p.head_size_v = head_size_v;
  p.softmax_scale = static_cast<float>(softmax_scale);
  p.is_causal = is_causal;
  p.kind = xllm::kernel::dcu::flash_mla::DenseDecodeKind::kQNopePe;
  torch::Tensor lse;
  if (latent_cache.has_value() && latent_cache->defined()) {   // the layer's store + decode in one call
    TORCH_CHECK(slot_mapping.has_value() && slot_mapping->defined(), "latent_cache and slot_mapping come together");
    torch::Tensor out = xllm::kernel::dcu::flash_mla::store_and_dense_decode(p, *latent_cache, *slot_mapping, plan, &lse);
    return {out, lse};
  }
  torch::Tensor out = plan.has_value() && plan->defined() ? xllm::kernel::dcu::flash_mla::dense_decode(p, *plan, &lse)
                                                          : xllm::kernel::dcu::flash_mla::dense_decode(p, &lse);
  return {out, lse};
}

torch::Tensor op_mla_decoding_metadata(torch::Tensor seqlens_k, torch::Tensor block_table, int64_t num_heads_per_head_k,
                                       int64_t block_size, std::optional<torch::Tensor> plan) {
  return xllm::kernel::dcu::flash_mla::get_mla_decoding_metadata(seqlens_k, block_table, num_heads_per_head_k, 1,
                                                                 block_size, plan)[0];
}

torch::Tensor op_paged_forward(torch::Tensor query, torch::Tensor output, torch::Tensor k_cache, torch::Tensor v_cache,
                               torch::Tensor block_table, torch::Tensor kv_seq_lens, torch::Tensor q_cu_seq_lens,
                               double scale, bool is_causal, int64_t max_seq_len, int64_t max_query_len) {
  xllm::kernel::mi355::paged_forward(query, output, k_cache, v_cache, block_table, kv_seq_lens, q_cu_seq_lens,
                                     static_cast<float>(scale), is_causal, max_seq_len, max_query_len);
  return output;
}

torch::Tensor op_gather_mla_latent_cache(torch::Tensor k_cache, torch::Tensor block_table,
                                         torch::Tensor kv_cu_seq_lens, int64_t total_kv_len, int64_t max_seq_len) {
  return xllm::kernel::mi355::gather_mla_latent_cache(k_cache, block_table, kv_cu_seq_lens, total_kv_len, max_seq_len);
}

torch::Tensor op_mask_block_table_padding(torch::Tensor block_table, torch::Tensor kv_seq_lens, int64_t page_block_size) {
  return xllm::kernel::mi355::mask_block_table_padding(block_table, kv_seq_lens, page_block_size);
}
torch::Tensor op_absorbed_bmm(torch::Tensor x, torch::Tensor w) { return xllm::kernel::mi355::absorbed_bmm(x, w); }

// (the reference's op returns the mutated qkv, xllm/core/kernels/cuda/cuda_ops_library.cpp:121-149, 280-284)
torch::Tensor op_fused_qk_norm_rope(torch::Tensor qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                           int64_t head_dim, double eps, torch::Tensor q_weight, torch::Tensor k_weight,
                           torch::Tensor cos_sin_cache, bool interleaved, torch::Tensor position_ids) {
  xllm::kernel::mi355::fused_qk_norm_rope(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight,
                                          cos_sin_cache, interleaved, position_ids);
  return qkv;
}

torch::Tensor op_fused_qk_norm_rope_and_cache(torch::Tensor qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                                     int64_t head_dim, double eps, torch::Tensor q_weight, torch::Tensor k_weight,
                                     torch::Tensor cos_sin_cache, bool interleaved, torch::Tensor position_ids,
                                     torch::Tensor slot_mapping, torch::Tensor key_cache, torch::Tensor value_cache,
                                     std::optional<torch::Tensor> k_scale, std::optional<torch::Tensor> v_scale) {
  xllm::kernel::ReshapePagedCacheParams p;
  p.k_cache = key_cache;
  p.v_cache = value_cache;
  p.slot_mapping = slot_mapping;
  p.k_cache_scale = k_scale;
  p.v_cache_scale = v_scale;
  xllm::kernel::mi355::fused_qk_norm_rope_and_cache(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight,
                                                    k_weight, cos_sin_cache, interleaved, position_ids, p);
  return qkv;
}

// xllm_ops::update_decode_graph_metadata of the reference, argument for argument
// (xllm/core/kernels/cuda/cuda_ops_library.cpp:161-252, schema :288-295): one token per sequence, the sizes
// taken from the tensors, returns dst_tokens.
torch::Tensor op_update_decode_graph_metadata(torch::Tensor tokens, torch::Tensor positions, torch::Tensor slot_mapping,
                                              torch::Tensor kv_seq_lens, torch::Tensor paged_kv_indptr,
                                              torch::Tensor paged_kv_indices, torch::Tensor paged_kv_last_page_len,
                                              torch::Tensor dst_tokens, torch::Tensor dst_positions,
                                              torch::Tensor dst_slot_mapping, torch::Tensor dst_kv_seq_lens,
                                              torch::Tensor dst_kv_seq_lens_delta, torch::Tensor dst_paged_kv_indptr,
                                              torch::Tensor dst_paged_kv_indices,
                                              torch::Tensor dst_paged_kv_last_page_len, int64_t padded_num_tokens) {
  for (const torch::Tensor* t : {&tokens, &positions, &slot_mapping, &kv_seq_lens, &paged_kv_indptr, &paged_kv_indices,
                                 &paged_kv_last_page_len, &dst_tokens, &dst_positions, &dst_slot_mapping,
                                 &dst_kv_seq_lens, &dst_kv_seq_lens_delta, &dst_paged_kv_indptr, &dst_paged_kv_indices,
                                 &dst_paged_kv_last_page_len})
    TORCH_CHECK(t->defined() && t->is_cuda() && t->scalar_type() == torch::kInt32 && t->is_contiguous(),
                "update_decode_graph_metadata takes contiguous int32 device tensors");
  const int64_t actual_num_tokens = tokens.numel();
  const int64_t actual_batch_size = paged_kv_last_page_len.numel();
  const int64_t actual_indices_size = paged_kv_indices.numel();
  TORCH_CHECK(actual_num_tokens == actual_batch_size, "decode graph requires one token per sequence");
  TORCH_CHECK(padded_num_tokens >= actual_num_tokens && positions.numel() >= actual_num_tokens &&
                  slot_mapping.numel() >= actual_num_tokens && kv_seq_lens.numel() >= actual_batch_size + 1 &&
                  paged_kv_indptr.numel() >= actual_batch_size + 1,
              "source tensors shorter than the step");
  TORCH_CHECK(dst_tokens.numel() >= padded_num_tokens && dst_positions.numel() >= padded_num_tokens &&
                  dst_slot_mapping.numel() >= padded_num_tokens && dst_kv_seq_lens.numel() >= padded_num_tokens + 1 &&
                  dst_kv_seq_lens_delta.numel() >= padded_num_tokens &&
                  dst_paged_kv_indptr.numel() >= padded_num_tokens + 1 &&
                  dst_paged_kv_indices.numel() >= actual_indices_size &&
                  dst_paged_kv_last_page_len.numel() >= padded_num_tokens,
              "persistent tensors shorter than the padded step");
  auto ptr = [](const torch::Tensor& t) { return t.numel() > 0 ? t.data_ptr<int32_t>() : nullptr; };
  xllm::kernel::mi355::LlmDecodeMetadataUpdateParams p{
      ptr(tokens), ptr(positions), ptr(slot_mapping), ptr(kv_seq_lens), ptr(paged_kv_indptr), ptr(paged_kv_indices),
      ptr(paged_kv_last_page_len), ptr(dst_tokens), ptr(dst_positions), ptr(dst_slot_mapping), ptr(dst_kv_seq_lens),
      ptr(dst_kv_seq_lens_delta), ptr(dst_paged_kv_indptr), ptr(dst_paged_kv_indices), ptr(dst_paged_kv_last_page_len),
      actual_num_tokens, padded_num_tokens, actual_batch_size, actual_indices_size};
  xllm::kernel::mi355::update_llm_decode_metadata(p, current_stream(dst_tokens));
  return dst_tokens;
}

std::tuple<torch::Tensor, torch::Tensor> op_merge(torch::Tensor partial_outputs, torch::Tensor partial_lse) {
  auto r = xllm::layer::merge_dcp_attention_shards(partial_outputs, partial_lse);
  return {r.output, r.lse};
}

}  // namespace

TORCH_LIBRARY(xllm_ops, m) {
  m.def("reshape_paged_cache(Tensor slot_mapping, Tensor keys, Tensor values, Tensor(a!) key_cache, "
        "Tensor(b!) value_cache) -> Tensor");
  m.def("quant_to_paged_cache(Tensor slot_mapping, Tensor keys, Tensor values, Tensor(a!) key_cache, "
        "Tensor(b!) value_cache, Tensor k_scale, Tensor v_scale) -> Tensor");
  m.def("batch_decode(Tensor query, Tensor k_cache, Tensor v_cache, Tensor(a!) output, Tensor block_table, "
        "Tensor seq_lens, Tensor? k_scale, Tensor? v_scale, int max_seq_len, float scale, Tensor? plan=None) -> (Tensor, Tensor)");
  m.def("update_decode_plan(Tensor block_table, Tensor seq_lens, int num_qo_heads, int num_kv_heads, int head_dim, "
        "int block_size, int window_left, bool fp8_cache, Tensor(a!)? plan=None) -> Tensor");
  m.def("mla_dense_decode(Tensor q_nope, Tensor q_pe, Tensor(a!) k_cache, Tensor seqlens_k, Tensor block_table, "
        "int head_size_v, float softmax_scale, bool is_causal=False, Tensor? plan=None, Tensor? latent_cache=None, "
        "Tensor? slot_mapping=None) -> (Tensor, Tensor)");
  m.def("mla_decoding_metadata(Tensor seqlens_k, Tensor block_table, int num_heads_per_head_k, int block_size, "
        "Tensor(a!)? plan=None) -> Tensor");
  m.def("lse_combine(Tensor(a!) output, Tensor shared_o, Tensor shared_lse, Tensor unshared_o, Tensor unshared_lse) -> Tensor");
  m.def("attention_layer_forward(Tensor query, Tensor key, Tensor value, Tensor(a!) k_cache, Tensor(b!) v_cache, "
        "Tensor? k_cache_scale, Tensor? v_cache_scale, Tensor slot_mapping, Tensor block_table, Tensor kv_seq_lens, "
        "Tensor? q_cu_seq_lens, int max_seq_len, int max_query_len, int num_heads, int head_size, int num_kv_heads, "
        "float scale, int sliding_window, bool is_causal, bool return_lse, Tensor(c!)? plan=None, int layer_id=-1) "
        "-> (Tensor, Tensor?)");
  m.def("merge_dcp_attention_shards(Tensor partial_outputs, Tensor partial_lse) -> (Tensor, Tensor)");
  m.def("paged_forward(Tensor query, Tensor(a!) output, Tensor k_cache, Tensor v_cache, Tensor block_table, "
        "Tensor kv_seq_lens, Tensor q_cu_seq_lens, float scale, bool is_causal, int max_seq_len, int max_query_len) -> Tensor");
  m.def("gather_mla_latent_cache(Tensor k_cache, Tensor block_table, Tensor kv_cu_seq_lens, int total_kv_len, "
        "int max_seq_len) -> Tensor");
  m.def("mla_absorbed_bmm(Tensor x, Tensor w) -> Tensor");
  m.def("mask_block_table_padding(Tensor block_table, Tensor kv_seq_lens, int page_block_size) -> Tensor");
  m.def("update_decode_graph_metadata(Tensor tokens, Tensor positions, Tensor slot_mapping, Tensor kv_seq_lens, "
        "Tensor paged_kv_indptr, Tensor paged_kv_indices, Tensor paged_kv_last_page_len, Tensor(a!) dst_tokens, "
        "Tensor(b!) dst_positions, Tensor(c!) dst_slot_mapping, Tensor(d!) dst_kv_seq_lens, "
        "Tensor(e!) dst_kv_seq_lens_delta, Tensor(f!) dst_paged_kv_indptr, Tensor(g!) dst_paged_kv_indices, "
        "Tensor(h!) dst_paged_kv_last_page_len, int padded_num_tokens) -> Tensor(a!)");
  m.def("fused_qk_norm_rope(Tensor(a!) qkv, int num_heads_q, int num_heads_k, int num_heads_v, int head_dim, "
        "float eps, Tensor q_weight, Tensor k_weight, Tensor cos_sin_cache, bool interleaved, Tensor position_ids) -> Tensor");
  m.def("fused_qk_norm_rope_and_cache(Tensor(a!) qkv, int num_heads_q, int num_heads_k, int num_heads_v, int head_dim, "
        "float eps, Tensor q_weight, Tensor k_weight, Tensor cos_sin_cache, bool interleaved, Tensor position_ids, "
        "Tensor slot_mapping, Tensor(b!) key_cache, Tensor(c!) value_cache, Tensor? k_scale, Tensor? v_scale) -> Tensor");
}

TORCH_LIBRARY_IMPL(xllm_ops, CUDA, m) {
  m.impl("reshape_paged_cache", &op_reshape_paged_cache);
  m.impl("quant_to_paged_cache", &op_quant_to_paged_cache);
  m.impl("batch_decode", &op_batch_decode);
  m.impl("update_decode_plan", &op_update_decode_plan);
  m.impl("mla_dense_decode", &op_mla_dense_decode);
  m.impl("mla_decoding_metadata", &op_mla_decoding_metadata);
  m.impl("lse_combine", &op_lse_combine);
  m.impl("attention_layer_forward", &op_attention_layer_forward);
  m.impl("merge_dcp_attention_shards", &op_merge);
  m.impl("paged_forward", &op_paged_forward);
  m.impl("gather_mla_latent_cache", &op_gather_mla_latent_cache);
  m.impl("mla_absorbed_bmm", &op_absorbed_bmm);
  m.impl("mask_block_table_padding", &op_mask_block_table_padding);
  m.impl("update_decode_graph_metadata", &op_update_decode_graph_metadata);
  m.impl("fused_qk_norm_rope", &op_fused_qk_norm_rope);
  m.impl("fused_qk_norm_rope_and_cache", &op_fused_qk_norm_rope_and_cache);
}
