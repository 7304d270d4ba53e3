/*
 * xllm_mi355.h -- C ABI of the MI355X (gfx950) paged-KV decode path.
 *
 * Two operations and their helpers:
 *   1. reshape_and_cache: scatter new K/V token rows into block-table-addressed
 *      cache pages, optionally quantising to fp8 e4m3fn with per-KV-head scales.
 *   2. paged decode attention: GQA (block-table and CSR addressing) and the MLA
 *      latent-KV variant, split over long contexts with a log-sum-exp merge.
 *
 * All pointers are DEVICE pointers unless a comment says "host".  Every entry
 * point only enqueues work on `stream` (a hipStream_t passed as void*); none of
 * them synchronises, allocates or frees device memory, or reads device memory
 * from the host, so they are legal inside a HIP graph capture.
 *
 * Return value of every int function: 0 = ok; negative = argument error
 * (XLLM_MI355_E*); positive = a hipError_t raised by a launch.
 * The reference aborts the process on a failed CHECK; the C++ shim above this
 * ABI turns a non-zero return into the same abort.
 *
 * Tensor layouts follow the reference (paths relative to the xLLM source tree):
 *   key/value          [T, Hkv, D]      last two dims contiguous, token stride free
 *                                       (xllm/core/kernels/param.h:126-161)
 *   k_cache/v_cache    [P, bs, Hkv, D]  contiguous
 *                                       (xllm/core/framework/kv_cache/kv_cache_shape.cpp:303-311)
 *   MLA latent cache   [P, bs, 1, d_latent + d_rope], no V cache
 *                                       (kv_cache_shape.cpp:433-441)
 *   slot_mapping       [T] int32, slot = page * bs + offset, negative = skip
 *                                       (xllm/core/kernels/cuda/reshape_paged_cache.cu:36-41)
 *   block_table        [B, >= ceil(L/bs)] int32 rows with a row stride; entries
 *                      past ceil(L/bs) are never read (padding may be 0 or -1)
 *   seq_lens           [B] int32, context length including the new token
 *   LSE                natural log, fp32, [B, Hq]
 *                                       (tests/core/layers/mlu/dcp_attention_merge_test.cpp:127-143)
 */
#ifndef XLLM_MI355_H_
#define XLLM_MI355_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types. */
enum {
  XLLM_MI355_BF16 = 0,
  XLLM_MI355_FP16 = 1,
  XLLM_MI355_FP32 = 2,
  XLLM_MI355_FP8_E4M3 = 3 /* OCP e4m3fn, the format of torch.float8_e4m3fn */
};

/* Argument errors. */
enum {
  XLLM_MI355_OK = 0,
  XLLM_MI355_EINVAL = -1,      /* null pointer, non-positive size, bad stride   */
  XLLM_MI355_EDTYPE = -2,      /* dtype combination not implemented             */
  XLLM_MI355_ESHAPE = -3,      /* head_dim / group / block size not implemented */
  XLLM_MI355_EWORKSPACE = -4,  /* workspace missing or too small                */
  XLLM_MI355_EALIGN = -5,      /* pointer or stride not 16-byte aligned         */
  XLLM_MI355_ESTALLED = -6,    /* xllm_mi355_decode_status: a bounded wait inside a decode kernel gave up */
  XLLM_MI355_ESCRATCH = -7,    /* the problem does not fit the static scratch of the no-allocation entry point */
  XLLM_MI355_EPLAN = -8        /* xllm_mi355_decode_status: a decode launch met a plan made for another shape or other lengths */
};

/* Human-readable text for a return code of this library (host pointer, static). */
const char* xllm_mi355_error_string(int code);

/* Library version, "major.minor.patch" (host pointer, static). */
const char* xllm_mi355_version(void);

/*
 * reshape_and_cache.
 * Replaces xllm::kernel::reshape_paged_cache (xllm/core/kernels/ops_api.h:31,
 * ops_api.cpp:248-278) and its CUDA kernel (kernels/cuda/reshape_paged_cache.cu:23-99).
 * With cache_dtype == XLLM_MI355_FP8_E4M3 it also covers the quantising store
 * selected where the cache carries scales (xllm/core/layers/mlu/attention.cpp:109-117),
 * using the reference's fp8 convention (kernels/cuda/fp8_quant.cu:92-103,
 * fp8_quant_utils.cuh:111-130):
 *     q = e4m3fn_rne(fmaxf(-448, fminf(float(x) * (1.0f / scale[h]), 448)))
 * `value` and `v_cache` may both be null (MLA latent store, the counterpart of
 * xllm/core/layers/dcu/deepseek_v2_attention.cpp:221-229).
 * Slots < 0 are skipped as in the reference; slots >= num_blocks * block_size
 * are skipped too (the reference leaves them undefined).
 * k_scale / v_scale: [Hkv] fp32, required iff cache_dtype is fp8.
 * Token strides are in elements.
 */
int xllm_mi355_reshape_and_cache(const void* key, const void* value,
                                 void* k_cache, void* v_cache,
                                 const int32_t* slot_mapping,
                                 const float* k_scale, const float* v_scale,
                                 int64_t n_tokens, int64_t n_kv_heads, int64_t head_dim,
                                 int64_t block_size, int64_t num_blocks,
                                 int64_t k_token_stride, int64_t v_token_stride,
                                 int in_dtype, int cache_dtype, void* stream);

/*
 * Per-KV-head fp8 scales: scale[h] = max(absmax(x[:, h, :]) / 448, 1e-12).
 * Replaces the dynamic branch of xllm::kernel::cuda::fp8_scaled_quantize
 * (xllm/core/kernels/cuda/fp8_scaled_quantize.cpp:38-42) at per-head granularity.
 * scales: [Hkv] fp32, fully overwritten.
 */
int xllm_mi355_kv_head_scales(const void* x, float* scales,
                              int64_t n_tokens, int64_t n_kv_heads, int64_t head_dim,
                              int64_t token_stride, int in_dtype, void* stream);

/*
 * Bytes of split-K workspace the decode entry points need for this problem.
 * max_seq_len is an upper bound on every seq_lens[b] (AttentionMetadata::max_seq_len,
 * xllm/core/layers/common/attention_metadata.h:99-156).  Counterpart of the
 * FlashInfer float workspace (xllm/core/layers/cuda/flashinfer_workspace.cpp:25-41).
 */
size_t xllm_mi355_paged_decode_gqa_workspace_bytes(int64_t batch, int64_t n_q_heads, int64_t head_dim);
size_t xllm_mi355_paged_decode_mla_workspace_bytes(int64_t batch, int64_t n_heads, int64_t max_seq_len);
/* The first form of the two above, kept for existing callers: it takes v_head_dim == 512 to mean the MLA latent
 * and every other width to be a GQA head dim.  New code names the variant. */
size_t xllm_mi355_paged_decode_workspace_bytes(int64_t batch, int64_t n_q_heads,
                                               int64_t v_head_dim, int64_t max_seq_len);

/*
 * The decode workspace.  Counterpart of the process-wide FlashInfer workspace of the reference
 * (xllm/core/layers/cuda/flashinfer_workspace.cpp:25-41: allocated once, handed to every layer's decode call).
 * Layout, the same for every decode entry point and independent of the batch, so that a launch recorded in a
 * HIP graph keeps meaning the same addresses whatever later calls ask for:
 *     256 bytes of header (word 0: status flags) | item prefix of up to 2048 sequences | fp32 partial slots
 * xllm_mi355_decode_workspace_bound() is a size that serves every GQA call, MLA calls with up to 1024 heads and
 * varlen calls of up to 65536 query tokens (about 135 MB on a GPU with 256 CUs): allocate that much once per
 * device and never replace it while graphs that captured a decode call are alive.
 * xllm_mi355_decode_workspace_init clears the header; call it once after allocating (it is a small fill kernel
 * on `stream`, legal under capture).
 * ONE workspace serves ONE stream at a time: two decode calls that use the same workspace and overlap in time
 * (two streams of one device, or two graphs replayed concurrently) overwrite each other's partial results.
 * Give every stream that decodes concurrently a workspace of its own.  The reference has the same rule: its
 * workspace is a per-process singleton used from the one worker thread and stream of a device.
 *
 * xllm_mi355_decode_status is the voice of the kernels: the wavefronts of the matrix-core GQA kernel wait for
 * each other with bounded polls; if a poll ever runs out, the wavefront sets a flag in the header and exits,
 * and the outputs of that launch are invalid.  The call waits for `stream`, reads the flag from the host and
 * clears it: 0 = no launch since the last call gave up, XLLM_MI355_ESTALLED otherwise (XLLM_MI355_EPLAN when the
 * flag is that of a planned call whose plan was made for another shape, see xllm_mi355_paged_decode_gqa_plan).  It synchronises, so it
 * is for use outside graph capture (for example once per step, or when a result looks wrong).  The reference
 * has no counterpart (its fast paths are closed libraries that abort on error).
 */
size_t xllm_mi355_decode_workspace_bound(void);
int xllm_mi355_decode_workspace_init(void* workspace, size_t workspace_bytes, void* stream);
int xllm_mi355_decode_status(void* workspace, void* stream);

/*
 * Paged decode attention, GQA, block-table addressing.
 * Replaces xllm::kernel::npu::batch_decode (xllm/core/kernels/npu/npu_ops_api.h:46,
 * npu/attention.cpp:26-78,141-167) and the block-table subset of
 * xllm::kernel::mlu::batch_decode (kernels/mlu/mlu_ops_api.h:127):
 *     out[b, h, :] = softmax(sm_scale * q[b, h, :] . K_b[:, h / group, :]^T) . V_b[:, h / group, :]
 * q/out: [B, Hq, D] with token strides in elements; lse: [B, Hq] fp32 natural log or null.
 * k_scale / v_scale: [Hkv] fp32, required iff cache_dtype is fp8 (dequantised value
 * = float(code) * scale[h]).  q_dtype also is the dtype of `out`: XLLM_MI355_BF16 or XLLM_MI355_FP16 over pages of the
 * same type or fp8 pages, or XLLM_MI355_FP32 over fp32 pages (what reshape_and_cache stores for an fp32 model: a
 * compatibility path, one workgroup per query head and sequence, no workspace needed).
 * max_seq_len <= 0 means "table_stride * block_size".
 * window_left: sliding window (window_left of xllm/core/kernels/cuda/cuda_ops_api.h:139; sliding_window_ of
 * xllm/core/layers/dcu/flash_attention.cpp:484): the query, at position L - 1, attends to positions
 * >= L - 1 - window_left; negative = the whole context.  Pages that lie wholly before the window are not read.
 * A sequence with seq_lens[b] <= 0 gets out = 0 and lse = -inf.
 */
int xllm_mi355_paged_decode_gqa(const void* q, const void* k_cache, const void* v_cache,
                                void* out, float* lse,
                                const int32_t* block_table, int64_t table_stride,
                                const int32_t* seq_lens,
                                const float* k_scale, const float* v_scale,
                                int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                int64_t q_token_stride, int64_t out_token_stride,
                                int64_t max_seq_len, int64_t window_left, float sm_scale,
                                void* workspace, size_t workspace_bytes,
                                int q_dtype, int cache_dtype, void* stream);

/*
 * xllm_mi355_paged_decode_gqa without a workspace argument and without any allocation, for callers that
 * cannot allocate: code under HIP graph capture whose workspace was not set up beforehand, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, same
 * kernels and bit-identical results; the partial results of contexts that span several workers go to a
 * scratch array inside the library's code object (XLLM_MI355_STATIC_SCRATCH_BYTES per GPU, held until the
 * process ends).  Limits: batch <= 2048, and a shape whose partial slots fit the scratch (every shape of the
 * matrix-core kernel does; XLLM_MI355_ESCRATCH otherwise).  Every call on a GPU shares that GPU's scratch:
 * calls that overlap in time on one GPU (two streams, two threads) race on it.  Nothing in it needs to start
 * at zero except the status word, which only xllm_mi355_decode_status(NULL, stream) clears.  The first call on
 * a device looks the scratch address up (hipGetSymbolAddress): make it outside graph capture.
 */
#define XLLM_MI355_STATIC_SCRATCH_BYTES (36u << 20)
int xllm_mi355_paged_decode_gqa_static(const void* q, const void* k_cache, const void* v_cache,
                                       void* out, float* lse,
                                       const int32_t* block_table, int64_t table_stride,
                                       const int32_t* seq_lens,
                                       const float* k_scale, const float* v_scale,
                                       int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                       int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                       int64_t q_token_stride, int64_t out_token_stride,
                                       int64_t max_seq_len, int64_t window_left, float sm_scale,
                                       int q_dtype, int cache_dtype, void* stream);

/*
 * Same, CSR addressing.  Replaces xllm::kernel::cuda::batch_decode
 * (xllm/core/kernels/cuda/cuda_ops_api.h:128-144, cuda/batch_decode.cpp:26-86) without
 * its FlashInfer plan/uri/workspace triple, and the decode branch of
 * TorchAttentionImpl::forward (xllm/core/layers/dcu/torch_attention.cpp:285-347):
 * pages of sequence b are paged_kv_indices[indptr[b] .. indptr[b+1]), the last of
 * them holds paged_kv_last_page_len[b] tokens.
 */
int xllm_mi355_paged_decode_gqa_csr(const void* q, const void* k_cache, const void* v_cache,
                                    void* out, float* lse,
                                    const int32_t* paged_kv_indptr,
                                    const int32_t* paged_kv_indices,
                                    const int32_t* paged_kv_last_page_len,
                                    const float* k_scale, const float* v_scale,
                                    int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                    int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                    int64_t q_token_stride, int64_t out_token_stride,
                                    int64_t max_seq_len, int64_t window_left, float sm_scale,
                                    void* workspace, size_t workspace_bytes,
                                    int q_dtype, int cache_dtype, void* stream);

/*
 * The plan of a decode step, made once and used by the decode calls of every layer: the counterpart of the
 * reference's FlashInfer plan, which update_decode_plan_info computes at layer 0 only and every layer's
 * batch_decode then takes (xllm/core/layers/cuda/flashinfer_planinfo.cpp:248-264 with the early return of :263-264
 * for layer_id != 0; plan_info argument of xllm/core/kernels/cuda/cuda_ops_api.h:128-144).
 * xllm_mi355_paged_decode_gqa_plan is one small launch that writes into `plan` (device memory of
 * xllm_mi355_paged_decode_plan_bytes() bytes, 256-byte aligned, the caller's): the prefix of the per-sequence work
 * items, where the work list is cut between the workers, and for every group of workers the page-table entries
 * its first loads need.  xllm_mi355_paged_decode_gqa_planned is xllm_mi355_paged_decode_gqa (block_table form,
 * paged_kv_indptr == NULL) or xllm_mi355_paged_decode_gqa_csr (paged_kv_indptr != NULL) that starts from the plan
 * instead of deriving all that in every launch: same kernels, same order of arithmetic, bit-identical results.
 * The plan holds for the sequence lengths, tables, head counts, head dim, block size, window and cache dtype it
 * was made with: make it again when any of them changes (every decode step).  Shapes that the matrix-core kernel
 * does not serve take no plan and are decoded as by the plain entry points.  A stale plan is reported, not
 * followed silently: a planned call whose shape differs from the plan's writes no output, and one whose sequence
 * lengths differ from those the plan was made with (the plan keeps them; the same shape one step later, a forgotten
 * re-plan) writes an output that is invalid; both raise a flag that xllm_mi355_decode_status reports as
 * XLLM_MI355_EPLAN.  Page ids that changed under unchanged lengths are not detected (page ids are clamped: the reads
 * of such a call stay inside the caches).  plan_bytes is the size of the caller's buffer: a planned call reads the
 * plan up to its last word, and a buffer below xllm_mi355_paged_decode_plan_bytes() is refused with
 * XLLM_MI355_EWORKSPACE before anything is launched.  Plan and planned calls are plain
 * launches on `stream` (legal under graph capture; a replay plans again from the current lengths).
 */
size_t xllm_mi355_paged_decode_plan_bytes(void);
int xllm_mi355_paged_decode_gqa_plan(void* plan, size_t plan_bytes,
                                     const int32_t* block_table, int64_t table_stride,
                                     const int32_t* seq_lens,
                                     const int32_t* paged_kv_indptr, const int32_t* paged_kv_indices,
                                     const int32_t* paged_kv_last_page_len,
                                     int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                     int64_t head_dim, int64_t block_size, int64_t window_left,
                                     int cache_dtype, void* stream);
int xllm_mi355_paged_decode_gqa_planned(const void* plan, size_t plan_bytes,
                                        const void* q, const void* k_cache, const void* v_cache,
                                        void* out, float* lse,
                                        const int32_t* block_table, int64_t table_stride,
                                        const int32_t* seq_lens,
                                        const int32_t* paged_kv_indptr, const int32_t* paged_kv_indices,
                                        const int32_t* paged_kv_last_page_len,
                                        const float* k_scale, const float* v_scale,
                                        int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                        int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                        int64_t q_token_stride, int64_t out_token_stride,
                                        int64_t max_seq_len, int64_t window_left, float sm_scale,
                                        void* workspace, size_t workspace_bytes,
                                        int q_dtype, int cache_dtype, void* stream);

/*
 * One decode step of an attention layer in one call: store the step's K / V rows, then attend.  Replaces the pair
 * that the reference's attention layer issues per layer and step, reshape_paged_cache followed by batch_decode
 * (xllm/core/layers/dcu/torch_attention.cpp:138-144 then :285-347; xllm/core/layers/cuda/flashinfer_attention.cpp
 * :136-142 then :329), with the arguments of xllm_mi355_reshape_and_cache (key, value [batch, Hkv, D]
 * of q's dtype, token strides in elements, slot_mapping [batch]) in front of those of
 * xllm_mi355_paged_decode_gqa_planned.  plan may be NULL (then plan_bytes is ignored and the call derives its
 * schedule itself).  Sequence b's slot must be the place of its token seq_lens[b] - 1 in its block table (what the
 * reference's slot mapping holds on a decode step); negative slots and slots beyond the cache are skipped, and such a
 * sequence attends to whatever its table holds.  The caches and `out` afterwards hold the same bytes as after
 * xllm_mi355_reshape_and_cache followed by the decode call.  Where the matrix-core kernel serves the shape (16-bit or
 * fp8 pages of a power-of-two block size >= 16, head dim 64 / 128 / 256; key / value 16-byte
 * aligned with strides that are multiples of 8 elements) the rows are written inside the decode launch, by the
 * worker that attends to the context's last tokens, and the step saves a launch; otherwise the library issues the
 * two launches itself.  The caches are written: a sequence with seq_lens[b] == 0 has no token to store and stores
 * none in the one-launch form.
 */
int xllm_mi355_write_and_decode_gqa(const void* key, const void* value, const int32_t* slot_mapping,
                                    int64_t k_token_stride, int64_t v_token_stride,
                                    const void* plan, size_t plan_bytes,
                                    const void* q, void* k_cache, void* v_cache, void* out, float* lse,
                                    const int32_t* block_table, int64_t table_stride,
                                    const int32_t* seq_lens,
                                    const int32_t* paged_kv_indptr, const int32_t* paged_kv_indices,
                                    const int32_t* paged_kv_last_page_len,
                                    const float* k_scale, const float* v_scale,
                                    int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                    int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                    int64_t q_token_stride, int64_t out_token_stride,
                                    int64_t max_seq_len, int64_t window_left, float sm_scale,
                                    void* workspace, size_t workspace_bytes,
                                    int q_dtype, int cache_dtype, void* stream);

/*
 * Rows of paged sequences gathered into one packed buffer, sequence after sequence.
 * Replaces xllm::kernel::dcu::gather_mla_latent_cache
 * (xllm/core/kernels/dcu/gather_mla_latent_cache.hip:32-75,124-190; declared in dcu_ops_api.h:74; called for
 * prefill with context at layers/dcu/deepseek_v2_attention.cpp:324):
 *     out[cu_seq_lens[b] + t, :] = cache[block_table[b, t / bs] * bs + t % bs, :]   for t < cu[b+1] - cu[b]
 * cache: [P, bs, row_bytes] contiguous (for the latent cache row_bytes = (kv_lora_rank + rope) * 2);
 * cu_seq_lens: [B + 1] int32 starting at 0; out: [total_rows, row_bytes].  Rows whose page id is negative
 * (table padding) or not below num_blocks are left untouched.
 */
int xllm_mi355_gather_paged_rows(const void* cache, const int32_t* block_table, int64_t table_stride,
                                 const int32_t* cu_seq_lens, void* out,
                                 int64_t batch, int64_t total_rows, int64_t block_size,
                                 int64_t num_blocks, int64_t row_bytes, void* stream);

/*
 * The per-head products either side of the MLA decode, on the matrix cores:
 *     y[t, h, :] = x[t, h, :] . w[h, :, :]
 * Replaces the two torch::bmm calls of the reference's absorbed MLA attention
 * (xllm/core/layers/dcu/deepseek_v2_attention.cpp:428-430: q_nope [T, H, 128] with w_kc_ [H, 128, 512] into the
 * q_nope operand of xllm_mi355_paged_decode_mla; :231-238: the decode output [T, H, 512] with w_vc_ [H, 512, 128]
 * into the input of o_proj), with the weights in the layouts the reference prepares at load time (:479-485).
 * x: [T, H, K] with free token and head strides (q_nope is a slice of q); w: [H, K, N] contiguous;
 * y: [T, H, N] with free token and head strides; strides in elements.  fp32 accumulation, one rounding to
 * dtype at the end.  dtype: XLLM_MI355_BF16.  K must be a multiple of 128, N of 64; pointers and strides
 * multiples of 16 bytes.
 */
int xllm_mi355_mla_absorbed_bmm(const void* x, const void* w, void* y,
                                int64_t n_tokens, int64_t n_heads, int64_t k, int64_t n,
                                int64_t x_token_stride, int64_t x_head_stride,
                                int64_t y_token_stride, int64_t y_head_stride,
                                int dtype, void* stream);

/*
 * Short query chunks through the decode kernels: chunked prefill and speculative-decoding
 * verification with a few query tokens per sequence.  Replaces the decode branch of
 * FlashAttentionImpl::paged_forward (xllm/core/layers/dcu/flash_attention.cpp:447-545: packed q
 * [total_tokens, Hq, D] with q_cu_seq_lens, hg_prefix_decode_varlen_fwd for chunks of up to 16 tokens):
 *     token j of the q_len = cu[b+1] - cu[b] tokens of sequence b attends to the first
 *     kv_seq_lens[b] - q_len + j + 1 tokens of its context when causal != 0 (the chunk is the
 *     tail of the context, AttentionMetadata::is_causal), to all kv_seq_lens[b] otherwise.
 * q/out: [n_tokens, Hq, D]; cu_seqlens_q: [B + 1] int32 starting at 0; block_table: [B, table_stride].
 * max_q_len is the caller's bound on the chunk lengths (AttentionMetadata::max_query_len), 0 if unknown.
 * With a bound (head dim 128, block size a power of two >= 16, Hq / Hkv <= 8 or the whole chunk in 16 columns)
 * the (token, head) pairs of a chunk share the 16 columns of the matrix-core kernel: the pages of a sequence
 * are read once per 16 / (Hq / Hkv) query tokens; the tokens of a chunk beyond the bound are left unwritten (the
 * others still attend to the right prefix), so the bound must hold.  Otherwise
 * (and always with a sliding window, window_left >= 0, which then counts from each token's own last attended
 * position) every query token is decoded as an entry of its own against its sequence's pages (read once per
 * token, partly from L2), which is correct for any length.
 * Workspace: xllm_mi355_paged_decode_varlen_workspace_bytes(max(n_tokens, batch), ...); the per-token arrays
 * take its last bytes, so pass the same workspace_bytes on every call that shares a captured graph.
 */
size_t xllm_mi355_paged_decode_varlen_workspace_bytes(int64_t n_tokens, int64_t n_q_heads,
                                                      int64_t head_dim);
int xllm_mi355_paged_decode_gqa_varlen(const void* q, const void* k_cache, const void* v_cache,
                                       void* out,
                                       const int32_t* cu_seqlens_q, const int32_t* kv_seq_lens,
                                       const int32_t* block_table, int64_t table_stride,
                                       const float* k_scale, const float* v_scale,
                                       int64_t batch, int64_t n_tokens, int64_t max_q_len,
                                       int64_t n_q_heads,
                                       int64_t n_kv_heads, int64_t head_dim, int64_t block_size,
                                       int64_t num_blocks, int64_t q_token_stride,
                                       int64_t out_token_stride, int64_t max_seq_len, int64_t window_left,
                                       float sm_scale, int causal, void* workspace, size_t workspace_bytes,
                                       int q_dtype, int cache_dtype, void* stream);

/*
 * Paged decode attention, MLA latent-KV variant.
 * Replaces xllm::kernel::dcu::flash_mla::dense_decode
 * (xllm/core/kernels/dcu/flash_mla_adapter.h:40-53, flash_mla_adapter.cpp:104-153):
 *     out[b, h, :] = softmax(sm_scale * [q_nope | q_pe][b, h, :] . C_b^T) . C_b[:, :d_latent]
 * with C_b the latent rows of sequence b, [L_b, d_latent + d_rope].
 * q_nope: [B, H, d_latent], q_pe: [B, H, d_rope], out: [B, H, d_latent], all contiguous and of `dtype`
 * (XLLM_MI355_BF16 or XLLM_MI355_FP16: "BF16/FP16", flash_mla_adapter.cpp:105-107); k_cache:
 * [P, bs, 1, d_latent + d_rope] of the same type.  d_latent 512, d_rope 64.  The S_q query tokens of a
 * multi-token step are passed as S_q * H heads (the adapter folds them the same way, :119-123).
 */
int xllm_mi355_paged_decode_mla(const void* q_nope, const void* q_pe, const void* k_cache,
                                void* out, float* lse,
                                const int32_t* block_table, int64_t table_stride,
                                const int32_t* seq_lens,
                                int64_t batch, int64_t n_heads,
                                int64_t d_latent, int64_t d_rope,
                                int64_t block_size, int64_t num_blocks,
                                int64_t max_seq_len, float sm_scale,
                                void* workspace, size_t workspace_bytes,
                                int dtype, void* stream);

/*
 * The plan of an MLA decode step, made once and used by the decode calls of every layer: the counterpart of the
 * tile-scheduler metadata that the reference computes apart from the decode call
 * (get_mla_decoding_metadata_dense_fp8, xllm/core/kernels/dcu/flash_mla_adapter.cpp:125-130) and of the plan that its
 * FlashInfer path makes at layer 0 only (xllm/core/layers/cuda/flashinfer_planinfo.cpp:248-264).  Same buffer as the
 * GQA plan (xllm_mi355_paged_decode_plan_bytes() bytes, 256-byte aligned, the caller's), same rules: one small launch
 * writes the schedule's prefix, the lengths and every workgroup team's first page-table entries;
 * xllm_mi355_paged_decode_mla_planned is xllm_mi355_paged_decode_mla that starts from them: same kernel, same order of
 * arithmetic, bit-identical results.  A plan serves the kernel for more than 64 heads with a block size that is a
 * power of two >= 16 and batches of at most 1024 sequences; other calls take no plan and are decoded as by the plain
 * entry point.  A planned call whose shape differs from the plan's writes no output, one whose lengths differ from
 * those the plan was made with writes an invalid one; both raise the flag that xllm_mi355_decode_status reports as
 * XLLM_MI355_EPLAN.  A plan buffer below xllm_mi355_paged_decode_plan_bytes() is refused with XLLM_MI355_EWORKSPACE.
 */
int xllm_mi355_paged_decode_mla_plan(void* plan, size_t plan_bytes,
                                     const int32_t* block_table, int64_t table_stride,
                                     const int32_t* seq_lens,
                                     int64_t batch, int64_t n_heads, int64_t block_size, void* stream);
int xllm_mi355_paged_decode_mla_planned(const void* plan, size_t plan_bytes,
                                        const void* q_nope, const void* q_pe, const void* k_cache,
                                        void* out, float* lse,
                                        const int32_t* block_table, int64_t table_stride,
                                        const int32_t* seq_lens,
                                        int64_t batch, int64_t n_heads,
                                        int64_t d_latent, int64_t d_rope,
                                        int64_t block_size, int64_t num_blocks,
                                        int64_t max_seq_len, float sm_scale,
                                        void* workspace, size_t workspace_bytes,
                                        int dtype, void* stream);

/*
 * One decode step of an MLA attention layer in one call: store the step's latent rows, then attend.  Replaces the
 * pair that the reference's MLA layer issues per layer and step, the latent store (store_latent_cache: the rows of
 * compressed KV and rope key copied into the cache by slot, xllm/core/layers/dcu/deepseek_v2_attention.cpp:221-229)
 * followed by dense_decode (decode_flash_mla, :242-263), with new_latent [batch] rows of 576 values of `dtype` (row stride in elements) and
 * slot_mapping [batch] in front of the arguments of xllm_mi355_paged_decode_mla_planned.  plan may be NULL.
 * Sequence b's slot must be the place of its token seq_lens[b] - 1 in its block table; negative slots and slots
 * beyond the cache are skipped.  The cache and `out` afterwards hold the same bytes as after
 * xllm_mi355_reshape_and_cache followed by the decode call.  Where the kernel for more than 64 heads serves the call
 * (block size a power of two >= 16; new_latent 16-byte aligned with a stride that is a multiple of 8 elements) the
 * rows are stored inside the decode launch, by the workgroup that attends to the context's last tokens; otherwise
 * the library issues the two launches itself.  A sequence with seq_lens[b] == 0 stores nothing in the one-launch form.
 */
int xllm_mi355_write_and_decode_mla(const void* new_latent, const int32_t* slot_mapping,
                                    int64_t latent_row_stride,
                                    const void* plan, size_t plan_bytes,
                                    const void* q_nope, const void* q_pe, void* k_cache,
                                    void* out, float* lse,
                                    const int32_t* block_table, int64_t table_stride,
                                    const int32_t* seq_lens,
                                    int64_t batch, int64_t n_heads, int64_t d_latent, int64_t d_rope,
                                    int64_t block_size, int64_t num_blocks, int64_t max_seq_len,
                                    float sm_scale, void* workspace, size_t workspace_bytes,
                                    int dtype, void* stream);

/*
 * Log-sum-exp merge of S partial attention results.
 * Replaces xllm::layer::merge_dcp_attention_shards
 * (xllm/core/layers/mlu/dcp_attention_merge.cpp:26-65):
 *     w_s = exp(lse_s - max_s lse_s);  out = sum_s w_s o_s / sum_s w_s;
 *     lse = max + log(sum_s w_s);  shards with lse = -inf are ignored;
 *     all shards empty -> out = 0, lse = -inf.
 * partial_out: [S, B, H, Dv] of `dtype`; partial_lse: [S, B, H] fp32 natural log;
 * out: [B, H, Dv] of `dtype`; lse: [B, H] fp32 or null.
 */
int xllm_mi355_lse_merge(const void* partial_out, const float* partial_lse,
                         void* out, float* lse,
                         int64_t n_shards, int64_t batch, int64_t n_heads, int64_t v_head_dim,
                         int dtype, void* stream);

/*
 * Two-way combine of attention results whose LSEs are in base 2 (the convention of FlashInfer).  Replaces
 * xllm::kernel::cuda::lse_combine (xllm/core/kernels/cuda/xattention/lse_combine.cu:41-85,99-166; caller
 * xllm/core/layers/cuda/xattention.cpp:315), in the reference's arithmetic order:
 *     m = max(a, b);  merged = m + log2(exp2(a - m) + exp2(b - m));
 *     out = exp2(a - merged) * shared_o + exp2(b - merged) * unshared_o
 * shared_o / unshared_o: [rows, head_dim] of in_dtype (rows = batch * heads); the LSEs: [rows] fp32;
 * out: [rows, head_dim] of out_dtype.  Like the reference it returns no merged LSE, and two empty inputs
 * (both LSEs -inf) give NaN.  A natural-log LSE of this library is this base-2 LSE times ln 2.
 */
int xllm_mi355_lse_combine(void* out, const void* shared_o, const float* shared_lse,
                           const void* unshared_o, const float* unshared_lse,
                           int64_t rows, int64_t head_dim, int in_dtype, int out_dtype, void* stream);

/*
 * CSR -> padded block table.  Replaces build_block_table_from_paged_kv
 * (xllm/core/kernels/dcu/build_block_table_from_paged_kv.hip:44-149):
 * block_table[b, j] = indices[indptr[b] + j] for j < pages(b), -1 elsewhere;
 * seq_lens[b] = (pages(b) - 1) * block_size + last_page_len[b] (0 if no pages).
 * seq_lens may be null.
 */
int xllm_mi355_build_block_table(const int32_t* paged_kv_indptr,
                                 const int32_t* paged_kv_indices,
                                 const int32_t* paged_kv_last_page_len,
                                 int32_t* block_table, int64_t table_stride,
                                 int32_t* seq_lens,
                                 int64_t batch, int64_t block_size, void* stream);

/*
 * Block-table hygiene for kernels that expect -1 in unused columns.  Replaces mask_block_table_padding
 * (xllm/core/layers/dcu/flash_attention.cpp:194-218; the reference pads its tables with the valid page id 0,
 * framework/batch/batch_input_builder.cpp:1233-1275):
 *     out[b, j] = block_table[b, j] for j < ceil(kv_seq_lens[b] / block_size), -1 elsewhere
 * for j < width.  Columns are masked by position only, never by page id.  out may be block_table itself.
 * The decode kernels of this library do not need it: they never read a column beyond a sequence's pages.
 */
int xllm_mi355_mask_block_table_padding(const int32_t* block_table, int64_t table_stride,
                                        const int32_t* kv_seq_lens,
                                        int32_t* out, int64_t out_stride,
                                        int64_t batch, int64_t width, int64_t block_size, void* stream);

/*
 * Per-head RMS norm + rotary embedding of the q and k heads of a fused qkv buffer, in place; with a cache,
 * also the cache write of the new k and v rows in the same launch.  Replaces
 * xllm::kernel::cuda::fused_qk_norm_rope (xllm/core/kernels/cuda/fused_qknorm_rope.cu:79-300, 388-470;
 * caller xllm/core/layers/common/qwen2_attention.cpp:144-186) and, with k_cache / v_cache / slot_mapping, the
 * reshape_paged_cache call that follows it (xllm/core/kernels/ops_api.h:31): the cache receives the bits
 * stored in place for k and the untouched v (quantised per KV head when cache_dtype is fp8), what
 * xllm_mi355_reshape_and_cache would write from the buffer afterwards.
 *   qkv            [T, token_stride] 16-bit: n_heads_q, then n_heads_k, then n_heads_v heads of head_dim
 *   q_weight, k_weight  [head_dim] of the qkv dtype, or both null (no norm)
 *   cos_sin_cache  [max_position, rotary_dim]: cos of the rotary_dim / 2 frequencies, then sin
 *   position_ids   [T] int64
 *   interleave     nonzero: pairs (2i, 2i + 1); zero: pairs (i, i + rotary_dim / 2)
 * head_dim 64, 128 or 256; rotary_dim a multiple of head_dim / 16.  k_cache null: no cache write.
 * qkv, the norm weights, cos_sin_cache and the caches 16-byte aligned.
 */
int xllm_mi355_rope_and_cache(void* qkv, const void* q_weight, const void* k_weight,
                              const void* cos_sin_cache, const int64_t* position_ids,
                              void* k_cache, void* v_cache, const int32_t* slot_mapping,
                              const float* k_scale, const float* v_scale,
                              int64_t n_tokens, int64_t token_stride,
                              int64_t n_heads_q, int64_t n_heads_k, int64_t n_heads_v,
                              int64_t head_dim, int64_t rotary_dim, float eps, int interleave,
                              int64_t block_size, int64_t num_blocks,
                              int dtype, int cos_sin_dtype, int cache_dtype, void* stream);

/*
 * Decode metadata into the persistent buffers of a captured step, with the padding a replay at a larger
 * batch expects.  Replaces xllm::kernel::cuda::update_llm_decode_metadata and its parameter struct,
 * field for field (xllm/core/kernels/cuda/llm_decode_metadata_update.h:33-56, .cu:27-71; caller
 * xllm/core/runtime/cuda_graph_executor_impl.cpp:243-284).  All arrays int32; src_kv_seq_lens and
 * src_paged_kv_indptr are cumulative, [actual_batch_size + 1].
 *   tokens, positions, new_cache_slots : [0, actual_num_tokens) copied; up to padded_num_tokens 0, 0, -1
 *   kv_seq_lens, paged_kv_indptr       : [0, actual_batch_size] copied; up to padded_num_tokens the last value
 *   kv_seq_lens_delta                  : src_kv_seq_lens[i + 1] - src_kv_seq_lens[i]; up to padded_num_tokens 0
 *   paged_kv_last_page_len             : copied; up to padded_num_tokens 1
 *   paged_kv_indices                   : [0, actual_indices_size) copied
 */
int xllm_mi355_decode_metadata_update(const int32_t* src_tokens, const int32_t* src_positions,
                                      const int32_t* src_new_cache_slots, const int32_t* src_kv_seq_lens,
                                      const int32_t* src_paged_kv_indptr, const int32_t* src_paged_kv_indices,
                                      const int32_t* src_paged_kv_last_page_len,
                                      int32_t* dst_tokens, int32_t* dst_positions, int32_t* dst_new_cache_slots,
                                      int32_t* dst_kv_seq_lens, int32_t* dst_kv_seq_lens_delta,
                                      int32_t* dst_paged_kv_indptr, int32_t* dst_paged_kv_indices,
                                      int32_t* dst_paged_kv_last_page_len,
                                      int64_t actual_num_tokens, int64_t padded_num_tokens,
                                      int64_t actual_batch_size, int64_t actual_indices_size, void* stream);

/*
 * Opt-in timing of the dominant decode kernel.  No counterpart in the reference, which
 * relies on external profilers (xllm/core/platform/cuda_profiler.cpp,
 * xllm/core/platform/torch_profiler.cpp).  After xllm_mi355_profile_enable(n) the next n
 * timed kernels carry a HIP event pair that the runtime fills with the kernel's own start and
 * end; a decode entry point times two kernels per launch pair, in this order: the decode kernel,
 * then the merge kernel (a batch of more than 2048 sequences is several launch pairs).
 * xllm_mi355_profile_collect waits for them, writes the elapsed milliseconds of each (host
 * pointer) and returns how many, or a value < -1000 on a HIP error.  Process-wide, single
 * caller thread, not usable under graph capture.
 */
int xllm_mi355_profile_enable(int capacity);
int xllm_mi355_profile_collect(float* ms_out, int max_n);

/*
 * Test hooks.  No counterpart in the reference.  XLLM_MI355_DEBUG_WAIT_SPINS: the bound of the polls described
 * at xllm_mi355_decode_status (negative = default, 2^22; 0 makes the first wait of a launch give up, which is
 * how the status path is tested: every wavefront still exits normally).  XLLM_MI355_DEBUG_MLA_KERNEL: the MLA
 * kernel choice, as the first letter of the environment variable XLLM_MI355_MLA_KERNEL, which the library reads
 * once per process (0 default, 'p' pairs, 'h' heads, 'n' narrow, 'w' the four-wavefront kernel).  XLLM_MI355_DEBUG_GQA_FOLD: 1 makes
 * the matrix-core GQA kernel merge the partial results itself instead of leaving them to a second launch (same
 * as XLLM_MI355_GQA_FOLD=1 in the environment; off by default because it measures slower).
 * XLLM_MI355_DEBUG_GQA_STREAM_STORES: 1 / 0 make the matrix-core GQA kernel write its output and partial rows with /
 * without non-temporal stores whatever the size of the launch, negative gives the choice back to the library (same
 * as XLLM_MI355_GQA_STREAM_STORES in the environment; the bytes written are the same either way).
 * XLLM_MI355_DEBUG_MLA_FOLD: 1 makes the MLA decode kernel for more than 64 heads merge the contexts that span several
 * workgroups itself, 0 leaves them to a second launch (the default: it measures the same, and the one launch needs every
 * workgroup resident at once), negative gives the choice back to the environment (XLLM_MI355_MLA_FOLD = 1 turns it on);
 * the outputs are the same bits either way.
 */
enum {
  XLLM_MI355_DEBUG_WAIT_SPINS = 0,
  XLLM_MI355_DEBUG_MLA_KERNEL = 1,
  XLLM_MI355_DEBUG_GQA_FOLD = 2,
  XLLM_MI355_DEBUG_GQA_STREAM_STORES = 3,
  XLLM_MI355_DEBUG_MLA_FOLD = 4
};
int xllm_mi355_debug_set(int what, int value);

/*
 * Plain streaming kernels of known size, the yardstick for the decode kernels.  No
 * counterpart in the reference (its own micro-benchmarks time block copies with device
 * events, tests/core/kernels/dcu/block_copy_test.cpp:195-215).  stream_read reads `bytes`
 * once (sink: 4 writable bytes or null); stream_copy reads and writes them once.  Pointers
 * 16-byte aligned, bytes a multiple of 16.  Both take part in the timing hook above.
 */
int xllm_mi355_stream_read(const void* src, size_t bytes, void* sink, void* stream);
int xllm_mi355_stream_copy(void* dst, const void* src, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* XLLM_MI355_H_ */
