/*
 * fandhe_rocm.h - C ABI of the MI355X (gfx950) quantized decode backend.
 *
 * Plain C, plain pointers and sizes.  Every entry point returns an fa_status;
 * none of them aborts or throws.  The entry points are what a `BackendOps` /
 * `MemoryOps` implementation for `Device::Rocm(0)` binds; each declaration
 * cites the reference interface it stands behind (paths are relative to the
 * reference repository root).
 *
 * Execution model (the contract of the reference's asynchronous backend,
 * docs/backend-cuda-async-execution-design.md:71-118): one in-order HIP stream
 * per context; submit calls do not block the host; the host-blocking points
 * are fa_download, fa_synchronize_device and calls documented as returning
 * host data.  Argument violations are reported before anything is written.
 * A HIP failure after validation poisons the context: every later call
 * returns FA_ERR_CONTEXT_POISONED until the context is destroyed.
 */
#ifndef FANDHE_ROCM_H
#define FANDHE_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ status */
/* Mirrors BackendError (crates/tensor-core/src/device.rs:225-371). */
typedef int32_t fa_status;
enum {
    FA_OK = 0,
    FA_ERR_INVALID_ARGUMENT = 1,       /* BackendError::InvalidArgument */
    FA_ERR_SHAPE_MISMATCH = 2,         /* BackendError::ShapeMismatch */
    FA_ERR_DEVICE_MISMATCH = 3,        /* BackendError::DeviceMismatch (foreign handle) */
    FA_ERR_ALLOCATION_FAILED = 4,      /* BackendError::DeviceAllocationFailed */
    FA_ERR_KERNEL_LAUNCH_FAILED = 5,   /* BackendError::KernelLaunchFailed */
    FA_ERR_DEVICE_UNAVAILABLE = 6,     /* BackendError::DeviceUnavailable */
    FA_ERR_TRANSFER_FAILED = 7,        /* BackendError::TransferFailed */
    FA_ERR_UNSUPPORTED = 8,            /* BackendError::Unsupported */
    FA_ERR_CONTEXT_POISONED = 9,       /* BackendError::DeviceContextPoisoned */
    FA_ERR_CAPTURE_IN_PROGRESS = 10,   /* BackendError::DeviceContextCaptureInProgress */
    FA_ERR_STORE_POISONED = 11         /* BackendError::StorePoisoned (a paged cache after a failed device write) */
};
/* Message of the last failure on the calling thread ("" if none). */
const char *fa_last_error_message(void);
const char *fa_status_name(fa_status s);
/* ABI version of this header; bumped on any incompatible change. */
uint32_t fa_abi_version(void);

/* ----------------------------------------------------------------- context */
/* DeviceProvider::{is_available, enumerate, select} for backend "rocm"
 * (crates/tensor-core/src/device.rs:149-168,
 *  crates/backend-rocm/src/device.rs:30-114).  Only gfx950 devices count. */
typedef struct fa_context fa_context;
fa_status fa_device_count(int32_t *count);
fa_status fa_context_create(int32_t ordinal, fa_context **out);
fa_status fa_context_destroy(fa_context *ctx);
typedef struct {
    int32_t ordinal;
    int32_t compute_units;
    int32_t clock_khz;
    int32_t wavefront_size;
    uint64_t total_memory_bytes;
    char arch[32];
    char name[128];
} fa_device_info;
fa_status fa_context_info(const fa_context *ctx, fa_device_info *out);

/* ------------------------------------------------------------------ memory */
/* MemoryOps + DeviceBuffer (crates/tensor-core/src/buffer.rs:91-373,389-521).
 * The reference's buffers are f32 only; the element type is explicit here so
 * that bf16 / int8 / fp8 storage sits behind the same opaque handle. */
typedef enum {
    FA_F32 = 0, FA_BF16 = 1, FA_I8 = 2, FA_E4M3 = 3, FA_I32 = 4, FA_U32 = 5
} fa_dtype;
typedef struct fa_buffer fa_buffer;

/* MemoryOps::alloc_zeroed (buffer.rs:395).  numel == 0 touches no device. */
fa_status fa_alloc_zeroed(fa_context *ctx, fa_dtype dtype, uint64_t numel, fa_buffer **out);
/* Same pool, contents unspecified (operator outputs are fully overwritten,
 * crates/tensor-core/src/backend_ops.rs:4343-4347). */
fa_status fa_alloc_uninit(fa_context *ctx, fa_dtype dtype, uint64_t numel, fa_buffer **out);
/* MemoryOps::upload (buffer.rs:404): host data is consumed on return. */
fa_status fa_upload(fa_context *ctx, fa_dtype dtype, const void *host, uint64_t numel, fa_buffer **out);
/* MemoryOps::upload_into (buffer.rs:446-459): dst_offset in elements. */
fa_status fa_upload_into(fa_context *ctx, const void *host, uint64_t numel, fa_buffer *dst,
                         uint64_t dst_offset);
/* MemoryOps::download (buffer.rs:417): host data is final on return (the
 * synchronization point).  src_offset / numel in elements. */
fa_status fa_download(fa_context *ctx, const fa_buffer *src, uint64_t src_offset, void *host,
                      uint64_t numel);
/* MemoryOps::download_owned (buffer.rs:414-430): the caller gives the buffer up; host data is final on return
 * and the handle is freed whether or not the copy succeeded (it is consumed either way, as in the trait). */
fa_status fa_download_owned(fa_context *ctx, fa_buffer *src, void *host, uint64_t numel);
/* MemoryOps::with_host_view (buffer.rs:486-521): calls f(user, data, numel) once with a host copy of the whole
 * buffer that is valid only during the call (numel == 0: an empty view, no device access). */
typedef void (*fa_host_view_fn)(void *user, const void *data, uint64_t numel);
fa_status fa_with_host_view(fa_context *ctx, const fa_buffer *src, fa_host_view_fn f, void *user);
/* Drop of the handle (buffer.rs:40-48): returns the block to the pool. */
fa_status fa_buffer_free(fa_context *ctx, fa_buffer *buf);
uint64_t fa_buffer_numel(const fa_buffer *buf);
fa_dtype fa_buffer_dtype(const fa_buffer *buf);
void *fa_buffer_device_ptr(const fa_buffer *buf);

/* BackendOps::synchronize_device (backend_ops.rs:4897). */
fa_status fa_synchronize_device(fa_context *ctx);
/* Whether an earlier device failure poisoned the context (1) or not (0); never fails on a live context and
 * does not touch the device.  With all work ordered on one stream this is what a caller re-checks after a
 * download where a batching backend would re-check a DispatchFailureCell (dispatch_failure.rs:1-40;
 * backend_ops.rs:4724-4726: a stream-ordered backend poisons the ordinal and keeps the *_tracked defaults). */
fa_status fa_context_poisoned(const fa_context *ctx, int32_t *poisoned);
/* The HIP stream (hipStream_t) every call of this context is ordered on. */
void *fa_context_stream(fa_context *ctx);

/* PoolStats (crates/tensor-core/src/pool_core.rs:122-139). */
typedef struct {
    uint64_t alloc_count, reuse_count, cached_bytes, pending_return_bytes,
        capacity_waste_bytes, released_bytes;
} fa_pool_stats;
/* BackendOps::device_memory_pool_stats (backend_ops.rs:5050). */
fa_status fa_device_memory_pool_stats(fa_context *ctx, fa_pool_stats *out);
/* BackendOps::release_cached_device_memory (backend_ops.rs:5038). */
fa_status fa_release_cached_device_memory(fa_context *ctx);
/* size_class_for with the default configuration (pool_core.rs:157-209). */
fa_status fa_size_class_for(uint64_t bytes, uint64_t *class_bytes);

/* ------------------------------------------------------------ f32 linear */
typedef enum { FA_ACT_NONE = 0, FA_ACT_RELU = 1 } fa_activation;
/* BackendOps::gemm_device (backend_ops.rs:1998): out[m,n] = a[m,k] @ b[k,n],
 * f32, one accumulator per output, k ascending, fused multiply-add. */
fa_status fa_gemm_device(fa_context *ctx, const fa_buffer *a, const fa_buffer *b, uint64_t m,
                         uint64_t n, uint64_t k, fa_buffer *out);
/* BackendOps::linear_forward_device (backend_ops.rs:4296-4308):
 * out = act(a @ w + bias); w / bias are views (buffer + element offset,
 * DeviceBufferView, buffer.rs:277-373) with w stored [k, n]. bias may be NULL. */
fa_status fa_linear_forward_device(fa_context *ctx, const fa_buffer *a, uint64_t m, uint64_t k,
                                   const fa_buffer *w, uint64_t w_offset, uint64_t n,
                                   const fa_buffer *bias, uint64_t bias_offset,
                                   fa_activation act, fa_buffer *out);

/* -------------------------------------------------------- quantized linear */
/* Not in the reference (design record only,
 * docs/backend-int8-quantization-decision.md:13,84); the contract is:
 * symmetric int8, scale = absmax / 127, q = clamp(rne(x / scale), -127, 127),
 * int32 accumulation, out = f32(acc) * (sx[m] * sw[n]) (+ bias[n]).
 * A quantized weight is an opaque object: int8 (or e4m3) codes in an
 * MFMA-friendly tile order plus f32 scales. */
typedef struct fa_qweight fa_qweight;
typedef enum { FA_QW_INT8_CHANNEL = 0, FA_QW_E4M3_TENSOR = 1, FA_QW_E4M3_CHANNEL = 2 } fa_qweight_kind;
/* Quantize an f32 weight view w[k, n] (the layout of linear_forward_device)
 * on the device.  INT8_CHANNEL: one scale per output column (absmax / 127).
 * E4M3_TENSOR: one scale (absmax / 448).  E4M3_CHANNEL: e4m3 codes with one
 * scale per output column (column absmax / 448). */
fa_status fa_qweight_from_f32(fa_context *ctx, const fa_buffer *w, uint64_t w_offset, uint64_t k,
                              uint64_t n, fa_qweight_kind kind, fa_qweight **out);
/* Import host codes q[k, n] (int8 or e4m3 bytes) with their scales
 * (n scales for INT8_CHANNEL and E4M3_CHANNEL, 1 for E4M3_TENSOR). */
fa_status fa_qweight_from_codes(fa_context *ctx, const void *codes, const float *scales,
                                uint64_t k, uint64_t n, fa_qweight_kind kind, fa_qweight **out);
/* Read back codes as [k, n] and scales (test / export path; synchronizes). */
fa_status fa_qweight_export(fa_context *ctx, const fa_qweight *qw, void *codes, float *scales);
fa_status fa_qweight_free(fa_context *ctx, fa_qweight *qw);
uint64_t fa_qweight_k(const fa_qweight *qw);
uint64_t fa_qweight_n(const fa_qweight *qw);

/* Dynamic per-token quantization of x[m, k] (f32 or bf16 buffer): writes
 * row-major int8 codes xq[m, k] and scales sx[m]. */
fa_status fa_quantize_rows_i8(fa_context *ctx, const fa_buffer *x, uint64_t m, uint64_t k,
                              fa_buffer *xq, fa_buffer *sx);
/* W8A8 linear on a weight of kind INT8_CHANNEL: quantizes x per token,
 * multiplies on the int8 matrix cores, dequantizes in the epilogue.
 * out: f32 or bf16 [m, n].  acc_out (nullable): i32 [m, n] raw accumulators.
 * bias (nullable): f32 view of n elements. */
fa_status fa_linear_w8a8(fa_context *ctx, const fa_buffer *x, uint64_t m, const fa_qweight *qw,
                         const fa_buffer *bias, uint64_t bias_offset, fa_buffer *acc_out,
                         fa_buffer *out);
/* Decode-shape int8-weight linear with bf16 activations a[m, k]:
 * out[m, n] = (sum_k a * w_int8) * sw[n], f32 accumulation; out f32 or bf16. */
fa_status fa_linear_w8a16(fa_context *ctx, const fa_buffer *a, uint64_t m, const fa_qweight *qw,
                          fa_buffer *out);
/* Per-tensor e4m3 quantization of x (f32): codes xq (E4M3, same shape) and a
 * one-element f32 scale buffer (absmax / 448). */
fa_status fa_quantize_tensor_e4m3(fa_context *ctx, const fa_buffer *x, uint64_t numel,
                                  fa_buffer *xq, fa_buffer *scale);
/* fp8 GEMM: out[m, n] = (aq[m, k] @ W) * (a_scale * w_scale), f32
 * accumulation; qw of kind E4M3_TENSOR; out f32 or bf16. */
fa_status fa_gemm_e4m3(fa_context *ctx, const fa_buffer *aq, const fa_buffer *a_scale, uint64_t m,
                       const fa_qweight *qw, fa_buffer *out);
/* fp8 linear with per-token activation and per-channel weight scales (the
 * e4m3 counterpart of fa_linear_w8a8; design record
 * docs/spec-proposal-fp8-int8-quant-gemm.md:95-97): dynamic per-token
 * quantization of x[m, k] (f32 or bf16) to e4m3, scale = row absmax / 448;
 * writes row-major codes xq[m, k] and scales sx[m]. */
fa_status fa_quantize_rows_e4m3(fa_context *ctx, const fa_buffer *x, uint64_t m, uint64_t k,
                                fa_buffer *xq, fa_buffer *sx);
/* out[m, n] = (xq @ W) * (sx[m] * sw[n]) (+ bias[n]) with f32 accumulation on
 * the fp8 matrix cores and the dequantization fused into the epilogue; qw of
 * kind E4M3_CHANNEL, x f32 or bf16 (quantized per token inside the call), out
 * f32 or bf16.  Rows up to 64 take a weight-streaming kernel (decode shape),
 * more rows the tiled GEMM kernels (k must then be a multiple of 128). */
fa_status fa_linear_e4m3(fa_context *ctx, const fa_buffer *x, uint64_t m, const fa_qweight *qw,
                         const fa_buffer *bias, uint64_t bias_offset, fa_buffer *out);
/* The same on activations quantized beforehand (fa_quantize_rows_e4m3). */
fa_status fa_gemm_e4m3_rows(fa_context *ctx, const fa_buffer *aq, const fa_buffer *sx, uint64_t m,
                            const fa_qweight *qw, const fa_buffer *bias, uint64_t bias_offset,
                            fa_buffer *out);
/* int8 GEMM on pre-quantized row-major activations aq[m, k] with scales
 * sx[m] (prefill shape); same epilogue as fa_linear_w8a8. */
fa_status fa_gemm_w8a8(fa_context *ctx, const fa_buffer *aq, const fa_buffer *sx, uint64_t m,
                       const fa_qweight *qw, fa_buffer *acc_out, fa_buffer *out);

/* ------------------------------------------------------------------ norms */
/* BackendOps::rmsnorm (backend_ops.rs:5113-5122; CPU contract
 * crates/backend-cpu/src/rmsnorm.rs:124-228): f64 sum of squares,
 * rstd = (f32)(1 / sqrt(sum * (f64)(1/hidden as f32) + eps)),
 * out = (x * rstd) * w.  w may be NULL.  x / out f32 [rows, hidden]. */
fa_status fa_rmsnorm(fa_context *ctx, const fa_buffer *x, const fa_buffer *w, float eps,
                     uint64_t rows, uint64_t hidden, fa_buffer *out);
/* Not in the reference: rotary embedding, rotate-half pairing (i, i + Dh/2),
 * inv_freq = theta^(-2i/Dh); x / out f32 [rows, heads, head_dim];
 * positions: i32 buffer [rows]. */
fa_status fa_rope(fa_context *ctx, const fa_buffer *x, const fa_buffer *positions, uint64_t rows,
                  uint64_t heads, uint64_t head_dim, double theta, fa_buffer *out);

/* ------------------------------------------------------------ elementwise */
/* BackendOps::scalar_unary(Silu) then mul (backend_ops.rs:2304,2276;
 * formula crates/tensor-core/src/scalar_op.rs:355,666-673). */
fa_status fa_silu_mul(fa_context *ctx, const fa_buffer *gate, const fa_buffer *up, uint64_t numel,
                      fa_buffer *out);
/* BackendOps::add (backend_ops.rs:2277). */
fa_status fa_add(fa_context *ctx, const fa_buffer *a, const fa_buffer *b, uint64_t numel,
                 fa_buffer *out);
/* BackendOps::argmax over the last axis (backend_ops.rs:2390): first index
 * on ties, NaN ignored, all-NaN row -> 0.  out: i32 [rows]. */
fa_status fa_argmax_rows(fa_context *ctx, const fa_buffer *x, uint64_t rows, uint64_t cols,
                         fa_buffer *out);
/* BackendOps::gather of rows (backend_ops.rs:3375): out[r, :] = table[idx[r], :]. */
fa_status fa_gather_rows(fa_context *ctx, const fa_buffer *table, uint64_t table_rows,
                         uint64_t cols, const fa_buffer *idx, uint64_t rows, fa_buffer *out);
/* Next-token sampling from logits [rows, vocab] (f32), on the device, with the
 * arithmetic of the reference's host sampler (crates/autodiff/src/generate/mod.rs:
 * 333-452, sample_step / sampling_weights_f32; crates/tensor-core/src/rng.rs:
 * 509-539 multinomial): strategy 0 greedy (first maximum), 1 temperature, 2
 * top-k (k largest by value descending, index ascending; temperature applies
 * too, the reference fixes it at 1).  rng: a U32 buffer of at least two
 * elements holding the 64-bit state of the xorshift64* generator
 * (fa_rng_seed); rows draw in row order, one draw each; greedy draws nothing.
 * tokens: I32 [rows].  A row with a non-finite logit gets token -1 (the
 * reference fails the step).  Asynchronous. */
typedef enum fa_sampling { FA_SAMPLE_GREEDY = 0, FA_SAMPLE_TEMPERATURE = 1, FA_SAMPLE_TOP_K = 2 } fa_sampling;
fa_status fa_sample_rows(fa_context *ctx, const fa_buffer *logits, uint64_t rows, uint64_t vocab,
                         fa_sampling strategy, float temperature, uint64_t top_k, fa_buffer *rng,
                         fa_buffer *tokens);
/* Generator::new(seed) (rng.rs:65-69, 684-689): seed 0 selects 0x9E3779B97F4A7C15. */
fa_status fa_rng_seed(fa_context *ctx, fa_buffer *rng, uint64_t seed);
/* The same rule as a plain host function: the generator state a seed starts. */
fa_status fa_rng_state_from_seed(uint64_t seed, uint64_t *state);
/* sampling_weights_f32 (crates/autodiff/src/generate/mod.rs:432-452) of `rows` rows of logits that start
 * `logits_offset` elements into `logits`: the f32 weights the sampler draws from, stored from `weights_offset` on
 * (greedy: one-hot at the first maximum).  status (I32 [rows]): 0, or 1 where a logit is not finite (that row of
 * weights is NaN; the reference rejects the step there). */
fa_status fa_sampling_weights(fa_context *ctx, const fa_buffer *logits, uint64_t logits_offset, uint64_t rows, uint64_t vocab,
                              fa_sampling strategy, float temperature, uint64_t top_k, fa_buffer *weights,
                              uint64_t weights_offset, fa_buffer *status);
/* Acceptance step of sampled speculative decoding for one sequence, on the device (verify_sampling,
 * crates/autodiff/src/generate/speculative.rs:246-279, with normalize_f64 / acceptance_prob_f32 /
 * residual_weights_f32 / accept_draw / sample_from, :111-189): p_weights holds the target's k + 1 weight rows of
 * the verification pass, q_weights the k rows every draft was drawn from, drafts the k draft tokens (host array,
 * k <= 32).  Draft i is accepted when the next uniform of `rng` is below (f32) min(1, p(d) / q(d)); at the first
 * refusal one token is drawn from max(0, p - q) and the call stops; when every draft is accepted one token is
 * drawn from row k of p_weights.  k == 0 is one multinomial draw from row 0 of p_weights (sample_from).
 * result (I32 [4]): accepted drafts, the token that follows them, status (0 ok; 2 q(d) <= 0 or a probability not
 * finite; 3 a weight row negative, not finite or summing to zero; 4 the residual sums to zero), unused.  The
 * generator advances by the draws the call consumed.  Nothing is read back: download `result`. */
fa_status fa_speculative_accept(fa_context *ctx, const fa_buffer *p_weights, uint64_t p_offset, const fa_buffer *q_weights,
                                uint64_t q_offset, const int32_t *drafts, uint64_t k, uint64_t vocab, fa_buffer *rng,
                                fa_buffer *result);

/* One row of a per-row sampling table: every row is a request with a
 * GenerateConfig and a Generator of its own, as in the reference's continuous
 * batching scheduler (crates/autodiff/src/generate/scheduler.rs:160-211: each
 * active request owns its config and its rng, one draw per generated token).
 * rng_state is advanced in place by one draw whenever a temperature / top-k row
 * is sampled; a greedy row draws nothing. */
typedef struct fa_row_sampling {
    uint64_t rng_state;   /* xorshift64* state, never zero (fa_rng_state_from_seed) */
    float temperature;    /* finite, > 0; 1 for greedy */
    uint32_t top_k;       /* 1..=vocab for FA_SAMPLE_TOP_K, ignored otherwise */
    int32_t strategy;     /* fa_sampling */
    uint32_t reserved;
} fa_row_sampling;
/* fa_sample_rows with one fa_row_sampling per row: table is a U32 buffer of
 * 6 * rows elements holding the rows' fa_row_sampling records. */
fa_status fa_sample_rows_per_row(fa_context *ctx, const fa_buffer *logits, uint64_t rows, uint64_t vocab,
                                 fa_buffer *table, fa_buffer *tokens);
/* dtype conversion f32 <-> bf16 (round to nearest even, once). */
fa_status fa_convert(fa_context *ctx, const fa_buffer *src, uint64_t numel, fa_buffer *dst);

/* --------------------------------------------------------------- paged KV */
/* PagedKvLayout (crates/tensor-core/src/paged_kv.rs:47-131). */
typedef struct {
    uint64_t num_blocks;
    uint64_t block_size;      /* power of two, 1..256 */
    uint64_t embed_dim;       /* width of one K / V row */
} fa_paged_layout;
/* PagedAttentionArgs (paged_kv.rs:137-214) + num_kv_heads for grouped-query
 * attention (0 or == num_heads: the reference's MHA; then embed_dim is the
 * query width too). */
typedef struct {
    fa_paged_layout layout;
    uint64_t batch;
    uint64_t l_new;
    uint64_t num_heads;
    uint64_t max_blocks_per_seq;
    float scale;
    uint64_t num_kv_heads;
} fa_paged_args;
/* PagedAttentionPlan (paged_kv.rs:201-213). */
typedef struct {
    uint64_t out_numel, s_max, query_rows, workspace_elems;
} fa_paged_plan;
/* validate_paged_kv_append / validate_paged_attention (paged_kv.rs:222-373);
 * pure host functions, callable without a device. */
fa_status fa_validate_paged_kv_append(uint64_t k_new_numel, uint64_t v_new_numel,
                                      uint64_t k_pool_numel, uint64_t v_pool_numel,
                                      const uint32_t *slot_mapping, uint64_t rows,
                                      const fa_paged_layout *layout);
fa_status fa_validate_paged_attention(uint64_t q_numel, uint64_t k_pool_numel,
                                      uint64_t v_pool_numel, const uint32_t *block_tables,
                                      uint64_t n_tables, const uint32_t *seq_lens, uint64_t n_seq,
                                      const fa_paged_args *args, fa_paged_plan *plan);
/* BackendOps::paged_kv_append (backend_ops.rs:4694-4709): copies row r of
 * k_new / v_new [rows, E] to pool row slot_mapping[r].  Buffers f32 or bf16
 * (all four the same type).  slot_mapping is a host array. */
fa_status fa_paged_kv_append(fa_context *ctx, const fa_buffer *k_new, const fa_buffer *v_new,
                             fa_buffer *k_pool, fa_buffer *v_pool, const uint32_t *slot_mapping,
                             uint64_t rows, const fa_paged_layout *layout);
/* BackendOps::paged_attention_forward (backend_ops.rs:4742-4757).  q / out
 * [B, L_new, H * Dh]; pools [num_blocks, block_size, H_kv * Dh]; f32 or bf16
 * (q, pools, out the same type).  block_tables [B, max_blocks_per_seq] and
 * seq_lens [B] are host arrays; unused table entries hold UINT32_MAX. */
fa_status fa_paged_attention_forward(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                     const fa_buffer *v_pool, const uint32_t *block_tables,
                                     uint64_t n_tables, const uint32_t *seq_lens, uint64_t n_seq,
                                     const fa_paged_args *args, fa_buffer *out);
/* Device-resident tables (U32 buffers) for callers that replay a captured
 * graph: nothing is read on the host, so table contents cannot be validated
 * before the launch; the kernels bounds-check every block id and slot and
 * write NaN / skip the row on a violation.  seq_lens may not exceed
 * max_blocks_per_seq * block_size. */
fa_status fa_paged_kv_append_device(fa_context *ctx, const fa_buffer *k_new, const fa_buffer *v_new,
                                    fa_buffer *k_pool, fa_buffer *v_pool,
                                    const fa_buffer *slot_mapping, uint64_t rows,
                                    const fa_paged_layout *layout);
fa_status fa_paged_attention_forward_device(fa_context *ctx, const fa_buffer *q,
                                            const fa_buffer *k_pool, const fa_buffer *v_pool,
                                            const fa_buffer *block_tables, const fa_buffer *seq_lens,
                                            const fa_paged_args *args, fa_buffer *out);

/* No counterpart in the reference.  fa_paged_attention_forward_device for callers that cannot allocate:
 * code under a HIP graph capture of its own, serving loops and harnesses that forbid hipMalloc.  The partial
 * results of the streamed decode kernel live in a static device array of the library (16 MiB per GPU, held
 * until the process ends) instead of the context's pooled workspace, and the call allocates and frees
 * nothing.  Decode shape of the streamed kernel only (bf16, head_dim 128, block_size 16, l_new 1, at most 16
 * query heads per kv head): FA_ERR_UNSUPPORTED otherwise; a shape whose partial results exceed the array
 * ((ranges + batch) * kv heads * 520 floats * padded group / 4; a batch of 64 with 8 kv heads needs 3.2 MB)
 * is FA_ERR_INVALID_ARGUMENT.  Same results, bit for bit, as fa_paged_attention_forward_device.  All calls
 * on one GPU share the array: calls that overlap on one GPU (two contexts, two streams) race. */
fa_status fa_paged_attention_decode_static(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                           const fa_buffer *v_pool, const fa_buffer *block_tables,
                                           const fa_buffer *seq_lens, const fa_paged_args *args, fa_buffer *out);
/* Size in bytes of that array. */
uint64_t fa_paged_attention_decode_static_max_bytes(void);

/* ---------------------------------------------------- paged KV cache (layer) */
/* The caller side of the paged operators: page table with free-block
 * bookkeeping and the one-layer device-resident cache built on it.
 * BlockTable (crates/autodiff/src/nn/paged_kv.rs:147-363): free blocks are the
 * stack of returned ids (last in, first out) and then the never-used ids in
 * ascending order; all rows of the batch have the same length; every call
 * either succeeds or leaves the table unchanged.  Pure host code: usable
 * without a device. */
typedef struct fa_block_table fa_block_table;
typedef struct {
    uint64_t seq_len;       /* BlockTable::seq_len (paged_kv.rs:192-195) */
    uint64_t has_batch;     /* batch fixed by the first append */
    uint64_t batch;
    uint64_t used_blocks;   /* sum of the rows' block counts */
    uint64_t free_blocks;   /* BlockTable::free_blocks (paged_kv.rs:167-169) */
    uint64_t next_unused, returned;
} fa_block_table_state;
fa_status fa_block_table_create(fa_block_table **out);
fa_status fa_block_table_destroy(fa_block_table *bt);
fa_status fa_block_table_clone(const fa_block_table *bt, fa_block_table **out);
/* BlockTable::alloc (paged_kv.rs:172-183); *got = 0 when no block is free. */
fa_status fa_block_table_alloc(fa_block_table *bt, uint64_t max_blocks, uint32_t *id, int32_t *got);
/* Pushes an id on the returned stack (what rewind_to does for every block it releases). */
fa_status fa_block_table_return(fa_block_table *bt, uint32_t id);
fa_status fa_block_table_reset(fa_block_table *bt);
fa_status fa_block_table_state_get(const fa_block_table *bt, uint64_t max_blocks, fa_block_table_state *out);
/* BlockTable::extend_for_append (paged_kv.rs:205-291): slots of the b * l_new
 * new tokens, rows first, slot = block_id * block_size + pos % block_size. */
fa_status fa_block_table_extend_for_append(fa_block_table *bt, uint64_t max_blocks, uint64_t block_size,
                                           uint64_t b, uint64_t l_new, uint32_t *slots,
                                           uint64_t slots_capacity, uint64_t *n_slots);
/* BlockTable::flatten_tables (paged_kv.rs:295-319): [rows, max_blocks_per_seq], UINT32_MAX in unused entries. */
fa_status fa_block_table_flatten(const fa_block_table *bt, uint64_t max_blocks_per_seq, uint32_t *out,
                                 uint64_t out_capacity, uint64_t *n_out);
/* BlockTable::rewind_to (paged_kv.rs:323-363). */
fa_status fa_block_table_rewind_to(fa_block_table *bt, uint64_t new_len, uint64_t block_size);

/* PagedKvCache (crates/autodiff/src/nn/paged_kv_device.rs:67-372): K / V pools
 * [max_blocks, block_size, embed_dim] on the device (f32 as in the reference,
 * or bf16), append and attention queued on the context's stream, the only
 * synchronization point is the download of the attention output.  A device
 * failure after validation poisons the cache (append / attention then return
 * FA_ERR_STORE_POISONED; rewind_to and clear stay allowed). */
typedef struct fa_paged_cache fa_paged_cache;
/* PagedKvCacheConfig::new (paged_kv.rs:79-108). */
fa_status fa_paged_cache_check_config(uint64_t block_size, uint64_t max_blocks, uint64_t embed_dim,
                                      fa_dtype dtype);
/* PagedKvCache::new (paged_kv_device.rs:91-123). */
fa_status fa_paged_cache_create(fa_context *ctx, uint64_t block_size, uint64_t max_blocks,
                                uint64_t embed_dim, fa_dtype dtype, fa_paged_cache **out);
fa_status fa_paged_cache_destroy(fa_context *ctx, fa_paged_cache *cache);
/* seq_len / batch / num_used_blocks / num_free_blocks / is_poisoned (paged_kv_device.rs:136-160). */
fa_status fa_paged_cache_state_get(const fa_paged_cache *cache, fa_block_table_state *out, int32_t *poisoned);
fa_status fa_paged_cache_pools(fa_paged_cache *cache, fa_buffer **k_pool, fa_buffer **v_pool);
fa_status fa_paged_cache_block_tables(const fa_paged_cache *cache, uint64_t max_blocks_per_seq, uint32_t *out,
                                      uint64_t out_capacity, uint64_t *n_out);
/* PagedKvCache::append (paged_kv_device.rs:187-247): k_new / v_new [b, l_new, embed_dim] of the pools' type. */
fa_status fa_paged_cache_append(fa_context *ctx, fa_paged_cache *cache, const fa_buffer *k_new,
                                const fa_buffer *v_new, uint64_t b, uint64_t l_new);
/* PagedKvCache::attention (paged_kv_device.rs:254-340): q / out [b, l_new, num_heads * head_dim] with
 * head_dim = embed_dim / num_kv_heads (num_kv_heads 0 or == num_heads: the reference's MHA). */
fa_status fa_paged_cache_attention(fa_context *ctx, const fa_paged_cache *cache, const fa_buffer *q, uint64_t b,
                                   uint64_t l_new, uint64_t num_heads, uint64_t num_kv_heads, float scale,
                                   fa_buffer *out);
/* PagedKvCache::rewind_to / clear (paged_kv_device.rs:346-371): logical state only. */
fa_status fa_paged_cache_rewind_to(fa_paged_cache *cache, uint64_t new_len);
fa_status fa_paged_cache_clear(fa_paged_cache *cache);
/* snapshot_table / restore_table (paged_kv_device.rs:356-363). */
fa_status fa_paged_cache_snapshot_table(const fa_paged_cache *cache, fa_block_table **out);
fa_status fa_paged_cache_restore_table(fa_paged_cache *cache, const fa_block_table *saved);

/* ------------------------------------------------------------------ graphs */
/* Counterpart of the reference's captured inference chain
 * (BackendOps::linear_chain_forward_captured, backend_ops.rs:4814;
 * docs/inference-chain-single-sync-design.md:175-186).  Between begin and end
 * every call on the context is recorded instead of executed; calls that
 * synchronize or allocate return FA_ERR_CAPTURE_IN_PROGRESS.  A graph belongs
 * to the context that recorded it: only that context may launch or destroy it
 * (another one gets FA_ERR_DEVICE_MISMATCH), the scratch blocks its kernels use
 * return to that context's pool when it is destroyed, and fa_context_destroy
 * refuses (FA_ERR_INVALID_ARGUMENT) while graphs of the context are alive. */
typedef struct fa_graph fa_graph;
fa_status fa_graph_capture_begin(fa_context *ctx);
fa_status fa_graph_capture_end(fa_context *ctx, fa_graph **out);
fa_status fa_graph_launch(fa_context *ctx, fa_graph *graph);
fa_status fa_graph_destroy(fa_context *ctx, fa_graph *graph);

/* ---------------------------------------------------------- decoder step */
/* Llama-style decoder (pre-norm RMSNorm, GQA attention with RoPE over a
 * paged bf16 KV cache, SwiGLU FFN), W8A8 int8 linears, one new token per
 * sequence, greedy argmax.  The reference has no such model; it is the
 * composition of the operators above that the benchmark names. */
typedef struct {
    uint32_t n_layers, d_model, n_heads, n_kv_heads, head_dim, d_ffn, vocab;
    uint32_t block_size, max_blocks_per_seq, num_blocks;
    uint32_t max_batch;           /* rows of a step: 1..=64 */
    float rms_eps;
    double rope_theta;
} fa_decoder_config;
typedef struct fa_decoder fa_decoder;
fa_status fa_decoder_create(fa_context *ctx, const fa_decoder_config *cfg, fa_decoder **out);
fa_status fa_decoder_destroy(fa_context *ctx, fa_decoder *dec);
/* Weights: norm vectors and embedding are f32 buffers (copied by reference,
 * the caller keeps them alive); linears are fa_qweight of kind INT8_CHANNEL
 * with shapes qkv [d_model, (H + 2 H_kv) Dh], o [H Dh, d_model],
 * gate_up [d_model, 2 d_ffn] (gate columns first), down [d_ffn, d_model],
 * lm_head [d_model, vocab]. */
fa_status fa_decoder_set_layer(fa_decoder *dec, uint32_t layer, const fa_buffer *attn_norm,
                               const fa_buffer *ffn_norm, const fa_qweight *wqkv,
                               const fa_qweight *wo, const fa_qweight *wgu, const fa_qweight *wdown);
fa_status fa_decoder_set_head(fa_decoder *dec, const fa_buffer *embed, const fa_buffer *final_norm,
                              const fa_qweight *lm_head);
/* K / V pools of one layer: bf16 [num_blocks, block_size, H_kv * Dh]. */
fa_status fa_decoder_kv_pools(fa_decoder *dec, uint32_t layer, fa_buffer **k_pool, fa_buffer **v_pool);
/* Installs block tables [batch, max_blocks_per_seq] and the current
 * sequence lengths [batch] (host arrays; validated here). */
fa_status fa_decoder_set_sequences(fa_context *ctx, fa_decoder *dec, uint32_t batch,
                                   const uint32_t *block_tables, const uint32_t *seq_lens);
/* Installs the tokens [batch] to feed to the next step (host array). */
fa_status fa_decoder_set_tokens(fa_context *ctx, fa_decoder *dec, const int32_t *tokens);
/* One decode step, asynchronous: consumes the resident tokens, appends K/V,
 * advances the sequence lengths by one and leaves the argmax tokens resident
 * as the next step's input.  use_graph != 0 replays a captured HIP graph of
 * the step (captured on first use). */
fa_status fa_decoder_step(fa_context *ctx, fa_decoder *dec, int32_t use_graph);
/* How fa_decoder_step and fa_decoder_prefill pick the next token from the
 * logits (fa_sample_rows; greedy until this is called) and the seed of the
 * decoder's generator, whose state stays on the device so that a sampled step
 * can be captured and replayed like a greedy one. */
fa_status fa_decoder_set_sampling(fa_context *ctx, fa_decoder *dec, fa_sampling strategy, float temperature,
                                  uint64_t top_k, uint64_t seed);
/* Per-request sampling for the installed sequences (rows [batch], host array):
 * each row picks its next token by its own strategy from its own generator
 * (scheduler.rs:160-211, 553-562).  The table stays on the device and its
 * generator states advance there; read it back before the batch is rearranged
 * and install the rearranged table after fa_decoder_set_sequences.
 * fa_decoder_set_sampling returns to one strategy for all rows. */
fa_status fa_decoder_set_row_sampling(fa_context *ctx, fa_decoder *dec, const fa_row_sampling *rows);
fa_status fa_decoder_read_row_sampling(fa_context *ctx, fa_decoder *dec, fa_row_sampling *rows);
/* Prompt ingestion: l_new tokens per installed sequence (tokens [batch, l_new],
 * host array), written behind what each sequence has cached, on the
 * prefill-shape GEMMs and the prefill form of the attention kernel, in chunks of
 * at most 8192 rows.  Leaves the logits of every sequence's last prompt token
 * and its greedy next token resident, exactly as a decode step does, so
 * fa_decoder_step continues from there.  The per-row arithmetic is the decode
 * step's: a prompt token leaves the K / V rows it would leave if it were
 * decoded.  Rejected before anything is queued if a row has no pages for its
 * prompt.  Asynchronous apart from the upload of the token ids.  The activation
 * buffers of a pass that are 32 MiB or larger stay with the decoder for its next
 * pass (grow only, released by fa_decoder_destroy; about 1.8 GB for 8192 rows at
 * d_model 4096 / d_ffn 14336); smaller ones come from the context's pool. */
fa_status fa_decoder_prefill(fa_context *ctx, fa_decoder *dec, const int32_t *tokens, uint32_t l_new);
/* Prompts of different lengths in one pass: tokens [batch, l_max] holds row b's
 * row_lens[b] prompt tokens followed by padding (any valid token id), row_lens
 * [batch] is a host array with 1 <= row_lens[b] <= l_max, batch * l_max <= 4096.
 * Every row ends as if it had been ingested alone with fa_decoder_prefill: its
 * length advances by row_lens[b], the logits and the next token are those of
 * its own last prompt token.  The padding is computed and thrown away: its
 * cache rows land past the sequence's length (in pages the row owns, if any;
 * positions without a page are skipped) and are overwritten by later tokens.
 * What a scheduler uses when several requests join in the same iteration
 * (crates/autodiff/src/generate/scheduler.rs:521-562 admits them one by one). */
fa_status fa_decoder_prefill_padded(fa_context *ctx, fa_decoder *dec, const int32_t *tokens, uint32_t l_max,
                                    const uint32_t *row_lens);
/* Speculative-decoding verification (crates/autodiff/src/generate/speculative.rs:
 * 484-490: the target model consumes the pending token and the draft's k tokens
 * in one forward pass and every position's logits decide): fa_decoder_prefill
 * that also returns, for every row b * l_new + t, the greedy token after token t
 * of sequence b (picked [batch, l_new], host array) and, if logits is not null,
 * that row's logits ([batch * l_new, vocab] f32, host array).  At most 4096 rows;
 * synchronous.  The sequence lengths advance by l_new as in a prompt pass; what
 * was rejected is dropped with fa_decoder_rewind. */
fa_status fa_decoder_verify(fa_context *ctx, fa_decoder *dec, const int32_t *tokens, uint32_t l_new,
                            int32_t *picked, float *logits);
/* Shortens the installed sequences to seq_lens [batch] (host array; a row may
 * keep its length, none may grow).  The pages stay where they are and cached
 * rows past the new length are simply overwritten by later tokens: the paged
 * counterpart of the reference's snapshot / restore / replay
 * (crates/autodiff/src/generate/kv_rewind.rs:60-215), without the replay. */
fa_status fa_decoder_rewind(fa_context *ctx, fa_decoder *dec, const uint32_t *seq_lens);
/* Host copies of the current tokens [batch] / logits [batch, vocab] /
 * sequence lengths [batch] (synchronize). */
fa_status fa_decoder_read_tokens(fa_context *ctx, fa_decoder *dec, int32_t *tokens);
fa_status fa_decoder_read_logits(fa_context *ctx, fa_decoder *dec, float *logits);
fa_status fa_decoder_read_seq_lens(fa_context *ctx, fa_decoder *dec, uint32_t *seq_lens);
/* The decoder's resident logits, f32 [max_batch, vocab] (rows of the last step, prompt pass or verification by
 * step; not a copy, do not free): what fa_sampling_weights reads when the sampled form of speculative decoding
 * (speculative.rs:334-531) keeps the probabilities on the device. */
fa_status fa_decoder_logits_buffer(fa_decoder *dec, fa_buffer **out);

#ifdef __cplusplus
}
#endif
#endif
