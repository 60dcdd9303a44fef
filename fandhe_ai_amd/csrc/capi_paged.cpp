// C ABI: paged KV append and paged attention (host-table and device-table
// variants).  Host tables are validated completely before any launch
// (crates/backend-rocm/src/ops/paged_kv.rs:11-13: no partial writes).
#include <mutex>
#include <string>

#include "kernels.hpp"
#include "runtime.hpp"
#include "validate.hpp"

using namespace fa;

namespace fa {
extern int g_decode_waves, g_prefill_generic;
}

// ------------------------------------------------ scratch of the entry point that allocates nothing
// Partial results of the decode attention for callers that cannot allocate (under a graph capture of their
// own, in a serving loop that forbids it).  One array per GPU, held until the process ends; every call on a
// GPU shares it, so calls that overlap on one GPU race.  `scratch` is a host-side stand-in for the symbol:
// the device address is looked up once per device (scratch_address) and only that address is handed to
// kernels.
constexpr uint64_t kStaticScratchBytes = 16ull << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
void *g_scratch_addr[kMaxDevices];      // per device: each GPU holds its own copy of the array
std::string g_scratch_error[kMaxDevices];   // what the last failed lookup on the device reported
std::mutex g_scratch_mu;

}  // namespace

namespace fa {
// Called with `device` current (context creation).  The lookup may initialise the module on that device,
// which is why it happens at set-up and not inside the entry point.
// A lookup that fails is tried again by the next context created on the device (only a success is remembered);
// the entry point reports the last failure's text.
void static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return;
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (g_scratch_addr[device]) return;
    void *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
        g_scratch_error[device] = e != hipSuccess ? hipGetErrorString(e) : "hipGetSymbolAddress returned a null address";
        (void)hipGetLastError();
        return;
    }
    g_scratch_error[device].clear();
    g_scratch_addr[device] = ptr;
}
}  // namespace fa

namespace {

// Device address of the array on `device`, or null with the reason in *why.
void *scratch_address(int device, std::string *why) {
    if (device < 0 || device >= kMaxDevices) {
        *why = "device ordinal " + std::to_string(device) + " is outside the " + std::to_string(kMaxDevices) + " devices this entry point keeps an address for";
        return nullptr;
    }
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (!g_scratch_addr[device]) *why = g_scratch_error[device].empty() ? "no context has been created on the device" : g_scratch_error[device];
    return g_scratch_addr[device];
}

fa_status same_storage(const fa_buffer *a, const fa_buffer *b, const char *what) {
    if (a->dtype != b->dtype) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": element types differ");
    return FA_OK;
}

fa_status storage_f32_or_bf16(const fa_buffer *a, const char *what) {
    if (a->dtype != FA_F32 && a->dtype != FA_BF16)
        return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": must be f32 or bf16");
    return FA_OK;
}

k::PagedShape make_shape(const fa_paged_args *a) {
    k::PagedShape ps;
    uint64_t hkv = paged_kv_heads(a);
    ps.num_blocks = (uint32_t)a->layout.num_blocks;
    ps.block_size = (uint32_t)a->layout.block_size;
    ps.e_kv = (uint32_t)a->layout.embed_dim;
    ps.batch = (uint32_t)a->batch;
    ps.l_new = (uint32_t)a->l_new;
    ps.num_heads = (uint32_t)a->num_heads;
    ps.num_kv_heads = (uint32_t)hkv;
    ps.head_dim = (uint32_t)(a->layout.embed_dim / hkv);
    ps.max_blocks_per_seq = (uint32_t)a->max_blocks_per_seq;
    ps.scale = a->scale;
    return ps;
}

// shapes of the streamed matrix-core kernel: one new token per row (decode) or several (prefill)
bool stream_fast_path(const k::PagedShape &ps, const fa_buffer *q) {
    uint32_t group = ps.num_heads / ps.num_kv_heads;
    return q->dtype == FA_BF16 && ps.head_dim == 128 && ps.block_size == 16 && ps.l_new >= 1 && group <= 16 &&
           ps.max_blocks_per_seq >= 1;
}

// shared tail of the two attention entry points: tables already on the device
fa_status launch_attention(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool, const fa_buffer *v_pool,
                           const uint32_t *d_tables, const uint32_t *d_lens, const fa_paged_args *args,
                           uint64_t s_stride, uint32_t ctx_hint, fa_buffer *out) {
    k::PagedShape ps = make_shape(args);
    ps.ctx_hint = ctx_hint;
    if (stream_fast_path(ps, q) && ps.l_new > 1 && !g_prefill_generic) {
        uint64_t need = k::paged_prefill_workspace_bytes(ps, (uint32_t)g_decode_waves);
        if (fa_status s = ensure_workspace(ctx, need)) return s;
        k::paged_attention_prefill_bf16((const uint16_t *)q->ptr, (const uint16_t *)k_pool->ptr,
                                        (const uint16_t *)v_pool->ptr, d_tables, d_lens, ps, (uint32_t)g_decode_waves,
                                        ctx->workspace, out->ptr, out->dtype == FA_BF16, ctx->stream);
        return after_launch(ctx, "paged_attention_prefill_bf16");
    }
    if (stream_fast_path(ps, q) && ps.l_new == 1) {
        uint64_t need = k::paged_decode_workspace_bytes(ps, (uint32_t)g_decode_waves);
        if (fa_status s = ensure_workspace(ctx, need)) return s;
        k::paged_attention_decode_bf16((const uint16_t *)q->ptr, (const uint16_t *)k_pool->ptr,
                                       (const uint16_t *)v_pool->ptr, d_tables, d_lens, ps, (uint32_t)g_decode_waves,
                                       ctx->workspace, out->ptr, out->dtype == FA_BF16, nullptr, ctx->stream);
        return after_launch(ctx, "paged_attention_decode_bf16");
    }
    if (out->dtype != q->dtype) return fail(FA_ERR_INVALID_ARGUMENT, "paged_attention: out must have the type of q");
    uint64_t rows = (uint64_t)ps.batch * ps.num_heads * ps.l_new;
    uint64_t need;
    if (__builtin_mul_overflow(rows, s_stride, &need) || __builtin_mul_overflow(need, (uint64_t)4, &need))
        return fail(FA_ERR_INVALID_ARGUMENT, "paged_attention: workspace size overflows");
    if (fa_status s = ensure_workspace(ctx, need)) return s;
    if ((uint64_t)ps.head_dim * 4 > 48 * 1024) return fail(FA_ERR_UNSUPPORTED, "paged_attention: head_dim too large");
    k::paged_attention_generic(q->ptr, k_pool->ptr, v_pool->ptr, d_tables, d_lens, ps, q->dtype == FA_BF16,
                               (float *)ctx->workspace, s_stride, out->ptr, ctx->stream);
    return after_launch(ctx, "paged_attention_generic");
}

fa_status check_attention_buffers(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                  const fa_buffer *v_pool, fa_buffer *out) {
    if (fa_status s = check_buf(ctx, q, "paged_attention: q")) return s;
    if (fa_status s = check_buf(ctx, k_pool, "paged_attention: k_pool")) return s;
    if (fa_status s = check_buf(ctx, v_pool, "paged_attention: v_pool")) return s;
    if (fa_status s = check_buf(ctx, out, "paged_attention: out")) return s;
    if (fa_status s = storage_f32_or_bf16(q, "paged_attention: q")) return s;
    if (fa_status s = same_storage(q, k_pool, "paged_attention: q / k_pool")) return s;
    if (fa_status s = same_storage(q, v_pool, "paged_attention: q / v_pool")) return s;
    if (fa_status s = storage_f32_or_bf16(out, "paged_attention: out")) return s;
    return FA_OK;
}

}  // namespace

extern "C" {

fa_status fa_paged_kv_append(fa_context *ctx, const fa_buffer *k_new, const fa_buffer *v_new, fa_buffer *k_pool,
                             fa_buffer *v_pool, const uint32_t *slot_mapping, uint64_t rows,
                             const fa_paged_layout *layout) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, k_new, "paged_kv_append: k_new")) return s;
    if (fa_status s = check_buf(ctx, v_new, "paged_kv_append: v_new")) return s;
    if (fa_status s = check_buf(ctx, k_pool, "paged_kv_append: k_pool")) return s;
    if (fa_status s = check_buf(ctx, v_pool, "paged_kv_append: v_pool")) return s;
    if (fa_status s = storage_f32_or_bf16(k_new, "paged_kv_append: k_new")) return s;
    if (fa_status s = same_storage(k_new, v_new, "paged_kv_append: k_new / v_new")) return s;
    if (fa_status s = same_storage(k_new, k_pool, "paged_kv_append: k_new / k_pool")) return s;
    if (fa_status s = same_storage(k_new, v_pool, "paged_kv_append: k_new / v_pool")) return s;
    if (fa_status s = fa_validate_paged_kv_append(k_new->numel, v_new->numel, k_pool->numel, v_pool->numel,
                                                  slot_mapping, rows, layout))
        return s;
    if (rows == 0) return FA_OK;
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "paged_kv_append with host tables during graph capture");
    if (fa_status s = ensure_table_stage(ctx, rows * 4)) return s;
    hipError_t e = hipMemcpyAsync(ctx->table_stage, slot_mapping, rows * 4, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);      // the host array is consumed on return
    if (e != hipSuccess) return hip_fail(ctx, e, "slot_mapping upload", FA_ERR_TRANSFER_FAILED);
    k::paged_kv_append(k_new->ptr, v_new->ptr, k_pool->ptr, v_pool->ptr, (const uint32_t *)ctx->table_stage, rows,
                       layout->embed_dim, layout->num_blocks * layout->block_size, (int)dtype_size(k_new->dtype),
                       ctx->stream);
    return after_launch(ctx, "paged_kv_append");
}

fa_status fa_paged_kv_append_device(fa_context *ctx, const fa_buffer *k_new, const fa_buffer *v_new, fa_buffer *k_pool,
                                    fa_buffer *v_pool, const fa_buffer *slot_mapping, uint64_t rows,
                                    const fa_paged_layout *layout) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = paged_layout_check(layout)) return s;
    if (fa_status s = check_buf(ctx, k_new, "paged_kv_append: k_new")) return s;
    if (fa_status s = check_buf(ctx, v_new, "paged_kv_append: v_new")) return s;
    if (fa_status s = check_buf(ctx, k_pool, "paged_kv_append: k_pool")) return s;
    if (fa_status s = check_buf(ctx, v_pool, "paged_kv_append: v_pool")) return s;
    if (fa_status s = storage_f32_or_bf16(k_new, "paged_kv_append: k_new")) return s;
    if (fa_status s = same_storage(k_new, v_new, "paged_kv_append: k_new / v_new")) return s;
    if (fa_status s = same_storage(k_new, k_pool, "paged_kv_append: k_new / k_pool")) return s;
    if (fa_status s = same_storage(k_new, v_pool, "paged_kv_append: k_new / v_pool")) return s;
    if (fa_status s = check_buf_typed(ctx, slot_mapping, FA_U32, rows, "paged_kv_append: slot_mapping")) return s;
    uint64_t expect = rows * layout->embed_dim;
    uint64_t pool = layout->num_blocks * layout->block_size * layout->embed_dim;
    if (k_new->numel != expect || v_new->numel != expect)
        return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: k_new / v_new do not hold rows * E elements");
    if (k_pool->numel != pool || v_pool->numel != pool)
        return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: pool sizes do not match the layout");
    if (rows == 0) return FA_OK;
    if (rows > (uint64_t)INT32_MAX) return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: more than i32::MAX appended rows");
    k::paged_kv_append(k_new->ptr, v_new->ptr, k_pool->ptr, v_pool->ptr, (const uint32_t *)slot_mapping->ptr, rows,
                       layout->embed_dim, layout->num_blocks * layout->block_size, (int)dtype_size(k_new->dtype),
                       ctx->stream);
    return after_launch(ctx, "paged_kv_append");
}

fa_status fa_paged_attention_forward(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                     const fa_buffer *v_pool, const uint32_t *block_tables, uint64_t n_tables,
                                     const uint32_t *seq_lens, uint64_t n_seq, const fa_paged_args *args,
                                     fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_attention_buffers(ctx, q, k_pool, v_pool, out)) return s;
    fa_paged_plan plan;
    if (fa_status s = fa_validate_paged_attention(q->numel, k_pool->numel, v_pool->numel, block_tables, n_tables,
                                                  seq_lens, n_seq, args, &plan))
        return s;
    if (out->numel < plan.out_numel) return fail(FA_ERR_SHAPE_MISMATCH, "paged_attention: out is too small");
    if (plan.out_numel == 0) return FA_OK;
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "paged_attention with host tables during graph capture");
    uint64_t tb = n_tables * 4, lb = n_seq * 4;
    uint64_t lens_off = (tb + 255) / 256 * 256;
    if (fa_status s = ensure_table_stage(ctx, lens_off + lb)) return s;
    hipError_t e = hipMemcpyAsync(ctx->table_stage, block_tables, tb, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess)
        e = hipMemcpyAsync((char *)ctx->table_stage + lens_off, seq_lens, lb, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "block table upload", FA_ERR_TRANSFER_FAILED);
    uint32_t longest = 0;
    for (uint64_t i = 0; i < n_seq; ++i) longest = seq_lens[i] > longest ? seq_lens[i] : longest;
    return launch_attention(ctx, q, k_pool, v_pool, (const uint32_t *)ctx->table_stage,
                            (const uint32_t *)((char *)ctx->table_stage + lens_off), args, plan.s_max, longest, out);
}

// argument checks shared by the two device-table entry points; *s_stride receives the longest sequence the
// tables can describe, *done is set when there is nothing to compute
static fa_status check_device_attention(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                        const fa_buffer *v_pool, const fa_buffer *block_tables,
                                        const fa_buffer *seq_lens, const fa_paged_args *args, fa_buffer *out,
                                        uint64_t *s_stride, bool *done) {
    *done = false;
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = paged_args_check(args)) return s;
    if (fa_status s = check_attention_buffers(ctx, q, k_pool, v_pool, out)) return s;
    const fa_paged_layout *l = &args->layout;
    uint64_t dh = l->embed_dim / paged_kv_heads(args);
    uint64_t out_numel = args->batch * args->l_new * args->num_heads * dh;
    uint64_t pool = l->num_blocks * l->block_size * l->embed_dim;
    if (q->numel != out_numel) return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: q does not hold B * L_new * E elements");
    if (k_pool->numel != pool || v_pool->numel != pool)
        return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: pool sizes do not match the layout");
    if (out->numel < out_numel) return fail(FA_ERR_SHAPE_MISMATCH, "paged_attention: out is too small");
    if (fa_status s = check_buf_typed(ctx, block_tables, FA_U32, args->batch * args->max_blocks_per_seq,
                                      "paged_attention: block_tables"))
        return s;
    if (fa_status s = check_buf_typed(ctx, seq_lens, FA_U32, args->batch, "paged_attention: seq_lens")) return s;
    if (out_numel == 0) {
        *done = true;
        return FA_OK;
    }
    uint64_t query_rows = args->batch * args->num_heads * args->l_new;
    if (query_rows > (uint64_t)INT32_MAX) return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: B * H * L_new exceeds i32::MAX");
    *s_stride = args->max_blocks_per_seq * l->block_size;
    return FA_OK;
}

fa_status fa_paged_attention_forward_device(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                            const fa_buffer *v_pool, const fa_buffer *block_tables,
                                            const fa_buffer *seq_lens, const fa_paged_args *args, fa_buffer *out) {
    uint64_t s_stride = 0;
    bool done = false;
    if (fa_status s = check_device_attention(ctx, q, k_pool, v_pool, block_tables, seq_lens, args, out, &s_stride, &done))
        return s;
    if (done) return FA_OK;
    return launch_attention(ctx, q, k_pool, v_pool, (const uint32_t *)block_tables->ptr,
                            (const uint32_t *)seq_lens->ptr, args, s_stride, 0, out);
}

fa_status fa_paged_attention_decode_static(fa_context *ctx, const fa_buffer *q, const fa_buffer *k_pool,
                                           const fa_buffer *v_pool, const fa_buffer *block_tables,
                                           const fa_buffer *seq_lens, const fa_paged_args *args, fa_buffer *out) {
    uint64_t s_stride = 0;
    bool done = false;
    if (fa_status s = check_device_attention(ctx, q, k_pool, v_pool, block_tables, seq_lens, args, out, &s_stride, &done))
        return s;
    if (done) return FA_OK;
    const k::PagedShape ps = make_shape(args);
    if (!(stream_fast_path(ps, q) && ps.l_new == 1))
        return fail(FA_ERR_UNSUPPORTED,
                    "paged_attention_decode_static: only the decode shape of the streamed kernel (bf16, head_dim 128, "
                    "block_size 16, one new token per row, at most 16 query heads per kv head)");
    const uint64_t need = k::paged_decode_workspace_bytes(ps, (uint32_t)g_decode_waves);
    if (need > kStaticScratchBytes)
        return fail(FA_ERR_INVALID_ARGUMENT,
                    "paged_attention_decode_static: the partial results of this shape need " + std::to_string(need) +
                        " bytes, the static scratch holds " + std::to_string(kStaticScratchBytes) +
                        " (fewer rows or kv heads, or fa_paged_attention_forward_device)");
    std::string why;
    void *ws = scratch_address(ctx->device, &why);
    if (!ws)
        return fail(FA_ERR_DEVICE_UNAVAILABLE, "paged_attention_decode_static: the address of the static scratch could not "
                                               "be resolved when the context was created (" + why + ")");
    k::paged_attention_decode_bf16((const uint16_t *)q->ptr, (const uint16_t *)k_pool->ptr, (const uint16_t *)v_pool->ptr,
                                   (const uint32_t *)block_tables->ptr, (const uint32_t *)seq_lens->ptr, ps,
                                   (uint32_t)g_decode_waves, ws, out->ptr, out->dtype == FA_BF16, nullptr, ctx->stream);
    return after_launch(ctx, "paged_attention_decode_static");
}

uint64_t fa_paged_attention_decode_static_max_bytes(void) { return kStaticScratchBytes; }

}  // extern "C"
