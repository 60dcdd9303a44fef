// C ABI: dense / quantized linears, norms and elementwise operators.
// Every entry point validates shapes against what the kernel and its grid
// assume before it launches anything.
#include <cmath>
#include <new>
#include <string>

#include "kernels.hpp"
#include "runtime.hpp"

using namespace fa;

namespace fa {
namespace k {
extern int g_gemm_f32_form, g_weight_prefetch, g_probe_plain_loads, g_rows_wide;
extern int g_skinny_ksplit, g_skinny_ksplit_s, g_row_fusion;
extern int g_rows_kernel;
extern int g_skinny_ntw, g_skinny_waves, g_skinny_astat, g_gemm_small_tiles, g_gemm_waves, g_gemm_ntb, g_gemm_split_fill;
}
int g_decode_waves = 0;
int g_prefill_generic = 0;
extern int g_prefill_rows, g_prefill_fused_rows, g_decode_partials_only, g_prefill_block_form, g_prefill_block_waves, g_prefill_block_split, g_prefill_block_cols;
}  // namespace fa

namespace {

uint64_t round_up(uint64_t v, uint64_t to) { return (v + to - 1) / to * to; }

bool mul3(uint64_t a, uint64_t b, uint64_t *r) { return !__builtin_mul_overflow(a, b, r); }

fa_status check_view(const fa_context *ctx, const fa_buffer *b, uint64_t offset, uint64_t numel, fa_dtype t,
                     const char *what) {
    if (fa_status s = check_buf(ctx, b, what)) return s;
    if (b->dtype != t) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": wrong element type");
    uint64_t end;
    if (__builtin_add_overflow(offset, numel, &end) || end > b->numel)
        return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": view range exceeds the backing buffer");
    return FA_OK;
}

fa_status check_qw(const fa_context *ctx, const fa_qweight *qw, fa_qweight_kind kind, const char *what) {
    if (!qw || qw->magic != kQwMagic) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": not a quantized weight");
    if (qw->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, std::string(what) + ": weight belongs to another context");
    if (qw->kind != kind) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": wrong weight kind");
    return FA_OK;
}

// scratch taken from the pool for the duration of one call; the block goes
// back right after the launch, which is safe because every later use is
// ordered after it on the context's stream.  A call recorded into a graph
// capture hands its scratch to the graph instead (scratch_release): the
// recorded kernels use those addresses on every replay.
struct Scratch {
    fa_context *ctx;
    void *ptr = nullptr;
    uint64_t bytes = 0, cls = 0;
    explicit Scratch(fa_context *c) : ctx(c) {}
    fa_status get(uint64_t n) {
        bytes = n;
        return pool_alloc(ctx, n, &ptr, &cls);
    }
    ~Scratch() {
        if (ptr) scratch_release(ctx, ptr, bytes, cls);
    }
};

}  // namespace

extern "C" {

// Tuning knobs for experiments (0 restores the built-in choice):
// key 0 = n-tiles per block of the skinny linears, 1 = wavefronts per block,
// 2 = wavefronts per compute unit of the decode attention, 3 = decode attention launches its streaming
// kernel only (timing aid), 4 = prefill GEMMs keep the 128 x 128 block tile for every shape,
// 5 = activation-stationary decode linears (1 never, 2 whenever they can run); the remaining keys are
// described beside the declaration.
fa_status fa_set_tuning(int32_t key, int32_t value) {
    switch (key) {
        case 0: k::g_skinny_ntw = value; return FA_OK;
        case 1: k::g_skinny_waves = value; return FA_OK;
        case 2: fa::g_decode_waves = value; return FA_OK;
        case 3: fa::g_decode_partials_only = value; return FA_OK;
        case 4: k::g_gemm_small_tiles = value; return FA_OK;
        case 5: k::g_skinny_astat = value; return FA_OK;
        case 6: k::g_gemm_waves = value; return FA_OK;
        case 7: k::g_gemm_ntb = value; return FA_OK;
        case 8: fa::g_prefill_generic = value; return FA_OK;
        case 9: k::g_gemm_split_fill = value; return FA_OK;
        case 10: fa::g_prefill_block_form = value; return FA_OK;
        case 11: fa::g_prefill_block_waves = value; return FA_OK;
        case 12: fa::g_prefill_block_split = value; return FA_OK;
        case 13: k::g_gemm_f32_form = value; return FA_OK;
        case 14: k::g_weight_prefetch = value; return FA_OK;
        case 15: k::g_probe_plain_loads = value; return FA_OK;
        case 16: k::g_skinny_ksplit = value; return FA_OK;
        case 17: k::g_skinny_ksplit_s = value; return FA_OK;
        case 18: k::g_rows_wide = value; return FA_OK;
        case 19: k::g_row_fusion = value; return FA_OK;
        case 20: k::g_decode_one = value; return FA_OK;
        case 21: k::g_rows_kernel = value; return FA_OK;
        case 22: k::g_gemm_swiglu = value; return FA_OK;
        case 23: fa::g_prefill_block_cols = value; return FA_OK;
        case 24: k::g_gemm_pair = value; return FA_OK;
        case 25: fa::g_prefill_rows = value; return FA_OK;
        case 26: fa::g_prefill_fused_rows = value; return FA_OK;
        case 27: k::g_rows_rope = value; return FA_OK;
    }
    return fail(FA_ERR_INVALID_ARGUMENT, "fa_set_tuning: unknown key");
}

fa_status fa_gemm_f32_form_query(uint64_t m, uint64_t n, uint64_t k, int32_t *form) {
    if (!form) return fail(FA_ERR_INVALID_ARGUMENT, "gemm_f32_form_query: null out");
    *form = k::gemm_f32_form(m, n, k);
    return FA_OK;
}

fa_status fa_gemm_plan_query(const fa_context *ctx, uint64_t m, const fa_qweight *qw, fa_gemm_plan *out) {
    if (!ctx || ctx->magic != kCtxMagic || !out) return fail(FA_ERR_INVALID_ARGUMENT, "gemm_plan_query: bad argument");
    if (!qw || qw->magic != kQwMagic) return fail(FA_ERR_INVALID_ARGUMENT, "gemm_plan_query: not a quantized weight");
    const k::GemmPlan p = k::gemm_plan(qw->kind != FA_QW_INT8_CHANNEL, m, qw->n_pad, qw->k_pad, ctx->props.multiProcessorCount);
    out->big_ntb = p.big_ntb;
    out->waves = p.waves;
    out->splits = p.splits;
    return FA_OK;
}

// ------------------------------------------------------------- f32 linear
fa_status fa_gemm_device(fa_context *ctx, const fa_buffer *a, const fa_buffer *b, uint64_t m, uint64_t n, uint64_t k,
                         fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t mk, kn, mn;
    if (!mul3(m, k, &mk) || !mul3(k, n, &kn) || !mul3(m, n, &mn)) return fail(FA_ERR_SHAPE_MISMATCH, "gemm: shape overflows");
    if (fa_status s = check_buf_typed(ctx, a, FA_F32, mk, "gemm: a")) return s;
    if (fa_status s = check_buf_typed(ctx, b, FA_F32, kn, "gemm: b")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, mn, "gemm: out")) return s;
    if (a->numel != mk || b->numel != kn) return fail(FA_ERR_SHAPE_MISMATCH, "gemm: operand sizes do not match m, n, k");
    if (mn == 0) return FA_OK;
    if ((m + 63) / 64 > 65535) return fail(FA_ERR_INVALID_ARGUMENT, "gemm: m too large for one launch");
    k::gemm_f32((const float *)a->ptr, (const float *)b->ptr, nullptr, (float *)out->ptr, m, n, k, 0, ctx->stream);
    return after_launch(ctx, "gemm_f32");
}

fa_status fa_linear_forward_device(fa_context *ctx, const fa_buffer *a, uint64_t m, uint64_t k, const fa_buffer *w,
                                   uint64_t w_offset, uint64_t n, const fa_buffer *bias, uint64_t bias_offset,
                                   fa_activation act, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t mk, kn, mn;
    if (!mul3(m, k, &mk) || !mul3(k, n, &kn) || !mul3(m, n, &mn))
        return fail(FA_ERR_SHAPE_MISMATCH, "linear_forward_device: shape overflows");
    if (fa_status s = check_buf_typed(ctx, a, FA_F32, mk, "linear_forward_device: a")) return s;
    if (a->numel != mk) return fail(FA_ERR_SHAPE_MISMATCH, "linear_forward_device: a is not [m, k]");
    if (fa_status s = check_view(ctx, w, w_offset, kn, FA_F32, "linear_forward_device: w")) return s;
    if (bias)
        if (fa_status s = check_view(ctx, bias, bias_offset, n, FA_F32, "linear_forward_device: bias")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, mn, "linear_forward_device: out")) return s;
    if (act != FA_ACT_NONE && act != FA_ACT_RELU)
        return fail(FA_ERR_UNSUPPORTED, "linear_forward_device: activation must be None or Relu");
    if (mn == 0) return FA_OK;
    if ((m + 63) / 64 > 65535) return fail(FA_ERR_INVALID_ARGUMENT, "linear_forward_device: m too large for one launch");
    k::gemm_f32((const float *)a->ptr, (const float *)w->ptr + w_offset,
                bias ? (const float *)bias->ptr + bias_offset : nullptr, (float *)out->ptr, m, n, k,
                act == FA_ACT_RELU ? 1 : 0, ctx->stream);
    return after_launch(ctx, "gemm_f32(linear)");
}

// ------------------------------------------------------- quantized weights
static fa_status qweight_alloc(fa_context *ctx, uint64_t kdim, uint64_t n, fa_qweight_kind kind, fa_qweight **out) {
    if (kind != FA_QW_INT8_CHANNEL && kind != FA_QW_E4M3_TENSOR && kind != FA_QW_E4M3_CHANNEL)
        return fail(FA_ERR_INVALID_ARGUMENT, "qweight: unknown kind");
    if (kdim == 0 || n == 0) return fail(FA_ERR_INVALID_ARGUMENT, "qweight: k and n must be positive");
    if (kdim > (1ull << 31) || n > (1ull << 31)) return fail(FA_ERR_INVALID_ARGUMENT, "qweight: dimension too large");
    uint64_t tk = kind == FA_QW_INT8_CHANNEL ? 64 : 128;
    fa_qweight *qw = new (std::nothrow) fa_qweight();
    if (!qw) return fail(FA_ERR_ALLOCATION_FAILED, "qweight: host allocation failed");
    qw->magic = kQwMagic;
    qw->ctx = ctx;
    qw->kind = kind;
    qw->k = kdim;
    qw->n = n;
    qw->k_pad = round_up(kdim, tk);
    qw->n_pad = round_up(n, 16);
    qw->codes = nullptr;
    qw->scales = nullptr;
    fa_status s = make_buffer(ctx, kind == FA_QW_INT8_CHANNEL ? FA_I8 : FA_E4M3, qw->k_pad * qw->n_pad, false, &qw->codes);
    if (s == FA_OK) s = make_buffer(ctx, FA_F32, kind == FA_QW_E4M3_TENSOR ? 1 : qw->n_pad, true, &qw->scales);
    if (s != FA_OK) {
        if (qw->codes) fa_buffer_free(ctx, qw->codes);
        delete qw;
        return s;
    }
    *out = qw;
    return FA_OK;
}

fa_status fa_qweight_from_f32(fa_context *ctx, const fa_buffer *w, uint64_t w_offset, uint64_t kdim, uint64_t n,
                              fa_qweight_kind kind, fa_qweight **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "qweight_from_f32: null output");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "qweight_from_f32 during graph capture");
    uint64_t kn;
    if (!mul3(kdim, n, &kn)) return fail(FA_ERR_SHAPE_MISMATCH, "qweight_from_f32: shape overflows");
    if (fa_status s = check_view(ctx, w, w_offset, kn, FA_F32, "qweight_from_f32: w")) return s;
    fa_qweight *qw = nullptr;
    if (fa_status s = qweight_alloc(ctx, kdim, n, kind, &qw)) return s;
    const float *wp = (const float *)w->ptr + w_offset;
    if (kind == FA_QW_INT8_CHANNEL) {
        k::weight_col_scales_i8(wp, kdim, n, qw->n_pad, (float *)qw->scales->ptr, ctx->stream);
        k::weight_quantize_pack_i8(wp, (const float *)qw->scales->ptr, kdim, n, qw->k_pad, qw->n_pad,
                                   (int8_t *)qw->codes->ptr, ctx->stream);
    } else if (kind == FA_QW_E4M3_CHANNEL) {
        k::weight_col_scales(wp, kdim, n, qw->n_pad, 448.0f, (float *)qw->scales->ptr, ctx->stream);
        k::weight_quantize_pack_e4m3_cols(wp, (const float *)qw->scales->ptr, kdim, n, qw->k_pad, qw->n_pad,
                                          (uint8_t *)qw->codes->ptr, ctx->stream);
    } else {
        Scratch am(ctx);
        if (fa_status s = am.get(4)) {
            fa_qweight_free(ctx, qw);
            return s;
        }
        k::tensor_absmax_f32(wp, kn, (float *)am.ptr, ctx->stream);
        k::scale_from_absmax((const float *)am.ptr, 448.0f, (float *)qw->scales->ptr, ctx->stream);
        k::weight_quantize_pack_e4m3(wp, (const float *)qw->scales->ptr, kdim, n, qw->k_pad, qw->n_pad,
                                     (uint8_t *)qw->codes->ptr, ctx->stream);
    }
    if (fa_status s = after_launch(ctx, "weight quantize/pack")) {
        fa_qweight_free(ctx, qw);
        return s;
    }
    *out = qw;
    return FA_OK;
}

fa_status fa_qweight_from_codes(fa_context *ctx, const void *codes, const float *scales, uint64_t kdim, uint64_t n,
                                fa_qweight_kind kind, fa_qweight **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!out || !codes || !scales) return fail(FA_ERR_INVALID_ARGUMENT, "qweight_from_codes: null argument");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "qweight_from_codes during graph capture");
    uint64_t kn;
    if (!mul3(kdim, n, &kn)) return fail(FA_ERR_SHAPE_MISMATCH, "qweight_from_codes: shape overflows");
    fa_qweight *qw = nullptr;
    if (fa_status s = qweight_alloc(ctx, kdim, n, kind, &qw)) return s;
    fa_buffer *tmp = nullptr;
    fa_status s = fa_upload(ctx, FA_I8, codes, kn, &tmp);
    if (s == FA_OK) s = fa_upload_into(ctx, scales, kind == FA_QW_E4M3_TENSOR ? 1 : n, qw->scales, 0);
    if (s == FA_OK) {
        k::weight_pack_codes((const uint8_t *)tmp->ptr, kdim, n, qw->k_pad, qw->n_pad,
                             kind == FA_QW_INT8_CHANNEL ? 64 : 128, (uint8_t *)qw->codes->ptr, ctx->stream);
        s = after_launch(ctx, "weight_pack_codes");
    }
    if (tmp) fa_buffer_free(ctx, tmp);
    if (s != FA_OK) {
        fa_qweight_free(ctx, qw);
        return s;
    }
    *out = qw;
    return FA_OK;
}

fa_status fa_qweight_export(fa_context *ctx, const fa_qweight *qw, void *codes, float *scales) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!qw || qw->magic != kQwMagic) return fail(FA_ERR_INVALID_ARGUMENT, "qweight_export: not a quantized weight");
    if (qw->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "qweight_export: weight belongs to another context");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "qweight_export during graph capture");
    if (codes) {
        fa_buffer *tmp = nullptr;
        if (fa_status s = make_buffer(ctx, FA_I8, qw->k * qw->n, false, &tmp)) return s;
        k::weight_unpack_codes((const uint8_t *)qw->codes->ptr, qw->k, qw->n, qw->k_pad, qw->n_pad,
                               qw->kind == FA_QW_INT8_CHANNEL ? 64 : 128, (uint8_t *)tmp->ptr, ctx->stream);
        fa_status s = after_launch(ctx, "weight_unpack_codes");
        if (s == FA_OK) s = fa_download(ctx, tmp, 0, codes, qw->k * qw->n);
        fa_buffer_free(ctx, tmp);
        if (s != FA_OK) return s;
    }
    if (scales) return fa_download(ctx, qw->scales, 0, scales, qw->kind == FA_QW_E4M3_TENSOR ? 1 : qw->n);
    return FA_OK;
}

fa_status fa_qweight_free(fa_context *ctx, fa_qweight *qw) {
    if (!qw) return FA_OK;
    if (qw->magic != kQwMagic) return fail(FA_ERR_INVALID_ARGUMENT, "qweight_free: not a quantized weight");
    if (qw->codes) fa_buffer_free(ctx, qw->codes);
    if (qw->scales) fa_buffer_free(ctx, qw->scales);
    qw->magic = 0;
    delete qw;
    return FA_OK;
}

uint64_t fa_qweight_k(const fa_qweight *qw) { return qw && qw->magic == kQwMagic ? qw->k : 0; }
uint64_t fa_qweight_n(const fa_qweight *qw) { return qw && qw->magic == kQwMagic ? qw->n : 0; }

// ------------------------------------------------------ quantized linears
fa_status fa_quantize_rows_i8(fa_context *ctx, const fa_buffer *x, uint64_t m, uint64_t kdim, fa_buffer *xq,
                              fa_buffer *sx) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t mk;
    if (!mul3(m, kdim, &mk)) return fail(FA_ERR_SHAPE_MISMATCH, "quantize_rows_i8: shape overflows");
    if (fa_status s = check_buf(ctx, x, "quantize_rows_i8: x")) return s;
    if (x->dtype != FA_F32 && x->dtype != FA_BF16) return fail(FA_ERR_INVALID_ARGUMENT, "quantize_rows_i8: x must be f32 or bf16");
    if (x->numel < mk) return fail(FA_ERR_SHAPE_MISMATCH, "quantize_rows_i8: x is smaller than [m, k]");
    if (fa_status s = check_buf_typed(ctx, xq, FA_I8, mk, "quantize_rows_i8: xq")) return s;
    if (fa_status s = check_buf_typed(ctx, sx, FA_F32, m, "quantize_rows_i8: sx")) return s;
    if (mk == 0) return FA_OK;
    if (m > (1ull << 31) - 1) return fail(FA_ERR_INVALID_ARGUMENT, "quantize_rows_i8: too many rows");
    k::quantize_rows_i8(x->ptr, x->dtype == FA_BF16, (int8_t *)xq->ptr, nullptr, (float *)sx->ptr, m, m, kdim,
                        round_up(kdim, 16), ctx->stream);
    return after_launch(ctx, "quantize_rows_i8");
}

static fa_status check_out_f32_or_bf16(const fa_context *ctx, const fa_buffer *out, uint64_t numel, const char *what) {
    if (fa_status s = check_buf(ctx, out, what)) return s;
    if (out->dtype != FA_F32 && out->dtype != FA_BF16)
        return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": must be f32 or bf16");
    if (out->numel < numel) return fail(FA_ERR_SHAPE_MISMATCH, std::string(what) + ": too small");
    return FA_OK;
}

fa_status fa_linear_w8a8(fa_context *ctx, const fa_buffer *x, uint64_t m, const fa_qweight *qw, const fa_buffer *bias,
                         uint64_t bias_offset, fa_buffer *acc_out, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_qw(ctx, qw, FA_QW_INT8_CHANNEL, "linear_w8a8: weight")) return s;
    uint64_t mk, mn;
    if (!mul3(m, qw->k, &mk) || !mul3(m, qw->n, &mn)) return fail(FA_ERR_SHAPE_MISMATCH, "linear_w8a8: shape overflows");
    if (fa_status s = check_buf(ctx, x, "linear_w8a8: x")) return s;
    if (x->dtype != FA_F32 && x->dtype != FA_BF16) return fail(FA_ERR_INVALID_ARGUMENT, "linear_w8a8: x must be f32 or bf16");
    if (x->numel != mk) return fail(FA_ERR_SHAPE_MISMATCH, "linear_w8a8: x is not [m, k]");
    if (bias)
        if (fa_status s = check_view(ctx, bias, bias_offset, qw->n, FA_F32, "linear_w8a8: bias")) return s;
    if (acc_out)
        if (fa_status s = check_buf_typed(ctx, acc_out, FA_I32, mn, "linear_w8a8: acc_out")) return s;
    if (fa_status s = check_out_f32_or_bf16(ctx, out, mn, "linear_w8a8: out")) return s;
    if (mn == 0) return FA_OK;
    if (m > (1ull << 22)) return fail(FA_ERR_INVALID_ARGUMENT, "linear_w8a8: m too large for one launch");

    Scratch sx(ctx), xq(ctx);
    if (fa_status s = sx.get(m * 4)) return s;
    k::EpilogueI8 ep;
    ep.sx = (const float *)sx.ptr;
    ep.sw = (const float *)qw->scales->ptr;
    ep.bias = bias ? (const float *)bias->ptr + bias_offset : nullptr;
    ep.residual = nullptr;
    ep.acc_out = acc_out ? (int32_t *)acc_out->ptr : nullptr;
    ep.out = out->ptr;
    ep.out_bf16 = out->dtype == FA_BF16;
    if (m <= 64) {
        uint64_t m_pad = round_up(m, 16);
        if (fa_status s = xq.get(m_pad * qw->k_pad)) return s;
        k::quantize_rows_i8(x->ptr, x->dtype == FA_BF16, nullptr, (int8_t *)xq.ptr, (float *)sx.ptr, m, m_pad, qw->k,
                            qw->k_pad, ctx->stream);
        k::linear_w8a8_skinny((const int8_t *)xq.ptr, (const int8_t *)qw->codes->ptr, m, qw->n, qw->n_pad, qw->k_pad,
                              ep, ctx->props.multiProcessorCount, ctx->stream, &ctx->splitk);
    } else if (qw->k == qw->k_pad &&
               k::linear_w8a8_rows_applies(m, qw->n_pad, qw->k_pad, ctx->props.multiProcessorCount, &ctx->splitk)) {
        uint64_t m_pad = round_up(m, 16);
        if (fa_status s = xq.get(m_pad * qw->k_pad)) return s;
        Scratch ws(ctx);
        if (uint64_t wsb = k::linear_w8a8_rows_workspace_bytes(m, qw->n_pad, qw->k_pad, ctx->props.multiProcessorCount, &ctx->splitk))
            if (fa_status s = ws.get(wsb)) return s;
        k::quantize_rows_i8(x->ptr, x->dtype == FA_BF16, nullptr, (int8_t *)xq.ptr, (float *)sx.ptr, m, m_pad, qw->k,
                            qw->k_pad, ctx->stream);
        k::linear_w8a8_rows((const int8_t *)xq.ptr, (const int8_t *)qw->codes->ptr, m, qw->n, qw->n_pad, qw->k_pad, ep,
                            ctx->props.multiProcessorCount, ctx->stream, &ctx->splitk, ws.ptr, ws.bytes);
    } else {
        if (qw->k != qw->k_pad) return fail(FA_ERR_UNSUPPORTED, "linear_w8a8: m > 64 needs k to be a multiple of 64");
        if (fa_status s = xq.get(mk)) return s;
        k::quantize_rows_i8(x->ptr, x->dtype == FA_BF16, (int8_t *)xq.ptr, nullptr, (float *)sx.ptr, m, m, qw->k,
                            qw->k_pad, ctx->stream);
        Scratch ws(ctx);
        if (uint64_t wsb = k::gemm_w8a8_workspace_bytes(m, qw->n, qw->n_pad, qw->k_pad, ctx->props.multiProcessorCount))
            if (fa_status s = ws.get(wsb)) return s;
        k::gemm_w8a8_mfma((const int8_t *)xq.ptr, (const int8_t *)qw->codes->ptr, m, qw->n, qw->n_pad, qw->k_pad, ep,
                          ctx->props.multiProcessorCount, ctx->stream, ws.ptr, ws.bytes, &ctx->splitk);
    }
    return after_launch(ctx, "linear_w8a8");
}

fa_status fa_gemm_w8a8(fa_context *ctx, const fa_buffer *aq, const fa_buffer *sx, uint64_t m, const fa_qweight *qw,
                       fa_buffer *acc_out, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_qw(ctx, qw, FA_QW_INT8_CHANNEL, "gemm_w8a8: weight")) return s;
    if (qw->k != qw->k_pad) return fail(FA_ERR_UNSUPPORTED, "gemm_w8a8: k must be a multiple of 64");
    uint64_t mk, mn;
    if (!mul3(m, qw->k, &mk) || !mul3(m, qw->n, &mn)) return fail(FA_ERR_SHAPE_MISMATCH, "gemm_w8a8: shape overflows");
    if (fa_status s = check_buf_typed(ctx, aq, FA_I8, mk, "gemm_w8a8: aq")) return s;
    if (fa_status s = check_buf_typed(ctx, sx, FA_F32, m, "gemm_w8a8: sx")) return s;
    if (acc_out)
        if (fa_status s = check_buf_typed(ctx, acc_out, FA_I32, mn, "gemm_w8a8: acc_out")) return s;
    if (fa_status s = check_out_f32_or_bf16(ctx, out, mn, "gemm_w8a8: out")) return s;
    if (mn == 0) return FA_OK;
    if (m > (1ull << 22)) return fail(FA_ERR_INVALID_ARGUMENT, "gemm_w8a8: m too large for one launch");
    k::EpilogueI8 ep;
    ep.sx = (const float *)sx->ptr;
    ep.sw = (const float *)qw->scales->ptr;
    ep.bias = nullptr;
    ep.residual = nullptr;
    ep.acc_out = acc_out ? (int32_t *)acc_out->ptr : nullptr;
    ep.out = out->ptr;
    ep.out_bf16 = out->dtype == FA_BF16;
    Scratch ws(ctx);
    if (uint64_t wsb = k::gemm_w8a8_workspace_bytes(m, qw->n, qw->n_pad, qw->k_pad, ctx->props.multiProcessorCount))
        if (fa_status s = ws.get(wsb)) return s;
    k::gemm_w8a8_mfma((const int8_t *)aq->ptr, (const int8_t *)qw->codes->ptr, m, qw->n, qw->n_pad, qw->k_pad, ep,
                      ctx->props.multiProcessorCount, ctx->stream, ws.ptr, ws.bytes, &ctx->splitk);
    return after_launch(ctx, "gemm_w8a8_mfma");
}

fa_status fa_linear_w8a16(fa_context *ctx, const fa_buffer *a, uint64_t m, const fa_qweight *qw, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_qw(ctx, qw, FA_QW_INT8_CHANNEL, "linear_w8a16: weight")) return s;
    if (m > 32) return fail(FA_ERR_UNSUPPORTED, "linear_w8a16: decode-shape kernel, m must be at most 32");
    if (qw->k != qw->k_pad) return fail(FA_ERR_UNSUPPORTED, "linear_w8a16: k must be a multiple of 64");
    uint64_t mk = m * qw->k, mn = m * qw->n;
    if (fa_status s = check_buf_typed(ctx, a, FA_BF16, mk, "linear_w8a16: a")) return s;
    if (a->numel != mk) return fail(FA_ERR_SHAPE_MISMATCH, "linear_w8a16: a is not [m, k]");
    if (fa_status s = check_out_f32_or_bf16(ctx, out, mn, "linear_w8a16: out")) return s;
    if (mn == 0) return FA_OK;
    k::linear_w8a16_skinny((const uint16_t *)a->ptr, (const int8_t *)qw->codes->ptr, (const float *)qw->scales->ptr, m,
                           qw->n, qw->n_pad, qw->k_pad, out->ptr, out->dtype == FA_BF16,
                           ctx->props.multiProcessorCount, ctx->stream, &ctx->splitk);
    return after_launch(ctx, "linear_w8a16_skinny");
}

fa_status fa_quantize_tensor_e4m3(fa_context *ctx, const fa_buffer *x, uint64_t numel, fa_buffer *xq, fa_buffer *scale) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf_typed(ctx, x, FA_F32, numel, "quantize_tensor_e4m3: x")) return s;
    if (fa_status s = check_buf_typed(ctx, xq, FA_E4M3, numel, "quantize_tensor_e4m3: xq")) return s;
    if (fa_status s = check_buf_typed(ctx, scale, FA_F32, 1, "quantize_tensor_e4m3: scale")) return s;
    Scratch am(ctx);
    if (fa_status s = am.get(4)) return s;
    k::quantize_tensor_e4m3((const float *)x->ptr, (uint8_t *)xq->ptr, (float *)scale->ptr, (float *)am.ptr, numel,
                            ctx->stream);
    return after_launch(ctx, "quantize_tensor_e4m3");
}

fa_status fa_gemm_e4m3(fa_context *ctx, const fa_buffer *aq, const fa_buffer *a_scale, uint64_t m, const fa_qweight *qw,
                       fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_qw(ctx, qw, FA_QW_E4M3_TENSOR, "gemm_e4m3: weight")) return s;
    if (qw->k != qw->k_pad) return fail(FA_ERR_UNSUPPORTED, "gemm_e4m3: k must be a multiple of 128");
    uint64_t mk, mn;
    if (!mul3(m, qw->k, &mk) || !mul3(m, qw->n, &mn)) return fail(FA_ERR_SHAPE_MISMATCH, "gemm_e4m3: shape overflows");
    if (fa_status s = check_buf_typed(ctx, aq, FA_E4M3, mk, "gemm_e4m3: aq")) return s;
    if (fa_status s = check_buf_typed(ctx, a_scale, FA_F32, 1, "gemm_e4m3: a_scale")) return s;
    if (fa_status s = check_out_f32_or_bf16(ctx, out, mn, "gemm_e4m3: out")) return s;
    if (mn == 0) return FA_OK;
    if (m > (1ull << 22)) return fail(FA_ERR_INVALID_ARGUMENT, "gemm_e4m3: m too large for one launch");
    k::gemm_e4m3_mfma((const uint8_t *)aq->ptr, (const uint8_t *)qw->codes->ptr, (const float *)a_scale->ptr,
                      (const float *)qw->scales->ptr, m, qw->n, qw->n_pad, qw->k_pad, out->ptr, out->dtype == FA_BF16,
                      ctx->props.multiProcessorCount, ctx->stream);
    return after_launch(ctx, "gemm_e4m3_mfma");
}

fa_status fa_quantize_rows_e4m3(fa_context *ctx, const fa_buffer *x, uint64_t m, uint64_t kdim, fa_buffer *xq,
                                fa_buffer *sx) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t mk;
    if (!mul3(m, kdim, &mk)) return fail(FA_ERR_SHAPE_MISMATCH, "quantize_rows_e4m3: shape overflows");
    if (fa_status s = check_buf(ctx, x, "quantize_rows_e4m3: x")) return s;
    if (x->dtype != FA_F32 && x->dtype != FA_BF16) return fail(FA_ERR_INVALID_ARGUMENT, "quantize_rows_e4m3: x must be f32 or bf16");
    if (x->numel < mk) return fail(FA_ERR_SHAPE_MISMATCH, "quantize_rows_e4m3: x is smaller than [m, k]");
    if (fa_status s = check_buf_typed(ctx, xq, FA_E4M3, mk, "quantize_rows_e4m3: xq")) return s;
    if (fa_status s = check_buf_typed(ctx, sx, FA_F32, m, "quantize_rows_e4m3: sx")) return s;
    if (mk == 0) return FA_OK;
    if (m > (1ull << 31) - 1) return fail(FA_ERR_INVALID_ARGUMENT, "quantize_rows_e4m3: too many rows");
    k::quantize_rows_e4m3(x->ptr, x->dtype == FA_BF16, (uint8_t *)xq->ptr, (float *)sx->ptr, m, kdim, kdim, ctx->stream);
    return after_launch(ctx, "quantize_rows_e4m3");
}

// shared tail of the two per-token x per-channel fp8 entry points: aq row-major e4m3 [m, k_pad]
static fa_status launch_e4m3_rows(fa_context *ctx, const uint8_t *aq, const float *sx, uint64_t m, const fa_qweight *qw,
                                  const fa_buffer *bias, uint64_t bias_offset, fa_buffer *out) {
    const float *bp = bias ? (const float *)bias->ptr + bias_offset : nullptr;
    if (m <= 64)
        k::linear_e4m3_skinny(aq, (const uint8_t *)qw->codes->ptr, sx, (const float *)qw->scales->ptr, bp, m, qw->n, qw->n_pad,
                              qw->k_pad, out->ptr, out->dtype == FA_BF16, ctx->stream);
    else
        k::gemm_e4m3_rows_mfma(aq, (const uint8_t *)qw->codes->ptr, sx, (const float *)qw->scales->ptr, bp, m, qw->n,
                               qw->n_pad, qw->k_pad, out->ptr, out->dtype == FA_BF16, ctx->props.multiProcessorCount,
                               ctx->stream);
    return after_launch(ctx, "linear_e4m3");
}

fa_status fa_gemm_e4m3_rows(fa_context *ctx, const fa_buffer *aq, const fa_buffer *sx, uint64_t m, const fa_qweight *qw,
                            const fa_buffer *bias, uint64_t bias_offset, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_qw(ctx, qw, FA_QW_E4M3_CHANNEL, "gemm_e4m3_rows: weight")) return s;
    if (qw->k != qw->k_pad) return fail(FA_ERR_UNSUPPORTED, "gemm_e4m3_rows: k must be a multiple of 128");
    uint64_t mk, mn;
    if (!mul3(m, qw->k, &mk) || !mul3(m, qw->n, &mn)) return fail(FA_ERR_SHAPE_MISMATCH, "gemm_e4m3_rows: shape overflows");
    if (fa_status s = check_buf_typed(ctx, aq, FA_E4M3, mk, "gemm_e4m3_rows: aq")) return s;
    if (fa_status s = check_buf_typed(ctx, sx, FA_F32, m, "gemm_e4m3_rows: sx")) return s;
    if (bias)
        if (fa_status s = check_view(ctx, bias, bias_offset, qw->n, FA_F32, "gemm_e4m3_rows: bias")) return s;
    if (fa_status s = check_out_f32_or_bf16(ctx, out, mn, "gemm_e4m3_rows: out")) return s;
    if (mn == 0) return FA_OK;
    if (m > (1ull << 22)) return fail(FA_ERR_INVALID_ARGUMENT, "gemm_e4m3_rows: m too large for one launch");
    return launch_e4m3_rows(ctx, (const uint8_t *)aq->ptr, (const float *)sx->ptr, m, qw, bias, bias_offset, out);
}

fa_status fa_linear_e4m3(fa_context *ctx, const fa_buffer *x, uint64_t m, const fa_qweight *qw, const fa_buffer *bias,
                         uint64_t bias_offset, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_qw(ctx, qw, FA_QW_E4M3_CHANNEL, "linear_e4m3: weight")) return s;
    uint64_t mk, mn, mkp;
    if (!mul3(m, qw->k, &mk) || !mul3(m, qw->n, &mn) || !mul3(m, qw->k_pad, &mkp))
        return fail(FA_ERR_SHAPE_MISMATCH, "linear_e4m3: shape overflows");
    if (fa_status s = check_buf(ctx, x, "linear_e4m3: x")) return s;
    if (x->dtype != FA_F32 && x->dtype != FA_BF16) return fail(FA_ERR_INVALID_ARGUMENT, "linear_e4m3: x must be f32 or bf16");
    if (x->numel != mk) return fail(FA_ERR_SHAPE_MISMATCH, "linear_e4m3: x is not [m, k]");
    if (bias)
        if (fa_status s = check_view(ctx, bias, bias_offset, qw->n, FA_F32, "linear_e4m3: bias")) return s;
    if (fa_status s = check_out_f32_or_bf16(ctx, out, mn, "linear_e4m3: out")) return s;
    if (mn == 0) return FA_OK;
    if (m > (1ull << 22)) return fail(FA_ERR_INVALID_ARGUMENT, "linear_e4m3: m too large for one launch");
    Scratch sx(ctx), xq(ctx);
    if (fa_status s = sx.get(m * 4)) return s;
    if (fa_status s = xq.get(mkp)) return s;
    // rows padded to the weight's k tiles with zero codes, so that any k is accepted
    k::quantize_rows_e4m3(x->ptr, x->dtype == FA_BF16, (uint8_t *)xq.ptr, (float *)sx.ptr, m, qw->k, qw->k_pad, ctx->stream);
    return launch_e4m3_rows(ctx, (const uint8_t *)xq.ptr, (const float *)sx.ptr, m, qw, bias, bias_offset, out);
}

// ------------------------------------------------------------------ norms
fa_status fa_rmsnorm(fa_context *ctx, const fa_buffer *x, const fa_buffer *w, float eps, uint64_t rows, uint64_t hidden,
                     fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    // crates/backend-cpu/src/rmsnorm.rs:90-120 (validate_rmsnorm_launch)
    if (!std::isfinite(eps) || eps < 0.0f) return fail(FA_ERR_INVALID_ARGUMENT, "rmsnorm: eps must be finite and non-negative");
    uint64_t numel;
    if (!mul3(rows, hidden, &numel)) return fail(FA_ERR_SHAPE_MISMATCH, "rmsnorm: rows * hidden overflows");
    if (fa_status s = check_buf_typed(ctx, x, FA_F32, numel, "rmsnorm: x")) return s;
    if (x->numel != numel) return fail(FA_ERR_SHAPE_MISMATCH, "rmsnorm: x length does not equal rows * hidden");
    if (w) {
        if (fa_status s = check_buf_typed(ctx, w, FA_F32, 0, "rmsnorm: weight")) return s;
        if (w->numel != hidden) return fail(FA_ERR_SHAPE_MISMATCH, "rmsnorm: weight length does not equal hidden");
    }
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, numel, "rmsnorm: out")) return s;
    if (numel == 0) return FA_OK;
    if (rows > (1ull << 31) - 1) return fail(FA_ERR_INVALID_ARGUMENT, "rmsnorm: too many rows");
    k::rmsnorm_f32((const float *)x->ptr, w ? (const float *)w->ptr : nullptr, (float *)out->ptr, rows, hidden, eps,
                   ctx->stream);
    return after_launch(ctx, "rmsnorm_f32");
}

fa_status fa_rope(fa_context *ctx, const fa_buffer *x, const fa_buffer *positions, uint64_t rows, uint64_t heads,
                  uint64_t head_dim, double theta, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (head_dim % 2 != 0) return fail(FA_ERR_INVALID_ARGUMENT, "rope: head_dim must be even");
    if (!(theta > 0.0) || !std::isfinite(theta)) return fail(FA_ERR_INVALID_ARGUMENT, "rope: theta must be positive and finite");
    uint64_t numel;
    if (!mul3(rows, heads, &numel) || !mul3(numel, head_dim, &numel)) return fail(FA_ERR_SHAPE_MISMATCH, "rope: shape overflows");
    if (fa_status s = check_buf_typed(ctx, x, FA_F32, numel, "rope: x")) return s;
    if (fa_status s = check_buf_typed(ctx, positions, FA_I32, rows, "rope: positions")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, numel, "rope: out")) return s;
    if (numel == 0) return FA_OK;
    if (rows > (1ull << 31) - 1 || heads > UINT32_MAX || head_dim > UINT32_MAX)
        return fail(FA_ERR_INVALID_ARGUMENT, "rope: dimension too large");
    k::rope_f32((const float *)x->ptr, (const int32_t *)positions->ptr, (float *)out->ptr, rows, heads, head_dim, theta,
                ctx->stream);
    return after_launch(ctx, "rope_f32");
}

// ------------------------------------------------------------ elementwise
fa_status fa_silu_mul(fa_context *ctx, const fa_buffer *gate, const fa_buffer *up, uint64_t numel, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf_typed(ctx, gate, FA_F32, numel, "silu_mul: gate")) return s;
    if (fa_status s = check_buf_typed(ctx, up, FA_F32, numel, "silu_mul: up")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, numel, "silu_mul: out")) return s;
    k::silu_mul_f32((const float *)gate->ptr, (const float *)up->ptr, (float *)out->ptr, numel, ctx->stream);
    return after_launch(ctx, "silu_mul_f32");
}

fa_status fa_add(fa_context *ctx, const fa_buffer *a, const fa_buffer *b, uint64_t numel, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf_typed(ctx, a, FA_F32, numel, "add: a")) return s;
    if (fa_status s = check_buf_typed(ctx, b, FA_F32, numel, "add: b")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, numel, "add: out")) return s;
    k::add_f32((const float *)a->ptr, (const float *)b->ptr, (float *)out->ptr, numel, ctx->stream);
    return after_launch(ctx, "add_f32");
}

fa_status fa_argmax_rows(fa_context *ctx, const fa_buffer *x, uint64_t rows, uint64_t cols, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t numel;
    if (!mul3(rows, cols, &numel)) return fail(FA_ERR_SHAPE_MISMATCH, "argmax_rows: shape overflows");
    if (cols == 0 && rows != 0) return fail(FA_ERR_INVALID_ARGUMENT, "argmax_rows: empty reduction axis");
    if (cols > (uint64_t)INT32_MAX) return fail(FA_ERR_INVALID_ARGUMENT, "argmax_rows: index does not fit i32");
    if (fa_status s = check_buf_typed(ctx, x, FA_F32, numel, "argmax_rows: x")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_I32, rows, "argmax_rows: out")) return s;
    if (rows == 0) return FA_OK;
    if (rows > (1ull << 31) - 1) return fail(FA_ERR_INVALID_ARGUMENT, "argmax_rows: too many rows");
    k::argmax_rows_f32((const float *)x->ptr, (int32_t *)out->ptr, rows, cols, ctx->stream);
    return after_launch(ctx, "argmax_rows_f32");
}

fa_status fa_gather_rows(fa_context *ctx, const fa_buffer *table, uint64_t table_rows, uint64_t cols,
                         const fa_buffer *idx, uint64_t rows, fa_buffer *out) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t tn, on;
    if (!mul3(table_rows, cols, &tn) || !mul3(rows, cols, &on)) return fail(FA_ERR_SHAPE_MISMATCH, "gather_rows: shape overflows");
    if (fa_status s = check_buf_typed(ctx, table, FA_F32, tn, "gather_rows: table")) return s;
    if (fa_status s = check_buf_typed(ctx, idx, FA_I32, rows, "gather_rows: idx")) return s;
    if (fa_status s = check_buf_typed(ctx, out, FA_F32, on, "gather_rows: out")) return s;
    if (on == 0) return FA_OK;
    if (rows > (1ull << 31) - 1) return fail(FA_ERR_INVALID_ARGUMENT, "gather_rows: too many rows");
    k::gather_rows_f32((const float *)table->ptr, table_rows, cols, (const int32_t *)idx->ptr, (float *)out->ptr, rows,
                       ctx->stream);
    return after_launch(ctx, "gather_rows_f32");
}

fa_status fa_fill_normal(fa_context *ctx, fa_buffer *buf, uint64_t offset, uint64_t numel, uint64_t seed, float mean,
                         float std) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, buf, "fill_normal: buf")) return s;
    if (buf->dtype != FA_F32 && buf->dtype != FA_BF16) return fail(FA_ERR_INVALID_ARGUMENT, "fill_normal: f32 or bf16 only");
    uint64_t end;
    if (__builtin_add_overflow(offset, numel, &end) || end > buf->numel)
        return fail(FA_ERR_INVALID_ARGUMENT, "fill_normal: range exceeds the buffer");
    if (offset % 2 != 0) return fail(FA_ERR_INVALID_ARGUMENT, "fill_normal: offset must be even");
    k::fill_normal((char *)buf->ptr + offset * dtype_size(buf->dtype), buf->dtype == FA_BF16, numel, seed, mean, std,
                   ctx->stream);
    return after_launch(ctx, "fill_normal");
}

static fa_status check_sampling(fa_sampling strategy, float temperature, uint64_t top_k, uint64_t vocab) {
    // GenerateConfig::validate (crates/autodiff/src/generate/mod.rs:170-215)
    if (strategy != FA_SAMPLE_GREEDY && strategy != FA_SAMPLE_TEMPERATURE && strategy != FA_SAMPLE_TOP_K)
        return fail(FA_ERR_INVALID_ARGUMENT, "sampling: unknown strategy");
    if (strategy != FA_SAMPLE_GREEDY && !(std::isfinite(temperature) && temperature > 0.0f))
        return fail(FA_ERR_INVALID_ARGUMENT, "sampling: temperature must be finite and positive");
    if (strategy == FA_SAMPLE_TOP_K && (top_k == 0 || top_k > vocab))
        return fail(FA_ERR_INVALID_ARGUMENT, "sampling: top_k must be in 1..=vocab");
    return FA_OK;
}

fa_status fa_sample_rows(fa_context *ctx, const fa_buffer *logits, uint64_t rows, uint64_t vocab, fa_sampling strategy,
                         float temperature, uint64_t top_k, fa_buffer *rng, fa_buffer *tokens) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t numel;
    if (!mul3(rows, vocab, &numel)) return fail(FA_ERR_SHAPE_MISMATCH, "sample_rows: shape overflows");
    if (fa_status s = check_buf_typed(ctx, logits, FA_F32, numel, "sample_rows: logits")) return s;
    if (fa_status s = check_buf_typed(ctx, tokens, FA_I32, rows, "sample_rows: tokens")) return s;
    if (vocab == 0 || vocab > (uint64_t)INT32_MAX) return fail(FA_ERR_INVALID_ARGUMENT, "sample_rows: vocab must be in 1..=i32::MAX");
    if (rows > 65535) return fail(FA_ERR_INVALID_ARGUMENT, "sample_rows: at most 65535 rows per call");
    if (fa_status s = check_sampling(strategy, temperature, top_k, vocab)) return s;
    if (rows == 0) return FA_OK;
    if (strategy == FA_SAMPLE_GREEDY) {
        k::argmax_rows_f32((const float *)logits->ptr, (int32_t *)tokens->ptr, rows, vocab, ctx->stream);
        return after_launch(ctx, "argmax_rows");
    }
    if (fa_status s = check_buf_typed(ctx, rng, FA_U32, 2, "sample_rows: rng")) return s;
    k::sample_rows((const float *)logits->ptr, (int32_t *)tokens->ptr, (uint64_t *)rng->ptr, (uint32_t)rows, (uint32_t)vocab,
                   strategy == FA_SAMPLE_TOP_K, temperature, (uint32_t)top_k, ctx->stream);
    return after_launch(ctx, "sample_rows");
}

fa_status fa_sampling_weights(fa_context *ctx, const fa_buffer *logits, uint64_t logits_offset, uint64_t rows, uint64_t vocab,
                              fa_sampling strategy, float temperature, uint64_t top_k, fa_buffer *weights,
                              uint64_t weights_offset, fa_buffer *status) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t numel, end;
    if (!mul3(rows, vocab, &numel) || __builtin_add_overflow(numel, logits_offset, &end))
        return fail(FA_ERR_SHAPE_MISMATCH, "sampling_weights: shape overflows");
    if (fa_status s = check_buf_typed(ctx, logits, FA_F32, end, "sampling_weights: logits")) return s;
    if (__builtin_add_overflow(numel, weights_offset, &end)) return fail(FA_ERR_SHAPE_MISMATCH, "sampling_weights: shape overflows");
    if (fa_status s = check_buf_typed(ctx, weights, FA_F32, end, "sampling_weights: weights")) return s;
    if (fa_status s = check_buf_typed(ctx, status, FA_I32, rows, "sampling_weights: status")) return s;
    if (vocab == 0 || vocab > (uint64_t)INT32_MAX)
        return fail(FA_ERR_INVALID_ARGUMENT, "sampling_weights: vocab must be in 1..=i32::MAX");
    if (rows > 65535) return fail(FA_ERR_INVALID_ARGUMENT, "sampling_weights: at most 65535 rows per call");
    if (fa_status s = check_sampling(strategy, temperature, top_k, vocab)) return s;
    if (rows == 0) return FA_OK;
    const int mode = strategy == FA_SAMPLE_GREEDY ? 2 : (strategy == FA_SAMPLE_TOP_K ? 1 : 0);
    k::sampling_weights((const float *)logits->ptr + logits_offset, (float *)weights->ptr + weights_offset, (int32_t *)status->ptr,
                        (uint32_t)rows, (uint32_t)vocab, mode, temperature, (uint32_t)top_k, ctx->stream);
    return after_launch(ctx, "sampling_weights");
}

fa_status fa_speculative_accept(fa_context *ctx, const fa_buffer *p_weights, uint64_t p_offset, const fa_buffer *q_weights,
                                uint64_t q_offset, const int32_t *drafts, uint64_t k, uint64_t vocab, fa_buffer *rng,
                                fa_buffer *result) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (k > k::kMaxDraftTokens) return fail(FA_ERR_INVALID_ARGUMENT, "speculative_accept: at most 32 draft tokens per call");
    if (vocab == 0 || vocab > (uint64_t)INT32_MAX)
        return fail(FA_ERR_INVALID_ARGUMENT, "speculative_accept: vocab must be in 1..=i32::MAX");
    uint64_t numel, end;
    if (!mul3(k + 1, vocab, &numel) || __builtin_add_overflow(numel, p_offset, &end))
        return fail(FA_ERR_SHAPE_MISMATCH, "speculative_accept: shape overflows");
    if (fa_status s = check_buf_typed(ctx, p_weights, FA_F32, end, "speculative_accept: p_weights")) return s;
    k::DraftTokens d{};
    if (k > 0) {
        if (!drafts) return fail(FA_ERR_INVALID_ARGUMENT, "speculative_accept: null drafts");
        if (!mul3(k, vocab, &numel) || __builtin_add_overflow(numel, q_offset, &end))
            return fail(FA_ERR_SHAPE_MISMATCH, "speculative_accept: shape overflows");
        if (fa_status s = check_buf_typed(ctx, q_weights, FA_F32, end, "speculative_accept: q_weights")) return s;
        for (uint64_t i = 0; i < k; ++i) {
            if (drafts[i] < 0 || (uint64_t)drafts[i] >= vocab)
                return fail(FA_ERR_INVALID_ARGUMENT, "speculative_accept: draft " + std::to_string(i) + " (" +
                                                         std::to_string(drafts[i]) + ") is outside the vocabulary");
            d.d[i] = drafts[i];
        }
    }
    if (fa_status s = check_buf_typed(ctx, rng, FA_U32, 2, "speculative_accept: rng")) return s;
    if (fa_status s = check_buf_typed(ctx, result, FA_I32, 4, "speculative_accept: result")) return s;
    k::speculative_accept((const float *)p_weights->ptr + p_offset, k ? (const float *)q_weights->ptr + q_offset : nullptr, d,
                          (uint32_t)k, (uint32_t)vocab, (uint64_t *)rng->ptr, (int32_t *)result->ptr, ctx->stream);
    return after_launch(ctx, "speculative_accept");
}

fa_status fa_rng_seed(fa_context *ctx, fa_buffer *rng, uint64_t seed) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf_typed(ctx, rng, FA_U32, 2, "rng_seed: rng")) return s;
    uint64_t state;
    (void)fa_rng_state_from_seed(seed, &state);
    const uint32_t words[2] = {(uint32_t)state, (uint32_t)(state >> 32)};
    return fa_upload_into(ctx, words, 2, rng, 0);
}

fa_status fa_rng_state_from_seed(uint64_t seed, uint64_t *state) {
    if (!state) return fail(FA_ERR_INVALID_ARGUMENT, "rng_state_from_seed: null state");
    *state = seed == 0 ? 0x9E3779B97F4A7C15ull : seed;
    return FA_OK;
}

fa_status fa_sample_rows_per_row(fa_context *ctx, const fa_buffer *logits, uint64_t rows, uint64_t vocab, fa_buffer *table,
                                 fa_buffer *tokens) {
    if (fa_status s = check_ctx(ctx)) return s;
    uint64_t numel;
    if (!mul3(rows, vocab, &numel)) return fail(FA_ERR_SHAPE_MISMATCH, "sample_rows_per_row: shape overflows");
    if (fa_status s = check_buf_typed(ctx, logits, FA_F32, numel, "sample_rows_per_row: logits")) return s;
    if (fa_status s = check_buf_typed(ctx, tokens, FA_I32, rows, "sample_rows_per_row: tokens")) return s;
    if (vocab == 0 || vocab > (uint64_t)INT32_MAX)
        return fail(FA_ERR_INVALID_ARGUMENT, "sample_rows_per_row: vocab must be in 1..=i32::MAX");
    if (rows > 65535) return fail(FA_ERR_INVALID_ARGUMENT, "sample_rows_per_row: at most 65535 rows per call");
    if (fa_status s = check_buf_typed(ctx, table, FA_U32, rows * 6, "sample_rows_per_row: table")) return s;
    if (rows == 0) return FA_OK;
    k::sample_rows_policy((const float *)logits->ptr, (int32_t *)tokens->ptr, (k::RowPolicy *)table->ptr, (uint32_t)rows,
                          (uint32_t)vocab, ctx->stream);
    return after_launch(ctx, "sample_rows_per_row");
}

fa_status fa_probe_matrix_rate(fa_context *ctx, int32_t kind, const fa_buffer *operands, uint32_t iters, fa_buffer *sink,
                               double *ops) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, operands, "probe_matrix_rate: operands")) return s;
    if (fa_status s = check_buf(ctx, sink, "probe_matrix_rate: sink")) return s;
    if (kind < 0 || kind > 2) return fail(FA_ERR_INVALID_ARGUMENT, "probe_matrix_rate: kind is 0, 1 or 2");
    if (operands->numel * dtype_size(operands->dtype) < 65536)
        return fail(FA_ERR_SHAPE_MISMATCH, "probe_matrix_rate: operands must hold 64 KiB");
    if (sink->numel * dtype_size(sink->dtype) < 4) return fail(FA_ERR_SHAPE_MISMATCH, "probe_matrix_rate: sink too small");
    if (!ops) return fail(FA_ERR_INVALID_ARGUMENT, "probe_matrix_rate: null ops");
    *ops = k::matrix_rate_probe(kind, operands->ptr, iters, ctx->props.multiProcessorCount, (int *)sink->ptr, ctx->stream);
    return after_launch(ctx, "matrix_rate_probe");
}

fa_status fa_probe_stream_read(fa_context *ctx, const fa_buffer *src, uint64_t offset_bytes, uint64_t bytes, int32_t blocks,
                               int32_t threads, fa_buffer *sink) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, src, "probe_stream_read: src")) return s;
    if (fa_status s = check_buf(ctx, sink, "probe_stream_read: sink")) return s;
    if (blocks <= 0 || blocks > 65536 || (threads != 256 && threads != 512))
        return fail(FA_ERR_INVALID_ARGUMENT, "probe_stream_read: blocks in 1..=65536, threads 256 or 512");
    const uint64_t have = src->numel * dtype_size(src->dtype);
    uint64_t end;
    if (offset_bytes % 16 != 0 || __builtin_add_overflow(offset_bytes, bytes, &end) || end > have)
        return fail(FA_ERR_INVALID_ARGUMENT, "probe_stream_read: range exceeds the buffer or is not 16-byte aligned");
    if (sink->numel * dtype_size(sink->dtype) < 4) return fail(FA_ERR_SHAPE_MISMATCH, "probe_stream_read: sink too small");
    if (bytes < 16ull * (uint64_t)blocks) return FA_OK;
    k::stream_read_probe((const char *)src->ptr + offset_bytes, bytes, blocks, threads, (int *)sink->ptr, ctx->stream);
    return after_launch(ctx, "stream_read_probe");
}

fa_status fa_probe_l2_path(fa_context *ctx, const fa_buffer *cold, uint64_t cold_offset_bytes, uint64_t cold_bytes,
                           const fa_buffer *hot, uint32_t hot_bytes, uint32_t hot_passes, int32_t in_flight,
                           int32_t hot_per_cold, int32_t blocks, int32_t threads, fa_buffer *sink) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, cold, "probe_l2_path: cold")) return s;
    if (fa_status s = check_buf(ctx, hot, "probe_l2_path: hot")) return s;
    if (fa_status s = check_buf(ctx, sink, "probe_l2_path: sink")) return s;
    if (blocks <= 0 || blocks > 65536 || threads < 64 || threads > 512 || threads % 64 != 0)
        return fail(FA_ERR_INVALID_ARGUMENT, "probe_l2_path: blocks in 1..=65536, threads a multiple of 64 up to 512");
    const uint64_t have = cold->numel * dtype_size(cold->dtype);
    uint64_t end;
    if (cold_offset_bytes % 16 != 0 || __builtin_add_overflow(cold_offset_bytes, cold_bytes, &end) || end > have)
        return fail(FA_ERR_INVALID_ARGUMENT, "probe_l2_path: cold range exceeds the buffer or is not 16-byte aligned");
    if (hot_bytes < 16u * 512u || hot_bytes % 16 != 0 || hot_bytes > hot->numel * dtype_size(hot->dtype))
        return fail(FA_ERR_INVALID_ARGUMENT, "probe_l2_path: hot region must hold 8 KiB .. its buffer, a multiple of 16 bytes");
    if (sink->numel * dtype_size(sink->dtype) < 4) return fail(FA_ERR_SHAPE_MISMATCH, "probe_l2_path: sink too small");
    if (cold_bytes == 0 && hot_passes == 0) return FA_OK;
    if (cold_bytes != 0 && cold_bytes < 16ull * (uint64_t)blocks) return FA_OK;
    if (!k::l2_path_probe((const char *)cold->ptr + cold_offset_bytes, cold_bytes, hot->ptr, hot_bytes, hot_passes, in_flight,
                          hot_per_cold, blocks, threads, (int *)sink->ptr, ctx->stream))
        return fail(FA_ERR_INVALID_ARGUMENT, "probe_l2_path: in_flight must be 8 or 16 and hot_per_cold 0 or 2");
    return after_launch(ctx, "l2_path_probe");
}

fa_status fa_convert(fa_context *ctx, const fa_buffer *src, uint64_t numel, fa_buffer *dst) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, src, "convert: src")) return s;
    if (fa_status s = check_buf(ctx, dst, "convert: dst")) return s;
    if (src->numel < numel || dst->numel < numel) return fail(FA_ERR_SHAPE_MISMATCH, "convert: buffer too small");
    if (src->dtype == FA_F32 && dst->dtype == FA_BF16)
        k::convert_f32_to_bf16((const float *)src->ptr, (uint16_t *)dst->ptr, numel, ctx->stream);
    else if (src->dtype == FA_BF16 && dst->dtype == FA_F32)
        k::convert_bf16_to_f32((const uint16_t *)src->ptr, (float *)dst->ptr, numel, ctx->stream);
    else
        return fail(FA_ERR_UNSUPPORTED, "convert: only f32 <-> bf16");
    return after_launch(ctx, "convert");
}

}  // extern "C"
