// One decode step of a Llama-style decoder on resident state: the
// composition of the quantized linears, RMSNorm, RoPE, paged attention and
// greedy argmax that the benchmark's full-step configuration names.  All
// buffers are allocated when the decoder is created; a step only enqueues
// kernels, so it can be captured once into a HIP graph and replayed.
#include <map>
#include <algorithm>
#include <cmath>
#include <exception>
#include <new>
#include <string>
#include <vector>

#include "kernels.hpp"
#include "runtime.hpp"
#include "validate.hpp"

using namespace fa;

namespace fa {
extern int g_decode_waves;
int g_prefill_rows = 0;      // rows per chunk of a prompt pass (tuning key 25; below 256: the built-in figure)
int g_prefill_fused_rows = 0;   // prompt passes of at most 64 rows: 0 the decode step's fused projections, 1 plain ones (tuning key 26)
namespace k {
extern int g_weight_prefetch;
}
}

struct fa_decoder {
    uint32_t magic;
    fa_context *ctx;
    fa_decoder_config cfg;
    struct Layer {
        const fa_buffer *attn_norm = nullptr, *ffn_norm = nullptr;
        const fa_qweight *wqkv = nullptr, *wo = nullptr, *wgu = nullptr, *wdown = nullptr;
        fa_buffer *k_pool = nullptr, *v_pool = nullptr;
    };
    std::vector<Layer> layers;
    // The large activation buffers of a prompt pass stay with the decoder from one pass to the next (grow only, until the
    // decoder goes): the context's pool keeps at most 128 MiB of idle blocks, so buffers of hundreds of megabytes went
    // back to the driver after every pass and were allocated again for the next (1024 prompt tokens: 12.9 -> 12.3 ms,
    // 4 x 2048: 71.4 -> 69.1 ms without those calls).  At most kRows rows of them: about 1.8 GB at the benchmark's width.
    struct KeptBlock {
        void *ptr = nullptr;
        uint64_t bytes = 0, cls = 0;
    };
    static constexpr int kKept = 8;
    KeptBlock kept[kKept];
    const fa_buffer *embed = nullptr, *final_norm = nullptr;
    const fa_qweight *lm_head = nullptr;
    uint32_t batch = 0;
    // resident state and activations
    fa_buffer *tokens = nullptr, *tables = nullptr, *seq_lens = nullptr, *pos = nullptr, *slots = nullptr;
    fa_buffer *cos_sin = nullptr, *h = nullptr, *xq = nullptr, *sx = nullptr, *q_bf = nullptr;
    fa_buffer *attn = nullptr, *act = nullptr, *pmax = nullptr, *logits = nullptr;
    // captured steps, one per batch size seen (a scheduler changes the batch as requests come and go)
    std::map<uint32_t, fa_graph *> graphs;
    int graph_waves = 0;
    // how the step and the prompt pass pick the next token; rng holds the generator state on the device
    fa_sampling strategy = FA_SAMPLE_GREEDY;
    float temperature = 1.0f;
    uint32_t top_k = 0;
    fa_buffer *rng = nullptr;
    // per-row sampling table (k::RowPolicy per row) and whether the pick uses it
    fa_buffer *policy = nullptr;
    bool per_row = false;
    // host mirror of the installed block tables and of the sequence lengths (advanced with every step and
    // prompt chunk), used to validate that a prompt fits before anything is queued
    std::vector<uint32_t> host_tables, host_lens;
};

namespace {

constexpr uint32_t kDecMagic = 0xFA0DEC01u;

uint64_t round_up(uint64_t v, uint64_t to) { return (v + to - 1) / to * to; }

void drop_graphs(fa_decoder *d) {
    for (auto &g : d->graphs) fa_graph_destroy(d->ctx, g.second);
    d->graphs.clear();
}

fa_status check_dec(const fa_decoder *d) {
    if (!d || d->magic != kDecMagic) return fail(FA_ERR_INVALID_ARGUMENT, "decoder: not a decoder");
    return FA_OK;
}

fa_status check_weight(const fa_decoder *d, const fa_qweight *qw, uint64_t k, uint64_t n, const char *what) {
    if (!qw || qw->magic != kQwMagic) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": not a quantized weight");
    if (qw->ctx != d->ctx) return fail(FA_ERR_DEVICE_MISMATCH, std::string(what) + ": weight belongs to another context");
    if (qw->kind != FA_QW_INT8_CHANNEL) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": must be an int8 weight");
    if (qw->k != k || qw->n != n)
        return fail(FA_ERR_SHAPE_MISMATCH, std::string(what) + ": expected [" + std::to_string(k) + ", " +
                                               std::to_string(n) + "], got [" + std::to_string(qw->k) + ", " +
                                               std::to_string(qw->n) + "]");
    return FA_OK;
}

fa_status check_vec(const fa_decoder *d, const fa_buffer *b, uint64_t numel, const char *what) {
    if (fa_status s = check_buf_typed(d->ctx, b, FA_F32, numel, what)) return s;
    if (b->numel != numel) return fail(FA_ERR_SHAPE_MISMATCH, std::string(what) + ": wrong length");
    return FA_OK;
}

void free_all(fa_context *ctx, fa_decoder *d) {
    for (auto &kb : d->kept) {
        if (kb.ptr) pool_free(ctx, kb.ptr, kb.bytes, kb.cls);
        kb = fa_decoder::KeptBlock{};
    }
    fa_buffer **bufs[] = {&d->tokens, &d->tables, &d->seq_lens, &d->pos, &d->slots, &d->cos_sin, &d->h, &d->xq,
                          &d->sx,     &d->q_bf,     &d->attn, &d->act,  &d->pmax, &d->logits, &d->rng, &d->policy};
    for (auto pb : bufs) {
        if (*pb) fa_buffer_free(ctx, *pb);
        *pb = nullptr;
    }
    for (auto &l : d->layers) {
        if (l.k_pool) fa_buffer_free(ctx, l.k_pool);
        if (l.v_pool) fa_buffer_free(ctx, l.v_pool);
        l.k_pool = l.v_pool = nullptr;
    }
}

// logits [batch, vocab] -> next tokens, by the decoder's sampling strategy
void enqueue_pick(fa_decoder *d, hipStream_t s) {
    if (d->per_row)
        k::sample_rows_policy((const float *)d->logits->ptr, (int32_t *)d->tokens->ptr, (k::RowPolicy *)d->policy->ptr,
                              d->batch, d->cfg.vocab, s);
    else if (d->strategy == FA_SAMPLE_GREEDY)
        k::argmax_rows_f32((const float *)d->logits->ptr, (int32_t *)d->tokens->ptr, d->batch, d->cfg.vocab, s);
    else
        k::sample_rows((const float *)d->logits->ptr, (int32_t *)d->tokens->ptr, (uint64_t *)d->rng->ptr, d->batch,
                       d->cfg.vocab, d->strategy == FA_SAMPLE_TOP_K, d->temperature, d->top_k, s);
}

// Whether the step about to be enqueued (the host lengths already count its token) sees only short contexts: its
// attention then takes the one-launch form, and the recorded graphs of the two kinds are kept apart.
// With at most one block (sequence x kv head) per compute unit: a scheduler's batch of up to a few dozen short
// conversations, whose few pages the streamed form would cut into ranges of a dozen, leaving partial results and a
// merge launch (measured through 32 layers at 4 .. 32 rows and contexts up to 1000: 2 - 14 % of the step; from 36 rows
// on, with more blocks than compute units and their unequal lengths, the streamed form is the faster one).
bool step_is_short(const fa_decoder *d) {
    if (k::g_decode_one == 1) return false;
    uint32_t longest = 0;
    for (uint32_t b = 0; b < d->batch && b < d->host_lens.size(); ++b) longest = std::max(longest, d->host_lens[b]);
    if (d->batch == 0 || longest > k::kDecodeOneMaxCtx) return false;
    const uint64_t blocks = (uint64_t)d->batch * d->cfg.n_kv_heads;
    return k::g_decode_one == 2 || blocks <= (uint64_t)d->ctx->props.multiProcessorCount;
}

// The kernels of one step, enqueued on the context's stream.  stop_after (test aid, -1 in normal use) ends the
// step after the given stage: stage 0 is the per-step bookkeeping and the embedding gather, stage
// 1 + 8 * layer + i (i = 0 .. 7) is the i-th launch of that layer (norm + quantizer, qkv projection with RoPE
// and cache append, attention with merge + quantizer, o projection, norm + quantizer, gate / up with SwiGLU,
// quantizer, down projection), and the three stages after the last layer are the final norm, the head and the pick.
fa_status enqueue_step(fa_context *ctx, fa_decoder *d, int stop_after = -1) {
    const fa_decoder_config &c = d->cfg;
    const uint32_t B = d->batch;
    const uint64_t D = c.d_model, H = c.n_heads, HKV = c.n_kv_heads, DH = c.head_dim, F = c.d_ffn, V = c.vocab;
    const uint64_t EQ = H * DH, EKV = HKV * DH;
    const uint64_t m_pad = round_up(B, 16);
    const int cus = ctx->props.multiProcessorCount;
    hipStream_t s = ctx->stream;
    const uint64_t pool_rows = (uint64_t)c.num_blocks * c.block_size;

    k::decode_prepare((const uint32_t *)d->tables->ptr, (uint32_t *)d->seq_lens->ptr, (int32_t *)d->pos->ptr,
                      (uint32_t *)d->slots->ptr, (float *)d->cos_sin->ptr, B, c.block_size, c.max_blocks_per_seq,
                      c.num_blocks, c.head_dim, c.rope_theta, s);
    k::gather_rows_f32((const float *)d->embed->ptr, V, D, (const int32_t *)d->tokens->ptr, (float *)d->h->ptr, B, s);
    int stage = 0;
    auto stop_here = [&]() { return stop_after >= 0 && stage++ == stop_after; };
    const bool short_ctx = step_is_short(d);
    if (stop_here()) return after_launch(ctx, "decoder step (partial)");

    k::PagedShape ps;
    ps.num_blocks = c.num_blocks;
    ps.block_size = c.block_size;
    ps.e_kv = (uint32_t)EKV;
    ps.batch = B;
    ps.l_new = 1;
    ps.num_heads = c.n_heads;
    ps.num_kv_heads = c.n_kv_heads;
    ps.head_dim = c.head_dim;
    ps.max_blocks_per_seq = c.max_blocks_per_seq;
    ps.scale = 1.0f / std::sqrt((float)c.head_dim);

    auto epilogue = [&](const fa_qweight *w, void *out, const float *residual) {
        k::EpilogueI8 ep;
        ep.sx = (const float *)d->sx->ptr;
        ep.sw = (const float *)w->scales->ptr;
        ep.bias = nullptr;
        ep.residual = residual;
        ep.acc_out = nullptr;
        ep.out = out;
        ep.out_bf16 = 0;
        return ep;
    };
    auto norm_prologue = [&](const float *norm_w) {
        k::RowPrologue pro;
        pro.x = (const float *)d->h->ptr;
        pro.norm_w = norm_w;
        pro.eps = c.rms_eps;
        pro.inv_n = 1.0f / (float)D;
        pro.xq_tiled_out = (int8_t *)d->xq->ptr;
        pro.sx_out = (float *)d->sx->ptr;
        return pro;
    };
    auto linear = [&](const fa_qweight *w, void *out, const float *residual) {
        k::linear_w8a8_skinny((const int8_t *)d->xq->ptr, (const int8_t *)w->codes->ptr, B, w->n, w->n_pad, w->k_pad,
                              epilogue(w, out, residual), cus, s, &ctx->splitk);
    };

    // The row kernels in front of the two small projections pull those projections' weights into L2 while they wait
    // on their own memory round trips (k::WeightPrefetch): all of the o projection (16.8 MB at the benchmark's width)
    // under the merge + quantizer, half of q | k | v under the norm + quantizer.  Measured in the step's kernel trace:
    // the o projection 6.7 -> 5.2 us, q | k | v 9.1 -> 8.0 us, their row kernels + 0.7 and + 0.3 us.  The same for
    // the wide projections (gate / up, down, the head) lengthens the row kernel by what the projection gains.
    const uint64_t pull_scale = k::g_weight_prefetch >= 2 ? (uint64_t)k::g_weight_prefetch : 12;
    const uint64_t kPullQkv = pull_scale << 20, kPullO = (2 * pull_scale) << 20;
    auto pull_plain = [&](const fa_qweight *w, uint64_t budget) {
        return k::prefetch_for_linear_w8a8_skinny((const int8_t *)w->codes->ptr, B, w->n_pad, w->k_pad, cus, budget, &ctx->splitk);
    };
    for (uint32_t li = 0; li < c.n_layers; ++li) {
        const fa_decoder::Layer &L = d->layers[li];
        const k::QkvRopeTargets t{(const float *)d->cos_sin->ptr, (const uint32_t *)d->slots->ptr, (uint16_t *)d->q_bf->ptr,
                                  (uint16_t *)L.k_pool->ptr, (uint16_t *)L.v_pool->ptr, c.n_heads, c.n_kv_heads,
                                  c.head_dim, pool_rows};
        // With one or two rows (by measurement; the kernels take four) the linears redo the row work in front of them
        // inside their own launch (k::RowPrologue): the row stage then launches nothing and its outputs (codes,
        // scales) appear with the linear's stage, written by one block of it.
        const bool fuse_qkv = k::qkv_rope_fuses_norm(B, L.wqkv->k_pad);
        // Short sequences: the attention finishes in one launch (a block per sequence and kv head; no
        // partial results, no merge launch) and leaves its output and the heads' maxima for the o projection, which
        // does the per-token quantizer itself when there is one row (a launch of its own otherwise).
        const bool one_form = short_ctx && c.n_heads <= 32 && F >= EQ && EQ % 64 == 0;
        const bool one_attn = one_form && k::plain_fuses_pmax_quantizer(B, L.wo->n_pad, L.wo->k_pad, cus);
        if (!fuse_qkv)
            k::rmsnorm_quantize_i8((const float *)d->h->ptr, (const float *)L.attn_norm->ptr, c.rms_eps, nullptr,
                                   (int8_t *)d->xq->ptr, (float *)d->sx->ptr, B, m_pad, D, s,
                                   k::prefetch_for_linear_w8a8_qkv_rope_skinny((const int8_t *)L.wqkv->codes->ptr, B, L.wqkv->n_pad,
                                                                               L.wqkv->k_pad, t, kPullQkv));
        if (stop_here()) break;
        {
            const k::RowPrologue pro = norm_prologue((const float *)L.attn_norm->ptr);
            k::linear_w8a8_qkv_rope_skinny((const int8_t *)d->xq->ptr, (const int8_t *)L.wqkv->codes->ptr,
                                           (const float *)d->sx->ptr, (const float *)L.wqkv->scales->ptr, B,
                                           L.wqkv->n_pad, L.wqkv->k_pad, t, s, fuse_qkv ? &pro : nullptr);
        }
        if (stop_here()) break;
        if (one_attn) {
            k::paged_attention_decode_one_bf16((const uint16_t *)d->q_bf->ptr, (const uint16_t *)L.k_pool->ptr,
                                               (const uint16_t *)L.v_pool->ptr, (const uint32_t *)d->tables->ptr,
                                               (const uint32_t *)d->seq_lens->ptr, ps, (float *)d->act->ptr,
                                               (float *)d->pmax->ptr, s);
        } else if (one_form) {
            // the same launch for more rows than the o projection quantizes for itself: the quantizer from the heads'
            // maxima is a launch of its own (the output is f32 values already rounded to bf16, the operator's output type)
            k::paged_attention_decode_one_bf16((const uint16_t *)d->q_bf->ptr, (const uint16_t *)L.k_pool->ptr,
                                               (const uint16_t *)L.v_pool->ptr, (const uint32_t *)d->tables->ptr,
                                               (const uint32_t *)d->seq_lens->ptr, ps, (float *)d->act->ptr,
                                               (float *)d->pmax->ptr, s);
            k::quantize_rows_from_pmax(d->act->ptr, false, (const float *)d->pmax->ptr, c.n_heads, (int8_t *)d->xq->ptr,
                                       (float *)d->sx->ptr, B, m_pad, EQ, s);
        } else if (c.n_heads <= 32) {
            k::paged_attention_decode_bf16((const uint16_t *)d->q_bf->ptr, (const uint16_t *)L.k_pool->ptr,
                                           (const uint16_t *)L.v_pool->ptr, (const uint32_t *)d->tables->ptr,
                                           (const uint32_t *)d->seq_lens->ptr, ps, (uint32_t)g_decode_waves, ctx->workspace,
                                           nullptr, 1, nullptr, (int8_t *)d->xq->ptr, (float *)d->sx->ptr, (uint32_t)m_pad,
                                           s, pull_plain(L.wo, kPullO));
        } else {
            k::paged_attention_decode_bf16((const uint16_t *)d->q_bf->ptr, (const uint16_t *)L.k_pool->ptr,
                                           (const uint16_t *)L.v_pool->ptr, (const uint32_t *)d->tables->ptr,
                                           (const uint32_t *)d->seq_lens->ptr, ps, (uint32_t)g_decode_waves, ctx->workspace,
                                           d->attn->ptr, 1, (float *)d->pmax->ptr, s);
            k::quantize_rows_from_pmax(d->attn->ptr, true, (const float *)d->pmax->ptr, c.n_heads, (int8_t *)d->xq->ptr,
                                       (float *)d->sx->ptr, B, m_pad, EQ, s);
        }
        if (stop_here()) break;
        if (one_attn) {
            k::RowPrologue pro;
            pro.x = (const float *)d->act->ptr;
            pro.pmax = (const float *)d->pmax->ptr;
            pro.parts = c.n_heads;
            pro.xq_tiled_out = (int8_t *)d->xq->ptr;
            pro.sx_out = (float *)d->sx->ptr;
            k::linear_w8a8_skinny(nullptr, (const int8_t *)L.wo->codes->ptr, B, L.wo->n, L.wo->n_pad, L.wo->k_pad,
                                  epilogue(L.wo, d->h->ptr, (const float *)d->h->ptr), cus, s, nullptr, &pro);
        } else {
            linear(L.wo, d->h->ptr, (const float *)d->h->ptr);
        }
        if (stop_here()) break;
        const bool fuse_gu = k::swiglu_fuses_norm(B, L.wgu->n_pad, L.wgu->k_pad, cus);
        if (!fuse_gu)
            k::rmsnorm_quantize_i8((const float *)d->h->ptr, (const float *)L.ffn_norm->ptr, c.rms_eps, nullptr,
                                   (int8_t *)d->xq->ptr, (float *)d->sx->ptr, B, m_pad, D, s);
        if (stop_here()) break;
        {
            const k::RowPrologue pro = norm_prologue((const float *)L.ffn_norm->ptr);
            k::linear_w8a8_swiglu_skinny((const int8_t *)d->xq->ptr, (const int8_t *)L.wgu->codes->ptr,
                                         (const float *)d->sx->ptr, (const float *)L.wgu->scales->ptr, B, L.wgu->n,
                                         L.wgu->n_pad, L.wgu->k_pad, (float *)d->act->ptr, (float *)d->pmax->ptr, 4, cus, s,
                                         fuse_gu ? &pro : nullptr);
        }
        if (stop_here()) break;
        const bool fuse_down = F % 64 == 0 && k::plain_fuses_pmax_quantizer(B, L.wdown->n_pad, L.wdown->k_pad, cus);
        if (!fuse_down)
            k::quantize_rows_from_pmax(d->act->ptr, false, (const float *)d->pmax->ptr, (uint32_t)(F / 16),
                                       (int8_t *)d->xq->ptr, (float *)d->sx->ptr, B, m_pad, F, s);
        if (stop_here()) break;
        if (fuse_down) {
            k::RowPrologue pro;
            pro.x = (const float *)d->act->ptr;
            pro.pmax = (const float *)d->pmax->ptr;
            pro.parts = (uint32_t)(F / 16);
            pro.xq_tiled_out = (int8_t *)d->xq->ptr;
            pro.sx_out = (float *)d->sx->ptr;
            k::linear_w8a8_skinny(nullptr, (const int8_t *)L.wdown->codes->ptr, B, L.wdown->n, L.wdown->n_pad, L.wdown->k_pad,
                                  epilogue(L.wdown, d->h->ptr, (const float *)d->h->ptr), cus, s, nullptr, &pro);
        } else {
            linear(L.wdown, d->h->ptr, (const float *)d->h->ptr);
        }
        if (stop_here()) break;
    }
    if (stop_after >= 0 && stage > stop_after) return after_launch(ctx, "decoder step (partial)");
    k::rmsnorm_quantize_i8((const float *)d->h->ptr, (const float *)d->final_norm->ptr, c.rms_eps, nullptr,
                           (int8_t *)d->xq->ptr, (float *)d->sx->ptr, B, m_pad, D, s);
    if (stop_here()) return after_launch(ctx, "decoder step (partial)");
    linear(d->lm_head, d->logits->ptr, nullptr);
    if (stop_here()) return after_launch(ctx, "decoder step (partial)");
    enqueue_pick(d, s);
    return after_launch(ctx, "decoder step");
}

// device memory from the context's pool, returned when the call that took it ends (the stream is in
// order, so a later user of the same memory is queued behind this call's kernels)
struct Temp {
    fa_context *ctx;
    void *ptr = nullptr;
    uint64_t bytes = 0, cls = 0;
    fa_decoder::KeptBlock *keep = nullptr;          // a block of the decoder's that this buffer borrows when it is large
    static constexpr uint64_t kKeepFrom = 32ull << 20;
    explicit Temp(fa_context *c, fa_decoder::KeptBlock *k = nullptr) : ctx(c), keep(k) {}
    fa_status get(uint64_t n) {
        bytes = n ? n : 16;
        if (keep && !ctx->capturing && (bytes >= kKeepFrom || keep->bytes >= bytes)) {
            if (keep->bytes < bytes) {
                if (keep->ptr) pool_free(ctx, keep->ptr, keep->bytes, keep->cls);
                *keep = fa_decoder::KeptBlock{};
                if (fa_status st = pool_alloc(ctx, bytes, &keep->ptr, &keep->cls)) return st;
                keep->bytes = bytes;
            }
            ptr = keep->ptr;
            return FA_OK;
        }
        keep = nullptr;
        return pool_alloc(ctx, bytes, &ptr, &cls);
    }
    ~Temp() {
        if (ptr && !keep) scratch_release(ctx, ptr, bytes, cls);
    }
    template <typename T>
    T *as() const { return (T *)ptr; }
};

// One pass of a prompt chunk (lc tokens per sequence, rows = batch * lc, row b * lc + t) through all layers
// on the prefill-shape GEMMs and the prefill form of the attention kernel.  The arithmetic per row is
// that of the decode step (same quantizers, same dequantization, same RoPE and SwiGLU expressions), so
// a prompt token leaves the same K / V rows in the cache as if it had been decoded.
struct PrefillBuffers {
    Temp tok, h, xq, sx, qkv, q_bf, attn, gu, slots, cos_sin, last_rows, splitk;
    // verification only: logits and greedy picks of every row
    Temp all_logits, all_picked;
    // padded pass only: the true prompt length of every row
    Temp row_lens;
    PrefillBuffers(fa_context *c, fa_decoder *d)
        : tok(c), h(c, &d->kept[0]), xq(c, &d->kept[1]), sx(c), qkv(c, &d->kept[2]), q_bf(c, &d->kept[3]), attn(c, &d->kept[4]),
          gu(c, &d->kept[5]), slots(c), cos_sin(c), last_rows(c), splitk(c, &d->kept[6]), all_logits(c, &d->kept[7]),
          all_picked(c), row_lens(c) {}
};

fa_status enqueue_prefill_chunk(fa_context *ctx, fa_decoder *d, PrefillBuffers &t, uint32_t lc, bool last_chunk,
                                bool every_row = false, bool padded = false) {
    const fa_decoder_config &c = d->cfg;
    const uint32_t B = d->batch;
    const uint64_t M = (uint64_t)B * lc;
    const uint64_t D = c.d_model, F = c.d_ffn, V = c.vocab;
    const uint64_t EKV = (uint64_t)c.n_kv_heads * c.head_dim;
    const int cus = ctx->props.multiProcessorCount;
    hipStream_t s = ctx->stream;
    const uint64_t pool_rows = (uint64_t)c.num_blocks * c.block_size;

    k::prefill_prepare((const uint32_t *)d->tables->ptr, (const uint32_t *)d->seq_lens->ptr, t.slots.as<uint32_t>(),
                       t.cos_sin.as<float>(), B, lc, c.block_size, c.max_blocks_per_seq, c.num_blocks, c.head_dim,
                       c.rope_theta, s);
    k::advance_seq_lens((uint32_t *)d->seq_lens->ptr, t.last_rows.as<int32_t>(), B, lc,
                        padded ? t.row_lens.as<uint32_t>() : nullptr, s);
    k::gather_rows_f32((const float *)d->embed->ptr, V, D, t.tok.as<int32_t>(), t.h.as<float>(), M, s);

    k::PagedShape ps;
    ps.num_blocks = c.num_blocks;
    ps.block_size = c.block_size;
    ps.e_kv = (uint32_t)EKV;
    ps.batch = B;
    ps.l_new = lc;
    ps.num_heads = c.n_heads;
    ps.num_kv_heads = c.n_kv_heads;
    ps.head_dim = c.head_dim;
    ps.max_blocks_per_seq = c.max_blocks_per_seq;
    ps.scale = 1.0f / std::sqrt((float)c.head_dim);
    for (uint32_t b = 0; b < B; ++b) ps.ctx_hint = std::max(ps.ctx_hint, d->host_lens[b] + lc);

    // A pass of 65 to a few hundred rows runs its narrow projections on the weight-stationary kernel, which takes
    // activation tiles (the decode kernels' layout) instead of row-major codes: the quantizer in front of such a
    // projection writes that layout.
    const uint64_t M_pad = round_up(M, 16);
    // (at most 64 rows: every projection on the decode kernels, which take the same layout)
    const bool decode_form = M <= 64 && k::g_rows_kernel != 1;
    auto rows_form = [&](const fa_qweight *w) { return decode_form || k::linear_w8a8_rows_applies(M, w->n_pad, w->k_pad, cus, &ctx->splitk); };
    // y = dequant(xq @ w) (+ residual) for the rows quantized into t.xq / t.sx just before
    auto gemm = [&](const fa_qweight *w, float *out, const float *residual) {
        k::EpilogueI8 ep;
        ep.sx = t.sx.as<float>();
        ep.sw = (const float *)w->scales->ptr;
        ep.bias = nullptr;
        ep.residual = residual;
        ep.acc_out = nullptr;
        ep.out = out;
        ep.out_bf16 = 0;
        if (decode_form)
            k::linear_w8a8_skinny(t.xq.as<int8_t>(), (const int8_t *)w->codes->ptr, M, w->n, w->n_pad, w->k_pad, ep, cus, s,
                                  &ctx->splitk);
        else if (rows_form(w))
            k::linear_w8a8_rows(t.xq.as<int8_t>(), (const int8_t *)w->codes->ptr, M, w->n, w->n_pad, w->k_pad, ep, cus, s,
                                &ctx->splitk, t.splitk.ptr, t.splitk.bytes);
        else
            k::gemm_w8a8_mfma(t.xq.as<int8_t>(), (const int8_t *)w->codes->ptr, M, w->n, w->n_pad, w->k_pad, ep, cus, s,
                              t.splitk.ptr, t.splitk.bytes, &ctx->splitk);
    };
    auto norm_quantize = [&](const float *norm_w, const fa_qweight *w) {
        if (rows_form(w))
            k::rmsnorm_quantize_i8(t.h.as<float>(), norm_w, c.rms_eps, nullptr, t.xq.as<int8_t>(), t.sx.as<float>(), M, M_pad, D, s);
        else
            k::rmsnorm_quantize_rows_i8(t.h.as<float>(), norm_w, c.rms_eps, t.xq.as<int8_t>(), t.sx.as<float>(), M, D, s);
    };

    for (uint32_t li = 0; li < c.n_layers; ++li) {
        const fa_decoder::Layer &L = d->layers[li];
        norm_quantize((const float *)L.attn_norm->ptr, L.wqkv);
        // at most 64 rows: the decode step's fused projection (RoPE, the bf16 rounding and the K / V append in the epilogue
        // of the decode kernel); on the large-tile GEMM the q | k | v projection does the same in its epilogue
        if (decode_form && g_prefill_fused_rows != 1) {
            const k::QkvRopeTargets qt{t.cos_sin.as<float>(), t.slots.as<uint32_t>(), t.q_bf.as<uint16_t>(), (uint16_t *)L.k_pool->ptr,
                                       (uint16_t *)L.v_pool->ptr, c.n_heads, c.n_kv_heads, c.head_dim, pool_rows};
            k::linear_w8a8_qkv_rope_skinny(t.xq.as<int8_t>(), (const int8_t *)L.wqkv->codes->ptr, t.sx.as<float>(),
                                           (const float *)L.wqkv->scales->ptr, M, L.wqkv->n_pad, L.wqkv->k_pad, qt, s);
        } else if (const k::QkvRopeTargets qt{t.cos_sin.as<float>(), t.slots.as<uint32_t>(), t.q_bf.as<uint16_t>(),
                                              (uint16_t *)L.k_pool->ptr, (uint16_t *)L.v_pool->ptr, c.n_heads, c.n_kv_heads,
                                              c.head_dim, pool_rows};
                   !decode_form && k::linear_w8a8_qkv_rope_rows_applies(M, L.wqkv->n_pad, L.wqkv->k_pad, cus, &ctx->splitk, qt)) {
            // 65 to a few hundred rows: the same in the epilogue of the weight-stationary kernel
            k::linear_w8a8_qkv_rope_rows(t.xq.as<int8_t>(), (const int8_t *)L.wqkv->codes->ptr, t.sx.as<float>(),
                                         (const float *)L.wqkv->scales->ptr, M, L.wqkv->n_pad, L.wqkv->k_pad, qt, s);
        } else if (!rows_form(L.wqkv) &&
            k::gemm_w8a8_qkv_rope_applies(M, L.wqkv->n, L.wqkv->n_pad, L.wqkv->k_pad, c.n_heads, c.n_kv_heads, c.head_dim, cus)) {
            const k::QkvRopeTargets qt{t.cos_sin.as<float>(), t.slots.as<uint32_t>(), t.q_bf.as<uint16_t>(), (uint16_t *)L.k_pool->ptr,
                                       (uint16_t *)L.v_pool->ptr, c.n_heads, c.n_kv_heads, c.head_dim, pool_rows};
            k::gemm_w8a8_qkv_rope_mfma(t.xq.as<int8_t>(), (const int8_t *)L.wqkv->codes->ptr, t.sx.as<float>(),
                                       (const float *)L.wqkv->scales->ptr, M, L.wqkv->k_pad, qt, s);
        } else {
            gemm(L.wqkv, t.qkv.as<float>(), nullptr);
            k::rope_append(t.qkv.as<float>(), t.cos_sin.as<float>(), t.slots.as<uint32_t>(), t.q_bf.as<uint16_t>(),
                           (uint16_t *)L.k_pool->ptr, (uint16_t *)L.v_pool->ptr, M, c.n_heads, c.n_kv_heads, c.head_dim,
                           pool_rows, s);
        }
        k::paged_attention_prefill_bf16(t.q_bf.as<uint16_t>(), (const uint16_t *)L.k_pool->ptr,
                                        (const uint16_t *)L.v_pool->ptr, (const uint32_t *)d->tables->ptr,
                                        (const uint32_t *)d->seq_lens->ptr, ps, (uint32_t)g_decode_waves, ctx->workspace,
                                        t.attn.ptr, 1, s);
        if (rows_form(L.wo))
            k::quantize_rows_i8(t.attn.ptr, true, nullptr, t.xq.as<int8_t>(), t.sx.as<float>(), M, M_pad, L.wo->k, L.wo->k_pad, s);
        else
            k::quantize_rows_i8(t.attn.ptr, true, t.xq.as<int8_t>(), nullptr, t.sx.as<float>(), M, M, L.wo->k, L.wo->k_pad, s);
        gemm(L.wo, t.h.as<float>(), t.h.as<float>());
        norm_quantize((const float *)L.ffn_norm->ptr, L.wgu);
        if (decode_form && g_prefill_fused_rows != 1 && L.wgu->n == 2 * F && F / 16 <= (uint64_t)c.n_heads * c.head_dim + 2 * EKV) {
            // at most 64 rows: the decode step's gate | up kernel (SwiGLU in the epilogue: products and their partial
            // maxima per 16 columns) and its quantizer from those maxima; t.qkv is free here and holds the maxima
            k::linear_w8a8_swiglu_skinny(t.xq.as<int8_t>(), (const int8_t *)L.wgu->codes->ptr, t.sx.as<float>(),
                                         (const float *)L.wgu->scales->ptr, M, L.wgu->n, L.wgu->n_pad, L.wgu->k_pad, t.gu.as<float>(),
                                         t.qkv.as<float>(), 4, cus, s, nullptr);
            k::quantize_rows_from_pmax(t.gu.ptr, false, t.qkv.as<float>(), (uint32_t)(F / 16), t.xq.as<int8_t>(), t.sx.as<float>(), M,
                                       M_pad, F, s);
            gemm(L.wdown, t.h.as<float>(), t.h.as<float>());
            continue;
        }
        // on the large-tile GEMM the gate | up projection takes SwiGLU into its epilogue and leaves the products
        // ([M, F] instead of [M, 2 F] written and read back); the quantizer behind it is the same either way
        const bool swiglu_in_gemm = !rows_form(L.wgu) && L.wgu->n == 2 * F && k::gemm_w8a8_swiglu_applies(M, F, L.wgu->n_pad, L.wgu->k_pad);
        if (swiglu_in_gemm)
            k::gemm_w8a8_swiglu_mfma(t.xq.as<int8_t>(), (const int8_t *)L.wgu->codes->ptr, t.sx.as<float>(),
                                     (const float *)L.wgu->scales->ptr, M, F, L.wgu->k_pad, t.gu.as<float>(), cus, s);
        else
            gemm(L.wgu, t.gu.as<float>(), nullptr);
        k::swiglu_quantize_rows_i8(t.gu.as<float>(), t.xq.as<int8_t>(), t.sx.as<float>(), M, F, s, rows_form(L.wdown), swiglu_in_gemm);
        gemm(L.wdown, t.h.as<float>(), t.h.as<float>());
    }
    if (padded) k::trim_seq_lens((uint32_t *)d->seq_lens->ptr, t.row_lens.as<uint32_t>(), B, lc, s);
    if (every_row) {
        // verification: the head over every row of the chunk (row b * lc + t is token t of sequence b)
        norm_quantize((const float *)d->final_norm->ptr, d->lm_head);
        gemm(d->lm_head, t.all_logits.as<float>(), nullptr);
        k::argmax_rows_f32(t.all_logits.as<float>(), t.all_picked.as<int32_t>(), M, V, s);
    }
    if (last_chunk) {
        // logits of every sequence's last prompt token, and the greedy next token, as a decode step leaves them
        const uint64_t m_pad = round_up(B, 16);
        k::gather_rows_f32(t.h.as<float>(), M, D, t.last_rows.as<int32_t>(), (float *)d->h->ptr, B, s);
        k::rmsnorm_quantize_i8((const float *)d->h->ptr, (const float *)d->final_norm->ptr, c.rms_eps, nullptr,
                               (int8_t *)d->xq->ptr, (float *)d->sx->ptr, B, m_pad, D, s);
        k::EpilogueI8 ep;
        ep.sx = (const float *)d->sx->ptr;
        ep.sw = (const float *)d->lm_head->scales->ptr;
        ep.bias = nullptr;
        ep.residual = nullptr;
        ep.acc_out = nullptr;
        ep.out = d->logits->ptr;
        ep.out_bf16 = 0;
        k::linear_w8a8_skinny((const int8_t *)d->xq->ptr, (const int8_t *)d->lm_head->codes->ptr, B, d->lm_head->n,
                              d->lm_head->n_pad, d->lm_head->k_pad, ep, cus, s);
        enqueue_pick(d, s);
    }
    return after_launch(ctx, "decoder prefill");
}

}  // namespace

extern "C" {

fa_status fa_decoder_create(fa_context *ctx, const fa_decoder_config *cfg, fa_decoder **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!cfg || !out) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_create: null argument");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "decoder_create during graph capture");
    const fa_decoder_config &c = *cfg;
    if (c.n_layers == 0 || c.d_model == 0 || c.n_heads == 0 || c.n_kv_heads == 0 || c.d_ffn == 0 || c.vocab == 0 ||
        c.max_batch == 0)
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder_create: zero dimension");
    if (c.head_dim != 128 || c.block_size != 16)
        return fail(FA_ERR_UNSUPPORTED, "decoder_create: head_dim must be 128 and block_size 16");
    if (c.n_heads % c.n_kv_heads != 0 || c.n_heads / c.n_kv_heads > 16)
        return fail(FA_ERR_UNSUPPORTED, "decoder_create: heads per kv head must be an integer of at most 16");
    if (c.d_model % 64 != 0 || c.d_ffn % 64 != 0)
        return fail(FA_ERR_UNSUPPORTED, "decoder_create: d_model and d_ffn must be multiples of 64");
    if (c.d_model > 16384) return fail(FA_ERR_UNSUPPORTED, "decoder_create: d_model above 16384");
    if (c.max_batch > 64) return fail(FA_ERR_UNSUPPORTED, "decoder_create: at most 64 sequences per step");
    if (!std::isfinite(c.rms_eps) || c.rms_eps < 0.0f) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_create: bad rms_eps");
    if (!(c.rope_theta > 0.0)) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_create: bad rope_theta");
    fa_paged_layout layout{c.num_blocks, c.block_size, (uint64_t)c.n_kv_heads * c.head_dim};
    if (fa_status s = paged_layout_check(&layout)) return s;
    if (c.max_blocks_per_seq == 0 || (uint64_t)c.max_blocks_per_seq * c.block_size > (uint64_t)INT32_MAX)
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder_create: bad max_blocks_per_seq");

    fa_decoder *d = new (std::nothrow) fa_decoder();
    if (!d) return fail(FA_ERR_ALLOCATION_FAILED, "decoder_create: host allocation failed");
    d->magic = kDecMagic;
    d->ctx = ctx;
    d->cfg = c;
    d->layers.resize(c.n_layers);
    const uint64_t B = c.max_batch, D = c.d_model, F = c.d_ffn, V = c.vocab;
    const uint64_t EQ = (uint64_t)c.n_heads * c.head_dim;
    const uint64_t kmax = std::max(std::max(D, F), EQ);
    fa_status s = FA_OK;
    auto mk = [&](fa_dtype t, uint64_t n, fa_buffer **b) {
        if (s == FA_OK) s = make_buffer(ctx, t, n, true, b);
    };
    mk(FA_I32, B, &d->tokens);
    mk(FA_U32, B * c.max_blocks_per_seq, &d->tables);
    mk(FA_U32, B, &d->seq_lens);
    mk(FA_I32, B, &d->pos);
    mk(FA_U32, B, &d->slots);
    mk(FA_F32, B * c.head_dim, &d->cos_sin);
    mk(FA_F32, B * D, &d->h);
    mk(FA_I8, round_up(B, 16) * kmax, &d->xq);
    mk(FA_F32, B, &d->sx);
    mk(FA_BF16, B * EQ, &d->q_bf);
    mk(FA_BF16, B * EQ, &d->attn);
    mk(FA_F32, B * F, &d->act);
    mk(FA_F32, B * std::max<uint64_t>(F / 16, c.n_heads), &d->pmax);
    mk(FA_F32, B * V, &d->logits);
    mk(FA_U32, 2, &d->rng);
    mk(FA_U32, 6 * (uint64_t)c.max_batch, &d->policy);
    for (auto &l : d->layers) {
        mk(FA_BF16, layout.num_blocks * layout.block_size * layout.embed_dim, &l.k_pool);
        mk(FA_BF16, layout.num_blocks * layout.block_size * layout.embed_dim, &l.v_pool);
    }
    if (s != FA_OK) {
        free_all(ctx, d);
        delete d;
        return s;
    }
    *out = d;
    return FA_OK;
}

fa_status fa_decoder_destroy(fa_context *ctx, fa_decoder *d) {
    if (!d) return FA_OK;
    if (fa_status s = check_dec(d)) return s;
    drop_graphs(d);
    free_all(ctx, d);
    d->magic = 0;
    delete d;
    return FA_OK;
}

fa_status fa_decoder_set_layer(fa_decoder *d, uint32_t layer, const fa_buffer *attn_norm, const fa_buffer *ffn_norm,
                               const fa_qweight *wqkv, const fa_qweight *wo, const fa_qweight *wgu,
                               const fa_qweight *wdown) {
    if (fa_status s = check_dec(d)) return s;
    const fa_decoder_config &c = d->cfg;
    if (layer >= c.n_layers) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_layer: layer out of range");
    const uint64_t D = c.d_model, EQ = (uint64_t)c.n_heads * c.head_dim, EKV = (uint64_t)c.n_kv_heads * c.head_dim;
    if (fa_status s = check_vec(d, attn_norm, D, "decoder_set_layer: attn_norm")) return s;
    if (fa_status s = check_vec(d, ffn_norm, D, "decoder_set_layer: ffn_norm")) return s;
    if (fa_status s = check_weight(d, wqkv, D, EQ + 2 * EKV, "decoder_set_layer: wqkv")) return s;
    if (fa_status s = check_weight(d, wo, EQ, D, "decoder_set_layer: wo")) return s;
    if (fa_status s = check_weight(d, wgu, D, 2ull * c.d_ffn, "decoder_set_layer: wgu")) return s;
    if (fa_status s = check_weight(d, wdown, c.d_ffn, D, "decoder_set_layer: wdown")) return s;
    fa_decoder::Layer &L = d->layers[layer];
    L.attn_norm = attn_norm;
    L.ffn_norm = ffn_norm;
    L.wqkv = wqkv;
    L.wo = wo;
    L.wgu = wgu;
    L.wdown = wdown;
    drop_graphs(d);
    return FA_OK;
}

fa_status fa_decoder_set_head(fa_decoder *d, const fa_buffer *embed, const fa_buffer *final_norm,
                              const fa_qweight *lm_head) {
    if (fa_status s = check_dec(d)) return s;
    const fa_decoder_config &c = d->cfg;
    if (fa_status s = check_vec(d, embed, (uint64_t)c.vocab * c.d_model, "decoder_set_head: embed")) return s;
    if (fa_status s = check_vec(d, final_norm, c.d_model, "decoder_set_head: final_norm")) return s;
    if (fa_status s = check_weight(d, lm_head, c.d_model, c.vocab, "decoder_set_head: lm_head")) return s;
    d->embed = embed;
    d->final_norm = final_norm;
    d->lm_head = lm_head;
    drop_graphs(d);
    return FA_OK;
}

fa_status fa_decoder_set_sampling(fa_context *ctx, fa_decoder *d, fa_sampling strategy, float temperature, uint64_t top_k,
                                  uint64_t seed) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "decoder_set_sampling: decoder belongs to another context");
    if (strategy != FA_SAMPLE_GREEDY && strategy != FA_SAMPLE_TEMPERATURE && strategy != FA_SAMPLE_TOP_K)
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_sampling: unknown strategy");
    if (strategy != FA_SAMPLE_GREEDY && !(std::isfinite(temperature) && temperature > 0.0f))
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_sampling: temperature must be finite and positive");
    if (strategy == FA_SAMPLE_TOP_K && (top_k == 0 || top_k > d->cfg.vocab))
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_sampling: top_k must be in 1..=vocab");
    if (fa_status s = fa_rng_seed(ctx, d->rng, seed)) return s;
    // the captured steps hold the choice (not the seed: the generator state is read from device memory)
    const bool same = !d->per_row && d->strategy == strategy &&
                      (strategy == FA_SAMPLE_GREEDY || (d->temperature == temperature && d->top_k == (uint32_t)top_k));
    d->strategy = strategy;
    d->temperature = temperature;
    d->top_k = (uint32_t)top_k;
    d->per_row = false;
    if (!same) drop_graphs(d);
    return FA_OK;
}

static_assert(sizeof(fa_row_sampling) == sizeof(k::RowPolicy) && sizeof(fa_row_sampling) == 24, "row sampling layout");

fa_status fa_decoder_set_row_sampling(fa_context *ctx, fa_decoder *d, const fa_row_sampling *rows) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "decoder_set_row_sampling: decoder belongs to another context");
    if (d->batch == 0) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_row_sampling: set the sequences first");
    if (!rows) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_row_sampling: null rows");
    for (uint32_t b = 0; b < d->batch; ++b) {
        const fa_row_sampling &r = rows[b];
        const std::string where = "decoder_set_row_sampling: row " + std::to_string(b);
        if (r.strategy != FA_SAMPLE_GREEDY && r.strategy != FA_SAMPLE_TEMPERATURE && r.strategy != FA_SAMPLE_TOP_K)
            return fail(FA_ERR_INVALID_ARGUMENT, where + ": unknown strategy");
        if (!(std::isfinite(r.temperature) && r.temperature > 0.0f))
            return fail(FA_ERR_INVALID_ARGUMENT, where + ": temperature must be finite and positive");
        if (r.strategy == FA_SAMPLE_TOP_K && (r.top_k == 0 || r.top_k > d->cfg.vocab))
            return fail(FA_ERR_INVALID_ARGUMENT, where + ": top_k must be in 1..=vocab");
        if (r.strategy != FA_SAMPLE_GREEDY && r.rng_state == 0)
            return fail(FA_ERR_INVALID_ARGUMENT, where + ": a generator state is never zero (fa_rng_state_from_seed)");
    }
    if (fa_status s = fa_upload_into(ctx, rows, (uint64_t)d->batch * 6, d->policy, 0)) return s;
    if (!d->per_row) drop_graphs(d);                    // the captured steps pick the other way
    d->per_row = true;
    return FA_OK;
}

fa_status fa_decoder_read_row_sampling(fa_context *ctx, fa_decoder *d, fa_row_sampling *rows) {
    if (fa_status s = check_dec(d)) return s;
    if (!rows) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_read_row_sampling: null rows");
    if (!d->per_row) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_read_row_sampling: no per-row table installed");
    return fa_download(ctx, d->policy, 0, rows, (uint64_t)d->batch * 6);
}

fa_status fa_decoder_kv_pools(fa_decoder *d, uint32_t layer, fa_buffer **k_pool, fa_buffer **v_pool) {
    if (fa_status s = check_dec(d)) return s;
    if (layer >= d->cfg.n_layers) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_kv_pools: layer out of range");
    if (k_pool) *k_pool = d->layers[layer].k_pool;
    if (v_pool) *v_pool = d->layers[layer].v_pool;
    return FA_OK;
}

fa_status fa_decoder_set_sequences(fa_context *ctx, fa_decoder *d, uint32_t batch, const uint32_t *block_tables,
                                   const uint32_t *seq_lens) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    const fa_decoder_config &c = d->cfg;
    if (batch == 0 || batch > c.max_batch) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_sequences: batch out of range");
    if (!block_tables || !seq_lens) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_sequences: null table");
    // the next step writes position seq_len and then attends to seq_len + 1 tokens
    for (uint32_t b = 0; b < batch; ++b) {
        uint64_t need = ((uint64_t)seq_lens[b] + 1 + c.block_size - 1) / c.block_size;
        if (need > c.max_blocks_per_seq)
            return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " has no room for one more token");
        for (uint64_t i = 0; i < need; ++i)
            if (block_tables[(uint64_t)b * c.max_blocks_per_seq + i] >= c.num_blocks)
                return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " entry " +
                                                         std::to_string(i) + " is not a valid block id");
    }
    if (fa_status s = fa_upload_into(ctx, block_tables, (uint64_t)batch * c.max_blocks_per_seq, d->tables, 0)) return s;
    if (fa_status s = fa_upload_into(ctx, seq_lens, batch, d->seq_lens, 0)) return s;
    d->batch = batch;
    try {
        d->host_tables.assign(block_tables, block_tables + (uint64_t)batch * c.max_blocks_per_seq);
        d->host_lens.assign(seq_lens, seq_lens + batch);
    } catch (const std::exception &) {
        d->batch = 0;
        return fail(FA_ERR_ALLOCATION_FAILED, "decoder_set_sequences: out of host memory");
    }
    return FA_OK;
}

fa_status fa_decoder_set_tokens(fa_context *ctx, fa_decoder *d, const int32_t *tokens) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->batch == 0) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_tokens: set the sequences first");
    if (!tokens) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_tokens: null tokens");
    for (uint32_t b = 0; b < d->batch; ++b)
        if (tokens[b] < 0 || (uint32_t)tokens[b] >= d->cfg.vocab)
            return fail(FA_ERR_INVALID_ARGUMENT, "decoder_set_tokens: token id outside the vocabulary");
    return fa_upload_into(ctx, tokens, d->batch, d->tokens, 0);
}

// The position every row writes in a decode step must have a page (validate_paged_kv_append rejects a row
// without a slot before anything is queued, crates/tensor-core/src/paged_kv.rs:222-290); checked on the host
// mirror of the installed tables by every entry point that runs the step's launches.
static fa_status check_step_room(const fa_decoder *d) {
    const fa_decoder_config &c = d->cfg;
    for (uint32_t b = 0; b < d->batch; ++b) {
        const uint64_t pos = d->host_lens[b];
        if (pos >= (uint64_t)c.max_blocks_per_seq * c.block_size)
            return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " has no room for one more token");
        if (d->host_tables[(uint64_t)b * c.max_blocks_per_seq + pos / c.block_size] >= c.num_blocks)
            return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " has no page for position " +
                                                     std::to_string(pos));
    }
    return FA_OK;
}

fa_status fa_decoder_step(fa_context *ctx, fa_decoder *d, int32_t use_graph) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "decoder_step: decoder belongs to another context");
    if (d->batch == 0) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_step: no sequences installed");
    if (!d->embed || !d->final_norm || !d->lm_head) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_step: head weights missing");
    for (auto &l : d->layers)
        if (!l.wqkv) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_step: layer weights missing");
    // attention workspace sized before anything is captured
    k::PagedShape ps{};
    ps.batch = d->batch;
    ps.num_heads = d->cfg.n_heads;
    ps.num_kv_heads = d->cfg.n_kv_heads;
    ps.max_blocks_per_seq = d->cfg.max_blocks_per_seq;
    if (fa_status s = ensure_workspace(ctx, k::paged_decode_workspace_bytes(ps, (uint32_t)g_decode_waves))) return s;
    if (fa_status s = check_step_room(d)) return s;
    // The host mirror of the lengths follows the device-side advance of this step; every return below that has
    // queued nothing takes the advance back.
    auto advance = [&](int by) {
        for (auto &len : d->host_lens) len += by;
    };
    if (!use_graph) {
        advance(1);
        fa_status es = enqueue_step(ctx, d);
        if (es != FA_OK) advance(-1);
        return es;
    }
    if (d->graph_waves != g_decode_waves) drop_graphs(d);
    // a graph per batch size and kind of step (bit 31: the short-context form, decided on the lengths after this step)
    advance(1);
    const uint32_t key = d->batch | (step_is_short(d) ? 0x80000000u : 0u);
    advance(-1);
    auto it = d->graphs.find(key);
    if (it == d->graphs.end()) {
        try {
            it = d->graphs.emplace(key, nullptr).first;
        } catch (const std::exception &) {
            return fail(FA_ERR_ALLOCATION_FAILED, "decoder_step: out of host memory");      // lengths not advanced yet
        }
    }
    advance(1);
    if (it->second == nullptr) {
        fa_status cs = fa_graph_capture_begin(ctx);
        fa_graph *g = nullptr;
        if (cs == FA_OK) {
            fa_status es = enqueue_step(ctx, d);
            cs = fa_graph_capture_end(ctx, &g);
            if (es != FA_OK) {
                if (g) fa_graph_destroy(ctx, g);
                g = nullptr;
                cs = es;
            }
        }
        if (cs != FA_OK || !g) {
            d->graphs.erase(it);
            advance(-1);                                // nothing ran
            return cs != FA_OK ? cs : fail(FA_ERR_KERNEL_LAUNCH_FAILED, "decoder_step: capture produced no graph");
        }
        it->second = g;
        d->graph_waves = g_decode_waves;
    }
    fa_status ls = fa_graph_launch(ctx, it->second);
    if (ls != FA_OK) advance(-1);
    return ls;
}

static fa_status prefill_impl(fa_context *ctx, fa_decoder *d, const int32_t *tokens, uint32_t l_new, int32_t *picked,
                              float *logits, const uint32_t *row_lens = nullptr) {
    const bool verify = picked != nullptr, padded = row_lens != nullptr;
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "decoder_prefill: decoder belongs to another context");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "decoder_prefill during graph capture");
    if (d->batch == 0) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill: no sequences installed");
    if (!d->embed || !d->final_norm || !d->lm_head) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill: head weights missing");
    for (auto &l : d->layers)
        if (!l.wqkv) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill: layer weights missing");
    if (!tokens || l_new == 0) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill: no tokens");
    const fa_decoder_config &c = d->cfg;
    const uint32_t B = d->batch;
    for (uint64_t i = 0; i < (uint64_t)B * l_new; ++i)
        if (tokens[i] < 0 || (uint32_t)tokens[i] >= c.vocab)
            return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill: token id outside the vocabulary");
    // every position the prompt writes must have a valid page
    for (uint32_t b = 0; b < B; ++b) {
        if (padded && (row_lens[b] == 0 || row_lens[b] > l_new))
            return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill: row " + std::to_string(b) + " has a length outside 1..=l_max");
        // the padding needs no pages, but its positions must stay inside the row of the block table
        if ((uint64_t)d->host_lens[b] + l_new > (uint64_t)c.max_blocks_per_seq * c.block_size)
            return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " has no room for the prompt");
        const uint64_t end = (uint64_t)d->host_lens[b] + (padded ? row_lens[b] : l_new);
        const uint64_t need = (end + c.block_size - 1) / c.block_size;
        if (need > c.max_blocks_per_seq)
            return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " has no room for the prompt");
        for (uint64_t i = 0; i < need; ++i)
            if (d->host_tables[(uint64_t)b * c.max_blocks_per_seq + i] >= c.num_blocks)
                return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: row " + std::to_string(b) + " entry " + std::to_string(i) +
                                                         " is not a valid block id");
    }
    // chunks of at most kRows rows per pass bound the activation memory (the widest is [rows, 2 d_ffn] f32: 0.9 GB at the
    // benchmark's width).  8192 rather than 4096: the q | k | v projection at 6144 columns is 24 column blocks of the
    // large-tile GEMM, 384 tiles = one and a half rounds of the device at 4096 rows, 768 = three whole rounds at 8192
    // (a prompt pass of 4 x 2048 tokens on one box: 75.9 ms in chunks of 4096 rows, 74.9 in one of 8192; tuning key 25).
    // Passes that keep every row's logits stay at 4096.
    const uint64_t kRows = g_prefill_rows >= 256 ? (uint64_t)g_prefill_rows : 8192;
    constexpr uint64_t kRowsChecked = 4096;
    if ((verify || padded) && (uint64_t)B * l_new > kRowsChecked)
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder: at most 4096 rows (batch x tokens) per verification or padded prompt pass");
    const uint32_t lc_max = (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>(l_new, kRows / B));
    const uint64_t M = (uint64_t)B * lc_max;
    const uint64_t D = c.d_model, F = c.d_ffn, EQ = (uint64_t)c.n_heads * c.head_dim, EKV = (uint64_t)c.n_kv_heads * c.head_dim;
    const uint64_t kmax = std::max(std::max(D, F), EQ);
    PrefillBuffers t(ctx, d);
    fa_status st = FA_OK;
    auto get = [&](Temp &b, uint64_t bytes) {
        if (st == FA_OK) st = b.get(bytes);
    };
    get(t.tok, M * 4);
    get(t.h, M * D * 4);
    get(t.xq, round_up(M, 16) * kmax);                    // row-major codes, or activation tiles with rows padded to 16
    get(t.sx, M * 4);
    get(t.qkv, M * (EQ + 2 * EKV) * 4);
    get(t.q_bf, M * EQ * 2);
    get(t.attn, M * EQ * 2);
    get(t.gu, M * 2 * F * 4);
    get(t.slots, M * 4);
    get(t.cos_sin, M * c.head_dim * 4);
    get(t.last_rows, (uint64_t)B * 4);
    {
        // short prompts leave the narrow projections too few tiles to fill the device: room for their k splits
        uint64_t need = 0;
        const int cus = ctx->props.multiProcessorCount;
        for (const auto &l : d->layers)
            for (const fa_qweight *w : {l.wqkv, l.wo, l.wgu, l.wdown})
                need = std::max({need, k::gemm_w8a8_workspace_bytes(M, w->n, w->n_pad, w->k_pad, cus),
                                 k::linear_w8a8_rows_workspace_bytes(M, w->n_pad, w->k_pad, cus, &ctx->splitk)});
        if (verify)
            need = std::max(need, k::gemm_w8a8_workspace_bytes(M, d->lm_head->n, d->lm_head->n_pad, d->lm_head->k_pad, cus));
        get(t.splitk, need);
    }
    if (verify) {
        get(t.all_logits, M * c.vocab * 4);
        get(t.all_picked, M * 4);
    }
    if (padded) get(t.row_lens, (uint64_t)B * 4);
    if (st != FA_OK) return st;
    k::PagedShape ps{};
    ps.batch = B;
    ps.l_new = lc_max;
    ps.num_heads = c.n_heads;
    ps.num_kv_heads = c.n_kv_heads;
    ps.max_blocks_per_seq = c.max_blocks_per_seq;
    if (fa_status s = ensure_workspace(ctx, k::paged_prefill_workspace_bytes(ps, (uint32_t)g_decode_waves))) return s;

    std::vector<int32_t> stage;
    try {
        stage.resize(M);
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "decoder_prefill: out of host memory");
    }
    for (uint32_t t0 = 0; t0 < l_new; t0 += lc_max) {
        const uint32_t lc = std::min(lc_max, l_new - t0);
        for (uint32_t b = 0; b < B; ++b)
            for (uint32_t i = 0; i < lc; ++i) stage[(uint64_t)b * lc + i] = tokens[(uint64_t)b * l_new + t0 + i];
        // the staging vector is reused by the next chunk: the copy must have consumed it before this call goes on
        hipError_t e = hipMemcpyAsync(t.tok.ptr, stage.data(), (uint64_t)B * lc * 4, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) return hip_fail(ctx, e, "prompt token upload", FA_ERR_TRANSFER_FAILED);
        if (padded) {
            e = hipMemcpyAsync(t.row_lens.ptr, row_lens, (uint64_t)B * 4, hipMemcpyHostToDevice, ctx->stream);
            if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
            if (e != hipSuccess) return hip_fail(ctx, e, "prompt lengths upload", FA_ERR_TRANSFER_FAILED);
        }
        if (fa_status s = enqueue_prefill_chunk(ctx, d, t, lc, t0 + lc == l_new, verify, padded)) return s;
        for (uint32_t b = 0; b < B; ++b) d->host_lens[b] += padded ? row_lens[b] : lc;
    }
    if (verify) {
        // one chunk; the buffers go back to the pool when this call returns, so the copies finish here
        hipError_t e = hipMemcpyAsync(picked, t.all_picked.ptr, (uint64_t)B * l_new * 4, hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess && logits)
            e = hipMemcpyAsync(logits, t.all_logits.ptr, (uint64_t)B * l_new * c.vocab * 4, hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) return hip_fail(ctx, e, "verification results download", FA_ERR_TRANSFER_FAILED);
    }
    return FA_OK;
}

fa_status fa_decoder_prefill(fa_context *ctx, fa_decoder *d, const int32_t *tokens, uint32_t l_new) {
    return prefill_impl(ctx, d, tokens, l_new, nullptr, nullptr);
}

fa_status fa_decoder_prefill_padded(fa_context *ctx, fa_decoder *d, const int32_t *tokens, uint32_t l_max,
                                    const uint32_t *row_lens) {
    if (!row_lens) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_prefill_padded: null lengths");
    return prefill_impl(ctx, d, tokens, l_max, nullptr, nullptr, row_lens);
}

fa_status fa_decoder_verify(fa_context *ctx, fa_decoder *d, const int32_t *tokens, uint32_t l_new, int32_t *picked,
                            float *logits) {
    if (!picked) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_verify: null picked");
    return prefill_impl(ctx, d, tokens, l_new, picked, logits);
}

fa_status fa_decoder_rewind(fa_context *ctx, fa_decoder *d, const uint32_t *seq_lens) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "decoder_rewind: decoder belongs to another context");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "decoder_rewind during graph capture");
    if (d->batch == 0 || !seq_lens) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_rewind: no sequences or null lengths");
    for (uint32_t b = 0; b < d->batch; ++b)
        if (seq_lens[b] > d->host_lens[b])
            return fail(FA_ERR_INVALID_ARGUMENT, "decoder_rewind: row " + std::to_string(b) + " cannot grow (" +
                                                     std::to_string(seq_lens[b]) + " > " + std::to_string(d->host_lens[b]) + ")");
    if (fa_status s = fa_upload_into(ctx, seq_lens, d->batch, d->seq_lens, 0)) return s;
    std::copy(seq_lens, seq_lens + d->batch, d->host_lens.begin());
    return FA_OK;
}

fa_status fa_decoder_debug_step_until(fa_context *ctx, fa_decoder *d, int32_t stop_after) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_dec(d)) return s;
    if (d->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "decoder_debug_step_until: decoder belongs to another context");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "decoder_debug_step_until during graph capture");
    if (d->batch == 0 || stop_after < 0) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_debug_step_until: no sequences or negative stage");
    if (!d->embed || !d->final_norm || !d->lm_head) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_debug_step_until: head weights missing");
    for (auto &l : d->layers)
        if (!l.wqkv) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_debug_step_until: layer weights missing");
    k::PagedShape ps{};
    ps.batch = d->batch;
    ps.num_heads = d->cfg.n_heads;
    ps.num_kv_heads = d->cfg.n_kv_heads;
    ps.max_blocks_per_seq = d->cfg.max_blocks_per_seq;
    if (fa_status s = ensure_workspace(ctx, k::paged_decode_workspace_bytes(ps, (uint32_t)g_decode_waves))) return s;
    if (fa_status s = check_step_room(d)) return s;
    for (auto &len : d->host_lens) len += 1;            // the bookkeeping stage advances the lengths on the device
    fa_status es = enqueue_step(ctx, d, stop_after);
    if (es != FA_OK)
        for (auto &len : d->host_lens) len -= 1;
    return es;
}

fa_status fa_decoder_debug_buffer(fa_decoder *d, int32_t which, fa_buffer **out) {
    if (fa_status s = check_dec(d)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_debug_buffer: null output");
    fa_buffer *table[] = {d->h, d->xq, d->sx, d->q_bf, d->act, d->pmax, d->logits, d->cos_sin, d->slots, d->pos};
    if (which < 0 || which >= (int32_t)(sizeof(table) / sizeof(table[0])))
        return fail(FA_ERR_INVALID_ARGUMENT, "decoder_debug_buffer: unknown buffer");
    *out = table[which];
    return FA_OK;
}

fa_status fa_decoder_read_tokens(fa_context *ctx, fa_decoder *d, int32_t *tokens) {
    if (fa_status s = check_dec(d)) return s;
    return fa_download(ctx, d->tokens, 0, tokens, d->batch);
}
fa_status fa_decoder_read_logits(fa_context *ctx, fa_decoder *d, float *logits) {
    if (fa_status s = check_dec(d)) return s;
    return fa_download(ctx, d->logits, 0, logits, (uint64_t)d->batch * d->cfg.vocab);
}
fa_status fa_decoder_logits_buffer(fa_decoder *d, fa_buffer **out) {
    if (fa_status s = check_dec(d)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "decoder_logits_buffer: null out");
    *out = d->logits;
    return FA_OK;
}
fa_status fa_decoder_read_seq_lens(fa_context *ctx, fa_decoder *d, uint32_t *seq_lens) {
    if (fa_status s = check_dec(d)) return s;
    return fa_download(ctx, d->seq_lens, 0, seq_lens, d->batch);
}

}  // extern "C"
