// CPU oracle (test infrastructure only, see oracle.h): one decode step of a
// Llama-style decoder assembled from the oracle's own operators.  The reference
// has no such model (its decoder layer is post-norm LayerNorm + MHA + ReLU/GELU
// FFN, crates/autodiff/src/nn/transformer_decoder_layer.rs:13-18); the
// dataflow and every rounding point are defined in oracle.h and the operators
// keep their reference semantics.
#include "oracle.h"

#include <cmath>
#include <cstring>
#include <vector>

extern "C" int orc_decode_step(const orc_decoder_config *cfg, const orc_decoder_weights *w,
                               uint16_t *const *k_pools, uint16_t *const *v_pools,
                               const uint32_t *block_tables, uint32_t *seq_lens,
                               const int32_t *tokens, uint32_t batch, int32_t *next_tokens,
                               float *logits_out) {
    const size_t B = batch, D = cfg->d_model, H = cfg->n_heads, HKV = cfg->n_kv_heads,
                 DH = cfg->head_dim, F = cfg->d_ffn, V = cfg->vocab;
    const size_t EQ = H * DH, EKV = HKV * DH, NQKV = EQ + 2 * EKV;

    std::vector<float> h(B * D), x(B * D), qkv(B * NQKV), q(B * EQ), k(B * EKV), v(B * EKV),
        qr(B * EQ), kr(B * EKV), attn(B * EQ), attn_in(B * EQ), o(B * D), gu(B * 2 * F),
        act(B * F), dn(B * D);
    std::vector<uint16_t> q_bf(B * EQ), k_bf(B * EKV), v_bf(B * EKV), attn_bf(B * EQ);
    std::vector<int32_t> pos(B);
    std::vector<uint32_t> slots(B), new_lens(B);

    for (size_t b = 0; b < B; ++b) {
        if (tokens[b] < 0 || (size_t)tokens[b] >= V) return -1;
        std::memcpy(&h[b * D], w->embed + (size_t)tokens[b] * D, D * sizeof(float));
        uint32_t p = seq_lens[b];
        if (p / cfg->block_size >= cfg->max_blocks_per_seq) return -1;
        uint32_t blk = block_tables[b * cfg->max_blocks_per_seq + p / cfg->block_size];
        if (blk >= cfg->num_blocks) return -1;
        pos[b] = (int32_t)p;
        slots[b] = blk * cfg->block_size + p % cfg->block_size;
        new_lens[b] = p + 1;
    }

    orc_paged_args pa;
    pa.layout.num_blocks = cfg->num_blocks;
    pa.layout.block_size = cfg->block_size;
    pa.layout.embed_dim = EKV;
    pa.batch = B;
    pa.l_new = 1;
    pa.num_heads = H;
    pa.num_kv_heads = HKV;
    pa.max_blocks_per_seq = cfg->max_blocks_per_seq;
    pa.scale = 1.0f / std::sqrt((float)DH);

    for (uint32_t l = 0; l < cfg->n_layers; ++l) {
        if (orc_rmsnorm_f32(h.data(), w->w_attn_norm[l], D, cfg->rms_eps, B, D, B * D, x.data())) return -1;
        orc_linear_w8a8(x.data(), w->wqkv[l], w->sqkv[l], nullptr, nullptr, qkv.data(), B, NQKV, D);
        for (size_t b = 0; b < B; ++b) {
            std::memcpy(&q[b * EQ], &qkv[b * NQKV], EQ * sizeof(float));
            std::memcpy(&k[b * EKV], &qkv[b * NQKV + EQ], EKV * sizeof(float));
            std::memcpy(&v[b * EKV], &qkv[b * NQKV + EQ + EKV], EKV * sizeof(float));
        }
        orc_rope_f32(q.data(), pos.data(), B, H, DH, cfg->rope_theta, qr.data());
        orc_rope_f32(k.data(), pos.data(), B, HKV, DH, cfg->rope_theta, kr.data());
        orc_f32_to_bf16_n(qr.data(), q_bf.data(), B * EQ);
        orc_f32_to_bf16_n(kr.data(), k_bf.data(), B * EKV);
        orc_f32_to_bf16_n(v.data(), v_bf.data(), B * EKV);
        if (orc_paged_kv_append(k_bf.data(), v_bf.data(), k_pools[l], v_pools[l], slots.data(), B,
                                &pa.layout, 2))
            return -1;
        if (orc_paged_attention_bf16(q_bf.data(), k_pools[l], v_pools[l], block_tables,
                                     new_lens.data(), &pa, attn.data()))
            return -1;
        orc_f32_to_bf16_n(attn.data(), attn_bf.data(), B * EQ);
        orc_bf16_to_f32_n(attn_bf.data(), attn_in.data(), B * EQ);
        orc_linear_w8a8(attn_in.data(), w->wo[l], w->so[l], nullptr, nullptr, o.data(), B, D, EQ);
        orc_add_f32(h.data(), o.data(), h.data(), B * D);

        if (orc_rmsnorm_f32(h.data(), w->w_ffn_norm[l], D, cfg->rms_eps, B, D, B * D, x.data())) return -1;
        orc_linear_w8a8(x.data(), w->wgu[l], w->sgu[l], nullptr, nullptr, gu.data(), B, 2 * F, D);
        for (size_t b = 0; b < B; ++b)
            orc_silu_mul_f32(&gu[b * 2 * F], &gu[b * 2 * F + F], &act[b * F], F);
        orc_linear_w8a8(act.data(), w->wdown[l], w->sdown[l], nullptr, nullptr, dn.data(), B, D, F);
        orc_add_f32(h.data(), dn.data(), h.data(), B * D);
    }

    if (orc_rmsnorm_f32(h.data(), w->w_final_norm, D, cfg->rms_eps, B, D, B * D, x.data())) return -1;
    std::vector<float> logits(B * V);
    orc_linear_w8a8(x.data(), w->wlm, w->slm, nullptr, nullptr, logits.data(), B, V, D);
    orc_argmax_rows_f32(logits.data(), B, V, next_tokens);
    if (logits_out) std::memcpy(logits_out, logits.data(), logits.size() * sizeof(float));
    for (size_t b = 0; b < B; ++b) seq_lens[b] = new_lens[b];
    return 0;
}
