"""Every fused stage of the decode step, at the benchmark's own width, against the matching oracle operator
on the stage's own input.

The chained-step tests hold the logits to a bar relative to the logit range, because one flipped int8 code
early in the chain moves a whole row.  Here nothing is chained: the step is run eagerly up to a stage
(fa_decoder_debug_step_until), what that stage left in the decoder's buffers is read back, and the oracle
operator is applied to what the *GPU* left one stage earlier.  Bars:
  * quantizer codes and scales: bit-exact;
  * outputs that are an exact function of the int32 accumulators (f32 projections with residual, logits, the V rows
    written to the cache): bit-exact, which pins the accumulators of the fused kernels bit for bit;
  * RoPE'd q / K rows (bf16 of an f32 the kernel does not store): equal to the oracle's bf16, or the adjacent bf16
    value in a vanishing fraction of elements (the cos / sin table is the device's double-precision cos / sin);
  * SwiGLU activations and attention: the reference's composite tolerance (rel < 1e-3 or abs < 1e-5); the fused
    attention + quantizer stage stores codes only, so its codes must be a round-to-nearest quantization, under its own
    scale, of a value within that tolerance (and one bf16 rounding) of the oracle's attention output.
One layer of d_model 4096, 32 / 8 heads, FFN 14336, vocab 32000, batch 32, contexts uniform in [1024, 8192]."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as o
from decoder_common import GpuDecoder, build_model
from gpu_common import assert_parity, ops

pytestmark = pytest.mark.gpu

H, XQ, SX, QBF, ACT, PMAX, LOGITS, COS_SIN, SLOTS, POS = range(10)


def _buf(fa, be, dec, which, dtype, count):
    h = fa.capi.buf_p()
    fa.check(fa.capi.lib.fa_decoder_debug_buffer(dec.h, which, C.byref(h)))
    out = np.empty(count, dtype=dtype)
    fa.check(fa.capi.lib.fa_download(be._ctx, h, 0, out.ctypes.data, count))
    return out


def _untile(codes, m, k):
    """Activation codes in tile order -> [m, k] (tiles [row tile][k tile] of 16 rows x 64 k, byte
    ((g * 16 + r) * 16 + j) of a tile = row r, k 16 g + j)."""
    m_pad = (m + 15) // 16 * 16
    t = codes[:m_pad * k].reshape(m_pad // 16, k // 64, 4, 16, 16)
    return np.ascontiguousarray(t.transpose(0, 3, 1, 2, 4).reshape(m_pad, k)[:m])


def _norm(x, w):
    rc, out = o.rmsnorm_f32(np.ascontiguousarray(x), w, 1e-5)
    assert rc == 0
    return out


def test_every_stage_of_the_step_against_its_oracle_operator_at_the_benchmark_width():
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    B, D, NH, NKV, DH, F, V = 32, 4096, 32, 8, 128, 14336, 32000
    EQ, EKV = NH * DH, NKV * DH
    ctxs = np.random.default_rng(0).integers(1024, 8193, size=B).tolist()
    m = build_model(seed=3, n_layers=1, d_model=D, n_heads=NH, n_kv_heads=NKV, d_ffn=F, vocab=V, batch=B, ctxs=ctxs,
                    steps=3, numpy_fill=True)
    L = m.layers[0]
    dec = GpuDecoder(be, m)
    o.set_threads(8)
    try:
        lens, tokens = m.seq_lens.copy(), m.tokens.copy()

        def run_until(stage):
            dec.set_state(lens, tokens)
            fa.check(lib.fa_decoder_debug_step_until(be._ctx, dec.h, stage))

        # ---- stage 0: bookkeeping + embedding gather
        run_until(0)
        h0 = _buf(fa, be, dec, H, np.float32, B * D).reshape(B, D)
        assert np.array_equal(h0, m.embed[tokens])
        pos = _buf(fa, be, dec, POS, np.int32, B)
        slots = _buf(fa, be, dec, SLOTS, np.uint32, B)
        assert np.array_equal(pos, lens.astype(np.int32))
        bs = m.cfg["block_size"]
        want_slots = np.array([m.tables[b, lens[b] // bs] * bs + lens[b] % bs for b in range(B)], dtype=np.uint32)
        assert np.array_equal(slots, want_slots)
        assert np.array_equal(dec.seq_lens(), lens + 1)
        cs = _buf(fa, be, dec, COS_SIN, np.float32, B * DH).reshape(B, DH)
        inv = 500000.0 ** (-2.0 * np.arange(DH // 2, dtype=np.float64) / DH)
        ang = lens.astype(np.float64)[:, None] * inv[None, :]
        want_cs = np.concatenate([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32)
        assert_parity("STAGE_PARITY", "cos_sin", cs, want_cs)

        # ---- stage 1: attention norm + per-token quantizer
        run_until(1)
        xq1 = _untile(_buf(fa, be, dec, XQ, np.int8, 32 * D), B, D)
        sx1 = _buf(fa, be, dec, SX, np.float32, B)
        want_q, want_s = o.quantize_rows_i8(_norm(h0, L["attn_norm"]))
        assert np.array_equal(sx1, want_s) and np.array_equal(xq1, want_q)

        # ---- stage 2: qkv projection + RoPE + cache append
        kp0, vp0 = L["k_pool"].copy(), L["v_pool"].copy()
        run_until(2)
        q_bf = _buf(fa, be, dec, QBF, np.uint16, B * EQ).reshape(B, EQ)
        kp, vp = dec.kv_pool(0)
        acc = o.gemm_i8_i32(xq1, L["wqkv"][0])
        qkv = o.dequant_i32(acc, sx1, L["wqkv"][1])
        q_f, k_f, v_f = qkv[:, :EQ], qkv[:, EQ:EQ + EKV], qkv[:, EQ + EKV:]
        want_q_bf = o.to_bf16(o.rope_f32(np.ascontiguousarray(q_f).reshape(B, NH, DH), pos, 500000.0)).reshape(B, EQ)
        want_k_bf = o.to_bf16(o.rope_f32(np.ascontiguousarray(k_f).reshape(B, NKV, DH), pos, 500000.0)).reshape(B, EKV)
        want_v_bf = o.to_bf16(np.ascontiguousarray(v_f))
        kp_rows, vp_rows = kp.reshape(-1, EKV)[slots], vp.reshape(-1, EKV)[slots]
        # V is an exact function of the accumulators: bit-exact
        assert np.array_equal(vp_rows, want_v_bf)
        for name, got, want in (("q", q_bf, want_q_bf), ("k", kp_rows, want_k_bf)):
            diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
            print("STAGE_PARITY\trope %s\tbf16 mismatches %d of %d" % (name, int((diff != 0).sum()), diff.size), flush=True)
            assert diff.max() <= 1 and (diff != 0).mean() < 2e-3, name
        # nothing but the appended rows changed
        untouched = np.ones(kp.shape[0] * kp.shape[1], bool)
        untouched[slots] = False
        assert np.array_equal(kp.reshape(-1, EKV)[untouched], kp0.reshape(-1, EKV)[untouched])
        assert np.array_equal(vp.reshape(-1, EKV)[untouched], vp0.reshape(-1, EKV)[untouched])

        # ---- stage 3: paged attention + merge + quantizer of the o projection's input
        run_until(3)
        xq3 = _untile(_buf(fa, be, dec, XQ, np.int8, 32 * EQ), B, EQ)
        sx3 = _buf(fa, be, dec, SX, np.float32, B)
        oargs = o.paged_args(m.cfg["num_blocks"], bs, EKV, B, 1, NH, m.cfg["max_blocks_per_seq"],
                             float(np.float32(1.0) / np.sqrt(np.float32(DH))), NKV)
        rc, attn = o.paged_attention_bf16(q_bf.reshape(B, 1, EQ), kp, vp, m.tables, lens + 1, oargs)
        assert rc == 0
        attn = attn.reshape(B, EQ)
        # the operator by itself on the same device state: composite tolerance
        kbuf, vbuf = fa.capi.buf_p(), fa.capi.buf_p()
        fa.check(lib.fa_decoder_kv_pools(dec.h, 0, C.byref(kbuf), C.byref(vbuf)))
        layout = fa.PagedKvLayout.new(m.cfg["num_blocks"], bs, EKV)
        args = fa.PagedAttentionArgs(layout, B, 1, NH, m.cfg["max_blocks_per_seq"], fa.default_scale(DH), NKV)
        out = be.alloc_uninit((B, 1, EQ), fa.capi.F32)
        dq, dt, dl = be.upload(q_bf.reshape(B, 1, EQ)), be.upload(m.tables), be.upload(lens + 1)
        fa.check(lib.fa_paged_attention_forward_device(be._ctx, dq._h, kbuf, vbuf, dt._h, dl._h, C.byref(args.c()), out._h))
        assert_parity("STAGE_PARITY", "attention", be.download(out).reshape(B, EQ), attn)
        # the fused stage: codes under its own scale are a round-to-nearest quantization of a value within the
        # tolerance (plus the one bf16 rounding of the attention output) of the oracle's output
        deq = xq3.astype(np.float32) * sx3[:, None]
        slack = sx3[:, None] * 0.5 * (1 + 1e-6) + np.maximum(1e-3 * np.abs(attn), 1e-5) + np.abs(attn) * 2.0 ** -8
        assert np.all(np.abs(deq - attn) <= slack)
        _, want_s3 = o.quantize_rows_i8(o.from_bf16(o.to_bf16(attn)))
        assert np.all(np.abs(sx3 - want_s3) <= 1e-3 * want_s3 + 2.0 ** -8 * want_s3)
        assert np.abs(xq3).max(axis=1).min() == 127              # every row uses its full range

        # ---- stage 4: o projection + residual (exact function of the accumulators)
        run_until(4)
        h4 = _buf(fa, be, dec, H, np.float32, B * D).reshape(B, D)
        want_h4 = o.dequant_i32(o.gemm_i8_i32(xq3, L["wo"][0]), sx3, L["wo"][1])
        want_h4 = (h0 + want_h4).astype(np.float32)
        assert np.array_equal(h4, want_h4)

        # ---- stage 5: ffn norm + quantizer
        run_until(5)
        xq5 = _untile(_buf(fa, be, dec, XQ, np.int8, 32 * D), B, D)
        sx5 = _buf(fa, be, dec, SX, np.float32, B)
        want_q, want_s = o.quantize_rows_i8(_norm(h4, L["ffn_norm"]))
        assert np.array_equal(sx5, want_s) and np.array_equal(xq5, want_q)

        # ---- stage 6: gate / up projection + SwiGLU
        run_until(6)
        act = _buf(fa, be, dec, ACT, np.float32, B * F).reshape(B, F)
        pmax = _buf(fa, be, dec, PMAX, np.float32, B * (F // 16)).reshape(B, F // 16)
        gu = o.dequant_i32(o.gemm_i8_i32(xq5, L["wgu"][0]), sx5, L["wgu"][1])
        want_act = o.silu_mul_f32(np.ascontiguousarray(gu[:, :F]), np.ascontiguousarray(gu[:, F:]))
        assert_parity("STAGE_PARITY", "swiglu", act, want_act)
        assert np.array_equal(pmax, np.abs(act).reshape(B, F // 16, 16).max(axis=2))

        # ---- stage 7: quantizer of the down projection's input
        run_until(7)
        xq7 = _untile(_buf(fa, be, dec, XQ, np.int8, 32 * F), B, F)
        sx7 = _buf(fa, be, dec, SX, np.float32, B)
        want_q, want_s = o.quantize_rows_i8(act)
        assert np.array_equal(sx7, want_s) and np.array_equal(xq7, want_q)

        # ---- stage 8: down projection + residual
        run_until(8)
        h8 = _buf(fa, be, dec, H, np.float32, B * D).reshape(B, D)
        want_h8 = (h4 + o.dequant_i32(o.gemm_i8_i32(xq7, L["wdown"][0]), sx7, L["wdown"][1])).astype(np.float32)
        assert np.array_equal(h8, want_h8)

        # ---- stages 9 - 11: final norm + quantizer, head, pick
        run_until(9)
        xq9 = _untile(_buf(fa, be, dec, XQ, np.int8, 32 * D), B, D)
        sx9 = _buf(fa, be, dec, SX, np.float32, B)
        want_q, want_s = o.quantize_rows_i8(_norm(h8, m.final_norm))
        assert np.array_equal(sx9, want_s) and np.array_equal(xq9, want_q)
        run_until(10)
        logits = _buf(fa, be, dec, LOGITS, np.float32, B * V).reshape(B, V)
        assert np.array_equal(logits, o.dequant_i32(o.gemm_i8_i32(xq9, m.lm[0]), sx9, m.lm[1]))
        run_until(11)
        assert np.array_equal(dec.tokens(), o.argmax_rows(logits))
        # the staged run is the step: a whole step from the same state ends with the same logits and tokens
        dec.set_state(lens, tokens)
        dec.step(False)
        assert np.array_equal(dec.logits(), logits) and np.array_equal(dec.tokens(), o.argmax_rows(logits))
    finally:
        o.set_threads(1)
        dec.close()
