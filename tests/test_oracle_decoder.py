"""The oracle's decode step is a composition of pinned operators; these checks
pin the composition itself: where K/V land, how lengths advance, and the
logits against an independent numpy float64 statement of the same model in
which only the int8 rounding of activations is shared."""
import numpy as np

import oracle_lib as o
from decoder_common import build_model, oracle_step


def _f64_step(m, seq_lens, tokens):
    c = m.cfg
    H, HKV, DH, F = c["n_heads"], c["n_kv_heads"], c["head_dim"], c["d_ffn"]
    EQ, EKV, bs = H * DH, HKV * DH, c["block_size"]

    def rms(x, w):
        inv_n = float(np.float32(1.0) / np.float32(x.shape[1]))
        r = 1.0 / np.sqrt((x * x).sum(axis=1) * inv_n + float(np.float32(c["rms_eps"])))
        return x * r[:, None] * w[None, :]

    def qlin(x, pair):
        q, s = o.quantize_rows_i8(x.astype(np.float32))
        return (q.astype(np.float64) @ pair[0].astype(np.float64)) * (s.astype(np.float64)[:, None] * pair[1].astype(np.float64)[None, :])

    def rope(x, heads):
        x = x.reshape(len(tokens), heads, DH)
        i = np.arange(DH // 2)
        ang = seq_lens.astype(np.float64)[:, None] * (c["rope_theta"] ** (-2.0 * i / DH))[None, :]
        cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        out = np.concatenate([x[..., :DH // 2] * cs - x[..., DH // 2:] * sn, x[..., DH // 2:] * cs + x[..., :DH // 2] * sn], -1)
        return out.reshape(len(tokens), heads * DH)

    h = m.embed[tokens].astype(np.float64)
    for L in m.layers:
        qkv = qlin(rms(h, L["attn_norm"]), L["wqkv"])
        q, k, v = rope(qkv[:, :EQ], H), rope(qkv[:, EQ:EQ + EKV], HKV), qkv[:, EQ + EKV:]
        attn = np.zeros((len(tokens), EQ))
        for b in range(len(tokens)):
            n = int(seq_lens[b])
            rows = [m.tables[b, j // bs] * bs + j % bs for j in range(n)]
            K = np.vstack([o.from_bf16(L["k_pool"].reshape(-1, EKV)[rows]).astype(np.float64), o.from_bf16(o.to_bf16(k[b:b + 1].astype(np.float32)))])
            V = np.vstack([o.from_bf16(L["v_pool"].reshape(-1, EKV)[rows]).astype(np.float64), o.from_bf16(o.to_bf16(v[b:b + 1].astype(np.float32)))])
            qb = o.from_bf16(o.to_bf16(q[b].astype(np.float32))).astype(np.float64)
            for hh in range(H):
                g = hh // (H // HKV)
                s = K[:, g * DH:(g + 1) * DH] @ qb[hh * DH:(hh + 1) * DH] / np.sqrt(DH)
                p = np.exp(s - s.max())
                attn[b, hh * DH:(hh + 1) * DH] = (p / p.sum()) @ V[:, g * DH:(g + 1) * DH]
        attn = o.from_bf16(o.to_bf16(attn.astype(np.float32))).astype(np.float64)
        h = h + qlin(attn, L["wo"])
        gu = qlin(rms(h, L["ffn_norm"]), L["wgu"])
        act = gu[:, :F] / (1.0 + np.exp(-gu[:, :F])) * gu[:, F:]
        h = h + qlin(act, L["wdown"])
    return qlin(rms(h, m.final_norm), m.lm)


def test_decode_step_composition():
    m = build_model(seed=3, n_layers=2, d_model=128, n_heads=2, n_kv_heads=1, d_ffn=192, vocab=300, batch=3,
                    ctxs=[5, 16, 33], steps=2, threads=2)
    lens = m.seq_lens.copy()
    want_logits = _f64_step(m, lens, m.tokens)
    pools_before = [(L["k_pool"].copy(), L["v_pool"].copy()) for L in m.layers]
    nxt, logits = oracle_step(m, lens, m.tokens, threads=2)
    assert lens.tolist() == [6, 17, 34]
    # the quantizer is discontinuous, so the f64 restatement can differ by a code here and there;
    # the logits still agree to a fraction of their spread
    assert np.abs(logits - want_logits).max() < 2e-2 * np.abs(want_logits).max()
    assert (nxt == want_logits.argmax(axis=1)).mean() >= 2 / 3
    assert np.array_equal(nxt, o.argmax_rows(logits))
    # exactly one new row per sequence and layer, at slot table[pos / bs] * bs + pos % bs
    for (kb, vb), L in zip(pools_before, m.layers):
        changed = np.argwhere((L["k_pool"] != kb).any(axis=2))
        want = sorted((int(m.tables[b, p // 16]), p % 16) for b, p in enumerate([5, 16, 33]))
        assert sorted(map(tuple, changed.tolist())) == want
        assert sorted(map(tuple, np.argwhere((L["v_pool"] != vb).any(axis=2)).tolist())) == want
    # deterministic, and a second step consumes the first one's state
    m2 = build_model(seed=3, n_layers=2, d_model=128, n_heads=2, n_kv_heads=1, d_ffn=192, vocab=300, batch=3,
                     ctxs=[5, 16, 33], steps=2, threads=1)
    lens2 = m2.seq_lens.copy()
    nxt2, logits2 = oracle_step(m2, lens2, m2.tokens, threads=1)
    assert np.array_equal(logits, logits2) and np.array_equal(nxt, nxt2)
    nxt3, _ = oracle_step(m, lens, nxt, threads=2)
    assert lens.tolist() == [7, 18, 35] and nxt3.shape == (3,)
