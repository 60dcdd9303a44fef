"""Pins the oracle's paged-KV validators, append and attention.

Validator tables are the reference's own unit tests
(crates/tensor-core/src/paged_kv.rs:387-521); attention is pinned by an f64
brute force written with a different loop structure, by closed-form special
cases and by invariances (block-table permutation, page size, GQA with one
group == MHA).
"""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as o

U32MAX = 0xFFFFFFFF


def _layout(nb=4, bs=2, e=4):
    return o.PagedLayout(nb, bs, e)


def _args(batch, l_new, max_blocks, heads=2, scale=0.5, layout=None):
    return o.PagedArgs(layout or _layout(), batch, l_new, heads, max_blocks, scale, 0)


def _val_append(kn, vn, kp, vp, slots, layout):
    s = np.array(slots, dtype=np.uint32)
    return o.lib.orc_validate_paged_kv_append(kn, vn, kp, vp, o.ptr(s, o.u32p), s.size, C.byref(layout))


def _val_attn(qn, kp, vp, tables, lens, args):
    t = np.array(tables, dtype=np.uint32)
    s = np.array(lens, dtype=np.uint32)
    plan = o.PagedPlan()
    rc = o.lib.orc_validate_paged_attention(qn, kp, vp, o.ptr(t, o.u32p), t.size, o.ptr(s, o.u32p), s.size,
                                            C.byref(args), C.byref(plan))
    return rc, plan


def test_layout_rejects_invalid_values():
    # paged_kv.rs:387-397
    chk = lambda *a: o.lib.orc_paged_layout_check(C.byref(o.PagedLayout(*a)))
    assert chk(0, 2, 4) != 0 and chk(4, 3, 4) != 0 and chk(4, 512, 4) != 0 and chk(4, 2, 0) != 0
    assert chk(U32MAX, 2, 4) != 0
    assert chk(4, 2, (1 << 64) - 1) != 0
    assert chk(1 << 20, 256, ((1 << 63) - 1) // (8 * 256) + 1) != 0
    assert chk(4, 256, 4) == 0


def test_args_reject_bad_heads_scale_and_sizes():
    # paged_kv.rs:399-408
    chk = lambda *a: o.lib.orc_paged_args_check(C.byref(o.PagedArgs(_layout(), *a)))
    assert chk(1, 1, 0, 2, 1.0, 0) != 0
    assert chk(1, 1, 3, 2, 1.0, 0) != 0
    assert chk(1, 1, 2, 2, float("nan"), 0) != 0
    assert chk(1, 1, 2, 2, float("inf"), 0) != 0
    assert chk((1 << 64) - 1, 1, 2, 2, 1.0, 0) != 0
    assert chk(1, 1, 2, 2, 1.0, 0) == 0
    # GQA extension: query heads must be a multiple of the kv heads, kv heads divide E_kv
    assert chk(1, 1, 8, 2, 1.0, 2) == 0 and chk(1, 1, 3, 2, 1.0, 2) != 0 and chk(1, 1, 6, 2, 1.0, 3) != 0


def test_append_accepts_valid_and_rejects_violations():
    # paged_kv.rs:410-435
    l, pool = _layout(), 4 * 2 * 4
    assert _val_append(8, 8, pool, pool, [0, 7], l) == 2
    assert _val_append(7, 8, pool, pool, [0, 7], l) < 0
    assert _val_append(8, 4, pool, pool, [0, 7], l) < 0
    assert _val_append(8, 8, pool - 1, pool, [0, 7], l) < 0
    assert _val_append(8, 8, pool, pool, [0, 8], l) < 0
    assert _val_append(4, 4, pool, pool, [U32MAX], l) < 0
    assert _val_append(8, 8, pool, pool, [3, 3], l) < 0
    assert _val_append(0, 0, pool, pool, [], l) == 0


def test_attention_plan_and_violations():
    # paged_kv.rs:437-474
    rc, plan = _val_attn(8, 32, 32, [0, 1, 2, 3], [3, 3], _args(2, 1, 2))
    assert rc == 0 and (plan.out_numel, plan.s_max, plan.query_rows, plan.workspace_elems) == (8, 3, 4, 12)
    a = _args(1, 2, 2)
    ok = [0, 1]
    assert _val_attn(8, 32, 32, ok, [3], a)[0] == 0
    assert _val_attn(7, 32, 32, ok, [3], a)[0] != 0
    assert _val_attn(8, 31, 32, ok, [3], a)[0] != 0
    assert _val_attn(8, 32, 32, [0], [3], a)[0] != 0
    assert _val_attn(8, 32, 32, ok, [3, 3], a)[0] != 0
    assert _val_attn(8, 32, 32, ok, [1], a)[0] != 0
    assert _val_attn(8, 32, 32, ok, [5], a)[0] != 0
    assert _val_attn(8, 32, 32, [0, 4], [3], a)[0] != 0
    assert _val_attn(8, 32, 32, [0, U32MAX], [3], a)[0] != 0
    assert _val_attn(8, 32, 32, [0, U32MAX], [2], a)[0] == 0


def test_attention_workspace_cap_mutated_fields_and_empty():
    # paged_kv.rs:476-521
    big = o.PagedArgs(_layout(), 1 << 20, 1 << 10, 1, 2, 1.0, 0)
    t = np.zeros((1 << 20) * 2, dtype=np.uint32)
    s = np.full(1 << 20, 2, dtype=np.uint32)
    plan = o.PagedPlan()
    assert o.lib.orc_validate_paged_attention((1 << 20) * (1 << 10) * 4, 32, 32, o.ptr(t, o.u32p), t.size,
                                              o.ptr(s, o.u32p), s.size, C.byref(big), C.byref(plan)) != 0
    a = _args(1, 1, 2)
    a.num_heads = 0
    assert _val_attn(4, 32, 32, [0, 1], [2], a)[0] != 0
    a = _args(1, 1, 2)
    a.layout.block_size = 0
    assert _val_attn(4, 32, 32, [0, 1], [2], a)[0] != 0
    l = _layout()
    l.block_size = 0
    assert _val_append(0, 0, 32, 32, [], l) < 0
    rc, plan = _val_attn(0, 32, 32, [], [], _args(0, 1, 2))
    assert rc == 0 and plan.out_numel == 0 and plan.workspace_elems == 0
    rc, plan = _val_attn(0, 32, 32, [0, 1], [3], _args(1, 0, 2))
    assert rc == 0 and plan.out_numel == 0 and plan.workspace_elems == 0


# ------------------------------------------------------------ append / attention
def _build_case(rng, batch, heads, kv_heads, dh, bs, ctxs, l_new=1, num_blocks=None, amp=1.0):
    e_kv, e_q = kv_heads * dh, heads * dh
    max_blocks = max((c + bs - 1) // bs for c in ctxs) + 1
    need = sum((c + bs - 1) // bs for c in ctxs)
    num_blocks = num_blocks or need + 3
    ids = rng.permutation(num_blocks)[:need].astype(np.uint32)
    tables = np.full((batch, max_blocks), U32MAX, dtype=np.uint32)
    pos = 0
    for b, c in enumerate(ctxs):
        nblk = (c + bs - 1) // bs
        tables[b, :nblk] = ids[pos:pos + nblk]
        pos += nblk
    k_pool = (rng.normal(size=(num_blocks, bs, e_kv)) * amp).astype(np.float32)
    v_pool = (rng.normal(size=(num_blocks, bs, e_kv)) * amp).astype(np.float32)
    q = (rng.normal(size=(batch, l_new, e_q)) * amp).astype(np.float32)
    lens = np.array(ctxs, dtype=np.uint32)
    args = o.paged_args(num_blocks, bs, e_kv, batch, l_new, heads, max_blocks,
                        float(np.float32(1.0) / np.sqrt(np.float32(dh))), kv_heads)
    return q, k_pool, v_pool, tables, lens, args


def test_append_is_a_bit_exact_row_scatter():
    rng = np.random.default_rng(0)
    l = o.PagedLayout(5, 4, 6)
    for dtype in (np.float32, np.uint16):
        kp = np.zeros((20, 6), dtype=dtype)
        vp = np.zeros((20, 6), dtype=dtype)
        kn = rng.integers(1, 60000, size=(3, 6)).astype(dtype)
        vn = rng.integers(1, 60000, size=(3, 6)).astype(dtype)
        assert o.paged_kv_append(kn, vn, kp, vp, [17, 0, 9], l) == 0
        assert np.array_equal(kp[[17, 0, 9]], kn) and np.array_equal(vp[[17, 0, 9]], vn)
        untouched = np.ones(20, bool)
        untouched[[17, 0, 9]] = False
        assert not kp[untouched].any() and not vp[untouched].any()
    assert o.paged_kv_append(kn, vn, kp, vp, [20, 0, 9], l) != 0


@pytest.mark.parametrize("bs,batch,embed,heads,ctxs,l_new", [
    # shapes of the reference's matrix (backend-cuda/tests/common/paged_attention_judgement.rs:58-97)
    (1, 1, 8, 2, [5], 1), (4, 2, 16, 2, [11, 11], 4), (16, 1, 64, 4, [19], 1), (16, 3, 48, 3, [32, 32, 32], 15),
    (16, 2, 16, 2, [15, 15], 1), (16, 2, 16, 2, [16, 16], 1), (16, 2, 16, 2, [17, 17], 1),
    (256, 2, 16, 2, [257, 257], 1), (16, 2, 32, 2, [301, 301], 1), (16, 1, 160, 1, [7], 1),
    (4, 2, 4, 4, [8, 8], 1), (4, 2, 16, 2, [13, 13], 5),
])
def test_attention_f32_matches_f64_brute_force_on_reference_shapes(bs, batch, embed, heads, ctxs, l_new):
    rng = np.random.default_rng(bs * 1000 + embed)
    q, kp, vp, tables, lens, args = _build_case(rng, batch, heads, heads, embed // heads, bs, ctxs, l_new)
    rc, got = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    assert rc == 0
    rc, want = o.paged_attention_f64(q.astype(np.float64), kp.astype(np.float64), vp.astype(np.float64),
                                     tables, lens, args)
    assert rc == 0
    r = o.compare(got, want)
    assert r.fail_count == 0, r.line("ORACLE_PAGED", f"bs{bs}")


def test_attention_numpy_softmax_restatement_with_causal_offset():
    # independent numpy statement of `j <= s_prev + i` (backend-cpu/src/paged_kv.rs:131)
    rng = np.random.default_rng(11)
    q, kp, vp, tables, lens, args = _build_case(rng, 2, 2, 2, 8, 4, [9, 9], l_new=3)
    rc, got = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    assert rc == 0
    for b in range(2):
        rows = np.array([tables[b, j // 4] * 4 + j % 4 for j in range(9)])
        K = kp.reshape(-1, 16)[rows].astype(np.float64)
        V = vp.reshape(-1, 16)[rows].astype(np.float64)
        for h in range(2):
            sl = slice(h * 8, (h + 1) * 8)
            for i in range(3):
                lim = 9 - 3 + i + 1
                s = (K[:lim, sl] @ q[b, i, sl].astype(np.float64)) * float(args.scale)
                p = np.exp(s - s.max())
                p /= p.sum()
                assert np.allclose(got[b, i, sl], p @ V[:lim, sl], rtol=1e-5, atol=1e-6)


def test_attention_special_cases_and_invariances():
    rng = np.random.default_rng(12)
    # context 1: the output is the V row (crates/backend-cuda/tests/paged_kv_real_device.rs:180)
    q, kp, vp, tables, lens, args = _build_case(rng, 3, 4, 2, 8, 16, [1, 1, 1])
    rc, got = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    assert rc == 0
    for b in range(3):
        vrow = vp[tables[b, 0], 0]                                   # [E_kv]
        for h in range(4):
            assert np.array_equal(got[b, 0, h * 8:(h + 1) * 8], vrow[(h // 2) * 8:(h // 2 + 1) * 8])
    # identical K rows: uniform weights, output = mean of V rows
    q, kp, vp, tables, lens, args = _build_case(rng, 1, 2, 2, 4, 4, [8])
    kp[:] = 0.25
    rc, got = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    rows = [tables[0, j // 4] * 4 + j % 4 for j in range(8)]
    assert np.allclose(got[0, 0], vp.reshape(-1, 8)[rows].mean(axis=0), rtol=1e-6, atol=1e-7)
    # block-table permutation invariance: move the pages, keep the logical order -> same bits
    q, kp, vp, tables, lens, args = _build_case(rng, 2, 4, 2, 8, 4, [13, 6], num_blocks=12)
    rc, base = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    perm = rng.permutation(12).astype(np.uint32)
    kp2, vp2 = np.empty_like(kp), np.empty_like(vp)
    kp2[perm], vp2[perm] = kp, vp
    t2 = tables.copy()
    used = tables != U32MAX
    t2[used] = perm[tables[used]]
    rc, moved = o.paged_attention_f32(q, kp2, vp2, t2, lens, args)
    assert np.array_equal(base, moved)
    # page size independence: regroup the same logical rows into pages of 2 and of 8
    outs = []
    for bs in (2, 8):
        nb = 40
        kpp = np.zeros((nb, bs, 16), np.float32)
        vpp = np.zeros((nb, bs, 16), np.float32)
        mb = 13 // bs + 2
        tt = np.full((2, mb), U32MAX, np.uint32)
        nxt = 0
        for b, c in enumerate([13, 6]):
            for j in range(c):
                if j % bs == 0:
                    tt[b, j // bs] = nxt
                    nxt += 1
                src = tables[b, j // 4] * 4 + j % 4
                kpp[tt[b, j // bs], j % bs] = kp.reshape(-1, 16)[src]
                vpp[tt[b, j // bs], j % bs] = vp.reshape(-1, 16)[src]
        a2 = o.paged_args(nb, bs, 16, 2, 1, 4, mb, args.scale, 2)
        rc, out = o.paged_attention_f32(q, kpp, vpp, tt, lens, a2)
        assert rc == 0
        outs.append(out)
    assert np.array_equal(outs[0], base) and np.array_equal(outs[1], base)
    # GQA with a group of one == MHA (num_kv_heads == num_heads vs the 0 default)
    q, kp, vp, tables, lens, args = _build_case(rng, 2, 3, 3, 4, 2, [5, 4])
    rc, a1 = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    args.num_kv_heads = 0
    rc, a0 = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    assert np.array_equal(a0, a1)
    # GQA == MHA on K/V with each kv head repeated `group` times
    q, kp, vp, tables, lens, args = _build_case(rng, 2, 4, 2, 4, 2, [5, 4])
    rc, g = o.paged_attention_f32(q, kp, vp, tables, lens, args)
    rep = lambda p: np.ascontiguousarray(np.repeat(p.reshape(p.shape[0], p.shape[1], 2, 4), 2, axis=2).reshape(p.shape[0], p.shape[1], 16))
    margs = o.paged_args(args.layout.num_blocks, 2, 16, 2, 1, 4, args.max_blocks_per_seq, args.scale, 0)
    rc, m = o.paged_attention_f32(q, rep(kp), rep(vp), tables, lens, margs)
    assert rc == 0 and np.array_equal(g, m)


def test_attention_bf16_is_the_f32_algorithm_on_promoted_inputs():
    rng = np.random.default_rng(13)
    q, kp, vp, tables, lens, args = _build_case(rng, 2, 8, 2, 16, 16, [40, 17])
    qb, kb, vb = o.to_bf16(q), o.to_bf16(kp), o.to_bf16(vp)
    rc, got = o.paged_attention_bf16(qb, kb, vb, tables, lens, args)
    assert rc == 0
    rc, want = o.paged_attention_f32(o.from_bf16(qb), o.from_bf16(kb), o.from_bf16(vb), tables, lens, args)
    assert np.array_equal(got, want)
    # out-of-range block id inside the used range is an error, not a silent zero
    bad = tables.copy()
    bad[0, 1] = args.layout.num_blocks
    assert o.paged_attention_bf16(qb, kb, vb, bad, lens, args)[0] != 0


def test_threads_do_not_change_results():
    rng = np.random.default_rng(14)
    q, kp, vp, tables, lens, args = _build_case(rng, 3, 4, 2, 8, 4, [13, 6, 9])
    a = rng.normal(size=(6, 40)).astype(np.float32)
    b = rng.normal(size=(40, 9)).astype(np.float32)
    o.set_threads(1)
    r1 = o.paged_attention_f32(q, kp, vp, tables, lens, args)[1]
    g1 = o.gemm_f32(a, b)
    o.set_threads(4)
    r4 = o.paged_attention_f32(q, kp, vp, tables, lens, args)[1]
    g4 = o.gemm_f32(a, b)
    o.set_threads(1)
    assert np.array_equal(r1, r4) and np.array_equal(g1, g4)
