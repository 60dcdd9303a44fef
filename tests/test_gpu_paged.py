"""GPU parity of paged-KV append and attention, through the C ABI.

The f32 / MHA path is checked on the reference's own shape matrix
(crates/backend-cuda/tests/common/paged_attention_judgement.rs:58-97,
crates/backend-cpu/tests/paged_kv_backend_parity.rs:84-122) driven step by
step (append -> attention) with non-contiguous block ids and sentinel entries
(crates/backend-rocm/src/ops/paged_kv.rs:277-328).  The bf16 grouped-query
decode path is checked against the oracle at reduced size, at the benchmark's
full size on sampled sequences, and through size-independent properties.
"""
from math import gcd

import numpy as np
import pytest

import oracle_lib as o
from gpu_common import assert_bf16_rounding_of, assert_parity, ops

pytestmark = pytest.mark.gpu
U32MAX = 0xFFFFFFFF


def _fa():
    import fandhe_ai_amd as fa
    return fa


def _data(shape, seed):
    out = np.empty(shape, dtype=np.float32)
    o.lib.orc_test_data_f32(o.ptr(out, o.f32p), out.size, seed)
    return out


# (id, block_size, batch, embed, heads, steps, input_scale)
CASES = [
    ("legacy_bs1_b1", 1, 1, 8, 2, [3, 1, 1], 1.0), ("legacy_bs4_b2", 4, 2, 16, 2, [5, 1, 1, 4], 1.0),
    ("legacy_bs16_b1", 16, 1, 64, 4, [17, 1, 1], 1.0), ("legacy_bs16_b3", 16, 3, 48, 3, [16, 1, 15], 1.0),
    ("bs1_prefill1", 1, 2, 16, 2, [1, 1, 1], 1.0), ("bs1_prefill2", 1, 2, 16, 2, [2, 1, 1], 1.0),
    ("bs2_prefill1", 2, 2, 16, 2, [1, 1, 1], 1.0), ("bs2_prefill2", 2, 2, 16, 2, [2, 1, 1], 1.0),
    ("bs2_prefill3", 2, 2, 16, 2, [3, 1, 1], 1.0), ("bs16_prefill15", 16, 2, 16, 2, [15, 1, 1], 1.0),
    ("bs16_prefill16", 16, 2, 16, 2, [16, 1, 1], 1.0), ("bs16_prefill17", 16, 2, 16, 2, [17, 1, 1], 1.0),
    ("bs256_prefill255", 256, 2, 16, 2, [255, 1, 1], 1.0), ("bs256_prefill256", 256, 2, 16, 2, [256, 1, 1], 1.0),
    ("bs256_prefill257", 256, 2, 16, 2, [257, 1, 1], 1.0), ("long_bs16_s301", 16, 2, 32, 2, [100, 100, 100, 1], 1.0),
    ("dh160_h1", 16, 1, 160, 1, [5, 1, 1], 1.0), ("dh1_e4_h4", 4, 2, 4, 4, [6, 1, 1], 1.0),
    ("multi_prefill_bs4", 4, 2, 16, 2, [3, 4, 5, 1], 1.0), ("large_amplitude", 16, 2, 32, 2, [17, 1, 1], 4.0),
    # crates/backend-cpu/tests/paged_kv_backend_parity.rs:86-93
    ("cpu_bs2", 2, 3, 4, 1, [3, 1, 1, 2], 1.0), ("cpu_bs4_long", 4, 2, 12, 3, [3, 1, 1, 1, 1, 5], 1.0),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_f32_append_then_attention_matches_the_reference_algorithm(case):
    fa = _fa()
    be = ops()
    cid, bs, batch, embed, heads, steps, amp = case
    max_blocks = (sum(steps) + bs - 1) // bs
    num_blocks = batch * max_blocks + 3
    stride = next(s for s in range(num_blocks - 1, 0, -1) if gcd(s, num_blocks) == 1)
    id_of = lambda b, slot: ((b * max_blocks + slot) * stride) % num_blocks
    layout = fa.PagedKvLayout.new(num_blocks, bs, embed)
    k_pool, v_pool = be.alloc_zeroed((num_blocks, bs, embed)), be.alloc_zeroed((num_blocks, bs, embed))
    hk = np.zeros((num_blocks * bs, embed), np.float32)
    hv = np.zeros((num_blocks * bs, embed), np.float32)
    scale = fa.default_scale(embed // heads)
    seq = 0
    for si, l in enumerate(steps):
        k = _data((batch, l, embed), 10 + si) * amp
        v = _data((batch, l, embed), 1010 + si) * amp
        q = _data((batch, l, embed), 2010 + si) * amp
        slots = [id_of(b, (seq + i) // bs) * bs + (seq + i) % bs for b in range(batch) for i in range(l)]
        seq += l
        used = (seq + bs - 1) // bs
        tables = np.array([[id_of(b, s) if s < used else U32MAX for s in range(max_blocks)] for b in range(batch)],
                          dtype=np.uint32)
        lens = np.full(batch, seq, dtype=np.uint32)
        be.paged_kv_append(be.upload(k.reshape(-1, embed)), be.upload(v.reshape(-1, embed)), k_pool, v_pool, slots, layout)
        assert o.paged_kv_append(k.reshape(-1, embed), v.reshape(-1, embed), hk, hv, slots, o.PagedLayout(num_blocks, bs, embed)) == 0
        assert np.array_equal(be.download(k_pool).reshape(-1, embed), hk)          # append is a bit-exact copy
        assert np.array_equal(be.download(v_pool).reshape(-1, embed), hv)
        args = fa.PagedAttentionArgs(layout, batch, l, heads, max_blocks, scale)
        got = be.download_owned(be.paged_attention_forward(be.upload(q), k_pool, v_pool, tables, lens, args))
        oargs = o.paged_args(num_blocks, bs, embed, batch, l, heads, max_blocks, scale, 0)
        rc, want = o.paged_attention_f32(q, hk.reshape(num_blocks, bs, embed), hv.reshape(num_blocks, bs, embed),
                                         tables, lens, oargs)
        assert rc == 0
        assert_parity("PAGED_PARITY", f"{cid}:step{si}", got, want)


def test_validation_errors_leave_the_pools_untouched():
    """crates/backend-rocm/src/ops/paged_kv.rs:418-447: typed errors before any write."""
    fa = _fa()
    be = ops()
    layout = fa.PagedKvLayout.new(4, 2, 4)
    kp, vp = be.alloc_zeroed((4, 2, 4)), be.alloc_zeroed((4, 2, 4))
    new = be.upload(np.ones((2, 4), np.float32))
    for slots in ([0, 8], [3, 3], [U32MAX, 0]):
        with pytest.raises(fa.InvalidArgument):
            be.paged_kv_append(new, new, kp, vp, slots, layout)
    with pytest.raises(fa.InvalidArgument):
        be.paged_kv_append(be.upload(np.ones((3, 4), np.float32)), new, kp, vp, [0, 1], layout)
    assert not be.download(kp).any() and not be.download(vp).any()
    be.paged_kv_append(be.upload(np.zeros((0, 4), np.float32)), be.upload(np.zeros((0, 4), np.float32)), kp, vp, [], layout)
    q = be.upload(np.ones((1, 2, 4), np.float32))
    args = fa.PagedAttentionArgs(layout, 1, 2, 2, 2, 0.5)
    for tables, lens in (([0, 4], [3]), ([0, U32MAX], [3]), ([0, 1], [1]), ([0, 1], [5]), ([0], [3])):
        with pytest.raises(fa.InvalidArgument):
            be.paged_attention_forward(q, kp, vp, tables, lens, args)
    out = be.paged_attention_forward(q, kp, vp, [0, U32MAX], [2], args)          # sentinel outside the used range
    assert np.all(np.isfinite(be.download(out)))
    for bad in ((0, 2, 4), (4, 3, 4), (4, 512, 4), (4, 2, 0), (U32MAX, 2, 4)):
        with pytest.raises(fa.InvalidArgument):
            fa.PagedKvLayout.new(*bad)
    with pytest.raises(fa.InvalidArgument):
        be.paged_attention_forward(q, kp, vp, [0, 1], [3], fa.PagedAttentionArgs(layout, 1, 2, 3, 2, 0.5))
    with pytest.raises(fa.InvalidArgument):
        be.paged_attention_forward(q, kp, vp, [0, 1], [3], fa.PagedAttentionArgs(layout, 1, 2, 2, 2, float("nan")))
    # mixed element types are rejected
    with pytest.raises(fa.InvalidArgument):
        be.paged_attention_forward(be.upload(np.ones((1, 2, 4), np.uint16)), kp, vp, [0, 1], [3], args)
    # empty batch is valid and launches nothing (crates/tensor-core/src/paged_kv.rs:510-521)
    e = be.paged_attention_forward(be.upload(np.zeros((0, 1, 4), np.float32)), kp, vp, [], [],
                                   fa.PagedAttentionArgs(layout, 0, 1, 2, 2, 0.5))
    assert be.download(e).size == 0


def _decode_case(rng, batch, heads, kv_heads, ctxs, num_blocks, dh=128, bs=16, extra_slots=1):
    e_kv, e_q = kv_heads * dh, heads * dh
    max_blocks = max((c + bs - 1) // bs for c in ctxs) + extra_slots
    need = sum((c + bs - 1) // bs for c in ctxs)
    assert need <= num_blocks
    ids = rng.permutation(num_blocks)[:need]
    tables = np.full((batch, max_blocks), U32MAX, dtype=np.uint32)
    p = 0
    for b, c in enumerate(ctxs):
        nb = (c + bs - 1) // bs
        tables[b, :nb] = ids[p:p + nb]
        p += nb
    return tables, np.array(ctxs, dtype=np.uint32), max_blocks, e_kv, e_q


@pytest.mark.parametrize("heads,kv_heads", [(32, 8), (8, 8), (16, 2), (4, 2)])
def test_bf16_gqa_decode_against_the_oracle(heads, kv_heads):
    fa = _fa()
    be = ops()
    rng = o.Rng(heads * 100 + kv_heads)
    batch, num_blocks = 6, 200
    ctxs = [1, 15, 16, 17, 130, 777]
    tables, lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, ctxs, num_blocks)
    kp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, 1, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    oargs = o.paged_args(num_blocks, 16, e_kv, batch, 1, heads, max_blocks, args.scale, kv_heads)
    o.set_threads(8)
    rc, want = o.paged_attention_bf16(q, kp, vp, tables, lens, oargs)
    o.set_threads(1)
    assert rc == 0
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    for ppc in (0, 1, 2, 8):          # wavefronts per compute unit: ranges of many / few pages
        fa.check(fa.capi.lib.fa_set_tuning(2, ppc))
        got = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, lens, args, out_dtype=fa.capi.F32))
        assert_parity("PAGED_DECODE_PARITY", f"H{heads}/{kv_heads}:waves{ppc}", got, want)
        got_bf = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, lens, args))
        assert_bf16_rounding_of("paged decode bf16", got_bf, got)
    fa.check(fa.capi.lib.fa_set_tuning(2, 0))
    # context 1: the output is the V row of the only token, exactly
    for h in range(heads):
        g = h // (heads // kv_heads)
        assert np.array_equal(got_bf[0, 0, h * 128:(h + 1) * 128], vp[tables[0, 0], 0, g * 128:(g + 1) * 128])
    # device-resident tables give the same bits as host tables (same launch shape)
    got_bf = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, lens, args))
    got_dev = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, be.upload(tables), be.upload(lens), args))
    assert np.array_equal(got_dev, got_bf)


def test_bf16_decode_properties_at_benchmark_size():
    """batch 64, 32 / 8 heads, head_dim 128, page 16, contexts uniform in [128, 4096], block tables a
    seeded permutation of a 40k-page pool; oracle on sampled sequences plus invariances on all."""
    fa = _fa()
    be = ops()
    rng = o.Rng(0)
    batch, heads, kv_heads, num_blocks = 64, 32, 8, 40000
    ctxs = rng.randint(128, 4097, batch).tolist()
    perm = rng.permutation(num_blocks)
    max_blocks = 256
    tables = np.full((batch, max_blocks), U32MAX, dtype=np.uint32)
    p = 0
    for b, c in enumerate(ctxs):
        nb = (c + 15) // 16
        tables[b, :nb] = perm[p:p + nb]
        p += nb
    lens = np.array(ctxs, dtype=np.uint32)
    e_kv, e_q = kv_heads * 128, heads * 128
    # pools are filled page by page to keep host memory modest: only the used pages matter
    kp = np.zeros((num_blocks, 16, e_kv), np.uint16)
    vp = np.zeros((num_blocks, 16, e_kv), np.uint16)
    used = perm[:p]
    kp[used] = o.to_bf16(rng.randn((p, 16, e_kv)))
    vp[used] = o.to_bf16(rng.randn((p, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, 1, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    got = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, lens, args, out_dtype=fa.capi.F32))
    assert np.all(np.isfinite(got))
    # oracle on a sample of sequences (shortest, longest, a few others)
    order = np.argsort(ctxs)
    sample = sorted(set([int(order[0]), int(order[-1]), 3, 17, 40]))
    sub_t = np.ascontiguousarray(tables[sample])
    sub_l = np.ascontiguousarray(lens[sample])
    oargs = o.paged_args(num_blocks, 16, e_kv, len(sample), 1, heads, max_blocks, args.scale, kv_heads)
    o.set_threads(8)
    rc, want = o.paged_attention_bf16(np.ascontiguousarray(q[sample]), kp, vp, sub_t, sub_l, oargs)
    o.set_threads(1)
    assert rc == 0
    assert_parity("PAGED_DECODE_PARITY", "bench:sampled", got[sample], want)
    # other launch shapes (1 and 8 wavefronts per compute unit: ranges of several hundred / a few dozen pages)
    for tune in (1, 8):
        fa.check(fa.capi.lib.fa_set_tuning(2, tune))
        alt = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, lens, args, out_dtype=fa.capi.F32))
        assert_parity("PAGED_DECODE_PARITY", f"bench:sampled:tune{tune}", alt[sample], want)
        assert np.allclose(alt, got, rtol=2e-3, atol=2e-5)
    fa.check(fa.capi.lib.fa_set_tuning(2, 0))
    # every output row is a convex combination of V rows: |out| <= max |V| per dim of its kv head
    vmax = np.abs(o.from_bf16(vp[used])).reshape(-1, kv_heads, 128).max(axis=0)
    assert np.all(np.abs(got.reshape(batch, heads, 128)) <= np.repeat(vmax, heads // kv_heads, axis=0)[None] + 1e-6)
    # block-table permutation invariance: moving pages to other physical blocks changes no bit
    perm2 = np.roll(np.arange(num_blocks), 7).astype(np.uint32)
    kp2, vp2 = np.empty_like(kp), np.empty_like(vp)
    kp2[perm2], vp2[perm2] = kp, vp
    t2 = tables.copy()
    m = tables != U32MAX
    t2[m] = perm2[tables[m]]
    got2 = be.download_owned(be.paged_attention_forward(dq, be.upload(kp2), be.upload(vp2), t2, lens, args,
                                                        out_dtype=fa.capi.F32))
    assert np.array_equal(got, got2)
    # a constant V gives that constant back (softmax weights sum to one)
    ones = np.full_like(vp, o.to_bf16(np.array([1.5], np.float32))[0])
    got3 = be.download_owned(be.paged_attention_forward(dq, dk, be.upload(ones), tables, lens, args,
                                                        out_dtype=fa.capi.F32))
    assert np.allclose(got3, 1.5, rtol=1e-5, atol=0)


PREFILL_CASES = [
    # heads, kv_heads, l_new, total lengths per row (>= l_new)
    (32, 8, 2, [2, 17, 300]), (32, 8, 3, [3, 16, 50]), (32, 8, 4, [4, 20, 33]), (32, 8, 5, [5, 21, 100]),
    (32, 8, 16, [16, 17, 64]), (32, 8, 17, [17, 31, 200]), (32, 8, 37, [37, 38, 500]), (32, 8, 200, [200, 333, 777]),
    (8, 8, 19, [19, 40]), (8, 4, 9, [9, 100]), (16, 2, 11, [11, 64]), (16, 1, 6, [6, 90]), (6, 2, 13, [13, 70]),
    (5, 1, 7, [7, 40]),
    # several tiles of the block form (256 / group new tokens per tile), ragged last tiles
    (32, 8, 300, [300, 1000]), (8, 8, 600, [600, 700]), (16, 2, 100, [100, 250]), (16, 1, 50, [50, 51, 333]),
    (4, 2, 129, [129, 640]),
]


@pytest.mark.parametrize("heads,kv_heads,l_new,lens", PREFILL_CASES,
                         ids=["H%d_%d_L%d" % c[:3] for c in PREFILL_CASES])
def test_bf16_prefill_on_the_streaming_kernel_against_the_oracle(heads, kv_heads, l_new, lens):
    """l_new > 1 with page 16 / head_dim 128: token tiles of 16 / group new tokens on the matrix cores,
    each masked at its own causal limit; rows differ in how much was cached before the new tokens."""
    fa = _fa()
    be = ops()
    rng = o.Rng(1000 * heads + 10 * l_new + kv_heads)
    batch, num_blocks = len(lens), 160
    tables, seq_lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, lens, num_blocks, extra_slots=2)
    kp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, l_new, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    oargs = o.paged_args(num_blocks, 16, e_kv, batch, l_new, heads, max_blocks, args.scale, kv_heads)
    o.set_threads(8)
    rc, want = o.paged_attention_bf16(q, kp, vp, tables, seq_lens, oargs)
    o.set_threads(1)
    assert rc == 0
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    for waves in (0, 1, 8):           # few long ranges / many short ones: different cuts through the token tiles
        fa.check(fa.capi.lib.fa_set_tuning(2, waves))
        got = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
        assert_parity("PAGED_PREFILL_PARITY", f"H{heads}/{kv_heads}:L{l_new}:waves{waves}", got, want)
    fa.check(fa.capi.lib.fa_set_tuning(2, 0))
    # the block form (one block per tile of 256 / group new tokens walks the cache once), forced for every
    # group size it supports whatever the shape heuristics would choose
    fa.check(fa.capi.lib.fa_set_tuning(10, 2))
    # tiles of 256 / group and of 128 / group new tokens; the smaller blocks also with the cache walk of a tile
    # shared by several blocks (as many as the shape allows, or two) and a merge pass
    # (cols: 32 columns per wavefront, key 23 = 2, or 16, key 23 = 1: half the multiplies per step, twice the blocks)
    for block_waves, split, cols in ((8, 1, 2), (4, 1, 2), (4, 1, 1), (4, 0, 2), (4, 2, 2)):
        fa.check(fa.capi.lib.fa_set_tuning(11, block_waves))
        fa.check(fa.capi.lib.fa_set_tuning(12, split))
        fa.check(fa.capi.lib.fa_set_tuning(23, cols))
        blk = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
        assert_parity("PAGED_PREFILL_PARITY", f"H{heads}/{kv_heads}:L{l_new}:block form, {block_waves} wavefronts, split {split}, cols {cols}", blk, want)
        blk_bf = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args))
        assert_bf16_rounding_of("paged prefill bf16, block form", blk_bf, blk)
        blk_dev = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, be.upload(tables), be.upload(seq_lens), args,
                                                                     out_dtype=fa.capi.F32))
        if split == 1:                # one block a tile: the same launch with host or device tables
            assert np.array_equal(blk_dev, blk)
        else:                         # the share count follows the longest row the host knows of
            assert_parity("PAGED_PREFILL_PARITY", f"H{heads}/{kv_heads}:L{l_new}:device tables, split {split}", blk_dev, want)
        for h in range(heads):
            gq = h // (heads // kv_heads)
            assert np.array_equal(blk_bf[0, 0, h * 128:(h + 1) * 128], vp[tables[0, 0], 0, gq * 128:(gq + 1) * 128])
    fa.check(fa.capi.lib.fa_set_tuning(11, 0))
    fa.check(fa.capi.lib.fa_set_tuning(12, 0))
    fa.check(fa.capi.lib.fa_set_tuning(23, 0))
    # whatever the shape selects by itself (host tables: the longest row is known; device tables: the table width)
    fa.check(fa.capi.lib.fa_set_tuning(10, 0))
    auto = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
    assert_parity("PAGED_PREFILL_PARITY", f"H{heads}/{kv_heads}:L{l_new}:form by shape", auto, want)
    fa.check(fa.capi.lib.fa_set_tuning(10, 1))
    got = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
    got_bf = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args))
    assert_bf16_rounding_of("paged prefill bf16", got_bf, got)      # same launch shape: same f32 values
    # the first new token of a row that had nothing cached sees only itself: its output is its own V row
    for h in range(heads):
        gq = h // (heads // kv_heads)
        assert np.array_equal(got_bf[0, 0, h * 128:(h + 1) * 128], vp[tables[0, 0], 0, gq * 128:(gq + 1) * 128])
    # device-resident tables: same bits
    got_dev = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, be.upload(tables), be.upload(seq_lens), args))
    assert np.array_equal(got_dev, got_bf)
    # the last new token equals a one-token decode call over the same cache
    q_last = np.ascontiguousarray(q[:, -1:, :])
    args1 = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    dec = be.download_owned(be.paged_attention_forward(be.upload(q_last), dk, dv, tables, seq_lens, args1,
                                                       out_dtype=fa.capi.F32))
    assert_parity("PREFILL_LAST_VS_DECODE", f"H{heads}/{kv_heads}:L{l_new}", got[:, -1:, :], dec)
    assert_parity("PREFILL_LAST_VS_DECODE", f"H{heads}/{kv_heads}:L{l_new}:block form", blk[:, -1:, :], dec)
    fa.check(fa.capi.lib.fa_set_tuning(10, 0))


def test_bf16_prefill_in_several_launches_matches_one_token_at_a_time():
    """More token tiles than one launch holds (batch 6 x 800 new tokens, 4 tokens per tile): the launches over
    successive token ranges together equal 800 single-token calls on sampled positions."""
    fa = _fa()
    be = ops()
    rng = o.Rng(77)
    heads, kv_heads, l_new, batch, num_blocks = 32, 8, 800, 6, 400
    lens = [800, 801, 815, 816, 900, 1000]
    tables, seq_lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, lens, num_blocks)
    kp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, l_new, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    oargs = o.paged_args(num_blocks, 16, e_kv, 1, l_new, heads, max_blocks, args.scale, kv_heads)
    o.set_threads(8)
    rc, want = o.paged_attention_bf16(np.ascontiguousarray(q[4:5]), kp, vp, np.ascontiguousarray(tables[4:5]),
                                      np.ascontiguousarray(seq_lens[4:5]), oargs)
    o.set_threads(1)
    assert rc == 0
    args1 = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    # 1: the streamed form in several launches; 0: what the shape selects by itself (the block form, 13 tiles a row)
    for form in (1, 0):
        fa.check(fa.capi.lib.fa_set_tuning(10, form))
        got = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
        assert np.all(np.isfinite(got))
        for t in (0, 1, 3, 4, 63, 64, 170, 171, 682, 683, 684, 799):
            lens_t = (seq_lens - l_new + t + 1).astype(np.uint32)
            dec = be.download_owned(be.paged_attention_forward(be.upload(np.ascontiguousarray(q[:, t:t + 1, :])), dk, dv,
                                                               tables, lens_t, args1, out_dtype=fa.capi.F32))
            assert_parity("PREFILL_VS_DECODE", f"form{form}:t{t}", got[:, t:t + 1, :], dec)
        assert_parity("PAGED_PREFILL_PARITY", f"form{form}:row4 of 6 x 800", got[4:5], want)
    fa.check(fa.capi.lib.fa_set_tuning(10, 0))


def test_bf16_generic_path_covers_shapes_outside_the_fast_path():
    fa = _fa()
    be = ops()
    rng = o.Rng(31)
    for heads, kv_heads, dh, bs, l_new, ctxs in ((4, 2, 64, 16, 1, [33, 5]), (8, 2, 128, 4, 1, [9, 30]),
                                                 (4, 4, 128, 16, 3, [20, 20]), (32, 1, 128, 16, 1, [40, 3])):
        batch, num_blocks = len(ctxs), 64
        tables, lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, ctxs, num_blocks, dh, bs)
        kp = o.to_bf16(rng.randn((num_blocks, bs, e_kv)))
        vp = o.to_bf16(rng.randn((num_blocks, bs, e_kv)))
        q = o.to_bf16(rng.randn((batch, l_new, e_q)))
        layout = fa.PagedKvLayout.new(num_blocks, bs, e_kv)
        args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(dh), kv_heads)
        oargs = o.paged_args(num_blocks, bs, e_kv, batch, l_new, heads, max_blocks, args.scale, kv_heads)
        rc, want = o.paged_attention_bf16(q, kp, vp, tables, lens, oargs)
        assert rc == 0
        got = be.download_owned(be.paged_attention_forward(be.upload(q), be.upload(kp), be.upload(vp), tables, lens, args))
        # the generic kernel keeps the reference's summation order, so after the single bf16 rounding
        # at most a last-bit difference of the f32 value can move an output by one bf16 step
        gf, wf = o.from_bf16(got), o.from_bf16(o.to_bf16(want))
        ulp = np.maximum(np.abs(wf), 2.0 ** -126) * 2.0 ** -7
        assert np.all(np.abs(gf - wf) <= ulp), (heads, kv_heads, dh, bs)
        assert (got != o.to_bf16(want)).mean() < 0.01


def test_device_tables_flag_violations_with_nan():
    fa = _fa()
    be = ops()
    rng = o.Rng(32)
    heads, kv_heads, num_blocks = 8, 2, 32
    tables, lens, max_blocks, e_kv, e_q = _decode_case(rng, 2, heads, kv_heads, [40, 20], num_blocks)
    kp, vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv))), o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((2, 1, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, 2, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    bad = tables.copy()
    bad[1, 0] = num_blocks + 5                      # row 1 points outside the pool
    got = o.from_bf16(be.download_owned(be.paged_attention_forward_device(
        be.upload(q), be.upload(kp), be.upload(vp), be.upload(bad), be.upload(lens), args)))
    assert np.all(np.isfinite(got[0])) and np.all(np.isnan(got[1]))
    # a row of length zero (device lengths are not validated) streams nothing and comes back as zeros
    got0 = o.from_bf16(be.download_owned(be.paged_attention_forward_device(
        be.upload(q), be.upload(kp), be.upload(vp), be.upload(tables), be.upload(np.array([0, 20], np.uint32)), args)))
    assert not got0[0].any() and np.all(np.isfinite(got0[1])) and got0[1].any()
    # append with device slots: out-of-range slots are skipped, valid ones written
    kpool, vpool = be.alloc_zeroed((num_blocks, 16, e_kv), fa.capi.BF16), be.alloc_zeroed((num_blocks, 16, e_kv), fa.capi.BF16)
    rows = o.to_bf16(rng.randn((2, e_kv)))
    slots = np.array([5, num_blocks * 16 + 1], dtype=np.uint32)
    be.paged_kv_append_device(be.upload(rows), be.upload(rows), kpool, vpool, be.upload(slots), layout)
    pool = be.download(kpool).reshape(-1, e_kv)
    assert np.array_equal(pool[5], rows[0]) and not np.delete(pool, 5, axis=0).any()


def test_block_form_prefill_flags_violations_per_column():
    """Device tables, 40 new tokens: a page id outside the pool gives NaN in exactly the columns whose causal
    range reaches that page; a row whose length is below its new tokens is NaN throughout."""
    fa = _fa()
    be = ops()
    rng = o.Rng(33)
    heads, kv_heads, num_blocks, l_new = 8, 2, 64, 40
    tables, lens, max_blocks, e_kv, e_q = _decode_case(rng, 3, heads, kv_heads, [100, 60, 60], num_blocks)
    kp, vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv))), o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((3, l_new, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, 3, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    oargs = o.paged_args(num_blocks, 16, e_kv, 3, l_new, heads, max_blocks, args.scale, kv_heads)
    rc, want = o.paged_attention_bf16(q, kp, vp, tables, lens, oargs)
    assert rc == 0
    bad_t = tables.copy()
    bad_t[1, 2] = num_blocks + 9                    # row 1: positions 32 .. 47 are unreachable
    bad_l = lens.copy()
    bad_l[2] = l_new - 1                            # row 2: fewer positions than new tokens
    fa.check(fa.capi.lib.fa_set_tuning(10, 2))
    try:
        for block_waves, split, cols in ((4, 1, 2), (4, 1, 1), (4, 0, 2), (8, 1, 2)):
            fa.check(fa.capi.lib.fa_set_tuning(11, block_waves))
            fa.check(fa.capi.lib.fa_set_tuning(12, split))
            fa.check(fa.capi.lib.fa_set_tuning(23, cols))
            got = be.download_owned(be.paged_attention_forward_device(
                be.upload(q), be.upload(kp), be.upload(vp), be.upload(bad_t), be.upload(bad_l), args, out_dtype=fa.capi.F32))
            assert_parity("PAGED_PREFILL_PARITY", "row 0 beside violations", got[0:1], want[0:1])
            # row 1: 20 positions were cached, token t sees positions < 21 + t: tokens 0 .. 11 stay below position 32
            assert_parity("PAGED_PREFILL_PARITY", "row 1 before the bad page", got[1:2, :12], want[1:2, :12])
            assert np.all(np.isnan(got[1, 12:])) and np.all(np.isnan(got[2]))
    finally:
        fa.check(fa.capi.lib.fa_set_tuning(10, 0))
        fa.check(fa.capi.lib.fa_set_tuning(11, 0))
        fa.check(fa.capi.lib.fa_set_tuning(12, 0))
        fa.check(fa.capi.lib.fa_set_tuning(23, 0))


def test_bf16_prefill_properties_at_prompt_size():
    """4 rows x 2048 new tokens, 32 / 8 heads (the prompt pass of the benchmark): both block sizes of the block
    form and the streamed form against each other and against one-token decode calls on sampled positions, plus
    the invariances that hold at any size."""
    fa = _fa()
    be = ops()
    rng = o.Rng(5)
    batch, heads, kv_heads, l_new, num_blocks = 4, 32, 8, 2048, 700
    lens = [2048, 2048 + 333, 2048 + 16, 2048 + 1]
    tables, seq_lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, lens, num_blocks)
    kp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, l_new, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    args1 = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    lib = fa.capi.lib
    outs = {}
    try:
        for name, form, waves in (("block8", 2, 8), ("block4", 2, 4), ("streamed", 1, 0), ("by shape", 0, 0)):
            fa.check(lib.fa_set_tuning(10, form))
            fa.check(lib.fa_set_tuning(11, waves))
            outs[name] = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
            assert np.all(np.isfinite(outs[name])), name
        fa.check(lib.fa_set_tuning(10, 0))
        fa.check(lib.fa_set_tuning(11, 0))
        for name in ("block8", "block4", "by shape"):
            assert_parity("PREFILL_FORMS", f"{name} vs streamed", outs[name], outs["streamed"])
        # sampled positions against one-token decode calls over the same cache (tile edges of both block sizes)
        for t in (0, 1, 31, 32, 63, 64, 1000, 2047):
            lens_t = (seq_lens - l_new + t + 1).astype(np.uint32)
            dec = be.download_owned(be.paged_attention_forward(be.upload(np.ascontiguousarray(q[:, t:t + 1, :])), dk, dv,
                                                               tables, lens_t, args1, out_dtype=fa.capi.F32))
            for name in ("block8", "block4"):
                assert_parity("PREFILL_VS_DECODE", f"{name}:t{t}", outs[name][:, t:t + 1, :], dec)
        # the oracle on the first 40 tokens of the row with the longest cache
        oargs = o.paged_args(num_blocks, 16, e_kv, 1, 40, heads, max_blocks, args.scale, kv_heads)
        o.set_threads(8)
        rc, want = o.paged_attention_bf16(np.ascontiguousarray(q[1:2, :40]), kp, vp, np.ascontiguousarray(tables[1:2]),
                                          np.array([lens[1] - l_new + 40], np.uint32), oargs)
        o.set_threads(1)
        assert rc == 0
        assert_parity("PAGED_PREFILL_PARITY", "row 1, tokens 0..39", outs["block8"][1:2, :40], want)
        got = outs["by shape"]
        # every output is a convex combination of V rows of its kv head
        used = tables[tables != U32MAX]
        vmax = np.abs(o.from_bf16(vp[used])).reshape(-1, kv_heads, 128).max(axis=0)
        bound = np.repeat(vmax, heads // kv_heads, axis=0)[None, None]
        assert np.all(np.abs(got.reshape(batch, l_new, heads, 128)) <= bound + 1e-6)
        # moving pages to other physical blocks changes no bit
        perm2 = np.roll(np.arange(num_blocks), 11).astype(np.uint32)
        kp2, vp2 = np.empty_like(kp), np.empty_like(vp)
        kp2[perm2], vp2[perm2] = kp, vp
        t2 = tables.copy()
        msk = tables != U32MAX
        t2[msk] = perm2[tables[msk]]
        got2 = be.download_owned(be.paged_attention_forward(dq, be.upload(kp2), be.upload(vp2), t2, seq_lens, args,
                                                            out_dtype=fa.capi.F32))
        assert np.array_equal(got, got2)
        # a constant V gives that constant back
        ones = np.full_like(vp, o.to_bf16(np.array([1.5], np.float32))[0])
        got3 = be.download_owned(be.paged_attention_forward(dq, dk, be.upload(ones), tables, seq_lens, args,
                                                            out_dtype=fa.capi.F32))
        assert np.allclose(got3, 1.5, rtol=1e-5, atol=0)
    finally:
        fa.check(lib.fa_set_tuning(10, 0))
        fa.check(lib.fa_set_tuning(11, 0))


def test_bf16_prefill_few_new_tokens_over_a_long_cache_share_the_walk():
    """64 new tokens per row over some thousand cached positions (a conversation that continues): few tiles, long
    walks.  The block form with shared walks, the block form without and the streamed form agree with each other
    and with one-token decode calls; the shape's own choice is one of them."""
    fa = _fa()
    be = ops()
    rng = o.Rng(9)
    batch, heads, kv_heads, l_new, num_blocks = 2, 32, 8, 64, 600
    lens = [4096 + 64, 1500 + 64]
    tables, seq_lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, lens, num_blocks)
    kp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, l_new, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    args1 = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    lib = fa.capi.lib
    outs = {}
    try:
        for name, form, split in (("shared walks", 2, 0), ("two shares", 2, 2), ("one block a tile", 2, 1), ("streamed", 1, 0), ("by shape", 0, 0)):
            fa.check(lib.fa_set_tuning(10, form))
            fa.check(lib.fa_set_tuning(12, split))
            outs[name] = be.download_owned(be.paged_attention_forward(dq, dk, dv, tables, seq_lens, args, out_dtype=fa.capi.F32))
            assert np.all(np.isfinite(outs[name])), name
    finally:
        fa.check(lib.fa_set_tuning(10, 0))
        fa.check(lib.fa_set_tuning(12, 0))
    for name in ("shared walks", "two shares", "one block a tile", "by shape"):
        assert_parity("PREFILL_FORMS", f"{name} vs streamed", outs[name], outs["streamed"])
    for t in (0, 31, 32, 63):
        lens_t = (seq_lens - l_new + t + 1).astype(np.uint32)
        dec = be.download_owned(be.paged_attention_forward(be.upload(np.ascontiguousarray(q[:, t:t + 1, :])), dk, dv,
                                                           tables, lens_t, args1, out_dtype=fa.capi.F32))
        assert_parity("PREFILL_VS_DECODE", f"shared walks:t{t}", outs["shared walks"][:, t:t + 1, :], dec)
    # the oracle on the shorter row
    oargs = o.paged_args(num_blocks, 16, e_kv, 1, l_new, heads, max_blocks, args.scale, kv_heads)
    o.set_threads(8)
    rc, want = o.paged_attention_bf16(np.ascontiguousarray(q[1:2]), kp, vp, np.ascontiguousarray(tables[1:2]),
                                      np.ascontiguousarray(seq_lens[1:2]), oargs)
    o.set_threads(1)
    assert rc == 0
    assert_parity("PAGED_PREFILL_PARITY", "row 1, shared walks", outs["shared walks"][1:2], want)


def test_shared_walks_flag_violations_per_column():
    """Device tables, 64 new tokens over a long cache, the walk of each tile shared by several blocks: a page id
    outside the pool gives NaN in exactly the columns whose causal range reaches that page, through the merge."""
    fa = _fa()
    be = ops()
    rng = o.Rng(10)
    batch, heads, kv_heads, l_new, num_blocks = 2, 8, 2, 64, 400
    lens = [4096 + 64, 1500 + 64]
    tables, seq_lens, max_blocks, e_kv, e_q = _decode_case(rng, batch, heads, kv_heads, lens, num_blocks)
    kp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, e_kv)))
    q = o.to_bf16(rng.randn((batch, l_new, e_q)))
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    dq, dk, dv = be.upload(q), be.upload(kp), be.upload(vp)
    bad = tables.copy()
    bad[0, 259] = num_blocks + 1                    # row 0: its last page, positions 4144 .. 4159
    bad[1, 10] = 0xFFFFFFF0                         # row 1: a page every new token sees
    lib = fa.capi.lib
    fa.check(lib.fa_set_tuning(10, 2))
    try:
        good = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, be.upload(tables), be.upload(seq_lens), args,
                                                                   out_dtype=fa.capi.F32))
        got = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, be.upload(bad), be.upload(seq_lens), args,
                                                                  out_dtype=fa.capi.F32))
    finally:
        fa.check(lib.fa_set_tuning(10, 0))
    assert np.all(np.isfinite(good))
    # row 0: 4096 positions were cached, token t sees positions < 4097 + t: tokens 0 .. 47 stay below position 4144
    assert np.array_equal(got[0, :48], good[0, :48]) and np.all(np.isnan(got[0, 48:]))
    assert np.all(np.isnan(got[1]))
