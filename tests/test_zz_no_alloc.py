"""The decode attention entry point that allocates nothing (fa_paged_attention_decode_static): same bits as
fa_paged_attention_forward_device, which is itself held to the oracle in test_gpu_paged.py, on two calls in a
row of which the second is smaller (the static scratch keeps the first call's partial results), and against
the oracle directly; pool statistics show that the calls took no device memory."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as o
from gpu_common import assert_parity, ops

pytestmark = pytest.mark.gpu
U32MAX = 0xFFFFFFFF


def _case(rng, batch, heads, kv_heads, ctxs, num_blocks):
    e_kv, e_q = kv_heads * 128, heads * 128
    max_blocks = max((c + 15) // 16 for c in ctxs) + 1
    need = sum((c + 15) // 16 for c in ctxs)
    assert need <= num_blocks
    ids = rng.permutation(num_blocks)[:need]
    tables = np.full((batch, max_blocks), U32MAX, dtype=np.uint32)
    p = 0
    for b, c in enumerate(ctxs):
        nb = (c + 15) // 16
        tables[b, :nb] = ids[p:p + nb]
        p += nb
    return tables, np.array(ctxs, dtype=np.uint32), max_blocks, e_kv, e_q


def _static(fa, be, q, kp, vp, tables, lens, args, out):
    fa.check(fa.capi.lib.fa_paged_attention_decode_static(be._ctx, q._h, kp._h, vp._h, tables._h, lens._h,
                                                          C.byref(args.c()), out._h))


def test_static_scratch_entry_point_matches_the_pooled_one_on_two_calls_in_a_row():
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    assert lib.fa_paged_attention_decode_static_max_bytes() == 16 << 20
    rng = o.Rng(77)
    heads, kv_heads, num_blocks = 32, 8, 1200
    big_ctx = [1, 15, 16, 17, 130, 777, 2049, 4000, 33, 640, 1234, 96]
    small_ctx = [300, 5, 48]
    kp = o.to_bf16(rng.randn((num_blocks, 16, kv_heads * 128)))
    vp = o.to_bf16(rng.randn((num_blocks, 16, kv_heads * 128)))
    dk, dv = be.upload(kp), be.upload(vp)
    layout = fa.PagedKvLayout.new(num_blocks, 16, kv_heads * 128)
    results = []
    for ctxs in (big_ctx, small_ctx):
        batch = len(ctxs)
        tables, lens, max_blocks, e_kv, e_q = _case(rng, batch, heads, kv_heads, ctxs, num_blocks)
        q = o.to_bf16(rng.randn((batch, 1, e_q)))
        args = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
        dq, dt, dl = be.upload(q), be.upload(tables), be.upload(lens)
        # the pooled entry point first (it sizes the context's workspace), then its result as the bar
        want_bf = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, dt, dl, args))
        want_f32 = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, dt, dl, args, out_dtype=fa.capi.F32))
        out_bf = be.alloc_zeroed((batch, 1, e_q), fa.capi.BF16)
        out_f32 = be.alloc_zeroed((batch, 1, e_q), fa.capi.F32)
        be.synchronize_device()
        before = be.device_memory_pool_stats()
        _static(fa, be, dq, dk, dv, dt, dl, args, out_bf)
        _static(fa, be, dq, dk, dv, dt, dl, args, out_f32)
        after = be.device_memory_pool_stats()
        # no allocation, no pool traffic at all
        assert (after.alloc_count, after.reuse_count, after.cached_bytes) == \
            (before.alloc_count, before.reuse_count, before.cached_bytes)
        got_bf, got_f32 = be.download(out_bf), be.download(out_f32)
        assert np.array_equal(got_bf, want_bf), ctxs
        assert np.array_equal(got_f32, want_f32), ctxs
        # and against the oracle itself
        oargs = o.paged_args(num_blocks, 16, e_kv, batch, 1, heads, max_blocks, args.scale, kv_heads)
        o.set_threads(8)
        rc, want = o.paged_attention_bf16(q, kp, vp, tables, lens, oargs)
        o.set_threads(1)
        assert rc == 0
        assert_parity("PAGED_DECODE_STATIC_PARITY", "B%d" % batch, got_f32, want)
        results.append(got_bf)
    # the second, smaller call ran over the first call's leftovers in the scratch; run the first shape's
    # small sibling once more under graph capture, where the pooled entry point could not grow its workspace
    batch = len(small_ctx)
    tables, lens, max_blocks, e_kv, e_q = _case(o.Rng(5), batch, heads, kv_heads, small_ctx, num_blocks)
    q = o.to_bf16(o.Rng(6).randn((batch, 1, e_q)))
    args = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads)
    dq, dt, dl = be.upload(q), be.upload(tables), be.upload(lens)
    want = be.download_owned(be.paged_attention_forward_device(dq, dk, dv, dt, dl, args))
    out = be.alloc_zeroed((batch, 1, e_q), fa.capi.BF16)
    g = C.c_void_p()
    fa.check(lib.fa_graph_capture_begin(be._ctx))
    try:
        _static(fa, be, dq, dk, dv, dt, dl, args, out)
    finally:
        st = lib.fa_graph_capture_end(be._ctx, C.byref(g))
    fa.check(st)
    try:
        for _ in range(2):
            fa.check(lib.fa_graph_launch(be._ctx, g))
            assert np.array_equal(be.download(out), want)
            be.upload_into(np.zeros(out.numel(), np.uint16), out, 0)
    finally:
        lib.fa_graph_destroy(be._ctx, g)


def test_static_scratch_entry_point_rejects_what_it_cannot_hold():
    import fandhe_ai_amd as fa
    be = ops()
    rng = o.Rng(78)
    # a shape outside the streamed decode kernel: f32 storage
    num_blocks, heads = 8, 2
    layout = fa.PagedKvLayout.new(num_blocks, 16, heads * 128)
    args = fa.PagedAttentionArgs(layout, 1, 1, heads, 2, 0.5)
    pool = be.upload(rng.randn((num_blocks, 16, heads * 128)))
    q = be.upload(rng.randn((1, 1, heads * 128)))
    t, l = be.upload(np.array([[0, 1]], np.uint32)), be.upload(np.array([20], np.uint32))
    out = be.alloc_zeroed((1, 1, heads * 128))
    with pytest.raises(fa.Unsupported):
        _static(fa, be, q, pool, pool, t, l, args, out)
    # too many partial results for the array: 64 kv heads x 16 query heads each at 64 rows
    heads, kv_heads, batch = 1024, 64, 64
    layout = fa.PagedKvLayout.new(4, 16, kv_heads * 128)
    args = fa.PagedAttentionArgs(layout, batch, 1, heads, 1, 0.5, kv_heads)
    pool = be.alloc_zeroed((4, 16, kv_heads * 128), fa.capi.BF16)
    q = be.alloc_zeroed((batch, 1, heads * 128), fa.capi.BF16)
    t, l = be.upload(np.zeros((batch, 1), np.uint32)), be.upload(np.ones(batch, np.uint32))
    out = be.alloc_zeroed((batch, 1, heads * 128), fa.capi.BF16)
    with pytest.raises(fa.InvalidArgument, match="static scratch holds"):
        _static(fa, be, q, pool, pool, t, l, args, out)
