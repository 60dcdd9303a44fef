"""GPU parity of the full decode step against the oracle's decode step.

The step chains quantizers, whose rounding is discontinuous: a last-bit
difference in an activation (attention's reduction order, exp) can flip an
int8 code, which moves a few accumulators by one weight code.  The operators
are each held to the reference's tolerance in their own tests; for the chained
step the logits are held, relative to the row's logit range, to a mean error
below 2e-4 and a maximum below 2e-2 (stated here; a flipped code shifts all
logits of that one sequence by a few 1e-3 of the range, the other sequences
stay bit-exact), and the greedy tokens must match wherever the oracle's
top-2 margin exceeds twice that maximum.  (Where a test has only a few rows, one flipped
row is not diluted by the others: there the bar is per row, mean below 4e-3 and median
row below 2e-4.)  Appended K/V rows are held
to 2^-6 of the row's largest magnitude (a code flip upstream moves a whole
row by a fraction of one quantization step).
"""
import numpy as np
import pytest

import oracle_lib as o
from decoder_common import GpuDecoder, build_model, oracle_step
from gpu_common import ops

pytestmark = pytest.mark.gpu


def _check_step(m, dec, lens, tokens, use_graph, tag):
    pools_before = [L["k_pool"].copy() for L in m.layers]
    want_next, want_logits = oracle_step(m, lens, tokens)
    dec.step(use_graph)
    got_logits, got_next = dec.logits(), dec.tokens()
    spread = want_logits.max(axis=1, keepdims=True) - want_logits.min(axis=1, keepdims=True)
    err = np.abs(got_logits - want_logits) / spread
    p999 = float(np.percentile(err, 99.9))
    exact_rows = int((err.max(axis=1) == 0).sum())
    print("DECODE_STEP_PARITY\t%s\tmax_err/range=%.3e\tp99.9=%.3e\tmean=%.3e\tbit_exact_rows=%d/%d"
          % (tag, err.max(), p999, err.mean(), exact_rows, err.shape[0]), flush=True)
    assert err.mean() < 2e-4 and err.max() < 2e-2
    top2 = np.sort(want_logits, axis=1)[:, -2:]
    decisive = (top2[:, 1] - top2[:, 0]) > 4e-2 * spread[:, 0]
    assert np.array_equal(got_next[decisive], want_next[decisive])
    assert np.array_equal(got_next, o.argmax_rows(got_logits))
    assert np.array_equal(dec.seq_lens(), lens)
    for li, L in enumerate(m.layers):
        gk, gv = dec.kv_pool(li)
        changed = (L["k_pool"] != pools_before[li]).any(axis=2)
        assert np.array_equal((gk != pools_before[li]).any(axis=2) | changed, changed)      # nothing else written
        for name, g, w in (("k", gk, L["k_pool"]), ("v", gv, L["v_pool"])):
            gf, wf = o.from_bf16(g[changed]), o.from_bf16(w[changed])
            assert np.all(np.abs(gf - wf) <= np.abs(wf).max(axis=1, keepdims=True) * 2.0 ** -6), (li, name)
        # keep the two caches identical from here on, so that later steps compare like with like
        L["k_pool"][:] = gk
        L["v_pool"][:] = gv
    return got_next


@pytest.mark.parametrize("shape", [
    dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, d_ffn=512, vocab=1000, batch=4, ctxs=[1, 15, 16, 200]),
    dict(n_layers=1, d_model=512, n_heads=8, n_kv_heads=8, d_ffn=256, vocab=333, batch=17, ctxs=list(range(3, 20))),
    dict(n_layers=2, d_model=1024, n_heads=8, n_kv_heads=1, d_ffn=1536, vocab=4000, batch=32, ctxs=[40 + 9 * i for i in range(32)]),
    # more than 32 rows: three and four row tiles per block in the decode-shape linears
    dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=2, d_ffn=1024, vocab=2000, batch=41, ctxs=[1 + 7 * i for i in range(41)]),
    dict(n_layers=1, d_model=1024, n_heads=8, n_kv_heads=2, d_ffn=1536, vocab=1500, batch=64, ctxs=[5 + 3 * i for i in range(64)]),
])
@pytest.mark.parametrize("astat", [1, 2], ids=["block-per-tile", "activation-stationary"])
def test_decode_steps_match_the_oracle_eager_and_graph(shape, astat):
    """Both families of decode-shape linears (the test models are narrow, so the activation-stationary
    kernels, which the shape heuristic reserves for wide weights, are forced for one of the runs)."""
    import fandhe_ai_amd as fa
    be = ops()
    fa.check(fa.capi.lib.fa_set_tuning(5, astat))
    m = build_model(seed=11, steps=4, **shape)
    dec = GpuDecoder(be, m)
    try:
        lens, tokens = m.seq_lens.copy(), m.tokens.copy()
        for step in range(3):
            tokens = _check_step(m, dec, lens, tokens, use_graph=(step > 0),
                                 tag="L%d:B%d:step%d:%d" % (shape["n_layers"], shape["batch"], step, astat))
            dec.set_state(lens, tokens)            # the oracle continues from the GPU's tokens
    finally:
        dec.close()
        fa.check(fa.capi.lib.fa_set_tuning(5, 0))


@pytest.mark.parametrize("shape", [
    dict(n_layers=2, d_model=2048, n_heads=16, n_kv_heads=4, d_ffn=3072, vocab=3000),
    # the benchmark's width, one layer: gate / up takes the activation-stationary kernel by shape
    dict(n_layers=1, d_model=4096, n_heads=32, n_kv_heads=8, d_ffn=14336, vocab=32000),
], ids=["2048-wide", "benchmark-wide"])
@pytest.mark.parametrize("batch", [1, 2, 3, 4])
def test_small_batches_do_the_row_work_inside_the_linears(shape, batch):
    """With one to four rows the q | k | v and gate | up projections do the norm + quantizer in front of them
    themselves, and with one or two rows the down projection does its quantizer (no launch of their own for the row
    kernels).  The steps must meet the oracle like any other batch, and every logit, token and cache row must be
    bit-identical to the same steps with the row kernels launched separately (tuning key 19 = 1): a sequence decodes to
    the same bits whatever batch it sits in.  The codes and scales the fused linears publish are those of the
    stand-alone kernels as well (read back after the step: the down projection's)."""
    import ctypes as C
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    wide = shape["d_model"] == 4096
    ctxs = [3, 130, 17, 64][:batch]
    m = build_model(seed=21 + batch, steps=4, batch=batch, ctxs=ctxs, numpy_fill=wide, **shape)
    if not wide:
        fa.check(lib.fa_set_tuning(5, 2))                 # narrow test model: force the kernel gate / up uses at full width
    outs, stages = {}, {}
    try:
        # (the attention keeps its usual form in both runs: how a sequence's pages are divided among wavefronts decides
        # the last bits of its output, and the one-launch form for short contexts divides them its own way)
        fa.check(lib.fa_set_tuning(20, 1))
        for fused in (True, False):
            fa.check(lib.fa_set_tuning(19, 2 if fused else 1))
            dec = GpuDecoder(be, m)
            try:
                # what the row stages leave behind, read after the linear that would consume it: the q | k | v projection
                # (stage 2: the attention norm's codes and scales), gate | up (stage 6: the ffn norm's) and the down
                # projection (stage 8: the SwiGLU quantizer's) of the first layer
                got = []
                for stage, k_cols in ((2, shape["d_model"]), (6, shape["d_model"]), (8, shape["d_ffn"])):
                    dec.set_state(m.seq_lens, m.tokens)
                    fa.check(lib.fa_decoder_debug_step_until(be._ctx, dec.h, stage))
                    xq, sx = C.c_void_p(), C.c_void_p()
                    fa.check(lib.fa_decoder_debug_buffer(dec.h, 1, C.byref(xq)))
                    fa.check(lib.fa_decoder_debug_buffer(dec.h, 2, C.byref(sx)))
                    codes = np.empty(16 * k_cols, np.int8)
                    scales = np.empty(batch, np.float32)
                    fa.check(lib.fa_download(be._ctx, xq, 0, codes.ctypes.data, codes.size))
                    fa.check(lib.fa_download(be._ctx, sx, 0, scales.ctypes.data, batch))
                    got.append((codes, scales))
                stages[fused] = got
                lens, tokens = m.seq_lens.copy(), m.tokens.copy()
                trace = []
                for step in range(3):
                    dec.set_state(lens, tokens)
                    dec.step(step > 0)
                    trace.append((dec.logits().copy(), dec.tokens().copy(), [tuple(x.copy() for x in dec.kv_pool(li))
                                                                             for li in range(shape["n_layers"])]))
                    lens = lens + 1
                    tokens = trace[-1][1]
                outs[fused] = trace
            finally:
                dec.close()
        for i, ((ca, sa), (cb, sb)) in enumerate(zip(stages[True], stages[False])):
            assert np.array_equal(sa, sb), "scales of row stage %d differ between the fused and the separate row work" % i
            assert np.array_equal(ca, cb), "codes of row stage %d differ between the fused and the separate row work" % i
            assert np.any(ca != 0)
        for step, (a, b) in enumerate(zip(outs[True], outs[False])):
            assert np.array_equal(a[0], b[0]), "logits of step %d differ between the fused and the separate row work" % step
            assert np.array_equal(a[1], b[1])
            for (ak, av), (bk, bv) in zip(a[2], b[2]):
                assert np.array_equal(ak, bk) and np.array_equal(av, bv)
        # against the oracle, with the fused path (and, for one and two rows, the one-launch attention)
        fa.check(lib.fa_set_tuning(19, 0))
        fa.check(lib.fa_set_tuning(20, 0))
        dec = GpuDecoder(be, m)
        try:
            lens, tokens = m.seq_lens.copy(), m.tokens.copy()
            for step in range(2):
                tokens = _check_small(m, dec, lens, tokens, step > 0, "fused rows:B%d:step%d" % (batch, step))
                dec.set_state(lens, tokens)
        finally:
            dec.close()
    finally:
        fa.check(lib.fa_set_tuning(19, 0))
        fa.check(lib.fa_set_tuning(20, 0))
        fa.check(lib.fa_set_tuning(5, 0))


_MANY_SHORT = [int(x) for x in np.random.default_rng(5).integers(1, 700, size=33)]


@pytest.mark.parametrize("ctxs", [[1], [16], [17, 3], [130, 64], [1000, 1], [1023, 777], [40, 7, 300, 1, 64], _MANY_SHORT],
                         ids=lambda c: "ctx" + "_".join(map(str, c[:6])) + ("_etc" if len(c) > 6 else ""))
def test_short_contexts_finish_the_attention_in_one_launch(ctxs):
    """Sequences of at most 1024 tokens: the attention runs as one launch (a block per sequence and kv head whose
    four wavefronts share the pages); with one or two sequences the o projection does the per-token quantizer, with
    more (up to one block per compute unit by itself; forced here for every batch, tuning key 20 = 2) the quantizer
    from the heads' maxima is a launch of its own.  The codes and scales of the attention output (stage 4
    of the first layer) must be what the streamed attention + merge + quantizer leave (tuning key 20 = 1) up to the
    last bits of the attention output: equal scales to 1e-6 relative and codes at most one step apart, nearly all
    equal.  The steps meet the oracle, eager and replayed, also when a context grows past the limit and the step
    changes form (1023 -> 1026)."""
    import ctypes as C
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    batch = len(ctxs)
    shape = dict(n_layers=2, d_model=2048, n_heads=16, n_kv_heads=4, d_ffn=3072, vocab=3000)
    m = build_model(seed=40 + sum(ctxs), steps=5, batch=batch, ctxs=ctxs, **shape)
    got = {}
    try:
        for one in (True, False):
            fa.check(lib.fa_set_tuning(20, 2 if one else 1))
            dec = GpuDecoder(be, m)
            try:
                dec.set_state(m.seq_lens, m.tokens)
                fa.check(lib.fa_decoder_debug_step_until(be._ctx, dec.h, 4))
                xq, sx = C.c_void_p(), C.c_void_p()
                fa.check(lib.fa_decoder_debug_buffer(dec.h, 1, C.byref(xq)))
                fa.check(lib.fa_decoder_debug_buffer(dec.h, 2, C.byref(sx)))
                codes = np.empty(16 * shape["d_model"], np.int8)
                scales = np.empty(batch, np.float32)
                fa.check(lib.fa_download(be._ctx, xq, 0, codes.ctypes.data, codes.size))
                fa.check(lib.fa_download(be._ctx, sx, 0, scales.ctypes.data, batch))
                got[one] = (codes.astype(np.int32), scales)
            finally:
                dec.close()
        (ca, sa), (cb, sb) = got[True], got[False]
        assert np.all(sb > 0) and np.allclose(sa, sb, rtol=1e-6, atol=0)
        assert np.abs(ca - cb).max() <= 1 and (ca != cb).mean() < 2e-3 and np.any(ca != 0)
        fa.check(lib.fa_set_tuning(20, 2))
        dec = GpuDecoder(be, m)
        try:
            lens, tokens = m.seq_lens.copy(), m.tokens.copy()
            for step in range(4):
                tokens = _check_small(m, dec, lens, tokens, step > 0, "one-launch attention:%s:step%d" % (ctxs, step))
                dec.set_state(lens, tokens)
        finally:
            dec.close()
    finally:
        fa.check(lib.fa_set_tuning(20, 0))


def _check_small(m, dec, lens, tokens, use_graph, tag):
    """_check_step with the bar for a handful of rows: a flipped code is not diluted by other rows, so every row is
    held to mean < 4e-3 of its logit range and, with three rows or more, the median row to 2e-4 (with one or two rows
    a single flipped code is the median)."""
    want_next, want_logits = oracle_step(m, lens, tokens)
    dec.step(use_graph)
    got_logits, got_next = dec.logits(), dec.tokens()
    spread = want_logits.max(axis=1, keepdims=True) - want_logits.min(axis=1, keepdims=True)
    err = np.abs(got_logits - want_logits) / spread
    rows = err.mean(axis=1)
    print("DECODE_STEP_PARITY\t%s\tmax_err/range=%.3e\trow means=%s" % (tag, err.max(), np.array2string(rows, precision=2)), flush=True)
    assert rows.max() < 4e-3 and (len(rows) < 3 or np.median(rows) < 2e-4) and err.max() < 2e-2
    top2 = np.sort(want_logits, axis=1)[:, -2:]
    decisive = (top2[:, 1] - top2[:, 0]) > 4e-2 * spread[:, 0]
    assert np.array_equal(got_next[decisive], want_next[decisive])
    assert np.array_equal(dec.seq_lens(), lens)
    for li, L in enumerate(m.layers):
        gk, gv = dec.kv_pool(li)
        L["k_pool"][:] = gk
        L["v_pool"][:] = gv
    return got_next


def test_decode_step_at_the_benchmark_width():
    """One layer of the benchmark's decoder at its full width (d_model 4096, 32 / 8 heads, FFN 14336, vocab
    32000), batch 32, contexts uniform in [1024, 8192]: the shapes at which the step's kernels are timed
    (activation-stationary gate/up and lm_head, deep-k down projection, long ragged contexts), eager and graph."""
    be = ops()
    ctxs = np.random.default_rng(0).integers(1024, 8193, size=32).tolist()
    m = build_model(seed=3, n_layers=1, d_model=4096, n_heads=32, n_kv_heads=8, d_ffn=14336, vocab=32000, batch=32,
                    ctxs=ctxs, steps=3, numpy_fill=True)
    dec = GpuDecoder(be, m)
    try:
        lens, tokens = m.seq_lens.copy(), m.tokens.copy()
        for step in range(2):
            tokens = _check_step(m, dec, lens, tokens, use_graph=(step > 0), tag="benchmark width:step%d" % step)
            dec.set_state(lens, tokens)
    finally:
        dec.close()


PREFILL_SHAPES = [
    dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, d_ffn=512, vocab=1000, batch=4, ctxs=[0, 5, 16, 40], l_new=7),
    dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=2, d_ffn=768, vocab=500, batch=3, ctxs=[0, 1, 31], l_new=33),
    dict(n_layers=1, d_model=256, n_heads=2, n_kv_heads=2, d_ffn=256, vocab=300, batch=2, ctxs=[0, 100], l_new=1),
    # d_ffn beyond 16384: the SwiGLU quantizer's two-pass form
    dict(n_layers=1, d_model=256, n_heads=2, n_kv_heads=1, d_ffn=16448, vocab=300, batch=2, ctxs=[0, 5], l_new=9),
    # the benchmark's width: 72 rows against 4096 / 6144 / 28672 / 4096-column weights (k split across blocks)
    dict(n_layers=1, d_model=4096, n_heads=32, n_kv_heads=8, d_ffn=14336, vocab=32000, batch=3, ctxs=[0, 37, 400], l_new=24,
         numpy_fill=True),
    # 8 x 1100 rows: two chunks (1024 + 76 tokens per sequence)
    dict(n_layers=1, d_model=256, n_heads=4, n_kv_heads=1, d_ffn=256, vocab=300, batch=8, ctxs=[0, 3, 9, 20, 0, 64, 7, 15],
         l_new=1100),
]


@pytest.mark.parametrize("shape", PREFILL_SHAPES, ids=["B%d_L%d" % (s["batch"], s["l_new"]) for s in PREFILL_SHAPES])
def test_prompt_prefill_matches_the_oracle_decoding_the_prompt_token_by_token(shape):
    """The oracle has no prompt path of its own: it decodes the prompt one token at a time (teacher forced),
    which is what the prefill is defined to equal.  Tolerances as for the chained decode step above."""
    be = ops()
    shape = dict(shape)
    l_new = shape.pop("l_new")
    m = build_model(seed=21, steps=l_new + 2, **shape)
    dec = GpuDecoder(be, m)
    try:
        rng = o.Rng(5)
        prompt = rng.randint(0, shape["vocab"], shape["batch"] * l_new).astype(np.int32).reshape(shape["batch"], l_new)
        pools_before = [(L["k_pool"].copy(), L["v_pool"].copy()) for L in m.layers]
        lens = m.seq_lens.copy()
        for t in range(l_new):
            want_next, want_logits = oracle_step(m, lens, np.ascontiguousarray(prompt[:, t]))
        dec.prefill(prompt)
        got_logits, got_next = dec.logits(), dec.tokens()
        spread = want_logits.max(axis=1, keepdims=True) - want_logits.min(axis=1, keepdims=True)
        err = np.abs(got_logits - want_logits) / spread
        row_mean = err.mean(axis=1)
        print("PREFILL_PARITY\tB%d:L%d\tmax_err/range=%.3e\tmean=%.3e\trows with mean error below 1e-6: %d/%d"
              % (shape["batch"], l_new, err.max(), err.mean(), int((row_mean < 1e-6).sum()), len(row_mean)), flush=True)
        # a batch of a few rows cannot dilute one flipped code (a row then sits at a few 1e-3 of its range
        # while the others are exact): the bar is per row, and the typical row must be far below it
        assert err.max() < 2e-2 and (row_mean < 4e-3).all() and np.median(row_mean) < 2e-4
        top2 = np.sort(want_logits, axis=1)[:, -2:]
        decisive = (top2[:, 1] - top2[:, 0]) > 4e-2 * spread[:, 0]
        assert np.array_equal(got_next[decisive], want_next[decisive])
        assert np.array_equal(got_next, o.argmax_rows(got_logits))
        assert np.array_equal(dec.seq_lens(), lens) and np.array_equal(lens, m.seq_lens + l_new)
        for li, L in enumerate(m.layers):
            gk, gv = dec.kv_pool(li)
            for name, g, w, before in (("k", gk, L["k_pool"], pools_before[li][0]), ("v", gv, L["v_pool"], pools_before[li][1])):
                changed = (w != before).any(axis=2)
                assert np.array_equal((g != before).any(axis=2) | changed, changed), (li, name)   # nothing else written
                gf, wf = o.from_bf16(g[changed]), o.from_bf16(w[changed])
                assert np.all(np.abs(gf - wf) <= np.abs(wf).max(axis=1, keepdims=True) * 2.0 ** -6), (li, name)
                if li == 0:
                    # the first layer's rows depend on nothing but the embedding and the projection: exact
                    assert np.array_equal(g[changed], w[changed]), name
            L["k_pool"][:] = gk
            L["v_pool"][:] = gv
        # decoding continues from the prefilled state
        _check_step(m, dec, lens, got_next.copy(), use_graph=False, tag="after prefill B%d:L%d" % (shape["batch"], l_new))
    finally:
        dec.close()


def test_prompt_pass_on_large_tiles_equals_the_pass_on_128_tiles_bit_for_bit():
    """The projections of a prompt pass on the large-tile GEMM (forced: 256 x 224 tiles; its epilogue adds the
    residual of the o and down projections from registers, four outputs of a row per lane, the gate | up projection
    takes SwiGLU into its epilogue and the q | k | v projection RoPE and the K / V append) against the same pass with
    SwiGLU left to the row quantizer and RoPE to its own pass, and against
    the pass on the 128 x 128 kernel (its own epilogue code): int32 sums are exact, the epilogues apply scale, then
    residual, in the same order, and the products are the same expressions of the same values, so logits, tokens and
    every cache row must be identical."""
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    shape = dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=2, d_ffn=1024, vocab=700, batch=3, ctxs=[0, 9, 40])
    l_new = 100                                           # 300 rows: two row blocks of 256, the second ragged
    m = build_model(seed=77, steps=l_new + 2, **shape)
    prompt = o.Rng(6).randint(0, shape["vocab"], shape["batch"] * l_new).astype(np.int32).reshape(shape["batch"], l_new)
    got = {}
    try:
        # (every projection on the tiled GEMMs: at this width the weight-stationary kernel would take them, key 21 = 1)
        fa.check(lib.fa_set_tuning(21, 1))
        # "big": large tiles, the gate | up GEMM with SwiGLU in its epilogue (256 x 256 tiles of eight gate and eight
        # up column tiles, products written) and the q | k | v GEMM with RoPE, the bf16 rounding and the K / V append
        # in its epilogue (a head per wavefront); "plain": large tiles, both left to their own passes (key 22 = 3);
        # "small": the 128 x 128 kernel everywhere
        for form in ("big", "plain", "small"):
            fa.check(lib.fa_set_tuning(7, 0 if form == "small" else 14))
            fa.check(lib.fa_set_tuning(4, 1 if form == "small" else 0))
            fa.check(lib.fa_set_tuning(22, 3 if form == "plain" else 0))
            dec = GpuDecoder(be, m)
            try:
                dec.prefill(prompt)
                got[form] = (dec.logits().copy(), dec.tokens().copy(), [tuple(x.copy() for x in dec.kv_pool(li)) for li in range(2)])
            finally:
                dec.close()
    finally:
        fa.check(lib.fa_set_tuning(7, 0))
        fa.check(lib.fa_set_tuning(4, 0))
        fa.check(lib.fa_set_tuning(22, 0))
        fa.check(lib.fa_set_tuning(21, 0))
    a = got["big"]
    assert np.all(np.isfinite(a[0])) and np.any(a[0] != 0)
    for other in ("plain", "small"):
        b = got[other]
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), other
        for (ak, av), (bk, bv) in zip(a[2], b[2]):
            assert np.array_equal(ak, bk) and np.array_equal(av, bv), other


@pytest.mark.parametrize("batch,l_new", [(1, 70), (3, 100), (2, 33)], ids=["70-rows", "300-rows", "66-rows"])
def test_prompt_pass_on_the_weight_stationary_kernel_equals_the_pass_on_the_tiled_gemm(batch, l_new):
    """A prompt pass of 66 to 300 rows with every projection on the weight-stationary kernel (forced, tuning key
    21 = 2: activation tiles from the quantizers, weights held in registers, rows in groups of 64) against the same
    pass on the tiled GEMMs (key 21 = 1): int32 sums are exact and the epilogues apply scale, then residual, in the
    same order, so logits, tokens and every cache row must be identical; the verification pass (head over every row)
    as well."""
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    shape = dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=2, d_ffn=1024, vocab=700, batch=batch, ctxs=[0, 9, 40][:batch])
    m = build_model(seed=78, steps=l_new + 2, **shape)
    prompt = o.Rng(7).randint(0, shape["vocab"], batch * l_new).astype(np.int32).reshape(batch, l_new)
    got = {}
    try:
        for rows in (True, False):
            fa.check(lib.fa_set_tuning(21, 2 if rows else 1))
            dec = GpuDecoder(be, m)
            try:
                dec.prefill(prompt)
                got[rows] = (dec.logits().copy(), dec.tokens().copy(), [tuple(x.copy() for x in dec.kv_pool(li)) for li in range(2)])
            finally:
                dec.close()
    finally:
        fa.check(lib.fa_set_tuning(21, 0))
    a, b = got[True], got[False]
    assert np.all(np.isfinite(a[0])) and np.any(a[0] != 0)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    for (ak, av), (bk, bv) in zip(a[2], b[2]):
        assert np.array_equal(ak, bk) and np.array_equal(av, bv)


@pytest.mark.parametrize("shape", [
    dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, d_ffn=512, vocab=1000, batch=3, ctxs=[0, 5, 40], l_new=6),
    dict(n_layers=1, d_model=256, n_heads=2, n_kv_heads=1, d_ffn=256, vocab=300, batch=1, ctxs=[21], l_new=40),
], ids=["B3_L6", "B1_L40"])
def test_verification_pass_matches_the_oracle_at_every_position_and_rewind_drops_the_tail(shape):
    """fa_decoder_verify returns the logits and the greedy token after every fed token: each row is held to
    the oracle decoding the same tokens one by one (chained-step tolerance); the last row is the resident
    result of the pass itself, bit for bit.  After a rewind the dropped positions are decoded again and
    must reproduce the verification's logits for them."""
    be = ops()
    shape = dict(shape)
    l_new = shape.pop("l_new")
    B, V = shape["batch"], shape["vocab"]
    m = build_model(seed=33, steps=l_new + 2, **shape)
    dec = GpuDecoder(be, m)
    try:
        rng = o.Rng(8)
        feed = rng.randint(0, V, B * l_new).astype(np.int32).reshape(B, l_new)
        lens = m.seq_lens.copy()
        want = []
        for t in range(l_new):
            want.append(oracle_step(m, lens, np.ascontiguousarray(feed[:, t])))
        picked, logits = dec.verify(feed)
        assert np.array_equal(dec.seq_lens(), m.seq_lens + l_new)
        assert logits[:, -1].tobytes() == dec.logits().tobytes() and np.array_equal(picked[:, -1], dec.tokens())
        worst = 0.0
        for t, (want_next, want_logits) in enumerate(want):
            spread = want_logits.max(axis=1, keepdims=True) - want_logits.min(axis=1, keepdims=True)
            err = np.abs(logits[:, t] - want_logits) / spread
            worst = max(worst, float(err.max()))
            assert err.mean() < 2e-4 and err.max() < 2e-2, (t, err.mean(), err.max())
            top2 = np.sort(want_logits, axis=1)[:, -2:]
            decisive = (top2[:, 1] - top2[:, 0]) > 4e-2 * spread[:, 0]
            assert np.array_equal(picked[decisive, t], want_next[decisive]), t
            assert np.array_equal(picked[:, t], o.argmax_rows(np.ascontiguousarray(logits[:, t])))
        print("VERIFY_PARITY\tB%d:L%d\tmax_err/range over all positions=%.3e" % (B, l_new, worst), flush=True)
        # drop the last three tokens of every row and decode them again, one step at a time
        keep = l_new - 3
        dec.rewind(m.seq_lens + keep)
        assert np.array_equal(dec.seq_lens(), m.seq_lens + keep)
        for t in range(keep, l_new):
            dec.set_state(m.seq_lens + t, feed[:, t])
            dec.step(True)
            got = dec.logits()
            spread = logits[:, t].max(axis=1, keepdims=True) - logits[:, t].min(axis=1, keepdims=True)
            err = np.abs(got - logits[:, t]) / spread
            assert err.mean() < 2e-4 and err.max() < 2e-2, (t, err.mean(), err.max())
        import fandhe_ai_amd as fa
        with pytest.raises(fa.InvalidArgument):
            dec.rewind(m.seq_lens + l_new + 1)                                # a rewind cannot grow a row
    finally:
        dec.close()


def test_prefill_argument_errors():
    import fandhe_ai_amd as fa
    be = ops()
    m = build_model(seed=1, n_layers=1, d_model=128, n_heads=2, n_kv_heads=1, d_ffn=128, vocab=50, batch=2,
                    ctxs=[3, 4], steps=6)
    dec = GpuDecoder(be, m)
    try:
        room = m.cfg["max_blocks_per_seq"] * 16 - 4
        with pytest.raises(fa.InvalidArgument):
            dec.prefill(np.zeros((2, room + 1), np.int32))                  # no pages for the whole prompt
        with pytest.raises(fa.InvalidArgument):
            dec.prefill(np.full((2, 2), 50, np.int32))                      # token outside the vocabulary
        with pytest.raises(fa.InvalidArgument):
            dec.prefill(np.zeros((2, 0), np.int32))
        assert dec.seq_lens().tolist() == [3, 4]
        dec.prefill(np.zeros((2, 5), np.int32))
        assert dec.seq_lens().tolist() == [8, 9]
    finally:
        dec.close()


def test_graph_replay_is_bit_identical_to_eager():
    be = ops()
    shape = dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, d_ffn=512, vocab=1000, batch=8,
                 ctxs=[7, 33, 64, 100, 5, 18, 250, 31])
    runs = []
    for use_graph in (False, True):
        m = build_model(seed=5, steps=6, **shape)
        dec = GpuDecoder(be, m)
        try:
            outs = []
            for _ in range(5):
                dec.step(use_graph)
                be.synchronize_device()
                outs.append((dec.logits().copy(), dec.tokens().copy(), dec.seq_lens().copy()))
            runs.append(outs)
        finally:
            dec.close()
    for (l0, t0, s0), (l1, t1, s1) in zip(*runs):
        assert np.array_equal(l0, l1) and np.array_equal(t0, t1) and np.array_equal(s0, s1)
    assert runs[0][-1][2].tolist() == [c + 5 for c in shape["ctxs"]]


def test_weight_pull_of_the_row_kernels_changes_no_bit():
    """The blocks appended to the row kernels only read the next projection's weights (an L2 warm-up): with the
    pull off, at its default and at a size that covers whole weights, every step leaves the same logits, tokens
    and lengths, eagerly and replayed; shapes with a ragged last q | k | v tile pair and a single row tile."""
    import fandhe_ai_amd as fa
    be = ops()
    for shape in (dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, d_ffn=512, vocab=1000, batch=8,
                       ctxs=[7, 33, 64, 100, 5, 18, 250, 31]),
                  dict(n_layers=1, d_model=384, n_heads=3, n_kv_heads=1, d_ffn=640, vocab=517, batch=3, ctxs=[1, 40, 17]),
                  dict(n_layers=1, d_model=256, n_heads=2, n_kv_heads=2, d_ffn=256, vocab=300, batch=19, ctxs=list(range(1, 20)))):
        runs = []
        try:
            for pull in (1, 0, 64):
                fa.check(fa.capi.lib.fa_set_tuning(14, pull))
                m = build_model(seed=6, steps=5, **shape)
                dec = GpuDecoder(be, m)
                try:
                    outs = []
                    for step in range(4):
                        dec.step(step >= 2)
                        be.synchronize_device()
                        outs.append((dec.logits().copy(), dec.tokens().copy(), dec.seq_lens().copy()))
                    runs.append(outs)
                finally:
                    dec.close()
        finally:
            fa.check(fa.capi.lib.fa_set_tuning(14, 0))
        for other in runs[1:]:
            for (l0, t0, s0), (l1, t1, s1) in zip(runs[0], other):
                assert np.array_equal(l0, l1) and np.array_equal(t0, t1) and np.array_equal(s0, s1)


def test_decoder_argument_errors():
    import ctypes as C
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    h = C.c_void_p()
    bad = fa.capi.DecoderConfig(1, 256, 4, 2, 64, 512, 100, 16, 8, 32, 4, 1e-5, 500000.0)       # head_dim 64
    assert lib.fa_decoder_create(be._ctx, C.byref(bad), C.byref(h)) == fa.capi.UNSUPPORTED
    bad = fa.capi.DecoderConfig(1, 256, 4, 2, 128, 512, 100, 16, 8, 32, 65, 1e-5, 500000.0)     # batch 65
    assert lib.fa_decoder_create(be._ctx, C.byref(bad), C.byref(h)) == fa.capi.UNSUPPORTED
    m = build_model(seed=1, n_layers=1, d_model=128, n_heads=2, n_kv_heads=1, d_ffn=128, vocab=50, batch=2,
                    ctxs=[3, 4], steps=1)
    dec = GpuDecoder(be, m)
    try:
        t = np.ascontiguousarray(m.tables)
        full = np.array([m.cfg["max_blocks_per_seq"] * 16, 3], dtype=np.uint32)       # no room for one more token
        assert lib.fa_decoder_set_sequences(be._ctx, dec.h, 2, t.ctypes.data_as(fa.capi.u32p),
                                            full.ctypes.data_as(fa.capi.u32p)) == fa.capi.INVALID_ARGUMENT
        tok = np.array([0, 50], dtype=np.int32)
        assert lib.fa_decoder_set_tokens(be._ctx, dec.h, tok.ctypes.data_as(fa.capi.i32p)) == fa.capi.INVALID_ARGUMENT
        wrong = be.import_quantized_weight(np.ones((64, 16), np.int8), np.ones(16, np.float32))
        assert lib.fa_decoder_set_head(dec.h, dec.keep[-3]._h, dec.keep[-2]._h, wrong._h) == fa.capi.SHAPE_MISMATCH
    finally:
        dec.close()


def test_step_without_a_page_for_the_next_position_is_refused():
    """A row that has used up its pages (or whose next table entry is the sentinel) is refused before
    anything is queued, with the row named; lengths and tokens stay as they were (the validators of the
    reference reject a row without a slot before the device is touched,
    crates/tensor-core/src/paged_kv.rs:222-290)."""
    import fandhe_ai_amd as fa
    be = ops()
    # row 0 ends exactly at a page boundary with no further page in its table; row 1 has room
    m = build_model(seed=9, n_layers=1, d_model=256, n_heads=4, n_kv_heads=2, d_ffn=512, vocab=300, batch=2,
                    ctxs=[30, 20], steps=1, threads=2)
    dec = GpuDecoder(be, m)
    try:
        bs = m.cfg["block_size"]
        tables = m.tables.copy()
        owned = int((tables[0] != 0xFFFFFFFF).sum())
        lens = np.array([owned * bs - 1, 20], dtype=np.uint32)
        dec.set_state(lens, m.tokens)
        for use_graph in (False, True):
            dec.step(use_graph)                       # writes the last free slot of row 0
            lens[0:2] += 1
            assert np.array_equal(dec.seq_lens(), lens)
            before = dec.tokens()
            with pytest.raises(fa.InvalidArgument, match="row 0"):
                dec.step(use_graph)
            assert np.array_equal(dec.seq_lens(), lens) and np.array_equal(dec.tokens(), before)
            dec.rewind(lens - 1)
            lens -= 1
    finally:
        dec.close()
