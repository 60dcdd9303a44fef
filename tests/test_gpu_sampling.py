"""GPU parity of the device sampler (fa_sample_rows) against the oracle restatement of the reference's
host sampler: the same tokens for the same logits, strategy and generator seed, over consecutive steps
(the generator state advances on the device), with ties in the logits, zero weights, and rows whose
logits are not finite."""
import os
import sys

import numpy as np
import pytest

import oracle_lib as o
from decoder_common import GpuDecoder, build_model
from gpu_common import ops

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import sampling as os_  # noqa: E402

pytestmark = pytest.mark.gpu


def _fa():
    import fandhe_ai_amd as fa
    return fa


def _logits(rng, rows, vocab, kind):
    x = rng.standard_normal((rows, vocab)).astype(np.float32) * 3
    if kind == "ties":
        x = np.round(x)                                    # many equal values: tie-breaking by index matters
    elif kind == "peaked":
        x *= 20                                            # most weights underflow to zero
    elif kind == "flat":
        x[:] = 1.25
    return x


CASES = [(rows, vocab, kind) for rows, vocab in ((1, 17), (5, 1000), (32, 32000), (3, 50257), (2, 1024), (7, 1))
         for kind in ("normal", "ties", "peaked", "flat")]


@pytest.mark.parametrize("rows,vocab,kind", CASES, ids=["%dx%d_%s" % c for c in CASES])
def test_sampled_tokens_equal_the_oracle(rows, vocab, kind):
    fa = _fa()
    be = ops()
    rng = np.random.default_rng(rows * 7 + vocab)
    strategies = [(fa.SAMPLE_TEMPERATURE, 1.0, 0), (fa.SAMPLE_TEMPERATURE, 0.6, 0), (fa.SAMPLE_TEMPERATURE, 1.7, 0),
                  (fa.SAMPLE_TOP_K, 1.0, 1), (fa.SAMPLE_TOP_K, 1.0, min(5, vocab)), (fa.SAMPLE_TOP_K, 0.8, min(50, vocab)),
                  (fa.SAMPLE_TOP_K, 1.0, vocab)]
    for strategy, temperature, k in strategies:
        seed = 11 + k
        gen = be.new_generator(seed)
        ref = os_.Generator(seed)
        for step in range(3):
            x = _logits(rng, rows, vocab, kind)
            got = be.download_owned(be.sample_rows(be.upload(x), strategy, temperature, k, gen))
            want = os_.sample_step(x, strategy, temperature, k or None, ref)
            assert np.array_equal(got, want), (strategy, temperature, k, step, got[:8], want[:8])
        state = be.download(gen)
        assert (int(state[1]) << 32 | int(state[0])) == ref.state


def test_greedy_top1_and_non_finite_rows():
    fa = _fa()
    be = ops()
    rng = np.random.default_rng(3)
    x = np.round(rng.standard_normal((6, 999)).astype(np.float32) * 2)
    greedy = be.download_owned(be.sample_rows(be.upload(x), fa.SAMPLE_GREEDY))
    assert np.array_equal(greedy, o.argmax_rows(x))
    gen = be.new_generator(0)
    top1 = be.download_owned(be.sample_rows(be.upload(x), fa.SAMPLE_TOP_K, 1.0, 1, gen))
    assert np.array_equal(top1, greedy)                    # first maximum, as the reference's ordering keeps it
    bad = x.copy()
    bad[1, 5] = np.nan
    bad[4, 998] = -np.inf
    got = be.download_owned(be.sample_rows(be.upload(bad), fa.SAMPLE_TEMPERATURE, 1.0, 0, gen))
    assert got[1] == -1 and got[4] == -1 and (got[[0, 2, 3, 5]] >= 0).all()
    for args in ((fa.SAMPLE_TEMPERATURE, 0.0, 0), (fa.SAMPLE_TEMPERATURE, float("nan"), 0), (fa.SAMPLE_TOP_K, 1.0, 0),
                 (fa.SAMPLE_TOP_K, 1.0, 1000), (7, 1.0, 0)):
        with pytest.raises(fa.InvalidArgument):
            be.sample_rows(be.upload(x), *args, generator=gen)


def test_decoder_steps_with_sampling_follow_the_oracle_generator():
    fa = _fa()
    be = ops()
    m = build_model(seed=4, n_layers=1, d_model=256, n_heads=2, n_kv_heads=1, d_ffn=256, vocab=700, batch=5,
                    ctxs=[3, 20, 9, 33, 1], steps=12)
    dec = GpuDecoder(be, m)
    try:
        for strategy, temperature, k, seed in ((fa.SAMPLE_TOP_K, 1.0, 40, 5), (fa.SAMPLE_TEMPERATURE, 0.9, 0, 0)):
            dec.set_sampling(strategy, temperature, k, seed)
            ref = os_.Generator(seed)
            for step in range(3):
                dec.step(use_graph=(step > 0))
                want = os_.sample_step(dec.logits(), strategy, temperature, k or None, ref)
                assert np.array_equal(dec.tokens(), want), (strategy, step)
        # the same choice with another seed keeps the captured step and draws from the new generator
        dec.set_sampling(fa.SAMPLE_TEMPERATURE, 0.9, 0, 77)
        ref = os_.Generator(77)
        for step in range(2):
            dec.step(True)
            assert np.array_equal(dec.tokens(), os_.sample_step(dec.logits(), fa.SAMPLE_TEMPERATURE, 0.9, None, ref)), step
        # another temperature re-captures
        dec.set_sampling(fa.SAMPLE_TEMPERATURE, 1.3, 0, 77)
        ref = os_.Generator(77)
        dec.step(True)
        assert np.array_equal(dec.tokens(), os_.sample_step(dec.logits(), fa.SAMPLE_TEMPERATURE, 1.3, None, ref))
        dec.set_sampling(fa.SAMPLE_GREEDY)
        dec.step(False)
        assert np.array_equal(dec.tokens(), o.argmax_rows(dec.logits()))
    finally:
        dec.close()


@pytest.mark.parametrize("rows,vocab,kind", [(9, 1000, "normal"), (32, 32000, "ties"), (6, 17, "peaked"), (5, 300, "flat")])
def test_per_row_policies_draw_from_their_own_generators(rows, vocab, kind):
    """One request per row (fa_sample_rows_per_row): every row follows its own strategy, temperature, k and
    generator; over consecutive calls each generator advances by exactly one draw per sampled token, a greedy
    row draws nothing, and a row with a non-finite logit yields -1."""
    fa = _fa()
    be = ops()
    rng = np.random.default_rng(rows + vocab)
    menu = [(fa.SAMPLE_GREEDY, 1.0, 0), (fa.SAMPLE_TEMPERATURE, 0.7, 0), (fa.SAMPLE_TOP_K, 1.0, min(5, vocab)),
            (fa.SAMPLE_TOP_K, 1.4, 1), (fa.SAMPLE_TEMPERATURE, 1.0, 0), (fa.SAMPLE_TOP_K, 0.5, vocab)]
    records = [menu[r % len(menu)] + (0 if r == 1 else 1000 + 17 * r,) for r in range(rows)]
    table = be.row_sampling_table(records)
    refs = [os_.Generator(seed) for _, _, _, seed in records]
    for step in range(4):
        x = _logits(rng, rows, vocab, kind)
        if step == 2:
            x[rows - 1, vocab // 2] = np.inf
        got = be.download_owned(be.sample_rows_per_row(be.upload(x), table))
        for r, (strategy, temperature, k, _) in enumerate(records):
            if not np.isfinite(x[r]).all():
                assert got[r] == -1                        # and its generator did not move
                continue
            want = os_.sample_step(x[r:r + 1], strategy, temperature, k or None, refs[r])[0]
            assert got[r] == want, (step, r, records[r], got[r], want)
    words = be.download(table).reshape(rows, 6)
    for r, (strategy, _, _, seed) in enumerate(records):
        state = int(words[r, 1]) << 32 | int(words[r, 0])
        assert state == refs[r].state
        if strategy == fa.SAMPLE_GREEDY:
            assert state == os_.Generator(seed).state
