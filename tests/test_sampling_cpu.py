"""Pins of the sampling oracle (oracle/sampling.py): the reference's own unit vectors and closed forms."""
import os
import sys

import numpy as np

import oracle_lib as o

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import sampling as os_  # noqa: E402


def test_reference_unit_vectors():
    # crates/autodiff/src/generate/mod.rs:776-826
    assert os_.greedy_argmax([1.0, 3.0, 3.0, 2.0]) == 1
    assert os_.greedy_argmax([5.0]) == 0
    assert os_.greedy_argmax([-1.0, -2.0, -0.5]) == 2
    w = os_.softmax_weights_f64([1.0, 2.0, 3.0], 1.0)
    assert abs(float(w.sum()) - 1.0) < 1e-5 and (w >= 0).all()
    w = os_.softmax_weights_f64([1e30, 1e30, -1e30], 1.0)
    assert np.isfinite(w).all() and abs(float(w.sum()) - 1.0) < 1e-4
    assert os_.softmax_weights_f64([1.0, 2.0], 0.1)[1] > os_.softmax_weights_f64([1.0, 2.0], 10.0)[1]
    assert os_.top_k_indices([1.0, 5.0, 5.0, 3.0, 0.0], 3) == [1, 2, 3]
    assert os_.top_k_indices([4.0, 1.0, 3.0, 2.0], 1) == [0]
    assert os_.top_k_indices([4.0, 1.0, 3.0, 2.0], 4) == [0, 2, 3, 1]


def test_generator_stream_equals_the_pinned_c_generator():
    for seed in (0, 1, 12345, 0xFFFFFFFFFFFFFFFF):
        g = os_.Generator(seed)
        import ctypes as C
        st = C.c_uint64(o.lib.orc_rng_init(C.c_uint64(seed)))
        o.lib.orc_rng_next_unit_f64.restype = C.c_double
        for _ in range(50):
            assert g.next_unit_f64() == o.lib.orc_rng_next_unit_f64(C.byref(st))
        assert g.state == st.value


def test_softmax_matches_a_float64_library_softmax():
    rng = np.random.default_rng(0)
    for t in (0.5, 1.0, 2.0):
        row = (rng.standard_normal(1000) * 3).astype(np.float32)
        z = (row.astype(np.float64) - row.max()) / float(np.float32(t))
        want = (np.exp(z) / np.exp(z).sum()).astype(np.float32)
        got = os_.softmax_weights_f64(row, t)
        assert np.max(np.abs(got.astype(np.float64) - want)) <= 2e-7 * want.max()


def test_top_k_weights_are_the_softmax_of_the_kept_values_in_place():
    row = np.array([0.5, 3.0, -1.0, 3.0, 2.0, 2.0], np.float32)
    w = os_.sampling_weights_f32(row, os_.TOP_K, 1.0, 3)
    assert (w[[0, 2, 5]] == 0).all()                       # of the two 2.0 only the one with the lower index stays
    kept = os_.softmax_weights_f64([3.0, 3.0, 2.0], 1.0)
    assert np.array_equal(w[[1, 3, 4]], kept)


class _Fixed:
    def __init__(self, u):
        self.u = u

    def next_unit_f64(self):
        return self.u


def test_multinomial_closed_forms():
    w = np.array([0.0, 0.25, 0.0, 0.5, 0.25, 0.0], np.float32)
    assert os_.multinomial_one(_Fixed(0.0), w) == 1       # first index whose cdf exceeds 0: zero weights are skipped
    assert os_.multinomial_one(_Fixed(0.2499999), w) == 1
    assert os_.multinomial_one(_Fixed(0.25), w) == 3       # cdf <= x is passed over: the boundary belongs to the next
    assert os_.multinomial_one(_Fixed(0.7499999), w) == 3
    assert os_.multinomial_one(_Fixed(0.75), w) == 4
    assert os_.multinomial_one(_Fixed(1.0 - 2.0 ** -53), w) == 4
    one_hot = np.zeros(7, np.float32)
    one_hot[5] = 3.0
    g = os_.Generator(9)
    assert all(os_.multinomial_one(g, one_hot) == 5 for _ in range(100))
    # frequencies on dyadic weights converge to the weights
    g = os_.Generator(3)
    draws = np.array([os_.multinomial_one(g, w) for _ in range(20000)])
    freq = np.bincount(draws, minlength=6) / draws.size
    assert np.max(np.abs(freq - w)) < 0.01


def test_sample_step_draws_rows_in_order_from_one_generator():
    rng = np.random.default_rng(1)
    logits = rng.standard_normal((5, 50)).astype(np.float32)
    got = os_.sample_step(logits, os_.TEMPERATURE, 0.8, None, os_.Generator(4))
    g = os_.Generator(4)
    want = [os_.multinomial_one(g, os_.softmax_weights_f64(r, 0.8)) for r in logits]
    assert got.tolist() == want
    assert os_.sample_step(logits, os_.GREEDY).tolist() == logits.argmax(axis=1).tolist()
    bad = logits.copy()
    bad[2, 3] = np.inf
    assert os_.sample_step(bad, os_.TOP_K, 1.0, 5, os_.Generator(0)) is None


# ---------------------------------------------------------------- sampled speculative decoding
def test_speculative_pure_functions_reference_vectors():
    # crates/autodiff/src/generate/speculative.rs:1019-1040
    import pytest
    p = os_.normalize_f64(np.array([0.1, 0.2, 0.3, 0.4], np.float32))
    for px in p:
        assert os_.acceptance_prob_f32(float(px), float(px)) == np.float32(1.0)
    for bad in (lambda: os_.residual_weights_f32(p, p), lambda: os_.residual_weights_f32(p, p[:2]),
                lambda: os_.acceptance_prob_f32(0.3, 0.0), lambda: os_.acceptance_prob_f32(0.3, float("nan")),
                lambda: os_.acceptance_prob_f32(float("nan"), 0.3), lambda: os_.acceptance_prob_f32(-0.1, 0.3),
                lambda: os_.normalize_f64([0.0, 0.0]), lambda: os_.normalize_f64([float("nan"), 1.0]),
                lambda: os_.normalize_f64([-1.0, 2.0])):
        with pytest.raises(os_.SamplingError):
            bad()
    r = os_.residual_weights_f32([0.7, 0.3, 0.0], [0.2, 0.3, 0.5])
    assert r.dtype == np.float32 and r.tolist() == [1.0, 0.0, 0.0]
    # speculative.rs:978-1017: against an independently written f64 form, on the reference's rows
    row_p, row_q = np.array([0.5, 1.5, -0.3, 2.0, 0.1], np.float32), np.array([1.0, 0.2, 0.7, -1.0, 0.4], np.float32)
    for temperature in (0.5, 1.0, 2.0):
        for strategy, k in ((os_.TEMPERATURE, None), (os_.TOP_K, 2), (os_.TOP_K, 3)):
            pw = os_.sampling_weights_f32(row_p, strategy, temperature, k)
            qw = os_.sampling_weights_f32(row_q, strategy, temperature, k)
            p, q = os_.normalize_f64(pw), os_.normalize_f64(qw)
            assert np.array_equal(p, pw.astype(np.float64) / sum(float(x) for x in pw))
            for x in range(5):
                if q[x] <= 0:
                    with pytest.raises(os_.SamplingError):
                        os_.acceptance_prob_f32(float(p[x]), float(q[x]))
                else:
                    assert abs(float(os_.acceptance_prob_f32(float(p[x]), float(q[x]))) - min(p[x] / q[x], 1.0)) < 1e-6
            try:
                res = os_.residual_weights_f32(p, q)
            except os_.SamplingError:
                continue
            raw = np.maximum(p - q, 0.0)
            assert np.allclose(res, raw / raw.sum(), rtol=1e-6, atol=0) and (res[p <= q] == 0).all()


def test_identical_distributions_accept_every_draft_and_draw_once_more_for_the_bonus():
    rng = np.random.default_rng(5)
    for seed in range(1, 40):
        logits = (rng.standard_normal((4, 9)) * 2).astype(np.float32)
        g = os_.Generator(seed)
        q_ws = [os_.sampling_weights_f32(logits[i], os_.TEMPERATURE, 0.8) for i in range(3)]
        drafts = [os_.sample_from(g, w) for w in q_ws]
        twin = os_.Generator(seed)
        for _ in range(3 + 3):                             # three draft draws, three acceptance draws
            twin.next_unit_f64()
        n_acc, tok = os_.verify_sampling(g, logits, drafts, q_ws, os_.TEMPERATURE, 0.8)
        assert n_acc == 3
        assert tok == os_.multinomial_one(twin, os_.sampling_weights_f32(logits[3], os_.TEMPERATURE, 0.8))
        assert g.state == twin.state                       # exactly one bonus draw after the acceptance draws


def test_first_token_of_a_round_is_distributed_as_the_target_whatever_the_draft():
    """The theorem speculative sampling rests on: draft x ~ q, accept with min(1, p/q), else resample from
    max(0, p - q) normalised => the emitted token ~ p.  A dropped clamp, p and q swapped, or a residual taken
    the wrong way round all fail this."""
    p = np.array([0.5, 0.05, 0.25, 0.2])
    q = np.array([0.1, 0.6, 0.05, 0.25])
    lp, lq = np.log(p).astype(np.float32), np.log(q).astype(np.float32)
    logits = np.stack([lp, lp])
    n, counts, accepted = 40000, np.zeros(4), 0
    seeds = np.random.default_rng(123).integers(1, 1 << 63, size=n)       # well-mixed 64-bit generator states
    for seed in seeds:
        g = os_.Generator(int(seed))
        qw = os_.sampling_weights_f32(lq, os_.TEMPERATURE, 1.0)
        d = os_.sample_from(g, qw)
        n_acc, tok = os_.verify_sampling(g, logits, [d], [qw], os_.TEMPERATURE, 1.0)
        counts[d if n_acc == 1 else tok] += 1
        accepted += n_acc
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 16.3, (counts / n, chi2)                 # 3 degrees of freedom, p = 0.001
    want_acc = float(np.minimum(p, q).sum())               # acceptance rate = 1 - total variation distance
    assert abs(accepted / n - want_acc) < 0.01


V7 = 7


def _target_next(t, p):
    # crates/autodiff/src/generate/speculative.rs:546-556
    return (3 * t + p + 1) % V7


def _wrong_next(t, p):
    return (_target_next(t, p) + 1) % V7


def _mixed_next(t, p):
    return _wrong_next(t, p) if p % 3 == 0 else _target_next(t, p)


class _TableModel:
    """speculative.rs:573-651: logits depend on (token, position) only: 10.0 at next(token, position)."""

    def __init__(self, nxt):
        self.nxt, self.calls, self.len = nxt, 0, 0

    def forward_step(self, ids):
        self.calls += 1
        out = np.zeros((len(ids), V7), np.float32)
        for i, t in enumerate(ids):
            out[i, self.nxt(int(t), self.len + i)] = 10.0
        self.len += len(ids)
        return out

    def seq_len(self):
        return self.len

    def truncate(self, n):
        assert n <= self.len
        self.len = n


def _expected(prompt, max_length):
    row = list(prompt)
    while len(row) < max_length:
        row.append(_target_next(row[-1], len(row) - 1))
    return row


def test_speculative_rounds_on_the_reference_table_model():
    # greedy: speculative.rs:672-706 (equal to the rule followed directly, for every draft)
    for nxt in (_target_next, _wrong_next, _mixed_next):
        for t, mx, k in ((3, 12, 1), (2, 12, 3), (3, 6, 8), (3, 4, 8), (3, 5, 8), (1, 9, 2), (4, 4, 3)):
            prompt = [i % V7 for i in range(t)]
            got = os_.generate_speculative(_TableModel(_target_next), _TableModel(nxt), prompt, mx, os_.GREEDY, k=k)
            assert got == _expected(prompt, mx), (nxt.__name__, t, mx, k)
            # speculative.rs:1097-1115: top-k 1 draws from a one-hot distribution and equals greedy
            got = os_.generate_speculative(_TableModel(_target_next), _TableModel(nxt), prompt, mx, os_.TOP_K, 1.0, 1, seed=7, k=k)
            assert got == _expected(prompt, mx), (nxt.__name__, t, mx, k)
    # speculative.rs:1064-1095: an identical draft is accepted throughout: prefill + 2 rounds + the last step
    for strategy, temperature, top_k, seed in ((os_.TEMPERATURE, 0.8, None, 11), (os_.TOP_K, 1.0, 3, 7)):
        target, draft = _TableModel(_target_next), _TableModel(_target_next)
        out = os_.generate_speculative(target, draft, [0, 1], 12, strategy, temperature, top_k, seed, 3)
        assert len(out) == 12 and target.calls == 4
        # speculative.rs:1041-1062: the same seed gives the same row
        again = os_.generate_speculative(_TableModel(_target_next), _TableModel(_mixed_next), [0, 1, 2], 14, strategy,
                                         temperature, top_k, seed, 3)
        assert again == os_.generate_speculative(_TableModel(_target_next), _TableModel(_mixed_next), [0, 1, 2], 14,
                                                 strategy, temperature, top_k, seed, 3) and len(again) == 14
