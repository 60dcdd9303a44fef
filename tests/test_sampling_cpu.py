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
