"""Oracle: next-token sampling from a step's logits.

TEST INFRASTRUCTURE ONLY: a CPU restatement of the reference's host-side sampler, written to be read next to
it; only tests, the smoke check and the benchmark's CPU leg may import it.  The shipped implementation is
the device kernel behind ``fa_sample_rows``.

Follows crates/autodiff/src/generate/mod.rs
  greedy_argmax            333-343   (first maximum)
  softmax_weights_f64      347-355   ((logit - max) / t in f64, exp, sequential f64 sum, cast to f32)
  top_k_indices            359-369   (value descending, index ascending, first k)
  sample_step              376-424   (rows in order, one draw per row from one generator)
  sampling_weights_f32     432-452   (top-k: softmax over the kept values, zeros elsewhere)
and crates/tensor-core/src/rng.rs
  Xorshift64Star           65-79     (seed 0 -> 0x9E3779B97F4A7C15; shifts 13 / 7 / 17; * 0x2545F4914F6CDD1D)
  next_unit_f64            101-104   (top 53 bits / 2^53)
  multinomial_core_with_replacement 509-539 (sequential f64 cumulative sum; x = u * total; first cdf > x;
                                             an index past the end falls to the last positive weight)

Pinned by the reference's unit vectors (generate/mod.rs:776-826) and by closed forms in
tests/test_sampling_cpu.py: one-hot weights, u = 0 and u -> 1 limits, exact frequencies over a full period
of draws on dyadic weights, and the generator stream already pinned for the C++ oracle.
"""
import math

import numpy as np

GREEDY, TEMPERATURE, TOP_K = 0, 1, 2
MASK64 = (1 << 64) - 1


class Generator:
    def __init__(self, seed=0):
        self.state = 0x9E3779B97F4A7C15 if seed == 0 else seed & MASK64

    def next_u64(self):
        x = self.state
        x ^= (x << 13) & MASK64
        x ^= x >> 7
        x ^= (x << 17) & MASK64
        self.state = x
        return (x * 0x2545F4914F6CDD1D) & MASK64

    def next_unit_f64(self):
        return (self.next_u64() >> 11) / float(1 << 53)


def greedy_argmax(row):
    best, best_val = 0, row[0]
    for i in range(1, len(row)):
        if row[i] > best_val:
            best, best_val = i, row[i]
    return best


def softmax_weights_f64(row, temperature):
    mx = -math.inf
    for v in row:
        mx = max(mx, float(v))
    t = float(np.float32(temperature))
    exps = [math.exp((float(v) - mx) / t) for v in row]
    total = 0.0
    for e in exps:
        total += e
    return np.array([e / total for e in exps], dtype=np.float64).astype(np.float32)


def top_k_indices(row, k):
    idx = sorted(range(len(row)), key=lambda i: (-float(row[i]), i))
    return idx[:k]


def sampling_weights_f32(row, strategy, temperature=1.0, k=None):
    if strategy == GREEDY:
        w = np.zeros(len(row), np.float32)
        w[greedy_argmax(row)] = 1.0
        return w
    if strategy == TEMPERATURE:
        return softmax_weights_f64(row, temperature)
    top = top_k_indices(row, k)
    w = np.zeros(len(row), np.float32)
    w[top] = softmax_weights_f64([row[i] for i in top], temperature)
    return w


def multinomial_one(rng, weights):
    """One draw with replacement (rng.rs:509-539)."""
    cdf = np.cumsum(weights.astype(np.float64))          # numpy's cumsum of f64 is the sequential sum
    total = float(cdf[-1])
    positive = np.nonzero(weights > 0)[0]
    last_positive = int(positive[-1]) if positive.size else len(weights) - 1
    x = rng.next_unit_f64() * total
    idx = int(np.searchsorted(cdf, x, side="right"))     # first index with cdf > x
    return last_positive if idx >= len(weights) else idx


def sample_step(logits, strategy, temperature=1.0, k=None, rng=None):
    """logits [B, V] (the last position of every row) -> tokens [B]; None if a logit is not finite
    (the reference returns an error there)."""
    logits = np.asarray(logits, dtype=np.float32)
    if not np.isfinite(logits).all():
        return None
    if strategy == GREEDY:
        return np.array([greedy_argmax(r) for r in logits], dtype=np.int32)
    return np.array([multinomial_one(rng, sampling_weights_f32(r, strategy, temperature, k)) for r in logits],
                    dtype=np.int32)
