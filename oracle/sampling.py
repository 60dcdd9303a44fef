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

and, for sampled speculative decoding, crates/autodiff/src/generate/speculative.rs
  normalize_f64            111-128   (f32 weights -> f64 probabilities, sequential f64 sum; negative / non-finite /
                                      zero-sum weights are errors)
  acceptance_prob_f32      132-140   (min(1, p / q) in f64, cast to f32; q <= 0 or non-finite is an error)
  residual_weights_f32     144-159   (max(0, p - q) / its f64 sum, cast to f32; a zero sum is an error)
  accept_draw              182-189   with rng.rs:348-355 (one uniform u, accepted when u < f64(a))
  verify_sampling          246-279   (drafts in order: accept, or resample from the residual and stop; all accepted:
                                      one bonus token from the target's next position)
  generate_speculative     334-531   (the round structure, k_eff = min(k, remaining - 1), the caches cut back by
                                      restoring a snapshot and replaying the accepted tokens)

Pinned by the reference's unit vectors (generate/mod.rs:776-826; speculative.rs:1019-1040, 1064-1115) and by
closed forms in tests/test_sampling_cpu.py: one-hot weights, u = 0 and u -> 1 limits, exact frequencies over
a full period of draws on dyadic weights, the generator stream already pinned for the C++ oracle; for the
speculative part: identical distributions accept every draft, the first emitted token of a round is
distributed as the target's p whatever the draft's q (chi-square over many seeds), top-k 1 reproduces the
greedy sequence, and the reference's table model (speculative.rs:546-556, 660-668) yields its expected rows
and its forward-call counts.
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


# ---------------------------------------------------------------- sampled speculative decoding
class SamplingError(ValueError):
    """AutodiffError::InvalidArgument of the sampled path (the reference fails closed)."""


def normalize_f64(weights):
    w = np.asarray(weights, dtype=np.float32)
    if not np.isfinite(w).all() or (w < 0).any():
        raise SamplingError("probability weights are negative or not finite")
    total = float(np.cumsum(w.astype(np.float64))[-1]) if w.size else 0.0      # sequential f64 sum
    if not math.isfinite(total) or total <= 0.0:
        raise SamplingError("probability weights sum to zero or are not finite")
    return w.astype(np.float64) / total


def acceptance_prob_f32(p_x, q_x):
    if not math.isfinite(q_x) or q_x <= 0.0 or not math.isfinite(p_x) or p_x < 0.0:
        raise SamplingError("q(x) is not positive, or a probability is not finite")
    return np.float32(min(max(p_x / q_x, 0.0), 1.0))


def residual_weights_f32(p, q):
    p, q = np.asarray(p, dtype=np.float64), np.asarray(q, dtype=np.float64)
    if p.shape != q.shape:
        raise SamplingError("p and q differ in length")
    r = np.maximum(p - q, 0.0)
    total = float(np.cumsum(r)[-1]) if r.size else 0.0
    if not math.isfinite(total) or total <= 0.0:
        raise SamplingError("the residual distribution sums to zero")
    return (r / total).astype(np.float32)


def accept_draw(rng, a):
    if not (math.isfinite(a) and 0.0 <= a <= 1.0):
        raise SamplingError("acceptance probability outside [0, 1]")
    return rng.next_unit_f64() < float(np.float32(a))


def sample_from(rng, weights):
    """One multinomial draw after the checks of rng.rs (nothing is drawn when a check fails)."""
    w = np.asarray(weights, dtype=np.float32)
    if w.size == 0 or not np.isfinite(w).all() or (w < 0).any():
        raise SamplingError("multinomial weights are empty, negative or not finite")
    if float(np.cumsum(w.astype(np.float64))[-1]) <= 0.0:
        raise SamplingError("multinomial weights sum to zero")
    return multinomial_one(rng, w)


def verify_sampling(rng, logits, drafts, q_ws, strategy, temperature=1.0, k=None):
    """logits [k_eff + 1, V] of the verification pass, drafts [k_eff], q_ws the f32 weights every draft was
    drawn from -> (accepted drafts, the token that follows them)."""
    logits = np.asarray(logits, dtype=np.float32)
    for i, d in enumerate(drafts):
        if not np.isfinite(logits[i]).all():
            raise SamplingError("logits hold non-finite values")
        p = normalize_f64(sampling_weights_f32(logits[i], strategy, temperature, k))
        q = normalize_f64(q_ws[i])
        if not 0 <= d < p.size:
            raise SamplingError("draft token outside the vocabulary")
        if accept_draw(rng, acceptance_prob_f32(float(p[d]), float(q[d]))):
            continue
        return i, sample_from(rng, residual_weights_f32(p, q))
    last = logits[len(drafts)]
    if not np.isfinite(last).all():
        raise SamplingError("logits hold non-finite values")
    return len(drafts), sample_from(rng, sampling_weights_f32(last, strategy, temperature, k))


def generate_speculative(target, draft, prompt, max_length, strategy, temperature=1.0, top_k=None, seed=0, k=1):
    """The round structure of generate_speculative for one sequence.  A model is an object with
    ``forward_step(ids) -> logits [len(ids), V]`` that appends ids to its cache, ``seq_len()`` and
    ``truncate(n)`` (the cache as it was when it held n tokens: the reference's snapshot + restore)."""
    if k < 1:
        raise SamplingError("k must be at least 1")
    row = [int(t) for t in prompt]
    if not row:
        raise SamplingError("the prompt is empty")
    if max_length < len(row):
        raise SamplingError("max_length is below the prompt length")
    if max_length == len(row):
        return row
    sampled = strategy != GREEDY

    def weights(r):
        if not np.isfinite(r).all():
            raise SamplingError("logits hold non-finite values")
        return sampling_weights_f32(r, strategy, temperature, top_k)

    def pick(rng, r):
        if not np.isfinite(r).all():
            raise SamplingError("logits hold non-finite values")
        return sample_from(rng, weights(r)) if sampled else greedy_argmax(r)

    t_logits = np.asarray(target.forward_step(row), dtype=np.float32)
    vocab = t_logits.shape[1]
    if strategy == TOP_K and top_k > vocab:
        raise SamplingError("top-k beyond the vocabulary")
    d_logits = np.asarray(draft.forward_step(row), dtype=np.float32)
    if d_logits.shape[1] != vocab:
        raise SamplingError("the models disagree on the vocabulary")
    rng = Generator(seed) if sampled else None
    row.append(pick(rng, t_logits[-1]))
    while len(row) < max_length:
        cur, last = len(row), row[-1]
        remaining = max_length - cur
        if remaining == 1:
            row.append(pick(rng, np.asarray(target.forward_step([last]), dtype=np.float32)[0]))
            break
        k_eff = min(k, remaining - 1)
        if draft.seq_len() + 1 != cur or target.seq_len() + 1 != cur:
            raise SamplingError("a cache does not hold cur_len - 1 tokens")
        drafts, q_ws, x = [], [], last
        for _ in range(k_eff):
            r = np.asarray(draft.forward_step([x]), dtype=np.float32)[0]
            if sampled:
                w = weights(r)
                x = sample_from(rng, w)
                q_ws.append(w)
            else:
                x = pick(rng, r)
            drafts.append(x)
        logits = np.asarray(target.forward_step([last] + drafts), dtype=np.float32)
        if sampled:
            n_acc, correction = verify_sampling(rng, logits, drafts, q_ws, strategy, temperature, top_k)
        else:
            n_acc = 0
            while True:
                if not np.isfinite(logits[n_acc]).all():
                    raise SamplingError("logits hold non-finite values")
                g = greedy_argmax(logits[n_acc])
                if n_acc < k_eff and drafts[n_acc] == g:
                    n_acc += 1
                else:
                    correction = g
                    break
        row.extend(drafts[:n_acc])
        row.append(int(correction))
        if len(row) >= max_length:
            break
        replay = [last] + drafts[:n_acc]
        if n_acc < k_eff:
            target.truncate(cur - 1)
            target.forward_step(replay)
        if n_acc == k_eff:
            draft.forward_step([x])
        elif n_acc + 1 < k_eff:
            draft.truncate(cur - 1)
            draft.forward_step(replay)
    return row[:max_length]
