"""Host logic of generation and continuous batching (fandhe_ai_amd/scheduler.py) replayed against the
reference's scheduler tests (crates/autodiff/src/generate/scheduler.rs:866-990) on a toy decoder that keeps
every fed token in a page pool, reads a row's history back through that row's block table, and picks tokens
with the oracle's sampler: a wrong table, length, page reuse or generator state changes the output."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import sampling as osamp  # noqa: E402

import fandhe_ai_amd as fa  # noqa: E402
from fandhe_ai_amd import capi  # noqa: E402
from fandhe_ai_amd.scheduler import (BatchScheduler, GenerateConfig, InvalidArgument, PageAllocator, RankMismatch,  # noqa: E402
                                     SamplingStrategy, SchedulerLimits, generate, generate_speculative)

VOCAB, BLOCK = 11, 16


class Cfg:
    def __init__(self, max_batch, num_blocks, max_blocks_per_seq):
        self.max_batch, self.num_blocks, self.max_blocks_per_seq = max_batch, num_blocks, max_blocks_per_seq
        self.block_size, self.vocab = BLOCK, VOCAB


def toy_logits(history, salt=0):
    """A table-like model: logits depend on every token seen so far and on the position."""
    if callable(salt):
        salt = salt(len(history))
    h = salt
    for i, t in enumerate(history):
        h = (h * 31 + (t + 1) * (i + 7)) % 1000003
    rng = np.random.default_rng(h)
    return rng.standard_normal(VOCAB).astype(np.float32) * 2.0


class ToyDecoder:
    """The surface of fandhe_ai_amd.Decoder that generation uses, on the host."""

    def __init__(self, max_batch=4, num_blocks=8, max_blocks_per_seq=4, salt=0):
        self.cfg = Cfg(max_batch, num_blocks, max_blocks_per_seq)
        self.salt = salt
        self.pool = np.full((num_blocks, BLOCK), -1, dtype=np.int64)
        self.calls = {"prefill": 0, "step": 0, "step_rows": 0}
        self.poison_token = None
        self.batch = 0
        self.per_row = False

    def set_sequences(self, tables, lens):
        self.tables, self.lens = np.array(tables, dtype=np.uint32), np.array(lens, dtype=np.int64)
        self.batch = len(self.lens)
        assert self.tables.shape == (self.batch, self.cfg.max_blocks_per_seq)
        self.cur = None

    def set_tokens(self, tokens):
        self.cur = [int(t) for t in tokens]
        assert len(self.cur) == self.batch

    def set_sampling(self, strategy, temperature=1.0, top_k=0, seed=0):
        self.per_row, self.uniform, self.rng = False, (strategy, temperature, top_k), osamp.Generator(seed)

    def set_row_sampling(self, rows):
        assert len(rows) == self.batch
        self.per_row = True
        self.policy = [[r.rng_state, r.temperature, r.top_k, r.strategy] for r in rows]

    def read_row_sampling(self):
        arr = (capi.RowSampling * self.batch)()
        for r, p in zip(arr, self.policy):
            r.rng_state, r.temperature, r.top_k, r.strategy = p
        return arr

    def _write(self, b, pos, tok):
        page = int(self.tables[b, pos // BLOCK])
        assert page < self.cfg.num_blocks, "position beyond the row's pages"
        self.pool[page, pos % BLOCK] = tok

    def _history(self, b):
        n = int(self.lens[b])
        return [int(self.pool[int(self.tables[b, p // BLOCK]), p % BLOCK]) for p in range(n)]

    def _pick(self):
        out = []
        for b in range(self.batch):
            hist = self._history(b)
            logits = toy_logits(hist, self.salt)
            if self.poison_token is not None and (hist[0], hist[-1]) == self.poison_token:
                out.append(-1)                             # the device reports a non-finite row this way
                continue
            if self.per_row:
                p = self.policy[b]
                g = osamp.Generator(1)
                g.state = p[0]
                tok = osamp.sample_step(logits[None, :], p[3], p[1], p[2], g)[0]
                p[0] = g.state
            else:
                s, t, k = self.uniform
                tok = osamp.sample_step(logits[None, :], s, t, k, self.rng)[0]
            out.append(int(tok))
        self.cur = out

    def prefill(self, prompt):
        self.calls["prefill"] += 1
        prompt = np.asarray(prompt)
        assert prompt.shape[0] == self.batch
        for b in range(self.batch):
            for t in prompt[b]:
                self._write(b, int(self.lens[b]), int(t))
                self.lens[b] += 1
        self._pick()

    def prefill_padded(self, prompts):
        self.calls["prefill"] += 1
        self.calls["padded_rows"] = self.calls.get("padded_rows", 0) + len(prompts)
        assert len(prompts) == self.batch and len(prompts) * max(len(p) for p in prompts) <= 4096
        for b, p in enumerate(prompts):
            for t in p:
                self._write(b, int(self.lens[b]), int(t))
                self.lens[b] += 1
        self._pick()

    def step(self, use_graph=True):
        self.calls["step"] += 1
        self.calls["step_rows"] += self.batch
        for b in range(self.batch):
            self._write(b, int(self.lens[b]), self.cur[b])
            self.lens[b] += 1
        self._pick()

    def tokens(self):
        return np.array(self.cur, dtype=np.int32)

    def verify(self, tokens):
        self.calls["verify"] = self.calls.get("verify", 0) + 1
        tokens = np.asarray(tokens)
        picked = np.empty(tokens.shape, dtype=np.int32)
        for b in range(self.batch):
            for i, t in enumerate(tokens[b]):
                self._write(b, int(self.lens[b]), int(t))
                self.lens[b] += 1
                picked[b, i] = osamp.greedy_argmax(toy_logits(self._history(b), self.salt))
        self.cur = [int(p[-1]) for p in picked]
        return picked

    def rewind(self, lens):
        lens = np.asarray(lens, dtype=np.int64)
        assert (lens <= self.lens).all(), "a rewind cannot grow a sequence"
        self.lens = lens.copy()


def cfg(max_length, strategy, seed):
    return GenerateConfig.new(max_length, strategy).with_seed(seed)


def run_to_end(s, limit=200):
    done = []
    for _ in range(limit):
        if s.active_len() == 0 and s.queued_len() == 0:
            break
        s.step()
        done += s.take_finished()
    assert s.active_len() == 0 and s.queued_len() == 0
    return done


def test_config_validation_matches_the_reference_rules():
    G, T, K = SamplingStrategy.Greedy, SamplingStrategy.Temperature, SamplingStrategy.TopK
    c = GenerateConfig.new(4, K(3))
    assert (c.temperature, c.top_k, c.seed) == (1.0, 3, 0)
    c.with_temperature(0.7).validate()                     # top-k with a temperature is allowed
    GenerateConfig.new(4, T(0.8)).validate()
    for bad in (GenerateConfig.new(4, G()).with_temperature(2.0), GenerateConfig.new(4, T(0.8)).with_temperature(0.9),
                GenerateConfig.new(4, T(0.0)), GenerateConfig.new(4, T(float("nan"))), GenerateConfig.new(4, T(float("inf"))),
                GenerateConfig.new(4, T(-1.0)), GenerateConfig.new(4, K(0))):
        with pytest.raises(InvalidArgument):
            bad.validate()
    c = GenerateConfig.new(4, K(3))
    c.top_k = 2
    with pytest.raises(InvalidArgument):
        c.validate()
    with pytest.raises(InvalidArgument):
        GenerateConfig.new(4, K(VOCAB + 1)).validate_top_k_le_vocab(VOCAB)
    GenerateConfig.new(4, K(VOCAB)).validate_top_k_le_vocab(VOCAB)


def test_limits_reject_zero_and_huge():
    for bad in ((0, 1, 1), (1, 0, 1), (1, 1, 0), (1, 1, (1 << 64) - 1), (1, 1, ((1 << 63) - 1) // 4 + 1)):
        with pytest.raises(InvalidArgument):
            SchedulerLimits(*bad)
    lim = SchedulerLimits(2, 3, 4)
    assert (lim.max_active, lim.max_queued, lim.max_length) == (2, 3, 4)
    with pytest.raises(InvalidArgument):                   # more rows than the decoder has
        BatchScheduler(ToyDecoder(max_batch=2), SchedulerLimits(3, 1, 8))


def test_submit_rejections_leave_state_unchanged():
    s = BatchScheduler(ToyDecoder(), SchedulerLimits(1, 2, 6))
    g = cfg(4, SamplingStrategy.Greedy(), 0)
    with pytest.raises(InvalidArgument):
        s.submit([1], cfg(4, SamplingStrategy.Greedy(), 0).with_temperature(2.0))
    with pytest.raises(RankMismatch):
        s.submit(np.array([[[1, 2]]]), g)
    with pytest.raises(InvalidArgument):
        s.submit(np.array([], dtype=np.int32), g)
    with pytest.raises(InvalidArgument):
        s.submit(np.array([[1], [2]]), g)
    with pytest.raises(InvalidArgument):
        s.submit([1, 2, 3, 4, 5], g)
    with pytest.raises(InvalidArgument):
        s.submit([1], cfg(7, SamplingStrategy.Greedy(), 0))
    assert s.queued_len() == 0
    a = s.submit([1], g)
    b = s.submit([1], g)
    assert a < b                                            # ids ascend
    with pytest.raises(InvalidArgument):
        s.submit([1], g)
    assert s.queued_len() == 2


def test_admission_is_bounded_by_max_active():
    m = ToyDecoder()
    s = BatchScheduler(m, SchedulerLimits(1, 2, 6))
    g = cfg(3, SamplingStrategy.Greedy(), 0)
    s.submit([1], g)
    s.submit([2], g)
    s.step()
    assert m.calls["prefill"] == 1 and m.calls["step"] == 0
    assert (s.active_len(), s.queued_len()) == (1, 1)
    done = s.take_finished() + run_to_end(s)
    assert len(done) == 2 and done[0][0] < done[1][0]


def test_prompt_only_request_finishes_without_forward_and_empty_step_is_free():
    m = ToyDecoder()
    s = BatchScheduler(m, SchedulerLimits(1, 1, 6))
    assert s.step() == 0
    s.submit(np.array([[3, 4]]), cfg(2, SamplingStrategy.Greedy(), 0))
    assert s.step() == 1
    assert m.calls == {"prefill": 0, "step": 0, "step_rows": 0}
    done = s.take_finished()
    assert done[0][1].shape == (1, 2) and done[0][1].tolist() == [[3, 4]]
    assert s.take_finished() == []


def test_interleaved_requests_match_single_generate():
    reqs = [([1, 2], cfg(6, SamplingStrategy.Greedy(), 0)),
            (np.array([[3]]), cfg(5, SamplingStrategy.TopK(3), 7)),
            ([5, 6, 7], cfg(7, SamplingStrategy.Temperature(0.8), 11)),
            ([9] * 20, cfg(40, SamplingStrategy.TopK(4), 0).with_temperature(0.5)),      # crosses page boundaries
            ([4, 4], cfg(9, SamplingStrategy.Temperature(1.3), 2 ** 64 - 1))]
    m = ToyDecoder(max_batch=3, num_blocks=6, max_blocks_per_seq=3)
    s = BatchScheduler(m, SchedulerLimits(3, 8, 40))
    ids = [s.submit(i, c) for i, c in reqs]
    done = dict((rid, out) for rid, out in run_to_end(s))
    assert len(done) == len(reqs) and s.take_failed() == []
    for rid, (i, c) in zip(ids, reqs):
        want = generate(ToyDecoder(), i, c)
        assert done[rid].shape == want.shape and done[rid].tolist() == want.tolist()
    assert m.calls["step_rows"] > m.calls["step"]          # decode steps really ran several requests at once
    assert m.calls.get("padded_rows", 0) >= 2              # and requests that joined together shared a prompt pass
    assert s.free_pages() == 6                             # every page came back


def test_generate_matches_a_direct_loop_and_batches_draw_in_row_order():
    prompt = np.array([[1, 2, 3], [4, 5, 6]])
    c = cfg(8, SamplingStrategy.Temperature(0.9), 5)
    got = generate(ToyDecoder(), prompt, c)
    # each row's next token is drawn from the logits of its history before this round's appends
    rng = osamp.Generator(5)
    rows = [list(r) for r in prompt]
    while len(rows[0]) < 8:
        nxt = [int(osamp.sample_step(toy_logits(r)[None, :], 1, 0.9, None, rng)[0]) for r in rows]
        for r, t in zip(rows, nxt):
            r.append(t)
    assert got.tolist() == rows
    assert generate(ToyDecoder(), [7, 8], cfg(2, SamplingStrategy.Greedy(), 0)).tolist() == [7, 8]
    with pytest.raises(InvalidArgument):
        generate(ToyDecoder(), [1, 2, 3], cfg(2, SamplingStrategy.Greedy(), 0))
    with pytest.raises(InvalidArgument):
        generate(ToyDecoder(max_blocks_per_seq=1), [1], cfg(40, SamplingStrategy.Greedy(), 0))
    with pytest.raises(InvalidArgument):
        generate(ToyDecoder(), [1], cfg(4, SamplingStrategy.TopK(VOCAB + 1), 0))


def test_failure_is_isolated_to_one_request():
    base = generate(ToyDecoder(), [2], cfg(8, SamplingStrategy.TopK(1), 3)).tolist()
    other = generate(ToyDecoder(), [1], cfg(8, SamplingStrategy.TopK(1), 3)).tolist()
    assert base != other
    m = ToyDecoder()
    m.poison_token = (2, base[4])                          # the request that started with 2 fails on a decode step
    s = BatchScheduler(m, SchedulerLimits(2, 4, 8))
    a = s.submit([1], cfg(8, SamplingStrategy.TopK(1), 3))
    c = s.submit([2], cfg(8, SamplingStrategy.TopK(1), 3))
    done = run_to_end(s)
    failed = s.take_failed()
    assert [rid for rid, _ in done] == [a] and done[0][1].tolist() == other
    assert [rid for rid, _ in failed] == [c] and isinstance(failed[0][1], InvalidArgument)
    assert s.free_pages() == m.cfg.num_blocks


def test_requests_wait_for_pages_and_impossible_ones_fail():
    m = ToyDecoder(max_batch=4, num_blocks=3, max_blocks_per_seq=2)
    s = BatchScheduler(m, SchedulerLimits(4, 8, 64))
    big = cfg(33, SamplingStrategy.Greedy(), 0)            # 32 written positions: two pages
    a, b = s.submit([1], big), s.submit([2], big)
    never = s.submit([3], cfg(34, SamplingStrategy.Greedy(), 0))     # three pages: more than a row's table holds
    bad_tok = s.submit([VOCAB], cfg(4, SamplingStrategy.Greedy(), 0))
    bad_k = s.submit([1], cfg(4, SamplingStrategy.TopK(VOCAB + 1), 0))
    s.step()
    assert (s.active_len(), s.queued_len()) == (1, 4)      # b waits for pages behind a
    done = dict(run_to_end(s))
    assert set(done) == {a, b}
    assert done[b].tolist() == generate(ToyDecoder(), [2], big).tolist()
    assert sorted(rid for rid, _ in s.take_failed()) == [never, bad_tok, bad_k]


def test_page_allocator_reuses_returned_pages_last_in_first_out():
    p = PageAllocator(6)
    assert p.take(3) == [0, 1, 2]
    p.give_back([0, 1])
    assert p.take(3) == [1, 0, 3] and p.free_pages() == 2
    with pytest.raises(InvalidArgument):
        p.take(3)


def test_rng_state_from_seed_is_the_generator_rule():
    for seed in (0, 1, 12345, 2 ** 64 - 1):
        st = capi.u64()
        assert capi.lib.fa_rng_state_from_seed(seed, st) == 0
        assert st.value == osamp.Generator(seed).state
    assert fa.scheduler.GREEDY == osamp.GREEDY and fa.scheduler.TOP_K == osamp.TOP_K


def test_speculative_greedy_equals_plain_generation_whatever_the_draft_proposes():
    # crates/autodiff/src/generate/speculative.rs tests: a draft that agrees, one that never does, one that
    # agrees on two positions out of three
    greedy = SamplingStrategy.Greedy()
    drafts = {"same": 0, "wrong": 12345, "mixed": lambda n: 12345 if n % 3 == 0 else 0}
    for prompt, max_length in (([3], 2), ([1, 2], 30), ([4] * 17, 40), ([5, 6, 7], 4), ([2], 3)):
        want = generate(ToyDecoder(), prompt, cfg(max_length, greedy, 0))
        for name, salt in drafts.items():
            for k in (1, 2, 4, 7):
                target, draft = ToyDecoder(num_blocks=4), ToyDecoder(num_blocks=4, salt=salt)
                got, rounds, accepted = generate_speculative(target, draft, prompt, cfg(max_length, greedy, 0), k)
                assert got.tolist() == want.tolist(), (prompt, max_length, name, k)
                new = max_length - len(prompt)
                if name == "same" and new > 2:
                    assert accepted > 0
                    if k + 1 <= target.cfg.max_batch:      # verification by one decode step over k + 1 rows
                        assert target.calls.get("verify", 0) == 0 and target.calls["step"] <= rounds + 1
                    else:                                  # verification by the prompt-shape pass
                        assert target.calls["verify"] == rounds and target.calls["step"] <= 1
                    assert rounds <= -(-new // (k + 1)) + 1
                assert 0 <= accepted <= new and rounds <= max(new - 1, 0)
    got, _, _ = generate_speculative(ToyDecoder(), ToyDecoder(), np.array([[1, 2]]), cfg(9, greedy, 0), 3)
    assert got.shape == (1, 9)
    got, rounds, _ = generate_speculative(ToyDecoder(), ToyDecoder(), [1, 2], cfg(2, greedy, 0), 3)
    assert got.tolist() == [1, 2] and rounds == 0


def test_speculative_argument_errors():
    greedy = SamplingStrategy.Greedy()
    T, D = ToyDecoder, ToyDecoder
    with pytest.raises(InvalidArgument):
        generate_speculative(T(), D(), [1], cfg(4, greedy, 0), 0)
    with pytest.raises(InvalidArgument):
        generate_speculative(T(), D(), np.array([[1], [2]]), cfg(4, greedy, 0), 2)
    with pytest.raises(InvalidArgument):
        generate_speculative(T(), D(), np.array([], dtype=np.int32), cfg(4, greedy, 0), 2)
    with pytest.raises(InvalidArgument):
        generate_speculative(T(), D(), [1, 2, 3], cfg(2, greedy, 0), 2)
    with pytest.raises(RankMismatch):
        generate_speculative(T(), D(), np.zeros((1, 1, 2), np.int32), cfg(4, greedy, 0), 2)
    with pytest.raises(InvalidArgument):                   # the sampled form: k beyond what one acceptance call takes
        generate_speculative(T(), D(), [1], cfg(4, SamplingStrategy.TopK(2), 0), 33)
    with pytest.raises(InvalidArgument):                   # speculative.rs:1117-1131: top-k beyond the vocabulary
        generate_speculative(T(), D(), [1], cfg(4, SamplingStrategy.TopK(VOCAB + 1), 0), 2)
    with pytest.raises(InvalidArgument):                   # a sequence longer than the page table of one model
        generate_speculative(T(), D(max_blocks_per_seq=1), [1], cfg(40, greedy, 0), 2)


@pytest.mark.parametrize("seed", range(6))
def test_random_arrivals_conserve_pages_and_match_single_generation(seed):
    """Requests of random length and strategy arrive at random iterations into a small decoder (few rows, few
    pages): whatever the interleaving, every request ends with exactly the tokens it gets alone, rows and pages
    never exceed their limits, and every page is back at the end."""
    rng = np.random.default_rng(100 + seed)
    S = SamplingStrategy
    max_active = int(rng.integers(1, 4))
    m = ToyDecoder(max_batch=3, num_blocks=int(rng.integers(3, 7)), max_blocks_per_seq=3)
    s = BatchScheduler(m, SchedulerLimits(max_active, 64, 48))
    todo = []
    for _ in range(int(rng.integers(5, 14))):
        plen = int(rng.integers(1, 20))
        max_length = plen + int(rng.integers(0, 28))
        strategy = (S.Greedy(), S.Temperature(float(rng.uniform(0.3, 2.0))), S.TopK(int(rng.integers(1, VOCAB + 1))))[int(rng.integers(0, 3))]
        c = cfg(max_length, strategy, int(rng.integers(0, 2 ** 63)))
        if strategy.kind == fa.scheduler.TOP_K and rng.random() < 0.5:
            c = c.with_temperature(float(rng.uniform(0.3, 2.0)))
        todo.append((int(rng.integers(0, 25)), rng.integers(0, VOCAB, plen).astype(np.int32), c))
    todo.sort(key=lambda e: e[0])
    submitted, done = {}, {}
    for it in range(600):
        while todo and todo[0][0] <= it:
            _, prompt, c = todo.pop(0)
            submitted[s.submit(prompt, c)] = (prompt, c)
        if not todo and s.active_len() == 0 and s.queued_len() == 0:
            break
        s.step()
        assert s.active_len() <= max_active and 0 <= s.free_pages() <= m.cfg.num_blocks
        used = [p for a in s._active for p in a.pages]
        assert len(used) == len(set(used)) == m.cfg.num_blocks - s.free_pages()          # no page is shared or lost
        done.update(dict(s.take_finished()))
    assert s.take_failed() == [] and sorted(done) == sorted(submitted)
    assert s.free_pages() == m.cfg.num_blocks
    for rid, (prompt, c) in submitted.items():
        assert done[rid].tolist() == generate(ToyDecoder(), prompt, c).tolist(), rid
