"""Autoregressive generation and continuous batching on the resident decoder.

Host-side mirror of the reference's generation layer (crates/autodiff/src/generate/mod.rs:101-215 config and
validation, :500-640 ``generate``; crates/autodiff/src/generate/scheduler.rs:75-127 limits, :445-508 ``submit``,
:521-562 admission, :571-590 ``step``, :712-720 ``take_*``) for a model whose state lives on the device: the KV
pages of all requests share the decoder's pools, every request owns a block-table row, a sampling record with
its own generator (seeded from its config, one draw per generated token) and its token list.  One ``step``
admits queued requests while rows and pages are free, ingests the prompts of the newly admitted requests
(whole prompts; requests that join together share padded passes) and advances all other active requests
together by one decode step of the batch they currently form; requests finish when they reach ``max_length`` (there is no end-of-sequence
stop, as in the reference) and leave the batch between steps.

What differs from the reference, by construction: the decode step is batched on the device (the reference's
opt-in ``step_batched``), so a request's tokens equal a stand-alone ``generate`` of the same request only as
far as its logits are decisive (the attention reduction is split differently when the batch changes); a
request that runs alone is identical to ``generate``.  Pages for the whole ``max_length`` are reserved at
admission, so a request that is admitted can always finish; a request that needs more pages than are free
waits at the head of the queue.
"""
import math
from collections import deque

import numpy as np

from . import capi
from .backend import SAMPLE_GREEDY as GREEDY
from .backend import SAMPLE_TEMPERATURE as TEMPERATURE
from .backend import SAMPLE_TOP_K as TOP_K
from .backend import BackendError, check

lib = capi.lib


class InvalidArgument(ValueError):
    """AutodiffError::InvalidArgument"""


class RankMismatch(ValueError):
    """AutodiffError::Shape(ShapeError::RankMismatch)"""


class SamplingStrategy:
    """``SamplingStrategy::{Greedy, TopK(k), Temperature(t)}`` (generate/mod.rs:101-113)."""

    def __init__(self, kind, value=None):
        self.kind, self.value = kind, value

    @classmethod
    def Greedy(cls):
        return cls(GREEDY)

    @classmethod
    def TopK(cls, k):
        return cls(TOP_K, k)

    @classmethod
    def Temperature(cls, t):
        return cls(TEMPERATURE, t)

    def __eq__(self, other):
        return isinstance(other, SamplingStrategy) and (self.kind, self.value) == (other.kind, other.value)

    def __repr__(self):
        return {GREEDY: "Greedy", TOP_K: "TopK(%r)" % (self.value,), TEMPERATURE: "Temperature(%r)" % (self.value,)}[self.kind]


class GenerateConfig:
    """``GenerateConfig`` (generate/mod.rs:124-168): ``max_length`` counts the prompt; ``temperature`` and
    ``top_k`` are derived from the strategy and may only be changed where the strategy allows it."""

    def __init__(self, max_length, strategy, seed=0):
        self.max_length, self.strategy, self.seed = max_length, strategy, seed
        self.temperature = float(strategy.value) if strategy.kind == TEMPERATURE else 1.0
        self.top_k = strategy.value if strategy.kind == TOP_K else None

    new = classmethod(lambda cls, max_length, strategy: cls(max_length, strategy))

    def with_temperature(self, temperature):
        self.temperature = temperature
        return self

    def with_seed(self, seed):
        self.seed = seed
        return self

    def clone(self):
        c = GenerateConfig(self.max_length, SamplingStrategy(self.strategy.kind, self.strategy.value), self.seed)
        c.temperature, c.top_k = self.temperature, self.top_k
        return c

    def validate(self):
        """generate/mod.rs:170-229: contradictory or non-finite settings are rejected, never repaired."""
        t = self.temperature
        if not (isinstance(t, (int, float)) and math.isfinite(t) and t > 0):
            raise InvalidArgument("GenerateConfig: temperature must be finite and positive (got %r)" % (t,))
        s = self.strategy
        if s.kind == GREEDY:
            if t != 1.0 or self.top_k is not None:
                raise InvalidArgument("GenerateConfig: Greedy requires temperature == 1.0 and top_k == None")
        elif s.kind == TOP_K:
            if self.top_k != s.value:
                raise InvalidArgument("GenerateConfig: TopK(%r) requires top_k == %r" % (s.value, s.value))
            if not isinstance(s.value, int) or s.value < 1:
                raise InvalidArgument("GenerateConfig: TopK needs k >= 1")
        elif s.kind == TEMPERATURE:
            if self.top_k is not None:
                raise InvalidArgument("GenerateConfig: Temperature requires top_k == None")
            if t != s.value:
                raise InvalidArgument("GenerateConfig: Temperature(%r) requires temperature == %r" % (s.value, s.value))
        else:
            raise InvalidArgument("GenerateConfig: unknown strategy")
        if not (isinstance(self.seed, int) and 0 <= self.seed < 1 << 64):
            raise InvalidArgument("GenerateConfig: seed must be a u64")

    def validate_top_k_le_vocab(self, vocab):
        """generate/mod.rs:236-248: k beyond the vocabulary is an error, not clamped."""
        if self.strategy.kind == TOP_K and self.strategy.value > vocab:
            raise InvalidArgument("GenerateConfig: TopK k (%d) exceeds vocab_size (%d)" % (self.strategy.value, vocab))


_I32_BYTES_MAX = (1 << 63) - 1


def _check_buffer_bytes(elems):
    if elems * 4 > _I32_BYTES_MAX:
        raise InvalidArgument("output of %d i32 elements exceeds the allocation limit" % elems)


def _prompt_shape(input_ids, what):
    ids = np.asarray(input_ids)
    if ids.ndim == 1:
        return ids.reshape(1, -1), 1, ids.shape[0], True
    if ids.ndim == 2:
        return ids, ids.shape[0], ids.shape[1], False
    raise RankMismatch("%s: input_ids must be [T] or [B, T] (rank %d)" % (what, ids.ndim))


def _pages_for(max_length, block_size):
    # positions 0 .. max_length - 2 are written (the last generated token is never fed back)
    return max(1, -(-(max_length - 1) // block_size))


def generate(decoder, input_ids, config):
    """``generate`` (generate/mod.rs:500-640) on a resident decoder: prompt pass, then one decode step per
    token until every row holds ``max_length`` tokens.  input_ids [T] or [B, T] int32; returns an int32 array
    of the same rank.  The B rows draw in row order from the one generator ``config.seed`` starts.  Uses
    pages 0 .. of the decoder's pools and replaces whatever sequences were installed."""
    config.validate()
    ids, b, prompt_len, want_rank1 = _prompt_shape(input_ids, "generate")
    if prompt_len == 0:
        raise InvalidArgument("generate: the prompt is empty")
    if b == 0:
        raise InvalidArgument("generate: the batch is empty")
    if config.max_length < prompt_len:
        raise InvalidArgument("generate: max_length (%d) must be at least the prompt length (%d)" % (config.max_length, prompt_len))
    _check_buffer_bytes(b * config.max_length)
    if config.max_length == prompt_len:                    # nothing to generate, no forward pass
        out = np.array(ids, dtype=np.int32)
        return out[0] if want_rank1 else out
    cfg = decoder.cfg
    pages = _pages_for(config.max_length, cfg.block_size)
    if b > cfg.max_batch or pages > cfg.max_blocks_per_seq or b * pages > cfg.num_blocks:
        raise InvalidArgument("generate: %d rows of %d tokens do not fit the decoder's batch or page pool" % (b, config.max_length))
    config.validate_top_k_le_vocab(cfg.vocab)
    out = np.empty((b, config.max_length), dtype=np.int32)
    out[:, :prompt_len] = ids
    tables = np.full((b, cfg.max_blocks_per_seq), 0xFFFFFFFF, dtype=np.uint32)
    tables[:, :pages] = np.arange(b * pages, dtype=np.uint32).reshape(b, pages)
    decoder.set_sequences(tables, np.zeros(b, np.uint32))
    decoder.set_sampling(config.strategy.kind, config.temperature, config.top_k or 0, config.seed)
    decoder.prefill(ids.astype(np.int32))
    for pos in range(prompt_len, config.max_length):
        if pos > prompt_len:
            decoder.step()
        tok = decoder.tokens()
        if (tok < 0).any():
            raise InvalidArgument("generate: logits hold non-finite values")
        out[:, pos] = tok
    return out[0] if want_rank1 else out


class _DeviceAcceptance:
    """The probabilities of sampled speculative decoding, kept on the device: the f32 weight rows of the target
    (k + 1) and of the draft (k), one generator for every draw of the call (speculative.rs:438-447), and the
    acceptance kernel behind ``fa_speculative_accept``.  Only (accepted, token, status) come back to the host."""

    _WHY = {2: "q(x) is not positive, or a probability is not finite", 3: "probability weights are negative, not finite or sum to zero",
            4: "the residual distribution sums to zero", 5: "a draft token lies outside the vocabulary"}

    def __init__(self, be, config, vocab, k):
        self.be, self.vocab = be, vocab
        self.kind, self.temperature, self.top_k = config.strategy.kind, config.temperature, config.top_k or 0
        self.gen = be.new_generator(config.seed)
        self.pw, self.qw = be.alloc_uninit((k + 1, vocab)), be.alloc_uninit((k, vocab))
        self.status, self.result = be.alloc_zeroed((k + 1,), capi.I32), be.alloc_zeroed((4,), capi.I32)

    def close(self):
        for b in (self.gen, self.pw, self.qw, self.status, self.result):
            b.free()

    def _raise_unless_ok(self, status, rows):
        if status == 0:
            return
        if status == 3 and self.be.download(self.status)[:rows].any():
            raise InvalidArgument("generate_speculative: logits hold non-finite values")
        raise InvalidArgument("generate_speculative: " + self._WHY.get(status, "acceptance failed (status %d)" % status))

    def draw(self, logits, row=0, keep_as_q=None):
        """One token from row `row` of `logits` (``sample_from`` over ``sampling_weights_f32``); the weights stay
        behind as draft row `keep_as_q` for the acceptance step when asked."""
        dst, dst_row = (self.pw, 0) if keep_as_q is None else (self.qw, keep_as_q)
        self.be.sampling_weights(logits, 1, self.vocab, self.kind, self.temperature, self.top_k, dst, self.status, row, dst_row)
        _, token, status = self.be.speculative_accept(dst, None, [], self.vocab, self.gen, self.result, p_row=dst_row)
        self._raise_unless_ok(status, 1)
        return token

    def verify(self, logits, drafts):
        """``verify_sampling``: rows 0 .. len(drafts) of `logits` are the verification pass."""
        rows = len(drafts) + 1
        self.be.sampling_weights(logits, rows, self.vocab, self.kind, self.temperature, self.top_k, self.pw, self.status)
        n_acc, token, status = self.be.speculative_accept(self.pw, self.qw, drafts, self.vocab, self.gen, self.result)
        self._raise_unless_ok(status, rows)
        return n_acc, token


def generate_speculative(target, draft, input_ids, config, k):
    """``generate_speculative`` (crates/autodiff/src/generate/speculative.rs:334-531) on two resident decoders:
    per round the draft decodes ``k_eff = min(k, remaining - 1)`` tokens, the target consumes the pending token
    and those drafts in one verification pass, a prefix of the drafts is kept and one more token from the
    target's own distribution is appended.  Greedy: the longest prefix that equals the target's greedy tokens,
    then the target's token at the first disagreement (or after the last draft).  Temperature / top-k:
    standard speculative sampling (draft i is kept with probability min(1, p / q), the first refused one is
    replaced by a draw from max(0, p - q), a fully accepted round ends with a bonus draw), with one generator
    seeded from ``config.seed`` for every draw of the call in the reference's order and all probabilities on
    the device (``fa_sampling_weights`` + ``fa_speculative_accept`` on the decoders' resident logits).
    Both caches are then cut back to the accepted length with ``Decoder.rewind``: paged rows past a sequence's
    length are dead, so nothing is replayed (the reference restores a snapshot and replays the accepted
    tokens, kv_rewind.rs:157-215).  One sequence per call, as in the reference.  When the pending token and
    the drafts fit the decoder's rows (``k + 1 <= min(32, max_batch)``) the verification is one decode step
    whose rows are the k + 1 positions of the one sequence (the same block table in every row, lengths ctx,
    ctx + 1, ...: every row appends its own position and attends to its own prefix), which costs about what a
    single decode step costs; longer look-aheads take the prompt-shape verification pass.  The greedy output
    equals ``generate(target, ...)`` wherever the target's greedy choice is decisive (int32 accumulators are
    identical in every form, attention sums are associated differently when the rows change).
    Returns (tokens, rounds, accepted drafts)."""
    config.validate()
    if not isinstance(k, int) or k < 1:
        raise InvalidArgument("generate_speculative: k must be at least 1")
    ids, b, prompt_len, want_rank1 = _prompt_shape(input_ids, "generate_speculative")
    if prompt_len == 0:
        raise InvalidArgument("generate_speculative: the prompt is empty")
    if b != 1:
        raise InvalidArgument("generate_speculative: one sequence only (got %d)" % b)
    max_length = config.max_length
    if max_length < prompt_len:
        raise InvalidArgument("generate_speculative: max_length (%d) must be at least the prompt length (%d)" % (max_length, prompt_len))
    _check_buffer_bytes(max_length)
    sampled = config.strategy.kind != GREEDY
    row = [int(t) for t in ids[0]]
    rounds = accepted = 0
    by_step = k + 1 <= min(32, target.cfg.max_batch)
    target_table = None
    acc = None
    if max_length > prompt_len:
        if target.cfg.vocab != draft.cfg.vocab:
            raise InvalidArgument("generate_speculative: the models disagree on the vocabulary (%d, %d)" % (draft.cfg.vocab, target.cfg.vocab))
        vocab = target.cfg.vocab
        config.validate_top_k_le_vocab(vocab)
        if sampled and k > 32:
            raise InvalidArgument("generate_speculative: the sampled form verifies at most 32 drafts per round (got %d)" % k)
        for dec in (target, draft):
            cfg = dec.cfg
            pages = _pages_for(max_length + 1, cfg.block_size)     # the verification pass also writes the last draft
            if pages > cfg.max_blocks_per_seq or pages > cfg.num_blocks:
                raise InvalidArgument("generate_speculative: %d tokens do not fit the decoder's page pool" % max_length)
        try:
            if sampled:
                acc = _DeviceAcceptance(target._ops, config, vocab, k)
            for dec in (target, draft):
                cfg = dec.cfg
                pages = _pages_for(max_length + 1, cfg.block_size)
                table = np.full((1, cfg.max_blocks_per_seq), 0xFFFFFFFF, dtype=np.uint32)
                table[0, :pages] = np.arange(pages, dtype=np.uint32)
                dec.set_sequences(table, np.zeros(1, np.uint32))
                dec.set_sampling(GREEDY)                           # the decoders' own picks are not used when sampling
                dec.prefill(ids.astype(np.int32))
                if dec is target:
                    target_table = table

            def pick(dec):
                """The next token from row 0 of a decoder's logits."""
                if sampled:
                    return acc.draw(dec.logits_buffer())
                tok = int(dec.tokens()[0])
                if tok < 0:
                    raise InvalidArgument("generate_speculative: logits hold non-finite values")
                return tok

            row.append(pick(target))
            while len(row) < max_length:
                cur, last = len(row), row[-1]
                remaining = max_length - cur
                if remaining == 1:
                    target.set_tokens([last])
                    target.step()
                    row.append(pick(target))
                    break
                k_eff = min(k, remaining - 1)
                drafts, x = [], last
                for i in range(k_eff):                         # the draft's cache grows by last, d1 .. d_{k_eff - 1}
                    draft.set_tokens([x])
                    draft.step()
                    x = acc.draw(draft.logits_buffer(), 0, keep_as_q=i) if sampled else pick(draft)
                    drafts.append(x)
                picked = staged = None
                if by_step:
                    n = k_eff + 1
                    target.set_sequences(np.repeat(target_table, n, axis=0), np.arange(cur - 1, cur - 1 + n, dtype=np.uint32))
                    target.set_tokens([last] + drafts)
                    target.step()
                    if sampled:
                        logits = target.logits_buffer()
                    else:
                        picked = target.tokens()
                        if (picked < 0).any():
                            raise InvalidArgument("generate_speculative: logits hold non-finite values")
                elif sampled:
                    _, host_logits = target.verify(np.array([[last] + drafts], dtype=np.int32), want_logits=True)
                    logits = staged = target._ops.upload(host_logits[0])
                else:
                    picked = target.verify(np.array([[last] + drafts], dtype=np.int32))[0]
                if sampled:
                    try:
                        n_acc, correction = acc.verify(logits, drafts)
                    finally:
                        if staged is not None:
                            staged.free()
                else:
                    n_acc = 0
                    while n_acc < k_eff and drafts[n_acc] == picked[n_acc]:
                        n_acc += 1
                    correction = int(picked[n_acc])
                row.extend(drafts[:n_acc])
                row.append(correction)
                rounds += 1
                accepted += n_acc
                if len(row) >= max_length:
                    break
                keep = cur + n_acc                             # tokens before the new pending one
                if by_step:
                    target.set_sequences(target_table, np.array([keep], dtype=np.uint32))
                else:
                    target.rewind([keep])
                if n_acc == k_eff:
                    draft.set_tokens([x])                      # the draft never consumed its own last token
                    draft.step()
                else:
                    draft.rewind([keep])
        finally:
            if acc is not None:
                acc.close()
    out = np.array(row[:max_length], dtype=np.int32)
    return (out if want_rank1 else out[None, :]), rounds, accepted


class SchedulerLimits:
    """scheduler.rs:80-127: every limit is mandatory and at least 1."""

    def __init__(self, max_active, max_queued, max_length):
        if min(max_active, max_queued, max_length) < 1:
            raise InvalidArgument("SchedulerLimits: every limit must be at least 1 (max_active=%d, max_queued=%d, max_length=%d)"
                                  % (max_active, max_queued, max_length))
        _check_buffer_bytes(max_length)
        self.max_active, self.max_queued, self.max_length = max_active, max_queued, max_length


class PageAllocator:
    """Page ids of the shared pools: pages that were returned are handed out again last-in first-out, then
    ids never used before in ascending order (the allocation order of the reference's block table,
    crates/autodiff/src/nn/paged_kv.rs:147-191)."""

    def __init__(self, num_blocks):
        self.num_blocks, self._next, self._returned = num_blocks, 0, []

    def free_pages(self):
        return len(self._returned) + self.num_blocks - self._next

    def take(self, n):
        if n > self.free_pages():
            raise InvalidArgument("page pool exhausted")
        out = []
        for _ in range(n):
            if self._returned:
                out.append(self._returned.pop())
            else:
                out.append(self._next)
                self._next += 1
        return out

    def give_back(self, pages):
        self._returned.extend(pages)


class _Pending:
    __slots__ = ("id", "prompt", "config", "want_rank1")

    def __init__(self, rid, prompt, config, want_rank1):
        self.id, self.prompt, self.config, self.want_rank1 = rid, prompt, config, want_rank1


class _Active:
    __slots__ = ("id", "tokens", "pages", "policy", "config", "want_rank1", "fresh")


class BatchScheduler:
    """``BatchScheduler`` (scheduler.rs:395-720) over a resident ``Decoder``."""

    def __init__(self, decoder, limits):
        cfg = decoder.cfg
        if limits.max_active > cfg.max_batch:
            raise InvalidArgument("scheduler: max_active (%d) exceeds the decoder's max_batch (%d)" % (limits.max_active, cfg.max_batch))
        self._dec, self.limits = decoder, limits
        self._queue, self._active, self._finished, self._failed = deque(), [], [], []
        self._next_id = 0
        self._pages = PageAllocator(cfg.num_blocks)
        self._resident = None                              # ids whose decode state is installed on the device, in row order
        # what the device was asked to do so far: prompt passes, their rows incl. padding, decode steps and their rows
        self.stats = {"prompt_passes": 0, "prompt_rows": 0, "decode_steps": 0, "decode_rows": 0}

    def queued_len(self):
        return len(self._queue)

    def active_len(self):
        return len(self._active)

    def free_pages(self):
        return self._pages.free_pages()

    def submit(self, input_ids, config):
        """Queues a request without touching the device; checks in the reference's order (config, rank, empty
        prompt, batch of one, max_length against the prompt and the limit, queue room); on any error the
        scheduler is unchanged.  Returns the request id (ascending)."""
        config.validate()
        ids, b, prompt_len, want_rank1 = _prompt_shape(input_ids, "scheduler")
        if prompt_len == 0:
            raise InvalidArgument("scheduler: the prompt is empty")
        if b != 1:
            raise InvalidArgument("scheduler: one sequence per request (got %d)" % b)
        if config.max_length < prompt_len:
            raise InvalidArgument("scheduler: max_length (%d) must be at least the prompt length (%d)" % (config.max_length, prompt_len))
        if config.max_length > self.limits.max_length:
            raise InvalidArgument("scheduler: max_length (%d) exceeds the limit (%d)" % (config.max_length, self.limits.max_length))
        _check_buffer_bytes(config.max_length)
        if len(self._queue) >= self.limits.max_queued:
            raise InvalidArgument("scheduler: the queue is full (%d)" % self.limits.max_queued)
        rid = self._next_id
        self._next_id += 1
        self._queue.append(_Pending(rid, [int(t) for t in ids[0]], config.clone(), want_rank1))
        return rid

    # ---- one iteration ------------------------------------------------------------------------------------

    def step(self):
        """Admits, ingests new prompts, advances everyone else by one token.  Returns how many requests
        finished successfully in this call; failures of single requests go to ``take_failed``."""
        completed = self._admit()
        n_fin, n_fail = len(self._finished), len(self._failed)
        fresh = [a for a in self._active if a.fresh]
        old = [a for a in self._active if not a.fresh]
        gone = set()
        if fresh:
            self._pull_resident_state()                    # the prompt passes overwrite the installed batch
            for group in self._prompt_groups(fresh):
                try:
                    bad = self._ingest(group)
                except BackendError as e:                  # a device failure takes the whole pass with it
                    for a in group:
                        self._fail(a, e, gone)
                    continue
                for a in group:
                    if a in bad:
                        self._fail(a, InvalidArgument("generate: logits hold non-finite values"), gone)
                    else:
                        completed += self._maybe_finish(a, gone)
        if old:
            try:
                if self._resident != [a.id for a in old]:
                    self._install(old)
                self._dec.step()
                picked = self._dec.tokens()
                self.stats["decode_steps"] += 1
                self.stats["decode_rows"] += len(old)
            except BackendError as e:                      # a device failure takes the whole batch with it
                for a in old:
                    self._fail(a, e, gone)
                self._resident = None
            else:
                for a, tok in zip(old, picked):
                    if tok < 0:
                        self._fail(a, InvalidArgument("generate: logits hold non-finite values"), gone)
                        continue
                    a.tokens.append(int(tok))
                    completed += self._maybe_finish(a, gone)
        if gone:
            self._pull_resident_state(skip=gone)           # the rows move: keep the survivors' generator states
            self._active = [a for a in self._active if a.id not in gone]
        # within one iteration requests are reported in request order, as if they had been advanced one by one
        self._finished[n_fin:] = sorted(self._finished[n_fin:], key=lambda e: e[0])
        self._failed[n_fail:] = sorted(self._failed[n_fail:], key=lambda e: e[0])
        return completed

    def take_finished(self):
        """[(request id, int32 tokens [max_length] or [1, max_length])] in completion order; drains."""
        out, self._finished = self._finished, []
        return out

    def take_failed(self):
        """[(request id, exception)]; drains."""
        out, self._failed = self._failed, []
        return out

    # ---- internals ----------------------------------------------------------------------------------------

    def _admit(self):
        cfg, completed = self._dec.cfg, 0
        while len(self._active) < self.limits.max_active and self._queue:
            p = self._queue[0]
            if p.config.max_length == len(p.prompt):       # nothing to generate: the prompt is the answer
                self._queue.popleft()
                self._finished.append((p.id, self._output(p.prompt, p.want_rank1)))
                completed += 1
                continue
            need = _pages_for(p.config.max_length, cfg.block_size)
            try:
                p.config.validate_top_k_le_vocab(cfg.vocab)
                if need > cfg.max_blocks_per_seq or need > cfg.num_blocks:
                    raise InvalidArgument("scheduler: max_length (%d) needs %d pages, the decoder holds %d per sequence, %d in all"
                                          % (p.config.max_length, need, cfg.max_blocks_per_seq, cfg.num_blocks))
                if any(t < 0 or t >= cfg.vocab for t in p.prompt):
                    raise InvalidArgument("scheduler: prompt token outside the vocabulary")
            except InvalidArgument as e:
                self._queue.popleft()
                self._failed.append((p.id, e))
                continue
            if need > self._pages.free_pages():
                break                                      # waits for pages, in order
            self._queue.popleft()
            a = _Active()
            a.id, a.tokens, a.config, a.want_rank1, a.fresh = p.id, list(p.prompt), p.config, p.want_rank1, True
            a.pages = self._pages.take(need)
            state = capi.u64()
            check(lib.fa_rng_state_from_seed(p.config.seed, state))
            a.policy = (state.value, float(p.config.temperature), int(p.config.top_k or 0), int(p.config.strategy.kind))
            self._active.append(a)
        return completed

    def _table_row(self, a):
        row = np.full(self._dec.cfg.max_blocks_per_seq, 0xFFFFFFFF, dtype=np.uint32)
        row[:len(a.pages)] = a.pages
        return row

    def _policy_rows(self, rows):
        arr = (capi.RowSampling * len(rows))()
        for r, a in zip(arr, rows):
            r.rng_state, r.temperature, r.top_k, r.strategy = a.policy
        return arr

    def _install(self, rows):
        self._pull_resident_state()
        self._dec.set_sequences(np.stack([self._table_row(a) for a in rows]),
                                np.array([len(a.tokens) - 1 for a in rows], dtype=np.uint32))
        self._dec.set_tokens(np.array([a.tokens[-1] for a in rows], dtype=np.int32))
        self._dec.set_row_sampling(self._policy_rows(rows))
        self._resident = [a.id for a in rows]

    def _pull_resident_state(self, skip=()):
        """Generator states advance on the device; fetch them before the installed batch is replaced."""
        if self._resident is None:
            return
        by_id = {a.id: a for a in self._active}
        rows = self._dec.read_row_sampling()
        for rid, r in zip(self._resident, rows):
            a = by_id.get(rid)
            if a is not None and rid not in skip:
                a.policy = (r.rng_state, r.temperature, r.top_k, r.strategy)
        self._resident = None

    MAX_PROMPT_ROWS = 4096                                  # rows (requests x longest prompt) of one padded pass

    def _prompt_groups(self, fresh):
        """Requests that join in the same iteration share prompt passes: sorted by prompt length and cut into
        groups whose padded size stays within one pass and whose longest prompt is at most twice the
        shortest (the padding is computed and thrown away)."""
        groups, cur = [], []
        for a in sorted(fresh, key=lambda a: (len(a.tokens), a.id)):
            n = len(a.tokens)
            if cur and ((len(cur) + 1) * n > self.MAX_PROMPT_ROWS or n > 2 * len(cur[0].tokens)
                        or len(cur) >= self._dec.cfg.max_batch):
                groups.append(cur)
                cur = []
            cur.append(a)
        if cur:
            groups.append(cur)
        return groups

    def _ingest(self, group):
        """One prompt pass for the group; returns the requests whose logits were not finite."""
        self._dec.set_sequences(np.stack([self._table_row(a) for a in group]), np.zeros(len(group), np.uint32))
        self._dec.set_row_sampling(self._policy_rows(group))
        self.stats["prompt_passes"] += 1
        self.stats["prompt_rows"] += len(group) * max(len(a.tokens) for a in group)
        if len(group) == 1:
            self._dec.prefill(np.array([group[0].tokens], dtype=np.int32))
        else:
            self._dec.prefill_padded([np.array(a.tokens, dtype=np.int32) for a in group])
        toks = self._dec.tokens()
        rows = self._dec.read_row_sampling()
        bad = []
        for a, tok, r in zip(group, toks, rows):
            a.policy = (r.rng_state, r.temperature, r.top_k, r.strategy)
            a.fresh = False
            if tok < 0:
                bad.append(a)
            else:
                a.tokens.append(int(tok))
        return bad

    def _maybe_finish(self, a, gone):
        if len(a.tokens) < a.config.max_length:
            return 0
        self._finished.append((a.id, self._output(a.tokens, a.want_rank1)))
        self._pages.give_back(a.pages)
        gone.add(a.id)
        return 1

    def _fail(self, a, err, gone):
        self._failed.append((a.id, err))
        self._pages.give_back(a.pages)
        gone.add(a.id)

    @staticmethod
    def _output(tokens, want_rank1):
        out = np.array(tokens, dtype=np.int32)
        return out if want_rank1 else out[None, :]
