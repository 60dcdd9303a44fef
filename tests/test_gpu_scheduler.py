"""Continuous batching on the resident decoder (fandhe_ai_amd/scheduler.py) on the GPU.

What is checked, and against what:
* every token a request receives is the oracle sampler's pick (oracle/sampling.py, the reference's host
  sampler) from the logits the decoder produced for that request at that step, with the request's own
  strategy and its own generator stream, in a batch whose composition changes while it runs;
* those logits equal the logits of the same request generated alone (`generate`), within the chained-step
  bar used for the decode step (mean error below 2e-4 of the logit range), for as long as the two token
  histories agree, which pins block tables, lengths, page reuse and row moves;
* a scheduler that runs one request at a time returns exactly `generate`'s tokens;
* replaying cached step graphs across batch-size changes, and across a growth of the attention workspace,
  gives bit-identical logits to eager launches.
"""
import os
import sys

import numpy as np
import pytest
from safetensors.numpy import save as st_save

from gpu_common import ops
from decoder_common import llama_checkpoint as _checkpoint

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import sampling as osamp  # noqa: E402

pytestmark = pytest.mark.gpu

L, D, HEADS, KV, F, VOCAB = 2, 256, 2, 1, 512, 320
_model = None


def _decoder(**geometry):
    import fandhe_ai_amd as fa
    global _model
    if _model is None:
        _model = st_save(_checkpoint(31, L, D, HEADS, KV, F, VOCAB))
    dec, store = fa.safetensors_io.load_decoder(ops(), _model, L, HEADS, KV, **geometry)
    store.free()
    return dec


def _recording(dec):
    """Wraps a decoder so that every prompt pass and step leaves (table row, logits row, picked token)."""
    import fandhe_ai_amd as fa

    class Recording(fa.Decoder):
        def set_sequences(self, tables, lens):
            self.rows = [tuple(int(x) for x in r) for r in np.asarray(tables)]
            super().set_sequences(tables, lens)

        def _record(self, kind, prompts=None):
            logits, toks = self.logits(), self.tokens()
            for r, row in enumerate(self.rows):
                tag = kind if prompts is None else (kind, tuple(int(t) for t in prompts[r]))
                self.trace.append((tag, row, logits[r].copy(), int(toks[r])))

        def prefill(self, prompt):
            super().prefill(prompt)
            self._record("prefill", list(np.asarray(prompt)))

        def prefill_padded(self, prompts):
            super().prefill_padded(prompts)
            self.padded_passes = getattr(self, "padded_passes", 0) + 1
            self._record("prefill", prompts)

        def step(self, use_graph=True):
            super().step(use_graph)
            self._record("step")

    dec.__class__ = Recording
    dec.trace, dec.rows = [], []
    return dec


def _cfg(max_length, strategy, seed):
    from fandhe_ai_amd.scheduler import GenerateConfig
    return GenerateConfig.new(max_length, strategy).with_seed(seed)


def _requests():
    from fandhe_ai_amd.scheduler import SamplingStrategy as S
    rng = np.random.default_rng(77)
    spec = [(1, 9, S.Greedy(), 0), (30, 60, S.TopK(5), 7), (2, 20, S.Temperature(0.8), 11), (17, 33, S.Greedy(), 0),
            (5, 48, S.TopK(40), 0), (12, 13, S.Temperature(1.5), 2 ** 63 + 5), (2, 2, S.Greedy(), 0), (8, 40, S.TopK(1), 3)]
    out = []
    for plen, max_length, strategy, seed in spec:
        cfg = _cfg(max_length, strategy, seed)
        if strategy.kind == 2 and strategy.value == 40:
            cfg = cfg.with_temperature(0.6)
        out.append((rng.integers(0, VOCAB, plen).astype(np.int32), cfg))
    return out


def _split_by_request(trace, reqs_by_prompt):
    """trace entries -> {request: [(logits, token)]}: a prompt pass names the request by its table row, which
    stays its row until it finishes."""
    owner, per = {}, {}
    for kind, row, logits, tok in trace:
        if kind[0] == "prefill":
            owner[row] = reqs_by_prompt[kind[1]]
        per.setdefault(owner[row], []).append((logits, tok))
    return per


def test_scheduler_tokens_are_the_oracle_picks_and_logits_match_stand_alone_generation():
    from fandhe_ai_amd.scheduler import BatchScheduler, SchedulerLimits, generate
    geometry = dict(max_blocks_per_seq=4, num_blocks=10, max_batch=4)
    dec = _recording(_decoder(**geometry))
    reqs = _requests()
    s = BatchScheduler(dec, SchedulerLimits(3, 16, 64))
    ids = [s.submit(p, c) for p, c in reqs]

    by_prompt = {tuple(int(t) for t in p): rid for rid, (p, _) in zip(ids, reqs)}      # the prompts are all different

    done, sizes = {}, []
    for _ in range(400):
        if s.active_len() == 0 and s.queued_len() == 0:
            break
        s.step()
        sizes.append(s.active_len())
        done.update(dict(s.take_finished()))
    assert s.take_failed() == [] and sorted(done) == ids and s.free_pages() == 10
    assert max(sizes) == 3 and len(set(sizes)) > 2          # the batch really changed size while running
    assert getattr(dec, "padded_passes", 0) >= 1            # requests that joined together shared a prompt pass
    per = _split_by_request(dec.trace, by_prompt)

    # (1) tokens = oracle picks from the produced logits, own generator stream per request
    for rid, (prompt, cfg) in zip(ids, reqs):
        out = done[rid]
        assert out.shape == (cfg.max_length,) and np.array_equal(out[:len(prompt)], prompt)
        steps = per.get(rid, [])
        assert len(steps) == cfg.max_length - len(prompt)
        gen = osamp.Generator(cfg.seed)
        for i, (logits, tok) in enumerate(steps):
            want = osamp.sample_step(logits[None, :], cfg.strategy.kind, cfg.temperature, cfg.top_k, gen)[0]
            assert tok == want == out[len(prompt) + i], (rid, i, tok, want)

    # (2) the same requests alone: same logits while the histories agree
    alone = _recording(_decoder(**geometry))
    compared = total = 0
    for rid, (prompt, cfg) in zip(ids, reqs):
        alone.trace = []
        want = generate(alone, prompt, cfg)
        mine = per.get(rid, [])
        total += len(mine)
        for i, ((kind, _, logits, tok), (got_logits, got_tok)) in enumerate(zip(alone.trace, mine)):
            spread = float(logits.max() - logits.min())
            err = np.abs(got_logits - logits) / spread
            assert err.mean() < 2e-4 and err.max() < 2e-2, (rid, i, err.mean(), err.max())
            compared += 1
            if got_tok != tok:
                break                                      # an indecisive pick: the histories part here
        if len(mine) == 0:
            assert np.array_equal(want, done[rid])
    print("SCHEDULER_PARITY\tcompared %d of %d generated tokens against stand-alone generation" % (compared, total), flush=True)
    assert compared >= 0.8 * total
    dec.close()
    alone.close()


def test_one_request_at_a_time_equals_generate_exactly():
    from fandhe_ai_amd.scheduler import BatchScheduler, SchedulerLimits, generate
    geometry = dict(max_blocks_per_seq=4, num_blocks=6, max_batch=2)
    dec = _decoder(**geometry)
    reqs = _requests()
    s = BatchScheduler(dec, SchedulerLimits(1, 16, 64))
    ids = [s.submit(p[None, :], c) for p, c in reqs]
    done = {}
    for _ in range(400):
        if s.active_len() == 0 and s.queued_len() == 0:
            break
        s.step()
        done.update(dict(s.take_finished()))
    assert s.take_failed() == [] and sorted(done) == ids
    for rid, (prompt, cfg) in zip(ids, reqs):
        want = generate(dec, prompt[None, :], cfg)
        assert done[rid].shape == want.shape == (1, cfg.max_length)
        assert np.array_equal(done[rid], want), rid
    # generate with several rows: each row equals its own oracle-checked stream is covered above; here the shape
    both = generate(dec, np.stack([reqs[2][0], reqs[2][0]]), _cfg(12, reqs[0][1].strategy, 0))
    assert both.shape == (2, 12) and np.array_equal(both[0], both[1])
    dec.close()


def test_cached_step_graphs_survive_batch_changes_and_workspace_growth():
    geometry = dict(max_blocks_per_seq=32, num_blocks=128, max_batch=4)
    dec = _decoder(**geometry)
    rng = np.random.default_rng(5)
    tables = np.arange(4 * 32, dtype=np.uint32).reshape(4, 32)
    p2 = rng.integers(0, VOCAB, (2, 5)).astype(np.int32)
    p_long = rng.integers(0, VOCAB, (2, 400)).astype(np.int32)

    def run(use_graph):
        seen = []
        dec.set_sequences(tables[:2], np.zeros(2, np.uint32))
        dec.prefill(p2)
        for _ in range(2):
            dec.step(use_graph)
            seen.append(dec.logits().copy())
        tok2 = dec.tokens().copy()
        dec.set_sequences(tables[2:4], np.zeros(2, np.uint32))      # a long prompt: the attention workspace grows
        dec.prefill(p_long)
        tok_long = dec.tokens().copy()
        dec.set_sequences(tables[:3], np.array([7, 7, 400], np.uint32))
        dec.set_tokens(np.concatenate([tok2, tok_long[:1]]))
        for _ in range(2):
            dec.step(use_graph)
            seen.append(dec.logits().copy())
        tok3 = dec.tokens().copy()
        dec.set_sequences(tables[:2], np.array([9, 9], np.uint32))  # back to two rows: the first graph again
        dec.set_tokens(tok3[:2])
        for _ in range(2):
            dec.step(use_graph)
            seen.append(dec.logits().copy())
        assert dec.seq_lens().tolist() == [11, 11]
        return seen

    eager = run(False)
    graph = run(True)
    again = run(True)                                      # every graph comes from the cache this time
    for a, b, c in zip(eager, graph, again):
        assert np.isfinite(a).all() and a.tobytes() == b.tobytes() == c.tobytes()
    dec.close()


@pytest.mark.parametrize("rows", [1, 8], ids=["verify-by-prompt-pass", "verify-by-decode-step"])
def test_speculative_generation_equals_the_target_generating_alone(rows):
    """Greedy speculative decoding with (a) a draft that is the target's twin and (b) a different, smaller
    draft: the tokens must be the target's own greedy tokens up to the first position where the target's
    two best logits are closer than the chained-step bar allows to tell apart (verification runs the
    prompt-shape kernels, plain generation the decode-shape ones)."""
    import fandhe_ai_amd as fa
    from fandhe_ai_amd.scheduler import SamplingStrategy, generate, generate_speculative
    geometry = dict(max_blocks_per_seq=8, num_blocks=8, max_batch=rows)
    target = _recording(_decoder(**geometry))
    twin = _decoder(**geometry)
    other_ckpt = st_save(_checkpoint(77, 1, D, HEADS, KV, F, VOCAB))
    other, store = fa.safetensors_io.load_decoder(ops(), other_ckpt, 1, HEADS, KV, **geometry)
    store.free()
    rng = np.random.default_rng(4)
    total = matched = 0
    for plen, max_length, k in ((5, 60, 4), (33, 80, 3), (1, 20, 7), (12, 14, 2)):
        prompt = rng.integers(0, VOCAB, plen).astype(np.int32)
        cfg = _cfg(max_length, SamplingStrategy.Greedy(), 0)
        target.trace = []
        want = generate(target, prompt, cfg)
        margins = []
        for _, _, logits, _ in list(target.trace):
            top2 = np.sort(logits)[-2:]
            margins.append(float(top2[1] - top2[0]) / float(logits.max() - logits.min()))
        assert len(margins) == max_length - plen
        for draft, name in ((twin, "twin"), (other, "other")):
            got, rounds, accepted = generate_speculative(target, draft, prompt, cfg, k)
            assert got.shape == want.shape and np.array_equal(got[:plen], prompt)
            new = max_length - plen
            agree = 0
            while agree < new and got[plen + agree] == want[plen + agree]:
                agree += 1
            if agree < new:
                assert margins[agree] < 4e-2, (name, plen, agree, margins[agree])     # only an indecisive pick may differ
            total += new
            matched += agree
            if name == "twin":
                assert accepted >= 0.5 * agree - k and rounds < new                   # most drafts are accepted
            print("SPECULATIVE\t%s\tprompt %d, %d new tokens, k %d: %d rounds, %d drafts accepted, %d tokens equal"
                  % (name, plen, new, k, rounds, accepted, agree), flush=True)
    assert matched >= 0.9 * total
    for d in (target, twin, other):
        d.close()


def _feeding(dec):
    """Wraps a decoder so that every prompt pass, step and verification pass leaves (kind, token ids fed, logits)."""
    import fandhe_ai_amd as fa

    class Feeding(fa.Decoder):
        def set_tokens(self, tokens):
            self.fed = [int(t) for t in tokens]
            super().set_tokens(tokens)

        def prefill(self, prompt):
            super().prefill(prompt)
            self.trace.append(("prefill", [int(t) for t in np.asarray(prompt)[0]], self.logits()[:1].copy()))

        def step(self, use_graph=True):
            super().step(use_graph)
            self.trace.append(("step", list(self.fed), self.logits()[:len(self.fed)].copy()))

        def verify(self, tokens, want_logits=False):
            picked, logits = super().verify(tokens, want_logits=True)
            self.trace.append(("step", [int(t) for t in np.asarray(tokens)[0]], logits[0].copy()))
            return (picked, logits) if want_logits else picked

    dec.__class__ = Feeding
    dec.trace, dec.fed = [], []
    return dec


class _Replay:
    """A model of the oracle's speculative loop that hands out the logits the device produced, call by call, and
    insists on being fed what the device was fed.  The oracle cuts a cache back by restoring a snapshot and
    replaying the accepted tokens (as the reference does); the device only shortens the sequence, so the one
    forward call after a ``truncate`` has no counterpart in the trace."""

    def __init__(self, trace):
        self.trace, self.len, self.replaying = list(trace), 0, False

    def forward_step(self, ids):
        ids = [int(t) for t in ids]
        self.len += len(ids)
        if self.replaying:
            self.replaying = False
            return np.zeros((len(ids), VOCAB), np.float32)
        kind, fed, logits = self.trace.pop(0)
        assert fed == ids, (kind, fed, ids)
        if kind == "prefill":
            out = np.zeros((len(ids), VOCAB), np.float32)
            out[-1] = logits[0]
            return out
        return logits

    def seq_len(self):
        return self.len

    def truncate(self, n):
        assert n <= self.len
        self.len, self.replaying = n, True


@pytest.mark.parametrize("rows", [1, 8], ids=["verify-by-prompt-pass", "verify-by-decode-step"])
def test_sampled_speculative_generation_takes_the_oracle_decisions(rows):
    """Temperature / top-k speculative decoding on the device (weights, acceptance, residual and bonus draws in
    fa_sampling_weights / fa_speculative_accept; rounds, rewinds and the draft's catch-up step in
    scheduler.generate_speculative) against the oracle's restatement of the reference loop run on the very
    logits the two decoders produced: the same tokens, the same sequence of forward calls with the same inputs."""
    import fandhe_ai_amd as fa
    from fandhe_ai_amd.scheduler import SamplingStrategy as S, generate_speculative
    geometry = dict(max_blocks_per_seq=8, num_blocks=8, max_batch=rows)
    target = _feeding(_decoder(**geometry))
    twin = _feeding(_decoder(**geometry))
    other_ckpt = st_save(_checkpoint(77, 1, D, HEADS, KV, F, VOCAB))
    other, store = fa.safetensors_io.load_decoder(ops(), other_ckpt, 1, HEADS, KV, **geometry)
    store.free()
    other = _feeding(other)
    rng = np.random.default_rng(9)
    drafted = {"twin": [0, 0], "other": [0, 0]}
    for plen, max_length, k, strategy, seed in ((5, 40, 4, S.Temperature(0.8), 11), (33, 60, 3, S.TopK(5), 7), (1, 20, 7, S.Temperature(1.4), 0),
                                                (12, 14, 2, S.TopK(40), 3), (3, 4, 5, S.Temperature(1.0), 5), (6, 30, 1, S.TopK(2), 2 ** 63 + 1)):
        prompt = rng.integers(0, VOCAB, plen).astype(np.int32)
        cfg = _cfg(max_length, strategy, seed)
        for draft, name in ((twin, "twin"), (other, "other")):
            target.trace, draft.trace = [], []
            got, rounds, accepted = generate_speculative(target, draft, prompt, cfg, k)
            assert got.shape == (max_length,) and np.array_equal(got[:plen], prompt)
            t_model, d_model = _Replay(target.trace), _Replay(draft.trace)
            want = osamp.generate_speculative(t_model, d_model, prompt, max_length, strategy.kind, cfg.temperature, cfg.top_k,
                                              seed, k)
            assert got.tolist() == want, (name, plen, max_length, k, strategy)
            assert not t_model.trace and not d_model.trace               # every device call was one the oracle makes
            drafted[name][0] += accepted
            drafted[name][1] += sum(len(fed) - 1 for kind, fed, _ in target.trace if kind == "step" and len(fed) > 1)
            again, r2, a2 = generate_speculative(target, draft, prompt, cfg, k)        # speculative.rs:1041-1062
            assert np.array_equal(again, got) and (r2, a2) == (rounds, accepted)
            print("SPECULATIVE_SAMPLED\t%s\t%s\tprompt %d, %d new tokens, k %d: %d rounds, %d drafts accepted"
                  % (name, strategy, plen, max_length - plen, k, rounds, accepted), flush=True)
    # a draft with the target's own weights is accepted almost always (its logits differ only by the rounding of
    # another batch shape); an unrelated one-layer draft is refused often
    assert drafted["twin"][0] >= 0.9 * drafted["twin"][1] and drafted["other"][0] < 0.9 * drafted["other"][1], drafted
    # speculative.rs:1097-1115: top-k 1 draws from one-hot weights and is the greedy sequence
    prompt = rng.integers(0, VOCAB, 7).astype(np.int32)
    greedy, _, _ = generate_speculative(target, other, prompt, _cfg(30, S.Greedy(), 0), 3)
    top1, _, _ = generate_speculative(target, other, prompt, _cfg(30, S.TopK(1), 9), 3)
    assert np.array_equal(greedy, top1)
    for d in (target, twin, other):
        d.close()


def test_padded_prompt_pass_leaves_every_row_as_its_own_prompt_pass_would():
    """Three prompts of different lengths in one padded pass against the same prompts ingested one by one:
    logits of every row's last prompt token within the chained-step bar (the rows of a GEMM and the ranges of
    the attention are cut differently), lengths exact, and decode steps continue from either state alike.
    One row has pages for its own prompt only, so part of its padding has no page to land on."""
    import fandhe_ai_amd as fa
    geometry = dict(max_blocks_per_seq=4, num_blocks=12, max_batch=4)
    dec = _decoder(**geometry)
    rng = np.random.default_rng(8)
    prompts = [rng.integers(0, VOCAB, n).astype(np.int32) for n in (5, 37, 16)]
    tables = np.full((3, 4), 0xFFFFFFFF, dtype=np.uint32)
    tables[0, :1] = [7]                                     # 5 tokens + a few steps fit one page; padding to 37 does not
    tables[1, :3] = [0, 1, 2]
    tables[2, :2] = [9, 4]
    alone_logits, alone_tokens = [], []
    for b in range(3):
        dec.set_sequences(tables[b:b + 1], np.zeros(1, np.uint32))
        dec.prefill(prompts[b][None, :])
        alone_logits.append(dec.logits()[0].copy())
        alone_tokens.append(int(dec.tokens()[0]))
    dec.set_sequences(tables, np.zeros(3, np.uint32))
    dec.prefill_padded(prompts)
    assert dec.seq_lens().tolist() == [5, 37, 16]
    got_logits, got_tokens = dec.logits(), dec.tokens()
    for b in range(3):
        spread = float(alone_logits[b].max() - alone_logits[b].min())
        err = np.abs(got_logits[b] - alone_logits[b]) / spread
        assert np.isfinite(got_logits[b]).all() and err.mean() < 2e-4 and err.max() < 2e-2, (b, err.mean(), err.max())
        top2 = np.sort(alone_logits[b])[-2:]
        if (top2[1] - top2[0]) / spread > 4e-2:
            assert got_tokens[b] == alone_tokens[b]
    # both states decode on: same logits within the bar for three more steps
    after_padded = []
    toks = got_tokens.copy()
    for _ in range(3):
        dec.step()
        after_padded.append(dec.logits().copy())
    fed = [toks] + [o.argmax(axis=1).astype(np.int32) for o in after_padded[:-1]]
    for b in range(3):                                      # replay row b alone, feeding what the padded run fed
        dec.set_sequences(tables[b:b + 1], np.zeros(1, np.uint32))
        dec.prefill(prompts[b][None, :])
        for s_i in range(3):
            dec.set_tokens(fed[s_i][b:b + 1])
            dec.step()
            ref = dec.logits()[0]
            spread = float(ref.max() - ref.min())
            err = np.abs(after_padded[s_i][b] - ref) / spread
            assert err.mean() < 2e-4 and err.max() < 2e-2, (b, s_i, err.mean(), err.max())
    # argument checks
    dec.set_sequences(tables, np.zeros(3, np.uint32))
    with pytest.raises(fa.InvalidArgument):
        dec.prefill_padded([prompts[0], prompts[1], np.zeros(70, np.int32)])          # beyond the row's block table
    with pytest.raises(fa.InvalidArgument):
        dec.prefill_padded([np.zeros(20, np.int32), prompts[1], prompts[2]])          # row 0 has one page
    lens = np.array([5, 0, 3], np.uint32)
    pad = np.zeros((3, 5), np.int32)
    assert fa.capi.lib.fa_decoder_prefill_padded(ops()._ctx, dec._h, pad.ctypes.data_as(fa.capi.i32p), 5,
                                                 lens.ctypes.data_as(fa.capi.u32p)) == fa.capi.INVALID_ARGUMENT
    dec.close()
