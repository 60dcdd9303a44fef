"""The C++ host layer on the device (tests/cpp/host_gpu_test.cpp) against the Python mirror: both build the same
decoder from device-generated weights (same seeds, same order) through the same C ABI and must produce the same
tokens from generate and from the continuous-batching scheduler."""
import ctypes as C
import json
import subprocess

import numpy as np
import pytest

from test_cpp_host_cpu import host_binary

pytestmark = pytest.mark.gpu


def _python_side():
    import fandhe_ai_amd as fa
    from fandhe_ai_amd import scheduler as sch
    be = fa.tape_for(fa.Device.Rocm(0))
    lib = fa.capi.lib
    n_layers, d, heads, kv, dh, f, vocab = 2, 256, 4, 2, 128, 512, 1000
    seed = [100]
    keep = []

    def filled(numel, mean, std):
        b = be.alloc_uninit((numel,), fa.capi.F32)
        fa.check(lib.fa_fill_normal(be._ctx, b._h, 0, numel, seed[0], mean, std))
        seed[0] += 1
        keep.append(b)
        return b

    def weight(k, n):
        w = filled(k * n, 0.0, 0.05)
        q = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)))
        keep.append(q)
        return q

    def decoder():
        return fa.Decoder(be, n_layers, d, heads, kv, f, vocab, max_blocks_per_seq=8, num_blocks=48, max_batch=8,
                          rms_eps=1e-5, rope_theta=10000.0)

    dec, draft = decoder(), decoder()                       # weights are borrowed: the two share them
    eq, ekv = heads * dh, kv * dh
    for l in range(n_layers):
        an, fn = filled(d, 1.0, 0.1), filled(d, 1.0, 0.1)
        ws = (weight(d, eq + 2 * ekv), weight(eq, d), weight(d, 2 * f), weight(f, d))
        dec.set_layer(l, an, fn, *ws)
        draft.set_layer(l, an, fn, *ws)
    embed, norm = filled(vocab * d, 0.0, 1.0), filled(d, 1.0, 0.1)
    head = weight(d, vocab)
    dec.set_head(embed, norm, head)
    draft.set_head(embed, norm, head)

    G, K, T = sch.SamplingStrategy.Greedy, sch.SamplingStrategy.TopK, sch.SamplingStrategy.Temperature
    out = {}
    prompts = np.array([[5, 17, 900, 3, 44], [1, 2, 3, 4, 5]], np.int32)
    out["generate_greedy"] = sch.generate(dec, prompts, sch.GenerateConfig(12, G())).tolist()
    out["generate_top_k"] = sch.generate(dec, np.array([[8, 9, 10]], np.int32), sch.GenerateConfig(14, K(5), seed=7)).tolist()
    out["generate_temperature"] = sch.generate(dec, prompts, sch.GenerateConfig(10, T(np.float32(0.8)), seed=3)).tolist()
    requests = [([5, 17, 900, 3, 44], sch.GenerateConfig(12, G())),
                ([11, 12], sch.GenerateConfig(20, K(5), seed=7)),
                ([21, 22, 23, 24, 25, 26, 27], sch.GenerateConfig(16, T(np.float32(0.8)), seed=3)),
                ([31], sch.GenerateConfig(9, G())),
                ([41, 42, 43], sch.GenerateConfig(3, G())),
                ([51, 52, 53, 54], sch.GenerateConfig(25, T(np.float32(1.3)), seed=11)),
                ([61, 62], sch.GenerateConfig(30, K(50), seed=13))]
    s = sch.BatchScheduler(dec, sch.SchedulerLimits(3, 16, 40))
    for p, c in requests:
        s.submit(np.array(p, np.int32), c)
    done = {}
    for _ in range(200):
        if not (s.queued_len() or s.active_len()):
            break
        s.step()
        for rid, toks in s.take_finished():
            done[rid] = toks.tolist()
    assert not s.take_failed() and len(done) == len(requests) and s.free_pages() == 48
    out["scheduler"] = [done[i] for i in sorted(done)]
    out["scheduler_prompt_passes"] = s.stats["prompt_passes"]
    out["scheduler_decode_steps"] = s.stats["decode_steps"]
    for k in (4, 9):
        toks, rounds, accepted = sch.generate_speculative(dec, draft, prompts[0], sch.GenerateConfig(24, G()), k)
        out["speculative_k%d" % k] = {"tokens": toks.tolist(), "rounds": rounds, "accepted": accepted}
    for name, c in (("speculative_temperature", sch.GenerateConfig(28, sch.SamplingStrategy.Temperature(0.8)).with_seed(11)),
                    ("speculative_top_k", sch.GenerateConfig(28, sch.SamplingStrategy.TopK(5)).with_seed(7))):
        for k in (3, 9):
            toks, rounds, accepted = sch.generate_speculative(dec, draft, prompts[1], c, k)
            out["%s_k%d" % (name, k)] = {"tokens": toks.tolist(), "rounds": rounds, "accepted": accepted}
    draft.close()
    dec.close()
    be.close()
    return out


def test_cpp_host_layer_matches_the_python_mirror_on_the_device():
    r = subprocess.run([host_binary("host_gpu_test")], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    cpp = json.loads(r.stdout)
    assert cpp["gemm_device_bit_exact"] and cpp["scheduler_clean"] and cpp["bad_table_rejected"]
    # a request that runs alone through the scheduler is generate of the same request
    assert cpp["scheduler_alone"] == cpp["generate_same_request"]
    assert cpp["scheduler"][4] == [41, 42, 43]                       # nothing to generate: the prompt is the answer
    for row, n in zip(cpp["scheduler"], (12, 20, 16, 9, 3, 25, 30)):
        assert len(row) == n and all(0 <= t < 1000 for t in row)
    # the draft is the target itself: all drafts are accepted and the tokens are plain greedy generation
    for k in (4, 9):
        sp = cpp["speculative_k%d" % k]
        assert sp["tokens"] == cpp["generate_greedy_24"][0] and sp["accepted"] > 0 and sp["rounds"] < 24 - 5
    # the one-layer cache against a double-precision host loop
    assert cpp["paged_cache_max_abs_err"] < 1e-5 and cpp["paged_cache_state_ok"]
    py = _python_side()
    for key in ("generate_greedy", "generate_top_k", "generate_temperature", "scheduler", "scheduler_prompt_passes",
                "scheduler_decode_steps", "speculative_k4", "speculative_k9", "speculative_temperature_k3",
                "speculative_temperature_k9", "speculative_top_k_k3", "speculative_top_k_k9"):
        assert cpp[key] == py[key], key


def test_cpp_checkpoint_loader_builds_the_decoder_the_python_loader_builds(tmp_path):
    """The same Llama-style safetensors file through the C++ loader (typed read, explicit transposes, flat resident
    store, device quantizer) and through the Python one: the two resident decoders generate the same tokens."""
    import fandhe_ai_amd as fa
    from decoder_common import llama_checkpoint
    from fandhe_ai_amd import safetensors_io as sio
    from fandhe_ai_amd import scheduler as sch
    n_layers, heads, kv = 2, 2, 1
    path = tmp_path / "tiny.safetensors"
    sio.save_safetensors_f32(str(path), llama_checkpoint(11, n_layers, 128, heads, kv, 256, 300))
    r = subprocess.run([host_binary("host_gpu_test"), str(path), str(n_layers), str(heads), str(kv)],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    cpp = json.loads(r.stdout)
    be = fa.tape_for(fa.Device.Rocm(0))
    dec, store = sio.load_decoder(be, str(path), n_layers, heads, kv, max_blocks_per_seq=4, num_blocks=16, max_batch=4,
                                  rms_eps=1e-5, rope_theta=10000.0)
    store.free()
    prompts = np.array([[3, 1, 4, 1, 5], [2, 7, 1, 8, 2]], np.int32)
    greedy = sch.generate(dec, prompts, sch.GenerateConfig(20, sch.SamplingStrategy.Greedy())).tolist()
    top_k = sch.generate(dec, prompts[:1], sch.GenerateConfig(20, sch.SamplingStrategy.TopK(8), seed=21)).tolist()
    dec.close()
    be.close()
    assert cpp["checkpoint_greedy"] == greedy and cpp["checkpoint_top_k"] == top_k
    assert len(set(greedy[0][5:])) > 3                     # not a degenerate model
