#!/usr/bin/env python3
"""Benchmark of the quantized decode path on one MI355X.

A step is one decode step of the benchmark's full-step configuration: a
random-init 32-layer Llama-style decoder (d_model 4096, 32 heads / 8 KV heads,
head_dim 128, SwiGLU 14336, RMSNorm eps 1e-5, RoPE theta 500000, vocab 32000),
W8A8 int8 linears, batch 32, paged bf16 KV (page 16) with contexts uniform in
[1024, 8192], greedy argmax.  All inputs are resident in HBM before the timed
region; the step runs as one captured HIP graph.

Prints ONE JSON line.  `value` is tokens/s of the whole step; `roofline`
covers the dominant operator (paged decode attention); `extras` holds the
other headline kernels (decode-shape int8-weight linears, the 64-sequence
attention configuration, prefill int8 / fp8 GEMM); `cpu_baseline` is the CPU
oracle timed on this host's cores on a bounded sample.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "int8/fp8 GEMM TOPS + decode tok/s (bs32, paged-KV) and % roofline, 1 GPU"
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TOPS = 5000.0          # dense int8 and fp8 on MI355X
# HBM bytes per launch of decode_stream_kernel at this benchmark's shape, from hardware counters
# (rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE, each scaled by the same counter's reading for a plain
# row-copy kernel of known size; the figures are in profiles/decode_stream_kernel_config5_pmc.txt).
ATTENTION_TRAFFIC_BYTES = 635875453
U32MAX = 0xFFFFFFFF
SERVING_ROWS = 64          # rows of the continuous-batching run (the decoder's limit)

MODEL = dict(n_layers=32, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ffn=14336, vocab=32000,
             block_size=16, rms_eps=1e-5, rope_theta=500000.0)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Timer:
    """HIP events recorded on the stream the kernels run on."""

    def __init__(self, fa, be):
        self.fa, self.be, self.h = fa, be, C.c_void_p()
        fa.check(fa.capi.lib.fa_timer_create(be._ctx, C.byref(self.h)))

    def start(self):
        self.fa.check(self.fa.capi.lib.fa_timer_start(self.be._ctx, self.h))

    def stop_ms(self):
        ms = C.c_float()
        self.fa.check(self.fa.capi.lib.fa_timer_stop(self.be._ctx, self.h))
        self.fa.check(self.fa.capi.lib.fa_timer_elapsed_ms(self.be._ctx, self.h, C.byref(ms)))
        return float(ms.value)


def time_launches(fa, be, fn, iters, warmup=5):
    """Seconds per launch of fn, from HIP events on the library's stream.  The launches are recorded
    into one HIP graph and the graph is replayed, so that the host's per-call cost (several microseconds
    through ctypes) does not show in kernels that take only a few microseconds."""
    lib = fa.capi.lib
    for _ in range(warmup):
        fn()
    be.synchronize_device()
    graph = C.c_void_p()
    fa.check(lib.fa_graph_capture_begin(be._ctx))
    try:
        for _ in range(iters):
            fn()
    finally:
        st = lib.fa_graph_capture_end(be._ctx, C.byref(graph))
    fa.check(st)
    try:
        fa.check(lib.fa_graph_launch(be._ctx, graph))
        be.synchronize_device()
        reps = 3
        t = Timer(fa, be)
        t.start()
        for _ in range(reps):
            fa.check(lib.fa_graph_launch(be._ctx, graph))
        return t.stop_ms() / (iters * reps) * 1e-3
    finally:
        lib.fa_graph_destroy(be._ctx, graph)


def make_tables(rng, ctxs, extra_tokens, bs, num_blocks=None):
    need = [(c + extra_tokens + bs - 1) // bs for c in ctxs]
    max_blocks = max(need) + 1
    total = sum(need)
    num_blocks = num_blocks or total + 8
    perm = rng.permutation(num_blocks).astype(np.uint32)
    tables = np.full((len(ctxs), max_blocks), U32MAX, dtype=np.uint32)
    p = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[p:p + n]
        p += n
    return tables, max_blocks, num_blocks


# ------------------------------------------------------------------ full step
def build_decoder(fa, be, cfg, batch, ctxs, steps_total, seed=0, max_batch=None):
    lib = fa.capi.lib
    rng = np.random.default_rng(seed)
    tables, max_blocks, num_blocks = make_tables(rng, ctxs, steps_total + 1, cfg["block_size"])
    dcfg = fa.capi.DecoderConfig(cfg["n_layers"], cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"],
                                 cfg["d_ffn"], cfg["vocab"], cfg["block_size"], max_blocks, num_blocks, max_batch or batch,
                                 cfg["rms_eps"], cfg["rope_theta"])
    dec = C.c_void_p()
    fa.check(lib.fa_decoder_create(be._ctx, C.byref(dcfg), C.byref(dec)))
    keep = []
    D, F, V = cfg["d_model"], cfg["d_ffn"], cfg["vocab"]
    EQ, EKV = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    scratch = be.alloc_uninit((max(D * 2 * F, D * V),))                    # f32 staging for one weight

    def qweight(k, n, s):
        fa.check(lib.fa_fill_normal(be._ctx, scratch._h, 0, k * n, s, 0.0, 0.02))
        q = be.quantize_weight(fa.DeviceBufferView(scratch, 0, (k, n)))
        keep.append(q)
        return q

    def norm(s):
        b = be.alloc_uninit((D,))
        fa.check(lib.fa_fill_normal(be._ctx, b._h, 0, D, s, 1.0, 0.1))
        keep.append(b)
        return b

    for li in range(cfg["n_layers"]):
        s = 1000 * (li + 1)
        fa.check(lib.fa_decoder_set_layer(dec, li, norm(s + 1)._h, norm(s + 2)._h, qweight(D, EQ + 2 * EKV, s + 3)._h,
                                          qweight(EQ, D, s + 4)._h, qweight(D, 2 * F, s + 5)._h,
                                          qweight(F, D, s + 6)._h))
        kp, vp = fa.capi.buf_p(), fa.capi.buf_p()
        fa.check(lib.fa_decoder_kv_pools(dec, li, C.byref(kp), C.byref(vp)))
        n = num_blocks * cfg["block_size"] * EKV
        fa.check(lib.fa_fill_normal(be._ctx, kp, 0, n, s + 7, 0.0, 1.0))
        fa.check(lib.fa_fill_normal(be._ctx, vp, 0, n, s + 8, 0.0, 1.0))
    embed = be.alloc_uninit((V, D))
    fa.check(lib.fa_fill_normal(be._ctx, embed._h, 0, V * D, 7, 0.0, 1.0))
    keep.append(embed)
    fa.check(lib.fa_decoder_set_head(dec, embed._h, norm(8)._h, qweight(D, V, 9)._h))
    scratch.free()
    lens = np.asarray(ctxs, dtype=np.uint32)
    fa.check(lib.fa_decoder_set_sequences(be._ctx, dec, batch, tables.ctypes.data_as(fa.capi.u32p),
                                          lens.ctypes.data_as(fa.capi.u32p)))
    tokens = rng.integers(0, V, size=batch).astype(np.int32)
    fa.check(lib.fa_decoder_set_tokens(be._ctx, dec, tokens.ctypes.data_as(fa.capi.i32p)))
    be.synchronize_device()
    return dec, keep, tables, max_blocks, num_blocks


def step_bytes(cfg, batch, sum_ctx):
    D, F, V = cfg["d_model"], cfg["d_ffn"], cfg["vocab"]
    EQ, EKV = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    w_layer = D * (EQ + 2 * EKV) + EQ * D + D * 2 * F + F * D
    weights = cfg["n_layers"] * w_layer + D * V
    kv = cfg["n_layers"] * sum_ctx * 2 * EKV * 2
    return weights + kv


def attention_bytes(sum_ctx, ctxs, heads, kv_heads, head_dim=128, bs=16):
    batch = len(ctxs)
    return (sum_ctx * 2 * kv_heads * head_dim * 2 + 2 * batch * heads * head_dim * 2 +
            sum((c + bs - 1) // bs for c in ctxs) * 4 + batch * 4)


# ------------------------------------------------------------------ operators
def bench_attention(fa, be, batch, heads, kv_heads, ctxs, num_blocks, iters, seed, kernel_only=False):
    lib = fa.capi.lib
    rng = np.random.default_rng(seed)
    tables, max_blocks, num_blocks = make_tables(rng, ctxs, 0, 16, num_blocks)
    e_kv, e_q = kv_heads * 128, heads * 128
    kp = be.alloc_uninit((num_blocks, 16, e_kv), fa.capi.BF16)
    vp = be.alloc_uninit((num_blocks, 16, e_kv), fa.capi.BF16)
    q = be.alloc_uninit((batch, 1, e_q), fa.capi.BF16)
    for b, s in ((kp, 1), (vp, 2), (q, 3)):
        fa.check(lib.fa_fill_normal(be._ctx, b._h, 0, b.numel(), seed * 10 + s, 0.0, 1.0))
    d_tables, d_lens = be.upload(tables), be.upload(np.asarray(ctxs, dtype=np.uint32))
    out = be.alloc_uninit((batch, 1, e_q), fa.capi.BF16)
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    args = fa.PagedAttentionArgs(layout, batch, 1, heads, max_blocks, fa.default_scale(128), kv_heads).c()

    def launch():
        fa.check(lib.fa_paged_attention_forward_device(be._ctx, q._h, kp._h, vp._h, d_tables._h, d_lens._h,
                                                       C.byref(args), out._h))
    sec = time_launches(fa, be, launch, iters)
    nbytes = attention_bytes(int(np.sum(ctxs)), ctxs, heads, kv_heads)
    sec_kernel = None
    if kernel_only:
        # the streaming kernel by itself (its merge kernel is not launched, the output stays unwritten)
        fa.check(lib.fa_set_tuning(3, 1))
        try:
            sec_kernel = time_launches(fa, be, launch, iters)
        finally:
            fa.check(lib.fa_set_tuning(3, 0))
    for b in (kp, vp, q, d_tables, d_lens, out):
        b.free()
    return (sec, nbytes, sec_kernel) if kernel_only else (sec, nbytes)


def bench_copy(fa, be, iters):
    """Plain row copy (identity gather) of 256 MiB: reads 256 MiB + 256 KiB of indices, writes 256 MiB."""
    lib = fa.capi.lib
    rows, cols = 65536, 1024
    src = be.alloc_uninit((rows, cols))
    fa.check(lib.fa_fill_normal(be._ctx, src._h, 0, rows * cols, 9, 0.0, 1.0))
    idx = be.upload(np.arange(rows, dtype=np.int32))
    dst = be.alloc_uninit((rows, cols))
    sec = time_launches(fa, be, lambda: fa.check(lib.fa_gather_rows(be._ctx, src._h, rows, cols, idx._h, rows, dst._h)),
                        iters)
    for b in (src, idx, dst):
        b.free()
    return sec, 2 * rows * cols * 4 + rows * 4


def bench_w8a8_decode(fa, be, cfg, m, iters):
    """W8A8 linears of one decoder layer at the step's batch (dynamic per-token quantizer + int8 GEMV)."""
    lib = fa.capi.lib
    D, F = cfg["d_model"], cfg["d_ffn"]
    EQ, EKV = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    res = []
    for k, n in ((D, EQ + 2 * EKV), (EQ, D), (D, 2 * F), (F, D)):
        w = be.alloc_uninit((k, n))
        fa.check(lib.fa_fill_normal(be._ctx, w._h, 0, k * n, k + n, 0.0, 0.02))
        qw = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)))
        w.free()
        x = be.alloc_uninit((m, k))
        fa.check(lib.fa_fill_normal(be._ctx, x._h, 0, m * k, 5, 0.0, 1.0))
        out = be.alloc_uninit((m, n))
        sec = time_launches(fa, be, lambda: fa.check(lib.fa_linear_w8a8(be._ctx, x._h, m, qw._h, None, 0, None, out._h)),
                            iters)
        nbytes = k * n + 4 * n + m * k + 4 * m * n
        res.append(dict(op="w8a8", m=m, k=k, n=n, us=sec * 1e6, gbs=nbytes / sec / 1e9))
        for b in (x, out, qw):
            b.free()
    return res


LINEAR_SHAPES = ((4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096))


def bench_linears(fa, be, iters, ms=(1, 8, 32), shapes=LINEAR_SHAPES):
    """Decode-shape int8-weight linears with bf16 activations (W8A16), Llama-7B layer shapes.  Consecutive
    launches walk over copies of the weight that together exceed the caches (32 MB of L2, 256 MB memory-side),
    as the layers of a model do: a launch that found its own weight of the previous launch still cached
    would be timed on traffic that a decode step never sees."""
    lib = fa.capi.lib
    res = []
    for k, n in shapes:
        w = be.alloc_uninit((k, n))
        fa.check(lib.fa_fill_normal(be._ctx, w._h, 0, k * n, k + n, 0.0, 0.02))
        copies = max(2, -(-(640 << 20) // (k * n)))
        qws = [be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n))) for _ in range(copies)]
        w.free()
        for m in ms:
            a = be.alloc_uninit((m, k), fa.capi.BF16)
            fa.check(lib.fa_fill_normal(be._ctx, a._h, 0, m * k, 5, 0.0, 1.0))
            out = be.alloc_uninit((m, n), fa.capi.BF16)
            counter = [0]

            def launch():
                qw = qws[counter[0] % copies]
                counter[0] += 1
                fa.check(lib.fa_linear_w8a16(be._ctx, a._h, m, qw._h, out._h))
            sec = time_launches(fa, be, launch, iters)
            nbytes = k * n + 4 * n + 2 * m * k + 2 * m * n
            res.append(dict(op="w8a16", m=m, k=k, n=n, us=sec * 1e6, gbs=nbytes / sec / 1e9,
                            frac=nbytes / sec / 1e9 / HBM_PEAK_GBS, weight_copies=copies))
            a.free()
            out.free()
        for qw in qws:
            qw.free()
    return res


def bench_prefill(fa, be, iters):
    lib = fa.capi.lib
    m, k, n = 2048, 4096, 14336
    ops_count = 2.0 * m * k * n
    res = []
    w = be.alloc_uninit((k, n))
    x = be.alloc_uninit((m, k))
    fa.check(lib.fa_fill_normal(be._ctx, w._h, 0, k * n, 11, 0.0, 1.0))
    fa.check(lib.fa_fill_normal(be._ctx, x._h, 0, m * k, 12, 0.0, 1.0))
    out = be.alloc_uninit((m, n), fa.capi.BF16)
    # int8 W8A8
    qw = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)))
    xq, sx = be.quantize_rows_i8(x)
    sec = time_launches(fa, be, lambda: fa.check(lib.fa_gemm_w8a8(be._ctx, xq._h, sx._h, m, qw._h, None, out._h)), iters)
    res.append(dict(op="gemm_w8a8", m=m, k=k, n=n, us=sec * 1e6, tops=ops_count / sec / 1e12,
                    frac=ops_count / sec / 1e12 / MFMA_PEAK_TOPS))
    qw.free(), xq.free(), sx.free()
    # fp8 e4m3
    qw = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)), fa.capi.QW_E4M3_TENSOR)
    xq, xs = be.quantize_tensor_e4m3(x)
    sec = time_launches(fa, be, lambda: fa.check(lib.fa_gemm_e4m3(be._ctx, xq._h, xs._h, m, qw._h, out._h)), iters)
    res.append(dict(op="gemm_e4m3", m=m, k=k, n=n, us=sec * 1e6, tops=ops_count / sec / 1e12,
                    frac=ops_count / sec / 1e12 / MFMA_PEAK_TOPS))
    for b in (qw, xq, xs, w, x, out):
        b.free()
    return res


F32_PEAK_TFLOPS = 157.3         # dense f32 matrix rate of MI355X


def bench_gemm_f32(fa, be, iters):
    """The order-fixed f32 GEMM (gemm_device / linear_forward_device: one fused multiply-add per k, k ascending)
    at a prompt shape and at a decode shape."""
    lib = fa.capi.lib
    res = []
    for m, k, n in ((2048, 4096, 4096), (32, 4096, 4096)):
        a, b, out = be.alloc_uninit((m, k)), be.alloc_uninit((k, n)), be.alloc_uninit((m, n))
        fa.check(lib.fa_fill_normal(be._ctx, a._h, 0, m * k, 21, 0.0, 1.0))
        fa.check(lib.fa_fill_normal(be._ctx, b._h, 0, k * n, 22, 0.0, 0.02))
        sec = time_launches(fa, be, lambda: fa.check(lib.fa_gemm_device(be._ctx, a._h, b._h, m, n, k, out._h)), iters)
        flops = 2.0 * m * k * n
        res.append(dict(op="gemm_device_f32", m=m, k=k, n=n, us=sec * 1e6, tflops=flops / sec / 1e12,
                        frac=flops / sec / 1e12 / F32_PEAK_TFLOPS))
        for x in (a, b, out):
            x.free()
    return res


def bench_prefill_attention(fa, be, batch=4, l_new=2048, heads=32, kv_heads=8):
    """Causal attention of `l_new` new tokens per row over their own pages (empty cache before them), bf16,
    page 16: the block form (what this shape selects), the streamed form and the generic kernel (reference
    summation order) beside it."""
    lib = fa.capi.lib
    rng = np.random.default_rng(5)
    tables, max_blocks, num_blocks = make_tables(rng, [l_new] * batch, 0, 16)
    e_kv, e_q = kv_heads * 128, heads * 128
    layout = fa.PagedKvLayout.new(num_blocks, 16, e_kv)
    pools = [be.alloc_uninit((num_blocks, 16, e_kv), fa.capi.BF16) for _ in range(2)]
    q = be.alloc_uninit((batch, l_new, e_q), fa.capi.BF16)
    for i, b in enumerate(pools + [q]):
        fa.check(lib.fa_fill_normal(be._ctx, b._h, 0, b.numel(), 21 + i, 0.0, 1.0))
    out = be.alloc_uninit((batch, l_new, e_q), fa.capi.BF16)
    args = fa.PagedAttentionArgs(layout, batch, l_new, heads, max_blocks, fa.default_scale(128), kv_heads)
    d_tables, d_lens = be.upload(tables), be.upload(np.full(batch, l_new, np.uint32))
    flops = 4.0 * batch * heads * 128 * l_new * (l_new + 1) / 2          # QK^T and PV over the causal triangle
    res = []
    for name, form, generic, reps in (("block", 0, 0, 5), ("streamed", 1, 0, 5), ("generic", 0, 1, 1)):
        fa.check(lib.fa_set_tuning(10, form))
        fa.check(lib.fa_set_tuning(8, generic))
        fn = lambda: fa.check(lib.fa_paged_attention_forward_device(be._ctx, q._h, pools[0]._h, pools[1]._h, d_tables._h,
                                                                    d_lens._h, C.byref(args.c()), out._h))
        fn()
        be.synchronize_device()
        t = Timer(fa, be)
        t.start()
        for _ in range(reps):
            fn()
        ms = t.stop_ms() / reps
        res.append(dict(kernel=name, ms=ms, tflops=flops / (ms * 1e-3) / 1e12))
    fa.check(lib.fa_set_tuning(8, 0))
    fa.check(lib.fa_set_tuning(10, 0))
    for b in pools + [q, out, d_tables, d_lens]:
        b.free()
    return res


def bench_prompt_prefill(fa, be, dec, cfg, tables, batch=4, l_new=2048, reps=2):
    """Prompt ingestion through the whole decoder: `batch` empty sequences, `l_new` prompt tokens each, on the
    resident model (the sequences borrow the first pages of the installed tables)."""
    lib = fa.capi.lib
    need = (l_new + 1 + cfg["block_size"] - 1) // cfg["block_size"]
    assert need <= tables.shape[1] and batch <= tables.shape[0]
    tb = np.ascontiguousarray(tables[:batch])
    lens = np.zeros(batch, dtype=np.uint32)
    prompt = np.random.default_rng(3).integers(0, cfg["vocab"], size=(batch, l_new)).astype(np.int32)

    def run():
        fa.check(lib.fa_decoder_set_sequences(be._ctx, dec, batch, tb.ctypes.data_as(fa.capi.u32p),
                                              lens.ctypes.data_as(fa.capi.u32p)))
        t = Timer(fa, be)
        t.start()
        fa.check(lib.fa_decoder_prefill(be._ctx, dec, prompt.ctypes.data_as(fa.capi.i32p), l_new))
        return t.stop_ms()

    run()
    ms = min(run() for _ in range(reps))
    toks = np.empty(batch, dtype=np.int32)
    fa.check(lib.fa_decoder_read_tokens(be._ctx, dec, toks.ctypes.data_as(fa.capi.i32p)))
    assert np.all((toks >= 0) & (toks < cfg["vocab"]))
    return dict(batch=batch, l_new=l_new, ms=ms, tokens_per_s=batch * l_new / (ms * 1e-3))


def bench_short_prompts(fa, be, dec, cfg, tables, lengths=(64, 300, 1024, (64, 4096)), reps=3):
    """One request's prompt pass (batch 1) on the resident model: what a scheduler runs when a request joins
    (an empty cache) or a conversation continues (new tokens after cached positions)."""
    lib = fa.capi.lib
    row = int(np.argmax((tables != 0xFFFFFFFF).sum(axis=1)))           # the row with the most pages
    tb = np.ascontiguousarray(tables[row:row + 1])
    out = []
    for item in lengths:                                               # l_new, or (l_new, positions cached before)
        l_new, cached = item if isinstance(item, tuple) else (item, 0)
        lens = np.full(1, cached, dtype=np.uint32)                     # the synthetic pools already hold K / V there
        assert (cached + l_new + 1 + cfg["block_size"] - 1) // cfg["block_size"] <= int((tb != 0xFFFFFFFF).sum())
        prompt = np.random.default_rng(l_new).integers(0, cfg["vocab"], size=(1, l_new)).astype(np.int32)
        best = None
        for _ in range(reps + 1):
            fa.check(lib.fa_decoder_set_sequences(be._ctx, dec, 1, tb.ctypes.data_as(fa.capi.u32p),
                                                  lens.ctypes.data_as(fa.capi.u32p)))
            t = Timer(fa, be)
            t.start()
            fa.check(lib.fa_decoder_prefill(be._ctx, dec, prompt.ctypes.data_as(fa.capi.i32p), l_new))
            ms = t.stop_ms()
            best = ms if best is None else min(best, ms)
        out.append(dict(l_new=l_new, cached=cached, ms=best, tokens_per_s=l_new / (best * 1e-3)))
    return out


def bench_single_stream(fa, be, dec, cfg, tables, prompt_len=128, steps=64):
    """One sequence decoding by itself (graph-replayed steps after a short prompt): the latency floor a
    speculative or interactive caller sees; dominated by streaming the weights once per token."""
    lib = fa.capi.lib
    row = int(np.argmax((tables != U32MAX).sum(axis=1)))
    tb = np.ascontiguousarray(tables[row:row + 1])
    lens = np.zeros(1, dtype=np.uint32)
    prompt = np.random.default_rng(5).integers(0, cfg["vocab"], size=(1, prompt_len)).astype(np.int32)
    fa.check(lib.fa_decoder_set_sequences(be._ctx, dec, 1, tb.ctypes.data_as(fa.capi.u32p), lens.ctypes.data_as(fa.capi.u32p)))
    fa.check(lib.fa_decoder_prefill(be._ctx, dec, prompt.ctypes.data_as(fa.capi.i32p), prompt_len))
    for _ in range(3):
        fa.check(lib.fa_decoder_step(be._ctx, dec, 1))
    t = Timer(fa, be)
    t.start()
    for _ in range(steps):
        fa.check(lib.fa_decoder_step(be._ctx, dec, 1))
    ms = t.stop_ms() / steps
    # speculative verification of a pending token and four drafts: one step whose five rows are five
    # consecutive positions of the one sequence (same block table, lengths ctx .. ctx + 4)
    ctx0 = prompt_len + 3 + steps
    rows = 5
    tb5 = np.ascontiguousarray(np.repeat(tb, rows, axis=0))
    lens5 = np.arange(ctx0, ctx0 + rows, dtype=np.uint32)
    toks5 = np.random.default_rng(6).integers(0, cfg["vocab"], size=rows).astype(np.int32)
    verify_ms = None
    for rep in range(3):
        fa.check(lib.fa_decoder_set_sequences(be._ctx, dec, rows, tb5.ctypes.data_as(fa.capi.u32p),
                                              lens5.ctypes.data_as(fa.capi.u32p)))
        fa.check(lib.fa_decoder_set_tokens(be._ctx, dec, toks5.ctypes.data_as(fa.capi.i32p)))
        t.start()
        fa.check(lib.fa_decoder_step(be._ctx, dec, 1))
        one = t.stop_ms()
        verify_ms = one if rep == 1 else (min(verify_ms, one) if rep > 1 else None)
    weights = cfg["n_layers"] * (cfg["d_model"] * (cfg["n_heads"] + 2 * cfg["n_kv_heads"]) * cfg["head_dim"] +
                                 cfg["n_heads"] * cfg["head_dim"] * cfg["d_model"] + 3 * cfg["d_model"] * cfg["d_ffn"]) + \
        cfg["d_model"] * cfg["vocab"]
    return dict(batch=1, context=prompt_len, ms_per_token=ms, tokens_per_s=1e3 / ms, weight_bytes=weights,
                weight_stream_gbs=weights / (ms * 1e-3) / 1e9, verify_5_positions_ms=verify_ms)


def bench_continuous_batching(fa, be, dec, dcfg, requests=96, max_active=32):
    """Continuous batching on the resident model: requests with prompts of 64..512 tokens that each generate
    64..192 tokens (greedy, temperature and top-k mixed) join and leave a batch of at most `max_active` rows;
    wall time from the first submit to the last finished request, prompts included."""
    from fandhe_ai_amd.scheduler import BatchScheduler, GenerateConfig, SamplingStrategy, SchedulerLimits
    rng = np.random.default_rng(12)
    d = fa.Decoder.from_handle(be, dec, dcfg)
    s = BatchScheduler(d, SchedulerLimits(max_active, requests, 1024))
    prompt_tokens = new_tokens = 0
    for i in range(requests):
        plen, gen = int(rng.integers(64, 513)), int(rng.integers(64, 193))
        strategy = (SamplingStrategy.Greedy(), SamplingStrategy.Temperature(0.8), SamplingStrategy.TopK(50))[i % 3]
        s.submit(rng.integers(0, dcfg.vocab, plen).astype(np.int32), GenerateConfig.new(plen + gen, strategy).with_seed(i + 1))
        prompt_tokens += plen
        new_tokens += gen
    be.synchronize_device()
    t0 = time.perf_counter()
    steps = rows = done = 0
    while s.active_len() or s.queued_len():
        done += s.step()
        rows += s.active_len()
        steps += 1
        assert steps < 100000
    be.synchronize_device()
    sec = time.perf_counter() - t0
    assert done == requests and not s.take_failed() and len(s.take_finished()) == requests
    return dict(requests=requests, max_active=max_active, prompt_tokens=prompt_tokens, generated_tokens=new_tokens,
                seconds=sec, generated_tokens_per_s=new_tokens / sec, iterations=steps, mean_active_rows=rows / steps,
                **s.stats)


def bench_sampling(fa, be, rows=32, vocab=32000, iters=50):
    """Device sampler at the decode step's logits shape, beside the greedy argmax it replaces."""
    lib = fa.capi.lib
    logits = be.alloc_uninit((rows, vocab))
    fa.check(lib.fa_fill_normal(be._ctx, logits._h, 0, rows * vocab, 5, 0.0, 3.0))
    gen = be.new_generator(1)
    out = be.alloc_uninit((rows,), fa.capi.I32)
    res = {}
    for name, strategy, temperature, k in (("greedy", 0, 1.0, 0), ("temperature", 1, 0.8, 0), ("top_k_50", 2, 1.0, 50)):
        sec = time_launches(fa, be, lambda: fa.check(lib.fa_sample_rows(be._ctx, logits._h, rows, vocab, strategy, temperature,
                                                                       k, gen._h, out._h)), iters)
        res[name + "_us"] = sec * 1e6
    for b in (logits, gen, out):
        b.free()
    return res


def bench_matrix_rate(fa, be, iters=20000):
    """Register-only rate of the matrix instructions the prefill GEMMs use, with all-zero and with
    random operand bits (the sustained clock of the part depends on the bits it multiplies)."""
    lib = fa.capi.lib
    rng = np.random.default_rng(7)
    rand = rng.integers(0, 256, size=65536, dtype=np.uint8)
    rand[(rand & 0x7F) == 0x7F] = 0x3C                  # no e4m3 NaN codes
    sink = be.alloc_zeroed((1,), fa.capi.I32)
    res = []
    for fill, data in (("zero operands", np.zeros(65536, np.uint8)), ("random operand bits", rand)):
        src = be.upload(data)
        for kind, name in enumerate(("v_mfma_i32_16x16x64_i8", "v_mfma_i32_32x32x32_i8", "v_mfma_scale_f32_16x16x128_f8f6f4 (e4m3)")):
            ops = C.c_double()
            fa.check(lib.fa_probe_matrix_rate(be._ctx, kind, src._h, 200, sink._h, C.byref(ops)))
            be.synchronize_device()
            t = Timer(fa, be)
            t.start()
            fa.check(lib.fa_probe_matrix_rate(be._ctx, kind, src._h, iters, sink._h, C.byref(ops)))
            ms = t.stop_ms()
            res.append(dict(instr=name, fill=fill, ms=ms, tops=ops.value / (ms * 1e-3) / 1e12))
        src.free()
    sink.free()
    return res


def bench_stream_floor(fa, be, sizes, reps=30):
    """Streaming read of `sizes` bytes (fa_probe_stream_read, 512 blocks of 512 threads, the non-temporal
    16-byte loads the kernels use for read-once data), each launch on a fresh window of a 4 GiB buffer so that
    nothing is served from the 256 MB memory-side cache: the best a memory-bound kernel that must fetch that
    many bytes can do on this part, launch ramp and tail included.  us_ordinary_loads: the same read with
    ordinary loads."""
    lib = fa.capi.lib
    total = 4 << 30
    buf = be.alloc_uninit((total // 4,))
    fa.check(lib.fa_fill_normal(be._ctx, buf._h, 0, total // 4, 3, 0.0, 1.0))
    sink = be.alloc_zeroed((1,), fa.capi.I32)
    res = []
    for name, nbytes in sizes:
        nb = nbytes // (16 * 512) * (16 * 512)
        win = (nb + 4095) // 4096 * 4096
        nwin = total // win

        counter = [0]

        def launch():
            # every launch of the replayed graph reads another window
            fa.check(lib.fa_probe_stream_read(be._ctx, buf._h, (counter[0] % nwin) * win, nb, 512, 512, sink._h))
            counter[0] += 1
        us = time_launches(fa, be, launch, reps, warmup=3) * 1e6
        fa.check(lib.fa_set_tuning(15, 1))
        try:
            us_plain = time_launches(fa, be, launch, reps, warmup=3) * 1e6
        finally:
            fa.check(lib.fa_set_tuning(15, 0))
        res.append(dict(what=name, bytes=nb, us=us, gbs=nb / us / 1e3, frac=nb / us / 1e3 / HBM_PEAK_GBS,
                        us_ordinary_loads=us_plain))
    buf.free()
    sink.free()
    return res


def bench_l2_path(fa, be, reps=20):
    """The path from L2 to the compute units (fa_probe_l2_path).  (1) A 1 MiB region that every block reads over and
    over (L2 hits after the first touch) at 2, 8 and 16 wavefronts per compute unit: what a compute unit can pull
    from L2.  (2) A 58.7 MB stream from memory no launch has touched (fresh windows of a 4 GiB buffer), 256 blocks
    of 512 threads as the decode linears launch, alone and with two L2-hit loads mixed in per streamed load, at 8
    and 16 streamed loads per thread in flight: what operand re-reads that hit in L2 cost an HBM stream."""
    lib = fa.capi.lib
    cus = be.info().compute_units
    total = 4 << 30
    cold = be.alloc_uninit((total // 4,))
    fa.check(lib.fa_fill_normal(be._ctx, cold._h, 0, total // 4, 3, 0.0, 1.0))
    hot = be.alloc_uninit(((1 << 20) // 4,))
    fa.check(lib.fa_fill_normal(be._ctx, hot._h, 0, (1 << 20) // 4, 4, 0.0, 1.0))
    sink = be.alloc_zeroed((1,), fa.capi.I32)
    res = []
    hot_bytes, passes = 1 << 20, 16
    for waves, blocks, threads in ((2, cus, 128), (8, cus, 512), (16, 2 * cus, 512)):
        def launch():
            fa.check(lib.fa_probe_l2_path(be._ctx, cold._h, 0, 0, hot._h, hot_bytes, passes, 8, 0, blocks, threads, sink._h))
        us = time_launches(fa, be, launch, reps, warmup=3) * 1e6
        nbytes = blocks * hot_bytes * passes
        res.append(dict(what="L2-resident region, %d wavefronts per compute unit" % waves, blocks=blocks, threads=threads,
                        us=us, gbs=nbytes / us / 1e3, gbs_per_cu=nbytes / us / 1e3 / cus))
    nb = 58720256
    win = (nb + 4095) // 4096 * 4096
    nwin = total // win
    for in_flight, ratio in ((8, 0), (16, 0), (8, 2), (16, 2)):
        counter = [0]

        def launch():
            fa.check(lib.fa_probe_l2_path(be._ctx, cold._h, (counter[0] % nwin) * win, nb, hot._h, 256 << 10, 0, in_flight, ratio,
                                          cus, 512, sink._h))
            counter[0] += 1
        us = time_launches(fa, be, launch, reps, warmup=3) * 1e6
        res.append(dict(what="58.7 MB from HBM, %d loads in flight per thread, %s" %
                             (in_flight, "alone" if ratio == 0 else "%d L2-hit loads per streamed load" % ratio),
                        blocks=cus, threads=512, us=us, gbs=nb / us / 1e3, gbs_per_cu=nb / us / 1e3 / cus,
                        l2_hit_gbs=ratio * nb / us / 1e3))
    for b in (cold, hot, sink):
        b.free()
    return res


def floor_sizes(cfg, att_bytes):
    D, F, V = cfg["d_model"], cfg["d_ffn"], cfg["vocab"]
    EQ, EKV = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    return [("o projection weight 4096x4096", EQ * D), ("qkv weight 4096x6144", D * (EQ + 2 * EKV)),
            ("config-2 weight 11008x4096", 11008 * 4096), ("config-2 weight 4096x12288", 4096 * 12288),
            ("down weight 14336x4096", F * D),
            ("config-2 weight 4096x22016", 4096 * 22016), ("gate/up weight 4096x28672", D * 2 * F),
            ("lm_head weight 4096x32000", D * V), ("decode attention K/V of one layer", att_bytes)]


# ---------------------------------------------------------------- CPU baseline
def cpu_baseline(fa, be, cfg, batch, ctxs, threads, keep, tables, max_blocks, num_blocks):
    """The CPU oracle (a restatement of the reference's backend-cpu algorithms; the Rust crate cannot be
    built on this host) on ONE layer plus the lm_head of the same workload, scaled to the full depth.  The operands
    are the GPU's own: layer 0's norms, quantized weights (codes and channel scales exported from the device), the
    embedding, the head, the block tables, and layer 0's K / V pools regenerated from the seeds that filled them."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as o
    from decoder_common import Model, oracle_step
    lib = fa.capi.lib
    one = dict(cfg, n_layers=1)
    m = Model()
    m.cfg, m.batch = dict(one), batch
    m.cfg["max_blocks_per_seq"], m.cfg["num_blocks"], m.tables = max_blocks, num_blocks, tables
    V = cfg["vocab"]
    EKV = cfg["n_kv_heads"] * cfg["head_dim"]
    # build_decoder keeps, per layer: attn norm, ffn norm, qkv, o, gate|up, down; then embedding, final norm, head
    n1, n2, wqkv, wo, wgu, wdown = keep[:6]
    embed, final_norm, lm = keep[-3:]
    m.embed = be.download(embed)
    m.final_norm = be.download(final_norm)
    m.lm = lm.export()

    def pool(seed):
        t = be.alloc_uninit((num_blocks, cfg["block_size"], EKV), fa.capi.BF16)
        fa.check(lib.fa_fill_normal(be._ctx, t._h, 0, t.numel(), seed, 0.0, 1.0))
        h = be.download(t)
        t.free()
        return h

    m.layers = [dict(attn_norm=be.download(n1), ffn_norm=be.download(n2), wqkv=wqkv.export(), wo=wo.export(),
                     wgu=wgu.export(), wdown=wdown.export(), k_pool=pool(1000 + 7), v_pool=pool(1000 + 8))]
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, V, size=batch).astype(np.int32)
    oracle_step(m, np.asarray(ctxs, dtype=np.uint32).copy(), tokens, threads=threads)   # warm-up
    times = []
    for _ in range(3):                                    # one iteration takes seconds: warm-up 1, 3 timed, median
        lens = np.asarray(ctxs, dtype=np.uint32).copy()
        t0 = time.perf_counter()
        oracle_step(m, lens, tokens, threads=threads)
        times.append(time.perf_counter() - t0)
    t_one = float(np.median(times))
    # separate the lm_head share: time a zero-layer-equivalent by timing the head alone
    x = rng.standard_normal((batch, cfg["d_model"]), dtype=np.float32)
    o.set_threads(threads)
    t0 = time.perf_counter()
    o.linear_w8a8(x, m.lm[0], m.lm[1])
    t_head = time.perf_counter() - t0
    o.set_threads(1)
    t_layer = max(t_one - t_head, 1e-9)
    t_full = t_layer * cfg["n_layers"] + t_head
    return dict(value=batch / t_full, unit="tokens/s", cores=threads, kind="port",
                sample="CPU oracle (C++ restatement of backend-cpu, not the Rust binary): 1 of %d layers + lm_head at "
                       "batch %d on the GPU's own layer-0 weights, head, tables and K / V contents, same contexts, warm-up 1 + "
                       "median of 3 timed passes, %.2f s per layer measured, scaled "
                       "to the full depth" % (cfg["n_layers"], batch, t_layer))


def _median_time(fn, min_iters, budget_s):
    """Median seconds of fn after one warm-up: at least min_iters timed calls, more while the budget lasts (up to 20)."""
    fn()
    times = []
    t_start = time.perf_counter()
    while len(times) < min_iters or (len(times) < 20 and time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times)), len(times)


def cpu_operator_baselines(fa, be, threads):
    """The CPU oracle beside the operator figures of `extras`, on the operands the GPU itself used (the codes and
    scales are read back from the device), with the GPU result judged against the CPU result in the same run.
    Each entry: CPU seconds (median, iterations stated), the GPU / CPU parity line, and what was sampled where one CPU
    pass over the full operator would take minutes."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as o
    lib = fa.capi.lib
    o.set_threads(threads)
    res = {"cores": threads, "kind": "port",
           "note": "C++ restatement of backend-cpu (not the Rust binary), OpenMP over independent rows / columns"}
    # decode-shape W8A16 sweep (config 2)
    gemv = []
    for k, n in ((4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)):
        w = be.alloc_uninit((k, n))
        fa.check(lib.fa_fill_normal(be._ctx, w._h, 0, k * n, k + n, 0.0, 0.02))
        qw = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)))
        w.free()
        codes, scales = qw.export()
        for m in (1, 8, 32):
            a = be.alloc_uninit((m, k), fa.capi.BF16)
            fa.check(lib.fa_fill_normal(be._ctx, a._h, 0, m * k, 5, 0.0, 1.0))
            out = be.alloc_uninit((m, n), fa.capi.F32)
            fa.check(lib.fa_linear_w8a16(be._ctx, a._h, m, qw._h, out._h))
            got, a_host = be.download(out), be.download(a)
            want = o.linear_w8a16(a_host, codes, scales)
            sec, iters = _median_time(lambda: o.linear_w8a16(a_host, codes, scales), 5, 0.5)
            r = o.compare(got, want)
            gemv.append(dict(op="w8a16", m=m, k=k, n=n, cpu_us=sec * 1e6, iters=iters, parity_fail=int(r.fail_count),
                             parity=r.line("W8A16_PARITY", "%dx%dx%d" % (m, n, k))))
            a.free(), out.free()
        qw.free()
    res["decode_linears"] = gemv
    # paged attention, config 3
    rng = np.random.default_rng(3)
    c3 = np.random.default_rng(0).integers(128, 4097, size=64).tolist()
    tables, max_blocks, num_blocks = make_tables(rng, c3, 0, 16, 40000)
    kp = be.alloc_uninit((num_blocks, 16, 1024), fa.capi.BF16)
    vp = be.alloc_uninit((num_blocks, 16, 1024), fa.capi.BF16)
    q = be.alloc_uninit((64, 1, 4096), fa.capi.BF16)
    for b, sd in ((kp, 31), (vp, 32), (q, 33)):
        fa.check(lib.fa_fill_normal(be._ctx, b._h, 0, b.numel(), sd, 0.0, 1.0))
    lens = np.asarray(c3, dtype=np.uint32)
    layout = fa.PagedKvLayout.new(num_blocks, 16, 1024)
    args = fa.PagedAttentionArgs(layout, 64, 1, 32, max_blocks, fa.default_scale(128), 8)
    got = be.download(be.paged_attention_forward(q, kp, vp, tables, lens, args, out_dtype=fa.capi.F32))
    kph, vph, qh = be.download(kp), be.download(vp), be.download(q)
    oargs = o.paged_args(num_blocks, 16, 1024, 64, 1, 32, max_blocks, args.scale, 8)
    rc, want = o.paged_attention_bf16(qh, kph, vph, tables, lens, oargs)
    sec, iters = _median_time(lambda: o.paged_attention_bf16(qh, kph, vph, tables, lens, oargs), 3, 3.0)
    r = o.compare(got, want)
    res["paged_attention_bs64"] = dict(cpu_us=sec * 1e6, iters=iters, parity_fail=int(r.fail_count),
                                       parity=r.line("PAGED_DECODE_PARITY", "bs64"))
    for b in (kp, vp, q):
        b.free()
    # prefill GEMMs, config 4: the CPU takes a sample of the rows (all columns, full k) and is scaled
    m, k, n, rows = 2048, 4096, 14336, 32
    w = be.alloc_uninit((k, n))
    x = be.alloc_uninit((m, k))
    fa.check(lib.fa_fill_normal(be._ctx, w._h, 0, k * n, 11, 0.0, 1.0))
    fa.check(lib.fa_fill_normal(be._ctx, x._h, 0, m * k, 12, 0.0, 1.0))
    sel = np.linspace(0, m - 1, rows).astype(np.int64)
    gemm = []
    qw = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)))
    xq, sx = be.quantize_rows_i8(x)
    out, acc = be.gemm_w8a8(xq, sx, qw, fa.capi.F32, want_acc=True)
    codes, scales = qw.export()
    a_rows = np.ascontiguousarray(be.download(xq)[sel])
    sec, iters = _median_time(lambda: o.gemm_i8_i32(a_rows, codes), 3, 2.0)
    want_acc = o.gemm_i8_i32(a_rows, codes)
    mism = int((be.download(acc)[sel] != want_acc).sum())
    gemm.append(dict(op="gemm_w8a8", m=m, k=k, n=n, cpu_ms_full=sec * m / rows * 1e3, sampled_rows=rows, iters=iters,
                     acc_bit_mismatch=mism))
    for b in (qw, xq, sx, out, acc):
        b.free()
    qw = be.quantize_weight(fa.DeviceBufferView(w, 0, (k, n)), fa.capi.QW_E4M3_TENSOR)
    xq, xs = be.quantize_tensor_e4m3(x)
    got = be.download(be.gemm_e4m3(xq, xs, qw, fa.capi.F32))[sel]
    codes, wscale = qw.export()
    a_rows = np.ascontiguousarray(be.download(xq)[sel])
    sa, sw = np.float32(be.download(xs)[0]), np.float32(wscale[0])
    sec, iters = _median_time(lambda: o.gemm_e4m3(a_rows, codes, sa, sw), 3, 2.0)
    want = o.gemm_e4m3(a_rows, codes, sa, sw)
    r = o.compare(got, want)
    # the fp8 bar: every output within 2^-15 * sum_k |a_k||b_k| * (sa * sw) of the exact-product f64 sum (the f32
    # accumulation of the matrix cores), and at least 98 % of them inside rel < 1e-3 or abs < 1e-5 as well
    absprod = np.abs(o.from_e4m3(a_rows)).astype(np.float64) @ np.abs(o.from_e4m3(codes)).astype(np.float64)
    bound = absprod * float(sa) * float(sw) * 2.0 ** -15 + 1e-30
    over = int((np.abs(got.astype(np.float64) - want.astype(np.float64)) > bound).sum())
    gemm.append(dict(op="gemm_e4m3", m=m, k=k, n=n, cpu_ms_full=sec * m / rows * 1e3, sampled_rows=rows, iters=iters,
                     parity_fail=over + (int(r.fail_count) if r.fail_count > 2e-2 * r.total else 0),
                     outside_fp8_bound=over, outside_composite=int(r.fail_count), total=int(r.total),
                     parity=r.line("FP8_PARITY", "%dx%dx%d" % (m, n, k))))
    for b in (qw, xq, xs, w, x):
        b.free()
    res["prefill_gemm"] = gemm
    o.set_threads(1)
    return res


# ------------------------------------------------------------------------ main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=MODEL["n_layers"], help="debug only: fewer layers (invalidates the metric)")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-serving", action="store_true",
                    help="skip the single-request prompt passes and the continuous-batching run (profiling aid: "
                         "keeps the decode kernels of the trace at the benchmark's own shape)")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--attn-waves", type=int, default=0,
                    help="tuning: wavefronts per compute unit of the decode attention (0 = built-in)")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="tuning: raw fa_set_tuning key/value pairs (experiments)")
    ap.add_argument("--rows", type=int, default=0,
                    help="with --only decode-linears: one row count of the sweep instead of 1, 8 and 32")
    ap.add_argument("--shape", type=int, default=-1,
                    help="with --only decode-linears: one of the four layer shapes (0 .. 3) instead of all, so that "
                         "a counter run sees launches of one shape only")
    ap.add_argument("--only", choices=("attention", "copy", "linears", "decode-linears", "prefill", "prefill-attention", "mfma",
                                       "prompt", "stream-floor", "gemm-f32", "l2-path", "single-stream"), default=None,
                    help="profiling aid: run only the dominant kernel at the workload's shape, or a plain "
                         "copy kernel of known size (counter calibration), a few launches, no JSON line")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); nothing here shards across devices")

    import fandhe_ai_amd as fa
    be = fa.tape_for(fa.Device.Rocm(0))
    info = be.info()
    log("device", info.arch.decode(), "CUs", info.compute_units, "clock_khz", info.clock_khz)
    lib = fa.capi.lib
    fa.check(lib.fa_set_tuning(2, a.attn_waves))
    for kv in a.tune:
        key, value = kv.split("=")
        fa.check(lib.fa_set_tuning(int(key), int(value)))
    cfg = dict(MODEL, n_layers=a.layers)
    batch = 32
    ctxs = np.random.default_rng(0).integers(1024, 8193, size=batch).tolist()
    if a.only is not None:
        mid_ctx = [c + a.warmup + a.steps // 2 for c in ctxs]
        if a.only in ("prefill", "prefill-attention"):
            if a.only == "prefill":
                for r in bench_prefill(fa, be, 20):
                    log("%s m=%d k=%d n=%d: %.1f us, %.0f TOPS (%.1f %% of peak)" %
                        (r["op"], r["m"], r["k"], r["n"], r["us"], r["tops"], 100 * r["frac"]))
            for r in bench_prefill_attention(fa, be):
                log("prefill attention 4 x 2048 new tokens, 32/8 heads, %s kernel: %.2f ms, %.1f TFLOP/s" %
                    (r["kernel"], r["ms"], r["tflops"]))
            be.close()
            return
        if a.only == "prompt":
            dec, keep, tables, _, _ = build_decoder(fa, be, cfg, batch, ctxs, 4)
            for r in bench_short_prompts(fa, be, dec, cfg, tables):
                log("one prompt of %d tokens%s through %d layers: %.2f ms, %.0f tokens/s" %
                    (r["l_new"], " after %d cached" % r["cached"] if r["cached"] else "", cfg["n_layers"], r["ms"], r["tokens_per_s"]))
            lib.fa_decoder_destroy(be._ctx, dec)
            be.close()
            return
        if a.only == "single-stream":
            dec, keep, tables, _, _ = build_decoder(fa, be, cfg, batch, ctxs, 300, max_batch=batch)
            r = bench_single_stream(fa, be, dec, cfg, tables)
            log("one sequence decoding alone through %d layers: %.3f ms per token; verifying 5 positions in one step: %.3f ms" %
                (cfg["n_layers"], r["ms_per_token"], r["verify_5_positions_ms"]))
            lib.fa_decoder_destroy(be._ctx, dec)
            be.close()
            return
        if a.only == "gemm-f32":
            for r in bench_gemm_f32(fa, be, 10):
                log("f32 gemm_device m=%d k=%d n=%d: %.1f us, %.1f TFLOP/s (%.1f %% of the f32 matrix peak)" %
                    (r["m"], r["k"], r["n"], r["us"], r["tflops"], 100 * r["frac"]))
            be.close()
            return
        if a.only == "mfma":
            for r in bench_matrix_rate(fa, be):
                log("%-42s %-20s: %.2f ms, %.0f T op/s (%.1f %% of peak)" %
                    (r["instr"], r["fill"], r["ms"], r["tops"], 100 * r["tops"] / MFMA_PEAK_TOPS))
            be.close()
            return
        if a.only == "l2-path":
            for r in bench_l2_path(fa, be):
                log("%-78s %4d x %3d threads: %8.2f us, %7.0f GB/s (%5.1f GB/s per compute unit)%s" %
                    (r["what"], r["blocks"], r["threads"], r["us"], r["gbs"], r["gbs_per_cu"],
                     ", L2 hits %.0f GB/s" % r["l2_hit_gbs"] if r.get("l2_hit_gbs") else ""))
            be.close()
            return
        if a.only == "stream-floor":
            for r in bench_stream_floor(fa, be, floor_sizes(cfg, attention_bytes(sum(mid_ctx), mid_ctx, cfg["n_heads"], cfg["n_kv_heads"]))):
                log("streaming read of %-36s %10d bytes: %7.2f us, %5.0f GB/s (%.1f %% of peak); ordinary loads %7.2f us" %
                    (r["what"], r["bytes"], r["us"], r["gbs"], 100 * r["frac"], r["us_ordinary_loads"]))
            be.close()
            return
        if a.only == "decode-linears":
            shapes = LINEAR_SHAPES if a.shape < 0 else LINEAR_SHAPES[a.shape:a.shape + 1]
            for r in bench_linears(fa, be, 20, (a.rows,) if a.rows else (1, 8, 32), shapes):
                log("w8a16 m=%d %5d->%5d: %.2f us, %.0f GB/s (%.1f %% of peak)" %
                    (r["m"], r["k"], r["n"], r["us"], r["gbs"], 100 * r["frac"]))
            be.close()
            return
        if a.only == "linears":
            for r in bench_w8a8_decode(fa, be, cfg, batch, 20):
                log("w8a8 m=%d %5d->%5d: %.2f us per call (quantizer + GEMV), %.0f GB/s" %
                    (r["m"], r["k"], r["n"], r["us"], r["gbs"]))
            be.close()
            return
        if a.only == "attention":
            sec, nb, sec_k = bench_attention(fa, be, batch, cfg["n_heads"], cfg["n_kv_heads"], mid_ctx, None, 10, seed=4,
                                             kernel_only=True)
            log("attention streaming kernel alone: %.2f us per launch, %.0f GB/s" % (sec_k * 1e6, nb / sec_k / 1e9))
        else:
            sec, nb = bench_copy(fa, be, 10)
        log("%s: %.2f us per launch, %d algorithmic bytes, %.0f GB/s" % (a.only, sec * 1e6, nb, nb / sec / 1e9))
        be.close()
        return
    t0 = time.time()
    # rows for twice the benchmark's batch: the serving run below fills them; the timed steps use `batch`
    dec, keep, tables, max_blocks, num_blocks = build_decoder(fa, be, cfg, batch, ctxs, a.steps + a.warmup,
                                                              max_batch=SERVING_ROWS)
    log("model resident in %.1f s; sum ctx = %d" % (time.time() - t0, sum(ctxs)))

    use_graph = 0 if a.no_graph else 1
    for _ in range(a.warmup):
        fa.check(lib.fa_decoder_step(be._ctx, dec, use_graph))
    be.synchronize_device()
    timer = Timer(fa, be)
    wall0 = time.perf_counter()
    timer.start()
    for _ in range(a.steps):
        fa.check(lib.fa_decoder_step(be._ctx, dec, use_graph))
    ms = timer.stop_ms()
    be.synchronize_device()
    wall = time.perf_counter() - wall0
    sec_per_step = max(ms * 1e-3, wall) / a.steps if abs(ms * 1e-3 - wall) > 0.2 * wall else ms * 1e-3 / a.steps
    toks = np.empty(batch, dtype=np.int32)
    fa.check(lib.fa_decoder_read_tokens(be._ctx, dec, toks.ctypes.data_as(fa.capi.i32p)))
    logits = np.empty((batch, cfg["vocab"]), dtype=np.float32)
    fa.check(lib.fa_decoder_read_logits(be._ctx, dec, logits.ctypes.data_as(fa.capi.f32p)))
    assert np.all(np.isfinite(logits)) and np.all((toks >= 0) & (toks < cfg["vocab"]))
    mid_ctx = [c + a.warmup + a.steps // 2 for c in ctxs]
    bytes_step = step_bytes(cfg, batch, sum(mid_ctx))
    log("step %.3f ms (events %.3f ms, wall %.3f ms); algorithmic bytes/step %.2f GB -> %.0f GB/s" %
        (sec_per_step * 1e3, ms / a.steps, wall / a.steps * 1e3, bytes_step / 1e9, bytes_step / sec_per_step / 1e9))
    prompt = None
    if not a.no_extras and min(ctxs) >= 2048 // 2:
        # the pages of the first sequences hold at least 2049 tokens each only if their context is that long;
        # pick the four longest rows of the table
        order = np.argsort(ctxs)[::-1][:4]
        if min(ctxs[i] for i in order) > 2048:
            prompt = bench_prompt_prefill(fa, be, dec, cfg, np.ascontiguousarray(tables[order]))
            log("prompt prefill %d x %d tokens: %.1f ms, %.0f tokens/s" %
                (prompt["batch"], prompt["l_new"], prompt["ms"], prompt["tokens_per_s"]))
    batching = short = single = None
    if not a.no_extras and not a.no_serving:
        short = bench_short_prompts(fa, be, dec, cfg, tables)
        log("one prompt, batch 1: " + ", ".join("%d tokens%s %.2f ms" % (r["l_new"], " after %d cached" % r["cached"] if r["cached"] else "", r["ms"])
                                                for r in short))
        single = bench_single_stream(fa, be, dec, cfg, tables)
        log("one sequence decoding alone: %.3f ms per token (%.0f tokens/s, weights streamed at %.0f GB/s); "
            "verifying 5 positions in one step: %.3f ms" %
            (single["ms_per_token"], single["tokens_per_s"], single["weight_stream_gbs"], single["verify_5_positions_ms"]))
        dcfg = fa.capi.DecoderConfig(cfg["n_layers"], cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"],
                                     cfg["d_ffn"], cfg["vocab"], cfg["block_size"], max_blocks, num_blocks, SERVING_ROWS,
                                     cfg["rms_eps"], cfg["rope_theta"])
        batching = bench_continuous_batching(fa, be, dec, dcfg, requests=3 * SERVING_ROWS, max_active=SERVING_ROWS)
        log("continuous batching: %d requests, %d generated tokens in %.2f s -> %.0f generated tokens/s "
            "(mean %.1f active rows)" % (batching["requests"], batching["generated_tokens"], batching["seconds"],
                                         batching["generated_tokens_per_s"], batching["mean_active_rows"]))
    threads = min(16, os.cpu_count() or 1)
    cpu_base = None
    if not a.no_cpu_baseline:                            # before the model's buffers go: the CPU is timed on them
        cpu_base = cpu_baseline(fa, be, cfg, batch, ctxs, threads, keep, tables, max_blocks, num_blocks)
    lib.fa_decoder_destroy(be._ctx, dec)
    for x in keep:
        x.free()
    be.release_cached_device_memory()

    # dominant operator at this workload's shape: paged decode attention of one layer
    att_sec, att_bytes, att_kernel_sec = bench_attention(fa, be, batch, cfg["n_heads"], cfg["n_kv_heads"], mid_ctx,
                                                         None, 50, seed=4, kernel_only=True)
    # Dominant kernel: decode_stream_kernel of the paged attention (about 60 % of the step).  Its launch
    # is timed by itself; the whole operator (that kernel + the merge of the partial results) is given
    # beside it.  traffic: HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE of this kernel at
    # this shape, scaled by a copy kernel of known size (profiles/decode_stream_kernel_config5_pmc.txt).
    roofline = dict(bound="hbm", kernel="decode_stream_kernel (paged GQA decode attention, one layer)",
                    achieved=att_bytes / att_kernel_sec / 1e9, peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=att_bytes / att_kernel_sec / 1e9 / HBM_PEAK_GBS, traffic=ATTENTION_TRAFFIC_BYTES,
                    bytes_per_launch=att_bytes, us_per_launch=att_kernel_sec * 1e6,
                    operator_us=att_sec * 1e6, operator_achieved=att_bytes / att_sec / 1e9)
    extras = {"step_algorithmic_gb": bytes_step / 1e9, "step_hbm_frac": bytes_step / sec_per_step / 1e9 / HBM_PEAK_GBS}
    if prompt is not None:
        extras["prompt_prefill"] = prompt
    if short is not None:
        extras["prompt_pass_one_request"] = short
        extras["single_stream_decode"] = single
    if batching is not None:
        extras["continuous_batching"] = batching
    if not a.no_extras:
        c3 = np.random.default_rng(0).integers(128, 4097, size=64).tolist()
        sec, nb = bench_attention(fa, be, 64, 32, 8, c3, 40000, 50, seed=3)
        extras["paged_attention_bs64"] = dict(us=sec * 1e6, gbs=nb / sec / 1e9, frac=nb / sec / 1e9 / HBM_PEAK_GBS,
                                              bytes=nb)
        extras["decode_linears"] = bench_linears(fa, be, 100)
        extras["sampling_32x32000"] = bench_sampling(fa, be)
        extras["prefill_gemm"] = bench_prefill(fa, be, 20)
        extras["gemm_device_f32"] = bench_gemm_f32(fa, be, 10)
        for r in extras["gemm_device_f32"]:
            log("f32 gemm_device m=%d k=%d n=%d: %.1f us, %.1f TFLOP/s (%.1f %% of the f32 matrix peak)" %
                (r["m"], r["k"], r["n"], r["us"], r["tflops"], 100 * r["frac"]))
        # what a plain streaming read of the same bytes reaches: the yardstick for the bandwidth-bound kernels
        extras["stream_read_floor"] = bench_stream_floor(fa, be, floor_sizes(cfg, att_bytes))
    out = {
        "metric": METRIC, "value": batch / sec_per_step, "unit": "tokens/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": sec_per_step * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 (int32 accumulate) linears, bf16 KV / f32 accumulate attention",
        "data": "synthetic: seeded N(0, 0.02) weights quantized per channel on the device, N(0, 1) bf16 KV cache, "
                "contexts uniform in [1024, 8192] (seed 0), block tables a seeded permutation",
        "config": {"workload": "full decode step, 32-layer Llama-style decoder, batch 32, paged KV page 16"
                               if a.layers == MODEL["n_layers"] else "DEBUG %d layers" % a.layers,
                   "batch": batch, "sum_ctx": int(sum(mid_ctx)), "graph": bool(use_graph)},
        "roofline": roofline, "extras": extras,
    }
    out["cpu_baseline"] = cpu_base
    if not a.no_cpu_baseline:
        if not a.no_extras:
            extras["cpu_operator_baselines"] = cpu_operator_baselines(fa, be, threads)
    be.close()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
