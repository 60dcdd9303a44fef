"""Builds a random-init Llama-style decoder both for the HIP library and for
the CPU oracle (same weights, same KV pools, same block tables)."""
import ctypes as C

import numpy as np

import oracle_lib as o

U32MAX = 0xFFFFFFFF


class Model:
    pass


def build_model(seed, n_layers, d_model, n_heads, n_kv_heads, d_ffn, vocab, batch, ctxs, steps, num_blocks=None,
                head_dim=128, block_size=16, quantize_on_host=True, threads=8, numpy_fill=False):
    """Weights ~N(0, 0.02) quantized per output channel; norm weights ~1; KV pools pre-filled for the
    given context lengths; block tables sized for `steps` more tokens.  numpy_fill: the large tensors come
    from numpy's generator instead of the reference's (for models of hundreds of millions of elements)."""
    rng = o.Rng(seed)
    if numpy_fill:
        class _Fast:
            def __init__(self, base, seed):
                self.base, self.np = base, np.random.default_rng(seed)

            def randn(self, shape, std=1.0):
                if int(np.prod(shape)) < 1 << 20:
                    return self.base.randn(shape, std=std) if std != 1.0 else self.base.randn(shape)
                return (self.np.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)

            def __getattr__(self, name):
                return getattr(self.base, name)
        rng = _Fast(rng, seed)
    m = Model()
    m.cfg = dict(n_layers=n_layers, d_model=d_model, n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim,
                 d_ffn=d_ffn, vocab=vocab, block_size=block_size, rms_eps=1e-5, rope_theta=500000.0)
    eq, ekv = n_heads * head_dim, n_kv_heads * head_dim
    m.batch = batch
    max_blocks = max((c + steps + block_size - 1) // block_size for c in ctxs) + 1
    need = sum((c + steps + block_size - 1) // block_size for c in ctxs)
    num_blocks = num_blocks or need + 5
    assert need <= num_blocks
    m.cfg["max_blocks_per_seq"], m.cfg["num_blocks"] = max_blocks, num_blocks
    perm = rng.permutation(num_blocks)
    m.tables = np.full((batch, max_blocks), U32MAX, dtype=np.uint32)
    p = 0
    for b, c in enumerate(ctxs):
        nb = (c + steps + block_size - 1) // block_size
        m.tables[b, :nb] = perm[p:p + nb]
        p += nb
    m.used_blocks = perm[:p]
    m.seq_lens = np.array(ctxs, dtype=np.uint32)
    m.tokens = rng.randint(0, vocab, batch).astype(np.int32)

    o.set_threads(threads)

    def qweight(k, n):
        w = rng.randn((k, n), std=0.02)
        return o.quantize_cols_i8(w)

    m.embed = rng.randn((vocab, d_model))
    m.final_norm = (1.0 + rng.randn((d_model,), std=0.1)).astype(np.float32)
    m.lm = qweight(d_model, vocab)
    m.layers = []
    for _ in range(n_layers):
        L = dict(attn_norm=(1.0 + rng.randn((d_model,), std=0.1)).astype(np.float32),
                 ffn_norm=(1.0 + rng.randn((d_model,), std=0.1)).astype(np.float32),
                 wqkv=qweight(d_model, eq + 2 * ekv), wo=qweight(eq, d_model),
                 wgu=qweight(d_model, 2 * d_ffn), wdown=qweight(d_ffn, d_model))
        kp = np.zeros((num_blocks, block_size, ekv), np.uint16)
        vp = np.zeros((num_blocks, block_size, ekv), np.uint16)
        kp[m.used_blocks] = o.to_bf16(rng.randn((p, block_size, ekv)))
        vp[m.used_blocks] = o.to_bf16(rng.randn((p, block_size, ekv)))
        L["k_pool"], L["v_pool"] = kp, vp
        m.layers.append(L)
    o.set_threads(1)
    return m


def oracle_step(m, seq_lens, tokens, threads=8):
    """One oracle decode step; updates the model's host KV pools and `seq_lens` in place."""
    cfg = o.DecoderConfig(m.cfg["n_layers"], m.cfg["d_model"], m.cfg["n_heads"], m.cfg["n_kv_heads"],
                          m.cfg["head_dim"], m.cfg["d_ffn"], m.cfg["vocab"], m.cfg["block_size"],
                          m.cfg["max_blocks_per_seq"], m.cfg["num_blocks"], m.cfg["rms_eps"], m.cfg["rope_theta"])
    nl = m.cfg["n_layers"]
    f32pp = o.f32p * nl
    i8pp = o.i8p * nl
    u16pp = o.u16p * nl

    def fpp(key, idx=None):
        return f32pp(*[o.ptr(L[key] if idx is None else L[key][idx], o.f32p) for L in m.layers])

    def ipp(key):
        return i8pp(*[o.ptr(L[key][0], o.i8p) for L in m.layers])

    w = o.DecoderWeights(o.ptr(m.embed, o.f32p), fpp("attn_norm"), fpp("ffn_norm"), o.ptr(m.final_norm, o.f32p),
                         ipp("wqkv"), fpp("wqkv", 1), ipp("wo"), fpp("wo", 1), ipp("wgu"), fpp("wgu", 1),
                         ipp("wdown"), fpp("wdown", 1), o.ptr(m.lm[0], o.i8p), o.ptr(m.lm[1], o.f32p))
    kps = u16pp(*[o.ptr(L["k_pool"], o.u16p) for L in m.layers])
    vps = u16pp(*[o.ptr(L["v_pool"], o.u16p) for L in m.layers])
    nxt = np.empty(m.batch, dtype=np.int32)
    logits = np.empty((m.batch, m.cfg["vocab"]), dtype=np.float32)
    o.set_threads(threads)
    rc = o.lib.orc_decode_step(C.byref(cfg), C.byref(w), kps, vps, o.ptr(m.tables, o.u32p), o.ptr(seq_lens, o.u32p),
                               o.ptr(tokens, o.i32p), m.batch, o.ptr(nxt, o.i32p), o.ptr(logits, o.f32p))
    o.set_threads(1)
    assert rc == 0
    return nxt, logits


class GpuDecoder:
    """The same model resident on the GPU behind fa_decoder_*."""

    def __init__(self, be, m):
        import fandhe_ai_amd as fa
        self.fa, self.be, self.m = fa, be, m
        lib = fa.capi.lib
        c = m.cfg
        cfg = fa.capi.DecoderConfig(c["n_layers"], c["d_model"], c["n_heads"], c["n_kv_heads"], c["head_dim"],
                                    c["d_ffn"], c["vocab"], c["block_size"], c["max_blocks_per_seq"],
                                    c["num_blocks"], m.batch, c["rms_eps"], c["rope_theta"])
        self.h = C.c_void_p()
        fa.check(lib.fa_decoder_create(be._ctx, C.byref(cfg), C.byref(self.h)))
        self.keep = []

        def qw(pair):
            q = be.import_quantized_weight(pair[0], pair[1])
            self.keep.append(q)
            return q

        def vec(a):
            b = be.upload(a)
            self.keep.append(b)
            return b

        for li, L in enumerate(m.layers):
            fa.check(lib.fa_decoder_set_layer(self.h, li, vec(L["attn_norm"])._h, vec(L["ffn_norm"])._h,
                                              qw(L["wqkv"])._h, qw(L["wo"])._h, qw(L["wgu"])._h, qw(L["wdown"])._h))
            kp, vp = fa.capi.buf_p(), fa.capi.buf_p()
            fa.check(lib.fa_decoder_kv_pools(self.h, li, C.byref(kp), C.byref(vp)))
            # fill only the used pages: one contiguous upload per pool is simplest at test sizes
            fa.check(lib.fa_upload_into(be._ctx, L["k_pool"].ctypes.data, L["k_pool"].size, kp, 0))
            fa.check(lib.fa_upload_into(be._ctx, L["v_pool"].ctypes.data, L["v_pool"].size, vp, 0))
        fa.check(lib.fa_decoder_set_head(self.h, vec(m.embed)._h, vec(m.final_norm)._h, qw(m.lm)._h))
        self.set_state(m.seq_lens, m.tokens)

    def set_state(self, seq_lens, tokens):
        fa, lib = self.fa, self.fa.capi.lib
        t = np.ascontiguousarray(self.m.tables)
        s = np.ascontiguousarray(seq_lens, dtype=np.uint32)
        fa.check(lib.fa_decoder_set_sequences(self.be._ctx, self.h, self.m.batch, t.ctypes.data_as(fa.capi.u32p),
                                              s.ctypes.data_as(fa.capi.u32p)))
        tk = np.ascontiguousarray(tokens, dtype=np.int32)
        fa.check(lib.fa_decoder_set_tokens(self.be._ctx, self.h, tk.ctypes.data_as(fa.capi.i32p)))

    def step(self, use_graph):
        self.fa.check(self.fa.capi.lib.fa_decoder_step(self.be._ctx, self.h, 1 if use_graph else 0))

    def set_sampling(self, strategy, temperature=1.0, top_k=0, seed=0):
        self.fa.check(self.fa.capi.lib.fa_decoder_set_sampling(self.be._ctx, self.h, strategy, temperature, top_k, seed))

    def prefill(self, prompt):
        """prompt: int32 [batch, l_new]"""
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        assert p.shape[0] == self.m.batch
        self.fa.check(self.fa.capi.lib.fa_decoder_prefill(self.be._ctx, self.h, p.ctypes.data_as(self.fa.capi.i32p),
                                                          p.shape[1]))

    def verify(self, tokens):
        """tokens int32 [batch, l_new] -> (picked [batch, l_new], logits [batch, l_new, vocab])"""
        p = np.ascontiguousarray(tokens, dtype=np.int32)
        picked = np.empty(p.shape, dtype=np.int32)
        logits = np.empty(p.shape + (self.m.cfg["vocab"],), dtype=np.float32)
        self.fa.check(self.fa.capi.lib.fa_decoder_verify(self.be._ctx, self.h, p.ctypes.data_as(self.fa.capi.i32p), p.shape[1],
                                                         picked.ctypes.data_as(self.fa.capi.i32p),
                                                         logits.ctypes.data_as(self.fa.capi.f32p)))
        return picked, logits

    def rewind(self, seq_lens):
        s = np.ascontiguousarray(seq_lens, dtype=np.uint32)
        self.fa.check(self.fa.capi.lib.fa_decoder_rewind(self.be._ctx, self.h, s.ctypes.data_as(self.fa.capi.u32p)))

    def tokens(self):
        out = np.empty(self.m.batch, dtype=np.int32)
        self.fa.check(self.fa.capi.lib.fa_decoder_read_tokens(self.be._ctx, self.h, out.ctypes.data_as(self.fa.capi.i32p)))
        return out

    def logits(self):
        out = np.empty((self.m.batch, self.m.cfg["vocab"]), dtype=np.float32)
        self.fa.check(self.fa.capi.lib.fa_decoder_read_logits(self.be._ctx, self.h, out.ctypes.data_as(self.fa.capi.f32p)))
        return out

    def seq_lens(self):
        out = np.empty(self.m.batch, dtype=np.uint32)
        self.fa.check(self.fa.capi.lib.fa_decoder_read_seq_lens(self.be._ctx, self.h, out.ctypes.data_as(self.fa.capi.u32p)))
        return out

    def kv_pool(self, layer):
        fa, lib = self.fa, self.fa.capi.lib
        kp, vp = fa.capi.buf_p(), fa.capi.buf_p()
        fa.check(lib.fa_decoder_kv_pools(self.h, layer, C.byref(kp), C.byref(vp)))
        shape = self.m.layers[layer]["k_pool"].shape
        k = np.empty(shape, np.uint16)
        v = np.empty(shape, np.uint16)
        fa.check(lib.fa_download(self.be._ctx, kp, 0, k.ctypes.data, k.size))
        fa.check(lib.fa_download(self.be._ctx, vp, 0, v.ctypes.data, v.size))
        return k, v

    def close(self):
        if self.h:
            self.fa.capi.lib.fa_decoder_destroy(self.be._ctx, self.h)
            self.h = None
        for x in self.keep:
            x.free()
        self.keep = []


def llama_checkpoint(seed, n_layers, d, heads, kv, f, vocab, dh=128):
    """Random float32 tensors under the names and [out, in] shapes of a Llama-style safetensors checkpoint."""
    rng = np.random.default_rng(seed)

    def w(*shape):
        return (rng.standard_normal(shape) / np.sqrt(shape[-1])).astype(np.float32)

    t = {"model.embed_tokens.weight": rng.standard_normal((vocab, d)).astype(np.float32),
         "model.norm.weight": (1 + 0.1 * rng.standard_normal(d)).astype(np.float32), "lm_head.weight": w(vocab, d)}
    for i in range(n_layers):
        p = "model.layers.%d." % i
        t[p + "input_layernorm.weight"] = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        t[p + "post_attention_layernorm.weight"] = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        t[p + "self_attn.q_proj.weight"] = w(heads * dh, d)
        t[p + "self_attn.k_proj.weight"] = w(kv * dh, d)
        t[p + "self_attn.v_proj.weight"] = w(kv * dh, d)
        t[p + "self_attn.o_proj.weight"] = w(d, heads * dh)
        t[p + "mlp.gate_proj.weight"] = w(f, d)
        t[p + "mlp.up_proj.weight"] = w(f, d)
        t[p + "mlp.down_proj.weight"] = w(d, f)
    return t
