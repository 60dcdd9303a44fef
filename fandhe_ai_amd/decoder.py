"""Host-side handle of the resident decoder behind ``fa_decoder_*``: a Llama-style stack of W8A8 linears,
RMSNorm, RoPE and paged GQA attention whose weights, KV pools, block tables and generator state stay on the
device; a decode step or a prompt pass only queues kernels."""
import ctypes as C

import numpy as np

from . import capi
from .backend import check

lib = capi.lib


class Decoder:
    def __init__(self, ops, n_layers, d_model, n_heads, n_kv_heads, d_ffn, vocab, max_blocks_per_seq, num_blocks,
                 max_batch, head_dim=128, block_size=16, rms_eps=1e-5, rope_theta=500000.0):
        self._ops = ops
        self.cfg = capi.DecoderConfig(n_layers, d_model, n_heads, n_kv_heads, head_dim, d_ffn, vocab, block_size,
                                      max_blocks_per_seq, num_blocks, max_batch, rms_eps, rope_theta)
        self._h = C.c_void_p()
        check(lib.fa_decoder_create(ops._ctx, C.byref(self.cfg), C.byref(self._h)))
        self._keep = []                                   # weights must outlive the decoder that points at them
        self.batch = 0

    @classmethod
    def from_handle(cls, ops, handle, cfg):
        """Wraps an fa_decoder created elsewhere (not destroyed by ``close``)."""
        d = cls.__new__(cls)
        d._ops, d._h, d.cfg, d._keep, d.batch, d._borrowed = ops, handle, cfg, [], 0, True
        return d

    def close(self):
        if getattr(self, "_borrowed", False):
            self._h = None
            return
        h, self._h = getattr(self, "_h", None), None
        if h and self._ops._ctx:
            lib.fa_decoder_destroy(self._ops._ctx, h)
        for w in self._keep:
            w.free()
        self._keep = []

    def set_layer(self, layer, attn_norm, ffn_norm, wqkv, wo, wgu, wdown):
        """attn_norm / ffn_norm: device buffers [d_model] f32; the others QuantizedWeight (int8, per channel):
        wqkv [d_model, (heads + 2 kv_heads) head_dim], wo [heads head_dim, d_model], wgu [d_model, 2 d_ffn]
        (gate columns first), wdown [d_ffn, d_model]."""
        check(lib.fa_decoder_set_layer(self._h, layer, attn_norm._h, ffn_norm._h, wqkv._h, wo._h, wgu._h, wdown._h))
        self._keep += [attn_norm, ffn_norm, wqkv, wo, wgu, wdown]

    def set_head(self, embed, final_norm, lm_head):
        check(lib.fa_decoder_set_head(self._h, embed._h, final_norm._h, lm_head._h))
        self._keep += [embed, final_norm, lm_head]

    def set_sequences(self, block_tables, seq_lens):
        t = np.ascontiguousarray(block_tables, dtype=np.uint32)
        s = np.ascontiguousarray(seq_lens, dtype=np.uint32)
        check(lib.fa_decoder_set_sequences(self._ops._ctx, self._h, s.size, t.ctypes.data_as(capi.u32p),
                                           s.ctypes.data_as(capi.u32p)))
        self.batch = int(s.size)

    def set_tokens(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        check(lib.fa_decoder_set_tokens(self._ops._ctx, self._h, t.ctypes.data_as(capi.i32p)))

    def set_sampling(self, strategy, temperature=1.0, top_k=0, seed=0):
        check(lib.fa_decoder_set_sampling(self._ops._ctx, self._h, strategy, temperature, top_k, seed))

    def set_row_sampling(self, rows):
        """rows: a ctypes array of ``capi.RowSampling``, one per installed sequence."""
        if len(rows) != self.batch:
            raise ValueError("one sampling record per installed sequence")
        check(lib.fa_decoder_set_row_sampling(self._ops._ctx, self._h, rows))

    def read_row_sampling(self):
        rows = (capi.RowSampling * self.batch)()
        check(lib.fa_decoder_read_row_sampling(self._ops._ctx, self._h, rows))
        return rows

    def prefill(self, prompt):
        """prompt: int32 [batch, l_new]; leaves the next tokens resident like a step."""
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        if p.ndim != 2 or p.shape[0] != self.batch:
            raise ValueError("prompt must be [batch, l_new]")
        check(lib.fa_decoder_prefill(self._ops._ctx, self._h, p.ctypes.data_as(capi.i32p), p.shape[1]))

    def prefill_padded(self, prompts):
        """prompts: one int32 sequence per installed row, of any lengths >= 1; they are padded to the longest
        and ingested in one pass (batch * longest <= 4096).  Every row ends as after its own ``prefill``."""
        if len(prompts) != self.batch:
            raise ValueError("one prompt per installed sequence")
        lens = np.array([len(p) for p in prompts], dtype=np.uint32)
        padded = np.zeros((self.batch, int(lens.max()) if len(prompts) else 0), dtype=np.int32)
        for b, p in enumerate(prompts):
            padded[b, :len(p)] = p
        check(lib.fa_decoder_prefill_padded(self._ops._ctx, self._h, padded.ctypes.data_as(capi.i32p), padded.shape[1],
                                            lens.ctypes.data_as(capi.u32p)))

    def verify(self, tokens, want_logits=False):
        """Speculative verification: feeds tokens [batch, l_new] like ``prefill`` and returns the greedy token
        after every one of them, int32 [batch, l_new] (and the logits [batch, l_new, vocab] if asked)."""
        p = np.ascontiguousarray(tokens, dtype=np.int32)
        if p.ndim != 2 or p.shape[0] != self.batch:
            raise ValueError("tokens must be [batch, l_new]")
        picked = np.empty(p.shape, dtype=np.int32)
        logits = np.empty(p.shape + (self.cfg.vocab,), dtype=np.float32) if want_logits else None
        check(lib.fa_decoder_verify(self._ops._ctx, self._h, p.ctypes.data_as(capi.i32p), p.shape[1],
                                    picked.ctypes.data_as(capi.i32p),
                                    logits.ctypes.data_as(capi.f32p) if want_logits else None))
        return (picked, logits) if want_logits else picked

    def rewind(self, seq_lens):
        """Shortens the installed sequences (no row may grow); the pages are kept."""
        s = np.ascontiguousarray(seq_lens, dtype=np.uint32)
        if s.size != self.batch:
            raise ValueError("one length per installed sequence")
        check(lib.fa_decoder_rewind(self._ops._ctx, self._h, s.ctypes.data_as(capi.u32p)))

    def step(self, use_graph=True):
        check(lib.fa_decoder_step(self._ops._ctx, self._h, 1 if use_graph else 0))

    def tokens(self):
        out = np.empty(self.batch, dtype=np.int32)
        check(lib.fa_decoder_read_tokens(self._ops._ctx, self._h, out.ctypes.data_as(capi.i32p)))
        return out

    def logits(self):
        out = np.empty((self.batch, self.cfg.vocab), dtype=np.float32)
        check(lib.fa_decoder_read_logits(self._ops._ctx, self._h, out.ctypes.data_as(capi.f32p)))
        return out

    def logits_buffer(self):
        """Raw handle of the resident logits [max_batch, vocab] (owned by the decoder)."""
        h = capi.buf_p()
        check(lib.fa_decoder_logits_buffer(self._h, C.byref(h)))
        return h

    def seq_lens(self):
        out = np.empty(self.batch, dtype=np.uint32)
        check(lib.fa_decoder_read_seq_lens(self._ops._ctx, self._h, out.ctypes.data_as(capi.u32p)))
        return out
