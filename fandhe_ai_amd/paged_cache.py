"""Caller side of the paged operators: ``BlockTable`` (page table and free-block bookkeeping, host
logic) and ``PagedKvCache`` (one layer's device-resident paged KV cache), with the names and the
error behaviour of the reference (crates/autodiff/src/nn/paged_kv.rs:147-363,
crates/autodiff/src/nn/paged_kv_device.rs:67-372) over the C ABI of ``libfandhe_rocm.so``.
"""
import ctypes as C

import numpy as np

from . import capi
from .backend import DeviceBuffer, InvalidArgument, check

U32MAX = 0xFFFFFFFF


class BlockTable:
    """Free blocks are the stack of returned ids (last in, first out) followed by the never-used
    ids in ascending order; a failed call leaves the table unchanged."""

    def __init__(self, _handle=None):
        if _handle is None:
            _handle = C.c_void_p()
            check(capi.lib.fa_block_table_create(C.byref(_handle)))
        self._h = _handle

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            capi.lib.fa_block_table_destroy(h)

    def clone(self):
        h = C.c_void_p()
        check(capi.lib.fa_block_table_clone(self._h, C.byref(h)))
        return BlockTable(h)

    def _state(self, max_blocks=0):
        st = capi.BlockTableState()
        check(capi.lib.fa_block_table_state_get(self._h, max_blocks, C.byref(st)))
        return st

    def free_blocks(self, max_blocks):
        return int(self._state(max_blocks).free_blocks)

    def alloc(self, max_blocks):
        """The next free block id, or None (crates/autodiff/src/nn/paged_kv.rs:172-183)."""
        bid, got = C.c_uint32(), C.c_int32()
        check(capi.lib.fa_block_table_alloc(self._h, max_blocks, C.byref(bid), C.byref(got)))
        return int(bid.value) if got.value else None

    def push_returned(self, block_id):
        check(capi.lib.fa_block_table_return(self._h, block_id))

    def reset(self):
        check(capi.lib.fa_block_table_reset(self._h))

    def seq_len(self):
        return int(self._state().seq_len)

    @property
    def batch(self):
        st = self._state()
        return int(st.batch) if st.has_batch else None

    def used_blocks(self):
        return int(self._state().used_blocks)

    def extend_for_append(self, max_blocks, block_size, b, l_new):
        # a request too large for any pool is left to the library's own checks (it fails before writing)
        cap = max(1, b * l_new) if b * l_new <= U32MAX else 1
        slots = np.empty(cap, dtype=np.uint32)
        n = C.c_uint64()
        check(capi.lib.fa_block_table_extend_for_append(self._h, max_blocks, block_size, b, l_new,
                                                        slots.ctypes.data_as(capi.u32p), cap, C.byref(n)))
        return slots[:n.value].copy()

    def flatten_tables(self, max_blocks_per_seq):
        st = self._state()
        rows = int(st.batch) if st.has_batch else 0
        cap = max(1, rows * max_blocks_per_seq)
        out = np.empty(cap, dtype=np.uint32)
        n = C.c_uint64()
        check(capi.lib.fa_block_table_flatten(self._h, max_blocks_per_seq, out.ctypes.data_as(capi.u32p), cap, C.byref(n)))
        return out[:n.value].copy()

    def rewind_to(self, new_len, block_size):
        check(capi.lib.fa_block_table_rewind_to(self._h, new_len, block_size))


class PagedKvCacheConfig:
    """Validated configuration (crates/autodiff/src/nn/paged_kv.rs:79-108)."""

    def __init__(self, block_size, max_blocks, embed_dim, dtype=capi.F32):
        check(capi.lib.fa_paged_cache_check_config(block_size, max_blocks, embed_dim, dtype))
        self.block_size, self.max_blocks, self.embed_dim, self.dtype = block_size, max_blocks, embed_dim, dtype

    @classmethod
    def new(cls, block_size, max_blocks, embed_dim, dtype=capi.F32):
        return cls(block_size, max_blocks, embed_dim, dtype)


class PagedKvCache:
    """One layer's K / V pools on the device with their page table.  ``append`` and ``attention`` are
    queued on the backend's stream; the download of the attention output is the only synchronization."""

    def __init__(self, ops, config):
        self._ops, self.config = ops, config
        self._h = C.c_void_p()
        check(capi.lib.fa_paged_cache_create(ops._ctx, config.block_size, config.max_blocks, config.embed_dim,
                                             config.dtype, C.byref(self._h)))

    @classmethod
    def new(cls, ops, config):
        return cls(ops, config)

    def close(self):
        h, self._h = getattr(self, "_h", None), None
        if h and self._ops._ctx:
            capi.lib.fa_paged_cache_destroy(self._ops._ctx, h)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _state(self):
        st, poisoned = capi.BlockTableState(), C.c_int32()
        check(capi.lib.fa_paged_cache_state_get(self._h, C.byref(st), C.byref(poisoned)))
        return st, bool(poisoned.value)

    def device(self):
        return self._ops.device()

    def seq_len(self):
        return int(self._state()[0].seq_len)

    def batch(self):
        st = self._state()[0]
        return int(st.batch) if st.has_batch else None

    def num_used_blocks(self):
        return int(self._state()[0].used_blocks)

    def num_free_blocks(self):
        return int(self._state()[0].free_blocks)

    def is_poisoned(self):
        return self._state()[1]

    def block_tables(self, max_blocks_per_seq):
        b = self.batch() or 0
        cap = max(1, b * max_blocks_per_seq)
        out = np.empty(cap, dtype=np.uint32)
        n = C.c_uint64()
        check(capi.lib.fa_paged_cache_block_tables(self._h, max_blocks_per_seq, out.ctypes.data_as(capi.u32p), cap,
                                                   C.byref(n)))
        return out[:n.value].reshape(b, max_blocks_per_seq).copy() if b else out[:0]

    def pools(self):
        """Host copies of the K and V pools [max_blocks, block_size, embed_dim] (synchronizes)."""
        k, v = capi.buf_p(), capi.buf_p()
        check(capi.lib.fa_paged_cache_pools(self._h, C.byref(k), C.byref(v)))
        shape = (self.config.max_blocks, self.config.block_size, self.config.embed_dim)
        views = [DeviceBuffer(self._ops, h, shape, self.config.dtype) for h in (k, v)]
        out = [self._ops.download(b).reshape(shape) for b in views]
        for b in views:
            b._h = None                                   # borrowed handles: the cache owns the pools
        return out

    def append(self, k_new, v_new):
        """k_new / v_new: host arrays or device buffers [B, L_new, E]."""
        kd = k_new if isinstance(k_new, DeviceBuffer) else self._ops.upload(np.ascontiguousarray(k_new), self.config.dtype)
        vd = v_new if isinstance(v_new, DeviceBuffer) else self._ops.upload(np.ascontiguousarray(v_new), self.config.dtype)
        if len(kd.shape) != 3:
            raise InvalidArgument("k_new must have rank 3")
        if tuple(vd.shape) != tuple(kd.shape):
            raise InvalidArgument("k_new and v_new differ in shape")
        b, l_new, e = kd.shape
        if e != self.config.embed_dim:
            raise InvalidArgument("last axis does not match embed_dim")
        check(capi.lib.fa_paged_cache_append(self._ops._ctx, self._h, kd._h, vd._h, b, l_new))

    def attention(self, q, num_heads, scale, num_kv_heads=0, out_dtype=None):
        """Attention over the cache for the last L_new positions (append first).  q: host array
        [B, L_new, num_heads * head_dim]; returns the host array of the same shape (in the cache's
        element type unless out_dtype names another)."""
        q = np.ascontiguousarray(q)
        if q.ndim != 3:
            raise InvalidArgument("q must have rank 3")
        b, l_new, e_q = q.shape
        if not num_kv_heads and e_q != self.config.embed_dim:
            raise InvalidArgument("last axis of q does not match embed_dim")
        if q.size == 0:
            check(capi.lib.fa_paged_cache_attention(self._ops._ctx, self._h, None, b, l_new, num_heads, num_kv_heads,
                                                    scale, None))
            return np.empty((b, l_new, e_q), dtype=q.dtype)
        out = self._ops.alloc_uninit((b, l_new, e_q), self.config.dtype if out_dtype is None else out_dtype)
        qd = self._ops.upload(q, self.config.dtype)
        check(capi.lib.fa_paged_cache_attention(self._ops._ctx, self._h, qd._h, b, l_new, num_heads, num_kv_heads,
                                                scale, out._h))
        return self._ops.download(out).reshape(b, l_new, e_q)

    def rewind_to(self, new_len):
        check(capi.lib.fa_paged_cache_rewind_to(self._h, new_len))

    def clear(self):
        check(capi.lib.fa_paged_cache_clear(self._h))

    def snapshot_table(self):
        h = C.c_void_p()
        check(capi.lib.fa_paged_cache_snapshot_table(self._h, C.byref(h)))
        return BlockTable(h)

    def restore_table(self, saved):
        check(capi.lib.fa_paged_cache_restore_table(self._h, saved._h))
