"""Host-side mirror of the reference's backend interface for ``Device::Rocm``.

Same names, argument meaning and error behaviour as the Rust traits the
reference's callers are written against:

* ``Device`` / ``RocmDeviceProvider``  - crates/tensor-core/src/device.rs:69-168,
  crates/backend-rocm/src/device.rs:30-114
* ``BackendError`` family              - crates/tensor-core/src/device.rs:225-371
* ``DeviceBuffer`` / ``DeviceBufferView`` / ``MemoryOps``
                                       - crates/tensor-core/src/buffer.rs:91-521
* ``PagedKvLayout`` / ``PagedAttentionArgs``
                                       - crates/tensor-core/src/paged_kv.rs:47-214
* ``RocmBackendOps``                   - the ``BackendOps`` methods of the decode path
                                         (crates/tensor-core/src/backend_ops.rs)

Everything is a thin call into the C ABI (include/fandhe_rocm.h); numpy arrays
stand in for the reference's host ``Tensor``.  There is no CPU fallback: a
missing library or device raises.
"""
import ctypes as C
import math

import numpy as np

from . import capi
from .capi import lib


# ------------------------------------------------------------------ errors
class BackendError(Exception):
    """crates/tensor-core/src/device.rs:225-371"""
    code = -1


class InvalidArgument(BackendError):
    code = capi.INVALID_ARGUMENT


class ShapeMismatch(BackendError):
    code = capi.SHAPE_MISMATCH


class DeviceMismatch(BackendError):
    code = capi.DEVICE_MISMATCH


class DeviceAllocationFailed(BackendError):
    code = capi.ALLOCATION_FAILED


class KernelLaunchFailed(BackendError):
    code = capi.KERNEL_LAUNCH_FAILED


class DeviceUnavailable(BackendError):
    code = capi.DEVICE_UNAVAILABLE


class TransferFailed(BackendError):
    code = capi.TRANSFER_FAILED


class Unsupported(BackendError):
    code = capi.UNSUPPORTED


class DeviceContextPoisoned(BackendError):
    code = capi.CONTEXT_POISONED


class DeviceContextCaptureInProgress(BackendError):
    code = capi.CAPTURE_IN_PROGRESS


class StorePoisoned(BackendError):
    code = capi.STORE_POISONED


_ERRORS = {e.code: e for e in (StorePoisoned, InvalidArgument, ShapeMismatch, DeviceMismatch, DeviceAllocationFailed,
                               KernelLaunchFailed, DeviceUnavailable, TransferFailed, Unsupported,
                               DeviceContextPoisoned, DeviceContextCaptureInProgress)}


def check(status):
    if status != capi.OK:
        raise _ERRORS.get(status, BackendError)(capi.last_error())


# ------------------------------------------------------------------ device
class Device:
    """``Device::Rocm(ordinal)`` (crates/tensor-core/src/device.rs:69-79)."""

    def __init__(self, kind, ordinal=0):
        self.kind, self.ordinal = kind, ordinal

    @staticmethod
    def Rocm(ordinal=0):
        return Device("rocm", ordinal)

    @staticmethod
    def Cuda(ordinal=0):
        """Another backend's device: this provider refuses it."""
        return Device("cuda", ordinal)

    def __eq__(self, other):
        return isinstance(other, Device) and (self.kind, self.ordinal) == (other.kind, other.ordinal)

    def __hash__(self):
        return hash((self.kind, self.ordinal))

    def __repr__(self):
        return "Device::Cpu" if self.kind == "cpu" else "Device::%s(%r)" % (self.kind.capitalize(), self.ordinal)


Device.Cpu = Device("cpu", 0)


class RocmDeviceProvider:
    """``DeviceProvider`` for backend "rocm" (crates/backend-rocm/src/device.rs:30-114); gfx950 only."""

    def backend_name(self):
        return "rocm"

    def is_available(self):
        return len(self.enumerate()) > 0

    def enumerate(self):
        n = C.c_int32(0)
        if lib.fa_device_count(C.byref(n)) != capi.OK:
            return []
        return [Device.Rocm(i) for i in range(n.value)]

    def select(self, device):
        # decided before HIP is touched (crates/backend-rocm/src/device.rs:52-63): another backend's device, or an
        # ordinal that is no device id at all
        if not isinstance(device, Device) or device.kind != "rocm":
            raise DeviceUnavailable("RocmDeviceProvider cannot select a non-ROCm device: %r" % (device,))
        n = device.ordinal
        if isinstance(n, bool) or not isinstance(n, int) or not 0 <= n < 2 ** 31:
            raise DeviceUnavailable("Device::Rocm ordinal %r is not a HIP device id" % (n,))
        return RocmBackendOps(n)


def tape_for(device):
    """Counterpart of ``fandhe_ai::tape_for(Device::Rocm(n))`` (crates/facade/src/lib.rs:3216): the
    backend object a tape would own."""
    return RocmDeviceProvider().select(device)


_NP = {capi.F32: np.float32, capi.BF16: np.uint16, capi.I8: np.int8, capi.E4M3: np.uint8,
       capi.I32: np.int32, capi.U32: np.uint32}


# ------------------------------------------------------------------ buffers
class DeviceBuffer:
    """Opaque device allocation with a shape (crates/tensor-core/src/buffer.rs:91-200); freed once."""

    def __init__(self, ops, handle, shape, dtype):
        self._ops, self._h, self.shape, self.dtype = ops, handle, tuple(int(s) for s in shape), dtype

    def numel(self):
        return int(np.prod(self.shape, dtype=np.uint64)) if self.shape else 1

    def device(self):
        return self._ops.device()

    def free(self):
        if self._h is not None and self._ops._ctx is not None:
            check(lib.fa_buffer_free(self._ops._ctx, self._h))
        self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class DeviceBufferView:
    """(buffer, element offset, shape) with the range checked at construction (buffer.rs:277-373)."""

    def __init__(self, buffer, offset, shape):
        numel = 1
        for d in shape:
            numel *= int(d)
        if offset < 0 or offset + numel > buffer.numel():
            raise InvalidArgument("DeviceBufferView::new: view range [%d, %d) exceeds backing buffer length (%d)"
                                  % (offset, offset + numel, buffer.numel()))
        self.buffer, self.offset, self.shape, self._numel = buffer, int(offset), tuple(shape), numel

    def numel(self):
        return self._numel


class QuantizedWeight:
    """int8 per-channel, e4m3 per-tensor or e4m3 per-channel weight in the kernels' tile order."""

    def __init__(self, ops, handle, k, n, kind):
        self._ops, self._h, self.k, self.n, self.kind = ops, handle, k, n, kind

    def export(self):
        codes = np.empty((self.k, self.n), dtype=np.int8 if self.kind == capi.QW_INT8_CHANNEL else np.uint8)
        scales = np.empty(1 if self.kind == capi.QW_E4M3_TENSOR else self.n, dtype=np.float32)
        check(lib.fa_qweight_export(self._ops._ctx, self._h, codes.ctypes.data,
                                    scales.ctypes.data_as(capi.f32p)))
        return codes, scales

    def free(self):
        if self._h is not None and self._ops._ctx is not None:
            check(lib.fa_qweight_free(self._ops._ctx, self._h))
        self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class PagedKvLayout:
    """crates/tensor-core/src/paged_kv.rs:47-131; ``new`` is the checked constructor."""

    def __init__(self, num_blocks, block_size, embed_dim):
        self.num_blocks, self.block_size, self.embed_dim = num_blocks, block_size, embed_dim

    @classmethod
    def new(cls, num_blocks, block_size, embed_dim):
        l = cls(num_blocks, block_size, embed_dim)
        check(lib.fa_validate_paged_kv_append(0, 0, l.pool_elems(), l.pool_elems(), None, 0, C.byref(l.c())))
        return l

    def pool_elems(self):
        return self.num_blocks * self.block_size * self.embed_dim

    def pool_rows(self):
        return self.num_blocks * self.block_size

    def c(self):
        return capi.PagedLayout(self.num_blocks & (2 ** 64 - 1), self.block_size, self.embed_dim & (2 ** 64 - 1))


class PagedAttentionArgs:
    """crates/tensor-core/src/paged_kv.rs:137-214 plus ``num_kv_heads`` (0 = the reference's MHA)."""

    def __init__(self, layout, batch, l_new, num_heads, max_blocks_per_seq, scale, num_kv_heads=0):
        self.layout, self.batch, self.l_new, self.num_heads = layout, batch, l_new, num_heads
        self.max_blocks_per_seq, self.scale, self.num_kv_heads = max_blocks_per_seq, scale, num_kv_heads

    def head_dim(self):
        hkv = self.num_kv_heads or self.num_heads
        return self.layout.embed_dim // hkv if hkv else 0

    def c(self):
        return capi.PagedArgs(self.layout.c(), self.batch, self.l_new, self.num_heads, self.max_blocks_per_seq,
                              self.scale, self.num_kv_heads)


class PoolStats:
    """crates/tensor-core/src/pool_core.rs:122-139"""

    def __init__(self, s):
        for f, _ in capi.PoolStats._fields_:
            setattr(self, f, int(getattr(s, f)))


# ----------------------------------------------------------------- the ops
class RocmBackendOps:
    """``BackendOps`` + ``MemoryOps`` of the decode path on one MI355X."""

    def __init__(self, ordinal=0):
        self._ctx = None
        ctx = capi.ctx_p()
        check(lib.fa_context_create(ordinal, C.byref(ctx)))
        self._ctx = ctx
        self._ordinal = ordinal

    # -- lifetime ----------------------------------------------------------
    def close(self):
        if self._ctx is not None:
            lib.fa_context_destroy(self._ctx)
            self._ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def device(self):
        return Device.Rocm(self._ordinal)

    def info(self):
        out = capi.DeviceInfo()
        check(lib.fa_context_info(self._ctx, C.byref(out)))
        return out

    def memory_ops(self):
        """``BackendOps::memory_ops`` - this backend implements ``MemoryOps`` itself."""
        return self

    # -- MemoryOps (buffer.rs:389-521) ---------------------------------------
    def _wrap(self, handle, shape, dtype):
        return DeviceBuffer(self, handle, shape, dtype)

    def alloc_zeroed(self, shape, dtype=capi.F32):
        h = capi.buf_p()
        check(lib.fa_alloc_zeroed(self._ctx, dtype, int(np.prod(shape, dtype=np.uint64)) if len(shape) else 1,
                                  C.byref(h)))
        return self._wrap(h, shape, dtype)

    def alloc_uninit(self, shape, dtype=capi.F32):
        h = capi.buf_p()
        check(lib.fa_alloc_uninit(self._ctx, dtype, int(np.prod(shape, dtype=np.uint64)) if len(shape) else 1,
                                  C.byref(h)))
        return self._wrap(h, shape, dtype)

    def upload(self, tensor, dtype=None):
        a = np.ascontiguousarray(tensor)
        if dtype is None:
            dtype = {np.dtype(np.float32): capi.F32, np.dtype(np.uint16): capi.BF16, np.dtype(np.int8): capi.I8,
                     np.dtype(np.uint8): capi.E4M3, np.dtype(np.int32): capi.I32,
                     np.dtype(np.uint32): capi.U32}[a.dtype]
        assert a.dtype == _NP[dtype]
        h = capi.buf_p()
        check(lib.fa_upload(self._ctx, dtype, a.ctypes.data, a.size, C.byref(h)))
        return self._wrap(h, a.shape, dtype)

    def download(self, buffer, offset=0, numel=None):
        n = buffer.numel() - offset if numel is None else numel
        out = np.empty(n, dtype=_NP[buffer.dtype])
        check(lib.fa_download(self._ctx, buffer._h, offset, out.ctypes.data, n))
        return out.reshape(buffer.shape) if (offset == 0 and numel is None) else out

    def download_owned(self, buffer):
        out = np.empty(buffer.numel(), dtype=_NP[buffer.dtype])
        h, buffer._h = buffer._h, None  # the library frees the handle whether or not the copy succeeds
        check(lib.fa_download_owned(self._ctx, h, out.ctypes.data, out.size))
        return out.reshape(buffer.shape)

    def upload_into(self, tensor, dst, dst_offset):
        a = np.ascontiguousarray(tensor, dtype=_NP[dst.dtype])
        check(lib.fa_upload_into(self._ctx, a.ctypes.data, a.size, dst._h, dst_offset))

    def with_host_view(self, buffer, f):
        dt = _NP[buffer.dtype]
        raised = []

        def thunk(_user, data, numel):
            try:
                if numel == 0:
                    f(np.empty(0, dtype=dt))
                else:
                    raw = (C.c_ubyte * (numel * np.dtype(dt).itemsize)).from_address(data)
                    view = np.frombuffer(raw, dtype=dt)
                    view.flags.writeable = False
                    f(view)
            except BaseException as e:  # an exception must not unwind through the C frame
                raised.append(e)

        cb = capi.HOST_VIEW_FN(thunk)
        check(lib.fa_with_host_view(self._ctx, buffer._h, C.cast(cb, C.c_void_p), None))
        if raised:
            raise raised[0]

    def is_poisoned(self):
        flag = C.c_int32()
        check(lib.fa_context_poisoned(self._ctx, C.byref(flag)))
        return bool(flag.value)

    def synchronize_device(self):
        check(lib.fa_synchronize_device(self._ctx))

    def release_cached_device_memory(self):
        check(lib.fa_release_cached_device_memory(self._ctx))

    def device_memory_pool_stats(self):
        s = capi.PoolStats()
        check(lib.fa_device_memory_pool_stats(self._ctx, C.byref(s)))
        return PoolStats(s)

    # -- f32 linears (backend_ops.rs:1998, 4296-4308) -------------------------
    def gemm_device(self, a, b):
        (m, k), (k2, n) = a.shape, b.shape
        if k != k2:
            raise ShapeMismatch("gemm_device: inner dimensions differ (%d vs %d)" % (k, k2))
        out = self.alloc_uninit((m, n))
        check(lib.fa_gemm_device(self._ctx, a._h, b._h, m, n, k, out._h))
        return out

    def linear_forward_device(self, a, w, bias=None, act="none"):
        """``y = act(a @ w + bias)``; ``w`` / ``bias`` are ``DeviceBufferView`` with ``w`` stored [k, n]."""
        m, k = a.shape
        if len(w.shape) != 2 or w.shape[0] != k:
            raise ShapeMismatch("linear_forward_device: w must be [k, n] with k = %d" % k)
        n = w.shape[1]
        if bias is not None and bias.numel() != n:
            raise ShapeMismatch("linear_forward_device: bias must hold n = %d elements" % n)
        acts = {"none": capi.ACT_NONE, "relu": capi.ACT_RELU}
        if act not in acts:
            raise Unsupported("linear_forward_device: activation %r" % (act,))
        out = self.alloc_uninit((m, n))
        check(lib.fa_linear_forward_device(self._ctx, a._h, m, k, w.buffer._h, w.offset, n,
                                           bias.buffer._h if bias is not None else None,
                                           bias.offset if bias is not None else 0, acts[act], out._h))
        return out

    # -- quantized linears (build-defined) --------------------------------------
    def quantize_weight(self, w_view, kind=capi.QW_INT8_CHANNEL):
        k, n = w_view.shape
        h = capi.qw_p()
        check(lib.fa_qweight_from_f32(self._ctx, w_view.buffer._h, w_view.offset, k, n, kind, C.byref(h)))
        return QuantizedWeight(self, h, k, n, kind)

    def import_quantized_weight(self, codes, scales, kind=capi.QW_INT8_CHANNEL):
        codes = np.ascontiguousarray(codes)
        scales = np.ascontiguousarray(scales, dtype=np.float32)
        k, n = codes.shape
        h = capi.qw_p()
        check(lib.fa_qweight_from_codes(self._ctx, codes.ctypes.data, scales.ctypes.data_as(capi.f32p), k, n, kind,
                                        C.byref(h)))
        return QuantizedWeight(self, h, k, n, kind)

    def quantize_rows_i8(self, x):
        m, k = x.shape
        xq, sx = self.alloc_uninit((m, k), capi.I8), self.alloc_uninit((m,), capi.F32)
        check(lib.fa_quantize_rows_i8(self._ctx, x._h, m, k, xq._h, sx._h))
        return xq, sx

    def linear_w8a8(self, x, qw, bias=None, out_dtype=capi.F32, want_acc=False):
        m = x.shape[0]
        out = self.alloc_uninit((m, qw.n), out_dtype)
        acc = self.alloc_uninit((m, qw.n), capi.I32) if want_acc else None
        check(lib.fa_linear_w8a8(self._ctx, x._h, m, qw._h, bias.buffer._h if bias is not None else None,
                                 bias.offset if bias is not None else 0, acc._h if acc is not None else None, out._h))
        return (out, acc) if want_acc else out

    def gemm_w8a8(self, aq, sx, qw, out_dtype=capi.BF16, want_acc=False):
        m = aq.shape[0]
        out = self.alloc_uninit((m, qw.n), out_dtype)
        acc = self.alloc_uninit((m, qw.n), capi.I32) if want_acc else None
        check(lib.fa_gemm_w8a8(self._ctx, aq._h, sx._h, m, qw._h, acc._h if acc is not None else None, out._h))
        return (out, acc) if want_acc else out

    def linear_w8a16(self, a, qw, out_dtype=capi.BF16):
        m = a.shape[0]
        out = self.alloc_uninit((m, qw.n), out_dtype)
        check(lib.fa_linear_w8a16(self._ctx, a._h, m, qw._h, out._h))
        return out

    def quantize_tensor_e4m3(self, x):
        xq, scale = self.alloc_uninit(x.shape, capi.E4M3), self.alloc_uninit((1,), capi.F32)
        check(lib.fa_quantize_tensor_e4m3(self._ctx, x._h, x.numel(), xq._h, scale._h))
        return xq, scale

    def gemm_e4m3(self, aq, a_scale, qw, out_dtype=capi.BF16):
        m = aq.shape[0]
        out = self.alloc_uninit((m, qw.n), out_dtype)
        check(lib.fa_gemm_e4m3(self._ctx, aq._h, a_scale._h, m, qw._h, out._h))
        return out

    def quantize_rows_e4m3(self, x):
        m, k = x.shape
        xq, sx = self.alloc_uninit((m, k), capi.E4M3), self.alloc_uninit((m,), capi.F32)
        check(lib.fa_quantize_rows_e4m3(self._ctx, x._h, m, k, xq._h, sx._h))
        return xq, sx

    def linear_e4m3(self, x, qw, bias=None, out_dtype=capi.F32):
        """Per-token x per-channel fp8 linear: x f32 / bf16 [m, k], qw of kind QW_E4M3_CHANNEL."""
        m = x.shape[0]
        out = self.alloc_uninit((m, qw.n), out_dtype)
        check(lib.fa_linear_e4m3(self._ctx, x._h, m, qw._h, bias.buffer._h if bias is not None else None,
                                 bias.offset if bias is not None else 0, out._h))
        return out

    def gemm_e4m3_rows(self, aq, sx, qw, bias=None, out_dtype=capi.F32):
        m = aq.shape[0]
        out = self.alloc_uninit((m, qw.n), out_dtype)
        check(lib.fa_gemm_e4m3_rows(self._ctx, aq._h, sx._h, m, qw._h, bias.buffer._h if bias is not None else None,
                                    bias.offset if bias is not None else 0, out._h))
        return out

    # -- norms / elementwise (backend_ops.rs:5113, 2276-2390, 3375) -------------
    def rmsnorm(self, x, weight, eps):
        """Host tensors in and out like ``BackendOps::rmsnorm``; x is [rows, hidden]."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, hidden = (x.shape if x.ndim == 2 else (int(np.prod(x.shape[:-1])), x.shape[-1]))
        dx = self.upload(x.reshape(rows, hidden))
        dw = self.upload(np.ascontiguousarray(weight, dtype=np.float32)) if weight is not None else None
        out = self.rmsnorm_device(dx, dw, eps)
        return self.download_owned(out).reshape(x.shape)

    def rmsnorm_device(self, x, weight, eps):
        rows, hidden = x.shape
        out = self.alloc_uninit((rows, hidden))
        check(lib.fa_rmsnorm(self._ctx, x._h, weight._h if weight is not None else None, eps, rows, hidden, out._h))
        return out

    def rope(self, x, positions, theta):
        rows, heads, dh = x.shape
        out = self.alloc_uninit(x.shape)
        check(lib.fa_rope(self._ctx, x._h, positions._h, rows, heads, dh, theta, out._h))
        return out

    def silu_mul(self, gate, up):
        out = self.alloc_uninit(gate.shape)
        check(lib.fa_silu_mul(self._ctx, gate._h, up._h, gate.numel(), out._h))
        return out

    def add(self, a, b):
        out = self.alloc_uninit(a.shape)
        check(lib.fa_add(self._ctx, a._h, b._h, a.numel(), out._h))
        return out

    def argmax(self, x):
        rows, cols = x.shape
        out = self.alloc_uninit((rows,), capi.I32)
        check(lib.fa_argmax_rows(self._ctx, x._h, rows, cols, out._h))
        return out

    def new_generator(self, seed=0):
        """Device-resident state of a ``Generator::new(seed)`` (crates/tensor-core/src/rng.rs:684-689)."""
        g = self.alloc_zeroed((2,), capi.U32)
        check(lib.fa_rng_seed(self._ctx, g._h, seed))
        return g

    def sample_rows(self, logits, strategy, temperature=1.0, top_k=0, generator=None):
        """Next tokens [rows] (device buffer) from logits [rows, vocab]; strategy: SAMPLE_GREEDY /
        SAMPLE_TEMPERATURE / SAMPLE_TOP_K (crates/autodiff/src/generate/mod.rs:376-424)."""
        rows, vocab = logits.shape
        out = self.alloc_uninit((rows,), capi.I32)
        check(lib.fa_sample_rows(self._ctx, logits._h, rows, vocab, strategy, temperature, top_k,
                                 generator._h if generator is not None else None, out._h))
        return out

    def sampling_weights(self, logits, rows, vocab, strategy, temperature, top_k, weights, status, logits_row=0, weights_row=0):
        """``sampling_weights_f32`` (crates/autodiff/src/generate/mod.rs:432-452) of `rows` rows of `logits` from row
        `logits_row` on, into rows `weights_row` .. of `weights`; `logits` may be a raw buffer handle."""
        check(lib.fa_sampling_weights(self._ctx, getattr(logits, "_h", logits), logits_row * vocab, rows, vocab, strategy,
                                      temperature, top_k, weights._h, weights_row * vocab, status._h))

    def speculative_accept(self, p_weights, q_weights, drafts, vocab, generator, result, p_row=0, q_row=0):
        """``verify_sampling`` (crates/autodiff/src/generate/speculative.rs:246-279) on the device; no drafts: one
        draw from row `p_row` of p_weights.  Returns (accepted drafts, next token, status) after a download."""
        d = np.ascontiguousarray(drafts, dtype=np.int32)
        check(lib.fa_speculative_accept(self._ctx, p_weights._h, p_row * vocab, q_weights._h if d.size else None, q_row * vocab,
                                        d.ctypes.data_as(capi.i32p) if d.size else None, d.size, vocab, generator._h, result._h))
        n_acc, token, status, _ = (int(v) for v in self.download(result))
        return n_acc, token, status

    def sample_rows_per_row(self, logits, table):
        """Next tokens [rows] where row r follows record r of `table`, a U32 device buffer of 6 * rows elements
        holding fa_row_sampling records (see ``row_sampling_table``); generator states advance in the table."""
        rows, vocab = logits.shape
        out = self.alloc_uninit((rows,), capi.I32)
        check(lib.fa_sample_rows_per_row(self._ctx, logits._h, rows, vocab, table._h, out._h))
        return out

    def row_sampling_table(self, records):
        """records: [(strategy, temperature, top_k, seed)] -> device table for ``sample_rows_per_row``."""
        arr = (capi.RowSampling * len(records))()
        for r, (strategy, temperature, top_k, seed) in zip(arr, records):
            st = capi.u64()
            check(lib.fa_rng_state_from_seed(seed, C.byref(st)))
            r.rng_state, r.temperature, r.top_k, r.strategy = st.value, temperature, top_k, strategy
        return self.upload(np.frombuffer(bytes(arr), dtype=np.uint32).copy(), capi.U32)

    def gather(self, table, idx):
        rows, cols = idx.shape[0], table.shape[1]
        out = self.alloc_uninit((rows, cols))
        check(lib.fa_gather_rows(self._ctx, table._h, table.shape[0], cols, idx._h, rows, out._h))
        return out

    def fill_normal(self, buf, seed, mean=0.0, std=1.0, offset=0, numel=None):
        """Synthetic N(mean, std) data generated on the device (benchmarks)."""
        check(lib.fa_fill_normal(self._ctx, buf._h, offset, buf.numel() - offset if numel is None else numel, seed,
                                 mean, std))

    def convert(self, src, dtype):
        out = self.alloc_uninit(src.shape, dtype)
        check(lib.fa_convert(self._ctx, src._h, src.numel(), out._h))
        return out

    # -- paged KV (backend_ops.rs:4694-4786) ---------------------------------------
    def paged_kv_append(self, k_new, v_new, k_pool, v_pool, slot_mapping, layout):
        slots = np.ascontiguousarray(slot_mapping, dtype=np.uint32)
        check(lib.fa_paged_kv_append(self._ctx, k_new._h, v_new._h, k_pool._h, v_pool._h,
                                     slots.ctypes.data_as(capi.u32p), slots.size, C.byref(layout.c())))

    def paged_attention_forward(self, q, k_pool, v_pool, block_tables, seq_lens, args, out_dtype=None):
        tables = np.ascontiguousarray(block_tables, dtype=np.uint32).ravel()
        lens = np.ascontiguousarray(seq_lens, dtype=np.uint32).ravel()
        hkv = args.num_kv_heads or args.num_heads
        e_q = args.num_heads * (args.layout.embed_dim // hkv) if hkv and args.layout.embed_dim % hkv == 0 else 0
        out = self.alloc_uninit((args.batch, args.l_new, e_q), q.dtype if out_dtype is None else out_dtype)
        check(lib.fa_paged_attention_forward(self._ctx, q._h, k_pool._h, v_pool._h, tables.ctypes.data_as(capi.u32p),
                                             tables.size, lens.ctypes.data_as(capi.u32p), lens.size,
                                             C.byref(args.c()), out._h))
        return out

    def paged_kv_append_device(self, k_new, v_new, k_pool, v_pool, slot_mapping, layout):
        check(lib.fa_paged_kv_append_device(self._ctx, k_new._h, v_new._h, k_pool._h, v_pool._h, slot_mapping._h,
                                            slot_mapping.numel(), C.byref(layout.c())))

    def paged_attention_forward_device(self, q, k_pool, v_pool, block_tables, seq_lens, args, out_dtype=None):
        e_q = args.num_heads * args.head_dim()
        out = self.alloc_uninit((args.batch, args.l_new, e_q), q.dtype if out_dtype is None else out_dtype)
        check(lib.fa_paged_attention_forward_device(self._ctx, q._h, k_pool._h, v_pool._h, block_tables._h,
                                                    seq_lens._h, C.byref(args.c()), out._h))
        return out


SAMPLE_GREEDY, SAMPLE_TEMPERATURE, SAMPLE_TOP_K = 0, 1, 2


def default_scale(head_dim):
    return float(np.float32(1.0) / np.sqrt(np.float32(head_dim)))
