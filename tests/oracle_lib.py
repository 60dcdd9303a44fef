"""ctypes binding of the CPU oracle (oracle/liboracle.so) for the tests.

The oracle is test infrastructure: it is the checker the HIP path is compared
with, never a fallback of the product.  The library is built by
``make -C oracle`` (``__graft_entry__.build()`` does it too); when the shared
object is missing it is built on first use because building the checker needs
no GPU.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_DIR = os.path.join(_ROOT, "oracle")
_SO = os.path.join(_DIR, "liboracle.so")


def _load():
    if not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _DIR, "-s"])
    return C.CDLL(_SO)


lib = _load()

u64p = C.POINTER(C.c_uint64)
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)
i32p = C.POINTER(C.c_int32)
u32p = C.POINTER(C.c_uint32)
u16p = C.POINTER(C.c_uint16)
u8p = C.POINTER(C.c_uint8)
i8p = C.POINTER(C.c_int8)


def ptr(a, t):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(t)


class CompareReport(C.Structure):
    _fields_ = [
        ("total", C.c_uint64), ("fail_count", C.c_uint64),
        ("max_abs_diff", C.c_double), ("mean_abs_diff", C.c_double),
        ("max_rel_err", C.c_double), ("mean_rel_err", C.c_double),
        ("p50_abs_diff", C.c_double), ("p99_abs_diff", C.c_double),
        ("p999_abs_diff", C.c_double), ("max_fail_abs_diff", C.c_double),
        ("bit_mismatch", C.c_uint64),
    ]

    def line(self, tag, shape):
        # same shape as the reference's real-device log line
        # (crates/backend-rocm/tests/gemm_real_device.rs:75-78)
        return ("%s\t%s\ttotal=%d\tfail=%d\tmax_abs=%e\tmax_rel=%e\tmean_abs=%e\tp99_abs=%e\tbit_mismatch=%d"
                % (tag, shape, self.total, self.fail_count, self.max_abs_diff, self.max_rel_err,
                   self.mean_abs_diff, self.p99_abs_diff, self.bit_mismatch))


class PagedLayout(C.Structure):
    _fields_ = [("num_blocks", C.c_uint64), ("block_size", C.c_uint64), ("embed_dim", C.c_uint64)]


class PagedArgs(C.Structure):
    _fields_ = [("layout", PagedLayout), ("batch", C.c_uint64), ("l_new", C.c_uint64),
                ("num_heads", C.c_uint64), ("max_blocks_per_seq", C.c_uint64),
                ("scale", C.c_float), ("num_kv_heads", C.c_uint64)]


class PagedPlan(C.Structure):
    _fields_ = [("out_numel", C.c_uint64), ("s_max", C.c_uint64), ("query_rows", C.c_uint64),
                ("workspace_elems", C.c_uint64)]


class DecoderConfig(C.Structure):
    _fields_ = [("n_layers", C.c_uint32), ("d_model", C.c_uint32), ("n_heads", C.c_uint32),
                ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("d_ffn", C.c_uint32),
                ("vocab", C.c_uint32), ("block_size", C.c_uint32),
                ("max_blocks_per_seq", C.c_uint32), ("num_blocks", C.c_uint32),
                ("rms_eps", C.c_float), ("rope_theta", C.c_double)]


class DecoderWeights(C.Structure):
    _fields_ = [("embed", f32p), ("w_attn_norm", C.POINTER(f32p)), ("w_ffn_norm", C.POINTER(f32p)),
                ("w_final_norm", f32p),
                ("wqkv", C.POINTER(i8p)), ("sqkv", C.POINTER(f32p)),
                ("wo", C.POINTER(i8p)), ("so", C.POINTER(f32p)),
                ("wgu", C.POINTER(i8p)), ("sgu", C.POINTER(f32p)),
                ("wdown", C.POINTER(i8p)), ("sdown", C.POINTER(f32p)),
                ("wlm", i8p), ("slm", f32p)]


lib.orc_set_threads.restype = C.c_int
lib.orc_rng_init.restype = C.c_uint64
lib.orc_rng_init.argtypes = [C.c_uint64]
lib.orc_rng_next_u64.restype = C.c_uint64
lib.orc_rng_next_u64.argtypes = [u64p]
lib.orc_rng_next_f32.restype = C.c_float
lib.orc_rng_next_f32.argtypes = [u64p]
lib.orc_rng_next_unit_f32.restype = C.c_float
lib.orc_rng_next_unit_f32.argtypes = [u64p]
lib.orc_rng_next_unit_f64.restype = C.c_double
lib.orc_rng_next_unit_f64.argtypes = [u64p]
lib.orc_randn_f32.argtypes = [u64p, f32p, C.c_size_t, C.c_float]
lib.orc_rand_unit_f32.argtypes = [u64p, f32p, C.c_size_t]
lib.orc_rand_pm1_f32.argtypes = [u64p, f32p, C.c_size_t]
lib.orc_randint.argtypes = [u64p, C.c_int32, C.c_int32, i32p, C.c_size_t]
lib.orc_permutation_u32.argtypes = [u64p, u32p, C.c_size_t]
lib.orc_test_data_f32.argtypes = [f32p, C.c_size_t, C.c_uint64]
lib.orc_composite_close_f32.argtypes = [C.c_float, C.c_float]
lib.orc_compare_f32.argtypes = [f32p, f32p, C.c_size_t, C.POINTER(CompareReport)]
lib.orc_f32_to_bf16.restype = C.c_uint16
lib.orc_f32_to_bf16.argtypes = [C.c_float]
lib.orc_bf16_to_f32.restype = C.c_float
lib.orc_bf16_to_f32.argtypes = [C.c_uint16]
lib.orc_f32_to_bf16_n.argtypes = [f32p, u16p, C.c_size_t]
lib.orc_bf16_to_f32_n.argtypes = [u16p, f32p, C.c_size_t]
lib.orc_e4m3_to_f32.restype = C.c_float
lib.orc_e4m3_to_f32.argtypes = [C.c_uint8]
lib.orc_f32_to_e4m3.restype = C.c_uint8
lib.orc_f32_to_e4m3.argtypes = [C.c_float]
lib.orc_f32_to_e4m3_n.argtypes = [f32p, u8p, C.c_size_t]
lib.orc_e4m3_to_f32_n.argtypes = [u8p, f32p, C.c_size_t]
lib.orc_gemm_f32.argtypes = [f32p, f32p, f32p, C.c_size_t, C.c_size_t, C.c_size_t]
lib.orc_linear_f32.argtypes = [f32p, f32p, f32p, f32p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int]
lib.orc_quantize_rows_i8.argtypes = [f32p, C.c_size_t, C.c_size_t, i8p, f32p]
lib.orc_quantize_cols_i8.argtypes = [f32p, C.c_size_t, C.c_size_t, i8p, f32p]
lib.orc_gemm_i8_i32.argtypes = [i8p, i8p, i32p, i32p, C.c_size_t, C.c_size_t, C.c_size_t]
lib.orc_dequant_i32.argtypes = [i32p, f32p, f32p, f32p, f32p, C.c_size_t, C.c_size_t]
lib.orc_linear_w8a8.argtypes = [f32p, i8p, f32p, f32p, i32p, f32p, C.c_size_t, C.c_size_t, C.c_size_t]
lib.orc_linear_w8a16.argtypes = [u16p, i8p, f32p, f32p, C.c_size_t, C.c_size_t, C.c_size_t]
lib.orc_quantize_tensor_e4m3.restype = C.c_float
lib.orc_quantize_tensor_e4m3.argtypes = [f32p, C.c_size_t, u8p]
lib.orc_gemm_e4m3.argtypes = [u8p, u8p, C.c_float, C.c_float, f32p, C.c_size_t, C.c_size_t, C.c_size_t]
lib.orc_quantize_rows_e4m3.argtypes = [f32p, C.c_size_t, C.c_size_t, u8p, f32p]
lib.orc_quantize_cols_e4m3.argtypes = [f32p, C.c_size_t, C.c_size_t, u8p, f32p]
lib.orc_linear_e4m3_rows.argtypes = [u8p, u8p, f32p, f32p, f32p, f32p, C.c_size_t, C.c_size_t, C.c_size_t]
lib.orc_rmsnorm_f32.argtypes = [f32p, f32p, C.c_size_t, C.c_float, C.c_size_t, C.c_size_t, C.c_size_t, f32p]
lib.orc_rope_f32.argtypes = [f32p, i32p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_double, f32p]
lib.orc_silu_f32.restype = C.c_float
lib.orc_silu_f32.argtypes = [C.c_float]
lib.orc_silu_mul_f32.argtypes = [f32p, f32p, f32p, C.c_size_t]
lib.orc_add_f32.argtypes = [f32p, f32p, f32p, C.c_size_t]
lib.orc_argmax_rows_f32.argtypes = [f32p, C.c_size_t, C.c_size_t, i32p]
lib.orc_paged_layout_check.argtypes = [C.POINTER(PagedLayout)]
lib.orc_paged_args_check.argtypes = [C.POINTER(PagedArgs)]
lib.orc_validate_paged_kv_append.restype = C.c_int64
lib.orc_validate_paged_kv_append.argtypes = [C.c_uint64] * 4 + [u32p, C.c_uint64, C.POINTER(PagedLayout)]
lib.orc_validate_paged_attention.argtypes = [C.c_uint64] * 3 + [u32p, C.c_uint64, u32p, C.c_uint64,
                                                               C.POINTER(PagedArgs), C.POINTER(PagedPlan)]
lib.orc_paged_kv_append.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, u32p, C.c_uint64,
                                    C.POINTER(PagedLayout), C.c_size_t]
lib.orc_paged_attention_f32.argtypes = [f32p, f32p, f32p, u32p, u32p, C.POINTER(PagedArgs), f32p]
lib.orc_paged_attention_bf16.argtypes = [u16p, u16p, u16p, u32p, u32p, C.POINTER(PagedArgs), f32p]
lib.orc_paged_attention_f64.argtypes = [f64p, f64p, f64p, u32p, u32p, C.POINTER(PagedArgs), f64p]
lib.orc_size_class_for.restype = C.c_uint64
lib.orc_size_class_for.argtypes = [C.c_uint64]
lib.orc_decode_step.argtypes = [C.POINTER(DecoderConfig), C.POINTER(DecoderWeights),
                                C.POINTER(u16p), C.POINTER(u16p), u32p, u32p, i32p, C.c_uint32,
                                i32p, f32p]


# ------------------------------------------------------------------ helpers
class Rng:
    """Xorshift64* stream of the reference (crates/tensor-core/src/rng.rs:62-105)."""

    def __init__(self, seed=0):
        self.state = C.c_uint64(lib.orc_rng_init(seed))

    def next_u64(self):
        return lib.orc_rng_next_u64(C.byref(self.state))

    def randn(self, shape, std=1.0):
        out = np.empty(shape, dtype=np.float32)
        lib.orc_randn_f32(C.byref(self.state), ptr(out, f32p), out.size, std)
        return out

    def rand_pm1(self, shape):
        out = np.empty(shape, dtype=np.float32)
        lib.orc_rand_pm1_f32(C.byref(self.state), ptr(out, f32p), out.size)
        return out

    def randint(self, low, high, n):
        out = np.empty(n, dtype=np.int32)
        assert lib.orc_randint(C.byref(self.state), low, high, ptr(out, i32p), n) == 0
        return out

    def permutation(self, n):
        out = np.empty(n, dtype=np.uint32)
        lib.orc_permutation_u32(C.byref(self.state), ptr(out, u32p), n)
        return out


def set_threads(n):
    return lib.orc_set_threads(n)


def compare(actual, reference):
    a = np.ascontiguousarray(actual, dtype=np.float32).ravel()
    b = np.ascontiguousarray(reference, dtype=np.float32).ravel()
    assert a.size == b.size
    r = CompareReport()
    lib.orc_compare_f32(ptr(a, f32p), ptr(b, f32p), a.size, C.byref(r))
    return r


def to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib.orc_f32_to_bf16_n(ptr(x, f32p), ptr(out, u16p), x.size)
    return out


def from_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib.orc_bf16_to_f32_n(ptr(x, u16p), ptr(out, f32p), x.size)
    return out


def to_e4m3(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib.orc_f32_to_e4m3_n(ptr(x, f32p), ptr(out, u8p), x.size)
    return out


def from_e4m3(x):
    x = np.ascontiguousarray(x, dtype=np.uint8)
    out = np.empty(x.shape, dtype=np.float32)
    lib.orc_e4m3_to_f32_n(ptr(x, u8p), ptr(out, f32p), x.size)
    return out


def gemm_f32(a, b):
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    c = np.empty((m, n), dtype=np.float32)
    lib.orc_gemm_f32(ptr(a, f32p), ptr(b, f32p), ptr(c, f32p), m, n, k)
    return c


def linear_f32(a, w, bias=None, act=0):
    m, k = a.shape
    n = w.shape[1]
    y = np.empty((m, n), dtype=np.float32)
    lib.orc_linear_f32(ptr(a, f32p), ptr(w, f32p), ptr(bias, f32p), ptr(y, f32p), m, n, k, act)
    return y


def quantize_rows_i8(x):
    rows, cols = x.shape
    q = np.empty((rows, cols), dtype=np.int8)
    s = np.empty(rows, dtype=np.float32)
    lib.orc_quantize_rows_i8(ptr(x, f32p), rows, cols, ptr(q, i8p), ptr(s, f32p))
    return q, s


def quantize_cols_i8(w):
    k, n = w.shape
    q = np.empty((k, n), dtype=np.int8)
    s = np.empty(n, dtype=np.float32)
    lib.orc_quantize_cols_i8(ptr(w, f32p), k, n, ptr(q, i8p), ptr(s, f32p))
    return q, s


def gemm_i8_i32(a, b, c_in=None):
    m, k = a.shape
    n = b.shape[1]
    acc = np.empty((m, n), dtype=np.int32)
    lib.orc_gemm_i8_i32(ptr(a, i8p), ptr(b, i8p), ptr(c_in, i32p), ptr(acc, i32p), m, n, k)
    return acc


def dequant_i32(acc, sx, sw, bias=None):
    m, n = acc.shape
    out = np.empty((m, n), dtype=np.float32)
    lib.orc_dequant_i32(ptr(acc, i32p), ptr(sx, f32p), ptr(sw, f32p), ptr(bias, f32p), ptr(out, f32p), m, n)
    return out


def linear_w8a8(x, wq, sw, bias=None):
    m, k = x.shape
    n = wq.shape[1]
    acc = np.empty((m, n), dtype=np.int32)
    out = np.empty((m, n), dtype=np.float32)
    lib.orc_linear_w8a8(ptr(x, f32p), ptr(wq, i8p), ptr(sw, f32p), ptr(bias, f32p), ptr(acc, i32p),
                        ptr(out, f32p), m, n, k)
    return acc, out


def linear_w8a16(a_bf16, wq, sw):
    m, k = a_bf16.shape
    n = wq.shape[1]
    out = np.empty((m, n), dtype=np.float32)
    lib.orc_linear_w8a16(ptr(a_bf16, u16p), ptr(wq, i8p), ptr(sw, f32p), ptr(out, f32p), m, n, k)
    return out


def quantize_tensor_e4m3(x):
    q = np.empty(x.shape, dtype=np.uint8)
    s = lib.orc_quantize_tensor_e4m3(ptr(x, f32p), x.size, ptr(q, u8p))
    return q, np.float32(s)


def quantize_rows_e4m3(x):
    rows, cols = x.shape
    q = np.empty((rows, cols), dtype=np.uint8)
    s = np.empty(rows, dtype=np.float32)
    lib.orc_quantize_rows_e4m3(ptr(x, f32p), rows, cols, ptr(q, u8p), ptr(s, f32p))
    return q, s


def quantize_cols_e4m3(w):
    k, n = w.shape
    q = np.empty((k, n), dtype=np.uint8)
    s = np.empty(n, dtype=np.float32)
    lib.orc_quantize_cols_e4m3(ptr(w, f32p), k, n, ptr(q, u8p), ptr(s, f32p))
    return q, s


def linear_e4m3_rows(a, b, sa, sb, bias=None):
    m, k = a.shape
    n = b.shape[1]
    out = np.empty((m, n), dtype=np.float32)
    lib.orc_linear_e4m3_rows(ptr(a, u8p), ptr(b, u8p), ptr(sa, f32p), ptr(sb, f32p), ptr(bias, f32p), ptr(out, f32p), m, n, k)
    return out


def gemm_e4m3(a, b, sa, sb):
    m, k = a.shape
    n = b.shape[1]
    out = np.empty((m, n), dtype=np.float32)
    lib.orc_gemm_e4m3(ptr(a, u8p), ptr(b, u8p), sa, sb, ptr(out, f32p), m, n, k)
    return out


def rmsnorm_f32(x, w, eps, rows=None, hidden=None):
    if rows is None:
        rows, hidden = x.shape
    out = np.zeros(x.size, dtype=np.float32)
    rc = lib.orc_rmsnorm_f32(ptr(x, f32p), ptr(w, f32p), 0 if w is None else w.size, eps, rows, hidden,
                             x.size, ptr(out, f32p))
    return rc, out.reshape(x.shape)


def rope_f32(x, positions, theta):
    rows, heads, dh = x.shape
    out = np.empty_like(x)
    pos = np.ascontiguousarray(positions, dtype=np.int32)
    lib.orc_rope_f32(ptr(x, f32p), ptr(pos, i32p), rows, heads, dh, theta, ptr(out, f32p))
    return out


def silu_mul_f32(gate, up):
    out = np.empty_like(gate)
    lib.orc_silu_mul_f32(ptr(gate, f32p), ptr(up, f32p), ptr(out, f32p), gate.size)
    return out


def argmax_rows(x):
    rows, cols = x.shape
    out = np.empty(rows, dtype=np.int32)
    lib.orc_argmax_rows_f32(ptr(x, f32p), rows, cols, ptr(out, i32p))
    return out


def paged_args(num_blocks, block_size, e_kv, batch, l_new, heads, max_blocks, scale, kv_heads=0):
    return PagedArgs(PagedLayout(num_blocks, block_size, e_kv), batch, l_new, heads, max_blocks,
                     scale, kv_heads)


def paged_attention_f32(q, k_pool, v_pool, tables, seq_lens, args):
    out = np.zeros(q.shape, dtype=np.float32)
    rc = lib.orc_paged_attention_f32(ptr(q, f32p), ptr(k_pool, f32p), ptr(v_pool, f32p),
                                     ptr(tables, u32p), ptr(seq_lens, u32p), C.byref(args), ptr(out, f32p))
    return rc, out


def paged_attention_bf16(q, k_pool, v_pool, tables, seq_lens, args):
    out = np.zeros(q.shape, dtype=np.float32)
    rc = lib.orc_paged_attention_bf16(ptr(q, u16p), ptr(k_pool, u16p), ptr(v_pool, u16p),
                                      ptr(tables, u32p), ptr(seq_lens, u32p), C.byref(args), ptr(out, f32p))
    return rc, out


def paged_attention_f64(q, k_pool, v_pool, tables, seq_lens, args):
    out = np.zeros(q.shape, dtype=np.float64)
    rc = lib.orc_paged_attention_f64(ptr(q, f64p), ptr(k_pool, f64p), ptr(v_pool, f64p),
                                     ptr(tables, u32p), ptr(seq_lens, u32p), C.byref(args), ptr(out, f64p))
    return rc, out


def paged_kv_append(k_new, v_new, k_pool, v_pool, slots, layout):
    slots = np.ascontiguousarray(slots, dtype=np.uint32)
    return lib.orc_paged_kv_append(k_new.ctypes.data, v_new.ctypes.data, k_pool.ctypes.data,
                                   v_pool.ctypes.data, ptr(slots, u32p), slots.size, C.byref(layout),
                                   k_new.dtype.itemsize)
