"""GPU parity: memory ops, pool, f32 GEMM / linear (reference summation order),
RMSNorm, RoPE and the small elementwise operators, all through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as o
from gpu_common import assert_parity, ops

pytestmark = pytest.mark.gpu


def test_device_is_gfx950_and_provider_surface():
    import fandhe_ai_amd as fa
    prov = fa.RocmDeviceProvider()
    assert prov.backend_name() == "rocm" and prov.is_available()
    assert prov.enumerate()[0] == fa.Device.Rocm(0)
    info = ops().info()
    assert info.arch.decode().startswith("gfx950") and info.wavefront_size == 64
    print("DEVICE", info.name.decode(), info.arch.decode(), "CUs", info.compute_units, "clock_khz", info.clock_khz)
    with pytest.raises(fa.DeviceUnavailable):
        fa.RocmBackendOps(99)


def test_memory_ops_round_trip_views_and_pool():
    import fandhe_ai_amd as fa
    be = ops()
    x = np.arange(1000, dtype=np.float32).reshape(10, 100)
    b = be.upload(x)
    assert np.array_equal(be.download(b), x) and not be.is_poisoned()
    z = be.alloc_zeroed((7, 5))
    assert not be.download(z).any()
    be.upload_into(np.array([1, 2, 3], np.float32), z, 4)
    got = be.download(z).ravel()
    assert got[4:7].tolist() == [1, 2, 3] and got[:4].sum() == 0 and got[7:].sum() == 0
    with pytest.raises(fa.InvalidArgument):
        be.upload_into(np.zeros(3, np.float32), z, 33)
    with pytest.raises(fa.InvalidArgument):
        fa.DeviceBufferView(z, 30, (2, 3))
    seen = []
    be.with_host_view(b, lambda s: seen.append(float(s.sum())))
    assert seen == [float(x.sum())]
    # the view is read-only and dies with the call; an exception of the closure comes back to the caller
    with pytest.raises(ValueError):
        be.with_host_view(b, lambda s: s.__setitem__(0, 1.0))
    with pytest.raises(KeyError):
        be.with_host_view(b, lambda s: {}["x"])
    # download_owned consumes the handle (crates/tensor-core/src/buffer.rs:414-430)
    c = be.upload(x)
    assert np.array_equal(be.download_owned(c), x) and c._h is None
    c.free()                                # a second release of a consumed buffer is a no-op
    # numel == 0 never touches the device (crates/tensor-core/src/buffer.rs:50-59)
    e = be.alloc_zeroed((0, 4))
    assert be.download(e).size == 0
    be.with_host_view(e, lambda s: seen.append(s.size))
    assert seen[-1] == 0
    # pool: a freed block is reused for the same size class, stats follow pool_core.rs:122-139
    s0 = be.device_memory_pool_stats()
    t = be.alloc_zeroed((1000,))            # 4000 B -> class 4096
    t.free()
    s1 = be.device_memory_pool_stats()
    t2 = be.alloc_zeroed((1010,))           # 4040 B -> the same class
    s2 = be.device_memory_pool_stats()
    assert s2.reuse_count == s1.reuse_count + 1
    assert s2.capacity_waste_bytes - s1.capacity_waste_bytes == 4096 - 4040
    t2.free()
    be.release_cached_device_memory()
    s3 = be.device_memory_pool_stats()
    assert s3.cached_bytes == 0 and s3.released_bytes > s0.released_bytes
    cls = C.c_uint64()
    for n in (0, 1, 255, 256, 1793, 200704, (1 << 20) + 1, (64 << 20) - 1, (64 << 20) + 7):
        assert fa.capi.lib.fa_size_class_for(n, C.byref(cls)) == 0 and cls.value == o.lib.orc_size_class_for(n)
    # a buffer of another context is a foreign handle
    other = fa.RocmBackendOps(0)
    try:
        fb = other.upload(np.zeros(4, np.float32))
        with pytest.raises(fa.DeviceMismatch):
            be.download(fb)
        fb.free()
    finally:
        other.close()


# crates/backend-rocm/tests/gemm_real_device.rs:16-38
GEMM_SHAPES = [(1, 1, 1), (1, 1, 0), (64, 64, 16), (63, 65, 17), (130, 70, 33), (5, 129, 200), (128, 128, 64),
               (257, 255, 513), (128, 128, 32), (65, 64, 16), (64, 63, 16), (64, 64, 15), (64, 64, 17), (1, 257, 33),
               (257, 1, 33), (193, 129, 48), (64, 64, 4096), (33, 17, 4097), (128, 96, 8192), (0, 5, 3), (5, 0, 3)]


def _data(n, seed):
    out = np.empty(n, dtype=np.float32)
    o.lib.orc_test_data_f32(o.ptr(out, o.f32p), n, seed)
    return out


def _gemm_form(fa, m, n, k):
    form = C.c_int32()
    fa.check(fa.capi.lib.fa_gemm_f32_form_query(m, n, k, C.byref(form)))
    return form.value


# shapes that take the matrix-core kernel by themselves: whole 128 x 128 tiles, ragged edges with k % 4 != 0
# (scalar slab loads), one tile row only
GEMM_SHAPES_WIDE = [(512, 4096, 33), (515, 4099, 70), (640, 3968, 16), (1024, 2048, 5)]


def test_gemm_device_is_bit_identical_to_the_fma_reference():
    """Both kernels of the order-fixed GEMM (a chain of v_fma_f32 on the vector ALUs; a chain of one-product
    matrix instructions) against the oracle's k-ascending fused multiply-add loop, bit for bit, on every shape."""
    import fandhe_ai_amd as fa
    be = ops()
    o.set_threads(8)
    try:
        for i, (m, n, k) in enumerate(GEMM_SHAPES + GEMM_SHAPES_WIDE):
            a = _data(m * k, 1 + i).reshape(m, k)
            b = _data(k * n, 100 + i).reshape(k, n)
            want = o.gemm_f32(a, b)
            da, db = be.upload(a), be.upload(b)
            if (m, n, k) in GEMM_SHAPES_WIDE:
                assert _gemm_form(fa, m, n, k) == 2
            for form in (0, 1, 2):
                fa.check(fa.capi.lib.fa_set_tuning(13, form))
                if form and k and m and n:
                    assert _gemm_form(fa, m, n, k) == form
                got = be.download_owned(be.gemm_device(da, db))
                r = assert_parity("ROCM_PARITY", f"{m}x{n}x{k} form {form}", got, want)
                assert r.bit_mismatch == 0
            da.free(), db.free()
    finally:
        fa.check(fa.capi.lib.fa_set_tuning(13, 0))
        o.set_threads(1)


def test_gemm_device_keeps_the_chain_on_special_values():
    """Subnormal inputs and products, cancellation, overflow to infinity and NaNs: one rounding per step on
    both kernels, as in the oracle's loop."""
    import fandhe_ai_amd as fa
    be = ops()
    rng = np.random.default_rng(7)
    m, n, k = 130, 192, 96
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    a[:, 0:16] *= np.float32(2.0 ** -80)                     # products near 2^-150: subnormal partial sums
    b[0:16, :] *= np.float32(2.0 ** -70)
    a[:, 16:32] *= np.float32(2.0 ** 70)                     # overflow to +-inf in some chains
    b[16:32, :] *= np.float32(2.0 ** 60)
    b[40, 5] = np.float32(np.nan)
    a[7, 50] = np.float32(np.inf)
    b[60:70, :] = -b[50:60, :]                               # exact cancellation against a[:, 50:60] below
    a[:, 60:70] = a[:, 50:60]
    want = o.gemm_f32(a, b)
    da, db = be.upload(a), be.upload(b)
    try:
        for form in (1, 2):
            fa.check(fa.capi.lib.fa_set_tuning(13, form))
            got = be.download_owned(be.gemm_device(da, db))
            same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
            assert same.all(), (form, int((~same).sum()))
    finally:
        fa.check(fa.capi.lib.fa_set_tuning(13, 0))
    assert np.isinf(want).any() and np.isnan(want).any()


def test_linear_forward_device_views_bias_relu():
    import fandhe_ai_amd as fa
    be = ops()
    rng = o.Rng(5)
    m, k, n = 16, 200, 72
    a = rng.randn((m, k))
    flat = rng.randn((37 + k * n + 11 + n,), std=0.1)       # one flat parameter buffer, weight and bias are views
    w = flat[37:37 + k * n].reshape(k, n)
    bias = flat[37 + k * n + 11:37 + k * n + 11 + n]
    store = be.upload(flat)
    wv = fa.DeviceBufferView(store, 37, (k, n))
    bv = fa.DeviceBufferView(store, 37 + k * n + 11, (n,))
    da = be.upload(a)
    for act, code in (("none", 0), ("relu", 1)):
        got = be.download_owned(be.linear_forward_device(da, wv, bv, act))
        want = o.linear_f32(a, np.ascontiguousarray(w), np.ascontiguousarray(bias), code)
        assert assert_parity("LINEAR_F32", f"{m}x{n}x{k}:{act}", got, want).bit_mismatch == 0
    got = be.download_owned(be.linear_forward_device(da, wv, None, "none"))
    assert np.array_equal(got, o.gemm_f32(a, np.ascontiguousarray(w)))
    with pytest.raises(fa.Unsupported):
        be.linear_forward_device(da, wv, bv, "gelu")
    with pytest.raises(fa.ShapeMismatch):
        be.linear_forward_device(da, fa.DeviceBufferView(store, 0, (k + 1, n)), None)


def test_rmsnorm_reference_fixtures_and_sweep():
    import fandhe_ai_amd as fa
    be = ops()
    # crates/backend-cpu/src/rmsnorm.rs:433-441
    x = np.array([[1, 2, 3, 4]], dtype=np.float32)
    got = be.rmsnorm(x, None, 0.0)
    assert np.array_equal(got, o.rmsnorm_f32(x, None, 0.0)[1])
    # NaN poisons its row only (rmsnorm.rs:443-462)
    x = np.array([[1, float("nan"), 3], [1, 2, 3]], dtype=np.float32)
    got = be.rmsnorm(x, None, 1e-5)
    assert np.all(np.isnan(got[0])) and np.all(np.isfinite(got[1]))
    with pytest.raises(fa.InvalidArgument):
        be.rmsnorm(x, None, -1.0)
    with pytest.raises(fa.ShapeMismatch):
        be.rmsnorm(x, np.ones(2, np.float32), 1e-5)
    x = np.array([[1e30, -1e30, 1e30, 1e-30]], dtype=np.float32)
    assert np.all(np.isfinite(be.rmsnorm(x, None, 1e-5)))
    rng = o.Rng(6)
    for rows, hidden in ((3, 1), (3, 4), (2, 8), (3, 1023), (3, 1024), (2, 4097), (32, 4096), (2048, 4096)):
        x = rng.randn((rows, hidden))
        w = rng.randn((hidden,))
        o.set_threads(8)
        rc, want = o.rmsnorm_f32(x, w, 1e-5)
        o.set_threads(1)
        got = be.rmsnorm(x, w, 1e-5)
        r = assert_parity("RMSNORM", f"{rows}x{hidden}", got, want)
        assert r.max_rel_err < 1e-6
    assert be.rmsnorm(np.zeros((0, 8), np.float32), None, 1e-5).size == 0


def test_rope_and_elementwise_against_the_oracle():
    be = ops()
    rng = o.Rng(7)
    x = rng.randn((6, 5, 128))
    pos = np.array([0, 1, 7, 100, 4095, 8191], dtype=np.int32)
    got = be.download_owned(be.rope(be.upload(x), be.upload(pos), 500000.0))
    want = o.rope_f32(x, pos, 500000.0)
    assert_parity("ROPE", "6x5x128", got, want)
    assert np.array_equal(got[0], x[0])
    g, u = rng.randn((32, 14336)), rng.randn((32, 14336))
    got = be.download_owned(be.silu_mul(be.upload(g), be.upload(u)))
    assert_parity("SILU_MUL", "32x14336", got, o.silu_mul_f32(g, u))
    a, b = rng.randn((32, 4096)), rng.randn((32, 4096))
    assert np.array_equal(be.download_owned(be.add(be.upload(a), be.upload(b))), a + b)
    # greedy argmax: first maximum, NaN ignored, all-NaN -> 0
    logits = rng.randn((32, 32000))
    logits[3, 100] = logits[3, 20000] = 50.0
    logits[4, :] = np.nan
    logits[5, 7] = np.nan
    got = be.download_owned(be.argmax(be.upload(logits)))
    assert np.array_equal(got, o.argmax_rows(logits)) and got[3] == 100 and got[4] == 0
    small = np.array([[1.0, 3.0, 3.0, 2.0], [-1.0, -2.0, -0.5, -9.0]], np.float32)
    assert be.download_owned(be.argmax(be.upload(small))).tolist() == [1, 2]
    for shape in ((7, 4099), (3, 50257), (5, 8192), (2, 3)):             # many ties; odd widths take the scalar loads
        tied = np.round(rng.randn(shape) * 2).astype(np.float32)
        assert np.array_equal(be.download_owned(be.argmax(be.upload(tied))), o.argmax_rows(tied)), shape
    table = rng.randn((50, 96))
    idx = np.array([3, 49, 0, 3], dtype=np.int32)
    assert np.array_equal(be.download_owned(be.gather(be.upload(table), be.upload(idx))), table[idx])
    v = rng.randn((1000,))
    import fandhe_ai_amd as fa
    bf = be.download_owned(be.convert(be.upload(v), fa.capi.BF16))
    assert np.array_equal(bf, o.to_bf16(v))
    assert np.array_equal(be.download_owned(be.convert(be.upload(bf), fa.capi.F32)), o.from_bf16(bf))


def test_bf16_conversion_equals_round_to_nearest_even_on_every_upper_half():
    """The device's f32 -> bf16 conversion (pairs on the hardware converter, an odd tail on the integer form) against
    the oracle's round-to-nearest-even on every 16-bit upper half combined with a zero, a below-tie, a tie, an
    above-tie and an all-ones lower half: normal numbers, subnormals, signed zeros, infinities, and every NaN pattern
    (a NaN must stay a NaN with its quiet bit set, as the integer form leaves it)."""
    import fandhe_ai_amd as fa
    be = ops()
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    bits = np.concatenate([hi | lo for lo in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF)] + [hi[:1]]).astype(np.uint32)
    v = bits.view(np.float32)                      # an odd count: the last element takes the scalar path
    got = be.download_owned(be.convert(be.upload(v), fa.capi.BF16))
    want = o.to_bf16(v)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(bits[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:8]]


def test_sync_points_are_rejected_during_graph_capture_and_graph_replays():
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    a = be.upload(np.full(256, 2.0, np.float32))
    b = be.upload(np.full(256, 3.0, np.float32))
    out = be.alloc_zeroed((256,))
    fa.check(lib.fa_graph_capture_begin(be._ctx))
    try:
        with pytest.raises(fa.DeviceContextCaptureInProgress):
            be.download(a)
        with pytest.raises(fa.DeviceContextCaptureInProgress):
            be.synchronize_device()
        with pytest.raises(fa.DeviceContextCaptureInProgress):
            be.alloc_zeroed((4,))
        fa.check(lib.fa_add(be._ctx, a._h, b._h, 256, out._h))
        fa.check(lib.fa_add(be._ctx, out._h, b._h, 256, out._h))
    finally:
        g = C.c_void_p()
        fa.check(lib.fa_graph_capture_end(be._ctx, C.byref(g)))
    assert not be.download(out).any()              # capture records, it does not execute
    for rep in range(3):
        fa.check(lib.fa_graph_launch(be._ctx, g))
        assert np.all(be.download(out) == 8.0)
        be.upload_into(np.zeros(256, np.float32), out, 0)
    fa.check(lib.fa_graph_destroy(be._ctx, g))


def test_a_graph_belongs_to_the_context_that_recorded_it():
    """Another context may neither replay nor destroy a graph (its scratch blocks would land in the wrong pool), and a
    context is not destroyed while one of its graphs is alive."""
    import fandhe_ai_amd as fa
    lib = fa.capi.lib
    one, two = C.c_void_p(), C.c_void_p()
    fa.check(lib.fa_context_create(0, C.byref(one)))
    fa.check(lib.fa_context_create(0, C.byref(two)))
    a, out = C.c_void_p(), C.c_void_p()
    host = np.full(64, 2.0, np.float32)
    fa.check(lib.fa_upload(one, fa.capi.F32, host.ctypes.data, 64, C.byref(a)))
    fa.check(lib.fa_alloc_zeroed(one, fa.capi.F32, 64, C.byref(out)))
    fa.check(lib.fa_graph_capture_begin(one))
    fa.check(lib.fa_add(one, a, a, 64, out))
    g = C.c_void_p()
    fa.check(lib.fa_graph_capture_end(one, C.byref(g)))
    assert lib.fa_graph_launch(two, g) == fa.capi.DEVICE_MISMATCH
    assert lib.fa_graph_destroy(two, g) == fa.capi.DEVICE_MISMATCH
    assert lib.fa_context_destroy(one) == fa.capi.INVALID_ARGUMENT and b"still alive" in lib.fa_last_error_message()
    fa.check(lib.fa_graph_launch(one, g))
    got = np.empty(64, np.float32)
    fa.check(lib.fa_download(one, out, 0, got.ctypes.data, 64))
    assert np.all(got == 4.0)
    fa.check(lib.fa_graph_destroy(one, g))
    for b in (a, out):
        fa.check(lib.fa_buffer_free(one, b))
    fa.check(lib.fa_context_destroy(one))
    fa.check(lib.fa_context_destroy(two))


def _capture(fa, be, fn):
    lib = fa.capi.lib
    g = C.c_void_p()
    fa.check(lib.fa_graph_capture_begin(be._ctx))
    try:
        fn()
    finally:
        st = lib.fa_graph_capture_end(be._ctx, C.byref(g))
    fa.check(st)
    return g


def _owned(fa, g):
    n = C.c_uint64()
    ptrs = (C.c_void_p * 16)()
    fa.check(fa.capi.lib.fa_graph_owned_blocks(g, ptrs, 16, C.byref(n)))
    return [ptrs[i] for i in range(min(n.value, 16))]


def test_captured_quantized_linear_owns_its_scratch():
    """A graph recorded over fa_linear_w8a8 keeps the addresses of the call's scratch (row scales, activation
    codes).  Those blocks belong to the graph until it is destroyed: a buffer of the same size class allocated
    afterwards gets other memory, replays leave it untouched bit for bit and still produce the eager result,
    and the pool never lists a block a live graph uses."""
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    rng = o.Rng(31)
    m, k, n = 32, 512, 256
    x, w = rng.randn((m, k)), rng.randn((k, n), std=0.05)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want = o.linear_w8a8(x, wq, ws)
    qw = be.import_quantized_weight(wq, ws)
    dx = be.upload(x)
    out = be.alloc_zeroed((m, n))
    be.release_cached_device_memory()        # every scratch request of the capture misses the pool
    s0 = be.device_memory_pool_stats()
    g = _capture(fa, be, lambda: fa.check(lib.fa_linear_w8a8(be._ctx, dx._h, m, qw._h, None, 0, None, out._h)))
    try:
        owned = _owned(fa, g)
        assert len(owned) == 2                       # row scales (128 B -> class 256) and codes (16 KiB)
        s1 = be.device_memory_pool_stats()
        assert s1.cached_bytes == s0.cached_bytes == 0          # nothing went back to the pool
        assert s1.pending_return_bytes - s0.pending_return_bytes == 256 + 16384
        # bystanders of both classes: must not share memory with the graph
        by_small = [be.upload(np.full(32, 7.25 + i, np.float32)) for i in range(4)]
        by_big = [be.upload(np.full(4096, -3.5 - i, np.float32)) for i in range(2)]
        addrs = [lib.fa_buffer_device_ptr(b._h) for b in by_small + by_big]
        assert not set(addrs) & set(owned)
        for rep in range(3):
            fa.check(lib.fa_graph_launch(be._ctx, g))
            got = be.download(out)
            assert np.array_equal(got, want), rep
            for i, b in enumerate(by_small):
                assert np.all(be.download(b) == np.float32(7.25 + i))
            for i, b in enumerate(by_big):
                assert np.all(be.download(b) == np.float32(-3.5 - i))
            be.upload_into(np.zeros(m * n, np.float32), out, 0)
            # the pool being emptied between replays must not touch the graph's blocks either
            be.release_cached_device_memory()
        for b in by_small + by_big:
            b.free()
    finally:
        fa.check(lib.fa_graph_destroy(be._ctx, g))
    s2 = be.device_memory_pool_stats()
    assert s2.pending_return_bytes == s0.pending_return_bytes    # the blocks came back with the graph
    # a second capture with a warm pool: hits are owned by the graph too
    g = _capture(fa, be, lambda: fa.check(lib.fa_linear_w8a8(be._ctx, dx._h, m, qw._h, None, 0, None, out._h)))
    try:
        owned = _owned(fa, g)
        assert len(owned) == 2
        fresh = be.upload(np.ones(32, np.float32))
        assert lib.fa_buffer_device_ptr(fresh._h) not in owned
        fa.check(lib.fa_graph_launch(be._ctx, g))
        assert np.array_equal(be.download(out), want)
        fresh.free()
    finally:
        fa.check(lib.fa_graph_destroy(be._ctx, g))
    # buffers cannot be made while a capture is open, whatever the pool holds
    t = be.alloc_zeroed((64,))
    t.free()
    fa.check(lib.fa_graph_capture_begin(be._ctx))
    try:
        h = C.c_void_p()
        assert lib.fa_alloc_zeroed(be._ctx, fa.capi.F32, 64, C.byref(h)) == fa.capi.CAPTURE_IN_PROGRESS
        assert lib.fa_alloc_uninit(be._ctx, fa.capi.F32, 64, C.byref(h)) == fa.capi.CAPTURE_IN_PROGRESS
    finally:
        g = C.c_void_p()
        lib.fa_graph_capture_end(be._ctx, C.byref(g))
        lib.fa_graph_destroy(be._ctx, g)


def test_stream_read_probe_runs_with_both_load_kinds_and_checks_its_range():
    """The read-floor probe of the benchmark (non-temporal and ordinary loads) reads only what it is given and
    writes nothing; ranges past the buffer, misaligned offsets and bad launch shapes are argument errors."""
    import fandhe_ai_amd as fa
    be = ops()
    lib = fa.capi.lib
    n = 1 << 20
    host = np.random.default_rng(5).standard_normal(n).astype(np.float32)
    src = be.upload(host)
    sink = be.alloc_zeroed((1,), fa.capi.I32)
    try:
        for plain in (0, 1):
            fa.check(lib.fa_set_tuning(15, plain))
            for blocks, threads, off, nbytes in ((512, 512, 0, 4 * n), (256, 256, 4096, 4 * n - 4096), (7, 512, 16, 16 * 7 * 513),
                                                 (64, 256, 0, 16 * 63), (1, 256, 4 * n - 16, 16)):
                fa.check(lib.fa_probe_stream_read(be._ctx, src._h, off, nbytes, blocks, threads, sink._h))
        be.synchronize_device()
        assert int(be.download(sink)[0]) == 0 and np.array_equal(be.download(src), host)
        for blocks, threads, off, nbytes in ((512, 512, 0, 4 * n + 16), (512, 512, 8, 1024), (0, 512, 0, 1024), (512, 128, 0, 1024),
                                             (70000, 512, 0, 1024), (512, 512, 4 * n, 16)):
            assert lib.fa_probe_stream_read(be._ctx, src._h, off, nbytes, blocks, threads, sink._h) == fa.capi.INVALID_ARGUMENT
    finally:
        fa.check(lib.fa_set_tuning(15, 0))
        src.free()
        sink.free()
