"""GPU parity of the quantized linears against the CPU oracle, through the C ABI.

int8: quantizer codes, scales and int32 accumulators are bit-exact; the
dequantized f32 output is bit-exact too (same single multiply).  bf16 outputs
are checked as the one round-to-nearest-even of the kernel's own f32 result,
whose parity with the oracle is judged with the composite tolerance.  fp8:
codes bit-exact, products judged against the exactly-summed oracle with the
bound stated in the test.
"""
import numpy as np
import pytest

import oracle_lib as o
from gpu_common import assert_bf16_rounding_of, assert_parity, ops

pytestmark = pytest.mark.gpu


def _fa():
    import fandhe_ai_amd as fa
    return fa


def test_per_token_quantizer_is_bit_exact():
    be = ops()
    rng = o.Rng(11)
    hand = np.array([[127.0, -127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, 63.5], [0.0] * 10,
                     [-8.0, 4.0, 2.0, 1.0, 0.0, 8.0, -4.0, -2.0, -1.0, 0.03]], dtype=np.float32)
    for x in (hand, rng.randn((16, 4096)), rng.randn((5, 100), std=3.0), rng.randn((33, 11008))):
        xq, sx = be.quantize_rows_i8(be.upload(x))
        wq, ws = o.quantize_rows_i8(x)
        assert np.array_equal(be.download_owned(sx), ws)
        assert np.array_equal(be.download_owned(xq), wq)
    xb = o.to_bf16(rng.randn((8, 512)))
    xq, sx = be.quantize_rows_i8(be.upload(xb))
    wq, ws = o.quantize_rows_i8(o.from_bf16(xb))
    assert np.array_equal(be.download_owned(sx), ws) and np.array_equal(be.download_owned(xq), wq)


def test_weight_quantizer_and_tile_packing_round_trip():
    fa = _fa()
    be = ops()
    rng = o.Rng(12)
    for k, n in ((64, 16), (4096, 4096), (100, 37), (130, 70), (11008, 64)):
        w = rng.randn((k, n), std=0.02)
        store = be.upload(w)
        qw = be.quantize_weight(fa.DeviceBufferView(store, 0, (k, n)))
        codes, scales = qw.export()
        o.set_threads(8)
        wq, ws = o.quantize_cols_i8(w)
        o.set_threads(1)
        assert np.array_equal(scales, ws), (k, n)
        assert np.array_equal(codes, wq), (k, n)
        qw2 = be.import_quantized_weight(wq, ws)
        c2, s2 = qw2.export()
        assert np.array_equal(c2, wq) and np.array_equal(s2, ws)
    w = rng.randn((256, 48))
    qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (256, 48)), fa.capi.QW_E4M3_TENSOR)
    codes, scale = qw.export()
    wq, ws = o.quantize_tensor_e4m3(w)
    assert scale[0] == ws and np.array_equal(codes, wq)


def test_int8_matrix_core_known_answers_from_the_reference_probe():
    """docs/perf/logs/int8-mma-probe-2608/RULE.txt:6-10,25-28 on the gfx950 int8 matrix instruction."""
    fa = _fa()
    be = ops()

    def acc_of(a, b):
        m, k = a.shape
        n = b.shape[1]
        kp = (k + 63) // 64 * 64
        ap = np.zeros((m, kp), np.int8)
        ap[:, :k] = a
        bp = np.zeros((kp, n), np.int8)
        bp[:k] = b
        qw = be.import_quantized_weight(bp, np.ones(n, np.float32))
        out, acc = be.gemm_w8a8(be.upload(ap), be.upload(np.ones(m, np.float32)), qw, fa.capi.F32, want_acc=True)
        acc = be.download_owned(acc)
        assert np.array_equal(be.download_owned(out), acc.astype(np.float32))
        return acc

    assert np.all(acc_of(np.ones((16, 32), np.int8), np.ones((32, 8), np.int8)) == 32)
    a127 = np.full((16, 128), 127, np.int8)
    assert np.all(acc_of(a127, np.full((128, 8), 127, np.int8)) == 2064512)
    assert np.all(acc_of(a127, np.full((128, 8), -127, np.int8)) == -2064512)
    r, kk, cc = np.arange(16)[:, None], np.arange(32)[None, :], np.arange(8)[None, :]
    pa = ((r * 37 + kk * 91 + 11) % 251 - 125).astype(np.int64)
    pb = ((np.arange(32)[:, None] * 53 + cc * 29 + 7) % 247 - 123).astype(np.int64)
    pa[0, 0], pa[1, 1], pb[0, 0], pb[31, 7] = -128, 127, -128, 127
    pc = np.arange(16)[:, None] * 1000003 - cc * 7919 - 5000000
    got = acc_of(pa.astype(np.int8), pb.astype(np.int8)).astype(np.int64) + pc
    assert np.array_equal(got, pc + pa @ pb)
    # asymmetric random operands: a transposed or permuted operand layout cannot pass
    rng = np.random.default_rng(0)
    a = rng.integers(-128, 128, size=(37, 192), dtype=np.int8)
    b = rng.integers(-128, 128, size=(192, 50), dtype=np.int8)
    assert np.array_equal(acc_of(a, b).astype(np.int64), a.astype(np.int64) @ b.astype(np.int64))


def test_w8a8_linear_benchmark_configuration_is_bit_exact():
    """x f32 [16,4096] ~N(0,1), W f32 [4096,4096] ~N(0,0.02), seed 0: int32 accumulators bit-exact."""
    fa = _fa()
    be = ops()
    rng = o.Rng(0)
    x = rng.randn((16, 4096))
    w = rng.randn((4096, 4096), std=0.02)
    qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (4096, 4096)))
    out, acc = be.linear_w8a8(be.upload(x), qw, want_acc=True)
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want_out = o.linear_w8a8(x, wq, ws)
    o.set_threads(1)
    got_acc, got_out = be.download_owned(acc), be.download_owned(out)
    assert np.array_equal(got_acc, want_acc)
    r = assert_parity("W8A8_PARITY", "16x4096x4096", got_out, want_out)
    assert r.bit_mismatch == 0
    # the quantized linear tracks the f32 linear it replaces
    ref = x.astype(np.float64) @ w.astype(np.float64)
    assert np.abs(got_out - ref).max() < 0.03 * np.abs(ref).max()


@pytest.mark.parametrize("m", [1, 8, 16, 17, 32, 33, 48, 49, 64, 65, 100, 300])
def test_w8a8_linear_row_sweep_bias_and_output_types(m):
    fa = _fa()
    be = ops()
    rng = o.Rng(100 + m)
    k, n = (4096, 6144) if m <= 64 else (512, 200)
    x = rng.randn((m, k))
    w = rng.randn((k, n), std=0.02)
    bias = rng.randn((n,))
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want = o.linear_w8a8(x, wq, ws, bias)
    o.set_threads(1)
    qw = be.import_quantized_weight(wq, ws)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    out, acc = be.linear_w8a8(be.upload(x), qw, bias=dbias, want_acc=True)
    assert np.array_equal(be.download_owned(acc), want_acc)
    got = be.download_owned(out)
    assert assert_parity("W8A8_PARITY", f"{m}x{n}x{k}", got, want).bit_mismatch == 0
    out_bf = be.linear_w8a8(be.upload(x), qw, bias=dbias, out_dtype=fa.capi.BF16)
    assert_bf16_rounding_of("w8a8 bf16", be.download_owned(out_bf), got)
    # bf16 activations are promoted exactly before the quantizer
    xb = o.to_bf16(x)
    out2 = be.download_owned(be.linear_w8a8(be.upload(xb), qw))
    assert np.array_equal(out2, o.linear_w8a8(o.from_bf16(xb), wq, ws)[1])


@pytest.mark.parametrize("m,k,n", [(33, 4096, 512), (100, 14336, 1030), (300, 2048, 768), (64, 1024, 4096), (200, 8192, 127)])
def test_w8a8_split_k_gemm_is_bit_exact(m, k, n):
    """A few hundred rows against a narrow weight: the GEMM splits k across blocks and adds the int32
    partial sums afterwards; accumulators and outputs must not depend on it."""
    fa = _fa()
    be = ops()
    rng = o.Rng(m + n)
    x = rng.randn((m, k))
    w = rng.randn((k, n), std=0.02)
    bias = rng.randn((n,))
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want = o.linear_w8a8(x, wq, ws, bias)
    o.set_threads(1)
    qw = be.import_quantized_weight(wq, ws)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    out, acc = be.linear_w8a8(be.upload(x), qw, bias=dbias, want_acc=True)
    assert np.array_equal(be.download_owned(acc), want_acc)
    got = be.download_owned(out)
    assert np.array_equal(got, want)
    out_bf = be.linear_w8a8(be.upload(x), qw, bias=dbias, out_dtype=fa.capi.BF16)
    assert_bf16_rounding_of("w8a8 split-k bf16", be.download_owned(out_bf), got)
    # the pre-quantized entry point takes the same path
    xq, sx = o.quantize_rows_i8(x)
    got2 = be.download_owned(be.gemm_w8a8(be.upload(xq), be.upload(sx), qw, out_dtype=fa.capi.F32))
    assert np.array_equal(got2, o.linear_w8a8(x, wq, ws)[1])


@pytest.mark.parametrize("m,k,n", [(65, 4096, 4096), (128, 4096, 6144), (300, 4096, 4096), (512, 4096, 4096), (100, 14336, 4096),
                                   (200, 2048, 1000), (77, 8192, 528), (260, 1024, 16), (512, 4096, 8192)])
def test_w8a8_weight_stationary_kernel_for_a_few_hundred_rows(m, k, n):
    """More rows than the decode kernels hold against a narrow weight: the weights stay in registers and the rows pass
    by in groups of 64 (forced here for every shape, tuning key 21 = 2).  Raw sums and outputs bit-exact against the
    oracle, with a bias, f32 and bf16 outputs, ragged row and column counts, one and two column tiles per block, all
    three register depths; and equal to what the tiled GEMM path (key 21 = 1) returns."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    rng = o.Rng(3 * m + n)
    x = rng.randn((m, k))
    w = rng.randn((k, n), std=0.02)
    bias = rng.randn((n,))
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want = o.linear_w8a8(x, wq, ws, bias)
    o.set_threads(1)
    qw = be.import_quantized_weight(wq, ws)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    dx = be.upload(x)
    try:
        fa.check(lib.fa_set_tuning(21, 2))
        for rep in range(2):
            out, acc = be.linear_w8a8(dx, qw, bias=dbias, want_acc=True)
            assert np.array_equal(be.download_owned(acc), want_acc), rep
            got = be.download_owned(out)
            assert np.array_equal(got, want), rep
        out_bf = be.linear_w8a8(dx, qw, bias=dbias, out_dtype=fa.capi.BF16)
        assert_bf16_rounding_of("w8a8 weight-stationary bf16", be.download_owned(out_bf), got)
        fa.check(lib.fa_set_tuning(21, 1))
        assert np.array_equal(be.download_owned(be.linear_w8a8(dx, qw, bias=dbias)), got)
    finally:
        fa.check(lib.fa_set_tuning(21, 0))


@pytest.mark.parametrize("m,k,n", [(300, 14336, 4096), (65, 8192, 4096), (512, 14336, 1000), (129, 11008, 528), (97, 14336, 16)])
def test_w8a8_weight_stationary_kernel_with_k_split_over_an_xcd(m, k, n):
    """Deep, narrow weights under more rows than the decode kernels hold: groups of four blocks keep a quarter of k of
    four column tiles in registers, every row group's partial sums meet in a workspace and the last arriver of a
    group finishes all rows (forced for every shape, tuning key 21 = 3; partial tiles exchanged inside the XCD's L2,
    key 16 = 3, and with agent-scope accesses, key 16 = 2).  Raw sums and outputs bit-exact against the oracle with a
    bias, f32 and bf16 outputs, ragged rows and columns, both register depths, three calls in a row (the counters
    return to zero), and equal to the tiled GEMM path (key 21 = 1)."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    rng = o.Rng(5 * m + n)
    x = rng.randn((m, k))
    w = rng.randn((k, n), std=0.02)
    bias = rng.randn((n,))
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want = o.linear_w8a8(x, wq, ws, bias)
    o.set_threads(1)
    qw = be.import_quantized_weight(wq, ws)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    dx = be.upload(x)
    try:
        fa.check(lib.fa_set_tuning(21, 3))
        for scope in (3, 2):
            fa.check(lib.fa_set_tuning(16, scope))
            for rep in range(3):
                out, acc = be.linear_w8a8(dx, qw, bias=dbias, want_acc=True)
                assert np.array_equal(be.download_owned(acc), want_acc), (scope, rep)
                got = be.download_owned(out)
                assert np.array_equal(got, want), (scope, rep)
        fa.check(lib.fa_set_tuning(16, 0))
        out_bf = be.linear_w8a8(dx, qw, bias=dbias, out_dtype=fa.capi.BF16)
        assert_bf16_rounding_of("w8a8 weight-stationary split-k bf16", be.download_owned(out_bf), got)
        fa.check(lib.fa_set_tuning(21, 1))
        assert np.array_equal(be.download_owned(be.linear_w8a8(dx, qw, bias=dbias)), got)
    finally:
        fa.check(lib.fa_set_tuning(21, 0))
        fa.check(lib.fa_set_tuning(16, 0))


def test_w8a8_ragged_shapes():
    """Shapes off every tile size, with and without a bias, under one and two column tiles per block and four and
    eight wavefronts (wavefronts without a k-tile, fewer k-tiles than ring slots, a clamped last column tile): the
    epilogue's operands are fetched ahead of the stream by index, so every edge has to agree with the tail's."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    rng = o.Rng(13)
    try:
        for m, k, n in ((3, 100, 37), (16, 64, 16), (32, 130, 70), (7, 4097, 33), (1, 64, 1), (64, 1000, 250), (33, 14336, 24)):
            x = rng.randn((m, k))
            w = rng.randn((k, n), std=0.05)
            bias = rng.randn((n,))
            wq, ws = o.quantize_cols_i8(w)
            qw = be.import_quantized_weight(wq, ws)
            dx = be.upload(x)
            dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
            for with_bias in (False, True):
                want_acc, want = o.linear_w8a8(x, wq, ws, bias if with_bias else None)
                for ntw, waves in ((0, 0), (1, 4), (1, 8), (2, 4), (2, 8)):
                    fa.check(lib.fa_set_tuning(0, ntw))
                    fa.check(lib.fa_set_tuning(1, waves))
                    out, acc = be.linear_w8a8(dx, qw, bias=dbias if with_bias else None, want_acc=True)
                    assert np.array_equal(be.download_owned(acc), want_acc), (m, k, n, with_bias, ntw, waves)
                    assert np.array_equal(be.download_owned(out), want), (m, k, n, with_bias, ntw, waves)
    finally:
        fa.check(lib.fa_set_tuning(0, 0))
        fa.check(lib.fa_set_tuning(1, 0))


def test_w8a8_activation_stationary_kernel_is_bit_exact():
    """The decode-shape linear that keeps the activations in registers and walks several column-tile
    pairs per block (chosen by shape for wide weights; forced here so that few units per block, ragged
    widths and k-tile counts that do not fill every wavefront are covered too).  33 to 64 rows take the form with one
    weight register set refilled behind every multiply (three and four row tiles, two items per wavefront)."""
    fa = _fa()
    be = ops()
    rng = o.Rng(77)
    lib = fa.capi.lib
    fa.check(lib.fa_set_tuning(5, 2))
    try:
        for m, k, n in ((32, 4096, 28672), (16, 4096, 6144), (3, 100, 37), (32, 130, 70), (7, 4096, 33), (17, 1000, 16400),
                        (1, 64, 16), (33, 4096, 6144), (48, 1000, 16400), (49, 130, 70), (64, 4096, 32000), (40, 64, 16)):
            x = rng.randn((m, k))
            w = rng.randn((k, n), std=0.05)
            bias = rng.randn((n,))
            o.set_threads(8)
            wq, ws = o.quantize_cols_i8(w)
            want_acc, want = o.linear_w8a8(x, wq, ws, bias)
            o.set_threads(1)
            qw = be.import_quantized_weight(wq, ws)
            dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
            out, acc = be.linear_w8a8(be.upload(x), qw, bias=dbias, want_acc=True)
            assert np.array_equal(be.download_owned(acc), want_acc), (m, k, n)
            assert np.array_equal(be.download_owned(out), want), (m, k, n)
    finally:
        fa.check(lib.fa_set_tuning(5, 0))


# Llama-7B layer shapes of the decode sweep: K -> N
GEMV_SHAPES = [(4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096)]


@pytest.mark.parametrize("k,n", GEMV_SHAPES)
def test_w8a16_decode_sweep(k, n):
    fa = _fa()
    be = ops()
    rng = o.Rng(k + n)
    w = rng.randn((k, n), std=0.02)
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    qw = be.import_quantized_weight(wq, ws)
    for m in (1, 8, 32):
        a = o.to_bf16(rng.randn((m, k)))
        want = o.linear_w8a16(a, wq, ws)
        da = be.upload(a)
        got = be.download_owned(be.linear_w8a16(da, qw, fa.capi.F32))
        assert_parity("W8A16_PARITY", f"{m}x{n}x{k}", got, want)
        assert_bf16_rounding_of("w8a16 bf16", be.download_owned(be.linear_w8a16(da, qw, fa.capi.BF16)), got)
        # the activation-stationary kernel keeps the k-split and summation order of the eight-wavefront
        # block-per-tile kernel: forced for every shape it can run, it must meet the same tolerance
        fa.check(fa.capi.lib.fa_set_tuning(5, 2))
        try:
            alt = be.download_owned(be.linear_w8a16(da, qw, fa.capi.F32))
        finally:
            fa.check(fa.capi.lib.fa_set_tuning(5, 0))
        assert_parity("W8A16_PARITY", f"{m}x{n}x{k}:stationary", alt, want)
    o.set_threads(1)


def test_w8a16_rejects_shapes_outside_its_contract():
    fa = _fa()
    be = ops()
    wq = np.ones((100, 16), np.int8)
    qw = be.import_quantized_weight(wq, np.ones(16, np.float32))
    with pytest.raises(fa.Unsupported):
        be.linear_w8a16(be.upload(np.zeros((1, 100), np.uint16)), qw)
    qw = be.import_quantized_weight(np.ones((128, 16), np.int8), np.ones(16, np.float32))
    with pytest.raises(fa.Unsupported):
        be.linear_w8a16(be.upload(np.zeros((33, 128), np.uint16)), qw)
    with pytest.raises(fa.ShapeMismatch):
        be.linear_w8a16(be.upload(np.zeros((2, 64), np.uint16)), qw)


def test_w8a16_ragged_shapes_under_every_launch_shape():
    """Row counts off the tile size, column counts that leave a half-filled last tile or an odd number of
    tiles, k of one to 172 tiles (wavefronts without a k-tile of their own, fewer k-tiles than ring slots,
    the deep-k loop form), under one and two column tiles per block and four and eight wavefronts."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    o.set_threads(8)
    try:
        for m, k, n in ((3, 128, 40), (17, 192, 16), (32, 4096, 1000), (5, 11008, 48), (16, 64, 8), (1, 320, 33),
                        (9, 1024, 272), (32, 11008, 100)):
            rng = o.Rng(m * 7 + k + n)
            wq, ws = o.quantize_cols_i8(rng.randn((k, n), std=0.02))
            qw = be.import_quantized_weight(wq, ws)
            a = o.to_bf16(rng.randn((m, k)))
            want = o.linear_w8a16(a, wq, ws)
            da = be.upload(a)
            for ntw in (1, 2):
                for waves in (4, 8):
                    fa.check(lib.fa_set_tuning(0, ntw))
                    fa.check(lib.fa_set_tuning(1, waves))
                    got = be.download_owned(be.linear_w8a16(da, qw, fa.capi.F32))
                    assert got.shape == (m, n)
                    assert_parity("W8A16_PARITY", f"{m}x{n}x{k}:ntw{ntw}:w{waves}", got, want)
    finally:
        fa.check(lib.fa_set_tuning(0, 0))
        fa.check(lib.fa_set_tuning(1, 0))
        o.set_threads(1)


def _topology(fa, be):
    import ctypes as C
    local, count = C.c_int32(), C.c_int32()
    fa.check(fa.capi.lib.fa_topology_query(be._ctx, C.byref(local), C.byref(count)))
    return local.value, count.value


def test_split_k_decode_linears_match_the_oracle():
    """The form of the decode-shape linears in which groups of two or four blocks divide k and add their partial
    tiles through a workspace, forced for every shape it accepts: partial tiles meeting in memory (key 16 = 2) and,
    where the device deals workgroups b and b + 8 to one XCD, in that XCD's L2 (key 16 = 3).  W8A8 accumulators and
    outputs bit-exact, W8A16 within the tolerance; every call three times in a row (the arrival counters must be
    back at zero) and on shapes with ragged rows, a clamped last column tile, groups past the last tile, k ranges
    that do not divide evenly and wavefronts with one k-tile more than others."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    local, count = _topology(fa, be)
    print("xcd_local", local, "xcd_count", count, flush=True)
    assert count >= 1
    modes = (2, 3) if local else (2,)
    o.set_threads(8)
    try:
        for m, k, n in ((32, 4096, 4096), (32, 14336, 4096), (7, 2048, 33), (17, 4160, 1000), (32, 11008, 100), (1, 4096, 16),
                        (20, 2112, 4112), (16, 8192, 528), (64, 14336, 4096), (33, 4096, 1000), (50, 2112, 4112)):
            rng = o.Rng(m + k + n)
            x = rng.randn((m, k))
            w = rng.randn((k, n), std=0.05)
            bias = rng.randn((n,))
            wq, ws = o.quantize_cols_i8(w)
            qw = be.import_quantized_weight(wq, ws)
            dx = be.upload(x)
            dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
            want_acc, want = o.linear_w8a8(x, wq, ws, bias)
            a16 = o.to_bf16(rng.randn((m, k))) if k % 64 == 0 and m <= 32 else None      # bf16 activations: at most 32 rows
            want16 = o.linear_w8a16(a16, wq, ws) if a16 is not None else None
            da16 = be.upload(a16) if a16 is not None else None
            for mode in modes:
                for s in (2, 4):
                    if (k + 63) // 64 // s < 16:
                        continue
                    fa.check(lib.fa_set_tuning(16, mode))
                    fa.check(lib.fa_set_tuning(17, s))
                    for rep in range(3):
                        out, acc = be.linear_w8a8(dx, qw, bias=dbias, want_acc=True)
                        assert np.array_equal(be.download_owned(acc), want_acc), (m, k, n, mode, s, rep)
                        assert np.array_equal(be.download_owned(out), want), (m, k, n, mode, s, rep)
                    if a16 is not None and m > 4:
                        first = None
                        for rep in range(3):
                            got = be.download_owned(be.linear_w8a16(da16, qw, fa.capi.F32))
                            assert_parity("W8A16_PARITY", f"{m}x{n}x{k}:ksplit{s}:mode{mode}", got, want16)
                            if first is None:
                                first = got
                            assert np.array_equal(got, first), "split-k f32 sums depend on the arrival order"
                        assert_bf16_rounding_of("w8a16 split-k bf16", be.download_owned(be.linear_w8a16(da16, qw, fa.capi.BF16)), first)
    finally:
        fa.check(lib.fa_set_tuning(16, 0))
        fa.check(lib.fa_set_tuning(17, 0))
        o.set_threads(1)


def test_w8a16_one_hot_rows_pick_weight_rows_exactly():
    fa = _fa()
    be = ops()
    rng = np.random.default_rng(3)
    k, n = 256, 48
    wq = rng.integers(-127, 128, size=(k, n), dtype=np.int8)
    ws = np.ones(n, np.float32)
    qw = be.import_quantized_weight(wq, ws)
    a = np.zeros((16, k), np.float32)
    picks = [0, 1, 15, 16, 17, 63, 64, 65, 100, 127, 128, 200, 254, 255, 7, 8]
    for r, p in enumerate(picks):
        a[r, p] = 1.0
    got = be.download_owned(be.linear_w8a16(be.upload(o.to_bf16(a)), qw, fa.capi.F32))
    assert np.array_equal(got, wq[picks].astype(np.float32))


def test_int8_prefill_gemm_rows_sampled_at_full_size():
    """M=2048, K=4096, N=14336: accumulators of sampled rows bit-exact against the oracle."""
    fa = _fa()
    be = ops()
    m, k, n = 2048, 4096, 14336
    rng = np.random.default_rng(5)
    aq = rng.integers(-127, 128, size=(m, k), dtype=np.int8)
    wq = rng.integers(-127, 128, size=(k, n), dtype=np.int8)
    sx = rng.uniform(0.01, 0.05, size=m).astype(np.float32)
    sw = rng.uniform(1e-4, 1e-3, size=n).astype(np.float32)
    qw = be.import_quantized_weight(wq, sw)
    out, acc = be.gemm_w8a8(be.upload(aq), be.upload(sx), qw, fa.capi.F32, want_acc=True)
    got_acc, got = be.download_owned(acc), be.download_owned(out)
    rows = np.r_[0:16, 127:130, 1000:1016, 2040:2048]
    o.set_threads(8)
    want_acc = o.gemm_i8_i32(np.ascontiguousarray(aq[rows]), wq)
    o.set_threads(1)
    assert np.array_equal(got_acc[rows], want_acc)
    assert np.array_equal(got[rows], o.dequant_i32(want_acc, np.ascontiguousarray(sx[rows]), sw))
    # checksum over the whole output: column sums of the accumulators equal (sum_m a[m, :]) @ w
    colsum = aq.astype(np.int64).sum(axis=0)
    assert np.array_equal(got_acc.astype(np.int64).sum(axis=0), colsum @ wq.astype(np.int64))
    out_bf = be.download_owned(be.gemm_w8a8(be.upload(aq), be.upload(sx), qw, fa.capi.BF16))
    assert_bf16_rounding_of("gemm_w8a8 bf16", out_bf, got)


@pytest.mark.parametrize("m,k,n", [(4000, 256, 2048), (8192, 128, 4096), (4096, 384, 6144)], ids=["16x8", "32x16", "16x24"])
def test_int8_large_tile_kernel_tile_order_with_many_row_blocks(m, k, n):
    """Sixteen and thirty-two row blocks of 256 against a multiple of eight column blocks: every XCD walks its column
    blocks for eight row blocks at a time.  Sampled rows of every row block bit-exact against the oracle, and the
    column sums of all accumulators equal (sum of the rows of a) @ w: every tile was written once, by the right block."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    rng = np.random.default_rng(m + n)
    aq = rng.integers(-127, 128, size=(m, k), dtype=np.int8)
    wq = rng.integers(-127, 128, size=(k, n), dtype=np.int8)
    sx = rng.uniform(0.01, 0.05, size=m).astype(np.float32)
    sw = rng.uniform(1e-4, 1e-3, size=n).astype(np.float32)
    qw = be.import_quantized_weight(wq, sw)
    try:
        fa.check(lib.fa_set_tuning(7, 16))                # 256 x 256 tiles whatever the shape would pick
        assert _gemm_plan(fa, be, m, qw).big_ntb == 16
        out, acc = be.gemm_w8a8(be.upload(aq), be.upload(sx), qw, fa.capi.F32, want_acc=True)
    finally:
        fa.check(lib.fa_set_tuning(7, 0))
    got_acc, got = be.download_owned(acc), be.download_owned(out)
    rows = np.unique(np.r_[np.arange(0, m, 256), np.arange(255, m, 256), m - 1, 1000:1003])
    want_acc = o.gemm_i8_i32(np.ascontiguousarray(aq[rows]), wq)
    assert np.array_equal(got_acc[rows], want_acc)
    assert np.array_equal(got[rows], o.dequant_i32(want_acc, np.ascontiguousarray(sx[rows]), sw))
    colsum = aq.astype(np.int64).sum(axis=0)
    assert np.array_equal(got_acc.astype(np.int64).sum(axis=0), colsum @ wq.astype(np.int64))


def test_fp8_quantizer_bit_exact_and_gemm_within_stated_bound():
    """e4m3 per-tensor: codes and scale bit-exact.  GEMM: the oracle sums the exact products in f64 and
    rounds once.  The f8f6f4 matrix instruction aligns the 128 products of one issue to their largest
    exponent before adding, which keeps about 17 bits below the largest term; measured on MI355X the
    worst error is 2^-17.0 of sum_k |a||b| at K = 256 and shrinks with K (2^-20.0 at K = 8192).
    Stated fp8 bound (looser than the composite tolerance, as the benchmark contract allows):
        |gpu - exact| <= 2^-15 * sum_k |a_k||b_k| * (sa * sb)     for every output,
    and the composite tolerance (rel < 1e-3 or abs < 1e-5) must still hold for >= 98 % of the outputs
    (the rest are outputs with heavy cancellation, |exact| << sum |a||b|)."""
    fa = _fa()
    be = ops()
    rng = o.Rng(21)
    for m, k, n in ((64, 256, 48), (130, 1024, 200), (2048, 4096, 512)):
        a, w = rng.randn((m, k)), rng.randn((k, n))
        aq, a_scale = be.quantize_tensor_e4m3(be.upload(a))
        want_aq, want_sa = o.quantize_tensor_e4m3(a)
        assert be.download(a_scale)[0] == want_sa and np.array_equal(be.download(aq), want_aq)
        qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (k, n)), fa.capi.QW_E4M3_TENSOR)
        wq, sw = qw.export()
        want_wq, want_sw = o.quantize_tensor_e4m3(w)
        assert sw[0] == want_sw and np.array_equal(wq, want_wq)
        got = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.F32))
        o.set_threads(8)
        want = o.gemm_e4m3(want_aq, want_wq, want_sa, want_sw)
        o.set_threads(1)
        absprod = (np.abs(o.from_e4m3(want_aq)).astype(np.float64) @ np.abs(o.from_e4m3(want_wq)).astype(np.float64))
        bound = absprod * float(want_sa) * float(want_sw) * 2.0 ** -15 + 1e-30
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        print("FP8_PARITY\t%dx%dx%d\tmax_err/bound=%.3e" % (m, n, k, float((err / bound).max())), flush=True)
        assert np.all(err <= bound)
        r = o.compare(got, want)
        print(r.line("FP8_PARITY", f"{m}x{n}x{k}"), flush=True)
        assert r.fail_count <= 2e-2 * r.total
        out_bf = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.BF16))
        assert_bf16_rounding_of("gemm_e4m3 bf16", out_bf, got)
    # e4m3-representable operands with absmax 448 (scale exactly 1): every product is a multiple of 2^9
    # and every partial sum stays below 2^33, so f32 accumulation in any order is exact
    a = np.tile(np.array([[64, 128, -256, 448]], np.float32), (16, 32))
    w = np.tile(np.array([[224], [-112], [56], [448]], np.float32), (32, 16))
    aq, sa = be.quantize_tensor_e4m3(be.upload(a))
    qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (128, 16)), fa.capi.QW_E4M3_TENSOR)
    assert be.download(sa)[0] == 1.0 and np.array_equal(o.from_e4m3(be.download(aq)), a)
    got = be.download_owned(be.gemm_e4m3(aq, sa, qw, fa.capi.F32))
    assert np.array_equal(got, (a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32))


def _gemm_plan(fa, be, m, qw):
    plan = fa.capi.GemmPlan()
    fa.check(fa.capi.lib.fa_gemm_plan_query(be._ctx, m, qw._h, __import__("ctypes").byref(plan)))
    return plan


def _fp8_rows_check(tag, got_rows, aq_rows, wq, sa, sw):
    """Sampled output rows of an e4m3 GEMM against the oracle's exact-product f64 sum rounded once, under the
    stated fp8 bound |gpu - exact| <= 2^-15 * sum_k |a_k||b_k| * (sa * sw), with >= 98 % of the outputs
    inside the composite tolerance (rel < 1e-3 or abs < 1e-5)."""
    o.set_threads(8)
    want = o.gemm_e4m3(np.ascontiguousarray(aq_rows), wq, sa, sw)
    o.set_threads(1)
    a_abs = np.abs(o.from_e4m3(np.ascontiguousarray(aq_rows))).astype(np.float64)
    n = wq.shape[1]
    absprod = np.empty((aq_rows.shape[0], n), np.float64)
    for c0 in range(0, n, 2048):
        absprod[:, c0:c0 + 2048] = a_abs @ np.abs(o.from_e4m3(np.ascontiguousarray(wq[:, c0:c0 + 2048]))).astype(np.float64)
    bound = absprod * float(sa) * float(sw) * 2.0 ** -15 + 1e-30
    err = np.abs(got_rows.astype(np.float64) - want.astype(np.float64))
    print("FP8_PARITY\t%s\tmax_err/bound=%.3e" % (tag, float((err / bound).max())), flush=True)
    assert np.all(err <= bound), tag
    r = o.compare(got_rows, want)
    print(r.line("FP8_PARITY", tag), flush=True)
    assert r.fail_count <= 2e-2 * r.total, tag


def test_fp8_prefill_gemm_large_tile_kernel_rows_sampled_at_full_size():
    """M=2048, K=4096, N=14336, N(0,1) operands cast to e4m3 per tensor (absmax / 448): the shape of the
    benchmark's fp8 GEMM, which the launcher sends to gemm_mfma_big_kernel<true, 14 | 16, waves / 2, EpiF8>.
    Sampled rows are compared with the oracle for 14 and 16 column tiles per block, 4 / 8 / 16 wavefronts per
    block and f32 / bf16 outputs; the plan query confirms the large-tile kernel is what ran."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    m, k, n = 2048, 4096, 14336
    rng = np.random.default_rng(44)
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((k, n), dtype=np.float32)
    aq, a_scale = be.quantize_tensor_e4m3(be.upload(a))
    o.set_threads(8)
    want_aq, want_sa = o.quantize_tensor_e4m3(a)
    want_wq, want_sw = o.quantize_tensor_e4m3(w)
    o.set_threads(1)
    assert be.download(a_scale)[0] == want_sa and np.array_equal(be.download(aq), want_aq)
    qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (k, n)), fa.capi.QW_E4M3_TENSOR)
    wq, sw = qw.export()
    assert sw[0] == want_sw and np.array_equal(wq, want_wq)
    del a, w
    # rows from every quarter of a 256-row block tile (both wavefront rows of it), first / middle / last blocks
    rows = np.r_[0:4, 60:68, 124:132, 188:196, 252:260, 1020:1028, 1500:1504, 2044:2048]
    try:
        for ntb, waves in ((0, 0), (14, 0), (16, 0), (14, 4), (16, 16), (14, 16)):
            fa.check(lib.fa_set_tuning(7, ntb))
            fa.check(lib.fa_set_tuning(6, waves))
            plan = _gemm_plan(fa, be, m, qw)
            assert plan.big_ntb in (14, 16) and (ntb == 0 or plan.big_ntb == ntb), (ntb, plan.big_ntb)
            assert plan.waves == (waves or 8) and plan.splits == 1
            got = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.F32))
            _fp8_rows_check("2048x14336x4096 ntb=%d waves=%d" % (plan.big_ntb, plan.waves), got[rows], want_aq[rows],
                            want_wq, want_sa, want_sw)
            # every output finite and the untested rows sane: row sums against a row-sum identity
            assert np.all(np.isfinite(got))
            out_bf = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.BF16))
            assert_bf16_rounding_of("gemm_e4m3 large tile bf16", out_bf, got)
            if ntb == 0:
                base = got
            else:
                # the tile shape changes which wavefront owns an output, not the order of its k sum
                assert np.array_equal(got, base), (ntb, waves)
    finally:
        fa.check(lib.fa_set_tuning(7, 0))
        fa.check(lib.fa_set_tuning(6, 0))
    # whole-output checksum: sum over rows of the exact result is (sum_m a[m, :]) @ w; the f32 outputs
    # summed in f64 must agree within the per-element bound summed over the rows
    a_f = o.from_e4m3(want_aq).astype(np.float64)
    colsum = a_f.sum(axis=0)
    exact = np.empty(n, np.float64)
    abs_col = np.abs(a_f).sum(axis=0)
    slack = np.empty(n, np.float64)
    for c0 in range(0, n, 2048):
        wf = o.from_e4m3(np.ascontiguousarray(want_wq[:, c0:c0 + 2048])).astype(np.float64)
        exact[c0:c0 + 2048] = colsum @ wf
        slack[c0:c0 + 2048] = abs_col @ np.abs(wf)
    scale = float(want_sa) * float(want_sw)
    assert np.all(np.abs(base.astype(np.float64).sum(axis=0) - exact * scale) <= slack * scale * 2.0 ** -14)


def test_fp8_large_tile_kernel_ragged_shape():
    """A shape with a ragged last row block (1000 rows), a column count that is not a multiple of the tile
    or of 8 (the row-band store path is off, the last tile is cut) which still selects the large-tile kernel."""
    fa = _fa()
    be = ops()
    m, k, n = 1000, 1024, 9004
    rng = np.random.default_rng(45)
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((k, n), dtype=np.float32)
    aq, a_scale = be.quantize_tensor_e4m3(be.upload(a))
    qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (k, n)), fa.capi.QW_E4M3_TENSOR)
    o.set_threads(8)
    want_aq, want_sa = o.quantize_tensor_e4m3(a)
    want_wq, want_sw = o.quantize_tensor_e4m3(w)
    o.set_threads(1)
    plan = _gemm_plan(fa, be, m, qw)
    assert plan.big_ntb in (14, 16), plan.big_ntb
    got = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.F32))
    rows = np.r_[0:8, 250:262, 760:776, 990:1000]
    _fp8_rows_check("1000x9004x1024 ntb=%d" % plan.big_ntb, got[rows], want_aq[rows], want_wq, want_sa, want_sw)
    assert np.all(np.isfinite(got))
    out_bf = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.BF16))
    assert_bf16_rounding_of("gemm_e4m3 ragged bf16", out_bf, got)
    # the 128 x 128 kernel on the same operands sums k in the same order: identical bits
    fa.check(fa.capi.lib.fa_set_tuning(4, 1))
    try:
        assert _gemm_plan(fa, be, m, qw).big_ntb == 0
        small = be.download_owned(be.gemm_e4m3(aq, a_scale, qw, fa.capi.F32))
    finally:
        fa.check(fa.capi.lib.fa_set_tuning(4, 0))
    assert np.array_equal(small, got)


@pytest.mark.parametrize("n", [9008, 9004], ids=["whole-tiles", "ragged-columns"])
def test_int8_large_tile_kernel_bias_without_raw_sums(n):
    """fa_linear_w8a8 on 1000 rows (quantizer + large-tile GEMM) with a bias and no raw-accumulator output: with a
    column count that is a multiple of 8 the epilogue adds the bias from registers and stores four outputs of a row
    per lane; otherwise it takes the general element-by-element form.  Both bit-exact against the oracle, f32 and
    bf16 outputs."""
    fa = _fa()
    be = ops()
    m, k = 1000, 1024
    rng = o.Rng(47 + n)
    x = rng.randn((m, k))
    w = rng.randn((k, n), std=0.05)
    bias = rng.randn((n,))
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    _, want = o.linear_w8a8(x, wq, ws, bias)
    o.set_threads(1)
    qw = be.import_quantized_weight(wq, ws)
    assert _gemm_plan(fa, be, m, qw).big_ntb in (14, 16)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    got = be.download_owned(be.linear_w8a8(be.upload(x), qw, bias=dbias))
    assert np.array_equal(got, want)
    out_bf = be.download_owned(be.linear_w8a8(be.upload(x), qw, bias=dbias, out_dtype=fa.capi.BF16))
    assert_bf16_rounding_of("w8a8 large tile bias bf16", out_bf, got)


@pytest.mark.parametrize("m,k,n", [(1024, 512, 4096), (1000, 1024, 6144), (800, 256, 4104), (1024, 4096, 4096), (800, 8320, 4096)])
def test_int8_large_tile_kernel_on_256_x_128_tiles(m, k, n):
    """About a thousand rows against a weight of 4096 to 6144 columns: too few 256 x 224 tiles for the device, so the
    large-tile kernel runs on 256 x 128 tiles (plan: 8 column tiles per block).  Raw sums and outputs bit-exact against
    the oracle with a bias and a residual-free epilogue, f32 and bf16 outputs, ragged rows and columns; equal to the
    128 x 128 kernel (key 4 = 1).  With k of 4096 and more and tiles for at most half the device, pairs of same-XCD blocks
    share a tile, half of k each, and meet in a workspace (the last two shapes, an odd number of k stages among them):
    three calls in a row, and identical to one block per tile (key 24 = 1)."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    rng = o.Rng(7 * m + n)
    x = rng.randn((m, k))
    w = rng.randn((k, n), std=0.05)
    bias = rng.randn((n,))
    o.set_threads(8)
    wq, ws = o.quantize_cols_i8(w)
    want_acc, want = o.linear_w8a8(x, wq, ws, bias)
    o.set_threads(1)
    qw = be.import_quantized_weight(wq, ws)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    dx = be.upload(x)
    try:
        fa.check(lib.fa_set_tuning(21, 1))                # no weight-stationary kernel: the tiled GEMMs
        assert _gemm_plan(fa, be, m, qw).big_ntb == 8
        out, acc = be.linear_w8a8(dx, qw, bias=dbias, want_acc=True)
        assert np.array_equal(be.download_owned(acc), want_acc)
        got = be.download_owned(be.linear_w8a8(dx, qw, bias=dbias))
        assert np.array_equal(be.download_owned(out), want) and np.array_equal(got, want)
        assert np.array_equal(be.download_owned(be.linear_w8a8(dx, qw, bias=dbias)), want)      # counters back at zero
        for scope in (2, 3):                              # partial sums exchanged with agent-scope accesses / in the XCD's L2
            fa.check(lib.fa_set_tuning(16, scope))
            assert np.array_equal(be.download_owned(be.linear_w8a8(dx, qw, bias=dbias)), want), scope
        fa.check(lib.fa_set_tuning(16, 0))
        fa.check(lib.fa_set_tuning(24, 1))
        assert np.array_equal(be.download_owned(be.linear_w8a8(dx, qw, bias=dbias)), want)
        fa.check(lib.fa_set_tuning(24, 0))
        out_bf = be.download_owned(be.linear_w8a8(dx, qw, bias=dbias, out_dtype=fa.capi.BF16))
        assert_bf16_rounding_of("w8a8 256 x 128 tiles bf16", out_bf, got)
        fa.check(lib.fa_set_tuning(4, 1))
        assert _gemm_plan(fa, be, m, qw).big_ntb == 0
        assert np.array_equal(be.download_owned(be.linear_w8a8(dx, qw, bias=dbias)), got)
    finally:
        fa.check(lib.fa_set_tuning(4, 0))
        fa.check(lib.fa_set_tuning(21, 0))
        fa.check(lib.fa_set_tuning(24, 0))
        fa.check(lib.fa_set_tuning(16, 0))


def test_int8_large_tile_kernel_wavefront_variants_are_bit_exact():
    """The 4- and 16-wavefront variants and both tile widths of the large-tile int8 kernel against the oracle
    on sampled rows of a ragged shape (exact integers: any difference is an indexing error)."""
    fa = _fa()
    be = ops()
    lib = fa.capi.lib
    m, k, n = 1000, 1024, 9004
    rng = np.random.default_rng(46)
    aq = rng.integers(-127, 128, size=(m, k), dtype=np.int8)
    wq = rng.integers(-127, 128, size=(k, n), dtype=np.int8)
    sx = rng.uniform(0.01, 0.05, size=m).astype(np.float32)
    sw = rng.uniform(1e-4, 1e-3, size=n).astype(np.float32)
    qw = be.import_quantized_weight(wq, sw)
    rows = np.r_[0:8, 250:262, 760:776, 990:1000]
    o.set_threads(8)
    want_acc = o.gemm_i8_i32(np.ascontiguousarray(aq[rows]), wq)
    o.set_threads(1)
    want = o.dequant_i32(want_acc, np.ascontiguousarray(sx[rows]), sw)
    daq, dsx = be.upload(aq), be.upload(sx)
    try:
        for ntb, waves in ((14, 4), (16, 4), (14, 16), (16, 16), (0, 0)):
            fa.check(lib.fa_set_tuning(7, ntb))
            fa.check(lib.fa_set_tuning(6, waves))
            plan = _gemm_plan(fa, be, m, qw)
            assert plan.big_ntb in (14, 16) and plan.waves == (waves or 8)
            out, acc = be.gemm_w8a8(daq, dsx, qw, fa.capi.F32, want_acc=True)
            assert np.array_equal(be.download_owned(acc)[rows], want_acc), (ntb, waves)
            assert np.array_equal(be.download_owned(out)[rows], want), (ntb, waves)
    finally:
        fa.check(lib.fa_set_tuning(7, 0))
        fa.check(lib.fa_set_tuning(6, 0))


def _fp8_rows_bound_check(tag, got, qa, qb, sa, sb, bias=None):
    """Stated fp8 bound for the per-token x per-channel linear: |gpu - exact| <= 2^-15 * sum_k |a_k||b_k| * sa[m] * sb[n]
    (+ one rounding of the bias add), and >= 98 % of the outputs inside the composite tolerance."""
    o.set_threads(8)
    want = o.linear_e4m3_rows(qa, qb, sa, sb, bias)
    o.set_threads(1)
    absprod = np.abs(o.from_e4m3(qa)).astype(np.float64) @ np.abs(o.from_e4m3(qb)).astype(np.float64)
    bound = absprod * sa[:, None].astype(np.float64) * sb[None, :].astype(np.float64) * 2.0 ** -15 + 1e-30
    if bias is not None:
        bound = bound + np.abs(want) * 2.0 ** -23
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    print("FP8_ROWS_PARITY\t%s\tmax_err/bound=%.3e" % (tag, float((err / bound).max())), flush=True)
    assert np.all(err <= bound), tag
    r = o.compare(got, want)
    print(r.line("FP8_ROWS_PARITY", tag), flush=True)
    assert r.fail_count <= 2e-2 * r.total, tag
    return want


@pytest.mark.parametrize("m,k,n", [(1, 4096, 6144), (8, 4096, 4096), (32, 4096, 6144), (33, 1024, 528), (64, 11008, 512),
                                   (17, 200, 70), (300, 1024, 520), (1000, 1024, 9004)])
def test_fp8_per_token_per_channel_linear(m, k, n):
    """fa_linear_e4m3: per-token e4m3 activations (row absmax / 448) against per-channel e4m3 weights (column
    absmax / 448), dequantization fused.  Rows up to 64 take the weight-streaming kernel, 300 rows the 128 x 128
    GEMM, 1000 x 9004 the large-tile GEMM; (17, 200, 70) has a k that is no multiple of the 128-wide tile."""
    fa = _fa()
    be = ops()
    rng = np.random.default_rng(m * 7 + n)
    x = rng.standard_normal((m, k), dtype=np.float32) * rng.uniform(0.1, 10.0, size=(m, 1)).astype(np.float32)
    w = rng.standard_normal((k, n), dtype=np.float32) * rng.uniform(0.005, 0.05, size=(1, n)).astype(np.float32)
    bias = rng.standard_normal(n, dtype=np.float32)
    o.set_threads(8)
    want_xq, want_sx = o.quantize_rows_e4m3(x)
    want_wq, want_sw = o.quantize_cols_e4m3(w)
    o.set_threads(1)
    dx = be.upload(x)
    xq, sx = be.quantize_rows_e4m3(dx)
    assert np.array_equal(be.download(sx), want_sx) and np.array_equal(be.download(xq), want_xq)
    qw = be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (k, n)), fa.capi.QW_E4M3_CHANNEL)
    codes, scales = qw.export()
    assert np.array_equal(scales, want_sw) and np.array_equal(codes, want_wq)
    qw2 = be.import_quantized_weight(want_wq, want_sw, fa.capi.QW_E4M3_CHANNEL)
    c2, s2 = qw2.export()
    assert np.array_equal(c2, want_wq) and np.array_equal(s2, want_sw)
    if m > 64:
        plan = _gemm_plan(fa, be, m, qw)
        assert (plan.big_ntb != 0) == (m == 1000)
    dbias = fa.DeviceBufferView(be.upload(bias), 0, (n,))
    got = be.download_owned(be.linear_e4m3(dx, qw, out_dtype=fa.capi.F32))
    _fp8_rows_bound_check("%dx%dx%d" % (m, n, k), got, want_xq, want_wq, want_sx, want_sw)
    got_b = be.download_owned(be.linear_e4m3(dx, qw, bias=dbias, out_dtype=fa.capi.F32))
    _fp8_rows_bound_check("%dx%dx%d+bias" % (m, n, k), got_b, want_xq, want_wq, want_sx, want_sw, bias)
    assert_bf16_rounding_of("linear_e4m3 bf16", be.download_owned(be.linear_e4m3(dx, qw, bias=dbias, out_dtype=fa.capi.BF16)),
                            got_b)
    # bf16 activations are promoted exactly before the quantizer
    xb = o.to_bf16(x)
    o.set_threads(8)
    qb16, sb16 = o.quantize_rows_e4m3(o.from_bf16(xb))
    o.set_threads(1)
    got16 = be.download_owned(be.linear_e4m3(be.upload(xb), qw, out_dtype=fa.capi.F32))
    _fp8_rows_bound_check("%dx%dx%d:bf16 in" % (m, n, k), got16, qb16, want_wq, sb16, want_sw)
    if k % 128 == 0:
        # the pre-quantized entry point takes the same path: identical bits
        again = be.download_owned(be.gemm_e4m3_rows(xq, sx, qw, out_dtype=fa.capi.F32))
        assert np.array_equal(again, got)
    # a weight of another kind is refused
    with pytest.raises(fa.InvalidArgument):
        be.linear_e4m3(dx, be.quantize_weight(fa.DeviceBufferView(be.upload(w), 0, (k, n)), fa.capi.QW_E4M3_TENSOR))
