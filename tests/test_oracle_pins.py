"""Pins the CPU oracle before anything is compared with it.

Every check here is independent of the oracle's own formulas: the reference's
golden vectors and known answers (cited per test), closed forms, brute force
in another precision or another language (pure Python integers / Fractions,
numpy float64, torch's CPU dtypes).
"""
import ctypes as C
import math
from fractions import Fraction

import numpy as np
import pytest

import oracle_lib as o

MASK = (1 << 64) - 1


# ------------------------------------------------------------------- rng
def _py_xorshift(state):
    x = state
    x ^= (x << 13) & MASK
    x ^= x >> 7
    x ^= (x << 17) & MASK
    return x, (x * 0x2545F4914F6CDD1D) & MASK


def test_rng_matches_python_bigint_xorshift64star():
    # crates/tensor-core/src/rng.rs:62-79; seed 0 maps to the golden-ratio constant
    for seed in (0, 1, 42, 0xDEADBEEF):
        st = 0x9E3779B97F4A7C15 if seed == 0 else seed
        r = o.Rng(seed)
        for _ in range(64):
            st, out = _py_xorshift(st)
            assert r.next_u64() == out


def test_rng_unit_floats_and_randn_follow_the_reference_recipe():
    # rng.rs:82-104 (24-bit / 53-bit mantissa draws) and rng.rs:231-255 (Box-Muller pairs)
    st = 42
    r = o.Rng(42)
    st, a = _py_xorshift(st)
    assert o.lib.orc_rng_next_unit_f32(C.byref(r.state)) == np.float32((a >> 40) / float(1 << 24))
    st, a = _py_xorshift(st)
    assert o.lib.orc_rng_next_f32(C.byref(r.state)) == np.float32(np.float32((a >> 40) / float(1 << 24)) * np.float32(2) - np.float32(1))
    st, a = _py_xorshift(st)
    assert o.lib.orc_rng_next_unit_f64(C.byref(r.state)) == (a >> 11) / float(1 << 53)

    st = 7
    got = o.Rng(7).randn(5)
    want = []
    while len(want) < 5:
        st, a = _py_xorshift(st)
        st, b = _py_xorshift(st)
        u1 = 1.0 - (a >> 11) / float(1 << 53)
        u2 = (b >> 11) / float(1 << 53)
        rad = math.sqrt(-2.0 * math.log(u1))
        th = math.tau * u2
        want.append(np.float32(rad * math.cos(th)))
        want.append(np.float32(rad * math.sin(th)))
    assert np.array_equal(got, np.array(want[:5], dtype=np.float32))
    # odd length consumes the same number of draws as the next even length (rng.rs:223-229)
    r5, r6 = o.Rng(9), o.Rng(9)
    r5.randn(5)
    r6.randn(6)
    assert r5.next_u64() == r6.next_u64()


def test_randint_rejection_sampling_and_permutation():
    # rng.rs:283-312
    r = o.Rng(1)
    v = r.randint(-3, 2, 2000)
    assert v.min() == -3 and v.max() == 1 and set(v.tolist()) == {-3, -2, -1, 0, 1}
    st = 5
    got = o.Rng(5).randint(10, 17, 50)
    rng_range = 7
    zone = (rng_range * (MASK // rng_range)) & MASK
    want = []
    while len(want) < 50:
        st, x = _py_xorshift(st)
        if x < zone:
            want.append(10 + x % rng_range)
    assert got.tolist() == want
    p = o.Rng(3).permutation(1000)
    assert sorted(p.tolist()) == list(range(1000)) and p.tolist() != list(range(1000))


def test_parity_test_generator():
    # crates/backend-cpu/tests/paged_kv_backend_parity.rs:21-31
    out = np.empty(8, dtype=np.float32)
    o.lib.orc_test_data_f32(o.ptr(out, o.f32p), 8, 100)
    s = ((100 * 0x9E3779B97F4A7C15) & MASK) | 1
    want = []
    for _ in range(8):
        s ^= (s << 13) & MASK
        s ^= s >> 7
        s ^= (s << 17) & MASK
        want.append(np.float32(np.float32((s >> 40) / float(1 << 24)) * np.float32(2) - np.float32(1)))
    assert out.tolist() == [float(w) for w in want]


# ------------------------------------------------------------- tolerance
def test_tolerance_boundary_table_of_the_reference():
    # crates/tensor-core/src/tolerance.rs:43-63
    cc = o.lib.orc_composite_close_f32
    assert cc(1.0010005, 1.0) and cc(1.0, 1.0010005)
    assert not cc(1.01, 1.0)
    assert cc(0.0, 0.0) and cc(5e-6, 0.0) and not cc(2e-5, 0.0)
    assert not cc(float("nan"), 1.0)
    assert not cc(float("inf"), 1.0)
    assert not cc(float("inf"), float("inf"))


def test_tolerance_formula_grid_and_report():
    # tolerance.rs:65-87 value grid, judged by the formula written in Python doubles
    vals = [0.0, 1e-12, 5e-6, 2e-5, 0.5, 1.0, 1.0005, 1.0010005, 1.002, -1.0, -1.0010005, 1e20, 1.0011e20]
    for a in vals:
        for b in vals:
            x, y = float(np.float32(a)), float(np.float32(b))
            diff = abs(x - y)
            rel = diff / max(abs(x), abs(y), 1e-12)
            assert bool(o.lib.orc_composite_close_f32(a, b)) == (rel < 1e-3 or diff < 1e-5)
    a = np.array([1.0, 2.0, 3.0, float("nan")], dtype=np.float32)
    b = np.array([1.0, 2.1, 3.0, 0.0], dtype=np.float32)
    r = o.compare(a, b)
    assert r.total == 4 and r.fail_count == 2 and r.bit_mismatch == 2
    assert math.isinf(r.max_abs_diff) and math.isinf(r.max_fail_abs_diff)
    r = o.compare(a[:3], b[:3])
    assert r.fail_count == 1 and abs(r.max_abs_diff - abs(float(np.float32(2.0)) - float(np.float32(2.1)))) < 1e-12


# --------------------------------------------------------- number formats
def test_bf16_rne_matches_torch_on_all_upper_halves():
    torch = pytest.importorskip("torch")
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    for low in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        bits = (hi | low).astype(np.uint32)
        f = bits.view(np.float32)
        want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        got = o.to_bf16(f)
        nan = np.isnan(f)
        assert np.array_equal(got[~nan], want[~nan])
        assert np.all(np.isnan(o.from_bf16(got[nan])))
    # promote is exact
    assert np.array_equal(o.from_bf16(np.arange(1 << 16, dtype=np.uint16)).view(np.uint32),
                          np.arange(1 << 16, dtype=np.uint32) << 16)


def test_e4m3_decode_table_and_encode_against_torch_and_brute_force():
    torch = pytest.importorskip("torch")
    codes = np.arange(256, dtype=np.uint8)
    dec = o.from_e4m3(codes)
    want = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.array_equal(np.isnan(dec), nan)
    assert np.array_equal(dec[~nan], want[~nan])
    assert dec[0x7E] == 448.0 and dec[0x01] == 2.0 ** -9 and dec[0x08] == 2.0 ** -6
    # encode: dense grid inside the finite range against torch (round-to-nearest-even)
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.uniform(-448, 448, 200000), rng.normal(0, 1, 200000), rng.normal(0, 0.01, 100000),
        dec[~nan].astype(np.float64),
        # exact midpoints between neighbouring codes: ties must go to the even mantissa
        (np.sort(dec[(~nan) & (dec >= 0)])[:-1] + np.sort(dec[(~nan) & (dec >= 0)])[1:]) / 2,
    ]).astype(np.float32)
    got = o.to_e4m3(x)
    want = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    # brute force nearest representable value on a sample (independent of torch)
    finite = np.sort(dec[~nan].astype(np.float64))
    for v in x[:2000]:
        best = finite[np.argmin(np.abs(finite - float(v)))]
        assert abs(float(o.lib.orc_e4m3_to_f32(o.lib.orc_f32_to_e4m3(float(v)))) - float(v)) <= abs(best - float(v)) + 0.0
    # saturation instead of NaN above the largest finite value
    assert o.lib.orc_f32_to_e4m3(1e9) == 0x7E and o.lib.orc_f32_to_e4m3(-500.0) == 0xFE
    assert o.lib.orc_f32_to_e4m3(float("nan")) & 0x7F == 0x7F


# --------------------------------------------------------- f32 GEMM/linear
def _round_f32(fr):
    """Correctly rounded float32 of an exact Fraction (ties to even)."""
    if fr == 0:
        return np.float32(0.0)
    d = float(fr)                       # float64, may be off by a double rounding ...
    c = np.float32(d)
    cands = {c, np.nextafter(c, np.float32(np.inf)), np.nextafter(c, np.float32(-np.inf))}
    best = None
    for x in cands:
        err = abs(Fraction(float(x)) - fr)
        even = (np.float32(x).view(np.uint32) & 1) == 0
        key = (err, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, x)
    return np.float32(best[1])


def test_gemm_f32_is_k_ascending_single_accumulator_fma():
    # crates/backend-cpu/src/parity.rs:340-361: exact-rational FMA emulation on a small case
    rng = np.random.default_rng(1)
    m, n, k = 3, 4, 9
    a = rng.normal(size=(m, k)).astype(np.float32)
    b = rng.normal(size=(k, n)).astype(np.float32)
    got = o.gemm_f32(a, b)
    for i in range(m):
        for j in range(n):
            acc = np.float32(0.0)
            for p in range(k):
                acc = _round_f32(Fraction(float(a[i, p])) * Fraction(float(b[p, j])) + Fraction(float(acc)))
            assert got[i, j] == acc
    # and a larger case against float64 matmul
    a = rng.normal(size=(17, 300)).astype(np.float32)
    b = rng.normal(size=(300, 33)).astype(np.float32)
    assert o.compare(o.gemm_f32(a, b), a.astype(np.float64) @ b.astype(np.float64)).fail_count == 0
    # k == 0 gives zeros (crates/backend-rocm/tests/gemm_real_device.rs:16-38 includes k=0)
    assert np.array_equal(o.gemm_f32(np.zeros((2, 0), np.float32), np.zeros((0, 3), np.float32)), np.zeros((2, 3), np.float32))


def test_linear_f32_bias_and_relu():
    rng = np.random.default_rng(2)
    a = rng.normal(size=(5, 7)).astype(np.float32)
    w = rng.normal(size=(7, 6)).astype(np.float32)
    bias = rng.normal(size=6).astype(np.float32)
    base = o.gemm_f32(a, w)
    assert np.array_equal(o.linear_f32(a, w, bias, 0), base + bias)
    assert np.array_equal(o.linear_f32(a, w, bias, 1), np.maximum(base + bias, 0))
    assert np.array_equal(o.linear_f32(a, w, None, 0), base)


# ------------------------------------------------------------ int8 pieces
def _probe_pattern(m=16, k=32, n=8):
    # docs/perf/logs/int8-mma-probe-2608/RULE.txt:25-28
    a = np.empty((m, k), dtype=np.int64)
    b = np.empty((k, n), dtype=np.int64)
    c = np.empty((m, n), dtype=np.int64)
    for r in range(m):
        for kk in range(k):
            a[r, kk] = ((r * 37 + kk * 91 + 11) % 251) - 125
    for kk in range(k):
        for cc in range(n):
            b[kk, cc] = ((kk * 53 + cc * 29 + 7) % 247) - 123
    a[0, 0], a[1, 1], b[0, 0], b[31, 7] = -128, 127, -128, 127
    for r in range(m):
        for cc in range(n):
            c[r, cc] = r * 1000003 - cc * 7919 - 5000000
    return a, b, c


def test_int8_gemm_reference_probe_vectors():
    # RULE.txt:6-10: ones -> 32; a=b=127 over K=128 -> +2064512; a=127,b=-127 -> -2064512
    ones = np.ones((16, 32), np.int8)
    assert np.all(o.gemm_i8_i32(ones, np.ones((32, 8), np.int8)) == 32)
    a = np.full((16, 128), 127, np.int8)
    assert np.all(o.gemm_i8_i32(a, np.full((128, 8), 127, np.int8)) == 2064512)
    assert np.all(o.gemm_i8_i32(a, np.full((128, 8), -127, np.int8)) == -2064512)
    pa, pb, pc = _probe_pattern()
    want = pc + pa @ pb                                    # int64, python-side naive GEMM
    got = o.gemm_i8_i32(pa.astype(np.int8), pb.astype(np.int8), pc.astype(np.int32))
    assert np.array_equal(got.astype(np.int64), want)
    # K_safe boundary (crates/backend-cuda/tests/int8_mma_probe_real_device.rs:566-572)
    assert (2 ** 31 - 1) // (127 * 127) == 133144
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, size=(9, 200), dtype=np.int8)
    b = rng.integers(-128, 128, size=(200, 11), dtype=np.int8)
    assert np.array_equal(o.gemm_i8_i32(a, b).astype(np.int64), a.astype(np.int64) @ b.astype(np.int64))


def test_quantize_rows_closed_forms():
    x = np.array([
        [127.0, -127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, 63.5],   # scale exactly 1: ties to even
        [0.0] * 10,                                                      # zero row: scale 0, q 0
        [-8.0, 4.0, 2.0, 1.0, 0.0, 8.0, -4.0, -2.0, -1.0, 0.03],
        [1e-30, -2e-30, 0, 0, 0, 0, 0, 0, 0, 0],
    ], dtype=np.float32)
    q, s = o.quantize_rows_i8(x)
    assert s[0] == 1.0 and q[0].tolist() == [127, -127, 0, 2, 2, 0, -2, -2, 3, 64]
    assert s[1] == 0.0 and not q[1].any()
    assert s[2] == np.float32(8.0) / np.float32(127.0) and q[2, 0] == -127 and q[2, 5] == 127
    assert q[3, 1] == -127 and q[3, 0] in (63, 64)
    rng = np.random.default_rng(4)
    x = rng.normal(size=(16, 4096)).astype(np.float32)
    q, s = o.quantize_rows_i8(x)
    assert np.array_equal(s, np.abs(x).max(axis=1) / np.float32(127.0))
    assert np.abs(q).max(axis=1).tolist() == [127] * 16
    # reconstruction error is at most half a step (plus one rounding of the division)
    assert np.all(np.abs(x - q.astype(np.float32) * s[:, None]) <= s[:, None] * 0.5000001)
    # monotone in x
    order = np.argsort(x[0], kind="stable")
    assert np.all(np.diff(q[0][order].astype(np.int32)) >= 0)
    # numpy restatement with IEEE float32 division + rint (half-even)
    want = np.clip(np.rint(x / s[:, None]), -127, 127).astype(np.int8)
    assert np.array_equal(q, want)


def test_quantize_cols_is_the_transpose_of_rows():
    rng = np.random.default_rng(5)
    w = (rng.normal(size=(64, 24)) * 0.02).astype(np.float32)
    q, s = o.quantize_cols_i8(w)
    qt, st = o.quantize_rows_i8(np.ascontiguousarray(w.T))
    assert np.array_equal(q, qt.T) and np.array_equal(s, st)


def test_dequant_single_multiply_and_linear_w8a8_composition():
    acc = np.array([[1, -2, 3], [1 << 24, (1 << 24) + 1, -(1 << 25) - 3]], dtype=np.int32)
    sx = np.array([0.5, 0.25], dtype=np.float32)
    sw = np.array([2.0, 3.0, 0.125], dtype=np.float32)
    out = o.dequant_i32(acc, sx, sw)
    want = acc.astype(np.float32) * (sx[:, None] * sw[None, :])     # int->f32 RNE, scales multiplied once
    assert np.array_equal(out, want)
    assert np.float32((1 << 24) + 1) == np.float32(1 << 24)        # RNE of a 25-bit accumulator
    bias = np.array([1.0, -1.0, 0.5], dtype=np.float32)
    assert np.array_equal(o.dequant_i32(acc, sx, sw, bias), want + bias)
    rng = np.random.default_rng(6)
    x = rng.normal(size=(4, 96)).astype(np.float32)
    w = (rng.normal(size=(96, 10)) * 0.02).astype(np.float32)
    wq, sw = o.quantize_cols_i8(w)
    acc, out = o.linear_w8a8(x, wq, sw)
    xq, sx = o.quantize_rows_i8(x)
    assert np.array_equal(acc.astype(np.int64), xq.astype(np.int64) @ wq.astype(np.int64))
    assert np.array_equal(out, acc.astype(np.float32) * (sx[:, None] * sw[None, :]))
    # the quantized linear approximates the f32 linear
    ref = x.astype(np.float64) @ w.astype(np.float64)
    assert np.abs(out - ref).max() < 0.02 * np.abs(ref).max()


def test_linear_w8a16_against_float64():
    rng = np.random.default_rng(7)
    a = o.to_bf16(rng.normal(size=(3, 128)).astype(np.float32))
    wq = rng.integers(-127, 128, size=(128, 300), dtype=np.int8)
    sw = rng.uniform(1e-4, 1e-3, size=300).astype(np.float32)
    got = o.linear_w8a16(a, wq, sw)
    want = (o.from_bf16(a).astype(np.float64) @ wq.astype(np.float64)) * sw.astype(np.float64)
    assert o.compare(got, want).fail_count == 0
    # one-hot activation picks a weight row exactly
    a1 = np.zeros((1, 128), np.float32)
    a1[0, 5] = 2.0
    got = o.linear_w8a16(o.to_bf16(a1), wq, sw)
    assert np.array_equal(got[0], (np.float32(2.0) * wq[5].astype(np.float32)) * sw)


def test_fp8_quantize_and_gemm():
    rng = np.random.default_rng(8)
    a = rng.normal(size=(5, 64)).astype(np.float32)
    b = rng.normal(size=(64, 7)).astype(np.float32)
    qa, sa = o.quantize_tensor_e4m3(a)
    qb, sb = o.quantize_tensor_e4m3(b)
    assert sa == np.abs(a).max() / np.float32(448.0)
    assert o.from_e4m3(qa).max() <= 448 and np.abs(o.from_e4m3(qa)).max() == 448.0
    got = o.gemm_e4m3(qa, qb, sa, sb)
    want = (o.from_e4m3(qa).astype(np.float64) @ o.from_e4m3(qb).astype(np.float64)).astype(np.float32) * (sa * sb)
    assert np.array_equal(got, want)
    # and the quantized product tracks the real one
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.abs(got - ref).max() < 0.1 * np.abs(ref).max()


def test_fp8_per_token_and_per_channel_quantizers_and_linear():
    """Closed forms for the per-row / per-column e4m3 quantizers and the double GEMM of the dequantized operands
    for the linear built on them."""
    rng = np.random.default_rng(18)
    x = rng.normal(size=(6, 96)).astype(np.float32) * np.array([[1e-3], [1.0], [50.0], [0.0], [3.0], [1e4]], np.float32)
    q, s = o.quantize_rows_e4m3(x)
    amax = np.abs(x).max(axis=1)
    assert np.array_equal(s, amax / np.float32(448.0))
    dec = o.from_e4m3(q)
    for r in range(6):
        if amax[r] == 0:
            assert s[r] == 0 and not q[r].any()                       # a zero row: scale 0, codes 0
            continue
        j = int(np.abs(x[r]).argmax())
        assert q[r, j] == (0x7E if x[r, j] > 0 else 0xFE)             # the absmax element is +-448
        assert np.abs(dec[r]).max() == 448.0
        # three mantissa bits: half an ulp is 2^-4 relative for normal codes; below 2^-6 the spacing is 2^-9
        err = np.abs(dec[r].astype(np.float64) * float(s[r]) - x[r].astype(np.float64))
        assert np.all(err <= np.abs(x[r]) * 2.0 ** -4 + float(s[r]) * 2.0 ** -10 + 1e-30)
        # every code is the nearest representable value of x / s (ties aside): re-encoding the scaled input agrees
        assert np.array_equal(q[r], o.to_e4m3((x[r] / s[r]).astype(np.float32)))
        # order is preserved
        order = np.argsort(x[r], kind="stable")
        assert np.all(np.diff(dec[r][order]) >= 0)
    # columns: the transpose of the row quantizer
    w = np.ascontiguousarray(x.T)
    qc, sc = o.quantize_cols_e4m3(w)
    assert np.array_equal(qc, q.T) and np.array_equal(sc, s)
    # linear: exact double sum of the decoded codes, one f32 scale product per output, bias added last
    a = rng.normal(size=(7, 128)).astype(np.float32)
    b = (rng.normal(size=(128, 9)) * np.linspace(0.01, 3.0, 9)).astype(np.float32)
    bias = rng.normal(size=9).astype(np.float32)
    qa, sa = o.quantize_rows_e4m3(a)
    qb, sb = o.quantize_cols_e4m3(b)
    got = o.linear_e4m3_rows(qa, qb, sa, sb, bias)
    exact = o.from_e4m3(qa).astype(np.float64) @ o.from_e4m3(qb).astype(np.float64)
    want = exact.astype(np.float32) * (sa[:, None] * sb[None, :]) + bias[None, :]
    assert np.array_equal(got, want.astype(np.float32))
    assert np.array_equal(o.linear_e4m3_rows(qa, qb, sa, sb), (exact.astype(np.float32) * (sa[:, None] * sb[None, :])))
    # with all scales equal it reduces to the per-tensor GEMM
    ones_a, ones_b = np.full(7, 0.5, np.float32), np.full(9, 0.25, np.float32)
    assert np.array_equal(o.linear_e4m3_rows(qa, qb, ones_a, ones_b), o.gemm_e4m3(qa, qb, np.float32(0.5), np.float32(0.25)))
    # and the quantized linear tracks the real one (per-channel scales keep the small columns accurate)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.all(np.abs(o.linear_e4m3_rows(qa, qb, sa, sb) - ref).max(axis=0) < 0.12 * np.abs(ref).max(axis=0))


# ----------------------------------------------------------------- RMSNorm
def test_rmsnorm_reference_fixtures():
    # crates/backend-cpu/src/rmsnorm.rs:433-441: [1,2,3,4], eps 0 -> x / sqrt(7.5)
    x = np.array([[1, 2, 3, 4]], dtype=np.float32)
    rc, out = o.rmsnorm_f32(x, None, 0.0)
    assert rc == 0
    rstd = np.float32(1.0 / math.sqrt(7.5))
    assert np.array_equal(out, x * rstd)
    # rmsnorm.rs:443-462: a NaN poisons its whole row and only that row
    x = np.array([[1, float("nan"), 3], [1, 2, 3]], dtype=np.float32)
    rc, out = o.rmsnorm_f32(x, None, 1e-5)
    assert np.all(np.isnan(out[0])) and np.all(np.isfinite(out[1]))
    # rmsnorm.rs:97-99: eps must be finite and non-negative; weight length must match
    assert o.rmsnorm_f32(x, None, -1.0)[0] == -1
    assert o.rmsnorm_f32(x, None, float("nan"))[0] == -1
    assert o.rmsnorm_f32(x, np.ones(2, np.float32), 1e-5)[0] == -3
    # crates/backend-cpu/tests/rmsnorm_parity.rs:86-92: extreme magnitudes stay finite (f64 statistic)
    x = np.array([[1e30, -1e30, 1e30, 1e-30]], dtype=np.float32)
    rc, out = o.rmsnorm_f32(x, None, 1e-5)
    assert rc == 0 and np.all(np.isfinite(out))


@pytest.mark.parametrize("hidden", [1, 4, 8, 1023, 1024, 4097])
def test_rmsnorm_shape_sweep_against_float64(hidden):
    # crates/backend-cpu/tests/rmsnorm_parity.rs:68-82
    rng = np.random.default_rng(hidden)
    x = rng.normal(size=(3, hidden)).astype(np.float32)
    w = rng.normal(size=hidden).astype(np.float32)
    rc, out = o.rmsnorm_f32(x, w, 1e-5)
    assert rc == 0
    inv_n = float(np.float32(1.0) / np.float32(hidden))
    x64 = x.astype(np.float64)
    rstd = (1.0 / np.sqrt((x64 * x64).sum(axis=1) * inv_n + float(np.float32(1e-5)))).astype(np.float32)
    want = (x * rstd[:, None]) * w[None, :]
    r = o.compare(out, want)
    assert r.fail_count == 0 and r.max_rel_err < 1e-6
    rc, out0 = o.rmsnorm_f32(np.zeros((0, hidden), np.float32), None, 1e-5, 0, hidden)
    assert rc == 0 and out0.size == 0


# -------------------------------------------------------------------- RoPE
def test_rope_textbook_properties():
    rng = np.random.default_rng(9)
    dh, theta = 128, 500000.0
    x = rng.normal(size=(6, 3, dh)).astype(np.float32)
    pos = np.array([0, 1, 7, 100, 4095, 8191], dtype=np.int32)
    out = o.rope_f32(x, pos, theta)
    assert np.array_equal(out[0], x[0])                              # position 0 is the identity
    half = dh // 2
    n_in = x[..., :half].astype(np.float64) ** 2 + x[..., half:].astype(np.float64) ** 2
    n_out = out[..., :half].astype(np.float64) ** 2 + out[..., half:].astype(np.float64) ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)            # each pair is rotated
    # f64 brute force with the rotate-half pairing (i, i + Dh/2)
    i = np.arange(half)
    inv = theta ** (-2.0 * i / dh)
    ang = pos[:, None].astype(np.float64) * inv[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x64 = x.astype(np.float64)
    want = np.concatenate([x64[..., :half] * c - x64[..., half:] * s,
                           x64[..., half:] * c + x64[..., :half] * s], axis=-1)
    assert o.compare(out, want).fail_count == 0
    # <R_m q, R_n k> depends only on m - n
    q = rng.normal(size=(1, 1, dh)).astype(np.float32)
    k = rng.normal(size=(1, 1, dh)).astype(np.float32)

    def dot(m, n):
        return float(np.dot(o.rope_f32(q, [m], theta).ravel().astype(np.float64),
                            o.rope_f32(k, [n], theta).ravel().astype(np.float64)))
    assert abs(dot(5, 3) - dot(102, 100)) < 1e-4 and abs(dot(5, 3) - dot(2, 0)) < 1e-4


# ------------------------------------------------------------ elementwise
def test_silu_and_argmax_fixtures():
    for v in (-100.0, -20.0, -1.0, -1e-3, 0.0, 1e-3, 1.0, 20.0, 100.0):
        want = v / (1.0 + math.exp(-v)) if v > -700 else 0.0
        assert abs(o.lib.orc_silu_f32(v) - want) <= 1e-6 * max(1.0, abs(want))
    assert o.lib.orc_silu_f32(-1e30) == 0.0 or o.lib.orc_silu_f32(-1e30) == -0.0
    g = np.array([1.0, -2.0, 0.5], np.float32)
    u = np.array([2.0, 3.0, -4.0], np.float32)
    got = o.silu_mul_f32(g, u)
    assert np.allclose(got, g / (1 + np.exp(-g.astype(np.float64))) * u, rtol=1e-6)
    # crates/autodiff/src/generate/mod.rs:777-781
    assert o.argmax_rows(np.array([[1.0, 3.0, 3.0, 2.0]], np.float32)).tolist() == [1]
    assert o.argmax_rows(np.array([[5.0]], np.float32)).tolist() == [0]
    assert o.argmax_rows(np.array([[-1.0, -2.0, -0.5]], np.float32)).tolist() == [2]
    # crates/backend-rocm/src/ops.rs:991-995: NaN ignored, all-NaN -> 0
    nan = float("nan")
    assert o.argmax_rows(np.array([[nan, 1.0, nan, 2.0], [nan, nan, nan, nan]], np.float32)).tolist() == [3, 0]


# ------------------------------------------------------------ memory pool
def test_size_classes_reference_examples():
    # crates/tensor-core/src/pool_core.rs:628-727
    sc = o.lib.orc_size_class_for
    assert sc(200704) == 229376 and sc(802816) == 917504 and sc(65536) == 65536
    assert sc(10240) == 10240 and sc(2560) == 2560 and sc(64 << 20) == 64 << 20
    assert sc(0) == 0 and sc(1) == 256 and sc(255) == 256 and sc(256) == 256
    assert sc(1 << 20) == 1 << 20 and sc((1 << 20) + 1) == 2 << 20
    assert sc((64 << 20) - 1) == 64 << 20
    assert sc(1024 + 768) == 1792 and sc(1793) == 2048 and sc(2048) == 2048
    assert sc((64 << 20) + 12345) == (64 << 20) + 12345
