"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, the host-only entry points (validators, size classes, error
reporting) behave like the reference's, and without a device every constructor
returns a typed error instead of crashing (the reference's `*_absent` tests,
crates/backend-rocm/tests/paged_kv_absent.rs:9-14).  No kernel is launched."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle_lib as o

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
U32MAX = 0xFFFFFFFF


def _fa():
    import fandhe_ai_amd as fa
    return fa


def test_library_exports_every_declared_symbol():
    fa = _fa()
    declared = set()
    for name in ("fandhe_rocm.h", "fandhe_rocm_bench.h"):
        header = open(os.path.join(ROOT, "include", name)).read()
        header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
        found = set(re.findall(r"\b(fa_[a-z0-9_]+)\s*\(", header))
        assert found, name
        declared |= found
    assert len(declared) > 60
    # the drop-in header holds nothing but what stands behind a reference interface: the aids live apart
    drop_in = open(os.path.join(ROOT, "include", "fandhe_rocm.h")).read()
    for aid in ("fa_set_tuning", "fa_fill_normal", "fa_probe_matrix_rate", "fa_timer_create", "fa_gemm_plan_query"):
        assert aid not in drop_in, aid
    missing = [n for n in sorted(declared) if not hasattr(fa.capi.lib, n)]
    assert not missing, missing
    assert declared == set(fa.capi.SIGNATURES), declared ^ set(fa.capi.SIGNATURES)
    assert fa.capi.lib.fa_abi_version() == 1
    assert fa.capi.lib.fa_status_name(fa.capi.UNSUPPORTED) == b"Unsupported"


def test_validators_follow_the_reference_tables():
    # crates/tensor-core/src/paged_kv.rs:387-521 through the C ABI
    fa = _fa()
    lib = fa.capi.lib

    def val_append(kn, vn, kp, vp, slots, layout):
        s = np.array(slots, dtype=np.uint32)
        return lib.fa_validate_paged_kv_append(kn, vn, kp, vp, s.ctypes.data_as(fa.capi.u32p), s.size, C.byref(layout))

    def val_attn(qn, kp, vp, tables, lens, args):
        t, s = np.array(tables, dtype=np.uint32), np.array(lens, dtype=np.uint32)
        plan = fa.capi.PagedPlan()
        rc = lib.fa_validate_paged_attention(qn, kp, vp, t.ctypes.data_as(fa.capi.u32p), t.size,
                                             s.ctypes.data_as(fa.capi.u32p), s.size, C.byref(args), C.byref(plan))
        return rc, plan

    L = lambda nb=4, bs=2, e=4: fa.capi.PagedLayout(nb, bs, e)
    A = lambda batch, l_new, mb, heads=2, scale=0.5, kvh=0, layout=None: fa.capi.PagedArgs(layout or L(), batch, l_new, heads, mb, scale, kvh)
    for bad in ((0, 2, 4), (4, 3, 4), (4, 512, 4), (4, 2, 0), (U32MAX, 2, 4), (4, 2, 2 ** 64 - 1),
                (1 << 20, 256, (2 ** 63 - 1) // (8 * 256) + 1)):
        assert val_append(0, 0, 0, 0, [], L(*bad)) == fa.capi.INVALID_ARGUMENT
    assert "paged_kv" in fa.capi.last_error()
    l, pool = L(), 32
    assert val_append(8, 8, pool, pool, [0, 7], l) == 0
    for args in ((7, 8, pool, pool, [0, 7]), (8, 4, pool, pool, [0, 7]), (8, 8, pool - 1, pool, [0, 7]),
                 (8, 8, pool, pool, [0, 8]), (4, 4, pool, pool, [U32MAX]), (8, 8, pool, pool, [3, 3])):
        assert val_append(*args, l) == fa.capi.INVALID_ARGUMENT
    assert val_append(0, 0, pool, pool, [], l) == 0
    rc, plan = val_attn(8, 32, 32, [0, 1, 2, 3], [3, 3], A(2, 1, 2))
    assert rc == 0 and (plan.out_numel, plan.s_max, plan.query_rows, plan.workspace_elems) == (8, 3, 4, 12)
    a = A(1, 2, 2)
    assert val_attn(8, 32, 32, [0, 1], [3], a)[0] == 0
    for args in ((7, 32, 32, [0, 1], [3]), (8, 31, 32, [0, 1], [3]), (8, 32, 32, [0], [3]), (8, 32, 32, [0, 1], [3, 3]),
                 (8, 32, 32, [0, 1], [1]), (8, 32, 32, [0, 1], [5]), (8, 32, 32, [0, 4], [3]),
                 (8, 32, 32, [0, U32MAX], [3])):
        assert val_attn(*args, a)[0] == fa.capi.INVALID_ARGUMENT
    assert val_attn(8, 32, 32, [0, U32MAX], [2], a)[0] == 0
    for bad in (A(1, 1, 2, heads=0), A(1, 1, 2, heads=3), A(1, 1, 2, scale=float("nan")), A(1, 1, 2, scale=float("inf")),
                A(2 ** 64 - 1, 1, 2), A(1, 1, 2, heads=3, kvh=2), A(1, 1, 2, heads=6, kvh=3)):
        assert val_attn(4, 32, 32, [0, 1], [2], bad)[0] == fa.capi.INVALID_ARGUMENT
    assert val_attn(16, 32, 32, [0, 1], [2], A(1, 1, 2, heads=8, kvh=2))[0] == 0         # q is 8 heads x Dh 2
    rc, plan = val_attn(0, 32, 32, [], [], A(0, 1, 2))
    assert rc == 0 and plan.out_numel == 0 and plan.workspace_elems == 0
    rc, plan = val_attn(0, 32, 32, [0, 1], [3], A(1, 0, 2))
    assert rc == 0 and plan.out_numel == 0
    big = A(1 << 20, 1 << 10, 2, heads=1)
    t = np.zeros((1 << 20) * 2, dtype=np.uint32)
    s = np.full(1 << 20, 2, dtype=np.uint32)
    assert lib.fa_validate_paged_attention((1 << 20) * (1 << 10) * 4, 32, 32, t.ctypes.data_as(fa.capi.u32p), t.size,
                                           s.ctypes.data_as(fa.capi.u32p), s.size, C.byref(big), None) == fa.capi.INVALID_ARGUMENT
    # the product validators agree with the oracle's on random tables
    rng = np.random.default_rng(0)
    for _ in range(200):
        nb, bs, e = int(rng.integers(1, 6)), int(2 ** rng.integers(0, 3)), int(rng.integers(1, 5)) * 2
        batch, mb = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        tables = rng.integers(0, nb + 1, size=batch * mb).astype(np.uint32)
        lens = rng.integers(0, mb * bs + 2, size=batch).astype(np.uint32)
        l_new = int(rng.integers(0, 3))
        fa_args = fa.capi.PagedArgs(fa.capi.PagedLayout(nb, bs, e), batch, l_new, 2, mb, 1.0, 0)
        o_args = o.PagedArgs(o.PagedLayout(nb, bs, e), batch, l_new, 2, mb, 1.0, 0)
        qn = batch * l_new * e
        got = val_attn(qn, nb * bs * e, nb * bs * e, tables, lens, fa_args)[0]
        want = o.lib.orc_validate_paged_attention(qn, nb * bs * e, nb * bs * e, o.ptr(tables, o.u32p), tables.size,
                                                  o.ptr(lens, o.u32p), lens.size, C.byref(o_args), None)
        assert (got == 0) == (want == 0)


def test_size_classes_follow_the_reference_examples():
    # crates/tensor-core/src/pool_core.rs:628-727
    fa = _fa()
    cls = C.c_uint64()
    table = {200704: 229376, 802816: 917504, 65536: 65536, 10240: 10240, 2560: 2560, 64 << 20: 64 << 20, 0: 0,
             1: 256, 255: 256, 256: 256, 1 << 20: 1 << 20, (1 << 20) + 1: 2 << 20, (64 << 20) - 1: 64 << 20,
             1792: 1792, 1793: 2048, 2048: 2048}
    for b, want in table.items():
        assert fa.capi.lib.fa_size_class_for(b, C.byref(cls)) == 0 and cls.value == want, b
    for b in np.random.default_rng(1).integers(0, 1 << 28, size=500):
        fa.capi.lib.fa_size_class_for(int(b), C.byref(cls))
        assert cls.value == o.lib.orc_size_class_for(int(b)) and cls.value >= b


def test_typed_errors_without_a_device_or_with_bad_handles():
    fa = _fa()
    lib = fa.capi.lib
    n = C.c_int32(-1)
    rc = lib.fa_device_count(C.byref(n))
    if rc == 0 and n.value > 0:
        pytest.skip("a gfx950 device is present; the absent-device path is covered on CPU hosts")
    assert n.value == 0
    assert not fa.RocmDeviceProvider().is_available() and fa.RocmDeviceProvider().enumerate() == []
    ctx = fa.capi.ctx_p()
    assert lib.fa_context_create(0, C.byref(ctx)) == fa.capi.DEVICE_UNAVAILABLE and not ctx.value
    assert fa.capi.last_error() != ""
    with pytest.raises(fa.DeviceUnavailable):
        fa.tape_for(fa.Device.Rocm(0))
    # null / foreign handles are argument errors, never a crash
    out = fa.capi.buf_p()
    assert lib.fa_alloc_zeroed(None, fa.capi.F32, 4, C.byref(out)) == fa.capi.INVALID_ARGUMENT
    assert lib.fa_synchronize_device(None) == fa.capi.INVALID_ARGUMENT
    assert lib.fa_buffer_free(None, None) == 0
    assert lib.fa_context_destroy(None) == fa.capi.INVALID_ARGUMENT
    assert lib.fa_set_tuning(99, 1) == fa.capi.INVALID_ARGUMENT


def test_device_provider_is_consistent_on_any_host():
    """crates/backend-rocm/tests/device_provider_absent.rs:9-58: the provider's name, enumerate / is_available /
    select agree with each other on any host, and devices that are not an existing ROCm ordinal are
    DeviceUnavailable before HIP is asked (this container has no device, a GPU host has one)."""
    fa = _fa()
    p = fa.RocmDeviceProvider()
    assert p.backend_name() == "rocm"
    listed = p.enumerate()                                   # never an error: an empty list without HIP
    assert p.is_available() == (len(listed) > 0)
    n = len(listed)
    for d in (fa.Device.Rocm(n), fa.Device.Rocm(2 ** 64 - 1), fa.Device.Rocm(-1), fa.Device.Rocm(True),
              fa.Device.Rocm(1.0), fa.Device.Cpu, fa.Device.Cuda(0), "rocm:0"):
        with pytest.raises(fa.DeviceUnavailable):
            p.select(d)
    assert fa.Device.Rocm(0) == fa.Device.Rocm(0) != fa.Device.Cuda(0) and repr(fa.Device.Cpu) == "Device::Cpu"
    if not listed:
        with pytest.raises(fa.DeviceUnavailable):
            p.select(fa.Device.Rocm(0))
    else:
        assert listed[0] == fa.Device.Rocm(0)
        ops = p.select(listed[0])
        assert ops.device() == fa.Device.Rocm(0)
        ops.close()
