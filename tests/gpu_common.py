"""Shared pieces of the GPU parity tests: one backend object per session and
comparison helpers built on the oracle's judge."""
import numpy as np
import pytest

import oracle_lib as o

_ops = None


def ops():
    """The backend under test; raises (never skips, never falls back) without the HIP library."""
    global _ops
    if _ops is None:
        import fandhe_ai_amd as fa
        _ops = fa.tape_for(fa.Device.Rocm(0))
    return _ops


def assert_parity(tag, shape, got, want):
    """Composite tolerance of the reference (rel < 1e-3 or abs < 1e-5,
    crates/tensor-core/src/tolerance.rs:15-37); prints the reference's log line."""
    r = o.compare(got, want)
    print(r.line(tag, shape), flush=True)
    assert r.fail_count == 0, r.line(tag, shape)
    return r


def assert_bf16_rounding_of(tag, got_bf16, f32_values):
    """bf16 output == the single round-to-nearest-even of the kernel's own f32 result."""
    want = o.to_bf16(np.ascontiguousarray(f32_values, dtype=np.float32))
    mism = int((np.asarray(got_bf16).ravel() != want.ravel()).sum())
    assert mism == 0, "%s: %d bf16 outputs differ from RNE(f32 output)" % (tag, mism)
