"""The reference's own known-answer vectors (tests/golden/reference_vectors.json, each with its file:line)
against the oracle and against the product's host-side code that implements the same rule."""
import json
import math
import os
import struct

import numpy as np
import pytest

import oracle_lib as o

with open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")) as f:
    G = json.load(f)


def _num(v):
    return float(v) if isinstance(v, str) else v


def test_tolerance_vectors():
    for c in G["composite_close_f32"]["cases"]:
        assert bool(o.lib.orc_composite_close_f32(_num(c["actual"]), _num(c["reference"]))) == c["close"], c


def test_int8_gemm_vectors():
    g = G["int8_gemm_i32"]
    for c in g["cases"]:
        a = np.full((c["m"], c["k"]), c["a"], np.int8)
        b = np.full((c["k"], c["n"]), c["b"], np.int8)
        assert np.all(o.gemm_i8_i32(a, b) == c["every_output"]), c
    assert (2 ** 31 - 1) // (127 * 127) == g["k_safe"]


def test_rmsnorm_vector():
    g = G["rmsnorm_f32"]
    x = np.array([g["x"]], dtype=np.float32)
    rc, out = o.rmsnorm_f32(x, None, g["eps"])
    assert rc == 0 and np.array_equal(out, x * np.float32(1.0 / math.sqrt(g["mean_square"])))


def test_argmax_and_top_k_vectors():
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
    import sampling as osamp
    for c in G["greedy_argmax"]["cases"]:
        row = np.array([[_num(v) for v in c["row"]]], dtype=np.float32)
        assert o.argmax_rows(row).tolist() == [c["index"]], c
    for c in G["top_k_indices"]["cases"]:
        assert osamp.top_k_indices(c["row"], c["k"]) == c["indices"], c
    for c in G["generator_seed"]["cases"]:
        assert osamp.Generator(c["seed"]).state == c["state"]


def test_product_host_code_follows_the_same_vectors():
    import fandhe_ai_amd as fa
    from fandhe_ai_amd import capi, safetensors_io as st
    from fandhe_ai_amd.scheduler import InvalidArgument, SchedulerLimits
    for c in G["generator_seed"]["cases"]:
        state = capi.u64()
        assert capi.lib.fa_rng_state_from_seed(c["seed"], state) == 0 and state.value == c["state"]
    for size, cls in G["size_class_for"]["cases"]:
        assert o.lib.orc_size_class_for(size) == cls
        got = capi.u64()
        assert capi.lib.fa_size_class_for(size, got) == 0 and got.value == cls
    g = G["safetensors_typed"]

    def one(dtype, shape, raw):
        h = json.dumps({"t": {"dtype": dtype, "shape": shape, "data_offsets": [0, len(raw)]}}).encode()
        return struct.pack("<Q", len(h)) + h + raw
    widths = {"U8": 1, "I8": 1, "U16": 2, "F8_E4M3": 1, "C64": 8, "U64": 8}
    for d in g["rejected_dtypes"]:
        with pytest.raises(st.UnsupportedDtype):
            st.load_safetensors_typed_from_bytes(one(d, [1], bytes(widths[d])))
    for c in g["invalid_bool"]:
        with pytest.raises(st.InvalidBoolValue) as e:
            st.load_safetensors_typed_from_bytes(one("BOOL", [len(c["bytes"])], bytes(c["bytes"])))
        assert (e.value.index, e.value.value) == (c["index"], c["value"])
    bits = np.array(g["f32_bits_preserved"], dtype=np.uint32)
    got = st.load_safetensors_typed_from_bytes(one("F32", [2, 2], bits.tobytes()))["t"]
    assert got.data.view(np.uint32).ravel().tolist() == g["f32_bits_preserved"]
    g = G["scheduler_limits"]
    for bad in g["rejected"]:
        with pytest.raises(InvalidArgument):
            SchedulerLimits(*bad)
    lim = SchedulerLimits(*g["accepted"])
    assert [lim.max_active, lim.max_queued, lim.max_length] == g["accepted"]
