"""safetensors typed loading: the reference's own loader tests (crates/onnx-interop/tests/st_typed.rs,
st_load.rs) replayed on hand-serialized files, and cross-checks against the safetensors library's reader and
writer (an independent implementation of the wire format)."""
import json
import struct

import numpy as np
import pytest
from safetensors.numpy import load as st_lib_load
from safetensors.numpy import save as st_lib_save

import fandhe_ai_amd  # noqa: F401  (the package needs the built library; the loader itself is host code)
from fandhe_ai_amd import safetensors_io as st


def ser(tensors, metadata=None, pad_header=0):
    """tensors: [(name, dtype_name, shape, raw bytes)] -> file bytes, offsets in the given order."""
    header, data, off = {}, b"", 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, dtype, shape, raw in tensors:
        header[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [off, off + len(raw)]}
        data += raw
        off += len(raw)
    h = json.dumps(header, separators=(",", ":")).encode() + b" " * pad_header
    return struct.pack("<Q", len(h)) + h + data


def test_all_reference_dtypes_round_trip_bit_exact():
    rng = np.random.default_rng(0)
    arrays = {"f32": rng.standard_normal((3, 4)).astype(np.float32), "f16": rng.standard_normal(5).astype(np.float16),
              "f64": rng.standard_normal((2, 2, 2)), "i32": rng.integers(-9, 9, 7).astype(np.int32),
              "i64": rng.integers(-9, 9, (1, 3)).astype(np.int64), "b": np.array([True, False, True]),
              "scalar": np.array(2.5, np.float32), "empty": np.zeros((0, 4), np.float32)}
    got = st.load_safetensors_typed_from_bytes(st_lib_save(arrays))
    tags = {"f32": "F32", "f16": "F16", "f64": "F64", "i32": "I32", "i64": "I64", "b": "BOOL", "scalar": "F32", "empty": "F32"}
    for k, a in arrays.items():
        assert got[k].dtype == tags[k] and got[k].shape == a.shape
        assert got[k].data.tobytes() == a.tobytes()
    # bf16: raw bits kept, to_f32 exact
    bits = np.array([0x3F80, 0xC000, 0x7FC0, 0x0001], np.uint16)
    got = st.load_safetensors_typed_from_bytes(ser([("w", "BF16", [4], bits.tobytes())]))
    assert np.array_equal(got["w"].data, bits)
    assert got["w"].to_f32().view(np.uint32).tolist() == [0x3F800000, 0xC0000000, 0x7FC00000, 0x00010000]
    # and the library reads what the hand serializer writes (the two agree on the wire format)
    a = rng.standard_normal((2, 3)).astype(np.float32)
    assert np.array_equal(st_lib_load(ser([("x", "F32", [2, 3], a.tobytes())]))["x"], a)


def test_unsupported_dtypes_are_rejected_fail_closed():
    # crates/onnx-interop/tests/st_typed.rs:194-208
    for d, width in (("U8", 1), ("I8", 1), ("U16", 2), ("F8_E4M3", 1), ("C64", 8), ("U64", 8)):
        with pytest.raises(st.UnsupportedDtype):
            st.load_safetensors_typed_from_bytes(ser([("t", d, [1], bytes(width))]))
    # already quantized checkpoints are an opt-in beyond the reference
    got = st.load_safetensors_typed_from_bytes(ser([("q", "I8", [2], b"\x7f\x81"), ("e", "F8_E4M3", [1], b"\x38")]),
                                               allow_quantized=True)
    assert got["q"].data.tolist() == [127, -127] and got["e"].data.tolist() == [0x38]


def test_invalid_bool_byte_is_rejected():
    # st_typed.rs:210-226
    with pytest.raises(st.InvalidBoolValue) as e:
        st.load_safetensors_typed_from_bytes(ser([("m", "BOOL", [3], bytes([0, 1, 2]))]))
    assert (e.value.key, e.value.index, e.value.value) == ("m", 2, 2)
    with pytest.raises(st.InvalidBoolValue) as e:
        st.load_safetensors_typed_from_bytes(ser([("m", "BOOL", [4], bytes([0, 7, 9, 1]))]))
    assert (e.value.index, e.value.value) == (1, 7)


def test_typed_f32_arm_matches_legacy_loader_bits():
    # st_typed.rs:228-252: NaN payload, -0.0, a subnormal
    vals = np.array([0x7FC00001, 0x80000000, 0x000116C2, 0x40600000], np.uint32)
    data = ser([("w", "F32", [2, 2], vals.tobytes())])
    legacy = st.load_safetensors_f32_from_bytes(data)["w"]
    typed = st.load_safetensors_typed_from_bytes(data)["w"]
    assert legacy.view(np.uint32).ravel().tolist() == vals.tolist() == typed.data.view(np.uint32).ravel().tolist()
    assert legacy.shape == typed.shape == (2, 2)
    with pytest.raises(st.UnsupportedDtype):                                   # st_typed.rs:254-259
        st.load_safetensors_f32_from_bytes(ser([("t", "I64", [1], bytes(8))]))


def test_require_keys_reports_all_missing():
    with pytest.raises(st.MissingKeys) as e:
        st.require_keys_typed({"b": 1}, ["a", "b", "c"])
    assert e.value.keys == ["a", "c"]
    st.require_keys({"a": 1, "b": 2}, ["a", "b"])


def test_layout_violations_are_format_errors_before_any_conversion():
    good = ser([("a", "F32", [2], bytes(8)), ("b", "I32", [1], bytes(4))])
    st.validate_safetensors_layout_from_bytes(good)
    st.validate_safetensors_layout_from_bytes(ser([("h", "U16", [3], bytes(6))]))      # any wire dtype passes the layout check
    bad = {
        "truncated data": good[:-1],
        "trailing bytes": good + b"\x00",
        "short file": good[:5],
        "header length beyond the file": struct.pack("<Q", 1 << 20) + good[8:],
        "header too large": struct.pack("<Q", 100_000_001) + good[8:],
        "not json": struct.pack("<Q", 4) + b"{,,}",
        "header not an object": struct.pack("<Q", 2) + b"[]",
        "shape and bytes disagree": ser([("a", "F32", [3], bytes(8))]),
        "unknown dtype": ser([("a", "F33", [2], bytes(8))]),
    }
    # a hole and an overlap between byte ranges
    h = {"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}, "b": {"dtype": "F32", "shape": [1], "data_offsets": [8, 12]}}
    hb = json.dumps(h).encode()
    bad["hole"] = struct.pack("<Q", len(hb)) + hb + bytes(12)
    h["b"]["data_offsets"] = [2, 6]
    hb = json.dumps(h).encode()
    bad["overlap"] = struct.pack("<Q", len(hb)) + hb + bytes(6)
    for what, data in bad.items():
        for fn in (st.validate_safetensors_layout_from_bytes, st.load_safetensors_typed_from_bytes,
                   st.load_safetensors_f32_from_bytes):
            with pytest.raises(st.SafetensorsFormat):
                fn(data)
        with pytest.raises(Exception):                     # the library rejects the same files
            st_lib_load(data)
        assert what
    meta = st.load_safetensors_typed_from_bytes(ser([("a", "F32", [1], bytes(4))], metadata={"format": "pt"}, pad_header=3))
    assert list(meta) == ["a"]


def test_llama_layout_transposes_explicitly_and_lists_every_missing_key():
    rng = np.random.default_rng(1)
    d, f, v, h, kv, dh = 8, 12, 20, 2, 1, 4
    t = {"model.embed_tokens.weight": rng.standard_normal((v, d)), "model.norm.weight": rng.standard_normal(d),
         "lm_head.weight": rng.standard_normal((v, d))}
    p = "model.layers.0."
    t.update({p + "input_layernorm.weight": rng.standard_normal(d), p + "post_attention_layernorm.weight": rng.standard_normal(d),
              p + "self_attn.q_proj.weight": rng.standard_normal((h * dh, d)), p + "self_attn.k_proj.weight": rng.standard_normal((kv * dh, d)),
              p + "self_attn.v_proj.weight": rng.standard_normal((kv * dh, d)), p + "self_attn.o_proj.weight": rng.standard_normal((d, h * dh)),
              p + "mlp.gate_proj.weight": rng.standard_normal((f, d)), p + "mlp.up_proj.weight": rng.standard_normal((f, d)),
              p + "mlp.down_proj.weight": rng.standard_normal((d, f))})
    t = {k: a.astype(np.float32) for k, a in t.items()}
    typed = st.load_safetensors_typed_from_bytes(st_lib_save(t))
    out = st.llama_decoder_tensors(typed, 1)
    assert out["layers.0.wqkv"].shape == (d, (h + 2 * kv) * dh)
    assert np.array_equal(out["layers.0.wqkv"][:, :h * dh], t[p + "self_attn.q_proj.weight"].T)
    assert np.array_equal(out["layers.0.wqkv"][:, -kv * dh:], t[p + "self_attn.v_proj.weight"].T)
    assert np.array_equal(out["layers.0.wgu"][:, f:], t[p + "mlp.up_proj.weight"].T)
    assert np.array_equal(out["lm_head"], t["lm_head.weight"].T) and out["layers.0.wdown"].shape == (f, d)
    del typed[p + "mlp.up_proj.weight"], typed["model.norm.weight"]
    with pytest.raises(st.MissingKeys) as e:
        st.llama_decoder_tensors(typed, 1)
    assert sorted(e.value.keys) == sorted([p + "mlp.up_proj.weight", "model.norm.weight"])


def test_writer_is_bit_identical_to_the_wire_formats_own_serializer_and_round_trips(tmp_path):
    # st_save.rs hands its sorted tensors to the safetensors serializer; the library's writer is that serializer
    rng = np.random.default_rng(3)
    mixes = [
        {"b": rng.standard_normal((2, 2)).astype(np.float32), "a": rng.integers(-5, 5, 3).astype(np.int64),
         "c": np.array([True, False, True]), "d": rng.standard_normal(1).astype(np.float16),
         "e": np.zeros((0, 3), np.float64), "aa": np.array([7], np.int32), "s": np.array(1.5, np.float32)},
        {"only": rng.standard_normal((5, 7, 3)).astype(np.float32)},
        {"w.%d" % i: rng.standard_normal((i + 1, 4)).astype(np.float32) for i in range(12)},
        {},
    ]
    for t in mixes:
        mine = st.save_safetensors_typed_to_bytes(t)
        assert mine == st_lib_save(t)
        assert mine == st.save_safetensors_typed_to_bytes(dict(reversed(list(t.items()))))       # deterministic
        back = st.load_safetensors_typed_from_bytes(mine)
        assert sorted(back) == sorted(t)
        for k, a in t.items():
            assert back[k].shape == a.shape and back[k].data.tobytes() == a.tobytes()
        assert st.save_safetensors_typed_to_bytes(back) == mine                                 # save -> load -> save
    # bf16 bits and special values survive (st_roundtrip.rs)
    special = np.array([0x7FC00001, 0x80000000, 0x00000001, 0x7F800000, 0xFF800000], np.uint32).view(np.float32)
    bf = st.TypedTensor("BF16", (3,), np.array([0x3F80, 0x7FC1, 0x8000], np.uint16))
    data = st.save_safetensors_typed_to_bytes({"x": special, "h": bf})
    back = st.load_safetensors_typed_from_bytes(data)
    assert back["x"].data.view(np.uint32).tolist() == special.view(np.uint32).tolist()
    assert back["h"].dtype == "BF16" and back["h"].data.tolist() == [0x3F80, 0x7FC1, 0x8000]
    # files: through a temporary name; the float32 entry points refuse anything else
    path = str(tmp_path / "ck.safetensors")
    st.save_safetensors_f32(path, {"x": special})
    assert st.load_safetensors_f32(path)["x"].view(np.uint32).tolist() == special.view(np.uint32).tolist()
    assert [p.name for p in tmp_path.iterdir()] == ["ck.safetensors"]
    with pytest.raises(st.SaveError):
        st.save_safetensors_f32_to_bytes({"i": np.array([1], np.int32)})
    with pytest.raises(st.SaveError):
        st.save_safetensors_typed_to_bytes({"u": np.array([1], np.uint16)})
    with pytest.raises(st.SaveError):
        st.save_safetensors_typed_to_bytes({"t": st.TypedTensor("F32", (3,), np.zeros(2, np.float32))})
    with pytest.raises(st.SaveError):
        st.save_safetensors_typed(str(tmp_path / "no" / "such" / "dir.safetensors"), {"x": special})
    meta = st.save_safetensors_typed_to_bytes({"x": special}, metadata={"format": "pt"})
    assert meta == st_lib_save({"x": special}, metadata={"format": "pt"})
