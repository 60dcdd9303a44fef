"""safetensors wire format -> typed host tensors -> device-resident parameters.

Mirrors the loading side of the reference (crates/onnx-interop/src/st_load.rs): the same dtype set
(F32 / F16 / BF16 / F64 / I32 / I64 / BOOL, lines 231-281), the same error kinds (``LoadError``, lines
47-87), the same validation order (layout first, then dtype, then data length, then shape; lines 24-31),
``require_keys`` reporting every missing key at once (lines 205-222, 568-590) and no implicit transposes
(lines 14-19: a caller that wants ``[in, out]`` transposes ``[out, in]`` itself).  The wire format is
parsed here (8-byte little-endian header length, JSON header, contiguous byte ranges covering the rest of
the file exactly: the checks of safetensors 0.7 ``Metadata::validate``), no third-party reader is needed.

Beyond the reference: with ``allow_quantized=True`` the typed loader also accepts ``I8`` and ``F8_E4M3``
tensors (already quantized checkpoints), which the reference rejects (tests/st_typed.rs:194-208); and
``DeviceParamStore`` / ``load_decoder`` put the tensors on the device (one flat resident buffer with
``DeviceBufferView`` offsets, crates/tensor-core/src/buffer.rs:277-303) and quantize the decoder's
projections per output channel there.
"""
import json
import os
import struct

import numpy as np

from . import capi
from .backend import DeviceBufferView

MAX_HEADER_BYTES = 100_000_000


class LoadError(Exception):
    """crates/onnx-interop/src/st_load.rs:47-87"""


class Io(LoadError):
    pass


class SafetensorsFormat(LoadError):
    pass


class MissingKeys(LoadError):
    def __init__(self, keys):
        super().__init__("missing tensor keys: " + ", ".join(keys))
        self.keys = list(keys)


class UnsupportedDtype(LoadError):
    def __init__(self, key, dtype):
        super().__init__("unsupported dtype (key=%s): %s" % (key, dtype))
        self.key, self.dtype = key, dtype


class InvalidBoolValue(LoadError):
    def __init__(self, key, index, value):
        super().__init__("BOOL tensor holds a value other than 0 / 1 (key=%s, index=%d): %d" % (key, index, value))
        self.key, self.index, self.value = key, index, value


class DataLengthMismatch(LoadError):
    def __init__(self, key, expected, actual):
        super().__init__("data length mismatch (key=%s): shape needs %d elements, data holds %d" % (key, expected, actual))
        self.key, self.expected, self.actual = key, expected, actual


class ShapeOverflow(LoadError):
    pass


# header name -> (element width, numpy dtype of the host array); bf16 and e4m3 are kept as raw bits
_REFERENCE_DTYPES = {"F32": (4, np.dtype("<f4")), "F16": (2, np.dtype("<f2")), "BF16": (2, np.dtype("<u2")),
                     "F64": (8, np.dtype("<f8")), "I32": (4, np.dtype("<i4")), "I64": (8, np.dtype("<i8")),
                     "BOOL": (1, np.dtype("u1"))}
_QUANTIZED_DTYPES = {"I8": (1, np.dtype("i1")), "F8_E4M3": (1, np.dtype("u1"))}
# widths of every dtype the wire format knows, for the layout check alone
_WIRE_WIDTH_BITS = {"BOOL": 8, "U8": 8, "I8": 8, "F8_E5M2": 8, "F8_E4M3": 8, "F8_E8M0": 8, "I16": 16, "U16": 16,
                    "F16": 16, "BF16": 16, "I32": 32, "U32": 32, "F32": 32, "C64": 64, "F64": 64, "I64": 64, "U64": 64,
                    "F4": 4, "F6_E2M3": 6, "F6_E3M2": 6}


class TypedTensor:
    """One tensor of a mixed-dtype file; ``data`` holds the file's bytes unchanged (bf16 / e4m3 as raw bit
    patterns in uint16 / uint8, BOOL as numpy bool)."""

    def __init__(self, dtype, shape, data):
        self.dtype, self.shape, self.data = dtype, tuple(shape), data

    def to_f32(self):
        """Explicit promotion (st_load.rs:369-391): F32 identity, F16 / BF16 exact, F64 / I64 / I32 rounded,
        BOOL 0 / 1."""
        if self.dtype == "BF16":
            return (self.data.astype(np.uint32) << 16).view(np.float32).reshape(self.shape)
        if self.dtype in _QUANTIZED_DTYPES:
            raise UnsupportedDtype("<to_f32>", self.dtype)
        return self.data.astype(np.float32).reshape(self.shape)


def _parse_layout(buf):
    """Header and byte ranges of every tensor, checked as safetensors' ``Metadata::validate`` checks them.
    Returns [(name, dtype_name, shape, begin, end)] with offsets relative to the start of the data section,
    and the data section's offset."""
    if len(buf) < 8:
        raise SafetensorsFormat("HeaderTooSmall")
    (n,) = struct.unpack("<Q", bytes(buf[:8]))
    if n > MAX_HEADER_BYTES:
        raise SafetensorsFormat("HeaderTooLarge")
    if 8 + n > len(buf):
        raise SafetensorsFormat("InvalidHeaderLength")
    raw = bytes(buf[8:8 + n])
    try:
        text = raw.decode("utf-8")
    except UnicodeDecodeError:
        raise SafetensorsFormat("InvalidHeader")
    if not text.startswith("{"):
        raise SafetensorsFormat("InvalidHeaderStart")
    try:
        header = json.loads(text)
    except ValueError as e:
        raise SafetensorsFormat("InvalidHeaderDeserialization: %s" % e)
    if not isinstance(header, dict):
        raise SafetensorsFormat("InvalidHeaderDeserialization: not an object")
    entries = []
    for name, info in header.items():
        if name == "__metadata__":
            if info is not None and not (isinstance(info, dict) and all(isinstance(v, str) for v in info.values())):
                raise SafetensorsFormat("InvalidHeaderDeserialization: __metadata__ must map strings to strings")
            continue
        try:
            dtype, shape, (begin, end) = info["dtype"], info["shape"], info["data_offsets"]
        except (KeyError, TypeError, ValueError):
            raise SafetensorsFormat("InvalidHeaderDeserialization: tensor %r" % name)
        if (not isinstance(dtype, str) or not isinstance(shape, list) or not all(isinstance(d, int) and d >= 0 for d in shape)
                or not isinstance(begin, int) or not isinstance(end, int)):
            raise SafetensorsFormat("InvalidHeaderDeserialization: tensor %r" % name)
        if dtype not in _WIRE_WIDTH_BITS:
            raise SafetensorsFormat("InvalidHeaderDeserialization: unknown dtype %r" % dtype)
        entries.append((name, dtype, shape, begin, end))
    entries.sort(key=lambda e: (e[3], e[4], e[0]))          # by byte range, as the wire format validates it
    data_len = len(buf) - 8 - n
    cursor = 0
    for name, dtype, shape, begin, end in entries:
        if begin != cursor or end < begin:
            raise SafetensorsFormat("InvalidOffset(%s)" % name)
        numel = 1
        for d in shape:
            numel *= d
            if numel > (1 << 64) - 1:
                raise SafetensorsFormat("ValidationOverflow")
        bits = numel * _WIRE_WIDTH_BITS[dtype]
        if bits % 8 != 0:
            raise SafetensorsFormat("MisalignedSlice")
        if bits // 8 != end - begin:
            raise SafetensorsFormat("TensorInvalidInfo(%s)" % name)
        cursor = end
    if cursor != data_len:
        raise SafetensorsFormat("MetadataIncompleteBuffer")
    return entries, 8 + n


def validate_safetensors_layout_from_bytes(buf):
    """Layout only, any dtype (st_load.rs:128-132)."""
    _parse_layout(memoryview(buf))


def load_safetensors_typed_from_bytes(buf, allow_quantized=False):
    """name -> TypedTensor (st_load.rs:433-559); tensors are visited in name order, so the first offending
    one reported is the alphabetically first."""
    view = memoryview(buf)
    entries, base = _parse_layout(view)
    out = {}
    for name, dtype, shape, begin, end in sorted(entries):
        spec = _REFERENCE_DTYPES.get(dtype) or (_QUANTIZED_DTYPES.get(dtype) if allow_quantized else None)
        if spec is None:
            raise UnsupportedDtype(name, dtype)
        width, np_dtype = spec
        expected = 1
        for d in shape:
            expected *= d
        if expected > (1 << 63) - 1:
            raise ShapeOverflow("element count overflows")
        nbytes = end - begin
        if nbytes % width != 0 or nbytes // width != expected:
            raise DataLengthMismatch(name, expected, nbytes // width)
        data = np.frombuffer(view[base + begin:base + end], dtype=np_dtype).reshape(shape)
        if dtype == "BOOL":
            bad = np.nonzero(data.ravel() > 1)[0]
            if bad.size:
                raise InvalidBoolValue(name, int(bad[0]), int(data.ravel()[bad[0]]))
            data = data.astype(np.bool_)
        out[name] = TypedTensor(dtype, shape, data)
    return out


def load_safetensors_typed(path, allow_quantized=False):
    try:
        with open(path, "rb") as f:
            buf = f.read()
    except OSError as e:
        raise Io(str(e))
    return load_safetensors_typed_from_bytes(buf, allow_quantized)


def load_safetensors_f32_from_bytes(buf):
    """name -> float32 array; anything but F32 is rejected (st_load.rs:144-192)."""
    view = memoryview(buf)
    entries, base = _parse_layout(view)
    out = {}
    for name, dtype, shape, begin, end in sorted(entries):
        if dtype != "F32":
            raise UnsupportedDtype(name, dtype)
        expected = int(np.prod(shape, dtype=object)) if shape else 1
        if (end - begin) % 4 != 0 or (end - begin) // 4 != expected:
            raise DataLengthMismatch(name, expected, (end - begin) // 4)
        out[name] = np.frombuffer(view[base + begin:base + end], dtype="<f4").reshape(shape)
    return out


def load_safetensors_f32(path):
    try:
        with open(path, "rb") as f:
            buf = f.read()
    except OSError as e:
        raise Io(str(e))
    return load_safetensors_f32_from_bytes(buf)


def require_keys(tensors, keys):
    """Every missing key at once, never only the first (st_load.rs:205-222)."""
    missing = [k for k in keys if k not in tensors]
    if missing:
        raise MissingKeys(missing)


require_keys_typed = require_keys


# ---- saving (crates/onnx-interop/src/st_save.rs) -----------------------------------------------------------

class SaveError(Exception):
    """st_save.rs:77-81"""


# the order in which the wire format's serializer lays tensors out: wider alignment first, then by name
_DTYPE_RANK = {n: i for i, n in enumerate(("BOOL", "U8", "I8", "F8_E5M2", "F8_E4M3", "I16", "U16", "F16", "BF16", "I32",
                                           "U32", "F32", "F64", "I64", "U64"))}
_NUMPY_TAGS = {np.dtype(np.float32): "F32", np.dtype(np.float16): "F16", np.dtype(np.float64): "F64",
               np.dtype(np.int32): "I32", np.dtype(np.int64): "I64", np.dtype(np.bool_): "BOOL"}


def _as_typed(key, t):
    if isinstance(t, TypedTensor):
        if t.dtype not in _REFERENCE_DTYPES and t.dtype not in _QUANTIZED_DTYPES:
            raise SaveError("%s: dtype %s cannot be written" % (key, t.dtype))
        return t
    a = np.asarray(t)
    tag = _NUMPY_TAGS.get(a.dtype)
    if tag is None:
        raise SaveError("%s: numpy dtype %s has no safetensors tag here (wrap bf16 bits in a TypedTensor)" % (key, a.dtype))
    return TypedTensor(tag, a.shape, a)


def save_safetensors_typed_to_bytes(tensors, metadata=None):
    """name -> TypedTensor (or a numpy array of a dtype the loader returns) -> file bytes, bit-identical to what
    the wire format's own serializer writes for the same tensors (st_save.rs:246-288 hands the sorted tensors
    to it): compact JSON header padded with spaces to a multiple of 8, tensors ordered by descending element
    alignment and then by name, data little-endian.  Nothing is transposed or renamed.  The output is
    deterministic.  metadata: optional str -> str map, written in sorted key order."""
    typed = {k: _as_typed(k, t) for k, t in tensors.items()}
    order = sorted(typed, key=lambda k: (-_DTYPE_RANK[typed[k].dtype], k))
    header, chunks, off = {}, [], 0
    if metadata:
        if not all(isinstance(k, str) and isinstance(v, str) for k, v in metadata.items()):
            raise SaveError("metadata must map strings to strings")
        header["__metadata__"] = {k: metadata[k] for k in sorted(metadata)}
    for k in order:
        t = typed[k]
        if k == "__metadata__":
            raise SaveError("__metadata__ is not a tensor name")
        width, npdt = (_REFERENCE_DTYPES.get(t.dtype) or _QUANTIZED_DTYPES[t.dtype])
        data = np.ascontiguousarray(t.data)
        if t.dtype == "BOOL":
            data = data.astype(np.uint8)
        if data.dtype.itemsize != width or int(np.prod(t.shape, dtype=np.int64)) != data.size:
            raise SaveError("%s: %s data of shape %s does not hold %d-byte elements of shape %s"
                            % (k, data.dtype, data.shape, width, t.shape))
        raw = data.astype(data.dtype.newbyteorder("<"), copy=False).tobytes()
        header[k] = {"dtype": t.dtype, "shape": [int(d) for d in t.shape], "data_offsets": [off, off + len(raw)]}
        chunks.append(raw)
        off += len(raw)
    h = json.dumps(header, separators=(",", ":"), ensure_ascii=False).encode("utf-8")
    h += b" " * (-len(h) % 8)
    return struct.pack("<Q", len(h)) + h + b"".join(chunks)


def save_safetensors_typed(path, tensors):
    """Writes through a temporary file in the same directory and a rename (st_save.rs:290-296): the final
    path never shows a partial file."""
    data = save_safetensors_typed_to_bytes(tensors)
    directory = os.path.dirname(os.path.abspath(path))
    tmp = os.path.join(directory, ".%s.%d.tmp" % (os.path.basename(path), os.getpid()))
    try:
        with open(tmp, "wb") as f:
            f.write(data)
        os.replace(tmp, path)
    except OSError as e:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise SaveError("io: %s" % e)


def save_safetensors_f32_to_bytes(tensors):
    """st_save.rs:118-190: float32 only."""
    for k, a in tensors.items():
        if np.asarray(a).dtype != np.float32:
            raise SaveError("%s: not float32" % k)
    return save_safetensors_typed_to_bytes(tensors)


def save_safetensors_f32(path, tensors):
    save_safetensors_f32_to_bytes(tensors)
    save_safetensors_typed(path, tensors)


class DeviceParamStore:
    """Parameters resident on the device in one flat f32 buffer; ``view(name)`` is a ``DeviceBufferView``
    (buffer, element offset, shape) into it.  Offsets are multiples of 64 elements so that vectorized
    kernels may read any parameter with 16-byte accesses."""

    ALIGN = 64

    def __init__(self, ops, tensors):
        """tensors: name -> float32 array (any shape); uploaded once, in name order."""
        self._ops = ops
        self.offsets, self.shapes = {}, {}
        total = 0
        for name in sorted(tensors):
            a = np.asarray(tensors[name])
            if a.dtype != np.float32:
                raise UnsupportedDtype(name, str(a.dtype))
            self.offsets[name], self.shapes[name] = total, tuple(a.shape)
            total += (a.size + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        self.buffer = ops.alloc_zeroed((max(total, 1),), capi.F32)
        for name in sorted(tensors):
            a = np.ascontiguousarray(tensors[name], dtype=np.float32)
            if a.size:
                ops.upload_into(a.ravel(), self.buffer, self.offsets[name])

    def view(self, name):
        return DeviceBufferView(self.buffer, self.offsets[name], self.shapes[name])

    def names(self):
        return sorted(self.offsets)

    def free(self):
        self.buffer.free()


def llama_decoder_keys(n_layers):
    """Tensor names of a Llama-style checkpoint as the Hugging Face exporters write them."""
    keys = ["model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"]
    for i in range(n_layers):
        p = "model.layers.%d." % i
        keys += [p + "input_layernorm.weight", p + "post_attention_layernorm.weight"]
        keys += [p + "self_attn.%s_proj.weight" % n for n in "qkvo"]
        keys += [p + "mlp.%s_proj.weight" % n for n in ("gate", "up", "down")]
    return keys


def llama_decoder_tensors(typed, n_layers):
    """Checks the key set and lays the checkpoint out as the decoder wants it: projection weights arrive as
    [out_features, in_features] and are transposed here, explicitly, to the [in, out] the linears multiply by;
    q | k | v and gate | up are concatenated along the output axis.  Returns name -> float32 array."""
    require_keys(typed, llama_decoder_keys(n_layers))

    def f32(key):
        return typed[key].to_f32()

    def t(key):
        w = f32(key)
        if w.ndim != 2:
            raise SafetensorsFormat("%s must be a matrix" % key)
        return np.ascontiguousarray(w.T)

    out = {"embed": f32("model.embed_tokens.weight"), "final_norm": f32("model.norm.weight"), "lm_head": t("lm_head.weight")}
    for i in range(n_layers):
        p, q = "model.layers.%d." % i, "layers.%d." % i
        out[q + "attn_norm"] = f32(p + "input_layernorm.weight")
        out[q + "ffn_norm"] = f32(p + "post_attention_layernorm.weight")
        out[q + "wqkv"] = np.concatenate([t(p + "self_attn.%s_proj.weight" % n) for n in "qkv"], axis=1)
        out[q + "wo"] = t(p + "self_attn.o_proj.weight")
        out[q + "wgu"] = np.concatenate([t(p + "mlp.gate_proj.weight"), t(p + "mlp.up_proj.weight")], axis=1)
        out[q + "wdown"] = t(p + "mlp.down_proj.weight")
    return out


def load_decoder(ops, checkpoint, n_layers, n_heads, n_kv_heads, max_blocks_per_seq, num_blocks, max_batch,
                 head_dim=128, block_size=16, rms_eps=1e-5, rope_theta=500000.0):
    """A resident ``Decoder`` from a Llama-style safetensors checkpoint (path or bytes): typed load, explicit
    transposes, one flat resident f32 parameter buffer, per-output-channel int8 quantization of every
    projection on the device.  Returns (decoder, store); the store may be freed once this returns (the
    quantized weights and the norm / embedding copies are the decoder's own)."""
    from .decoder import Decoder
    typed = load_safetensors_typed(checkpoint) if isinstance(checkpoint, str) else load_safetensors_typed_from_bytes(checkpoint)
    tensors = llama_decoder_tensors(typed, n_layers)
    vocab, d_model = tensors["embed"].shape
    d_ffn = tensors["layers.0.wdown"].shape[0]
    eq, ekv = n_heads * head_dim, n_kv_heads * head_dim
    expect = {"lm_head": (d_model, vocab), "final_norm": (d_model,)}
    for i in range(n_layers):
        q = "layers.%d." % i
        expect.update({q + "attn_norm": (d_model,), q + "ffn_norm": (d_model,), q + "wqkv": (d_model, eq + 2 * ekv),
                       q + "wo": (eq, d_model), q + "wgu": (d_model, 2 * d_ffn), q + "wdown": (d_ffn, d_model)})
    for name, shape in expect.items():
        if tensors[name].shape != shape:
            raise SafetensorsFormat("%s has shape %s, the configuration needs %s" % (name, tensors[name].shape, shape))
    store = DeviceParamStore(ops, tensors)
    dec = Decoder(ops, n_layers, d_model, n_heads, n_kv_heads, d_ffn, vocab, max_blocks_per_seq, num_blocks, max_batch,
                  head_dim, block_size, rms_eps, rope_theta)

    def own(name):                                        # norms and the embedding: buffers of the decoder's own
        return ops.upload(np.ascontiguousarray(tensors[name], dtype=np.float32))

    try:
        for i in range(n_layers):
            q = "layers.%d." % i
            dec.set_layer(i, own(q + "attn_norm"), own(q + "ffn_norm"), ops.quantize_weight(store.view(q + "wqkv")),
                          ops.quantize_weight(store.view(q + "wo")), ops.quantize_weight(store.view(q + "wgu")),
                          ops.quantize_weight(store.view(q + "wdown")))
        dec.set_head(own("embed"), own("final_norm"), ops.quantize_weight(store.view("lm_head")))
    except Exception:
        dec.close()
        store.free()
        raise
    return dec, store
