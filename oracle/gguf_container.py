"""CPU restatement of the reference's GGUF container writer and reader.  Test infrastructure only: the
test-suite compares the product's C++ container code (include/pmetal_gguf_file.hpp) with this, byte for byte;
the product never imports it.

Follows, function by function (paths under crates/pmetal-gguf/src/):
  ``GgufBuilder``                  writer.rs:14-538   ``write`` :180-224, ``validate`` :226-293,
                                   ``write_metadata_value[_data]`` :344-480, ``write_tensor_info`` :483-511,
                                   ``calculate_tensor_offsets`` :514-537, ``align_offset_checked`` :591-606
  ``read`` / ``read_tensor_data``  reader.rs:189-333, :371-407, ``read_string`` :446-479, ``read_value`` :493-560
  type table                       types.rs:16-187

What pins it without the reference running: the GGUF layout itself is fixed by the reference's own reader tests,
which assemble files byte by byte (reader.rs:631-666), by the writer tests (writer.rs:617-723: magic, version and
tensor count at fixed offsets, alignment examples 0/1/32/33 -> 0/32/32/64, row-major dimensions round trip, the four
rejections) and by a file whose every byte is derived by hand in tests/test_gguf_container.py.

Values are (type, payload) pairs: ``("u32", 7)``, ``("str", "x")``, ``("arr", [("i32", 1), ...])``.
"""
from __future__ import annotations

import struct

GGUF_MAGIC = 0x46554747  # types.rs:4
GGUF_VERSION = 3  # types.rs:7
GGUF_DEFAULT_ALIGNMENT = 32  # types.rs:10
MAX_STRING_LENGTH = 10 * 1024 * 1024  # reader.rs:58-77
MAX_ARRAY_LENGTH = 1_000_000
MAX_TENSOR_COUNT = 100_000
MAX_METADATA_COUNT = 100_000
MAX_TENSOR_DIMS = 16
MAX_ARRAY_DEPTH = 8  # reader.rs:485

# types.rs:193-220: value type name -> (id, struct format)
VALUE_TYPES = {
    "u8": (0, "<B"), "i8": (1, "<b"), "u16": (2, "<H"), "i16": (3, "<h"), "u32": (4, "<I"), "i32": (5, "<i"),
    "f32": (6, "<f"), "bool": (7, "<B"), "str": (8, None), "arr": (9, None), "u64": (10, "<Q"), "i64": (11, "<q"),
    "f64": (12, "<d"),
}
VALUE_NAMES = {v[0]: k for k, v in VALUE_TYPES.items()}

# types.rs:16-187: id -> (bytes per block, elements per block)
TYPE_TABLE = {
    0: (4, 1), 1: (2, 1), 2: (18, 32), 3: (20, 32), 6: (22, 32), 7: (24, 32), 8: (34, 32), 9: (36, 32),
    10: (84, 256), 11: (110, 256), 12: (144, 256), 13: (176, 256), 14: (210, 256), 15: (292, 256),
    16: (66, 256), 17: (74, 256), 18: (98, 256), 19: (50, 256), 20: (18, 32), 21: (110, 256), 22: (82, 256),
    23: (136, 256), 24: (1, 1), 25: (2, 1), 26: (4, 1), 27: (8, 1), 28: (8, 1), 29: (56, 256), 30: (2, 1),
    31: (18, 32), 32: (18, 32), 33: (18, 32), 34: (54, 256), 35: (66, 256), 36: (18, 32), 37: (18, 32),
    38: (18, 32), 39: (17, 32), 40: (36, 64), 41: (18, 128),
}


class InvalidArgument(ValueError):
    """PMetalError::InvalidArgument"""


class GgufReadError(ValueError):
    """reader.rs:80-170; ``kind`` is the variant name."""

    def __init__(self, kind: str, message: str = ""):
        super().__init__(f"{kind}: {message}" if message else kind)
        self.kind = kind


def tensor_size(dtype: int, n_elements: int) -> int:  # types.rs:173-177
    type_size, block = TYPE_TABLE[dtype]
    return -(-n_elements // block) * type_size


def align_offset(offset: int, alignment: int) -> int:  # writer.rs:591-606
    if alignment == 0:
        raise InvalidArgument("GGUF alignment must be greater than zero")
    rem = offset % alignment
    out = offset if rem == 0 else offset + (alignment - rem)
    if out >= 1 << 64:
        raise InvalidArgument("GGUF aligned offset overflows u64")
    return out


class GgufBuilder:
    """writer.rs:14-538.  ``dimensions`` are row-major; tensor data are bytes."""

    def __init__(self):  # :33-50
        self.metadata = {}
        self.tensors = []  # (name, dimensions, dtype id, bytes)
        self._alignment = GGUF_DEFAULT_ALIGNMENT
        self.add_metadata("general.alignment", ("u32", GGUF_DEFAULT_ALIGNMENT))
        self.add_metadata("general.quantization_version", ("u32", 2))

    @classmethod
    def with_model(cls, architecture: str, name: str):  # :53-64
        b = cls()
        b.add_metadata("general.architecture", ("str", architecture))
        b.add_metadata("general.name", ("str", name))
        return b

    def alignment(self, alignment: int):  # :67-74
        self._alignment = alignment
        self.metadata["general.alignment"] = ("u32", alignment)
        return self

    def add_metadata(self, key: str, value):  # :77-80
        self.metadata[key] = value
        return self

    def add_raw_tensor(self, name: str, dimensions, dtype: int, data: bytes):  # :167-177
        self.tensors.append((name, list(dimensions), dtype, bytes(data)))
        return self

    # ---- :226-293 ----
    def validate(self):
        if self._alignment == 0 or self._alignment > 1_048_576:
            raise InvalidArgument(f"GGUF alignment must be in 1..=1048576, got {self._alignment}")
        for key, value in self.metadata.items():
            if len(key.encode()) > MAX_STRING_LENGTH:
                raise InvalidArgument("GGUF metadata key too long")
            _validate_value(value)
        names = set()
        for name, dims, dtype, data in self.tensors:
            if name in names:
                raise InvalidArgument(f"Duplicate GGUF tensor name: {name}")
            names.add(name)
            if len(name.encode()) > MAX_STRING_LENGTH:
                raise InvalidArgument("GGUF tensor name too long")
            if len(dims) > MAX_TENSOR_DIMS:
                raise InvalidArgument(f"GGUF tensor {name} has {len(dims)} dimensions")
            n = 1
            for d in dims:
                n *= d
            if n >= 1 << 64 or tensor_size(dtype, n) >= 1 << 64:
                raise InvalidArgument(f"GGUF tensor {name} has invalid dimensions or dtype")
            if tensor_size(dtype, n) != len(data):
                raise InvalidArgument(f"GGUF tensor {name} has {len(data)} bytes but requires {tensor_size(dtype, n)}")

    # ---- :180-224 ----
    def build_to_bytes(self) -> bytes:
        self.validate()
        out = bytearray()
        out += struct.pack("<IIQQ", GGUF_MAGIC, GGUF_VERSION, len(self.tensors), len(self.metadata))  # :303-327
        # BTreeMap<String, _> iterates in byte-wise key order
        for key in sorted(self.metadata, key=lambda k: k.encode()):
            out += _string(key)
            value = self.metadata[key]
            out += struct.pack("<I", VALUE_TYPES[value[0]][0])  # :346-351
            out += _value_data(value)
        offset = 0  # :514-537
        for name, dims, dtype, data in self.tensors:
            out += _string(name)  # :483-511
            out += struct.pack("<I", len(dims))
            for d in reversed(dims):
                out += struct.pack("<Q", d)
            out += struct.pack("<IQ", dtype, offset)
            offset = align_offset(offset + len(data), self._alignment)
        out += bytes(align_offset(len(out), self._alignment) - len(out))
        for i, (_, _, _, data) in enumerate(self.tensors):
            out += data
            if i < len(self.tensors) - 1:  # :213-220: nothing behind the last tensor
                out += bytes(align_offset(len(out), self._alignment) - len(out))
        return bytes(out)


def _string(s: str) -> bytes:  # :330-341
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _validate_array(arr):  # :559-576
    if len(arr) > MAX_ARRAY_LENGTH:
        raise InvalidArgument(f"GGUF metadata array has {len(arr)} elements")
    if arr and any(e[0] != arr[0][0] for e in arr):
        raise InvalidArgument("GGUF metadata arrays must contain a single value type")


def _validate_value(value):  # :540-557
    kind, payload = value
    if kind == "str" and len(payload.encode()) > MAX_STRING_LENGTH:
        raise InvalidArgument("GGUF string metadata value too long")
    if kind == "arr":
        _validate_array(payload)
        for e in payload:
            _validate_value(e)


def _value_data(value) -> bytes:  # :418-480 (and the value part of :353-413)
    kind, payload = value
    if kind == "str":
        return _string(payload)
    if kind == "arr":
        _validate_array(payload)
        elem_type = VALUE_TYPES[payload[0][0]][0] if payload else 0  # empty array: Uint8 (:393-396)
        return struct.pack("<IQ", elem_type, len(payload)) + b"".join(_value_data(e) for e in payload)
    if kind == "bool":
        return struct.pack("<B", 1 if payload else 0)
    return struct.pack(VALUE_TYPES[kind][1], payload)


# ------------------------------------------------------------------------------------------------
# reader.rs
# ------------------------------------------------------------------------------------------------
class _Cursor:
    def __init__(self, data: bytes):
        self.data, self.pos = data, 0

    def take(self, fmt: str):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.data):
            raise GgufReadError("Io", "failed to fill whole buffer")
        (v,) = struct.unpack_from(fmt, self.data, self.pos)
        self.pos += size
        return v

    def raw(self, n: int) -> bytes:
        if self.pos + n > len(self.data):
            raise GgufReadError("Io", "failed to fill whole buffer")
        b = self.data[self.pos:self.pos + n]
        self.pos += n
        return b


def _read_string(c: _Cursor, v1: bool) -> str:  # :446-479
    n = c.take("<I") if v1 else c.take("<Q")
    if n > MAX_STRING_LENGTH:
        raise GgufReadError("StringTooLarge", str(n))
    b = c.raw(n).rstrip(b"\x00")
    try:
        return b.decode("utf-8")
    except UnicodeDecodeError:
        raise GgufReadError("InvalidUtf8") from None


def _read_value(c: _Cursor, vt: int, v1: bool, depth: int):  # :493-560
    if vt not in VALUE_NAMES:
        raise GgufReadError("InvalidValueType", str(vt))
    kind = VALUE_NAMES[vt]
    if kind == "str":
        return ("str", _read_string(c, v1))
    if kind == "arr":
        if depth >= MAX_ARRAY_DEPTH:
            raise GgufReadError("ArrayNestingTooDeep")
        et = c.take("<I")
        n = c.take("<I") if v1 else c.take("<Q")
        if n > MAX_ARRAY_LENGTH:
            raise GgufReadError("ArrayTooLarge", str(n))
        return ("arr", [_read_value(c, et, v1, depth + 1) for _ in range(n)])
    v = c.take(VALUE_TYPES[kind][1])
    return (kind, bool(v)) if kind == "bool" else (kind, v)


class GgufContent:
    """reader.rs:176-444"""

    def __init__(self):
        self.version = 0
        self.metadata = {}
        self.tensor_infos = {}  # name -> dict(dimensions (row-major), dtype, offset)
        self.tensor_order = []
        self.tensor_data_offset = 0

    @classmethod
    def read(cls, data: bytes):  # :189-333
        c, g = _Cursor(data), cls()
        magic = c.take("<I")
        if magic != GGUF_MAGIC:
            raise GgufReadError("InvalidMagic", hex(magic))
        g.version = c.take("<I")
        if g.version not in (1, 2, 3):
            raise GgufReadError("UnsupportedVersion", str(g.version))
        v1 = g.version == 1
        n_tensors = c.take("<I") if v1 else c.take("<Q")
        n_kv = c.take("<I") if v1 else c.take("<Q")
        if n_tensors > MAX_TENSOR_COUNT:
            raise GgufReadError("TooManyTensors", str(n_tensors))
        if n_kv > MAX_METADATA_COUNT:
            raise GgufReadError("TooManyMetadata", str(n_kv))
        for _ in range(n_kv):
            key = _read_string(c, v1)
            value = _read_value(c, c.take("<I"), v1, 0)
            if key in g.metadata:
                raise GgufReadError("DuplicateMetadataKey", key)
            g.metadata[key] = value
        for _ in range(n_tensors):
            name = _read_string(c, v1)
            n_dims = c.take("<I")
            if n_dims > MAX_TENSOR_DIMS:
                raise GgufReadError("TooManyTensorDimensions", name)
            dims = [c.take("<I") if v1 else c.take("<Q") for _ in range(n_dims)]
            dims.reverse()  # fastest axis first on disk
            dtype = c.take("<I")
            if dtype not in TYPE_TABLE:
                raise GgufReadError("InvalidDtype", str(dtype))
            offset = c.take("<Q")
            n = 1
            for d in dims:
                n *= d
            if n >= 1 << 64 or tensor_size(dtype, n) >= 1 << 64:
                raise GgufReadError("IntegerOverflow")
            if name in g.tensor_infos:
                raise GgufReadError("DuplicateTensorName", name)
            g.tensor_infos[name] = dict(dimensions=dims, dtype=dtype, offset=offset)
            g.tensor_order.append(name)
        alignment = GGUF_DEFAULT_ALIGNMENT  # :305-312
        a = g.metadata.get("general.alignment")
        if a is not None and a[0] in ("u32", "u64"):
            alignment = a[1]
        if alignment == 0 or alignment > 1_048_576:
            raise GgufReadError("InvalidAlignment", str(alignment))
        g.tensor_data_offset = align_offset(c.pos, alignment)
        return g

    def read_tensor_data(self, data: bytes, name: str) -> bytes:  # :371-407
        if name not in self.tensor_infos:
            raise GgufReadError("TensorNotFound", name)
        info = self.tensor_infos[name]
        n = 1
        for d in info["dimensions"]:
            n *= d
        size = tensor_size(info["dtype"], n)
        begin = self.tensor_data_offset + info["offset"]
        if begin + size > len(data):
            raise GgufReadError("Io", "failed to fill whole buffer")
        return data[begin:begin + size]


# crates/pmetal-models/src/weight_format.rs:389-435
_HF_SUFFIX = {
    "input_layernorm.weight": "attn_norm.weight", "self_attn.q_proj.weight": "attn_q.weight",
    "self_attn.k_proj.weight": "attn_k.weight", "self_attn.v_proj.weight": "attn_v.weight",
    "self_attn.o_proj.weight": "attn_output.weight", "post_attention_layernorm.weight": "ffn_norm.weight",
    "mlp.gate.weight": "ffn_gate_inp.weight", "mlp.router.weight": "ffn_gate_inp.weight",
    "mlp.gate_proj.weight": "ffn_gate.weight", "mlp.up_proj.weight": "ffn_up.weight",
    "mlp.down_proj.weight": "ffn_down.weight", "mlp.experts.gate_proj.weight": "ffn_gate_exps.weight",
    "mlp.experts.up_proj.weight": "ffn_up_exps.weight", "mlp.experts.down_proj.weight": "ffn_down_exps.weight",
    "mlp.shared_expert.gate_proj.weight": "ffn_gate_shexp.weight", "mlp.shared_expert.up_proj.weight": "ffn_up_shexp.weight",
    "mlp.shared_expert.down_proj.weight": "ffn_down_shexp.weight",
    "mlp.shared_experts.gate_proj.weight": "ffn_gate_shexp.weight", "mlp.shared_experts.up_proj.weight": "ffn_up_shexp.weight",
    "mlp.shared_experts.down_proj.weight": "ffn_down_shexp.weight",
    "mlp.shared_expert_gate.weight": "ffn_gate_inp_shexp.weight", "self_attn.q_norm.weight": "attn_q_norm.weight",
    "self_attn.k_norm.weight": "attn_k_norm.weight",
}


def hf_to_gguf_name(hf_name: str) -> str:
    top = {"model.embed_tokens.weight": "token_embd.weight", "model.norm.weight": "output_norm.weight",
           "lm_head.weight": "output.weight"}
    if hf_name in top:
        return top[hf_name]
    if not hf_name.startswith("model.layers."):
        return hf_name
    rest = hf_name[len("model.layers."):]
    if "." not in rest:
        return hf_name
    layer, suffix = rest.split(".", 1)
    # usize::from_str: decimal digits with an optional leading '+'
    digits = layer[1:] if layer.startswith("+") else layer
    if not digits or not all("0" <= ch <= "9" for ch in digits) or int(digits) >= 1 << 64:
        return hf_name
    return f"blk.{layer}.{_HF_SUFFIX.get(suffix, suffix)}"


# crates/pmetal-models/src/weight_format.rs:332-386
_GGUF_SUFFIX = {
    "attn_norm.weight": "input_layernorm.weight", "attn_q.weight": "self_attn.q_proj.weight",
    "attn_k.weight": "self_attn.k_proj.weight", "attn_v.weight": "self_attn.v_proj.weight",
    "attn_output.weight": "self_attn.o_proj.weight", "ffn_norm.weight": "post_attention_layernorm.weight",
    "ffn_gate.weight": "mlp.gate_proj.weight", "ffn_up.weight": "mlp.up_proj.weight", "ffn_down.weight": "mlp.down_proj.weight",
    "ffn_gate_inp.weight": "mlp.gate.weight", "ffn_gate_exps.weight": "mlp.experts.gate_proj.weight",
    "ffn_up_exps.weight": "mlp.experts.up_proj.weight", "ffn_down_exps.weight": "mlp.experts.down_proj.weight",
    "ffn_gate_shexp.weight": "mlp.shared_expert.gate_proj.weight", "ffn_up_shexp.weight": "mlp.shared_expert.up_proj.weight",
    "ffn_down_shexp.weight": "mlp.shared_expert.down_proj.weight", "ffn_gate_inp_shexp.weight": "mlp.shared_expert_gate.weight",
    "attn_q_norm.weight": "self_attn.q_norm.weight", "attn_k_norm.weight": "self_attn.k_norm.weight",
}


def gguf_to_hf_name(gguf_name: str) -> str:
    top = {"token_embd.weight": "model.embed_tokens.weight", "output_norm.weight": "model.norm.weight",
           "output.weight": "lm_head.weight"}
    if gguf_name in top:
        return top[gguf_name]
    if gguf_name.startswith("blk."):
        parts = gguf_name.split(".", 2)  # splitn(3, '.')
        if len(parts) >= 3:
            return f"model.layers.{parts[1]}.{_GGUF_SUFFIX.get(parts[2], parts[2])}"
    return gguf_name


def load_gguf(data: bytes, dequantize, supported):
    """WeightLoader::load_gguf (weight_format.rs:258-313) over a file image: {hugging face name: (shape, f32 values)} of
    every tensor whose type ``supported(dtype)`` accepts, decoded by ``dequantize(raw bytes, dtype, shape)``; a dimension
    beyond i32 is an error (:142-153).  Returns the dict and the names skipped."""
    content = GgufContent.read(data)
    weights, skipped = {}, []
    for name in content.tensor_order:
        info = content.tensor_infos[name]
        if not supported(info["dtype"]):
            skipped.append(name)
            continue
        for d in info["dimensions"]:
            if d > 2**31 - 1:
                raise ValueError(f"Tensor {name} dimension {d} exceeds MLX i32 shape limits")
        shape = list(info["dimensions"])
        weights[gguf_to_hf_name(name)] = (shape, dequantize(content.read_tensor_data(data, name), info["dtype"], shape))
    return weights, skipped
