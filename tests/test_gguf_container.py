"""The GGUF container beside the quantizer: the C++ writer / reader (include/pmetal_gguf_file.hpp) against the
oracle's restatement (oracle/gguf_container.py), the oracle against what pins it, and -- on the GPU -- the Q4_K_M
model driver (quantize_model_q4_k_m) against oracle quantizer + oracle writer, byte for byte."""
import os
import struct
import subprocess

import numpy as np
import pytest

from oracle import gguf_container as og

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cpp", "test_gguf_file.cpp")
LIBDIR = os.path.join(ROOT, "pmetal_amd")


@pytest.fixture(scope="module")
def host_exe(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("gguf") / "test_gguf_file_host")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-DPMETAL_TEST_HOST_ONLY", "-I", os.path.join(ROOT, "include"),
                    SRC, "-o", exe], check=True)
    return exe


def hx(s) -> str:
    b = s.encode() if isinstance(s, str) else s
    return b.hex() or "-"


def tensor_bytes(seed: int, n: int) -> bytes:
    i = np.arange(n, dtype=np.uint64)
    return ((np.uint64(seed * 131) + i * np.uint64(7) + (i >> np.uint64(8))) & np.uint64(0xFF)).astype(np.uint8).tobytes()


def spec_value(v) -> str:
    kind, payload = v
    if kind == "arr":
        return " ".join(["arr", str(len(payload))] + [spec_value(e) for e in payload])
    if kind == "str":
        return f"str {hx(payload)}"
    if kind == "f32":
        return f"f32 {struct.unpack('<I', struct.pack('<f', payload))[0]}"
    if kind == "f64":
        return f"f64 {struct.unpack('<Q', struct.pack('<d', payload))[0]}"
    if kind == "bool":
        return f"bool {1 if payload else 0}"
    return f"{kind} {payload}"


def write_spec(path, scenario):
    lines = []
    if "align" in scenario:
        lines.append(f"align {scenario['align']}")
    for key, value in scenario.get("meta", []):
        lines.append(f"meta {hx(key)} {spec_value(value)}")
    for name, dtype, dims, seed in scenario.get("tensors", []):
        lines.append(f"tensor {hx(name)} {dtype} {len(dims)} {' '.join(map(str, dims))} {seed}")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def oracle_build(scenario) -> bytes:
    b = og.GgufBuilder()
    if "align" in scenario:
        b.alignment(scenario["align"])
    for key, value in scenario.get("meta", []):
        b.add_metadata(key, value)
    for name, dtype, dims, seed in scenario.get("tensors", []):
        n = int(np.prod(dims, dtype=np.uint64)) if dims else 1
        b.add_raw_tensor(name, dims, dtype, tensor_bytes(seed, og.tensor_size(dtype, n)))
    return b.build_to_bytes()


def oracle_dump(data: bytes) -> str:
    c = og.GgufContent.read(data)
    out = [f"version {c.version}", f"data_offset {c.tensor_data_offset}"]
    for key in sorted(c.metadata, key=lambda k: k.encode()):
        out.append(f"meta {hx(key)} {spec_value(c.metadata[key])}")
    for name in c.tensor_order:
        t = c.tensor_infos[name]
        raw = c.read_tensor_data(data, name)
        h = 1469598103934665603
        for byte in raw:
            h = ((h ^ byte) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
        dims = "".join(f" {d}" for d in t["dimensions"])
        out.append(f"tensor {hx(name)} {t['dtype']} {len(t['dimensions'])}{dims} offset {t['offset']} bytes {len(raw)} fnv {h}")
    return "\n".join(out) + "\n"


SCENARIOS = {
    "empty": {},
    "model_header": {"meta": [("general.architecture", ("str", "llama")), ("general.name", ("str", "quantized-model"))]},
    "every_value_type": {"meta": [
        ("k.u8", ("u8", 255)), ("k.i8", ("i8", -128)), ("k.u16", ("u16", 65535)), ("k.i16", ("i16", -32768)),
        ("k.u32", ("u32", 4294967295)), ("k.i32", ("i32", -2147483648)), ("k.u64", ("u64", 2**64 - 1)),
        ("k.i64", ("i64", -2**63)), ("k.f32", ("f32", 1.5)), ("k.f64", ("f64", -2.25)), ("k.t", ("bool", True)),
        ("k.f", ("bool", False)), ("k.str", ("str", "héllo wörld ✓")), ("k.empty_str", ("str", "")),
        ("k.empty_arr", ("arr", [])), ("k.ints", ("arr", [("i32", v) for v in (-1, 0, 7)])),
        ("k.floats", ("arr", [("f32", 0.5), ("f32", -0.0)])),
        ("k.strings", ("arr", [("str", "hello"), ("str", ""), ("str", "world")])),
        ("k.nested", ("arr", [("arr", [("u8", 1), ("u8", 2)]), ("arr", []), ("arr", [("u8", 3)])])),
        # BTreeMap order is byte order: upper case before lower case, "a.b" before "a/b" before "ab"
        ("Zebra", ("u32", 1)), ("a/b", ("u32", 2)), ("a.b", ("u32", 3)), ("ab", ("u32", 4)), ("é", ("u32", 5)),
    ]},
    "tensors_default_alignment": {"tensors": [
        ("blk.0.attn_q.weight", 12, [4, 512], 1), ("blk.0.attn_v.weight", 14, [3, 256], 2),
        ("blk.0.attn_norm.weight", 1, [5], 3), ("scalar", 0, [], 4), ("blk.0.ffn_up.weight", 8, [2, 3, 32], 5),
        ("last.weight", 0, [7], 6),
    ]},
    "alignment_1": {"align": 1, "tensors": [("a", 24, [3], 1), ("b", 24, [5], 2)]},
    "alignment_4096": {"align": 4096, "tensors": [("a", 24, [3], 1), ("b", 25, [5], 2), ("c", 0, [1, 1], 3)]},
    "exact_multiple": {"tensors": [("a", 0, [8], 1), ("b", 0, [16], 2)]},  # 32 and 64 bytes: no padding between
    "zero_elements": {"tensors": [("none", 0, [0, 4], 1), ("some", 0, [2], 2)]},
    "alignment_replaced_by_metadata": {"align": 64, "meta": [("general.alignment", ("u32", 16))],
                                       "tensors": [("a", 24, [3], 1), ("b", 24, [5], 2)]},
}


def test_oracle_against_a_file_derived_by_hand():
    """Every byte of a small file, written out from the GGUF layout: header (magic, version 3, counts as u64), the four
    default keys in byte order, one tensor info with its dimensions reversed, padding to 32, the data."""
    b = og.GgufBuilder.with_model("llama", "t")
    b.add_raw_tensor("w", [2, 3], 0, struct.pack("<6f", 1, 2, 3, 4, 5, 6))
    got = b.build_to_bytes()

    def s(x):
        return struct.pack("<Q", len(x)) + x

    want = b"GGUF" + struct.pack("<I", 3) + struct.pack("<QQ", 1, 4)
    want += s(b"general.alignment") + struct.pack("<II", 4, 32)
    want += s(b"general.architecture") + struct.pack("<I", 8) + s(b"llama")
    want += s(b"general.name") + struct.pack("<I", 8) + s(b"t")
    want += s(b"general.quantization_version") + struct.pack("<II", 4, 2)
    want += s(b"w") + struct.pack("<I", 2) + struct.pack("<QQ", 3, 2) + struct.pack("<I", 0) + struct.pack("<Q", 0)
    assert len(want) == 220
    want += bytes(4) + struct.pack("<6f", 1, 2, 3, 4, 5, 6)
    assert got == want and len(got) == 248


def test_oracle_reference_unit_tests():
    """writer.rs:617-723 and reader.rs:631-669, restated against the oracle."""
    bytes_ = og.GgufBuilder.with_model("llama", "test-model").build_to_bytes()
    assert bytes_[0:4] == struct.pack("<I", og.GGUF_MAGIC) and bytes_[4:8] == struct.pack("<I", og.GGUF_VERSION)
    b = og.GgufBuilder.with_model("llama", "test-model")
    b.add_raw_tensor("test.weight", [2, 3], 0, struct.pack("<6f", 1, 2, 3, 4, 5, 6))
    bytes_ = b.build_to_bytes()
    assert struct.unpack("<Q", bytes_[8:16])[0] == 1
    assert og.GgufContent.read(bytes_).tensor_infos["test.weight"]["dimensions"] == [2, 3]
    assert [og.align_offset(v, 32) for v in (0, 1, 32, 33)] == [0, 32, 32, 64]
    with pytest.raises(og.InvalidArgument):
        og.GgufBuilder.with_model("llama", "test-model").alignment(0).build_to_bytes()
    with pytest.raises(og.InvalidArgument):
        og.GgufBuilder().add_metadata("bad.array", ("arr", [("u32", 1), ("str", "two")])).build_to_bytes()
    with pytest.raises(og.InvalidArgument):
        og.GgufBuilder().add_raw_tensor("bad.weight", [2], 0, bytes(4)).build_to_bytes()
    with pytest.raises(og.InvalidArgument):
        og.GgufBuilder().add_raw_tensor("dup", [1], 0, bytes(4)).add_raw_tensor("dup", [1], 0, bytes(4)).build_to_bytes()

    def s(x):
        return struct.pack("<Q", len(x)) + x

    dup = struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 0, 2) + (s(b"dup") + struct.pack("<II", 4, 1)) + (s(b"dup") + struct.pack("<II", 4, 2))
    with pytest.raises(og.GgufReadError) as e:
        og.GgufContent.read(dup)
    assert e.value.kind == "DuplicateMetadataKey"
    rank = struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 1, 0) + s(b"bad.weight") + struct.pack("<I", og.MAX_TENSOR_DIMS + 1)
    with pytest.raises(og.GgufReadError) as e:
        og.GgufContent.read(rank)
    assert e.value.kind == "TooManyTensorDimensions"


def test_cpp_reference_unit_tests(host_exe):
    r = subprocess.run([host_exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.parametrize("name", sorted(SCENARIOS))
def test_cpp_writer_equals_oracle_and_readers_agree(host_exe, tmp_path, name):
    scenario = SCENARIOS[name]
    spec, out = str(tmp_path / "spec.txt"), str(tmp_path / "out.gguf")
    write_spec(spec, scenario)
    r = subprocess.run([host_exe, "--build", spec, out], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    want = oracle_build(scenario)
    got = open(out, "rb").read()
    assert got == want, f"{name}: first difference at byte {next(i for i, (a, b) in enumerate(zip(got, want)) if a != b) if len(got) == len(want) else (len(got), len(want))}"
    # the C++ reader on the file and the oracle reader on the same bytes print the same thing
    r = subprocess.run([host_exe, "--dump", out], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout == oracle_dump(want)
    assert "MISMATCH" not in r.stdout


def test_random_scenarios(host_exe, tmp_path):
    rng = np.random.default_rng(11)
    kinds = ["u8", "i8", "u16", "i16", "u32", "i32", "u64", "i64", "f32", "f64", "bool", "str"]
    ranges = {"u8": (0, 2**8), "i8": (-2**7, 2**7), "u16": (0, 2**16), "i16": (-2**15, 2**15), "u32": (0, 2**32),
              "i32": (-2**31, 2**31), "u64": (0, 2**63), "i64": (-2**62, 2**62)}

    def scalar(kind):
        if kind in ranges:
            return (kind, int(rng.integers(*ranges[kind])))
        if kind == "f32":
            return ("f32", float(np.float32(rng.standard_normal())))
        if kind == "f64":
            return ("f64", float(rng.standard_normal()))
        if kind == "bool":
            return ("bool", bool(rng.integers(0, 2)))
        return ("str", "".join(chr(int(c)) for c in rng.integers(32, 0x2FF, int(rng.integers(0, 12)))))

    for case in range(12):
        meta = []
        for k in range(int(rng.integers(0, 12))):
            kind = kinds[int(rng.integers(len(kinds)))]
            if rng.random() < 0.3:
                value = ("arr", [scalar(kind) for _ in range(int(rng.integers(0, 6)))])
            else:
                value = scalar(kind)
            meta.append((f"key.{case}.{int(rng.integers(1000))}.{k}", value))
        tensors = []
        for t in range(int(rng.integers(0, 6))):
            dtype = int(rng.choice([0, 1, 8, 12, 14, 24, 30]))
            dims = [int(d) for d in rng.integers(1, 40, int(rng.integers(1, 4)))]
            tensors.append((f"t{t}.weight", dtype, dims, int(rng.integers(1, 1000))))
        scenario = {"align": int(rng.choice([1, 8, 32, 64, 256])), "meta": meta, "tensors": tensors}
        spec, out = str(tmp_path / f"spec{case}.txt"), str(tmp_path / f"out{case}.gguf")
        write_spec(spec, scenario)
        r = subprocess.run([host_exe, "--build", spec, out], capture_output=True, text=True)
        assert r.returncode == 0, r.stdout + r.stderr
        want = oracle_build(scenario)
        assert open(out, "rb").read() == want, case
        r = subprocess.run([host_exe, "--dump", out], capture_output=True, text=True)
        assert r.stdout == oracle_dump(want), case


def test_writer_rejections_agree(host_exe, tmp_path):
    bad = {
        "alignment_zero": {"align": 0},
        "alignment_too_large": {"align": 1048577},
        "mixed_array": {"meta": [("bad", ("arr", [("u32", 1), ("str", "two")]))]},
        "duplicate_tensor": {"tensors": [("dup", 0, [1], 1), ("dup", 0, [2], 2)]},
        "rank_17": {"tensors": [("deep", 24, [1] * 17, 1)]},
    }
    for name, scenario in bad.items():
        with pytest.raises(og.InvalidArgument):
            oracle_build(scenario)
        spec, out = str(tmp_path / f"{name}.txt"), str(tmp_path / f"{name}.gguf")
        write_spec(spec, scenario)
        r = subprocess.run([host_exe, "--build", spec, out], capture_output=True, text=True)
        assert r.returncode == 3 and "InvalidArgument" in r.stdout, (name, r.stdout, r.stderr)


def test_reader_errors_agree(host_exe, tmp_path):
    def s(x, v1=False):
        return struct.pack("<I" if v1 else "<Q", len(x)) + x

    good = oracle_build(SCENARIOS["tensors_default_alignment"])
    head = struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 0, 1)
    nested = struct.pack("<I", 9) + struct.pack("<IQ", 9, 1) * 8 + struct.pack("<IQ", 4, 0)  # eight arrays deep
    cases = {
        "bad_magic": b"GGUG" + good[4:],
        "version_4": good[:4] + struct.pack("<I", 4) + good[8:],
        "truncated_header": good[:20],
        "truncated_infos": good[:120],
        "too_many_tensors": struct.pack("<IIQQ", og.GGUF_MAGIC, 3, og.MAX_TENSOR_COUNT + 1, 0),
        "too_many_metadata": struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 0, og.MAX_METADATA_COUNT + 1),
        "bad_value_type": head + s(b"k") + struct.pack("<I", 13),
        "string_too_large": head + struct.pack("<Q", og.MAX_STRING_LENGTH + 1),
        "array_too_large": head + s(b"k") + struct.pack("<IIQ", 9, 4, og.MAX_ARRAY_LENGTH + 1),
        "nested_nine_deep": head + s(b"k") + struct.pack("<I", 9) + struct.pack("<IQ", 9, 1) * 8 + struct.pack("<IQ", 4, 0),
        "nested_eight_deep_is_fine": head + s(b"k") + nested[:4] + struct.pack("<IQ", 9, 1) * 7 + struct.pack("<IQ", 4, 0),
        "invalid_utf8": head + s(b"\xff\xfe") + struct.pack("<II", 4, 1),
        "overlong_utf8": head + s(b"\xc0\xaf") + struct.pack("<II", 4, 1),
        "surrogate_utf8": head + s(b"\xed\xa0\x80") + struct.pack("<II", 4, 1),
        "bad_dtype": struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 1, 0) + s(b"w") + struct.pack("<IQIQ", 1, 4, 4, 0),
        "size_overflow": struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 1, 0) + s(b"w") + struct.pack("<IQQIQ", 2, 2**40, 2**40, 0, 0),
        "duplicate_tensor": struct.pack("<IIQQ", og.GGUF_MAGIC, 3, 2, 0) + (s(b"w") + struct.pack("<IQIQ", 1, 4, 0, 0)) * 2,
        "alignment_zero": head + s(b"general.alignment") + struct.pack("<II", 4, 0),
        "alignment_u64": head + s(b"general.alignment") + struct.pack("<IQ", 10, 128),
        "alignment_as_string_is_ignored": head + s(b"general.alignment") + struct.pack("<I", 8) + s(b"64"),
        "trailing_nulls_in_key": head + s(b"key\x00\x00") + struct.pack("<II", 4, 9),
        "version_1_counts_and_strings_are_u32": struct.pack("<IIII", og.GGUF_MAGIC, 1, 1, 1) + s(b"k", True) + struct.pack("<II", 4, 7)
        + s(b"w", True) + struct.pack("<IIIIQ", 2, 3, 2, 0, 0) + bytes(64),
        "version_2": good[:4] + struct.pack("<I", 2) + good[8:],
    }
    for name, data in cases.items():
        try:
            og.GgufContent.read(data)
            want = "none"
        except og.GgufReadError as e:
            want = e.kind
        path = str(tmp_path / f"{name}.gguf")
        open(path, "wb").write(data)
        r = subprocess.run([host_exe, "--read-error", path], capture_output=True, text=True)
        assert r.returncode == 0 and r.stdout.strip() == want, (name, want, r.stdout, r.stderr)
        if want == "none":
            r = subprocess.run([host_exe, "--dump", path], capture_output=True, text=True)
            assert r.stdout == oracle_dump(data), name
    expected_kinds = {"bad_magic": "InvalidMagic", "version_4": "UnsupportedVersion", "truncated_header": "Io",
                      "nested_nine_deep": "ArrayNestingTooDeep", "nested_eight_deep_is_fine": "none",
                      "overlong_utf8": "InvalidUtf8", "size_overflow": "IntegerOverflow", "alignment_zero": "InvalidAlignment",
                      "version_1_counts_and_strings_are_u32": "none", "alignment_as_string_is_ignored": "none"}
    for name, kind in expected_kinds.items():  # the oracle's own answers, spelled out
        try:
            og.GgufContent.read(cases[name])
            got = "none"
        except og.GgufReadError as e:
            got = e.kind
        assert got == kind, name


def test_host_f16_conversion_is_round_to_nearest_even(host_exe, tmp_path):
    """f32_to_f16_bits (the F16 tensors of a quantized model) against numpy's IEEE conversion: every f16 value, its
    neighbours and the midpoints between neighbours (ties), subnormals, overflow, infinities, and random bit patterns."""
    rng = np.random.default_rng(3)
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    halves = halves[np.isfinite(halves)].astype(np.float32)
    up, down = np.nextafter(halves, np.float32(np.inf)), np.nextafter(halves, np.float32(-np.inf))
    mids = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([halves, up, down, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                        np.array([65504, 65519.99, 65520, 65536, 1e10, -1e10, np.inf, -np.inf, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001,
                                  2.0**-26, 0.0, -0.0, 5.9604645e-08, 6.1e-05], dtype=np.float32),
                        rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    x = x[~np.isnan(x)]
    src, dst = str(tmp_path / "f32.bin"), str(tmp_path / "f16.bin")
    x.tofile(src)
    r = subprocess.run([host_exe, "--f16", src, dst], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(dst, dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (x[bad[:5]], got[bad[:5]], want[bad[:5]])
    # NaN stays NaN (quiet), with its sign
    nan = np.array([0x7FC00000, 0xFFC00001, 0x7F800001], dtype=np.uint32).view(np.float32)
    nan.tofile(src)
    subprocess.run([host_exe, "--f16", src, dst], check=True)
    got = np.fromfile(dst, dtype=np.uint16)
    assert all((g & 0x7C00) == 0x7C00 and (g & 0x03FF) != 0 for g in got) and (got[1] & 0x8000)


def test_hf_to_gguf_name_examples():
    """weight_format.rs:389-435"""
    f = og.hf_to_gguf_name
    assert f("model.embed_tokens.weight") == "token_embd.weight"
    assert f("model.norm.weight") == "output_norm.weight"
    assert f("lm_head.weight") == "output.weight"
    assert f("model.layers.12.self_attn.q_proj.weight") == "blk.12.attn_q.weight"
    assert f("model.layers.0.mlp.down_proj.weight") == "blk.0.ffn_down.weight"
    assert f("model.layers.3.self_attn.rotary_emb.inv_freq") == "blk.3.self_attn.rotary_emb.inv_freq"
    assert f("model.layers.x.mlp.up_proj.weight") == "model.layers.x.mlp.up_proj.weight"
    assert f("model.layers.7") == "model.layers.7"
    assert f("visual.blocks.0.attn.qkv.weight") == "visual.blocks.0.attn.qkv.weight"


def test_gguf_to_hf_name_reference_examples():
    """The reference's own examples, weight_format.rs:668-786, and the pass-through cases its code implies."""
    f = og.gguf_to_hf_name
    assert f("token_embd.weight") == "model.embed_tokens.weight"
    assert f("output_norm.weight") == "model.norm.weight"
    assert f("output.weight") == "lm_head.weight"
    assert f("blk.0.attn_q.weight") == "model.layers.0.self_attn.q_proj.weight"
    assert f("blk.15.attn_k.weight") == "model.layers.15.self_attn.k_proj.weight"
    assert f("blk.7.attn_v.weight") == "model.layers.7.self_attn.v_proj.weight"
    assert f("blk.0.attn_output.weight") == "model.layers.0.self_attn.o_proj.weight"
    assert f("blk.0.ffn_gate.weight") == "model.layers.0.mlp.gate_proj.weight"
    assert f("blk.0.ffn_up.weight") == "model.layers.0.mlp.up_proj.weight"
    assert f("blk.0.ffn_down.weight") == "model.layers.0.mlp.down_proj.weight"
    assert f("blk.0.attn_norm.weight") == "model.layers.0.input_layernorm.weight"
    assert f("blk.0.ffn_norm.weight") == "model.layers.0.post_attention_layernorm.weight"
    assert f("blk.0.attn_q_norm.weight") == "model.layers.0.self_attn.q_norm.weight"
    assert f("blk.0.attn_k_norm.weight") == "model.layers.0.self_attn.k_norm.weight"
    for name in ROUND_TRIP_NAMES:  # test_hf_to_gguf_name_round_trip_core_tensors
        assert f(og.hf_to_gguf_name(name)) == name
    assert og.hf_to_gguf_name("model.layers.0.mlp.gate.weight") == "blk.0.ffn_gate_inp.weight"  # test_hf_to_gguf_name_moe_tensors
    assert og.hf_to_gguf_name("model.layers.0.mlp.experts.gate_proj.weight") == "blk.0.ffn_gate_exps.weight"
    assert og.hf_to_gguf_name("model.layers.0.mlp.shared_expert.up_proj.weight") == "blk.0.ffn_up_shexp.weight"
    # unknown tensors and names that are not blk.N.rest pass through; the block number is not parsed
    assert f("blk.3.attn_rot_embd") == "model.layers.3.attn_rot_embd"
    assert f("blk.5") == "blk.5" and f("blk.x.ffn_up.weight") == "model.layers.x.mlp.up_proj.weight"
    assert f("rope_freqs.weight") == "rope_freqs.weight" and f("blk..attn_q.weight") == "model.layers..self_attn.q_proj.weight"


ROUND_TRIP_NAMES = ["model.embed_tokens.weight", "model.norm.weight", "lm_head.weight", "model.layers.0.self_attn.q_proj.weight",
                    "model.layers.1.self_attn.k_proj.weight", "model.layers.2.self_attn.v_proj.weight",
                    "model.layers.3.self_attn.o_proj.weight", "model.layers.4.input_layernorm.weight",
                    "model.layers.5.post_attention_layernorm.weight", "model.layers.6.mlp.gate_proj.weight",
                    "model.layers.7.mlp.up_proj.weight", "model.layers.8.mlp.down_proj.weight",
                    "model.layers.9.self_attn.q_norm.weight", "model.layers.10.self_attn.k_norm.weight"]


def test_host_f16_to_f32_is_exact(host_exe, tmp_path):
    """f16_bits_to_f32 (the F16 tensors of a file that is loaded) on all 65536 bit patterns against numpy."""
    bits = np.arange(65536, dtype=np.uint16)
    src, dst = str(tmp_path / "f16.bin"), str(tmp_path / "f32.bin")
    bits.tofile(src)
    subprocess.run([host_exe, "--f16-to-f32", src, dst], check=True)
    got = np.fromfile(dst, dtype=np.float32)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all() and np.array_equal(got[nan].view(np.uint32) >> 31, want[nan].view(np.uint32) >> 31)


# ---------------------------------------------------------------------------------------------------------------------
# GPU: the Q4_K_M model driver end to end
# ---------------------------------------------------------------------------------------------------------------------
def synth_tensor(seed: int, n: int) -> np.ndarray:
    i = np.arange(n, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15) + i * np.uint64(0xBF58476D1CE4E5B9) + np.uint64(0x94D049BB133111EB)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    u = (z >> np.uint64(40)).astype(np.float64) / 16777216.0 - 0.5
    return (u * 0.125).astype(np.float32)


@pytest.mark.gpu
def test_quantize_model_q4_k_m_file_equals_oracle(oracle, tmp_path):
    if not os.path.exists(os.path.join(LIBDIR, "libpmetal_hip.so")):
        pytest.fail("libpmetal_hip.so is not built")
    exe = str(tmp_path / "test_gguf_file")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"), SRC, "-o", exe, "-L", LIBDIR,
                    "-lpmetal_hip", f"-Wl,-rpath,{LIBDIR}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    layers, hidden, inter, kv, vocab = 9, 512, 1280, 256, 1000
    tensors = [("model.embed_tokens.weight", [vocab, hidden]), ("model.norm.weight", [hidden]), ("lm_head.weight", [vocab, hidden]),
               ("blk.1.attn_qkv.weight", [3 * 256, hidden])]  # already GGUF-named, fused: the recipe gives it Q5_K
    for layer in range(layers):
        p = f"model.layers.{layer}."
        tensors += [(p + "input_layernorm.weight", [hidden]), (p + "post_attention_layernorm.weight", [hidden]),
                    (p + "self_attn.q_proj.weight", [hidden, hidden]), (p + "self_attn.k_proj.weight", [kv, hidden]),
                    (p + "self_attn.v_proj.weight", [kv, hidden]), (p + "self_attn.o_proj.weight", [hidden, hidden]),
                    (p + "self_attn.q_norm.weight", [64]), (p + "mlp.gate_proj.weight", [inter, hidden]),
                    (p + "mlp.up_proj.weight", [inter, hidden]), (p + "mlp.down_proj.weight", [hidden, inter])]
    rng = np.random.default_rng(5)
    order = rng.permutation(len(tensors))  # the driver sorts by name whatever order it is given
    spec = str(tmp_path / "model.txt")
    with open(spec, "w") as f:
        f.write(f"arch {hx('qwen3')}\nlayers {layers}\n")
        for idx in order:
            name, dims = tensors[idx]
            f.write(f"tensor {hx(name)} {len(dims)} {' '.join(map(str, dims))} {1000 + idx}\n")
    out = str(tmp_path / "model.gguf")
    r = subprocess.run([exe, "--quantize-model", spec, out], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr

    # the same job by the oracle: commands/quantize.rs:1390-1433 (sorted Hugging Face names, recipe type, quantize)
    b = og.GgufBuilder.with_model("qwen3", "quantized-model")
    types = {}
    for idx in sorted(range(len(tensors)), key=lambda i: tensors[i][0].encode()):
        name, dims = tensors[idx]
        gguf_name = og.hf_to_gguf_name(name)
        t = oracle.lib().pmo_q4km_tensor_type(gguf_name.encode(), len(dims), layers)
        x = synth_tensor(1000 + idx, int(np.prod(dims)))
        data = x.astype(np.float16).tobytes() if t == 1 else oracle.quantize(t, x).tobytes()
        b.add_raw_tensor(gguf_name, dims, t, data)
        types[t] = types.get(t, 0) + 1
    b.add_metadata("qwen3.block_count", ("u32", layers))
    want = b.build_to_bytes()
    assert set(types) == {1, 12, 13, 14} and types[14] >= 4  # F16 norms, Q4_K, Q5_K (fused qkv), Q6_K on the embedding / output / more-bits layers
    got = open(out, "rb").read()
    assert len(got) == len(want)
    assert got == want
    # and the file reads back: the C++ reader's view of it equals the oracle's
    r = subprocess.run([exe, "--dump", out], capture_output=True, text=True)
    assert r.stdout == oracle_dump(want)

    # the way back, WeightLoader::load_gguf (weight_format.rs:258-313): every tensor dequantized to f32 under its Hugging
    # Face name, bit for bit what the oracle's dequantizers give for the same bytes (F16 by numpy)
    vals = str(tmp_path / "loaded.bin")
    r = subprocess.run([exe, "--load-model", out, vals], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr

    def oracle_dequantize(raw, dtype, shape):
        raw = np.frombuffer(raw, dtype=np.uint8)
        if dtype == 1:
            return raw.view(np.float16).astype(np.float32)
        return oracle.dequantize(dtype, raw, shape)

    loaded, skipped = og.load_gguf(want, oracle_dequantize, lambda dt: dt in (0, 1, 30, 8, 10, 11, 12, 13, 14, 15))
    assert not skipped and len(loaded) == len(tensors)
    flat = np.fromfile(vals, dtype=np.float32)
    lines = r.stdout.strip().split("\n")
    assert len(lines) == len(loaded)
    pos = 0
    for line, name in zip(lines, sorted(loaded, key=lambda s: s.encode())):
        f = line.split()
        assert bytes.fromhex(f[0]).decode() == name
        shape, values = loaded[name]
        assert [int(v) for v in f[2:2 + int(f[1])]] == shape and int(f[-1]) == values.size
        assert np.array_equal(flat[pos:pos + values.size].view(np.uint32), values.view(np.uint32)), name
        pos += values.size
    assert pos == flat.size
    # the loaded names are the Hugging Face names the model was given (the fused tensor keeps its GGUF-style name under
    # model.layers.N.)
    assert set(loaded) == {n if not n.startswith("blk.") else og.gguf_to_hf_name(n) for n, _ in tensors}
    # both name mappings of the C++ mirror against the oracle's, over the reference's examples and some odd names
    names = ROUND_TRIP_NAMES + [og.hf_to_gguf_name(n) for n in ROUND_TRIP_NAMES] + [
        "blk.3.attn_rot_embd", "blk.5", "blk.x.ffn_up.weight", "rope_freqs.weight", "blk..attn_q.weight", "model.layers.7",
        "model.layers.+3.mlp.up_proj.weight", "model.layers.0.mlp.shared_experts.down_proj.weight", "blk.2.ffn_gate_inp_shexp.weight"]
    listing = str(tmp_path / "names.txt")
    open(listing, "w").write("\n".join(hx(n) for n in names) + "\n")
    r = subprocess.run([exe, "--names", listing], capture_output=True, text=True)
    got_names = [tuple(bytes.fromhex(h).decode() for h in l.split()) for l in r.stdout.strip().split("\n")]
    assert got_names == [(og.gguf_to_hf_name(n), og.hf_to_gguf_name(n)) for n in names]
