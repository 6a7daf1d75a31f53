"""CPU-side checks of the C ABI: the library loads, exports every declared symbol, and its host-side
logic (sizes, validation, recipe, error slot) behaves like the reference -- no compute calls."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import pmetal_amd as pm
from pmetal_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
Q8_0, Q4K, Q6K = 8, 12, 14


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from pmetal_amd import build
        build.build()
    return _lib.load()


def test_header_and_library_agree(lib):
    header = open(os.path.join(ROOT, "include", "pmetal_hip.h")).read()
    declared = set(re.findall(r"\b(pmetal_hip_[a-z0-9_]+)\s*\(", header))
    bound = {name for name, _, _ in _lib.SYMBOLS}
    assert declared == bound, declared ^ bound
    for name in declared:
        assert hasattr(lib, name), name


def test_sizes_match_types_rs(lib):
    # crates/pmetal-gguf/src/types.rs:102-187 and k_quants.rs:1334-1342
    assert [lib.pmetal_hip_type_size(t) for t in (Q8_0, Q4K, Q6K)] == [34, 144, 210]
    assert [lib.pmetal_hip_block_size(t) for t in (Q8_0, Q4K, Q6K)] == [32, 256, 256]
    assert lib.pmetal_hip_tensor_size(Q4K, 14336 * 4096) == 33030144
    assert lib.pmetal_hip_tensor_size(Q8_0, 33) == 68
    assert lib.pmetal_hip_tensor_size(99, 1000) == 0 and lib.pmetal_hip_type_size(0) == 0
    assert [lib.pmetal_hip_is_supported(t) for t in (Q8_0, Q4K, Q6K, 2, 13, 15, 11, 10, 16, 41)] == [1, 1, 1, 1, 1, 1, 1, 1, 0, 0]
    # the 32-element formats beside Q8_0 (types.rs:106-111, :150)
    assert [lib.pmetal_hip_type_size(t) for t in (2, 3, 6, 7, 9)] == [18, 20, 22, 24, 36]
    assert [lib.pmetal_hip_block_size(t) for t in (2, 3, 6, 7, 9)] == [32] * 5
    assert lib.pmetal_hip_type_size(13) == 176 and lib.pmetal_hip_block_size(13) == 256  # Q5_K: quantize / dequantize only
    assert lib.pmetal_hip_type_size(15) == 292 and lib.pmetal_hip_block_size(15) == 256  # Q8_K likewise


def test_sizes_agree_with_oracle(lib, oracle):
    for t in (Q8_0, Q4K, Q6K):
        for n in (0, 1, 31, 32, 33, 255, 256, 257, 10**6 + 7):
            assert lib.pmetal_hip_tensor_size(t, n) == oracle.tensor_size(t, n)


def test_validation_order_and_error_slot(lib):
    shape = (C.c_int32 * 2)(4, -1)
    nb, ne = C.c_size_t(), C.c_size_t()
    assert lib.pmetal_hip_expected_byte_size(Q4K, shape, 2, C.byref(nb), C.byref(ne)) == 6
    assert lib.pmetal_hip_last_error_code() == 6
    assert b"non-negative" in lib.pmetal_hip_last_error_message()
    big = (C.c_int32 * 3)(2**31 - 1, 2**31 - 1, 2**31 - 1)
    assert lib.pmetal_hip_expected_byte_size(Q4K, big, 3, C.byref(nb), C.byref(ne)) == 7
    ok = (C.c_int32 * 2)(3, 256)
    assert lib.pmetal_hip_expected_byte_size(Q6K, ok, 2, C.byref(nb), C.byref(ne)) == 0
    assert (nb.value, ne.value) == (630, 768)
    assert lib.pmetal_hip_last_error_code() == 0 and lib.pmetal_hip_last_error_message() == b""
    # size mismatch is reported before anything touches a device
    raw = np.zeros(10, np.uint8)
    one = (C.c_int32 * 1)(256)
    assert lib.pmetal_hip_dequantize(Q4K, raw.ctypes.data, 10, one, 1, None, 0, 0) == 3
    assert b"expected 144 bytes, got 10" in lib.pmetal_hip_last_error_message()
    assert lib.pmetal_hip_quantize(16, None, 256, None, 66) == 2  # IQ2_XXS: no kernel here
    assert lib.pmetal_hip_quantize(Q4K, None, 256, None, 100) == 3
    lib.pmetal_hip_clear_error()
    assert lib.pmetal_hip_last_error_code() == 0


def test_no_silent_cpu_fallback(lib):
    if lib.pmetal_hip_device_count() > 0:
        pytest.skip("a GPU is present")
    x = np.zeros(256, np.float32)
    with pytest.raises(pm.NoDeviceError):
        pm.quantize(x, Q4K)
    with pytest.raises(pm.NoDeviceError):
        pm.dequantize(np.zeros(144, np.uint8), Q4K, [256])


def test_recipe_matches_reference_kats_and_oracle(lib, oracle):
    t = lambda name, nd, nl: lib.pmetal_hip_q4km_tensor_type(name.encode(), nd, nl)
    # crates/pmetal/src/commands/quantize.rs:1561-1608
    assert t("blk.0.ffn_down.weight", 2, 32) == Q6K
    assert t("blk.0.attn_norm.weight", 1, 32) == 1
    assert t("output.weight", 2, 32) == Q6K
    names = ["token_embd.weight", "output.weight", "output_norm.weight", "blk.X.attn_q.weight", "blk.X.attn_k.weight",
             "blk.X.attn_v.weight", "blk.X.attn_output.weight", "blk.X.ffn_gate.weight", "blk.X.ffn_up.weight",
             "blk.X.ffn_down.weight", "blk.X.attn_norm.weight", "blk.X.ffn_gate_inp.weight", "blk.X.attn_qkv.weight",
             "blk.X.ffn_down_exps.weight", "blk.X.FFN_DOWN.weight", "blk..ffn_down.weight", "blk.7x.ffn_down.weight"]
    O = oracle.lib()
    for nl in (0, 28, 32, 80):
        for layer in range(max(nl, 1)):
            assert lib.pmetal_hip_use_more_bits(layer, nl) == O.pmo_use_more_bits(layer, nl)
            for nm in names:
                nm = nm.replace("X", str(layer))
                for nd in (1, 2, 3):
                    assert t(nm, nd, nl) == O.pmo_q4km_tensor_type(nm.encode(), nd, nl), (nm, nd, nl)
    more = [l for l in range(28) if pm.use_more_bits(l, 28)]
    assert more == [0, 1, 2, 5, 8, 11, 14, 17, 20, 23, 24, 25, 26, 27]
