"""Committed block vectors (tests/golden/blocks.npz, written by tests/golden/make_golden.py): the oracle must
keep reproducing them on the CPU, and the HIP library must reproduce them bit for bit on the GPU."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "blocks.npz")
TYPES = {"q8_0": 8, "q4k": 12, "q6k": 14, "q5k": 13, "q3k": 11, "q2k": 10, "q8k": 15}
TWO_ORDERS = (12, 13)


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(GOLD, allow_pickle=False))


@pytest.mark.parametrize("name", sorted(TYPES))
def test_oracle_reproduces_golden(oracle, gold, name):
    t = TYPES[name]
    q = oracle.quantize(t, gold["x"])
    assert np.array_equal(q, gold[name + "_bytes"])
    assert np.array_equal(oracle.dequantize(t, q, [gold["x"].size]).view(np.uint32), gold[name + "_deq"])
    if t in TWO_ORDERS:
        got = oracle.dequantize(t, q, [gold["x"].size], order=1).view(np.uint32)
        assert np.array_equal(got, gold[name + "_deq_ggml"])


def test_golden_zero_superblock(gold):
    """The all-zero super-block of the fixture: Q4_K emits zero bytes, Q6_K emits d = f16(-0.0)
    (crates/pmetal-gguf/src/k_quants.rs:1096-1097 has no zero guard)."""
    assert not gold["q4k_bytes"][144:288].any()
    blk = gold["q6k_bytes"][210:420]
    assert not blk[:208].any() and blk[208] == 0x00 and blk[209] == 0x80


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(TYPES))
def test_hip_reproduces_golden(gold, name):
    from gpu_util import gpu_dequantize_dev, gpu_quantize_dev
    t = TYPES[name]
    q = gpu_quantize_dev(t, gold["x"])
    assert np.array_equal(q, gold[name + "_bytes"])
    assert np.array_equal(gpu_dequantize_dev(t, q, gold["x"].size).view(np.uint32), gold[name + "_deq"])
    if t in TWO_ORDERS:
        assert np.array_equal(gpu_dequantize_dev(t, q, gold["x"].size, order=1).view(np.uint32), gold[name + "_deq_ggml"])
