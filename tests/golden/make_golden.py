"""Writes tests/golden/blocks.npz: seeded inputs and the block bytes / dequantized values the CPU oracle
produces for them.  The reference holds no byte-level vectors for this path (its tests are tolerance and
KAT checks, restated in tests/test_oracle.py), so these are regression pins of the oracle and of the HIP
path against each other, not evidence from the reference.  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding as ob  # noqa: E402

TYPES = {"q8_0": 8, "q4k": 12, "q6k": 14, "q5k": 13, "q3k": 11, "q2k": 10, "q8k": 15}
TWO_ORDERS = (12, 13)  # Q4_K and Q5_K: the reference dequantizer's order and the inverse of the packing


def inputs():
    rng = np.random.default_rng(20240607)
    n = 6 * 256
    x = (rng.standard_normal(n) * 0.02).astype(np.float32)
    x[256:512] = np.float32(0.0)                                 # an all-zero super-block
    x[512:768] = (np.arange(256, dtype=np.float32) - 128) * np.float32(0.01)  # the reference's ramp
    x[768:800] = np.float32(0.37)                                # a constant sub-block (max == min)
    x[1024] = np.float32(0.5)                                    # an outlier
    x[1025] = np.float32(-0.5)
    x[1300] = np.float32(1e-41)                                  # a subnormal
    return x


def main():
    ob.build()
    x = inputs()
    out = {"x": x}
    for name, t in TYPES.items():
        q = ob.quantize(t, x)
        out[name + "_bytes"] = q
        out[name + "_deq"] = ob.dequantize(t, q, [x.size]).view(np.uint32)
        if t in TWO_ORDERS:
            out[name + "_deq_ggml"] = ob.dequantize(t, q, [x.size], order=1).view(np.uint32)
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "blocks.npz"), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
