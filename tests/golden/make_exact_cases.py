#!/usr/bin/env python3
"""Writes ``exact_cases.json``: inputs of the three scale searches and of the five k-quant block quantizers together with the
results that rational arithmetic gives for them (``tests/exact_ref.py``: the reference's algorithms restated from the Rust
over ``fractions.Fraction``, every binary32 operation rounded once by the IEEE-754 definition).

Nothing here runs the CPU oracle or the HIP library: the expected values are independent of both.

Two families of inputs:

* ``order_free``: dyadic / small-integer inputs for which every accumulated sum of the search is exact in any order of its
  terms (checked by the rational reference, see ``Trace.order_free``), so that the result follows from the algorithm's
  definition and from single correctly rounded operations only.  The patterns were found by random search over eight-element
  patterns on a 1/8 grid (make_qkx1_quants; a sub-block is the pattern repeated, which leaves scale, min and quants unchanged)
  and over sixteen small integers or half-integers (make_qx_quants, make_q3_quants) and are kept below as data; what makes
  them fixtures is that the rational reference confirms the property and records the branches taken when this script runs.
* ``ordered``: Gaussian inputs (N(0, 0.02^2), a fixed seed) where the sums do round and the order of the terms matters; the
  expected bits come from the rational reference adding in the reference's order (element 0 first), one rounding per
  addition.

Usage:  python tests/golden/make_exact_cases.py            (rewrites tests/golden/exact_cases.json)
"""
import json
import os
import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import exact_ref as E  # noqa: E402

# ---- make_qkx1_quants: (nmax, repeat, pattern); the sub-block is the pattern repeated `repeat` times -------------------
QKX1_PATTERNS = [
    # two tries, nothing rounds at all
    (3, 2, [-1.375, 1.625, 0.5, 0.625, -0.75, -0.125, -0.25, 0.75]),
    (3, 2, [0.0, 3.0, 2.75, 2.375, 2.0, 2.25, 1.75, 2.0]),
    (15, 4, [-2.25, 12.75, 0.0, 9.75, -1.25, -0.5, 2.75, 0.75]),
    (15, 4, [0.0, 15.0, 0.0, 12.25, 6.0, 11.5, 3.25, 9.25]),
    (31, 4, [-0.5, 30.5, 17.75, 17.25, 26.5, 22.5, 11.5, 23.5]),
    (31, 4, [0.0, 31.0, 6.25, 28.75, 16.75, 20.0, 25.25, 15.25]),
    # two tries with a quant above nmax before the clamp
    (3, 2, [-1.375, 1.625, -0.625, -1.375, -1.125, -0.875, 0.125, -0.875]),
    (15, 4, [-2.75, 12.25, 3.75, 8.875, -0.125, 10.75, 8.875, -2.125]),
    # three tries
    (3, 2, [-3.5, -0.5, -2.25, -2.25, -3.125, -1.625, -2.25, -3.0]),
    (3, 2, [-0.125, 2.875, 1.375, 0.25, 0.25, 0.0, 1.0, 0.125]),
    (3, 2, [-1.75, 1.25, -0.25, -1.375, -0.25, -0.125, 0.75, -0.375]),
    (15, 4, [-3.75, 11.25, 1.5, 1.5, -2.25, 10.0, 2.5, -1.5]),
    (15, 4, [-0.125, 14.875, 0.25, 4.25, 1.25, 1.0, 3.375, 1.875]),
    (31, 4, [-0.5, 30.5, 29.0, 8.75, 20.75, 29.75, 1.5, 5.5]),
    # four tries
    (3, 2, [-0.125, 2.875, 0.5, 0.0, 0.25, 1.125, 1.25, 1.375]),
    (3, 2, [0.0, 3.0, 1.125, 1.5, 1.625, 2.375, 1.375, 2.5]),
    (3, 1, [-3.25, -0.25, -3.0, -1.75, -2.0, -2.75, -2.75, -2.0, -3.0, -1.75, -2.0, -3.0, -0.5, -1.0, -3.25, -2.0]),
    # five tries (the fifth confirms that nothing changes any more)
    (3, 2, [-0.125, 2.875, 0.375, 1.25, 0.25, 0.5, 1.125, 2.0]),
    (3, 2, [-0.125, 2.875, 0.375, 0.25, 1.125, 2.0, 1.25, 0.5]),
    # all elements positive: the minimum starts at 0 (quantize.rs:601), scale exactly 1
    (15, 2, [15.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 9.0, 10.0, 11.0, 12.0, 13.0, 14.0, 1.0]),
    (3, 2, [3.0, 1.0, 2.0, 1.0, 3.0, 2.0, 1.0, 2.0]),
]

# ---- make_qx_quants(16, 32, x, 1) and make_q3_quants(x, 4, true): sixteen small integers or half-integers ---------------
QX_INPUTS = [
    [-1.0, 1.0, 13.0, 22.0, -23.0, -17.0, 16.0, 22.0, -12.0, -9.0, 18.0, -4.0, -11.0, 16.0, -12.0, -4.0],
    [3.0, 3.0, 0.0, 5.0, -7.0, -2.0, -5.0, 6.0, 0.0, -3.0, -8.0, -2.0, 0.0, -3.0, 12.0, 10.0],
    [-14.0, 4.0, -2.0, 17.0, 10.0, 11.0, 4.0, -7.0, -11.0, -3.0, 4.0, -6.0, -17.0, -19.0, -22.0, -15.0],
    [0.0, 11.0, -7.0, -14.0, -17.0, -16.0, -5.0, 10.0, 2.0, -6.0, -10.0, -5.0, -4.0, -5.0, -14.0, -5.0],
    [-3.0, -12.0, 7.0, -5.0, -1.5, 12.0, -3.0, -6.0, -6.5, 8.5, -7.0, 2.5, -6.5, 7.5, 5.5, 3.0],
    [7.0, -10.5, -1.0, -3.5, 6.5, 6.0, 7.0, -2.5, 9.0, -9.0, 0.5, 10.0, -2.0, 10.5, -2.5, -2.0],
    [-12.0, 4.0, 6.0, -6.0, 16.0, -19.0, 8.0, 1.0, 21.0, 15.0, 17.0, 19.0, -23.0, 23.0, -19.0, -6.0],
    [7.5, -9.5, -4.5, -7.0, 7.5, -3.0, -11.0, 9.5, 10.5, -4.0, 11.0, -1.0, -4.5, -0.5, 0.0, -4.5],
    [10.0, 0.0, -5.5, 7.0, 11.0, -5.0, 10.0, 6.5, 7.0, 0.5, 10.0, -8.5, -10.0, 11.5, 0.0, -2.5],
    [-23.0, -9.0, 10.0, -19.0, 8.0, 19.0, 11.0, -4.0, 23.0, 6.0, -23.0, -9.0, -14.0, 6.0, -8.0, 11.0],
    [6.0, -8.5, 5.0, 5.5, 12.0, -5.5, -1.5, -9.0, -12.0, -11.0, -1.5, -8.0, 6.0, -7.5, 3.0, 1.0],
    [-7.5, -2.5, 1.0, -2.0, -1.0, 7.0, -6.5, -5.5, 1.0, -5.0, 3.0, 3.5, 3.0, -2.5, 7.5, 0.0],
    [-7.5, -4.0, -1.5, -3.5, 7.0, -1.0, 0.0, 7.0, -7.0, -0.5, -3.5, 7.5, 5.5, -5.0, -2.0, 7.0],
    [7.0, -6.0, 4.0, -5.0, 10.0, -3.0, -12.0, 8.0, -15.0, -6.0, -6.0, -2.0, 4.0, 11.0, -11.0, 2.0],
    [-12.0, 4.0, -4.5, 12.0, 6.0, -7.5, -4.0, 5.5, 11.5, 1.5, -10.5, -1.5, -3.0, -4.5, -9.0, 5.0],
    # an exact grid: x = l for l in [-32, 31] with the largest magnitude negative: scale exactly 1, nothing moves
    [-32.0, 31.0, -1.0, 0.0, 5.0, -7.0, 12.0, -20.0, 3.0, 2.0, 1.0, -3.0, 8.0, -8.0, 16.0, -16.0],
    # the largest magnitude twice with both signs: the first one (positive) decides, the other is clamped to 31
    [24.0, -24.0, 3.0, -5.0, 7.0, 1.0, 0.0, 2.0, -9.0, 11.0, 4.0, -6.0, 8.0, -2.0, 5.0, -1.0],
]
# the new quants of a rescale pass differ from the old ones and slx^2 == best * sl2 exactly (quantize.rs:798 refuses the pass on a
# tie); found by a search over sub-blocks of small integers and half-integers
QX_TIE_INPUTS = [
    [-19.0, -21.0, -16.0, 19.0, -3.0, 13.0, 0.0, 22.0, 14.0, 6.0, -14.0, -23.0, -5.0, -14.0, 4.0, -2.0],
    [11.0, 11.0, -13.0, -11.0, 23.0, 13.0, 5.0, -1.0, -9.0, -13.0, -21.0, -21.0, 10.0, -7.0, -23.0, 4.0],
    [17.0, 8.0, -24.0, 22.0, 4.0, 24.0, 5.0, 10.0, 7.0, -3.0, -10.0, 13.0, -2.0, -14.0, 19.0, -4.0],
    [12.0, -1.5, -3.0, 2.5, 6.0, -1.0, -4.5, -0.5, 1.5, 3.0, -6.5, 0.0, -12.0, -9.5, -10.0, -9.5],
    [10.5, -11.5, -1.5, 11.0, 7.0, -11.5, -1.0, 8.0, 6.5, 3.5, -4.5, 11.5, -4.0, 0.5, 2.0, 8.5],
]
# one element carries the whole of sumlx (every other quant is 0): slx == 0 exactly for it (quantize.rs:819), both signs
QX_SLX_ZERO_INPUTS = [
    [-32.0, 0.25, -0.25, 0.125, 0.0, 0.375, -0.125, 0.25, 0.0, 0.0, 0.125, -0.375, 0.25, 0.0, -0.25, 0.125],
    [0.125, 0.125, 16.0, -0.125, 0.0, 0.0, 0.125, -0.125, 0.0, 0.125, 0.0, 0.0, -0.125, 0.0, 0.125, 0.0],
]
# Gaussian super-blocks (block `index` of gaussian(default_rng(seed), blocks * elements)) whose bytes change when a step of the
# block quantizer is done differently; found by a search, kept as (type, blocks in the stream, seed, index, what they pin)
GAUSS_PICKS = [
    (12, 64, 7000, 3, "requantize with the decoded f16 d / dmin (k_quants.rs:935-937)"),
    (12, 64, 7000, 4, "requantize with the decoded f16 d / dmin (k_quants.rs:935-937)"),
    (13, 64, 7000, 0, "requantize with the decoded f16 d / dmin (k_quants.rs:1016-1018)"),
    (13, 64, 7000, 1, "requantize with the decoded f16 d / dmin (k_quants.rs:1016-1018)"),
    (10, 64, 7000, 19, "requantize with the decoded f16 d / dmin (k_quants.rs:1300-1304)"),
    (10, 64, 7000, 43, "requantize with the decoded f16 d / dmin (k_quants.rs:1300-1304)"),
    (11, 64, 7000, 42, "requantize with the decoded f16 d (k_quants.rs:1199)"),
    (11, 64, 7001, 26, "requantize with the decoded f16 d (k_quants.rs:1199)"),
    (14, 64, 7000, 1, "requantize with the decoded f16 d (k_quants.rs:1106)"),
    (14, 64, 7000, 3, "requantize with the decoded f16 d (k_quants.rs:1106)"),
    (12, 20000, 7000, 7616, "(x + dm) / d is a division, not a product with 1 / d (k_quants.rs:939)"),
    (12, 20000, 7001, 6501, "(x + dm) / d is a division, not a product with 1 / d (k_quants.rs:939)"),
    (14, 20000, 7000, 15395, "x / d is a division, not a product with 1 / d (k_quants.rs:1109)"),
    (14, 20000, 7000, 17017, "x / d is a division, not a product with 1 / d (k_quants.rs:1109)"),
    (8, 100000, 7000, 54099, "iscale = 127 / amax, not 1 / (amax / 127) (quantize.rs:282)"),
    (8, 100000, 7001, 58597, "iscale = 127 / amax, not 1 / (amax / 127) (quantize.rs:282)"),
    (8, 100000, 7001, 86130, "iscale = 127 / amax, not 1 / (amax / 127) (quantize.rs:282)"),
]
Q3_INPUTS = [
    [27.0, -19.0, -32.0, -16.0, -7.0, 25.0, -4.0, -33.0, -13.0, 8.0, 25.0, 19.0, 40.0, -25.0, 31.0, -36.0],
    [-1.0, 32.0, -5.0, 9.0, -34.0, 27.0, -5.0, 0.0, -33.0, 16.0, 11.0, -13.0, 22.0, 2.0, -36.0, -23.0],
    [-32.0, -20.0, -35.0, 10.0, -37.0, -9.0, 1.0, -4.0, 8.0, 25.0, 31.0, 26.0, 20.0, 4.0, 8.0, 24.0],
    [15.0, 11.0, 4.0, -16.0, 5.0, 6.0, -14.0, 17.0, 8.0, -32.0, 2.0, -20.0, 18.0, 13.0, -18.0, -14.0],
    [34.0, -9.0, -11.0, 6.0, -39.0, 37.0, 28.0, 17.0, -32.0, 19.0, -10.0, 38.0, 22.0, -19.0, -24.0, -19.0],
    [-4.0, -12.0, 17.0, 17.5, 9.5, 12.5, 18.0, -14.5, -12.0, -11.5, -11.0, -20.0, 20.0, 18.0, -13.5, -13.0],
    [6.0, -17.0, -17.0, 11.5, 3.0, -3.5, -7.5, -1.5, -3.5, -7.0, 4.0, 17.0, 0.0, -14.0, 16.0, -6.5],
    [-18.0, -17.0, 14.0, -17.5, 19.5, -11.5, -18.5, 15.5, 3.0, 13.5, -9.5, 16.0, -14.5, 0.5, -13.0, -20.0],
    [-15.0, 2.0, -19.0, -19.0, 19.0, 7.5, 4.0, 19.0, 16.0, 4.5, -5.5, -12.5, 6.0, -5.5, -9.0, -9.0],
    [18.0, -14.5, 14.0, 9.5, -20.0, -7.5, -15.0, -11.0, 19.0, 20.0, 7.5, 1.5, -15.0, -3.0, -13.5, -18.0],
    [5.0, -21.0, -27.0, 30.0, -25.0, 22.0, 9.0, -30.0, -34.0, -6.0, -8.0, 12.0, -23.0, 22.0, -6.0, 33.0],
    # an exact grid: x = l for l in [-4, 3], largest magnitude negative: scale exactly 1
    [-4.0, 3.0, -1.0, 0.0, 1.0, 2.0, -2.0, -3.0, 3.0, 1.0, 0.0, -1.0, 2.0, -2.0, 1.0, -3.0],
]


def f32(v):
    return E.F32.of(Fraction(v) if not isinstance(v, Fraction) else v)


def bits_of(xs):
    return [x.bits() for x in xs]


def trace_dict(tr):
    return {"order_free": tr.order_free, "inexact": tr.inexact, "branches": sorted(tr.branches)}


def case_qkx1(name, nmax, xs, family):
    tr = E.new_trace()
    s, m, L = E.make_qkx1_quants(nmax, 5, xs)
    d = {"name": name, "family": family, "nmax": nmax, "x_bits": bits_of(xs), "scale_bits": s.bits(), "min_bits": m.bits(),
         "L": L, "tries": tr.tries}
    d.update(trace_dict(tr))
    return d


def case_qx(name, xs, family, n=16, nmax=32, rmse_type=1):
    tr = E.new_trace()
    s, ls = E.make_qx_quants(n, nmax, xs, rmse_type)
    d = {"name": name, "family": family, "n": n, "nmax": nmax, "rmse_type": rmse_type, "x_bits": bits_of(xs),
         "scale_bits": s.bits(), "ls": ls}
    d.update(trace_dict(tr))
    return d


def case_q3(name, xs, family, nmax=4, do_rmse=True):
    tr = E.new_trace()
    s, ls = E.make_q3_quants(xs, nmax, do_rmse)
    d = {"name": name, "family": family, "nmax": nmax, "do_rmse": do_rmse, "x_bits": bits_of(xs), "scale_bits": s.bits(), "ls": ls}
    d.update(trace_dict(tr))
    return d


def gaussian(rng, n, std=0.02):
    return [E.F32.from_bits(int(u)) for u in (rng.standard_normal(n) * std).astype(np.float32).view(np.uint32)]


def scaled(xs, e):
    """x * 2^e (exact)."""
    return [E.F32.of(x.q * Fraction(2) ** e) for x in xs]


def block_case(name, t, xs, family, parts):
    tr = E.new_trace()
    raw = E.BLOCK_QUANTIZERS[t](xs)
    return {"name": name, "family": family, "type": t, "x_bits": bits_of(xs), "bytes": raw.hex(), "sub_blocks": parts,
            "order_free": tr.order_free}


def main():
    out = {"qkx1": [], "qx": [], "q3": [], "blocks": [], "tensors": [], "dequant": []}
    rng = np.random.default_rng(20240607)

    # ---- make_qkx1_quants ----
    pats = QKX1_PATTERNS
    subs = {3: [], 15: [], 31: []}  # order-free sub-blocks of the formats' sizes, for the block vectors
    for i, (nmax, rep, pat) in enumerate(pats):
        xs = [f32(v) for v in pat] * rep
        c = case_qkx1(f"qkx1_grid_{i}_nmax{nmax}", nmax, xs, "order_free")
        assert c["order_free"], c["name"]
        out["qkx1"].append(c)
        if len(xs) == (16 if nmax == 3 else 32):
            subs[nmax].append((c["name"], xs))
    out["qkx1"].append(case_qkx1("qkx1_constant", 15, [f32(1)] * 32, "special"))
    out["qkx1"].append(case_qkx1("qkx1_two_values", 15, [f32(0), f32(15)] * 16, "order_free"))
    big = E.F32.from_bits(0x7F61B1E6)  # 3e38: max - min overflows, every quant is 0, the loop leaves at suml2 == 0
    out["qkx1"].append(case_qkx1("qkx1_overflow_suml2_zero", 15, [big, -big] + [f32(0)] * 30, "special"))
    for nmax, n in ((15, 32), (31, 32), (3, 16)):
        got = {}
        for _ in range(400):  # Gaussian sub-blocks until every number of tries has been seen a few times
            xs = gaussian(rng, n)
            c = case_qkx1("", nmax, xs, "ordered")
            key = (c["tries"], "qkx1:all_tries_changed" in c["branches"], "qkx1:clamp_low" in c["branches"])
            if got.get(key, 0) < 2:
                got[key] = got.get(key, 0) + 1
                c["name"] = f"qkx1_gauss_nmax{nmax}_{len(out['qkx1'])}"
                out["qkx1"].append(c)
            if len(got) >= 5 and all(v >= 2 for v in got.values()):
                break

    # ---- make_qx_quants ----
    qsubs = []
    for i, pat in enumerate(QX_INPUTS):
        xs = [f32(v) for v in pat]
        c = case_qx(f"qx_int_{i}", xs, "order_free")
        assert c["order_free"], c["name"]
        out["qx"].append(c)
        qsubs.append((c["name"], xs))
    for i, pat in enumerate(QX_TIE_INPUTS):
        c = case_qx(f"qx_rescale_tie_{i}", [f32(v) for v in pat], "order_free")
        assert c["order_free"] and "qx:rescale:tie_rejected" in c["branches"], c["name"]
        out["qx"].append(c)
    for i, pat in enumerate(QX_SLX_ZERO_INPUTS):
        c = case_qx(f"qx_slx_zero_{i}", [f32(v) for v in pat], "order_free")
        assert c["order_free"] and "qx:descent:slx==0" in c["branches"], c["name"]
        out["qx"].append(c)
    out["qx"].append(case_qx("qx_all_zero", [f32(0)] * 16, "special"))
    out["qx"].append(case_qx("qx_rmse_type_0", [f32(v) for v in QX_INPUTS[0]], "order_free", rmse_type=0))
    for i in range(24):
        out["qx"].append(case_qx(f"qx_gauss_{i}", gaussian(rng, 16), "ordered"))

    # ---- make_q3_quants ----
    q3subs = []
    for i, pat in enumerate(Q3_INPUTS):
        xs = [f32(v) for v in pat]
        c = case_q3(f"q3_int_{i}", xs, "order_free")
        assert c["order_free"], c["name"]
        out["q3"].append(c)
        q3subs.append((c["name"], xs))
    out["q3"].append(case_q3("q3_all_zero", [f32(0)] * 16, "special"))
    out["q3"].append(case_q3("q3_no_rmse", [f32(v) for v in Q3_INPUTS[0]], "order_free", do_rmse=False))
    # the reference's own known answers (quantize.rs:1020-1032): zeros and a ramp
    out["q3"].append(case_q3("q3_reference_ramp", [f32(v) for v in range(-8, 8)], "order_free"))
    for i in range(24):
        out["q3"].append(case_q3(f"q3_gauss_{i}", gaussian(rng, 16), "ordered"))

    # ---- whole super-blocks built from the order-free sub-blocks, each at its own power-of-two magnitude ----
    def compose(pool, count, exps):
        xs, parts = [], []
        for j in range(count):
            name, sub = pool[(j * 7 + 3) % len(pool)]
            e = exps[j % len(exps)]
            xs += scaled(sub, e)
            parts.append(f"{name} * 2^{e}")
        return xs, parts

    for rot in range(3):
        e4 = [[-6, -7, -6, -8, -5, -6, -7, -6], [-3, -3, -3, -3, -3, -3, -3, -3], [0, -9, -4, -1, -12, -2, -6, -3]][rot]
        for t, nmax in ((12, 15), (13, 31)):
            pool = subs[nmax][rot:] + subs[nmax][:rot]
            xs, parts = compose(pool, 8, e4)
            out["blocks"].append(block_case(f"block_type{t}_grid_{rot}", t, xs, "order_free", parts))
        pool = subs[3][rot:] + subs[3][:rot]
        xs, parts = compose(pool, 16, e4)
        out["blocks"].append(block_case(f"block_type10_grid_{rot}", 10, xs, "order_free", parts))
        e6 = [[-9, -10, -9, -11, -8, -9, -10, -9], [-5] * 8, [-4, -13, -8, -5, -16, -6, -10, -7]][rot]
        pool = qsubs[rot:] + qsubs[:rot]
        xs, parts = compose(pool, 16, e6)
        out["blocks"].append(block_case(f"block_type14_grid_{rot}", 14, xs, "order_free", parts))
        pool = q3subs[rot:] + q3subs[:rot]
        xs, parts = compose(pool, 16, e6)
        out["blocks"].append(block_case(f"block_type11_grid_{rot}", 11, xs, "order_free", parts))
    for b in out["blocks"]:
        assert b["order_free"], b["name"]
    for t in (12, 13, 14, 11, 10):
        for i in range(2):
            xs = gaussian(rng, 256)
            if i == 1:  # the benchmark's outliers
                xs[17], xs[200] = f32(0.5), f32(-0.5)
            out["blocks"].append(block_case(f"block_type{t}_gauss_{i}", t, xs, "ordered", []))

    # ---- super-blocks that single out one step of the block quantizers ----
    # Q4_K / Q5_K / Q2_K with every element positive: each sub-block returns the min -0.0, and max_min folds from +0.0
    # (k_quants.rs:904-905), so dmin is 0x0000 and not 0x8000
    pos15 = [xs for name, xs in subs[15] if all(x.q > 0 for x in xs)]
    pos3 = [xs for name, xs in subs[3] if all(x.q > 0 for x in xs)]
    assert pos15 and pos3
    allpos32 = sum((scaled(pos15[0], -(j % 3) - 4) for j in range(8)), [])
    allpos16 = sum((scaled(pos3[0], -(j % 3) - 4) for j in range(16)), [])
    for t, xs in ((12, allpos32), (13, allpos32), (10, allpos16)):
        c = block_case(f"block_type{t}_all_positive", t, xs, "order_free", ["all-positive sub-blocks"])
        raw = bytes.fromhex(c["bytes"])
        assert (raw[2:4] if t != 10 else raw[82:84]) == bytes(2), "dmin must be +0.0"
        out["blocks"].append(c)
    # Q6_K: two sub-blocks whose scales are +1 and -1 exactly (an exact grid and its mirror image), the others smaller: the
    # first of the two decides the sign of d (k_quants.rs:1090), and the other one's scale code 128 is cut to 127 (:1101)
    grid = [f32(v) for v in QX_INPUTS[15]]
    assert case_qx("", grid, "order_free")["scale_bits"] == f32(1).bits()
    mirror = [-x for x in grid]
    assert case_qx("", mirror, "order_free")["scale_bits"] == f32(-1).bits()
    small = [scaled(qsubs[(3 * j) % 15][1], -7 - j % 4) for j in range(14)]
    for name, first, second in (("plus_first", grid, mirror), ("minus_first", mirror, grid)):
        xs = sum(small[:5], []) + first + sum(small[5:9], []) + second + sum(small[9:], [])
        c = block_case(f"block_type14_equal_scales_{name}", 14, xs, "order_free", ["scales +1 and -1"])
        raw = bytes.fromhex(c["bytes"])
        codes = sorted(v - 256 if v > 127 else v for v in (raw[192 + 5], raw[192 + 10]))
        assert codes == [-128, 127], codes
        out["blocks"].append(c)
    # a sub-block far below the largest one gets the scale code 0 and keeps its quants: all 0 in Q4_K (k_quants.rs:936), the ones
    # make_qx_quants left in Q6_K (:1107)
    tiny4 = sum((scaled(subs[15][j % len(subs[15])][1], -3 if j != 2 else -20) for j in range(8)), [])
    tiny6 = sum((scaled(qsubs[j % len(qsubs)][1], -5 if j != 4 else -24) for j in range(16)), [])
    out["blocks"].append(block_case("block_type12_scale_code_zero", 12, tiny4, "order_free", ["sub-block 2 at 2^-17 of the others"]))
    out["blocks"].append(block_case("block_type14_scale_code_zero", 14, tiny6, "order_free", ["sub-block 4 at 2^-19 of the others"]))
    # all-zero super-blocks: Q4_K / Q5_K / Q3_K / Q2_K all-zero bytes, Q6_K d = f16(-0.0) = 0x8000 (k_quants.rs:1096-1097)
    for t in (12, 13, 14, 11, 10):
        c = block_case(f"block_type{t}_all_zero", t, [f32(0)] * 256, "special", [])
        assert (bytes.fromhex(c["bytes"])[208:210] == bytes([0, 0x80])) if t == 14 else not any(bytes.fromhex(c["bytes"]))
        out["blocks"].append(c)
    # the Gaussian picks
    for t, nblocks, seed, index, why in GAUSS_PICKS:
        el = 32 if t == 8 else 256
        stream = (np.random.default_rng(seed).standard_normal(nblocks * el) * 0.02).astype(np.float32)
        xs = [E.F32.from_bits(int(u)) for u in stream[index * el:(index + 1) * el].view(np.uint32)]
        E.new_trace()
        c = {"name": f"pick_type{t}_seed{seed}_{index}", "family": "ordered", "type": t, "x_bits": bits_of(xs),
             "bytes": E.quantize_tensor(t, xs).hex(), "pins": why}
        out["blocks" if t != 8 else "tensors"].append(c)

    # ---- whole tensors: ragged lengths and Q8_0 ----
    def tensor_case(name, t, xs, family):
        E.new_trace()
        return {"name": name, "family": family, "type": t, "x_bits": bits_of(xs), "bytes": E.quantize_tensor(t, xs).hex()}

    tail = [f32(Fraction(v, 8)) for v in range(-22, 22)]  # 44 elements past the last whole super-block: emitted as zeros
    for t, blk in ((12, tiny4), (13, allpos32), (14, tiny6), (11, sum((scaled(q3subs[j % len(q3subs)][1], -5) for j in range(16)), [])),
                   (10, allpos16)):
        c = tensor_case(f"tensor_type{t}_300_elements", t, blk + tail, "order_free")
        assert len(c["bytes"]) == 4 * E.BLOCK_BYTES[t] and not any(bytes.fromhex(c["bytes"])[E.BLOCK_BYTES[t]:])
        out["tensors"].append(c)
    ramp = [f32(Fraction(v - 16, 8)) for v in range(40)]  # Q8_0: a whole block and 8 elements of a second one
    out["tensors"].append(tensor_case("tensor_q8_0_40_elements", 8, ramp, "order_free"))
    out["tensors"].append(tensor_case("tensor_q8_0_zero_block", 8, [f32(0)] * 32, "special"))
    neg = [f32(-127)] + [f32(v) for v in range(-15, 16)]  # the largest magnitude is negative: amax = |x|, codes reach -127
    out["tensors"].append(tensor_case("tensor_q8_0_negative_maximum", 8, neg, "order_free"))
    out["tensors"].append(tensor_case("tensor_q8_0_gauss", 8, gaussian(rng, 96), "ordered"))

    # ---- dequantizers: block bytes -> values, every product and difference rounded on its own ----
    def dequant_case(name, t, raw, n, order):
        fn = {8: lambda: E.dequantize_q8_0(raw, n), 12: lambda: E.dequantize_q4k(raw, n, order == 1), 14: lambda: E.dequantize_q6k(raw, n)}[t]
        E.new_trace()
        return {"name": name, "type": t, "order": order, "n": n, "bytes": raw.hex(), "y_bits": [y.bits() for y in fn()]}

    drng = np.random.default_rng(4242)
    for t, size in ((12, 144), (14, 210), (8, 34)):
        nblk = 2 if t != 8 else 5
        raw = bytearray(drng.integers(0, 256, nblk * size, dtype=np.uint8).tobytes())
        for b in range(nblk):  # finite f16 scales (clear the top exponent bit)
            for off in {12: (1, 3), 14: (209,), 8: (1,)}[t]:
                raw[b * size + off] &= 0xBF
        n = nblk * (32 if t == 8 else 256) - 7  # the output is cut to n elements
        for order in ((0, 1) if t == 12 else (0,)):
            out["dequant"].append(dequant_case(f"dequant_type{t}_order{order}_random_bytes", t, bytes(raw), n, order))
    for c in out["blocks"]:  # and what the quantizers wrote for the Gaussian blocks
        if c["name"] in ("block_type12_gauss_0", "block_type14_gauss_0"):
            for order in ((0, 1) if c["type"] == 12 else (0,)):
                out["dequant"].append(dequant_case(f"dequant_{c['name']}_order{order}", c["type"], bytes.fromhex(c["bytes"]), 256, order))

    path = os.path.join(HERE, "exact_cases.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, {k: len(v) for k, v in out.items()}, os.path.getsize(path), "bytes")
    hit = set()
    for k in ("qkx1", "qx", "q3"):
        for c in out[k]:
            if c["order_free"]:
                hit |= set(c["branches"])
    print("branches reached by order-free cases:", sorted(hit))


if __name__ == "__main__":
    main()
