"""Pins the oracle's scale searches and k-quant block quantizers against results that rational arithmetic fixes.

Expected values: ``tests/golden/exact_cases.json``, written by ``tests/golden/make_exact_cases.py`` from ``tests/exact_ref.py``
-- the reference's ``make_qkx1_quants`` (crates/pmetal-gguf/src/quantize.rs:583-644), ``make_q3_quants`` (:655-726),
``make_qx_quants`` (:738-841) and ``quantize_q4k / _q5k / _q6k / _q3k / _q2k`` (crates/pmetal-gguf/src/k_quants.rs:876-1323)
restated from the Rust over ``fractions.Fraction`` with one IEEE-754 rounding per binary32 operation.  Neither the C oracle nor
numpy's float32 takes part in producing them.

Families (field ``family`` of a case):
  order_free  every accumulated sum of the search is exact in ANY order of its terms (all terms on one power-of-two grid,
              the sum of magnitudes below 2^24 grid steps), so the expected (scale, min, quants) do not depend on the
              summation order; what is left are single operations (a product, a quotient, a comparison) that IEEE-754 fixes.
              Cases with ``inexact == 0`` do not round anywhere: their results are the ones real arithmetic gives.
  ordered     Gaussian inputs; sums round, the expected bits are those of the reference's order (element 0 first).
  special     constant input, all-zero input, an overflowing range (the suml2 == 0 exit).

Which order-free case reaches which lines of the reference (asserted by ``test_order_free_cases_reach_every_branch``):
  quantize.rs:596       max == min -> (0, 0)                               qkx1_constant
  quantize.rs:601       min.min(0.0) with an all-positive sub-block        qkx1:min0=0       (grid cases 19, 20)
  quantize.rs:613       clamp of a quant above nmax                        qkx1:clamp_high
  quantize.rs:622-624   suml2 == 0 exit                                    qkx1_overflow_suml2_zero (special: needs max - min = inf)
  quantize.rs:627-637   re-estimated min, min > 0 -> 0                     qkx1:min>0->0
  quantize.rs:639-641   did_change == false after try 2 / 3 / 4 / 5        qkx1:stop_after_try_2 .. _5
  quantize.rs:607       all five tries change something                    ordered family only (qkx1:all_tries_changed)
  quantize.rs:752-754   amax == 0                                          qx_all_zero
  quantize.rs:758-764   rmse_type == 0                                     qx_rmse_type_0
  quantize.rs:756       sign of iscale                                     qx:max<0, qx:max>0
  quantize.rs:771       clamp at nmax - 1                                  qx:clamp_high
  quantize.rs:798       rescale pass: unchanged / rejected / accepted      qx:rescale1..2:unchanged, qx:rescale1..2:rejected,
                        (first, second, third pass, all three accepted)    qx:rescale1..3:accepted, qx:rescale:three_accepted
  quantize.rs:819       slx <= 0 skips the element                         qx:descent:slx<=0
  quantize.rs:825-831   single-element move accepted / rejected            qx:descent1..5:accepted, qx:descent1..4:rejected
  quantize.rs:835-837   sweeps until nothing changes (1 .. 5 sweeps),      qx:descent:stop_after_sweep_1 .. _5,
                        and five sweeps that all change                    qx:descent:five_sweeps_changed
  quantize.rs:669-671   amax == 0                                          q3_all_zero
  quantize.rs:720-725   do_rmse == false                                   q3_no_rmse
  quantize.rs:680       clamp at nmax - 1                                  q3:clamp_high
  quantize.rs:693       slx <= 0 skips the element                         q3:descent:slx<=0
  quantize.rs:700-705   move accepted / rejected in sweeps 1 .. 5          q3:descent1..5:accepted, q3:descent1..5:rejected
  quantize.rs:709-711   1 .. 5 sweeps, and five sweeps that all change     q3:descent:stop_after_sweep_1 .. _5, q3:descent:five_sweeps_changed
  quantize.rs:798       slx^2 == best * sl2 exactly with changed quants: refused    qx:rescale:tie_rejected  (qx_rescale_tie_0 .. _4)
  quantize.rs:819       slx == 0 exactly                                   qx:descent:slx==0        (qx_slx_zero_0, _1)
Whole super-blocks (``blocks``): 8 or 16 of the order-free sub-blocks above, each scaled by its own power of two (exact), so
that the super-block steps (largest scale, 6-bit / 4-bit / signed scale codes, f16 d and dmin, requantization with the
decoded scales, bit packing) run on known sub-block results; those steps hold no sums, only single operations.  Blocks that
single out one step each:
  k_quants.rs:904-905   max_min folds from +0.0 (all sub-blocks return -0.0)         block_type12/13/10_all_positive
  k_quants.rs:1090      the first of two scales of equal magnitude decides d's sign  block_type14_equal_scales_plus_first, _minus_first
  k_quants.rs:1101      a scale code of 128 is cut to 127 before `as i8`             the same two blocks
  k_quants.rs:936,1107  `if d != 0.0`: a sub-block with scale code 0 keeps its quants block_type12/14_scale_code_zero
  k_quants.rs:1096-97   all-zero Q6_K block: d = f16(-0.0) = 0x8000                  block_type14_all_zero (and the other types' zero blocks)
  k_quants.rs:935-937, :1016-1018, :1106, :1199, :1300-1304   requantization with the decoded f16 d / dmin: Gaussian blocks whose
                        bytes differ if the unrounded value is used                  pick_type12/13/14/11/10_seed7000_*
  k_quants.rs:939,1109  the quotient is an IEEE division (blocks with a quotient next to a rounding boundary)   pick_type12/14_seed700x_*
Whole tensors (``tensors``): a trailing partial super-block is emitted as zeros (k_quants.rs:890-892 and the like; 300 elements
of every k-quant type), Q8_0 (quantize.rs:268-300) with a short last block, a zero block, a negative maximum, and Gaussian
blocks where round(x * (127 / amax)) differs from round(x * (1 / (amax / 127))) (:282, pick_type8_*).
Dequantizers (``dequant``): random block bytes and quantized Gaussian blocks -> values in rational arithmetic, both element
orders for Q4_K, the output cut to n elements.
``tests/test_oracle_mutations.py`` edits the oracle one line at a time and checks that these cases notice.
"""
import json
import os

import numpy as np
import pytest

import exact_ref as E

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = json.load(open(os.path.join(HERE, "golden", "exact_cases.json")))
BLOCK_BYTES = {12: 144, 13: 176, 14: 210, 11: 110, 10: 84}

REQUIRED_ORDER_FREE = {
    "qkx1:constant", "qkx1:min0=0", "qkx1:clamp_high", "qkx1:min>0->0", "qkx1:stop_after_try_2", "qkx1:stop_after_try_3",
    "qkx1:stop_after_try_4", "qkx1:stop_after_try_5",
    "qx:amax==0", "qx:rmse_type==0", "qx:max<0", "qx:max>0", "qx:clamp_high", "qx:rescale1:unchanged", "qx:rescale1:accepted",
    "qx:rescale2:unchanged", "qx:rescale2:rejected", "qx:rescale2:accepted", "qx:rescale3:accepted", "qx:rescale:three_accepted",
    "qx:descent:slx<=0", "qx:descent1:accepted", "qx:descent1:rejected", "qx:descent2:accepted", "qx:descent2:rejected",
    "qx:descent3:accepted", "qx:descent4:accepted", "qx:rescale1:rejected", "qx:descent3:rejected", "qx:descent4:rejected",
    "qx:descent5:accepted", "qx:descent:five_sweeps_changed", "qx:descent:stop_after_sweep_1", "qx:descent:stop_after_sweep_2",
    "qx:descent:stop_after_sweep_3", "qx:descent:stop_after_sweep_4", "qx:descent:stop_after_sweep_5",
    "q3:amax==0", "q3:no_rmse", "q3:max<0", "q3:max>0", "q3:clamp_high", "q3:descent:slx<=0", "q3:descent1:accepted",
    "q3:descent1:rejected", "q3:descent2:accepted", "q3:descent2:rejected", "q3:descent3:accepted", "q3:descent3:rejected",
    "q3:descent4:accepted", "q3:descent4:rejected", "q3:descent5:accepted", "q3:descent5:rejected",
    "q3:descent:stop_after_sweep_1",
    "q3:descent:stop_after_sweep_2", "q3:descent:stop_after_sweep_3", "q3:descent:stop_after_sweep_4",
    "q3:descent:stop_after_sweep_5", "q3:descent:five_sweeps_changed",
    "qx:rescale:tie_rejected", "qx:descent:slx==0",
}


def f32_from_bits(bits):
    return np.array(bits, dtype=np.uint32).view(np.float32)


def bits(v):
    return int(np.float32(v).view(np.uint32))


# ---- the rational reference itself: IEEE-754 by definition against the hardware's binary32 / numpy's binary16 ----------
def test_rational_binary32_matches_hardware_arithmetic():
    rng = np.random.default_rng(7)
    specials = np.array([0x00000000, 0x80000000, 0x00000001, 0x807FFFFF, 0x00800000, 0x7F7FFFFF, 0xFF7FFFFF, 0x3F800000,
                         0x3F800001, 0x3FFFFFFF, 0x33800000, 0x4B000000, 0x4B800000, 0x7F800000, 0xFF800000], dtype=np.uint32)
    a = np.concatenate([specials.repeat(len(specials)), rng.integers(0, 0x7F800000, 600, dtype=np.uint32) | (
        rng.integers(0, 2, 600, dtype=np.uint32) << 31)])
    b = np.concatenate([np.tile(specials, len(specials)), rng.integers(0, 0x7F800000, 600, dtype=np.uint32) | (
        rng.integers(0, 2, 600, dtype=np.uint32) << 31)])
    # operands of nearby magnitude as well (cancellation, ties)
    a = np.concatenate([a, rng.integers(0x3F000000, 0x40000000, 600, dtype=np.uint32)])
    b = np.concatenate([b, rng.integers(0x3F000000, 0x40000000, 600, dtype=np.uint32) | 0x80000000])
    fa, fb = a.view(np.float32), b.view(np.float32)
    E.new_trace()
    with np.errstate(all="ignore"):
        for name, op in (("add", lambda x, y: x + y), ("sub", lambda x, y: x - y), ("mul", lambda x, y: x * y),
                         ("div", lambda x, y: x / y)):
            want = op(fa, fb)
            for i in range(a.size):
                got = op(E.F32.from_bits(int(a[i])), E.F32.from_bits(int(b[i])))
                if np.isnan(want[i]):
                    assert got.kind == E.NAN, (name, hex(a[i]), hex(b[i]))
                else:
                    assert got.bits() == int(want[i].view(np.uint32)), (name, hex(a[i]), hex(b[i]))


def test_rational_f16_conversion_matches_numpy():
    rng = np.random.default_rng(8)
    u = np.concatenate([rng.integers(0, 2**32, 3000, dtype=np.uint64).astype(np.uint32),
                        np.array([0, 0x80000000, 0x477FE000, 0x477FEFFF, 0x477FF000, 0x33000000, 0x33000001, 0x32FFFFFF,
                                  0x38800000, 0x387FFFFF, 0x3F801000, 0x3F803000], dtype=np.uint32)])
    f = u.view(np.float32)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    for i in range(u.size):
        if np.isnan(f[i]):
            continue
        assert E.f32_to_f16_bits(E.F32.from_bits(int(u[i]))) == int(want[i]), hex(u[i])
    for h in range(0, 65536, 7):
        v = np.array([h], dtype=np.uint16).view(np.float16).astype(np.float32)[0]
        if not np.isnan(v):
            assert E.f16_bits_to_f32(h).bits() == bits(v)


def test_nearest_int_reference_known_answers_in_the_rational_reference():
    # quantize.rs:862-868
    vals = {0.5: 1, 0.4: 0, -0.5: -1, -0.6: -1, 1.5: 2, 2.5: 3, -2.5: -3}
    for v, want in vals.items():
        assert E.nearest_int(E.F32.of(float(np.float32(v)))) == want


# ---- the fixture is what the rational reference gives (guards against a stale or edited file) ------------------------------
def _xs(case):
    return [E.F32.from_bits(u) for u in case["x_bits"]]


def test_fixture_function_cases_reproduce_from_the_rational_reference():
    for c in CASES["qkx1"]:
        tr = E.new_trace()
        s, m, L = E.make_qkx1_quants(c["nmax"], 5, _xs(c))
        assert (s.bits(), m.bits(), L, tr.tries, tr.order_free, tr.inexact, sorted(tr.branches)) == (
            c["scale_bits"], c["min_bits"], c["L"], c["tries"], c["order_free"], c["inexact"], c["branches"]), c["name"]
    for c in CASES["qx"]:
        tr = E.new_trace()
        s, ls = E.make_qx_quants(c["n"], c["nmax"], _xs(c), c["rmse_type"])
        assert (s.bits(), ls, tr.order_free, sorted(tr.branches)) == (c["scale_bits"], c["ls"], c["order_free"], c["branches"]), c["name"]
    for c in CASES["q3"]:
        tr = E.new_trace()
        s, ls = E.make_q3_quants(_xs(c), c["nmax"], c["do_rmse"])
        assert (s.bits(), ls, tr.order_free, sorted(tr.branches)) == (c["scale_bits"], c["ls"], c["order_free"], c["branches"]), c["name"]


def test_fixture_block_cases_reproduce_from_the_rational_reference():
    for c in CASES["blocks"][::3]:  # a third of them: a block takes 0.1-0.3 s in rational arithmetic
        E.new_trace()
        assert E.BLOCK_QUANTIZERS[c["type"]](_xs(c)).hex() == c["bytes"], c["name"]


def test_order_free_cases_reach_every_branch():
    hit = set()
    for key in ("qkx1", "qx", "q3"):
        for c in CASES[key]:
            if c["family"] == "order_free" or c["name"] in ("qkx1_constant", "qx_all_zero", "q3_all_zero"):
                assert c["order_free"], c["name"]
                hit |= set(c["branches"])
    assert REQUIRED_ORDER_FREE <= hit, sorted(REQUIRED_ORDER_FREE - hit)
    # nothing rounds at all in some multi-try cases: their results are those of real arithmetic
    exact = [c for c in CASES["qkx1"] if c["family"] == "order_free" and c["inexact"] <= 1 and c["tries"] >= 2]
    assert {c["nmax"] for c in exact} == {3, 15, 31} and max(c["tries"] for c in exact) >= 3
    # the ordered family adds what no order-free input reaches
    ordered = set()
    for c in CASES["qkx1"]:
        if c["family"] == "ordered":
            ordered |= set(c["branches"])
            ordered.add(f"tries={c['tries']}")
    assert {"qkx1:all_tries_changed", "tries=2", "tries=3", "tries=4", "tries=5"} <= ordered, ordered
    assert any(c["name"] == "qkx1_overflow_suml2_zero" and "qkx1:suml2==0" in c["branches"] for c in CASES["qkx1"])


# ---- the oracle against the fixture -------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", CASES["qkx1"], ids=[c["name"] for c in CASES["qkx1"]])
def test_oracle_make_qkx1_quants(oracle, case):
    s, m = oracle.make_qkx1_quants(case["nmax"], 5, f32_from_bits(case["x_bits"]))
    assert (bits(s), bits(m)) == (case["scale_bits"], case["min_bits"]), (s, m)


@pytest.mark.parametrize("case", CASES["qx"], ids=[c["name"] for c in CASES["qx"]])
def test_oracle_make_qx_quants(oracle, case):
    s, ls = oracle.make_qx_quants(case["n"], case["nmax"], f32_from_bits(case["x_bits"]), case["rmse_type"])
    assert bits(s) == case["scale_bits"] and [int(v) for v in ls] == case["ls"]


@pytest.mark.parametrize("case", CASES["q3"], ids=[c["name"] for c in CASES["q3"]])
def test_oracle_make_q3_quants(oracle, case):
    s, ls = oracle.make_q3_quants(f32_from_bits(case["x_bits"]), case["nmax"], case["do_rmse"])
    assert bits(s) == case["scale_bits"] and [int(v) for v in ls] == case["ls"]


@pytest.mark.parametrize("case", CASES["blocks"], ids=[c["name"] for c in CASES["blocks"]])
def test_oracle_block_bytes(oracle, case):
    got = oracle.quantize(case["type"], f32_from_bits(case["x_bits"]))
    want = np.frombuffer(bytes.fromhex(case["bytes"]), dtype=np.uint8)
    assert got.size == BLOCK_BYTES[case["type"]]
    assert np.array_equal(got, want), np.nonzero(got != want)[0][:8]


@pytest.mark.parametrize("case", CASES["tensors"], ids=[c["name"] for c in CASES["tensors"]])
def test_oracle_tensor_bytes(oracle, case):
    got = oracle.quantize(case["type"], f32_from_bits(case["x_bits"]))
    assert got.tobytes().hex() == case["bytes"]


@pytest.mark.parametrize("case", CASES["dequant"], ids=[c["name"] for c in CASES["dequant"]])
def test_oracle_dequantized_bits(oracle, case):
    raw = np.frombuffer(bytes.fromhex(case["bytes"]), dtype=np.uint8)
    got = oracle.dequantize(case["type"], raw, [case["n"]], order=case["order"])
    assert [int(v) for v in got.view(np.uint32)] == case["y_bits"]


def test_fixture_tensor_and_dequant_cases_reproduce_from_the_rational_reference():
    for c in CASES["tensors"]:
        E.new_trace()
        assert E.quantize_tensor(c["type"], _xs(c)).hex() == c["bytes"], c["name"]
    for c in CASES["dequant"][:3]:
        raw = bytes.fromhex(c["bytes"])
        fn = {8: lambda: E.dequantize_q8_0(raw, c["n"]), 12: lambda: E.dequantize_q4k(raw, c["n"], c["order"] == 1),
              14: lambda: E.dequantize_q6k(raw, c["n"])}[c["type"]]
        E.new_trace()
        assert [y.bits() for y in fn()] == c["y_bits"], c["name"]


# ---- the HIP quantizers against the fixture (not against the oracle) ------------------------------------------------------
@pytest.mark.gpu
def test_gpu_block_bytes_equal_the_rational_reference():
    import pmetal_amd as pm

    pm.init(0)
    for t in sorted(BLOCK_BYTES):
        cases = [c for c in CASES["blocks"] if c["type"] == t]
        x = np.concatenate([f32_from_bits(c["x_bits"]) for c in cases])
        want = np.concatenate([np.frombuffer(bytes.fromhex(c["bytes"]), dtype=np.uint8) for c in cases])
        got = pm.quantize(x, pm.GgmlType(t))
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, (t, cases[int(bad[0]) // BLOCK_BYTES[t]]["name"], int(bad[0]) % BLOCK_BYTES[t])
        for c in cases:  # and one block at a time (a tensor of a single super-block)
            one = pm.quantize(f32_from_bits(c["x_bits"]), pm.GgmlType(t))
            assert np.array_equal(one, np.frombuffer(bytes.fromhex(c["bytes"]), dtype=np.uint8)), c["name"]


@pytest.mark.gpu
def test_gpu_tensor_bytes_and_dequantized_bits_equal_the_rational_reference():
    """Ragged tensors, Q8_0 and the dequantizers through the HIP library against the rational fixture."""
    import pmetal_amd as pm

    pm.init(0)
    for c in CASES["tensors"]:
        got = pm.quantize(f32_from_bits(c["x_bits"]), pm.GgmlType(c["type"]))
        assert got.tobytes().hex() == c["bytes"], c["name"]
    for c in CASES["dequant"]:
        raw = np.frombuffer(bytes.fromhex(c["bytes"]), dtype=np.uint8)
        got = pm.dequantize(raw, pm.GgmlType(c["type"]), [c["n"]], order=c["order"])
        assert [int(v) for v in got.view(np.uint32)] == c["y_bits"], c["name"]
