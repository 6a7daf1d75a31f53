"""One-line mistakes that a restatement of the reference's quantizers could plausibly contain, as text edits of
``oracle/pmetal_oracle.c``, and the machinery to build the edited oracle and run the rational fixtures through it.

``tests/test_oracle_mutations.py`` asserts that every one of them makes at least one case of
``tests/golden/exact_cases.json`` fail: a mistake of that kind in the oracle cannot hide behind the fixtures.  Each entry
names the step of the reference it perturbs (file:line of the Rust) and the item of the bit-exactness checklist it
belongs to:

   1  nearest_int rounds half away from zero               2  no fused multiply-add in quantize / dequantize
   3  divisions are IEEE divisions                          4  requantize with the decoded f16 d / dmin; Q8_0 with 127/amax
   5  float sums run in element order                       6  max_scale / max_min fold from +0.0
   7  make_qkx1_quants returns (scale, -min)                8  Q6_K: first strictly greater |scale|; all-zero block d = 0x8000
   9  `.min(127) as i8` before the truncation              10  `if d != 0.0` guards of the requantization loops
  11  a trailing partial super-block is emitted as zeros

``EQUIVALENT`` lists edits that cannot change a result (or are not known to), with the argument; no fixture can tell them from
the original.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_C = os.path.join(os.path.dirname(HERE), "oracle", "pmetal_oracle.c")
CFLAGS = ["-O2", "-std=c11", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-fno-unsafe-math-optimizations", "-frounding-math"]

# (name, checklist item, reference lines, [(old text, new text), ...]); every old text must occur exactly once
MUTATIONS = [
    ("nearest_int_half_even", 1, "quantize.rs:567",
     [("int32_t pmo_nearest_int(float v) { return f32_as_i32(roundf(v)); }",
       "int32_t pmo_nearest_int(float v) { return f32_as_i32(rintf(v)); }")]),
    ("qkx1_sum_fused", 2, "quantize.rs:630",
     [("for (int32_t i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];",
       "for (int32_t i = 0; i < n; i++) sum += fmaf(-scale, (float)l[i], x[i]);")]),
    ("q4k_requant_reciprocal", 3, "k_quants.rs:939",
     [("int32_t lv = pmo_nearest_int((x[32 * j + ii] + dm) / d);",
       "int32_t lv = pmo_nearest_int((x[32 * j + ii] + dm) * (1.0f / d));")]),
    ("q6k_requant_reciprocal", 3, "k_quants.rs:1109",
     [("int32_t ll = clamp_i32(pmo_nearest_int(x[16 * j + ii] / d), -32, 31);",
       "int32_t ll = clamp_i32(pmo_nearest_int(x[16 * j + ii] * (1.0f / d)), -32, 31);")]),
    ("qkx1_scale_reciprocal", 3, "quantize.rs:625",
     [("scale = sumlx / (float)suml2;", "scale = sumlx * (1.0f / (float)suml2);")]),
    ("q4k_requant_undecoded_d", 4, "k_quants.rs:935-937",
     [("float df = pmo_f16_to_f32(d16), dminf = pmo_f16_to_f32(dmin16);",
       "float df = max_scale / 63.0f, dminf = max_min / 63.0f;")]),
    ("q5k_requant_undecoded_d", 4, "k_quants.rs:1016-1018",
     [("float d = pmo_f16_to_f32(d16) * (float)sc;", "float d = (max_scale / 63.0f) * (float)sc;"),
      ("float dm = pmo_f16_to_f32(dmin16) * (float)m;", "float dm = (max_min / 63.0f) * (float)m;")]),
    ("q6k_requant_undecoded_d", 4, "k_quants.rs:1106",
     [("float df = pmo_f16_to_f32(d16);", "float df = 1.0f / iscale;")]),
    ("q2k_requant_undecoded_d", 4, "k_quants.rs:1300-1304",
     [("float d = pmo_f16_to_f32(d16) * (float)(bscales[j] & 0xF);", "float d = (max_scale / 15.0f) * (float)(bscales[j] & 0xF);"),
      ("float dm = pmo_f16_to_f32(dmin16) * (float)(bscales[j] >> 4);", "float dm = (max_min / 15.0f) * (float)(bscales[j] >> 4);")]),
    ("q3k_requant_undecoded_d", 4, "k_quants.rs:1199",
     [("float d = pmo_f16_to_f32(d16) * (float)scs;",
       "float d = (max_scale != 0.0f ? 1.0f / (-32.0f / max_scale) : 0.0f) * (float)scs;")]),
    ("q8_0_iscale_from_scale", 4, "quantize.rs:282",
     [("float iscale = amax == 0.0f ? 0.0f : 127.0f / amax;\n        uint16_t d = pmo_f32_to_f16(scale);",
       "float iscale = amax == 0.0f ? 0.0f : 1.0f / scale;\n        uint16_t d = pmo_f32_to_f16(scale);")]),
    ("qkx1_sum_reversed", 5, "quantize.rs:627-632",
     [("for (int32_t i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];",
       "for (int32_t i = n - 1; i >= 0; i--) sum += x[i] - scale * (float)l[i];")]),
    ("q4k_fold_from_first", 6, "k_quants.rs:904-905",
     [("float max_scale = 0.0f, max_min = 0.0f;\n        for (int j = 0; j < 8; j++) max_scale = rust_max(scales[j], max_scale);",
       "float max_scale = scales[0], max_min = mins[0];\n        for (int j = 0; j < 8; j++) max_scale = rust_max(scales[j], max_scale);")]),
    ("qkx1_returns_zero_minus_min", 7, "quantize.rs:643",
     [("*min_out = -min;", "*min_out = 0.0f - min;")]),
    ("q6k_last_of_equal_scales", 8, "k_quants.rs:1090",
     [("if (abs_scale > max_abs_scale) {", "if (abs_scale >= max_abs_scale) {")]),
    ("q6k_zero_block_guarded", 8, "k_quants.rs:1096-1097",
     [("uint16_t d16 = pmo_f32_to_f16(1.0f / iscale);\n        blk[208]",
       "uint16_t d16 = max_scale == 0.0f ? 0 : pmo_f32_to_f16(1.0f / iscale);\n        blk[208]")]),
    ("q6k_scale_code_wraps", 9, "k_quants.rs:1101",
     [("if (v > 127) v = 127;", "")]),
    ("q4k_requant_unguarded", 10, "k_quants.rs:936",
     [("float d = df * (float)sc;\n            if (d != 0.0f) {", "float d = df * (float)sc;\n            if (1) {")]),
    ("q6k_requant_unguarded", 10, "k_quants.rs:1107",
     [("float d = df * (float)bscales[j];\n            if (d != 0.0f) {", "float d = df * (float)bscales[j];\n            if (1) {")]),
    ("q4k_partial_block_not_zeroed", 11, "k_quants.rs:878-892",
     [("memset(dst, 0, n_blocks * 144);", "memset(dst, 0, (n / QK_K) * 144);")]),
    ("q6k_partial_block_not_zeroed", 11, "k_quants.rs:1058-1072",
     [("memset(dst, 0, n_blocks * 210);", "memset(dst, 0, (n / QK_K) * 210);")]),
    # further one-line edits of the searches
    ("qkx1_min_not_clamped", 0, "quantize.rs:635",
     [("if (min > 0.0f) min = 0.0f;", "")]),
    ("qx_descent_accepts_ties", 0, "quantize.rs:825",
     [("                    if (sl2 > 0.0f && slx * slx * suml2 > sumlx * sumlx * sl2) {\n                        ls[i] = (int8_t)(nmax + new_l);",
       "                    if (sl2 > 0.0f && slx * slx * suml2 >= sumlx * sumlx * sl2) {\n                        ls[i] = (int8_t)(nmax + new_l);")]),
    ("qx_last_of_equal_magnitudes", 0, "quantize.rs:746",
     [("    /* :742-750 */\n    float max = 0.0f, amax = 0.0f;\n    for (int32_t i = 0; i < n; i++) {\n        float ax = fabsf(x[i]);\n        if (ax > amax) {",
       "    /* :742-750 */\n    float max = 0.0f, amax = 0.0f;\n    for (int32_t i = 0; i < n; i++) {\n        float ax = fabsf(x[i]);\n        if (ax >= amax) {")]),
    ("qx_rescale_accepts_ties", 0, "quantize.rs:798",
     [("if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;", "if (!changed || sl2 == 0.0f || slx * slx < best * sl2) break;")]),
    ("q8_0_amax_signed", 0, "quantize.rs:279",
     [("amax = rust_max(amax, fabsf(x[i])); /* acc.max(x.abs()) */", "amax = rust_max(amax, x[i]);")]),
]

# Edits that change no result, so that no fixture can catch them: (name, reference lines, edits, why).  The test checks that
# they indeed pass every fixture case.
EQUIVALENT = [
    ("q4k_dequant_fused", "k_quants.rs:381",
     [("for (int l = 0; l < 16; l++) out[idx++] = d1 * (float)(q[l] & 0xF) - dm1;",
       "for (int l = 0; l < 16; l++) out[idx++] = fmaf(d1, (float)(q[l] & 0xF), -dm1);")],
     "d (11 significant bits) * sc (6 bits) * q (4 bits) has at most 21 significant bits: the products are exact in binary32, and "
     "the subtraction is the only rounding with or without fusing.  The same holds for Q5_K (22 bits), Q6_K's d * sc * q (24 bits) "
     "and Q8_0's q * d (19 bits)."),
    ("qx_descent_slx_zero_enters", "quantize.rs:819",
     [("            if (slx > 0.0f) {\n                float sl2 = suml2 - w * (float)(l * l);",
       "            if (slx >= 0.0f) {\n                float sl2 = suml2 - w * (float)(l * l);")],
     "slx is sumlx minus the element's own term, and every term w*x*l has the sign of -max (l is rounded from -nmax/max * x).  On "
     "the sums as first accumulated, slx == 0 needs every other term to be exactly zero (a non-zero quant means |x| >= |max|/64, a "
     "term of at least 2^-18 of the largest, which no rounding of the running sum absorbs), so every other w*l*l is zero too and "
     "sl2 == 0: the candidate is nearest_int(NaN) = 0 and `sl2 > 0.0` refuses the move.  After accepted moves the sums carry "
     "rounding residues and the argument is no proof; a search over 6.4e7 sub-blocks (integers, half-integers, one dominant "
     "element beside small ones, sparse and Gaussian data) found no input on which the two differ.  The fixture holds two "
     "sub-blocks that reach slx == 0 (qx_slx_zero_0, _1)."),
    ("qkx1_sum_seed_plus_zero", "quantize.rs:627-632",
     [("float sum = -0.0f;", "float sum = 0.0f;")],
     "Iterator::sum folds from -0.0; every term x - scale*l that is zero is +0.0 in round-to-nearest, and -0.0 + (+0.0) = +0.0 = "
     "+0.0 + (+0.0): with n >= 1 terms the seed's sign never reaches the result."),
    ("qkx1_first_maximum", "quantize.rs:593",
     [("if (total_cmp(max, x[i]) <= 0) max = x[i];", "if (total_cmp(max, x[i]) < 0) max = x[i];")],
     "max_by(total_cmp) returns the last of equal maxima, but values that total_cmp calls equal have the same bits."),
    ("qx_rescale_without_change_test", "quantize.rs:798",
     [("if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;", "if (sl2 == 0.0f || slx * slx <= best * sl2) break;")],
     "when no quant changed, slx and sl2 are sums of the same terms in the same order as sumlx and suml2: whether the pass is "
     "then taken or not, ls, sumlx, suml2 and scale keep their values."),
    ("q4k_scale_code_unclamped", "k_quants.rs:917",
     [("uint8_t ls = (uint8_t)(a < 63 ? a : 63);\n            uint8_t lm = (uint8_t)(c < 63 ? c : 63);",
       "uint8_t ls = (uint8_t)a;\n            uint8_t lm = (uint8_t)c;")],
     "inv_scale * scale_j <= fl(63 / max) * max <= 63 * (1 + 2^-23): nearest_int never exceeds 63, the min never binds."),
]


def edited_source(edits, what):
    src = open(ORACLE_C).read()
    for old, new in edits:
        assert src.count(old) == 1, f"{what}: the text to edit occurs {src.count(old)} times in pmetal_oracle.c: {old[:60]!r}"
        src = src.replace(old, new)
    return src


def mutated_source(name):
    for mname, _, _, edits in MUTATIONS:
        if mname == name:
            return edited_source(edits, name)
    raise KeyError(name)


def build(src_text, workdir, tag):
    """Compile an oracle source text into workdir/liboracle_<tag>.so and return the loaded library."""
    c_path = os.path.join(workdir, f"oracle_{tag}.c")
    so_path = os.path.join(workdir, f"liboracle_{tag}.so")
    with open(c_path, "w") as f:
        f.write(src_text)
    subprocess.run(["gcc", *CFLAGS, "-I", os.path.dirname(ORACLE_C), "-shared", "-o", so_path, c_path, "-lm", "-lpthread"],
                   check=True, capture_output=True)
    return bind(C.CDLL(so_path))


def bind(L):
    f32p, u8p, i8p, i32p = C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_int8), C.POINTER(C.c_int32)
    L.pmo_make_qkx1_quants.argtypes, L.pmo_make_qkx1_quants.restype = [C.c_int32, C.c_int32, f32p, C.c_int32, f32p, f32p], None
    L.pmo_make_qx_quants.argtypes, L.pmo_make_qx_quants.restype = [C.c_int32, C.c_int32, f32p, C.c_int32, i8p], C.c_float
    L.pmo_make_q3_quants.argtypes, L.pmo_make_q3_quants.restype = [f32p, C.c_int32, C.c_int32, C.c_int32, i8p], C.c_float
    L.pmo_tensor_size.argtypes, L.pmo_tensor_size.restype = [C.c_uint32, C.c_size_t], C.c_size_t
    L.pmo_quantize.argtypes, L.pmo_quantize.restype = [C.c_uint32, f32p, C.c_size_t, u8p, C.c_size_t], C.c_int32
    L.pmo_dequantize.argtypes = [C.c_uint32, u8p, C.c_size_t, i32p, C.c_size_t, f32p, C.c_size_t, C.c_uint32]
    L.pmo_dequantize.restype = C.c_int32
    return L


def _f32(bits):
    return np.ascontiguousarray(np.array(bits, dtype=np.uint32).view(np.float32))


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def lib_quantize(L, t, x):
    """pmo_quantize into a poisoned buffer (a byte the library does not write stays 0xA5)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    nbytes = L.pmo_tensor_size(t, x.size)
    out = np.full(nbytes, 0xA5, dtype=np.uint8)
    rc = L.pmo_quantize(t, _p(x, C.c_float), x.size, _p(out, C.c_uint8), nbytes)
    assert rc == 0, rc
    return out


def lib_dequantize(L, t, raw, n, order):
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.full(n, np.nan, dtype=np.float32)
    shape = np.array([n], dtype=np.int32)
    rc = L.pmo_dequantize(t, _p(raw, C.c_uint8), raw.size, _p(shape, C.c_int32), 1, _p(out, C.c_float), n, order)
    assert rc == 0, rc
    return out


def failing_cases(L, cases):
    """Names of the fixture cases whose expected bits the library `L` does not return."""
    bad = []
    for c in cases["qkx1"]:
        x = _f32(c["x_bits"])
        s, m = C.c_float(), C.c_float()
        L.pmo_make_qkx1_quants(c["nmax"], 5, _p(x, C.c_float), x.size, C.byref(s), C.byref(m))
        got = (int(np.float32(s.value).view(np.uint32)), int(np.float32(m.value).view(np.uint32)))
        if got != (c["scale_bits"], c["min_bits"]):
            bad.append(c["name"])
    for c in cases["qx"]:
        x = _f32(c["x_bits"])
        ls = np.zeros(c["n"], dtype=np.int8)
        s = L.pmo_make_qx_quants(c["n"], c["nmax"], _p(x, C.c_float), c["rmse_type"], _p(ls, C.c_int8))
        if int(np.float32(s).view(np.uint32)) != c["scale_bits"] or [int(v) for v in ls] != c["ls"]:
            bad.append(c["name"])
    for c in cases["q3"]:
        x = _f32(c["x_bits"])
        ls = np.zeros(x.size, dtype=np.int8)
        s = L.pmo_make_q3_quants(_p(x, C.c_float), x.size, c["nmax"], 1 if c["do_rmse"] else 0, _p(ls, C.c_int8))
        if int(np.float32(s).view(np.uint32)) != c["scale_bits"] or [int(v) for v in ls] != c["ls"]:
            bad.append(c["name"])
    for c in cases["blocks"] + cases.get("tensors", []):
        got = lib_quantize(L, c["type"], _f32(c["x_bits"]))
        if got.tobytes().hex() != c["bytes"]:
            bad.append(c["name"])
    for c in cases.get("dequant", []):
        raw = np.frombuffer(bytes.fromhex(c["bytes"]), dtype=np.uint8)
        got = lib_dequantize(L, c["type"], raw, c["n"], c["order"])
        if [int(v) for v in got.view(np.uint32)] != c["y_bits"]:
            bad.append(c["name"])
    return bad
