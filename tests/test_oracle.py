"""Pins the CPU oracle without the reference running (it is Rust; no toolchain here).

Each block of tests names what it pins and against what: the reference's own
known-answer tests (cited file:line under /root/reference), closed forms that the
algorithm must hit exactly, invariants, numpy's IEEE half conversion, and an
independent numpy-float32 twin of the two scale searches (tests/np_twin.py).
"""
import numpy as np
import pytest

import np_twin

Q8_0, Q4K, Q6K = 8, 12, 14


# ----------------------------------------------------------------------------------------------
# half conversions (half 2.7.1; reference call sites k_quants.rs:928-929, :1097, dequant.rs:482)
# ----------------------------------------------------------------------------------------------
def test_f16_to_f32_all_65536_against_numpy(oracle):
    L = oracle.lib()
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([L.pmo_f16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_against_numpy_rne(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(1)
    bits = [rng.integers(0, 2**32, 60000, dtype=np.uint64).astype(np.uint32)]
    # every f16 value, its neighbours, and every exact midpoint between adjacent f16 values
    h = np.arange(0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo[:-1] + hi[:-1]) / 2).astype(np.float32)
    for arr in (lo.astype(np.float32), mid, np.nextafter(mid, np.float32(np.inf)),
                np.nextafter(mid, np.float32(-np.inf))):
        bits += [arr.view(np.uint32), (-arr).view(np.uint32)]
    bits.append(np.array([0, 0x80000000, 0x7F800000, 0xFF800000, 0x477FE000, 0x477FEFFF, 0x477FF000,
                          0x33000000, 0x33000001, 0x32FFFFFF, 0x00000001, 0x007FFFFF], dtype=np.uint32))
    u = np.concatenate(bits)
    f = u.view(np.float32)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([L.pmo_f32_to_f16(float(v)) for v in f], dtype=np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    assert all((int(g) & 0x7C00) == 0x7C00 and (int(g) & 0x3FF) != 0 for g in got[nan])


def test_bf16_rne(oracle):
    L = oracle.lib()
    # 1.0 + 2^-8 is the midpoint between bf16(1.0) and the next value: ties to even (down);
    # 1.0 + 3*2^-8 ties to even (up).
    assert L.pmo_f32_to_bf16(1.0) == 0x3F80
    assert L.pmo_f32_to_bf16(float(np.float32(1.0 + 2.0**-8))) == 0x3F80
    assert L.pmo_f32_to_bf16(float(np.float32(1.0 + 2.0**-8 + 2.0**-20))) == 0x3F81
    assert L.pmo_f32_to_bf16(float(np.float32(1.0 + 3 * 2.0**-8))) == 0x3F82
    assert L.pmo_f32_to_bf16(float("inf")) == 0x7F80
    rng = np.random.default_rng(2)
    x = rng.standard_normal(20000).astype(np.float32)
    vec = oracle.f32_to_bf16_bits(x)
    assert np.array_equal(vec, np.array([L.pmo_f32_to_bf16(float(v)) for v in x], dtype=np.uint16))
    back = oracle.bf16_bits_to_f32(vec)
    assert np.max(np.abs(back - x) / np.abs(x)) <= 2.0**-8


# ----------------------------------------------------------------------------------------------
# nearest_int: reference KATs quantize.rs:862-868 + saturation / NaN of `as i32`
# ----------------------------------------------------------------------------------------------
def test_nearest_int_reference_kats(oracle):
    f = oracle.lib().pmo_nearest_int
    assert [f(0.5), f(0.4), f(-0.5), f(-0.6), f(1.5)] == [1, 0, -1, -1, 2]
    assert f(2.5) == 3 and f(-2.5) == -3  # half away from zero, not half-even
    assert f(float(np.float32(0.49999997))) == 0
    assert f(float("nan")) == 0 and f(1e20) == 2**31 - 1 and f(-1e20) == -(2**31)


# ----------------------------------------------------------------------------------------------
# get_scale_min_k4: reference KATs quantize.rs:1035-1047, k_quants.rs:1386-1396; pack identity
# ----------------------------------------------------------------------------------------------
def pack_scales_k4(ls, lm):
    """6-bit packing as stated at k_quants.rs:915-926 (independent of the oracle)."""
    s = [0] * 12
    for j in range(8):
        if j < 4:
            s[j], s[j + 4] = ls[j], lm[j]
        else:
            s[j + 4] = (ls[j] & 0xF) | ((lm[j] & 0xF) << 4)
            s[j - 4] |= (ls[j] >> 4) << 6
            s[j] |= (lm[j] >> 4) << 6
    return np.array(s, dtype=np.uint8)


def test_get_scale_min_k4(oracle):
    g = oracle.get_scale_min_k4
    assert g(0, np.array([63] * 8 + [0] * 4)) == (63, 63)
    assert g(0, np.array([0x3F] * 8 + [0] * 4)) == (63, 63)
    sc, _ = g(4, np.array([0xC0, 0, 0, 0, 0, 0, 0, 0, 0x03, 0, 0, 0]))
    assert sc == 51  # (0x03 & 0xF) | ((0xC0 >> 6) << 4)
    rng = np.random.default_rng(3)
    for _ in range(2000):
        ls, lm = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
        packed = pack_scales_k4(ls, lm)
        assert [g(j, packed) for j in range(8)] == [(int(a), int(b)) for a, b in zip(ls, lm)]


# ----------------------------------------------------------------------------------------------
# make_qkx1_quants: reference tests quantize.rs:998-1017, exact closed forms, twin
# ----------------------------------------------------------------------------------------------
def test_qkx1_reference_kats(oracle):
    s, m = oracle.make_qkx1_quants(15, 5, np.ones(32))
    assert s == 0.0 and m == 0.0
    s, m = oracle.make_qkx1_quants(15, 5, np.arange(16))
    assert s == 1.0 and m == 0.0  # closed form: l_i = i, sumlx = suml2 = 1240


@pytest.mark.parametrize("k,mm", [(1, 0), (7, 3), (63, 63), (40, 1)])
def test_qkx1_exact_affine_grid(oracle, k, mm):
    # x = k*2^-10 * q - mm*2^-9 with q covering 0..15: every operation is exact, so the search must
    # return exactly (k*2^-10, mm*2^-9).  A sign error on min or a dropped term breaks this.
    rng = np.random.default_rng(k)
    q = np.concatenate([np.arange(16), rng.integers(0, 16, 16)])
    rng.shuffle(q)
    x = (k * 2.0**-10 * q - mm * 2.0**-9).astype(np.float32)
    s, m = oracle.make_qkx1_quants(15, 5, x)
    assert s == np.float32(k * 2.0**-10) and m == np.float32(mm * 2.0**-9)


def test_qkx1_all_positive_keeps_min_zero(oracle):
    x = (np.arange(32) * 0.125 + 3.0).astype(np.float32)  # min > 0 -> min forced to 0 (quantize.rs:601,635)
    s, m = oracle.make_qkx1_quants(15, 5, x)
    assert m == 0.0 and s > 0.0


def test_qkx1_matches_numpy_twin_and_never_worsens(oracle):
    rng = np.random.default_rng(4)
    for t in range(300):
        scale = [0.02, 1.0, 50.0][t % 3]
        x = (rng.standard_normal(32) * scale).astype(np.float32)
        if t % 7 == 0:
            x[rng.integers(0, 32)] = 0.5
        s, m = oracle.make_qkx1_quants(15, 5, x)
        ts, tm = np_twin.qkx1(15, 5, x)
        assert s.view(np.uint32) == ts.view(np.uint32) and m.view(np.uint32) == tm.view(np.uint32)
        assert s > 0 and m >= 0

        def err(sc, mn):
            q = np.clip(np.round((x.astype(np.float64) + mn) / sc), 0, 15)
            return float(np.sum((sc * q - mn - x) ** 2))

        lo = min(float(x.min()), 0.0)
        s0 = (float(x.max()) - lo) / 15
        assert err(float(s), float(m)) <= err(s0, -lo) * (1 + 1e-4) + 1e-12


# ----------------------------------------------------------------------------------------------
# make_qx_quants: closed forms (quantize.rs:752-764), exact grids, invariant, twin
# ----------------------------------------------------------------------------------------------
def test_qx_zero_and_rmse0(oracle):
    s, ls = oracle.make_qx_quants(16, 32, np.zeros(16), 1)
    assert s == 0.0 and not ls.any()
    l = np.array([-32, 31, 0, 5, -7, 12, -1, 1, 30, -31, 16, -16, 8, -8, 2, -2])
    x = (l * 2.0**-6).astype(np.float32)
    s, ls = oracle.make_qx_quants(16, 32, x, 0)
    assert s == np.float32(2.0**-6) and np.array_equal(ls, l + 32)


@pytest.mark.parametrize("sign", [1, -1])
def test_qx_exact_grid(oracle, sign):
    # x = sign * 2^-6 * l with the unique max-|x| element at l = -32.  The search must keep the grid:
    # sign=+1: max is negative -> scale > 0, ls = l + 32; sign=-1: max is positive -> scale < 0 and the
    # same ls (x / scale = l).
    rng = np.random.default_rng(5)
    l = np.concatenate([[-32], rng.integers(-31, 32, 15)])
    rng.shuffle(l)
    x = (sign * l * 2.0**-6).astype(np.float32)
    s, ls = oracle.make_qx_quants(16, 32, x, 1)
    assert np.array_equal(ls, l + 32)
    assert abs(float(s) - sign * 2.0**-6) <= 2.0**-6 * 1e-5 and np.sign(s) == sign


def test_qx_matches_numpy_twin_and_never_worsens(oracle):
    rng = np.random.default_rng(6)
    for t in range(400):
        x = (rng.standard_normal(16) * [0.02, 1.0, 300.0][t % 3]).astype(np.float32)
        if t % 5 == 0:
            x[rng.integers(0, 16)] = -0.5
        if t % 11 == 0:
            x[rng.integers(0, 16, 4)] = 0.0
        s, ls = oracle.make_qx_quants(16, 32, x, 1)
        ts, tls = np_twin.qx(16, 32, x, 1)
        assert s.view(np.uint32) == ts.view(np.uint32) and list(ls) == tls
        assert ls.min() >= 0 and ls.max() <= 63
        x64 = x.astype(np.float64)
        w = x64 * x64
        l0 = np.clip(np.round(-32.0 / x64[np.argmax(np.abs(x64))] * x64), -32, 31)
        s0 = np.sum(w * x64 * l0) / np.sum(w * l0 * l0)
        e0 = np.sum(w * (x64 - s0 * l0) ** 2)
        e1 = np.sum(w * (x64 - float(s) * (ls.astype(np.float64) - 32)) ** 2)
        assert e1 <= e0 * (1 + 1e-4) + 1e-30


# ----------------------------------------------------------------------------------------------
# sizes: types.rs:102-187, k_quants.rs:1334-1342
# ----------------------------------------------------------------------------------------------
def test_sizes(oracle):
    L = oracle.lib()
    assert [L.pmo_type_size(t) for t in (Q8_0, Q4K, Q6K)] == [34, 144, 210]
    assert [L.pmo_block_size(t) for t in (Q8_0, Q4K, Q6K)] == [32, 256, 256]
    assert oracle.tensor_size(Q4K, 14336 * 4096) == 33030144
    assert oracle.tensor_size(Q8_0, 3072 * 1024) == 3342336
    assert oracle.tensor_size(Q8_0, 33) == 68 and oracle.tensor_size(Q6K, 257) == 420
    assert oracle.tensor_size(Q4K, 0) == 0


# ----------------------------------------------------------------------------------------------
# Q8_0: closed form (4 IEEE ops + RNE f16); dequant KAT dequant.rs:1016-1036
# ----------------------------------------------------------------------------------------------
def q8_0_numpy(x):
    x = np.asarray(x, dtype=np.float32)
    nb = -(-x.size // 32)
    xp = np.zeros(nb * 32, dtype=np.float32)
    xp[: x.size] = x
    xb = xp.reshape(nb, 32)
    amax = np.max(np.abs(xb), axis=1)
    with np.errstate(divide="ignore", invalid="ignore"):
        scale = (amax / np.float32(127.0)).astype(np.float32)
        iscale = np.where(amax == 0, np.float32(0), np.float32(127.0) / amax).astype(np.float32)
    v = (xb * iscale[:, None]).astype(np.float32)
    r = np.trunc(v)
    r = r + np.where(np.abs(v - r) >= 0.5, np.copysign(np.float32(1), v), np.float32(0))
    q = np.clip(r, -127, 127).astype(np.int8)
    out = np.zeros((nb, 34), dtype=np.uint8)
    out[:, :2] = scale.astype(np.float16).view(np.uint8).reshape(nb, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def test_q8_0_quantize_closed_form(oracle):
    rng = np.random.default_rng(7)
    for n in (32, 1024, 3072 * 8, 33, 1, 95):
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        if n >= 64:
            x[32:64] = 0.0  # amax == 0 block -> iscale 0, d 0
        assert np.array_equal(oracle.quantize(Q8_0, x), q8_0_numpy(x))
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1], x[2] = 1.0, -1.0, 0.5 / 127  # 0.5/127*127 -> 0.5 -> rounds away to 1
    out = oracle.quantize(Q8_0, x)
    assert out[2] == 127 and out[3] == 0x81 and out[4] in (0, 1)


def test_q8_0_dequant_reference_kat(oracle):
    data = np.concatenate([np.array([0.5], dtype=np.float16).view(np.uint8), np.arange(32, dtype=np.uint8)])
    out = oracle.dequantize(Q8_0, data, [32])
    assert np.array_equal(out, np.arange(32, dtype=np.float32) * 0.5)
    data[2] = 0x80  # -128
    assert oracle.dequantize(Q8_0, data, [32])[0] == -64.0
    assert oracle.dequantize(Q8_0, np.concatenate([data, data]), [40]).size == 40  # truncation


# ----------------------------------------------------------------------------------------------
# Q4_K
# ----------------------------------------------------------------------------------------------
def test_q4k_dequant_reference_kat_fixes_the_order(oracle):
    # Block of k_quants.rs:1370-1375; the REF order (k_quants.rs:365-403) puts, per 64 outputs,
    # 16 low nibbles, 16 high nibbles of bytes 0..15, then the same for bytes 16..31.
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    blk[4:8] = 1
    blk[16:] = 0x21
    ref = oracle.dequantize(Q4K, blk, [256], order=oracle.ORDER_REF)
    assert np.all((ref >= 0) & (ref <= 15))
    chunk = [1.0] * 16 + [2.0] * 16 + [1.0] * 16 + [2.0] * 16
    assert list(ref) == chunk * 2 + [0.0] * 128
    ggml = oracle.dequantize(Q4K, blk, [256], order=oracle.ORDER_GGML)
    assert list(ggml) == ([1.0] * 32 + [2.0] * 32) * 2 + [0.0] * 128


def q4k_decode_numpy(blk, order):
    """Independent vectorised decode from the element<->byte map (not the oracle's loop)."""
    d = blk[0:2].view(np.float16).astype(np.float32)[0]
    dmin = blk[2:4].view(np.float16).astype(np.float32)[0]
    s = blk[4:16]
    sc = np.zeros(8, np.float32)
    mn = np.zeros(8, np.float32)
    for j in range(8):
        if j < 4:
            sc[j], mn[j] = s[j] & 63, s[j + 4] & 63
        else:
            sc[j] = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
            mn[j] = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
    qs = blk[16:]
    e = np.arange(256)
    c, p = e // 64, e % 64
    if order == 0:
        byte = 32 * c + (p % 16) + 16 * (p // 32)
        hi = (p // 16) % 2
        sb = 2 * c + p // 32
    else:
        byte = 32 * c + p % 32
        hi = p // 32
        sb = 2 * c + p // 32
    nib = np.where(hi == 1, qs[byte] >> 4, qs[byte] & 0xF).astype(np.float32)
    d1 = (d * sc).astype(np.float32)
    dm = (dmin * mn).astype(np.float32)
    return ((d1[sb] * nib).astype(np.float32) - dm[sb]).astype(np.float32)


def test_q4k_dequant_random_bytes_both_orders(oracle):
    rng = np.random.default_rng(8)
    for _ in range(50):
        blk = rng.integers(0, 256, 144, dtype=np.uint8)
        blk[0:4] = (rng.standard_normal(2) * 0.01).astype(np.float16).view(np.uint8)
        for order in (0, 1):
            got = oracle.dequantize(Q4K, blk, [256], order=order)
            assert np.array_equal(got.view(np.uint32), q4k_decode_numpy(blk, order).view(np.uint32))


def exact_q4k_block(rng):
    k = rng.integers(1, 64, 8)
    mm = rng.integers(0, 64, 8)
    k[rng.integers(0, 8)] = 63
    mm[rng.integers(0, 8)] = 63
    q = np.zeros((8, 32), dtype=np.int64)
    for j in range(8):
        row = np.concatenate([[0, 15], rng.integers(0, 16, 30)])
        rng.shuffle(row)
        q[j] = row
    x = (k[:, None] * 2.0**-10 * q - mm[:, None] * 2.0**-9).astype(np.float32).reshape(-1)
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([2.0**-10], dtype=np.float16).view(np.uint8)
    blk[2:4] = np.array([2.0**-9], dtype=np.float16).view(np.uint8)
    blk[4:16] = pack_scales_k4(k, mm)
    L = q.reshape(-1)
    for c in range(4):  # k_quants.rs:946-951
        for l in range(32):
            blk[16 + 32 * c + l] = L[64 * c + l] | (L[64 * c + l + 32] << 4)
    return x, blk


def test_q4k_quantize_exact_grid_bytes(oracle):
    # Every sub-block lies exactly on a representable (scale, min) grid, so the whole super-block's
    # bytes are determined by the format alone: d = 2^-10, dmin = 2^-9, 6-bit (k, m), nibbles = q.
    rng = np.random.default_rng(9)
    xs, blks = zip(*[exact_q4k_block(rng) for _ in range(20)])
    got = oracle.quantize(Q4K, np.concatenate(xs))
    assert np.array_equal(got, np.concatenate(blks))
    # the inverse of the quantizer's packing is the GGML order, and it restores x exactly
    back = oracle.dequantize(Q4K, got, [20 * 256], order=oracle.ORDER_GGML)
    assert np.array_equal(back, np.concatenate(xs))
    # the reference's own dequantize order is NOT that inverse (documented reference quirk)
    back_ref = oracle.dequantize(Q4K, got, [20 * 256], order=oracle.ORDER_REF)
    assert not np.array_equal(back_ref, np.concatenate(xs))
    perm = np.concatenate([64 * c + np.concatenate([np.arange(16), 32 + np.arange(16), 16 + np.arange(16),
                                                     48 + np.arange(16)]) for c in range(4)])
    # REF order reads element positions through a fixed permutation and pairs them with the scale of
    # the half they are emitted in; check the permutation part on a block with one (k, m) everywhere
    q = rng.integers(0, 16, 256)
    q[:2] = [0, 15]
    x1 = (63 * 2.0**-10 * q - 63 * 2.0**-9).astype(np.float32)
    for j in range(8):
        x1[32 * j], x1[32 * j + 1] = np.float32(-63 * 2.0**-9), np.float32(63 * 2.0**-10 * 15 - 63 * 2.0**-9)
    b1 = oracle.quantize(Q4K, x1)
    assert np.array_equal(oracle.dequantize(Q4K, b1, [256], order=0), x1[perm])


def test_q4k_reference_roundtrip_bounds_and_edges(oracle):
    ramp = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)  # k_quants.rs:1446-1465
    b = oracle.quantize(Q4K, ramp)
    assert b.size == 144
    r = oracle.dequantize(Q4K, b, [256])
    assert np.sqrt(np.mean((r - ramp) ** 2)) < 0.15 and np.max(np.abs(r - ramp)) < 0.5
    g = oracle.dequantize(Q4K, b, [256], order=oracle.ORDER_GGML)
    assert np.sqrt(np.mean((g - ramp) ** 2)) < 0.02 and np.max(np.abs(g - ramp)) < 0.06
    assert not oracle.quantize(Q4K, np.zeros(512)).any()  # all-zero block -> all-zero bytes
    # trailing partial super-block is left all-zero (k_quants.rs:890-892)
    x = np.concatenate([ramp, ramp[:100]])
    out = oracle.quantize(Q4K, x)
    assert out.size == 288 and np.array_equal(out[:144], b) and not out[144:].any()
    rng = np.random.default_rng(10)
    w = (rng.standard_normal(256 * 64) * 0.02).astype(np.float32)
    bw = oracle.quantize(Q4K, w)
    gw = oracle.dequantize(Q4K, bw, [w.size], order=oracle.ORDER_GGML)
    assert np.sqrt(np.mean((gw - w) ** 2)) < 0.1 * 0.02


# ----------------------------------------------------------------------------------------------
# Q6_K
# ----------------------------------------------------------------------------------------------
def q6k_decode_numpy(blk):
    """Independent vectorised decode from the layout stated in the doc comment k_quants.rs:465-473."""
    d = blk[208:210].view(np.float16).astype(np.float32)[0]
    sc = blk[192:208].view(np.int8).astype(np.float32)
    e = np.arange(256)
    h, r = e // 128, e % 128
    g, l = r // 32, r % 32
    qlb = blk[64 * h + l + 32 * (g & 1)]
    nib = np.where(g >= 2, qlb >> 4, qlb & 0xF)
    hi2 = (blk[128 + 32 * h + l] >> (2 * g)) & 3
    q = (nib | (hi2 << 4)).astype(np.int32) - 32
    dsc = (d * sc[8 * h + 2 * g + l // 16]).astype(np.float32)
    return (dsc * q.astype(np.float32)).astype(np.float32)


def test_q6k_dequant_single_byte_probes_and_random(oracle):
    base = np.zeros(210, dtype=np.uint8)
    base[208:210] = np.array([1.0], dtype=np.float16).view(np.uint8)
    base[192:208] = 1
    zero = oracle.dequantize(Q6K, base, [256])
    assert np.all(zero == -32.0)
    b = base.copy()
    b[5] = 0x0F  # ql[5] low nibble -> element 5 (ys[l] uses ql[l] low)
    out = oracle.dequantize(Q6K, b, [256])
    assert out[5] == -17.0 and np.count_nonzero(out != -32.0) == 1
    b = base.copy()
    b[32 + 7] = 0xF0  # ql[l+32] high nibble -> ys[l+96]
    out = oracle.dequantize(Q6K, b, [256])
    assert out[96 + 7] == -17.0 and np.count_nonzero(out != -32.0) == 1
    b = base.copy()
    b[128 + 32 + 3] = 0b00001100  # qh of the second half, l=3, bits 2-3 -> ys[l+32] of chunk 1
    out = oracle.dequantize(Q6K, b, [256])
    assert out[128 + 32 + 3] == 16.0 and np.count_nonzero(out != -32.0) == 1
    b = base.copy()
    b[192 + 8 + 4 + 1] = 0xFE  # scale -2 for chunk 1, group 2, l >= 16
    out = oracle.dequantize(Q6K, b, [256])
    assert np.all(out[128 + 64 + 16: 128 + 64 + 32] == 64.0) and np.count_nonzero(out != -32.0) == 16
    rng = np.random.default_rng(11)
    for _ in range(50):
        blk = rng.integers(0, 256, 210, dtype=np.uint8)
        blk[208:210] = (rng.standard_normal(1) * 0.001).astype(np.float16).view(np.uint8)
        assert np.array_equal(oracle.dequantize(Q6K, blk, [256]).view(np.uint32),
                              q6k_decode_numpy(blk).view(np.uint32))


def exact_q6k_block(rng):
    k = rng.integers(1, 129, 16)
    k[rng.integers(0, 16)] = 128
    l = np.zeros((16, 16), dtype=np.int64)
    for j in range(16):
        row = np.concatenate([[-32], rng.integers(-31, 32, 15)])
        rng.shuffle(row)
        l[j] = row
    x = (k[:, None] * 2.0**-12 * l).astype(np.float32).reshape(-1)
    L = (l.reshape(-1) + 32).astype(np.uint8)
    blk = np.zeros(210, dtype=np.uint8)
    for h in range(2):  # k_quants.rs:1116-1130
        for i in range(32):
            a, c, e, g = (L[128 * h + i + 32 * t] for t in range(4))
            blk[64 * h + i] = (a & 0xF) | ((e & 0xF) << 4)
            blk[64 * h + i + 32] = (c & 0xF) | ((g & 0xF) << 4)
            blk[128 + 32 * h + i] = (a >> 4) | ((c >> 4) << 2) | ((e >> 4) << 4) | ((g >> 4) << 6)
    blk[192:208] = (-k).astype(np.int8).view(np.uint8)
    blk[208:210] = np.array([-(2.0**-12)], dtype=np.float16).view(np.uint8)
    return x, blk


def test_q6k_quantize_exact_grid_bytes(oracle):
    # x = k_j * 2^-12 * l on every 16-element sub-block with max k = 128: d must come out as
    # f16(-2^-12), the i8 scales as -k_j (k_quants.rs:1096-1102), and ql/qh must hold l + 32.
    rng = np.random.default_rng(12)
    xs, blks = zip(*[exact_q6k_block(rng) for _ in range(20)])
    got = oracle.quantize(Q6K, np.concatenate(xs))
    assert np.array_equal(got, np.concatenate(blks))
    assert np.array_equal(oracle.dequantize(Q6K, got, [20 * 256]), np.concatenate(xs))


def test_q6k_reference_roundtrip_bounds_and_edges(oracle):
    ramp = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)  # k_quants.rs:1490-1509
    b = oracle.quantize(Q6K, ramp)
    assert b.size == 210
    r = oracle.dequantize(Q6K, b, [256])
    assert np.sqrt(np.mean((r - ramp) ** 2)) < 0.1 and np.max(np.abs(r - ramp)) < 0.3
    assert np.max(np.abs(r - ramp)) < 0.025  # 6 bits over +-1.28
    z = oracle.quantize(Q6K, np.zeros(256))
    # all-zero block: iscale = -inf, d = f16(-0.0) (no zero guard in k_quants.rs:1096-1097)
    assert z[209] == 0x80 and z[208] == 0 and not z[:208].any()
    out = oracle.quantize(Q6K, np.concatenate([ramp, ramp[:17]]))
    assert out.size == 420 and np.array_equal(out[:210], b) and not out[210:].any()
    rng = np.random.default_rng(13)
    w = (rng.standard_normal(256 * 64) * 0.02).astype(np.float32)
    w[rng.integers(0, w.size, 16)] = 0.5
    bw = oracle.quantize(Q6K, w)
    assert np.all(bw.reshape(-1, 210)[:, 192:208].view(np.int8) >= -128)
    gw = oracle.dequantize(Q6K, bw, [w.size])
    assert np.sqrt(np.mean((gw - w) ** 2)) < 0.05 * 0.02 * 3


# ----------------------------------------------------------------------------------------------
# dispatchers and validation: quantize.rs:82-85, dequant.rs:184-216, tests dequant.rs:1139-1150
# ----------------------------------------------------------------------------------------------
def test_dispatch_errors(oracle):
    with pytest.raises(ValueError) as e:
        oracle.dequantize(Q4K, np.zeros(10, dtype=np.uint8), [256])
    assert e.value.args[0] == oracle.ERR_INVALID_SIZE
    with pytest.raises(ValueError) as e:
        oracle.dequantize(Q4K, np.zeros(0, dtype=np.uint8), [-1])
    assert e.value.args[0] == oracle.ERR_INVALID_SHAPE
    with pytest.raises(ValueError) as e:
        oracle.dequantize(Q4K, np.zeros(0, dtype=np.uint8), [2**31 - 1] * 3)
    assert e.value.args[0] == oracle.ERR_SHAPE_TOO_LARGE
    with pytest.raises(ValueError) as e:
        oracle.dequantize(99, np.zeros(0, dtype=np.uint8), [0])
    assert e.value.args[0] == oracle.ERR_UNSUPPORTED_TYPE
    assert oracle.dequantize(Q4K, np.zeros(0, dtype=np.uint8), [0, 5]).size == 0
    assert oracle.dequantize(Q6K, np.zeros(210 * 4, dtype=np.uint8), [2, 512]).size == 1024


# ----------------------------------------------------------------------------------------------
# Q4_K_M recipe: KATs crates/pmetal/src/commands/quantize.rs:1561-1608
# ----------------------------------------------------------------------------------------------
def test_recipe(oracle):
    L = oracle.lib()
    t = lambda name, nd, nl: L.pmo_q4km_tensor_type(name.encode(), nd, nl)
    assert t("blk.0.ffn_down.weight", 2, 32) == Q6K
    assert t("blk.0.attn_norm.weight", 1, 32) == 1  # F16
    assert t("output.weight", 2, 32) == Q6K and t("token_embd.weight", 2, 32) == Q6K
    assert t("blk.3.attn_q.weight", 2, 32) == Q4K and t("blk.4.ffn_down.weight", 2, 32) == Q4K
    assert t("blk.4.attn_v.weight", 2, 32) == Q4K and t("blk.6.attn_v.weight", 2, 32) == Q6K
    assert t("blk.6.attn_output.weight", 2, 32) == Q4K and t("blk.1.ffn_gate_inp.weight", 2, 32) == 1
    more = lambda n: [l for l in range(n) if L.pmo_use_more_bits(l, n)]
    assert more(28) == [0, 1, 2, 5, 8, 11, 14, 17, 20, 23, 24, 25, 26, 27]
    assert more(32) == [0, 1, 2, 3, 6, 9, 12, 15, 18, 21, 24, 27, 28, 29, 30, 31]
    assert more(0) == []
    # direct evaluation of the rule at commands/quantize.rs:988-993
    for n in (1, 7, 8, 16, 40):
        assert more(n) == [l for l in range(n) if l < n // 8 or l >= 7 * n // 8 or max(l - n // 8, 0) % 3 == 2]


# ----------------------------------------------------------------------------------------------
# dequantize-then-matmul against exact arithmetic on tiny shapes
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("t,k", [(Q8_0, 64), (Q4K, 512), (Q6K, 256)])
def test_qmatvec_brute_force(oracle, t, k):
    rng = np.random.default_rng(14)
    n = 5
    w = (rng.standard_normal(n * k) * 0.02).astype(np.float32)
    wq = oracle.quantize(t, w)
    x = rng.standard_normal(k).astype(np.float32)
    for order in ((0, 1) if t == Q4K else (0,)):
        deq = oracle.dequantize(t, wq, [n, k], order=order).reshape(n, k).astype(np.float64)
        want = (deq @ x.astype(np.float64)).astype(np.float32)
        assert np.array_equal(oracle.qmatvec(t, wq, n, k, x, order=order), want)
        f32 = oracle.qmatvec(t, wq, n, k, x, order=order, acc="f32")
        assert np.allclose(f32, want, rtol=1e-4, atol=1e-6)
        xm = rng.standard_normal((3, k)).astype(np.float32)
        ym = oracle.qmatmul(t, wq, n, k, xm, order=order)
        assert np.array_equal(ym, (xm.astype(np.float64) @ deq.T).astype(np.float32))
