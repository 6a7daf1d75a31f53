"""The 32-element formats beside Q8_0 (Q4_0, Q4_1, Q5_0, Q5_1, Q8_1): the oracle against the reference's own block
tests and against values that follow from the format definitions by hand; the HIP kernels against the oracle, bit for
bit.  Reference: crates/pmetal-gguf/src/quantize.rs:93-230, :302-359 and dequant.rs:300-463, :505-528."""
import numpy as np
import pytest

Q4_0, Q4_1, Q5_0, Q5_1, Q8_1 = 2, 3, 6, 7, 9
TYPES = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_1]
BYTES = {Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_1: 36}


def f16(v) -> bytes:
    return np.array([v], np.float16).tobytes()


def u8(b: bytes) -> np.ndarray:
    return np.frombuffer(b, dtype=np.uint8)


def test_sizes(oracle):
    for t in TYPES:
        assert oracle.lib().pmo_type_size(t) == BYTES[t] and oracle.lib().pmo_block_size(t) == 32  # types.rs:106-111, :150
        assert oracle.tensor_size(t, 33) == 2 * BYTES[t]


def test_reference_block_structure_tests(oracle):
    """dequant.rs:935-961 (Q4_0), :976-989 (Q4_1), :991-1017 (Q5_0, Q5_1), :1039-1053 (Q8_1), values as asserted there."""
    data = f16(1.0) + bytes(((i % 16 + 8) & 0xF) | ((((i + 1) % 16 + 8) & 0xF) << 4) for i in range(16))
    r = oracle.dequantize(Q4_0, u8(data), (32,))
    assert r.size == 32 and (r[0], r[1], r[16]) == (0.0, 1.0, 1.0)
    r = oracle.dequantize(Q4_1, u8(f16(0.5) + f16(1.0) + bytes([2 | (4 << 4)]) + bytes(15)), (32,))
    assert (r[0], r[16]) == (2.0, 3.0)
    r = oracle.dequantize(Q5_0, u8(f16(1.0) + (1).to_bytes(4, "little") + bytes([1 | (15 << 4)]) + bytes(15)), (32,))
    assert (r[0], r[16]) == (1.0, -1.0)
    r = oracle.dequantize(Q5_1, u8(f16(1.0) + f16(0.25) + (1).to_bytes(4, "little") + bytes([1 | (15 << 4)]) + bytes(15)), (32,))
    assert (r[0], r[16]) == (17.25, 15.25)
    r = oracle.dequantize(Q8_1, u8(f16(0.25) + f16(0.0) + bytes(range(32))), (32,))
    assert r.size == 32 and r[4] == 1.0


def test_dequantize_every_code_of_every_position(oracle):
    """Blocks written by hand from the format definitions: element i takes the low (i < 16) or high nibble of byte i % 16,
    its fifth bit is bit i of qh, and the value is (q - 8) d, q d + m, (q - 16) d, q d + m, q d.  Scales are powers of two
    and minima multiples of them, so every product and sum is exact and the expected values need no rounding model."""
    rng = np.random.default_rng(7)
    for t in TYPES:
        for trial in range(20):
            d = float(2.0 ** rng.integers(-6, 4))
            m = float(rng.integers(-40, 40)) * d
            if t == Q8_1:
                q = rng.integers(-128, 128, 32)
                blk = f16(d) + f16(123.0) + q.astype(np.int8).tobytes()  # the sum field is not read
                want = q * d
            else:
                qmax = 32 if t in (Q5_0, Q5_1) else 16
                q = rng.integers(0, qmax, 32)
                qs = bytes(int(q[i] & 15) | (int(q[i + 16] & 15) << 4) for i in range(16))
                qh = sum(int(q[i] >> 4) << i for i in range(32)).to_bytes(4, "little")
                if t == Q4_0:
                    blk, want = f16(d) + qs, (q - 8) * d
                elif t == Q4_1:
                    blk, want = f16(d) + f16(m) + qs, q * d + m
                elif t == Q5_0:
                    blk, want = f16(d) + qh + qs, (q - 16) * d
                else:
                    blk, want = f16(d) + f16(m) + qh + qs, q * d + m
            assert len(blk) == BYTES[t]
            got = oracle.dequantize(t, u8(blk), (32,))
            assert np.array_equal(got, want.astype(np.float32)), (t, trial)
            # truncation to the shape's element count (dequant.rs:330-331)
            assert np.array_equal(oracle.dequantize(t, u8(blk), (19,)), want[:19].astype(np.float32))


def grid_block(rng, lo, hi, step):
    """32 multiples of `step` between lo * step and hi * step, with both ends present."""
    k = rng.integers(lo, hi + 1, 32)
    k[rng.integers(0, 32)] = lo
    k[(np.argmin(k) + 5) % 32 if np.argmin(k) == np.argmax(k) else np.argmax(k)] = hi
    k[np.argmin(k)] = lo
    return k, (k * step).astype(np.float32)


def test_quantize_on_exact_grids(oracle):
    """Inputs on a power-of-two grid, where scale, reciprocal and every product are exact, so the codes follow from the
    definitions alone: Q4_1 / Q5_1 map k s -> k - kmin; Q8_1 with amax = 127 s maps k s -> k and stores the sum of the
    codes times d; Q4_0 / Q5_0 take d = max / -8 (-16) of the largest magnitude WITH ITS SIGN and round x / d + 8.5
    (16.5) half away from zero -- one above the unbiased code, which is what the reference computes."""
    rng = np.random.default_rng(11)
    for trial in range(50):
        s = float(2.0 ** rng.integers(-8, 6))
        # Q4_1: range exactly 15 steps
        k, x = grid_block(rng, -7, 8, s)
        got = oracle.quantize(Q4_1, x)
        q = k + 7
        want = f16(s) + f16(-7 * s) + bytes(int(q[i]) | (int(q[i + 16]) << 4) for i in range(16))
        assert got.tobytes() == want
        # Q5_1: range exactly 31 steps
        k, x = grid_block(rng, -10, 21, s)
        got = oracle.quantize(Q5_1, x)
        q = k + 10
        want = (f16(s) + f16(-10 * s) + sum(int(q[i] >> 4) << i for i in range(32)).to_bytes(4, "little") +
                bytes(int(q[i] & 15) | (int(q[i + 16] & 15) << 4) for i in range(16)))
        assert got.tobytes() == want
        # Q8_1: amax = 127 s
        k, x = grid_block(rng, -127, 100, s)
        got = oracle.quantize(Q8_1, x)
        want = f16(s) + f16(float(np.float32(int(k.sum())) * np.float32(s))) + k.astype(np.int8).tobytes()
        assert got.tobytes() == want
        # Q4_0: largest magnitude -8 s (negative), so d = s; code = round_half_away(k + 8.5) clamped to 15 = min(k + 9, 15)
        k, x = grid_block(rng, -8, 7, s)
        got = oracle.quantize(Q4_0, x)
        q = np.minimum(k + 9, 15)
        assert got.tobytes() == f16(s) + bytes(int(q[i]) | (int(q[i + 16]) << 4) for i in range(16))
        # the same magnitudes with the largest positive: d = -s, codes mirror: round_half_away(-k + 8.5)
        got = oracle.quantize(Q4_0, -x)
        q = np.minimum(k + 9, 15)
        assert got.tobytes() == f16(-s) + bytes(int(q[i]) | (int(q[i + 16]) << 4) for i in range(16))
        # Q5_0 likewise with -16 s
        k, x = grid_block(rng, -16, 15, s)
        got = oracle.quantize(Q5_0, x)
        q = np.minimum(k + 17, 31)
        assert got.tobytes() == (f16(s) + sum(int(q[i] >> 4) << i for i in range(32)).to_bytes(4, "little") +
                                 bytes(int(q[i] & 15) | (int(q[i + 16] & 15) << 4) for i in range(16)))


def test_quantize_special_blocks(oracle):
    zeros = np.zeros(32, np.float32)
    # all zeros: max = +0.0, d = +0.0 / -8.0 = -0.0 (Q4_0, Q5_0); codes round(0 * 0 + 8.5) = 9 and 17
    assert oracle.quantize(Q4_0, zeros).tobytes() == bytes([0x00, 0x80]) + bytes([0x99] * 16)
    assert oracle.quantize(Q5_0, zeros).tobytes() == bytes([0x00, 0x80]) + (0xFFFFFFFF).to_bytes(4, "little") + bytes([0x11] * 16)
    assert oracle.quantize(Q4_1, zeros).tobytes() == bytes(20) and oracle.quantize(Q5_1, zeros).tobytes() == bytes(24)
    assert oracle.quantize(Q8_1, zeros).tobytes() == bytes(36)
    # the first of two equal magnitudes gives the sign (strict > in the scan)
    x = zeros.copy()
    x[3], x[9] = 4.0, -4.0
    assert oracle.quantize(Q4_0, x)[:2].tobytes() == f16(-0.5)
    x[3], x[9] = -4.0, 4.0
    assert oracle.quantize(Q4_0, x)[:2].tobytes() == f16(0.5)
    # a short last block: minimum and maximum over the elements that exist, 0.0 quantized in the empty places
    x = np.array([3.0, 4.5, 6.0], np.float32)  # min 3, scale 3 / 15 = 0.2
    got = oracle.quantize(Q4_1, x)
    sc = np.float32(3.0) / np.float32(15.0)
    isc = np.float32(1.0) / sc
    code = lambda v: int(min(15, max(0, np.floor(abs(np.float32((np.float32(v) - np.float32(3.0)) * isc)) + np.float32(0.5)) * np.sign((v - 3.0) * 1.0))))
    want = f16(sc) + f16(3.0) + bytes([code(3.0) | (code(0.0) << 4), code(4.5) | (code(0.0) << 4), code(6.0) | (code(0.0) << 4)] +
                                      [code(0.0) | (code(0.0) << 4)] * 13)
    assert got.tobytes() == want and code(0.0) == 0 and code(6.0) == 15
    # non-finite values take no part in min / max (Q4_1, Q5_1) or the signed maximum (Q5_0); Q4_0 lets infinity in
    x = np.linspace(-1, 1, 32).astype(np.float32)
    y = x.copy()
    y[5], y[20] = np.inf, np.nan
    for t in (Q4_1, Q5_1, Q5_0):
        a, b = oracle.quantize(t, x), oracle.quantize(t, y)
        hdr = {Q4_1: 4, Q5_1: 4, Q5_0: 2}[t]
        assert a[:hdr].tobytes() == b[:hdr].tobytes()
    assert oracle.quantize(Q4_0, y)[:2].tobytes() == f16(-np.inf)


def test_round_trip_error_bounds(oracle):
    """|dequantize(quantize(x)) - x| stays within one step of the format (one and a half for the biased Q4_0 / Q5_0;
    the f16 rounding of the scale adds up to 2^-11 of the largest code)."""
    x = (np.random.default_rng(3).standard_normal(4096) * 0.3).astype(np.float32)
    for t, bound in ((Q4_0, 1.6 / 8), (Q5_0, 1.6 / 16), (Q4_1, 0.55 / 15 * 2), (Q5_1, 0.55 / 31 * 2), (Q8_1, 0.6 / 127)):
        y = oracle.dequantize(t, oracle.quantize(t, x), (4096,))
        blocks = np.abs(x.reshape(-1, 32)).max(axis=1, keepdims=True)
        assert (np.abs(y - x).reshape(-1, 32) <= bound * blocks * 1.02 + 1e-6).all(), t


def edge_inputs():
    rng = np.random.default_rng(5)
    cases = {
        "normal": (rng.standard_normal(32 * 97) * 0.02).astype(np.float32),
        "ragged": rng.standard_normal(32 * 5 + 19).astype(np.float32),
        "short": rng.standard_normal(3).astype(np.float32),
        "zeros": np.zeros(64, np.float32),
        "signed_zeros": np.where(np.arange(64) % 3 == 0, np.float32(-0.0), np.float32(0.0)).astype(np.float32),
        "constant": np.full(96, -0.37, np.float32),
        "ties": ((rng.integers(-31, 32, 32 * 40)) * 0.5).astype(np.float32),
        "equal_magnitudes": np.tile(np.array([2.0, -2.0, 1.0, -2.0], np.float32), 64) * np.repeat(rng.choice([-1.0, 1.0], 8), 32).astype(np.float32),
        "tiny": (rng.standard_normal(256) * 1e-41).astype(np.float32),
        "huge": (rng.standard_normal(256) * 1e37).astype(np.float32),
        "scale_spread": (rng.standard_normal(32 * 64) * np.repeat(np.exp(rng.uniform(-60, 60, 64)), 32)).astype(np.float32),
    }
    for name, bad in (("with_inf", np.inf), ("with_nan", np.nan)):
        x = rng.standard_normal(32 * 64).astype(np.float32)
        x[rng.integers(0, x.size, 30)] = bad
        x[rng.integers(0, x.size, 30)] = -bad
        x[32 * 7:32 * 8] = bad  # a whole block of it
        cases[name] = x
    return cases


@pytest.mark.gpu
@pytest.mark.parametrize("t", TYPES)
def test_gpu_quantize_and_dequantize_bit_exact(oracle, t):
    import pmetal_amd as pm
    from gpu_util import first_mismatch, gpu_dequantize_dev, gpu_quantize_dev
    pm.init(0)
    for name, x in edge_inputs().items():
        want = oracle.quantize(t, x)
        got = gpu_quantize_dev(t, x)
        assert np.array_equal(got, want), f"{name}: {first_mismatch(got, want, BYTES[t])}"
        assert np.array_equal(pm.quantize(x, t), want), name  # the host-pointer entry point
        back = gpu_dequantize_dev(t, want, x.size)
        assert np.array_equal(back.view(np.uint32), oracle.dequantize(t, want, (x.size,)).view(np.uint32)), name
    # arbitrary block bytes (every header pattern, NaN and infinite scales included)
    raw = np.random.default_rng(9).integers(0, 256, BYTES[t] * 4096, dtype=np.uint8)
    n = 32 * 4096 - 7
    got = gpu_dequantize_dev(t, raw, n)
    want = oracle.dequantize(t, raw, (n,))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(pm.dequantize(raw, t, (n,)).view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
def test_gpu_legacy_types_have_no_linear_kernels():
    import pmetal_amd as pm
    from pmetal_amd import _lib
    pm.init(0)
    lib = _lib.load()
    buf = pm.DeviceBuffer(4096)
    for t in TYPES:
        assert lib.pmetal_hip_is_supported(t) == 1
        assert lib.pmetal_hip_qgemv(t, buf.ptr, 4, 32, buf.ptr, 1, buf.ptr, 0, None) == 2  # unsupported type
