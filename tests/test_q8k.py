"""Q8_K activation blocks and the integer dot products over them (crates/pmetal-gguf/src/k_quants.rs:815-871,
vec_dot.rs:617-810): the oracle against what pins it, then the HIP kernels against the oracle, bit for bit."""
import struct

import numpy as np
import pytest

Q4K, Q6K = 12, 14
Q2K, Q3K, Q5K = 10, 11, 13


# ---------------------------------------------------------------------------------------------------------------------
# oracle pins (CPU)
# ---------------------------------------------------------------------------------------------------------------------
def q8k_block(d: float, qs) -> bytes:
    """make_test_q8k (vec_dot.rs:892-909): the block a list of int8 values makes, sums included."""
    q = np.zeros(256, dtype=np.int8)
    q[:len(qs)] = qs
    bsums = q.reshape(16, 16).astype(np.int32).sum(axis=1).astype(np.int16)
    return struct.pack("<f", d) + q.tobytes() + bsums.tobytes()


def q4k_block(d: float, dmin: float, sc, m, nibbles) -> bytes:
    """A Q4_K super-block from its parts: 8 scales and mins (6 bits), 256 quants in the quantizer's packing
    (k_quants.rs:915-926 and :946-951): qs[32 c + l] = L[64 c + l] | L[64 c + l + 32] << 4."""
    scales = np.zeros(12, dtype=np.uint8)
    for j in range(8):
        if j < 4:
            scales[j] |= sc[j] & 63
            scales[j + 4] |= m[j] & 63
        else:
            scales[j + 4] = (sc[j] & 0xF) | ((m[j] & 0xF) << 4)
            scales[j - 4] |= (sc[j] >> 4) << 6
            scales[j] |= (m[j] >> 4) << 6
    L = np.asarray(nibbles, dtype=np.uint8).reshape(4, 2, 32)
    qs = (L[:, 0, :] | (L[:, 1, :] << 4)).reshape(-1)
    return np.float16(d).tobytes() + np.float16(dmin).tobytes() + scales.tobytes() + qs.tobytes()


def q6k_block_linear(d: float, scales, q) -> bytes:
    """A Q6_K super-block whose element idx, *in the order the reference's dot product reads it* (vec_dot.rs:665-686),
    is q[idx] (0..63): nibble idx % 2 of ql[idx / 2], bits 2 (idx % 4) of qh[idx / 4]."""
    q = np.asarray(q, dtype=np.uint8)
    ql, qh = np.zeros(128, dtype=np.uint8), np.zeros(64, dtype=np.uint8)
    for idx in range(256):
        ql[idx // 2] |= (q[idx] & 0xF) << (4 * (idx % 2))
        qh[idx // 4] |= (q[idx] >> 4) << (2 * (idx % 4))
    return ql.tobytes() + qh.tobytes() + np.asarray(scales, dtype=np.int8).tobytes() + np.float16(d).tobytes()


def test_quantize_q8k_known_answers(oracle):
    assert oracle.lib().pmo_q8k_size(256) == 292 and oracle.lib().pmo_q8k_size(257) == 584 and oracle.lib().pmo_q8k_size(0) == 0
    # all zeros -> an all-zero block (k_quants.rs:846-851, :1557-1559)
    assert not oracle.quantize_q8k(np.zeros(256, np.float32)).any()
    # the reference's round-trip ramp (k_quants.rs:1421-1443): x = (i - 128) / 100; the largest magnitude is x[0] =
    # -1.28, so iscale = -128 / -1.28 = 100 (to a rounding), q[i] = round(100 x[i]) = i - 128 with 127 the cap
    x = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    blk = oracle.quantize_q8k(x)
    d, = struct.unpack("<f", blk[:4].tobytes())
    q = blk[4:260].view(np.int8)
    assert np.array_equal(q, np.arange(256) - 128)
    assert abs(d - 0.01) < 1e-8
    assert np.array_equal(blk[260:].view(np.int16), (np.arange(256) - 128).reshape(16, 16).sum(axis=1))
    restored = d * q.astype(np.float32)
    assert np.sqrt(np.mean((restored - x) ** 2)) < 0.01 and np.abs(restored - x).max() < 0.02
    # positive maximum: it maps to -128 and the scale is negative; an equal negative value would be +128, capped at 127
    x = np.zeros(256, np.float32)
    x[3], x[9], x[200] = 2.0, -2.0, 1.0
    blk = oracle.quantize_q8k(x)
    d, = struct.unpack("<f", blk[:4].tobytes())
    q = blk[4:260].view(np.int8)
    assert d == np.float32(-1.0 / 64.0) and q[3] == -128 and q[9] == 127 and q[200] == -64
    # the first of two equal magnitudes decides the sign
    x[3], x[9] = -2.0, 2.0
    q = oracle.quantize_q8k(x)[4:260].view(np.int8)
    assert q[3] == -128 and q[9] == 127 and q[200] == 64
    # a trailing partial block stays zero, full blocks before it are quantized (k_quants.rs:829-834)
    blk = oracle.quantize_q8k(np.ones(300, np.float32))
    assert blk.size == 584 and not blk[292:].any() and (blk[4:260].view(np.int8) == -128).all()
    # half-away rounding and the cap: max 128 -> iscale -1; 0.5 -> -0.5 -> -1 (away); -126.5 -> 126.5 -> 127
    x = np.zeros(256, np.float32)
    x[0], x[1], x[2], x[3] = 128.0, 0.5, -126.5, -127.6
    q = oracle.quantize_q8k(x)[4:260].view(np.int8)
    assert list(q[:4]) == [-128, -1, 127, 127]


def test_vec_dot_q4k_q8k_known_answers(oracle):
    ones = q8k_block(1.0, [1] * 256)
    # quants 1 (low half of each 64-chunk) and 2 (high half), all scales 1, no mins: sum = 128 * 1 + 128 * 2
    L = np.tile(np.concatenate([np.full(32, 1), np.full(32, 2)]), 4)
    blk = q4k_block(1.0, 0.0, [1] * 8, [0] * 8, L)
    assert oracle.vec_dot_q8k(Q4K, np.frombuffer(blk, np.uint8), np.frombuffer(ones, np.uint8), 1) == 384.0
    # the min term: m_j = 3 on the first four sub-blocks, dmin = 1 -> minus 3 * 32 * 4
    blk = q4k_block(1.0, 1.0, [1] * 8, [3, 3, 3, 3, 0, 0, 0, 0], L)
    assert oracle.vec_dot_q8k(Q4K, np.frombuffer(blk, np.uint8), np.frombuffer(ones, np.uint8), 1) == 0.0
    # one non-zero quant and one non-zero activation: only the matching position counts, with its sub-block's scale
    rng = np.random.default_rng(0)
    for _ in range(200):
        e, f = int(rng.integers(256)), int(rng.integers(256))
        sc = [int(v) for v in rng.integers(1, 64, 8)]
        L = np.zeros(256, np.uint8)
        L[e] = 7
        a = np.zeros(256, np.int8)
        a[f] = -5
        blk = q4k_block(2.0, 0.0, sc, [0] * 8, L)
        got = oracle.vec_dot_q8k(Q4K, np.frombuffer(blk, np.uint8), np.frombuffer(q8k_block(0.5, a), np.uint8), 1)
        assert got == (2.0 * 0.5 * 7 * -5 * sc[e // 32] if e == f else 0.0), (e, f)
    # against dequantize-then-dot in f64: the dot product is sum W[i] (yd q8[i]) with W in the quantizer's order
    x = (rng.standard_normal(4 * 256) * 0.05).astype(np.float32)
    w = oracle.quantize(Q4K, x)
    act = rng.standard_normal(4 * 256).astype(np.float32)
    xq = oracle.quantize_q8k(act)
    got = oracle.vec_dot_q8k(Q4K, w, xq, 4)
    wd = oracle.dequantize(Q4K, w, [4 * 256], order=oracle.ORDER_GGML).astype(np.float64)
    blocks = xq.reshape(4, 292)
    aq = np.concatenate([b[:4].view(np.float32).astype(np.float64) * b[4:260].view(np.int8).astype(np.float64) for b in blocks])
    want = float(wd @ aq)
    assert abs(got - want) <= 1e-5 * np.abs(wd * aq).sum()
    # ... and NOT in the reference dequantizer's own order (the two orders differ on real data)
    wr = oracle.dequantize(Q4K, w, [4 * 256], order=oracle.ORDER_REF).astype(np.float64)
    assert abs(got - float(wr @ aq)) > 1e-3 * abs(want)


def test_vec_dot_q6k_q8k_known_answers(oracle):
    ones = q8k_block(1.0, [1] * 256)
    # q = 33 everywhere (value +1 after the -32), scales 2: 256 * 1 * 2
    blk = q6k_block_linear(1.0, [2] * 16, [33] * 256)
    assert oracle.vec_dot_q8k(Q6K, np.frombuffer(blk, np.uint8), np.frombuffer(ones, np.uint8), 1) == 512.0
    # q = 32 is zero: nothing, whatever the scales; q = 0 is -32
    blk = q6k_block_linear(1.0, list(range(-8, 8)), [32] * 256)
    assert oracle.vec_dot_q8k(Q6K, np.frombuffer(blk, np.uint8), np.frombuffer(ones, np.uint8), 1) == 0.0
    blk = q6k_block_linear(0.5, [1] * 16, [0] * 256)
    assert oracle.vec_dot_q8k(Q6K, np.frombuffer(blk, np.uint8), np.frombuffer(ones, np.uint8), 1) == 0.5 * -32 * 256
    rng = np.random.default_rng(1)
    for _ in range(200):  # a single position: its scale is scales[idx / 16], negative scales included
        e, f = int(rng.integers(256)), int(rng.integers(256))
        scales = [int(v) for v in rng.integers(-128, 128, 16)]
        q = np.full(256, 32, np.uint8)
        q[e] = int(rng.integers(0, 64))
        a = np.zeros(256, np.int8)
        a[f] = 9
        blk = q6k_block_linear(1.0, scales, q)
        got = oracle.vec_dot_q8k(Q6K, np.frombuffer(blk, np.uint8), np.frombuffer(q8k_block(1.0, a), np.uint8), 1)
        assert got == (float((int(q[e]) - 32) * 9 * scales[e // 16]) if e == f else 0.0), (e, f)
    # several blocks: the float sum runs over the blocks in order (an f32 sum of exact per-block products)
    blocks_w, blocks_a, want = b"", b"", np.float32(0)
    for b in range(5):
        scales = [int(v) for v in rng.integers(-20, 20, 16)]
        q = rng.integers(0, 64, 256).astype(np.uint8)
        a = rng.integers(-127, 128, 256).astype(np.int8)
        d, yd = np.float16(rng.uniform(0.001, 0.01)), np.float32(rng.uniform(0.01, 0.1))
        blocks_w += q6k_block_linear(float(d), scales, q)
        blocks_a += q8k_block(float(yd), a)
        sumi = int(((q.astype(np.int64) - 32) * a.astype(np.int64) * np.repeat(scales, 16)).sum())
        want = np.float32(want + np.float32(np.float32(np.float32(d) * yd) * np.float32(sumi)))
    got = oracle.vec_dot_q8k(Q6K, np.frombuffer(blocks_w, np.uint8), np.frombuffer(blocks_a, np.uint8), 5)
    assert np.float32(got) == want


def k4_scales(sc, m) -> bytes:
    """The 12 scale bytes of a Q4_K / Q5_K super-block from 8 scales and 8 mins of 6 bits (k_quants.rs:915-926)."""
    scales = np.zeros(12, dtype=np.uint8)
    for j in range(8):
        if j < 4:
            scales[j] |= sc[j] & 63
            scales[j + 4] |= m[j] & 63
        else:
            scales[j + 4] = (sc[j] & 0xF) | ((m[j] & 0xF) << 4)
            scales[j - 4] |= (sc[j] >> 4) << 6
            scales[j] |= (m[j] >> 4) << 6
    return scales.tobytes()


def q5k_block_linear(d: float, dmin: float, sc, m, q) -> bytes:
    """A Q5_K super-block (d, dmin, scales[12], qh[32], qs[128]) whose element j, in the order the reference's dot product
    reads it (vec_dot.rs:712-731), is q[j] (0..31): nibble j % 2 of qs[j / 2], bit j % 8 of qh[j / 8]."""
    q = np.asarray(q, dtype=np.uint8)
    qs, qh = np.zeros(128, dtype=np.uint8), np.zeros(32, dtype=np.uint8)
    for j in range(256):
        qs[j // 2] |= (q[j] & 0xF) << (4 * (j % 2))
        qh[j // 8] |= (q[j] >> 4) << (j % 8)
    return np.float16(d).tobytes() + np.float16(dmin).tobytes() + k4_scales(sc, m) + qh.tobytes() + qs.tobytes()


def q2k_block_linear(d: float, dmin: float, sc, m, q) -> bytes:
    """A Q2_K super-block (scales[16], qs[64], d, dmin) whose element j, in the order of vec_dot.rs:796-803, is q[j]
    (0..3): bits 2 (j % 4) of qs[j / 4]; scales[g] = sc[g] | m[g] << 4."""
    q = np.asarray(q, dtype=np.uint8)
    qs = np.zeros(64, dtype=np.uint8)
    for j in range(256):
        qs[j // 4] |= (q[j] & 3) << (2 * (j % 4))
    scales = np.array([(sc[g] & 0xF) | ((m[g] & 0xF) << 4) for g in range(16)], dtype=np.uint8)
    return scales.tobytes() + qs.tobytes() + np.float16(d).tobytes() + np.float16(dmin).tobytes()


def q3k_block_linear(d: float, scale_bytes, q) -> bytes:
    """A Q3_K super-block (hmask[32], qs[64], scales[12], d) whose element j, in the order of vec_dot.rs:757-771, is
    q[j] (0..7, value q - 4): bits 2 (j % 4) of qs[j / 4], bit j % 8 of hmask[j / 8]."""
    q = np.asarray(q, dtype=np.uint8)
    qs, hm = np.zeros(64, dtype=np.uint8), np.zeros(32, dtype=np.uint8)
    for j in range(256):
        qs[j // 4] |= (q[j] & 3) << (2 * (j % 4))
        hm[j // 8] |= (q[j] >> 2) << (j % 8)
    return hm.tobytes() + qs.tobytes() + np.asarray(scale_bytes, dtype=np.uint8).tobytes() + np.float16(d).tobytes()


def test_vec_dot_q5k_q8k_known_answers(oracle):
    ones = np.frombuffer(q8k_block(1.0, [1] * 256), np.uint8)
    # q = 17 everywhere (fifth bit and low nibble 1), all scales 2, no mins: 256 * 17 * 2
    blk = q5k_block_linear(1.0, 0.0, [2] * 8, [0] * 8, [17] * 256)
    assert oracle.vec_dot_q8k(Q5K, np.frombuffer(blk, np.uint8), ones, 1) == 256 * 17 * 2
    # the min term: m = 5 on sub-blocks 0 and 7 (the two forms of the 6-bit packing), dmin = 0.5 -> minus 0.5 * 5 * 32 * 2
    blk = q5k_block_linear(1.0, 0.5, [0] * 8, [5, 0, 0, 0, 0, 0, 0, 5], [31] * 256)
    assert oracle.vec_dot_q8k(Q5K, np.frombuffer(blk, np.uint8), ones, 1) == -160.0
    rng = np.random.default_rng(5)
    for _ in range(300):  # a single position: quant, activation and the scale of sub-block e / 32 (scales up to 63)
        e, f = int(rng.integers(256)), int(rng.integers(256))
        sc = [int(v) for v in rng.integers(1, 64, 8)]
        q = np.zeros(256, np.uint8)
        q[e] = int(rng.integers(1, 32))
        a = np.zeros(256, np.int8)
        a[f] = -7
        blk = q5k_block_linear(2.0, 0.0, sc, [0] * 8, q)
        got = oracle.vec_dot_q8k(Q5K, np.frombuffer(blk, np.uint8), np.frombuffer(q8k_block(0.5, a), np.uint8), 1)
        assert got == (2.0 * 0.5 * int(q[e]) * -7 * sc[e // 32] if e == f else 0.0), (e, f)
    # several blocks, every field random: integer sums per block, then the f32 recurrence of the routine in block order
    w, x, want = b"", b"", np.float32(0)
    for b in range(4):
        sc, m = [int(v) for v in rng.integers(0, 64, 8)], [int(v) for v in rng.integers(0, 64, 8)]
        q = rng.integers(0, 32, 256).astype(np.uint8)
        a = rng.integers(-127, 128, 256).astype(np.int8)
        d, dmin, yd = np.float16(rng.uniform(0.001, 0.01)), np.float16(rng.uniform(0.001, 0.01)), np.float32(rng.uniform(0.01, 0.1))
        w += q5k_block_linear(float(d), float(dmin), sc, m, q)
        x += q8k_block(float(yd), a)
        mins = int((np.array(m, np.int64) * a.astype(np.int64).reshape(8, 32).sum(1)).sum())
        sumi = int((q.astype(np.int64) * a.astype(np.int64) * np.repeat(sc, 32)).sum())
        want = np.float32(want - np.float32(np.float32(np.float32(dmin) * yd) * np.float32(mins)))
        want = np.float32(want + np.float32(np.float32(np.float32(d) * yd) * np.float32(sumi)))
    assert np.float32(oracle.vec_dot_q8k(Q5K, np.frombuffer(w, np.uint8), np.frombuffer(x, np.uint8), 4)) == want


def test_vec_dot_q2k_q8k_known_answers(oracle):
    ones = np.frombuffer(q8k_block(1.0, [1] * 256), np.uint8)
    blk = q2k_block_linear(1.0, 0.0, [3] * 16, [0] * 16, [2] * 256)   # 256 * 2 * 3
    assert oracle.vec_dot_q8k(Q2K, np.frombuffer(blk, np.uint8), ones, 1) == 1536.0
    blk = q2k_block_linear(1.0, 0.25, [0] * 16, [15] + [0] * 14 + [1], [3] * 256)  # minus 0.25 * (15 * 16 + 1 * 16)
    assert oracle.vec_dot_q8k(Q2K, np.frombuffer(blk, np.uint8), ones, 1) == -64.0
    rng = np.random.default_rng(6)
    for _ in range(300):
        e, f = int(rng.integers(256)), int(rng.integers(256))
        sc = [int(v) for v in rng.integers(1, 16, 16)]
        q = np.zeros(256, np.uint8)
        q[e] = int(rng.integers(1, 4))
        a = np.zeros(256, np.int8)
        a[f] = 11
        blk = q2k_block_linear(1.0, 0.0, sc, [0] * 16, q)
        got = oracle.vec_dot_q8k(Q2K, np.frombuffer(blk, np.uint8), np.frombuffer(q8k_block(1.0, a), np.uint8), 1)
        assert got == (float(int(q[e]) * 11 * sc[e // 16]) if e == f else 0.0), (e, f)
    w, x, want = b"", b"", np.float32(0)
    for b in range(4):
        sc, m = [int(v) for v in rng.integers(0, 16, 16)], [int(v) for v in rng.integers(0, 16, 16)]
        q = rng.integers(0, 4, 256).astype(np.uint8)
        a = rng.integers(-127, 128, 256).astype(np.int8)
        d, dmin, yd = np.float16(rng.uniform(0.001, 0.01)), np.float16(rng.uniform(0.001, 0.01)), np.float32(rng.uniform(0.01, 0.1))
        w += q2k_block_linear(float(d), float(dmin), sc, m, q)
        x += q8k_block(float(yd), a)
        mins = int((np.array(m, np.int64) * a.astype(np.int64).reshape(16, 16).sum(1)).sum())
        sumi = int((q.astype(np.int64) * a.astype(np.int64) * np.repeat(sc, 16)).sum())
        want = np.float32(want - np.float32(np.float32(np.float32(dmin) * yd) * np.float32(mins)))
        want = np.float32(want + np.float32(np.float32(np.float32(d) * yd) * np.float32(sumi)))
    assert np.float32(oracle.vec_dot_q8k(Q2K, np.frombuffer(w, np.uint8), np.frombuffer(x, np.uint8), 4)) == want


def test_vec_dot_q3k_q8k_known_answers(oracle):
    ones = np.frombuffer(q8k_block(1.0, [1] * 256), np.uint8)
    # scale nibbles 9 (value +1) in the first four bytes, q = 7 (value 3) everywhere: the first 128 elements count with
    # scale 1, the last 128 with the zero that the routine leaves there -> 128 * 3
    blk = q3k_block_linear(1.0, [0x99] * 4 + [0xFF] * 8, [7] * 256)
    assert oracle.vec_dot_q8k(Q3K, np.frombuffer(blk, np.uint8), ones, 1) == 384.0
    # nibble 0 is scale -8; q = 0 is value -4: 128 * (-4) * (-8)
    blk = q3k_block_linear(0.5, [0x00] * 12, [0] * 256)
    assert oracle.vec_dot_q8k(Q3K, np.frombuffer(blk, np.uint8), ones, 1) == 0.5 * 128 * 32
    rng = np.random.default_rng(7)
    for _ in range(300):  # a single position: every other quant is 4 (value 0)
        e, f = int(rng.integers(256)), int(rng.integers(256))
        sb = [int(v) for v in rng.integers(0, 256, 12)]
        q = np.full(256, 4, np.uint8)
        q[e] = int(rng.integers(0, 8))
        a = np.zeros(256, np.int8)
        a[f] = 13
        blk = q3k_block_linear(1.0, sb, q)
        got = oracle.vec_dot_q8k(Q3K, np.frombuffer(blk, np.uint8), np.frombuffer(q8k_block(1.0, a), np.uint8), 1)
        g = e // 16
        scale = (((sb[g // 2] >> (4 * (g % 2))) & 0xF) - 8) if g < 8 else 0
        assert got == (float((int(q[e]) - 4) * 13 * scale) if e == f else 0.0), (e, f, g)
    w, x, want = b"", b"", np.float32(0)
    for b in range(4):
        sb = [int(v) for v in rng.integers(0, 256, 12)]
        q = rng.integers(0, 8, 256).astype(np.uint8)
        a = rng.integers(-127, 128, 256).astype(np.int8)
        d, yd = np.float16(rng.uniform(0.001, 0.01)), np.float32(rng.uniform(0.01, 0.1))
        w += q3k_block_linear(float(d), sb, q)
        x += q8k_block(float(yd), a)
        scales = np.array([(((sb[g // 2] >> (4 * (g % 2))) & 0xF) - 8) if g < 8 else 0 for g in range(16)], np.int64)
        sumi = int(((q.astype(np.int64) - 4) * a.astype(np.int64) * np.repeat(scales, 16)).sum())
        want = np.float32(want + np.float32(np.float32(np.float32(d) * yd) * np.float32(sumi)))
    assert np.float32(oracle.vec_dot_q8k(Q3K, np.frombuffer(w, np.uint8), np.frombuffer(x, np.uint8), 4)) == want


# ---------------------------------------------------------------------------------------------------------------------
# HIP kernels against the oracle (GPU)
# ---------------------------------------------------------------------------------------------------------------------
def gpu_quantize_q8k(x):
    import pmetal_amd as pm
    from pmetal_amd import gguf
    x = np.ascontiguousarray(x, dtype=np.float32)
    dx = pm.DeviceBuffer.from_host(x) if x.size else pm.DeviceBuffer(16)
    nbytes = gguf.q8k_size(x.size)
    out = pm.DeviceBuffer(max(nbytes, 16))
    pm.check(pm._lib.load().pmetal_hip_memset(out.ptr, 0xA5, max(nbytes, 16), None))  # every byte must be written
    gguf.quantize_q8k_dev(dx, x.size, out)
    pm.check(pm._lib.load().pmetal_hip_sync(None))
    return out.to_host(np.uint8, nbytes)


@pytest.mark.gpu
def test_gpu_quantize_q8k_bit_exact(oracle):
    import pmetal_amd as pm
    pm.init(0)
    rng = np.random.default_rng(4)
    ties = np.zeros(512, np.float32)
    ties[0], ties[256] = 128.0, -64.0
    ties[1:200] = (np.arange(199) - 99) * 0.5
    ties[257:400] = (np.arange(143) - 71) * 0.25
    equal = np.zeros(256, np.float32)
    equal[77], equal[13], equal[200] = 3.0, -3.0, 3.0  # the first of equal magnitudes (index 13) decides
    cases = {
        "normal": rng.standard_normal(1 << 18).astype(np.float32),
        "ramp": ((np.arange(256) - 128.0) * 0.01).astype(np.float32),
        "zeros": np.zeros(512, np.float32),
        "ties": ties, "equal_magnitudes": equal,
        "ragged": rng.standard_normal(256 * 3 + 100).astype(np.float32), "short": rng.standard_normal(17).astype(np.float32),
        "scales": (rng.standard_normal(1 << 14) * np.repeat(np.exp(rng.uniform(-60, 60, 64)), 256)).astype(np.float32),
        "denormal": (rng.standard_normal(512) * 1e-41).astype(np.float32),
        "signed_zero": np.where(np.arange(512) % 2 == 0, np.float32(0.0), np.float32(-0.0)).astype(np.float32),
    }
    for bad in (np.inf, np.nan):
        x = rng.standard_normal(1 << 12).astype(np.float32)
        x[rng.integers(0, x.size, 9)] = bad
        x[rng.integers(0, x.size, 9)] = -bad
        cases[f"with_{bad}"] = x
    for name, x in cases.items():
        want, got = oracle.quantize_q8k(x), gpu_quantize_q8k(x)
        bad = np.nonzero(want != got)[0]
        assert bad.size == 0, (name, bad[:8], want[bad[:8]], got[bad[:8]])
    assert gpu_quantize_q8k(np.zeros(0, np.float32)).size == 0
    lib = pm._lib.load()
    assert lib.pmetal_hip_quantize_q8k_dev(None, 256, None, 291, None) == 3  # wrong size comes first
    lib.pmetal_hip_clear_error()


@pytest.mark.gpu
@pytest.mark.parametrize("t", [Q4K, Q6K, Q5K, Q3K, Q2K])
@pytest.mark.parametrize("n,k", [(1, 256), (7, 512), (300, 1024), (64, 4096), (1000, 2048), (4096, 4096), (33, 32768), (513, 2304)])
def test_gpu_qgemv_q8k_bit_exact(oracle, t, n, k):
    import pmetal_amd as pm
    from gpu_util import weights
    from pmetal_amd import gguf
    pm.init(0)
    rng = np.random.default_rng(n * 31 + k + t)
    wq = oracle.quantize(t, weights(n + k + t, n * k, outliers=1e-3))
    act = (rng.standard_normal(k) * np.repeat(np.exp(rng.uniform(-3, 3, k // 256)), 256)).astype(np.float32)
    xq = oracle.quantize_q8k(act)
    want = oracle.qmatvec_q8k(t, wq, n, k, xq)
    dw, dxq = pm.DeviceBuffer.from_host(wq), pm.DeviceBuffer.from_host(xq)
    dy = pm.DeviceBuffer(max(4 * n, 16))
    pm.check(pm._lib.load().pmetal_hip_memset(dy.ptr, 0xFF, max(4 * n, 16), None))
    gguf.qgemv_q8k(t, dw, n, k, dxq, dy)
    pm.check(pm._lib.load().pmetal_hip_sync(None))
    got = dy.to_host(np.float32, n)
    bad = np.nonzero(got.view(np.uint32) != want.view(np.uint32))[0]
    assert bad.size == 0, (bad[:5], got[bad[:5]], want[bad[:5]])
    # the activation quantizer on the device feeds the same bits
    dact = pm.DeviceBuffer.from_host(act)
    dxq2 = gguf.quantize_q8k_dev(dact, k)
    pm.check(pm._lib.load().pmetal_hip_sync(None))
    assert np.array_equal(dxq2.to_host(np.uint8, xq.size), xq)


@pytest.mark.gpu
@pytest.mark.parametrize("t,block,d_at", [(Q5K, 176, (0, 2)), (Q3K, 110, (108,)), (Q2K, 84, (80, 82))])
def test_gpu_qgemv_q8k_random_block_bytes(oracle, t, block, d_at):
    """Every scale, min, quant and high-bit pattern: random block bytes with finite d / dmin of both signs, rows that start
    at every alignment the block size allows (odd numbers of super-blocks), activations over the whole int8 range."""
    import pmetal_amd as pm
    from pmetal_amd import gguf
    pm.init(0)
    rng = np.random.default_rng(t)
    for n, k in ((37, 256 * 3), (260, 256 * 7), (1025, 2048)):
        spr = k // 256
        raw = rng.integers(0, 256, size=(n * spr, block), dtype=np.uint8)
        for off in d_at:
            vals = (rng.uniform(0.001, 0.05, n * spr) * rng.choice([-1.0, 1.0], n * spr)).astype(np.float16)
            raw[:, off:off + 2] = vals.view(np.uint8).reshape(-1, 2)
        raw = raw.reshape(-1)
        xq = np.concatenate([np.frombuffer(q8k_block(float(rng.uniform(0.01, 0.1)), rng.integers(-128, 128, 256).astype(np.int8)), np.uint8)
                             for _ in range(spr)])
        want = oracle.qmatvec_q8k(t, raw, n, k, xq)
        dw, dxq, dy = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer.from_host(xq), pm.DeviceBuffer(max(4 * n, 16))
        gguf.qgemv_q8k(t, dw, n, k, dxq, dy)
        pm.check(pm._lib.load().pmetal_hip_sync(None))
        got = dy.to_host(np.float32, n)
        bad = np.nonzero(got.view(np.uint32) != want.view(np.uint32))[0]
        assert bad.size == 0, (t, n, k, bad[:5], got[bad[:5]], want[bad[:5]])


@pytest.mark.gpu
def test_gpu_qgemv_q8k_argument_errors():
    import pmetal_amd as pm
    pm.init(0)
    lib = pm._lib.load()
    buf = pm.DeviceBuffer(1 << 16)
    assert lib.pmetal_hip_qgemv_q8k(8, buf.ptr, 4, 256, buf.ptr, buf.ptr, None) == 2      # Q8_0 weights: no such product
    assert lib.pmetal_hip_qgemv_q8k(15, buf.ptr, 4, 256, buf.ptr, buf.ptr, None) == 2     # nor Q8_K against Q8_K
    assert lib.pmetal_hip_qgemv_q8k(Q4K, buf.ptr, 4, 300, buf.ptr, buf.ptr, None) == 6    # k not a multiple of 256
    assert lib.pmetal_hip_qgemv_q8k(Q4K, buf.ptr, 4, 65536, buf.ptr, buf.ptr, None) == 6  # k too long for LDS
    assert lib.pmetal_hip_qgemv_q8k(Q4K, None, 4, 256, buf.ptr, buf.ptr, None) == 1
    assert lib.pmetal_hip_qgemv_q8k(Q4K, buf.ptr, 0, 256, buf.ptr, buf.ptr, None) == 0    # no rows: nothing to do
    lib.pmetal_hip_clear_error()
