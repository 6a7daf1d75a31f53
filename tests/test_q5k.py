"""Q5_K quantize / dequantize (crates/pmetal-gguf/src/k_quants.rs:960-1051, :407-462): the oracle against what pins it,
the HIP kernels against the oracle bit for bit.  Q5_K is what the Q4_K_M recipe gives a fused attn_qkv tensor."""
import numpy as np
import pytest

Q5K = 13


def q5k_block(d, dmin, sc, m, L):
    """A block from its parts, packed as quantize_q5k packs (k_quants.rs:997-1008, :1027-1047)."""
    scales = np.zeros(12, dtype=np.uint8)
    for j in range(8):
        if j < 4:
            scales[j] |= sc[j] & 63
            scales[j + 4] |= m[j] & 63
        else:
            scales[j + 4] = (sc[j] & 0xF) | ((m[j] & 0xF) << 4)
            scales[j - 4] |= (sc[j] >> 4) << 6
            scales[j] |= (m[j] >> 4) << 6
    L = np.asarray(L, dtype=np.uint8).reshape(4, 2, 32)
    qs = ((L[:, 0, :] & 15) | ((L[:, 1, :] & 15) << 4)).reshape(-1)
    qh = np.zeros(32, dtype=np.uint8)
    for c in range(4):
        qh |= ((L[c, 0, :] >> 4) << (2 * c)).astype(np.uint8) | ((L[c, 1, :] >> 4) << (2 * c + 1)).astype(np.uint8)
    return np.frombuffer(np.float16(d).tobytes() + np.float16(dmin).tobytes() + scales.tobytes() + qh.tobytes() + qs.tobytes(),
                         dtype=np.uint8)


def test_q5k_sizes_and_zero_blocks(oracle):
    assert oracle.tensor_size(Q5K, 256) == 176 and oracle.tensor_size(Q5K, 257) == 352  # k_quants.rs:162, types.rs:115
    assert not oracle.quantize(Q5K, np.zeros(512, np.float32)).any()
    assert not oracle.quantize(Q5K, np.full(256, 0.37, np.float32)).any()  # max == min in every sub-block -> (0, 0)
    blk = oracle.quantize(Q5K, np.ones(300, np.float32))
    assert blk.size == 352 and not blk[176:].any()  # a partial trailing block stays zero (k_quants.rs:975-977)


def test_q5k_exact_grid_block_is_packed_as_derived_by_hand(oracle):
    """x = 0, 1, ..., 31 in every sub-block: min 0, max 31, iscale 1 -> l = x, scale 1.0, min -0.0 (quantize.rs:583-644).
    All eight scales are 1.0 -> max_scale 1, ls = 63 each, lm = 0, d = f16(1 / 63); requantizing with the decoded d:
    d * 63 is 1 to within 2e-4, so L = x again.  The bytes follow from the packing rules."""
    x = np.tile(np.arange(32, dtype=np.float32), 8)
    got = oracle.quantize(Q5K, x)
    want = q5k_block(1.0 / 63.0, 0.0, [63] * 8, [0] * 8, np.tile(np.arange(32), 8))
    assert np.array_equal(got, want)
    # qh: elements 16..31 of every sub-block carry the fifth bit: bytes 16..31 of qh are 0xFF, bytes 0..15 are 0
    assert (got[16:32] == 0).all() and (got[32:48] == 0xFF).all()
    # and both dequantization orders: the inverse of the packing gives the grid back; the reference's own order does not
    d = np.float32(np.float16(1.0 / 63.0)) * np.float32(63)
    back = oracle.dequantize(Q5K, got, [256], order=oracle.ORDER_GGML)
    assert np.array_equal(back, (d * x).astype(np.float32))
    ref = oracle.dequantize(Q5K, got, [256], order=oracle.ORDER_REF)
    assert not np.array_equal(ref, back)


def test_q5k_dequantize_single_positions(oracle):
    """One non-zero quant: where the reference's order (k_quants.rs:414-459) and the packing's inverse put it."""
    rng = np.random.default_rng(2)
    for _ in range(300):
        e = int(rng.integers(256))
        q = int(rng.integers(1, 32))
        sc = [int(v) for v in rng.integers(1, 64, 8)]
        L = np.zeros(256, np.uint8)
        L[e] = q
        blk = q5k_block(1.0, 0.0, sc, [0] * 8, L)
        ggml = oracle.dequantize(Q5K, blk, [256], order=oracle.ORDER_GGML)
        assert np.count_nonzero(ggml) == 1 and ggml[e] == float(sc[e // 32] * q)
        # the reference's order: nibble and fifth bit are looked up separately, so one stored quant can surface as a
        # nibble at one output and as a 16 at another.  Follow the lookups by hand:
        c, p = e // 64, e % 64
        byte, hi_nibble = 32 * c + (p % 32), p >= 32          # where the packing put the low four bits
        half, r = (byte % 32) // 16, byte % 16                 # REF reads qs[32 c + 16 half + l / 2]: l = 2 r (+ 1 for the high nibble)
        out_nib = 64 * c + 32 * half + 2 * r + (1 if hi_nibble else 0)
        qh_byte, qh_bit = p % 32, 2 * c + (1 if p >= 32 else 0)  # where the packing put the fifth bit
        c2, rest = qh_byte // 8, qh_byte % 8                   # REF reads qh[8 c2 + 4 half2 + l / 8] bit l % 8
        half2, l2 = rest // 4, 8 * (rest % 4) + qh_bit
        out_bit = 64 * c2 + 32 * half2 + l2
        want = np.zeros(256, np.float32)
        if q & 15:
            want[out_nib] += float(sc[out_nib // 32] * (q & 15))
        if q >> 4:
            want[out_bit] += float(sc[out_bit // 32] * 16)
        ref = oracle.dequantize(Q5K, blk, [256], order=oracle.ORDER_REF)
        assert np.array_equal(ref, want), (e, q)


def test_q5k_round_trip_bounds(oracle):
    """The reference's round-trip style bound (k_quants.rs:1446-1509 for its siblings), in the packing's order."""
    x = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    back = oracle.dequantize(Q5K, oracle.quantize(Q5K, x), [256], order=oracle.ORDER_GGML)
    assert np.sqrt(np.mean((back - x) ** 2)) < 0.05 and np.abs(back - x).max() < 0.15
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(256 * 64) * 0.02).astype(np.float32)
    q = oracle.quantize(Q5K, x)
    back = oracle.dequantize(Q5K, q, [x.size], order=oracle.ORDER_GGML)
    rel = np.sqrt(np.mean((back - x) ** 2)) / np.sqrt(np.mean(x ** 2))
    assert rel < 0.04  # 5 bits: about half the error of Q4_K
    q4 = oracle.dequantize(12, oracle.quantize(12, x), [x.size], order=oracle.ORDER_GGML)
    assert rel < 0.7 * np.sqrt(np.mean((q4 - x) ** 2)) / np.sqrt(np.mean(x ** 2))


@pytest.mark.gpu
def test_gpu_q5k_quantize_and_dequantize_bit_exact(oracle):
    import pmetal_amd as pm
    from gpu_util import first_mismatch, gpu_dequantize_dev, gpu_quantize_dev, weights
    from test_gpu_codec import edge_inputs
    pm.init(0)
    cases = dict(edge_inputs(256))
    cases["random"] = weights(55, 1 << 20, outliers=1e-3)
    cases["grid"] = np.tile(np.arange(32, dtype=np.float32), 64)
    for name, x in cases.items():
        want = oracle.quantize(Q5K, x)
        got = gpu_quantize_dev(Q5K, x)
        assert np.array_equal(got, want), f"{name}: {first_mismatch(got, want, 176)}"
        if x.size == 0:
            continue
        for order in (0, 1):
            wd = oracle.dequantize(Q5K, want, [x.size], order=order)
            gd = gpu_dequantize_dev(Q5K, want, x.size, order=order)
            nan = np.isnan(wd)
            assert np.array_equal(np.isnan(gd), nan), (name, order)
            assert np.array_equal(gd[~nan].view(np.uint32), wd[~nan].view(np.uint32)), (name, order)
    # every bit pattern of a block, including f16 infinities and NaNs in d / dmin
    rng = np.random.default_rng(9)
    raw = rng.integers(0, 256, 176 * 4096, dtype=np.uint8)
    for order in (0, 1):
        wd = oracle.dequantize(Q5K, raw, [4096 * 256], order=order)
        gd = gpu_dequantize_dev(Q5K, raw, 4096 * 256, order=order)
        nan = np.isnan(wd)
        assert np.array_equal(np.isnan(gd), nan)
        assert np.array_equal(gd[~nan].view(np.uint32), wd[~nan].view(np.uint32))
    # ragged lengths through the host-pointer entry points
    for n in (1, 255, 257, 1000):
        x = weights(n, n)
        assert np.array_equal(pm.quantize(x, Q5K), oracle.quantize(Q5K, x))
        assert np.array_equal(pm.dequantize(oracle.quantize(Q5K, x), Q5K, [n]), oracle.dequantize(Q5K, oracle.quantize(Q5K, x), [n]))


Q5K_GEMV_CASES = [(6144, 4096), (3072, 1024), (7, 256), (33, 1792), (1001, 2304), (6001, 3584), (301, 11008), (4096, 14336), (20, 32768)]


@pytest.mark.gpu
@pytest.mark.parametrize("n,k", Q5K_GEMV_CASES)
def test_gpu_q5k_gemv_matches_dequantize_then_matmul(oracle, n, k):
    """Fused Q5_K GEMV against the oracle's dequantize-then-matmul in f64, both element orders and both activation types:
    the fused attn_qkv shape of an 8B-class model, small and ragged shapes (rows of 1 to 128 super-blocks, short last
    chunks, fewer rows than compute units), random block bytes."""
    import pmetal_amd as pm
    from gpu_util import gpu_qgemv, rel_errors
    pm.init(0)
    rng = np.random.default_rng(n * 7 + k)
    raw = rng.integers(0, 256, size=(n * (k // 256), 176), dtype=np.uint8)
    raw[:, 0:4] = np.frombuffer(np.array([0.01, 0.02], np.float16).tobytes(), np.uint8)  # d, dmin small and finite
    raw = raw.reshape(-1)
    x = rng.standard_normal(k).astype(np.float32)
    x[rng.integers(0, k, max(1, k // 300))] *= 1000.0
    x[rng.integers(0, k, max(1, k // 300))] *= 1e-6
    x[5:21] = 0.0
    bits = oracle.f32_to_bf16_bits(x)
    for x_dtype, x_dev, x_ref in ((pm.DTYPE_F32, x, x), (pm.DTYPE_BF16, bits, oracle.bf16_bits_to_f32(bits))):
        for order in (0, 1):
            want = oracle.qmatvec(Q5K, raw, n, k, x_ref, order=order)
            got = gpu_qgemv(Q5K, raw, n, k, x_dev, x_dtype, order)
            elem, norm = rel_errors(got, want)
            assert elem <= 1e-3 and norm <= 1e-3, (n, k, x_dtype, order, elem, norm)


@pytest.mark.gpu
def test_gpu_q5k_gemv_unit_vectors_quantized_weights_and_linear(oracle):
    import pmetal_amd as pm
    from gpu_util import gpu_qgemv, rel_errors, weights
    pm.init(0)
    n, k = 300, 2048
    wq = pm.quantize(weights(77, n * k, outliers=1e-3), Q5K)
    for order in (0, 1):
        w = oracle.dequantize(Q5K, wq, [n, k], order=order).reshape(n, k)
        for j in list(range(0, 70)) + [255, 256, 511, 1023, 1024, 2047]:
            x = np.zeros(k, np.float32)
            x[j] = 1.0
            got = gpu_qgemv(Q5K, wq, n, k, x, pm.DTYPE_F32, order)
            assert np.allclose(got, w[:, j], rtol=1e-6, atol=1e-9), (order, j)
    assert not gpu_qgemv(Q5K, wq, n, k, np.zeros(k, np.float32), pm.DTYPE_F32, 1).any()
    x = np.random.default_rng(5).standard_normal(k).astype(np.float32)
    x[100] = np.inf
    assert np.isnan(gpu_qgemv(Q5K, wq, n, k, x, pm.DTYPE_F32, 1)).all()
    # qlinear with two activation rows runs one fused GEMV per row (from three rows on: the matrix kernel)
    lib = pm._lib.load()
    m = 2
    xs = np.random.default_rng(6).standard_normal((m, k)).astype(np.float32)
    dw, dx, dy = pm.DeviceBuffer.from_host(wq), pm.DeviceBuffer.from_host(xs), pm.DeviceBuffer(4 * m * n)
    pm.check(lib.pmetal_hip_qlinear(Q5K, dw.ptr, n, k, dx.ptr, pm.DTYPE_F32, m, dy.ptr, pm.DTYPE_F32, 1, None))
    pm.check(lib.pmetal_hip_sync(None))
    got = dy.to_host(np.float32).reshape(m, n)
    for r in range(m):
        want = oracle.qmatvec(Q5K, wq, n, k, xs[r], order=1)
        elem, norm = rel_errors(got[r], want)
        assert elem <= 1e-3 and norm <= 1e-3
    # the GEMM entry point takes Q5_K too (tests/test_gpu_gemm.py) and agrees with the row loop
    pm.check(lib.pmetal_hip_qgemm(Q5K, dw.ptr, n, k, dx.ptr, pm.DTYPE_F32, m, dy.ptr, pm.DTYPE_F32, 1, None))
    pm.check(lib.pmetal_hip_sync(None))
    assert np.allclose(dy.to_host(np.float32).reshape(m, n), got, rtol=0, atol=1e-3 * np.abs(got).max())  # f32 activations: f16-rounded in the GEMM
