"""Q2_K and Q3_K quantize / dequantize (crates/pmetal-gguf/src/k_quants.rs:1242-1321, :230-266 and :1139-1237,
:281-355; make_q3_quants quantize.rs:655-727): the oracle against what pins it, the HIP kernels against the oracle bit
for bit.  These are the two low-bit candidates of the KL calibration's default list (dynamic.rs:958-965)."""
import numpy as np
import pytest

Q2K, Q3K = 10, 11


def pack_qs2(L):
    """qs[32 h + l] = L[128 h + l] | L[128 h + l + 32] << 2 | ... << 4 | ... << 6 (k_quants.rs:1227-1234, :1313-1320)."""
    L = np.asarray(L, dtype=np.uint8).reshape(2, 4, 32)
    return (L[:, 0] | (L[:, 1] << 2) | (L[:, 2] << 4) | (L[:, 3] << 6)).astype(np.uint8).reshape(-1)


def q2k_block(d, dmin, sc, m, L):
    scales = (np.asarray(sc, dtype=np.uint8) & 15) | ((np.asarray(m, dtype=np.uint8) & 15) << 4)
    return np.frombuffer(scales.astype(np.uint8).tobytes() + pack_qs2(L).tobytes() + np.float16(d).tobytes() + np.float16(dmin).tobytes(),
                         dtype=np.uint8)


def q3k_block(d, sc6, L):
    """sc6: sixteen values 0..63 (scale + 32); L: 256 values 0..7 (quant + 4).  Packed as quantize_q3k packs
    (k_quants.rs:1176-1184, :1209-1234)."""
    sc6 = [int(v) for v in sc6]
    scales = np.zeros(12, dtype=np.uint8)
    for j in range(16):
        if j < 8:
            scales[j] |= sc6[j] & 15
        else:
            scales[j - 8] |= (sc6[j] & 15) << 4
        scales[8 + j % 4] |= (sc6[j] >> 4) << (2 * (j // 4))
    L = np.asarray(L, dtype=np.uint8)
    hmask = np.zeros(32, dtype=np.uint8)
    for e in range(256):
        if L[e] > 3:
            hmask[e % 32] |= 1 << (e // 32)
    return np.frombuffer(hmask.tobytes() + pack_qs2(L & 3).tobytes() + scales.tobytes() + np.float16(d).tobytes(), dtype=np.uint8)


def test_sizes_and_degenerate_blocks(oracle):
    assert oracle.tensor_size(Q2K, 256) == 84 and oracle.tensor_size(Q2K, 257) == 168    # k_quants.rs:158
    assert oracle.tensor_size(Q3K, 256) == 110 and oracle.tensor_size(Q3K, 513) == 330   # k_quants.rs:159
    for t, nb in ((Q2K, 84), (Q3K, 110)):
        assert not oracle.quantize(t, np.zeros(512, np.float32)).any()
        blk = oracle.quantize(t, np.ones(300, np.float32))
        assert blk.size == 2 * nb and not blk[nb:].any()  # a partial trailing block stays zero (:1154-1156, :1259-1261)
    assert not oracle.quantize(Q2K, np.full(256, 0.37, np.float32)).any()  # max == min in every sub-block -> (0, 0)


def test_make_q3_quants_known_answers(oracle):
    s, ls = oracle.make_q3_quants(np.zeros(16, np.float32), 4, True)  # quantize.rs:1020-1024
    assert s == 0.0 and not ls.any()
    s, _ = oracle.make_q3_quants(np.arange(-4, 4, dtype=np.float32), 4, True)  # quantize.rs:1027-1032
    assert abs(s) > 0.0
    # closed form: x = s * (-4 .. 3) twice.  The element of largest magnitude is -4 s, iscale = -4 / (-4 s) = 1 / s, so
    # l = x / s exactly; sumlx / suml2 = s sum(l^4 s^2 ...) / ... = s; every refinement proposes round(x / s) = l.
    for sc in (1.0, 0.5, 3.0, 0.0625):
        x = np.tile(np.arange(-4, 4, dtype=np.float32) * np.float32(sc), 2)
        s, ls = oracle.make_q3_quants(x, 4, True)
        assert np.array_equal(ls, np.tile(np.arange(0, 8, dtype=np.int8), 2)) and s == np.float32(sc)
        s2, ls2 = oracle.make_q3_quants(x, 4, False)  # no refinement: 1 / iscale
        assert np.array_equal(ls2, ls) and s2 == np.float32(sc)
    # mirrored: the largest magnitude is positive, so iscale is negative and so is the returned scale
    s, ls = oracle.make_q3_quants(np.arange(-3, 5, dtype=np.float32), 4, True)
    assert s == -1.0 and np.array_equal(ls, 4 - np.arange(-3, 5))


def test_make_q3_quants_invariants(oracle):
    """On random input: the scale is the weighted least-squares scale of the returned quants (w = x^2), and the sweeps
    never end on a worse weighted error than the plain rounding they start from."""
    rng = np.random.default_rng(4)
    for trial in range(400):
        x = (rng.standard_normal(16) * 10.0 ** rng.uniform(-3, 2)).astype(np.float32)
        if trial % 7 == 0:
            x[rng.integers(16)] *= 8
        s, ls = oracle.make_q3_quants(x, 4, True)
        l = ls.astype(np.float64) - 4
        assert l.min() >= -4 and l.max() <= 3
        xd = x.astype(np.float64)
        w = xd * xd
        assert s == pytest.approx((w * xd * l).sum() / (w * l * l).sum(), rel=2e-5)
        _, ls0 = oracle.make_q3_quants(x, 4, False)
        l0 = ls0.astype(np.float64) - 4

        def best_err(lq):  # weighted error at the optimal scale for these quants
            return (w * xd * xd).sum() - (w * xd * lq).sum() ** 2 / (w * lq * lq).sum()
        assert best_err(l) <= best_err(l0) * (1 + 1e-5) + 1e-30


def test_q2k_grid_blocks_are_packed_as_derived_by_hand(oracle):
    """Sub-block j holds (e % 4) * s_j - 1.5 s_j with s_j = (j % 15 + 1) / 15: make_qkx1_quants finds min -1.5 s_j,
    l = e % 4 and scale s_j (quantize.rs:583-644), so max_scale = 1, max_min = 1.5, the 4-bit scale is j % 15 + 1 and the
    4-bit min round(15 * 1.5 s_j / 1.5) = j % 15 + 1; d = f16(1 / 15), dmin = f16(0.1).  Requantizing with the decoded
    values moves every quotient by less than 1e-3, so L = e % 4."""
    k = np.arange(16) % 15 + 1
    s = (k / 15.0).astype(np.float32)
    x = ((np.arange(256) % 4).astype(np.float32).reshape(16, 16) * s[:, None] - np.float32(1.5) * s[:, None]).astype(np.float32).reshape(-1)
    got = oracle.quantize(Q2K, x)
    want = q2k_block(1.0 / 15.0, 0.1, k, k, np.arange(256) % 4)
    assert np.array_equal(got, want)
    assert (got[16:80].reshape(-1, 4) == np.array([0x00, 0x55, 0xAA, 0xFF], np.uint8)).all()
    back = oracle.dequantize(Q2K, got, [256])
    d, dmin = np.float32(np.float16(1 / 15.0)), np.float32(np.float16(0.1))
    exp = ((d * k.astype(np.float32))[:, None] * (np.arange(256) % 4).astype(np.float32).reshape(16, 16)
           - (dmin * k.astype(np.float32))[:, None]).astype(np.float32).reshape(-1)
    assert np.array_equal(back, exp)
    # all-positive grid: min stays 0 and the scale byte has no high nibble
    got = oracle.quantize(Q2K, np.tile(np.arange(4, dtype=np.float32), 64))
    assert np.array_equal(got, q2k_block(1.0 / 15.0, 0.0, [15] * 16, [0] * 16, np.arange(256) % 4))


def test_q3k_grid_block_is_packed_as_derived_by_hand(oracle):
    """Sub-block j holds s_j * (-4 .. 3) twice with s_j = (j + 1) / 32 (j < 15) and -1 for j = 15 (so that sub-block's
    scale is the one of largest magnitude and negative... its data is +4 .. -3): make_q3_quants returns s_j; iscale =
    -32 / (-1) = 32; the 6-bit value is round(32 s_j) + 32 = j + 33 (j < 15) and 0 for j = 15; d = f16(1 / 32).
    Requantizing: x / (d * (l - 32)) is the grid value exactly, so L = grid + 4."""
    s = np.array([(j + 1) / 32.0 for j in range(15)] + [-1.0], dtype=np.float32)
    grid = np.tile(np.arange(-4, 4, dtype=np.float32), 2)
    x = (s[:, None] * grid[None, :]).astype(np.float32).reshape(-1)
    got = oracle.quantize(Q3K, x)
    sc6 = [j + 33 for j in range(15)] + [0]
    want = q3k_block(1.0 / 32.0, sc6, np.tile(np.arange(0, 8), 32))
    assert np.array_equal(got, want)
    back = oracle.dequantize(Q3K, got, [256])
    assert np.array_equal(back, x)  # every value is on the grid: the round trip is exact


def test_dequantize_single_positions(oracle):
    """One non-zero quant per block: element e reads qs[32 (e / 128) + e % 32] at bit 2 ((e % 128) / 32), the scale of
    sub-block e / 16 and (Q3_K) bit e / 32 of hmask[e % 32]."""
    rng = np.random.default_rng(6)
    for _ in range(200):
        e = int(rng.integers(256))
        sc = [int(v) for v in rng.integers(1, 16, 16)]
        L = np.zeros(256, np.uint8)
        L[e] = q = int(rng.integers(1, 4))
        out = oracle.dequantize(Q2K, q2k_block(1.0, 0.0, sc, [0] * 16, L), [256])
        assert np.count_nonzero(out) == 1 and out[e] == float(sc[e // 16] * q)
        # mins: every element of sub-block j reads -dmin * m_j
        m = [int(v) for v in rng.integers(0, 16, 16)]
        out = oracle.dequantize(Q2K, q2k_block(0.0, 1.0, sc, m, L), [256])
        assert np.array_equal(out, -np.repeat(np.array(m, np.float32), 16))
        # Q3_K: all quants at 4 (value 0) except one
        sc6 = [int(v) for v in rng.integers(0, 64, 16)]
        L3 = np.full(256, 4, np.uint8)
        L3[e] = q3 = int(rng.choice([0, 1, 2, 3, 5, 6, 7]))
        out = oracle.dequantize(Q3K, q3k_block(1.0, sc6, L3), [256])
        want = np.zeros(256, np.float32)
        want[e] = float((sc6[e // 16] - 32) * (q3 - 4))
        assert np.array_equal(out, want), e


def test_round_trip_bounds(oracle):
    """The reference's own round-trip tests (k_quants.rs:1512-1553) and tighter sanity bounds on Gaussian data."""
    x = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    for t, rmse_max, err_max in ((Q3K, 1.5, 4.0), (Q2K, 1.0, 2.0)):
        back = oracle.dequantize(t, oracle.quantize(t, x), [256])
        assert np.sqrt(np.mean((back - x) ** 2)) < rmse_max and np.abs(back - x).max() < err_max
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(256 * 64) * 0.02).astype(np.float32)
    rel = {}
    for t in (Q2K, Q3K, 12):
        back = oracle.dequantize(t, oracle.quantize(t, x), [x.size], order=oracle.ORDER_GGML)
        rel[t] = np.sqrt(np.mean((back - x) ** 2)) / np.sqrt(np.mean(x ** 2))
    assert rel[12] < rel[Q3K] < rel[Q2K] and rel[Q3K] < 0.2 and rel[Q2K] < 0.35


@pytest.mark.gpu
def test_gpu_q2k_q3k_quantize_and_dequantize_bit_exact(oracle):
    import pmetal_amd as pm
    from gpu_util import first_mismatch, gpu_dequantize_dev, gpu_quantize_dev, weights
    from test_gpu_codec import edge_inputs
    pm.init(0)
    cases = dict(edge_inputs(256))
    cases["random"] = weights(56, 1 << 20, outliers=1e-3)
    cases["grid2"] = np.tile(np.arange(4, dtype=np.float32), 1024)
    cases["grid3"] = np.tile(np.arange(-4, 4, dtype=np.float32), 512)
    rng = np.random.default_rng(12)
    cases["wide"] = (rng.standard_normal(1 << 16) * 10.0 ** rng.uniform(-6, 4, 1 << 16)).astype(np.float32)
    cases["negative_heavy"] = (-np.abs(rng.standard_normal(1 << 16)) * 0.05).astype(np.float32)
    for t, nb in ((Q2K, 84), (Q3K, 110)):
        for name, x in cases.items():
            want = oracle.quantize(t, x)
            got = gpu_quantize_dev(t, x)
            assert np.array_equal(got, want), f"type {t} {name}: {first_mismatch(got, want, nb)}"
            if x.size == 0:
                continue
            wd = oracle.dequantize(t, want, [x.size])
            gd = gpu_dequantize_dev(t, want, x.size)
            nan = np.isnan(wd)
            assert np.array_equal(np.isnan(gd), nan), (t, name)
            assert np.array_equal(gd[~nan].view(np.uint32), wd[~nan].view(np.uint32)), (t, name)
        # every bit pattern of a block, including f16 infinities and NaNs in d / dmin
        raw = np.random.default_rng(9).integers(0, 256, nb * 4096, dtype=np.uint8)
        wd = oracle.dequantize(t, raw, [4096 * 256])
        gd = gpu_dequantize_dev(t, raw, 4096 * 256)
        nan = np.isnan(wd)
        assert np.array_equal(np.isnan(gd), nan)
        assert np.array_equal(gd[~nan].view(np.uint32), wd[~nan].view(np.uint32))
        # ragged lengths through the host-pointer entry points
        for n in (1, 255, 257, 1000):
            x = weights(n, n)
            assert np.array_equal(pm.quantize(x, t), oracle.quantize(t, x))
            assert np.array_equal(pm.dequantize(oracle.quantize(t, x), t, [n]), oracle.dequantize(t, oracle.quantize(t, x), [n]))


GEMV_CASES = [(6144, 4096), (3072, 1024), (7, 256), (33, 1792), (1001, 2304), (3001, 3584), (301, 11008), (2048, 14336), (20, 32768),
              (5, 6400)]


@pytest.mark.gpu
@pytest.mark.parametrize("t", [Q2K, Q3K])
@pytest.mark.parametrize("n,k", GEMV_CASES)
def test_gpu_q2k_q3k_gemv_matches_dequantize_then_matmul(oracle, t, n, k):
    """Fused Q2_K / Q3_K GEMV against the oracle's dequantize-then-matmul in f64, both activation types: large, small and
    ragged shapes (rows of 1 to 128 super-blocks, odd counts so that rows start at every alignment, short last chunks,
    fewer rows than compute units), random block bytes."""
    import pmetal_amd as pm
    from gpu_util import gpu_qgemv, rel_errors
    pm.init(0)
    nb = {Q2K: 84, Q3K: 110}[t]
    rng = np.random.default_rng(n * 7 + k + t)
    raw = rng.integers(0, 256, size=(n * (k // 256), nb), dtype=np.uint8)
    if t == Q2K:
        raw[:, 80:84] = np.frombuffer(np.array([0.01, 0.02], np.float16).tobytes(), np.uint8)  # d, dmin small and finite
    else:
        raw[:, 108:110] = np.frombuffer(np.array([0.01], np.float16).tobytes(), np.uint8)
    raw = raw.reshape(-1)
    x = rng.standard_normal(k).astype(np.float32)
    x[rng.integers(0, k, max(1, k // 300))] *= 1000.0
    x[rng.integers(0, k, max(1, k // 300))] *= 1e-6
    x[5:21] = 0.0
    bits = oracle.f32_to_bf16_bits(x)
    for x_dtype, x_dev, x_ref in ((pm.DTYPE_F32, x, x), (pm.DTYPE_BF16, bits, oracle.bf16_bits_to_f32(bits))):
        want = oracle.qmatvec(t, raw, n, k, x_ref)
        got = gpu_qgemv(t, raw, n, k, x_dev, x_dtype, 0)
        elem, norm = rel_errors(got, want)
        assert elem <= 1e-3 and norm <= 1e-3, (t, n, k, x_dtype, elem, norm)


@pytest.mark.gpu
@pytest.mark.parametrize("t", [Q2K, Q3K])
def test_gpu_q2k_q3k_gemv_unit_vectors_and_linear(oracle, t):
    import pmetal_amd as pm
    from gpu_util import gpu_qgemv, rel_errors, weights
    pm.init(0)
    n, k = 301, 2304  # nine super-blocks per row: rows start at every alignment, the second chunk holds one super-block
    wq = pm.quantize(weights(78, n * k, outliers=1e-3), t)
    w = oracle.dequantize(t, wq, [n, k]).reshape(n, k)
    for j in list(range(0, 140)) + [255, 256, 511, 1023, 1024, 2047, 2048, 2303]:
        x = np.zeros(k, np.float32)
        x[j] = 1.0
        got = gpu_qgemv(t, wq, n, k, x, pm.DTYPE_F32, 0)
        assert np.allclose(got, w[:, j], rtol=1e-6, atol=1e-9), (t, j)
    assert not gpu_qgemv(t, wq, n, k, np.zeros(k, np.float32), pm.DTYPE_F32, 0).any()
    x = np.random.default_rng(5).standard_normal(k).astype(np.float32)
    x[100] = np.inf
    assert np.isnan(gpu_qgemv(t, wq, n, k, x, pm.DTYPE_F32, 0)).all()
    # qlinear with two activation rows runs one fused GEMV per row (from three rows on: the matrix kernel)
    lib = pm._lib.load()
    m = 2
    xs = np.random.default_rng(6).standard_normal((m, k)).astype(np.float32)
    dw, dx, dy = pm.DeviceBuffer.from_host(wq), pm.DeviceBuffer.from_host(xs), pm.DeviceBuffer(4 * m * n)
    pm.check(lib.pmetal_hip_qlinear(t, dw.ptr, n, k, dx.ptr, pm.DTYPE_F32, m, dy.ptr, pm.DTYPE_F32, 0, None))
    pm.check(lib.pmetal_hip_sync(None))
    got = dy.to_host(np.float32).reshape(m, n)
    for r in range(m):
        elem, norm = rel_errors(got[r], oracle.qmatvec(t, wq, n, k, xs[r]))
        assert elem <= 1e-3 and norm <= 1e-3
    # the GEMM entry point takes these types too (tests/test_gpu_gemm.py) and agrees with the row loop
    pm.check(lib.pmetal_hip_qgemm(t, dw.ptr, n, k, dx.ptr, pm.DTYPE_F32, m, dy.ptr, pm.DTYPE_F32, 0, None))
    pm.check(lib.pmetal_hip_sync(None))
    assert np.allclose(dy.to_host(np.float32).reshape(m, n), got, rtol=0, atol=1e-3 * np.abs(got).max())  # f32 activations: f16-rounded in the GEMM


@pytest.mark.gpu
@pytest.mark.parametrize("t", [Q3K, Q2K, 13])
def test_gpu_gemv_vocabulary_sized_matrix(oracle, t):
    """An output projection of 128256 x 4096 (501 rows per workgroup): the row sums go through LDS one float per row and
    chunk, so the row count of a matrix does not limit the kernel.  Random block bytes; the reference covers the first
    and last 256 rows and 512 rows drawn at random."""
    import pmetal_amd as pm
    from gpu_util import gpu_qgemv, rel_errors
    n, k = 128256, 4096
    ts = {Q3K: 110, Q2K: 84, 13: 176}[t]
    rng = np.random.default_rng(40 + t)
    raw = rng.integers(0, 256, n * (k // 256) * ts, dtype=np.uint8)
    blocks = raw.reshape(-1, ts)
    for off in {Q3K: (109,), Q2K: (81, 83), 13: (1, 3)}[t]:  # keep the f16 scales finite and small
        blocks[:, off] &= 0x3F
    x = rng.standard_normal(k).astype(np.float32)
    got = gpu_qgemv(t, raw, n, k, x, pm.DTYPE_F32)
    rows = np.unique(np.concatenate([np.arange(256), np.arange(n - 256, n), rng.choice(n, 512, replace=False)]))
    row_bytes = k // 256 * ts
    want = oracle.qmatvec(t, raw.reshape(n, row_bytes)[rows].reshape(-1), rows.size, k, x)
    elem, norm = rel_errors(got[rows], want)
    assert elem <= 1e-3 and norm <= 1e-3, (elem, norm)
    assert np.isfinite(got).all()
