"""GPU parity on seeded random shapes: the launch geometry of the GEMV / GEMM kernels (which kernel a shape takes, rows per
workgroup, ragged tails, chunks per row, groups of the batch entry point) is chosen from the shape, so shapes nobody
picked by hand go through the same checks as the fixed cases: dequantize-then-matmul in f64 by the oracle, <= 1e-3.

Block bytes are random (every byte pattern is a valid block; the f16 scales are set to small finite values), so no
quantizer is involved."""
import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import Q4K, Q6K, Q8_0, gpu_qgemv, rel_errors

pytestmark = pytest.mark.gpu
TOL = 1e-3
Q5K, Q3K, Q2K = 13, 11, 10
BLOCK = {Q8_0: (32, 34), Q4K: (256, 144), Q6K: (256, 210), Q5K: (256, 176), Q3K: (256, 110), Q2K: (256, 84)}
# byte offsets of the f16 scale fields of a block (d, and dmin where the type has one)
SCALES = {Q8_0: (0,), Q4K: (0, 2), Q5K: (0, 2), Q6K: (208,), Q3K: (108,), Q2K: (80, 82)}


@pytest.fixture(scope="module", autouse=True)
def _device():
    pm.init(0)


def random_blocks(rng, t, n, k):
    bs, ts = BLOCK[t]
    raw = rng.integers(0, 256, size=(n * (k // bs), ts), dtype=np.uint8)
    for i, off in enumerate(SCALES[t]):
        v = rng.uniform(0.5, 2.0, raw.shape[0]) * (0.01 if i == 0 else 0.02)
        raw[:, off:off + 2] = v.astype(np.float16).view(np.uint8).reshape(-1, 2)
    return raw.reshape(-1)


def random_shape(rng, t, max_elems):
    bs = BLOCK[t][0]
    # rows: a few super-blocks, thousands of elements, tens of thousands; row counts: 1 .. tens of thousands, never round
    k = bs * int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 14, 16, 17, 24, 32, 43, 56, 64]) * (8 if bs == 32 and rng.random() < 0.7 else 1))
    kind = rng.integers(0, 4)
    n = int({0: rng.integers(1, 40), 1: rng.integers(40, 600), 2: rng.integers(600, 6000), 3: rng.integers(6000, 40000)}[int(kind)])
    n = max(1, min(n, max_elems // k))
    return n, k


def check(oracle, t, raw, n, k, x_ref, order, got, want):
    """Normwise <= 1e-3 always; element-wise <= 1e-3 over the outputs above 1e-3 of the largest, or -- where cancellation
    makes small outputs out of large terms (activations with x300 outliers) -- <= 1e-4 of sum |w| |x|, the scale on which any
    summation of these terms is accurate."""
    elem, norm = rel_errors(got.reshape(-1), want.reshape(-1))
    assert norm <= TOL, (t, n, k, order, elem, norm)
    if elem > TOL:
        w = np.abs(oracle.dequantize(t, raw, [n * k], order=order).reshape(n, k))
        cond = (w @ np.abs(x_ref.astype(np.float32)).reshape(-1, k).T).T.reshape(-1).astype(np.float64)
        err = np.abs(got.reshape(-1).astype(np.float64) - want.reshape(-1).astype(np.float64))
        worst = float((err / np.maximum(cond, 1e-300)).max())
        assert worst <= 1e-4, (t, n, k, order, elem, norm, worst)


def activations(oracle, rng, k, x_dtype):
    x = rng.standard_normal(k).astype(np.float32)
    if rng.random() < 0.3:
        x[rng.integers(0, k, max(1, k // 200))] *= 300.0
    if x_dtype == pm.DTYPE_BF16:
        bits = oracle.f32_to_bf16_bits(x)
        return bits, oracle.bf16_bits_to_f32(bits)
    return x, x


@pytest.mark.parametrize("t", [Q4K, Q6K, Q8_0, Q5K, Q3K, Q2K])
@pytest.mark.parametrize("seed", range(20))
def test_qgemv_random_shapes(oracle, t, seed):
    rng = np.random.default_rng(1000 * t + seed)
    for _ in range(3):
        n, k = random_shape(rng, t, 48 << 20)
        x_dtype = pm.DTYPE_BF16 if rng.random() < 0.6 else pm.DTYPE_F32
        order = int(rng.integers(0, 2)) if t in (Q4K, Q5K) else 0
        raw = random_blocks(rng, t, n, k)
        x_dev, x_ref = activations(oracle, rng, k, x_dtype)
        print(f"type {t} {n}x{k} x_dtype {x_dtype} order {order}", flush=True)
        want = oracle.qmatvec(t, raw, n, k, x_ref, order=order, threads=8)
        got = gpu_qgemv(t, raw, n, k, x_dev, x_dtype, order)
        check(oracle, t, raw, n, k, x_ref, order, got, want)


@pytest.mark.parametrize("seed", range(30))
def test_qgemv_batch_random_groups(oracle, seed):
    """Descriptor lists as a model forward issues them: runs of Q4_K matrices over one activation vector, a Q6_K matrix
    behind some of them, single matrices of other types in between, outputs one float off 16-byte alignment now and then.
    Every output against the oracle and against the matrix's own launch."""
    from pmetal_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77 + seed)
    k = 256 * int(rng.choice([2, 4, 8, 16]))
    x_dtype = pm.DTYPE_BF16 if seed % 2 == 0 else pm.DTYPE_F32
    order = seed % 2
    x_dev, x_ref = activations(oracle, rng, k, x_dtype)
    dx = pm.DeviceBuffer.from_host(x_dev)
    budget = (24 << 20) // k
    types = []
    for _ in range(int(rng.integers(1, 4))):  # groups
        types += [Q4K] * int(rng.integers(1, 5))
        r = rng.random()
        if r < 0.5:
            types.append(Q6K)
        elif r < 0.7:
            types.append(int(rng.choice([Q8_0, Q5K, Q3K, Q2K])))
    descs = (_lib.LinearDesc * len(types))()
    keep = []
    for i, t in enumerate(types):
        n = int(rng.choice([rng.integers(1, 64), rng.integers(64, 1500), rng.integers(1500, max(1501, budget))]))
        raw = random_blocks(rng, t, n, k)
        shift = int(rng.integers(0, 2))
        dw, dy = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer(4 * (n + 4))
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, 4 * (n + 4), None))
        keep.append((t, dw, dy, raw, n, shift))
        descs[i] = _lib.LinearDesc(t, x_dtype, order if t in (Q4K, Q5K) else 0, 0, n, k, dw.ptr, dx.ptr, dy.ptr + 4 * shift)
    print("k", k, "x_dtype", x_dtype, "order", order, [(t, n) for t, _, _, _, n, _ in keep], flush=True)
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(types), None))
    pm.check(lib.pmetal_hip_sync(None))
    for t, dw, dy, raw, n, shift in keep:
        o = order if t in (Q4K, Q5K) else 0
        whole = dy.to_host(np.float32)
        got = whole[shift:shift + n]
        assert np.isnan(whole[shift + n:]).all() and np.isnan(whole[:shift]).all()  # nothing written outside
        want = oracle.qmatvec(t, raw, n, k, x_ref, order=o, threads=8)
        check(oracle, t, raw, n, k, x_ref, o, got, want)
        single = gpu_qgemv(t, raw, n, k, x_dev, x_dtype, o)
        assert np.abs(got - single).max() <= 2e-6 * max(np.abs(single).max(), 1e-30), (t, n, k)


@pytest.mark.parametrize("t", [Q4K, Q6K, Q8_0, Q5K, Q3K, Q2K])
@pytest.mark.parametrize("seed", range(12))
def test_qgemm_random_shapes(oracle, t, seed):
    from pmetal_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(5000 + 100 * t + seed)
    k = 256 * int(rng.choice([1, 2, 3, 5, 8, 14, 16, 24]))
    n = int(rng.choice([rng.integers(1, 100), rng.integers(100, 3000)]))
    m = int(rng.choice([rng.integers(2, 17), rng.integers(17, 130), rng.integers(130, 700)]))
    m = max(2, min(m, (6 << 20) // (n * k // 256 + 1) + 2))
    x_dtype = pm.DTYPE_BF16 if rng.random() < 0.6 else pm.DTYPE_F32
    y_dtype = pm.DTYPE_BF16 if rng.random() < 0.5 else pm.DTYPE_F32
    order = int(rng.integers(0, 2)) if t in (Q4K, Q5K) else 0
    raw = random_blocks(rng, t, n, k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if x_dtype == pm.DTYPE_BF16:
        x_dev = oracle.f32_to_bf16_bits(x.reshape(-1))
        x_ref = oracle.bf16_bits_to_f32(x_dev).reshape(m, k)
    else:
        # the GEMM rounds f32 activations once to f16 at the row's power-of-two scale (row maximum in [2^9, 2^10)): the
        # element-wise check is against the reference fed the same rounded activations
        e = np.floor(np.log2(np.max(np.abs(x), axis=1, keepdims=True))) - 9
        x_ref = (np.ldexp(x, (-e).astype(np.int32)).astype(np.float16).astype(np.float32) * np.exp2(e)).astype(np.float32)
        x_dev = x.reshape(-1)
    print(f"type {t} m={m} {n}x{k} x_dtype {x_dtype} y_dtype {y_dtype} order {order}", flush=True)
    dw, dx = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer.from_host(x_dev)
    esize = 2 if y_dtype == pm.DTYPE_BF16 else 4
    dy = pm.DeviceBuffer(esize * m * n)
    pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, esize * m * n, None))
    pm.check(lib.pmetal_hip_qgemm(t, dw.ptr, n, k, dx.ptr, x_dtype, m, dy.ptr, y_dtype, order, None))
    pm.check(lib.pmetal_hip_sync(None))
    if y_dtype == pm.DTYPE_BF16:
        got = oracle.bf16_bits_to_f32(dy.to_host(np.uint16, m * n)).reshape(m, n)
    else:
        got = dy.to_host(np.float32, m * n).reshape(m, n)
    want = oracle.qmatmul(t, raw, n, k, x_ref, order=order, threads=8)
    tol = TOL + (4e-3 if y_dtype == pm.DTYPE_BF16 else 0.0)  # a bf16 output carries its own rounding (2^-8 relative)
    elem, norm = rel_errors(got.reshape(-1), want.reshape(-1))
    assert elem <= tol and norm <= tol, (t, m, n, k, elem, norm)


CODEC_TYPES = [2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14]  # Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K
CODEC_BLOCK = {2: 32, 3: 32, 6: 32, 7: 32, 8: 32, 9: 32, 10: 256, 11: 256, 12: 256, 13: 256, 14: 256}


def same_floats(got, want):
    """Bit for bit, except that a NaN only has to be a NaN (a block whose f16 scale overflowed decodes inf * 0, and the
    sign and payload of that NaN are the machine's)."""
    nan = np.isnan(want)
    return np.array_equal(np.isnan(got), nan) and np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


@pytest.mark.parametrize("t", CODEC_TYPES)
@pytest.mark.parametrize("seed", range(6))
def test_codec_random_lengths(oracle, t, seed):
    """Quantize and dequantize at lengths nobody picked (whole blocks, ragged tails, a single element, lengths around the
    host entry points' staging threshold), data of mixed character: bytes and values equal the oracle's, bit for bit,
    through the device entry points and through the host entry points."""
    from gpu_util import gpu_dequantize_dev, gpu_quantize_dev
    rng = np.random.default_rng(9000 + 50 * t + seed)
    bs = CODEC_BLOCK[t]
    n = int(rng.choice([rng.integers(1, 3 * bs), rng.integers(3 * bs, 50000), rng.integers(50000, 700000),
                        (1 << 18) + rng.integers(-bs - 3, bs + 3)]))
    x = (rng.standard_normal(n) * np.exp(rng.uniform(-6, 3))).astype(np.float32)
    kind = int(rng.integers(0, 4))
    if kind == 1:  # runs of zeros and of one value
        for _ in range(1 + n // 5000):
            a = int(rng.integers(0, n))
            x[a:a + int(rng.integers(1, 600))] = 0.0 if rng.random() < 0.5 else np.float32(rng.standard_normal())
    elif kind == 2:  # magnitudes spread over many orders
        x *= np.exp(rng.uniform(-20, 20, n)).astype(np.float32)
    elif kind == 3:  # a coarse grid: many rounding ties
        x = (np.round(x * 8) / 8).astype(np.float32)
    print(f"type {t} n {n} kind {kind}", flush=True)
    want_q = oracle.quantize(t, x, threads=8)
    got_q = gpu_quantize_dev(t, x)
    assert np.array_equal(got_q, want_q), (t, n, kind)
    assert np.array_equal(pm.quantize(x, t), want_q)  # host entry point
    orders = (0, 1) if t in (Q4K, Q5K) else (0,)
    for order in orders:
        want = oracle.dequantize(t, want_q, [n], order=order)
        got = gpu_dequantize_dev(t, want_q, n, order)
        assert same_floats(got, want), (t, n, kind, order)
    assert same_floats(pm.dequantize(want_q, t, (n,)), oracle.dequantize(t, want_q, [n]))


@pytest.mark.parametrize("t", [Q4K, Q6K, Q5K, Q3K, Q2K])
@pytest.mark.parametrize("seed", range(8))
def test_qgemv_q8k_random_shapes(oracle, t, seed):
    """The integer-dot GEMV over Q8_K activations at drawn shapes: bit-identical to the reference's scalar dot products."""
    from pmetal_amd import gguf
    lib = pm._lib.load()
    rng = np.random.default_rng(12000 + 40 * t + seed)
    for _ in range(2):
        n, k = random_shape(rng, t, 24 << 20)
        raw = random_blocks(rng, t, n, k)
        act = (rng.standard_normal(k) * np.repeat(np.exp(rng.uniform(-3, 3, k // 256)), 256)).astype(np.float32)
        xq = oracle.quantize_q8k(act)
        print(f"type {t} {n}x{k}", flush=True)
        want = oracle.qmatvec_q8k(t, raw, n, k, xq)
        dw, dxq = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer.from_host(xq)
        dy = pm.DeviceBuffer(max(4 * n, 16))
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, max(4 * n, 16), None))
        gguf.qgemv_q8k(t, dw, n, k, dxq, dy)
        pm.check(lib.pmetal_hip_sync(None))
        got = dy.to_host(np.float32, n)
        bad = np.nonzero(got.view(np.uint32) != want.view(np.uint32))[0]
        assert bad.size == 0, (t, n, k, bad[:5], got[bad[:5]], want[bad[:5]])
