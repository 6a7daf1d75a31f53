"""GPU parity: dequant-fused GEMV against the oracle's dequantize-then-matmul (f64 accumulation).

Tolerance: max relative error <= 1e-3 (the bound BASELINE.json's north_star states), measured
element-wise over outputs with |y| > 1e-3 * max|y| and normwise (max|dy| / max|y|)."""
import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import Q4K, Q6K, Q8_0, gpu_qgemv, rel_errors, weights

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module", autouse=True)
def _device():
    pm.init(0)


def activations(oracle, seed, k, x_dtype):
    x = np.random.default_rng(seed).standard_normal(k).astype(np.float32)
    if x_dtype == pm.DTYPE_BF16:
        bits = oracle.f32_to_bf16_bits(x)
        return bits, oracle.bf16_bits_to_f32(bits)
    return x, x


CASES = [
    # (type, n, k): Qwen3-0.6B projections, one Llama-3-8B slice of each orientation, odd shapes
    (Q8_0, 3072, 1024), (Q8_0, 37, 32), (Q8_0, 5, 96), (Q8_0, 64, 2048 + 64),
    (Q4K, 3072, 1024), (Q4K, 1024, 3072), (Q4K, 1024, 2048), (Q4K, 2048, 4096), (Q4K, 512, 14336),
    (Q4K, 3, 256), (Q4K, 67, 768), (Q4K, 9, 1280),
    (Q6K, 1024, 1024), (Q6K, 1024, 3072), (Q6K, 2048, 4096), (Q6K, 7, 256), (Q6K, 33, 1792),
]


@pytest.mark.parametrize("t,n,k", CASES)
@pytest.mark.parametrize("x_dtype", [pm.DTYPE_BF16, pm.DTYPE_F32])
def test_qgemv_matches_dequantize_then_matmul(oracle, t, n, k, x_dtype):
    wq = oracle.quantize(t, weights(n * 31 + k, n * k, outliers=1e-3))
    x_dev, x_ref = activations(oracle, k, k, x_dtype)
    for order in ((0, 1) if t == Q4K else (0,)):
        want = oracle.qmatvec(t, wq, n, k, x_ref, order=order)
        got = gpu_qgemv(t, wq, n, k, x_dev, x_dtype, order)
        elem, norm = rel_errors(got, want)
        print(f"type {t} {n}x{k} x_dtype {x_dtype} order {order}: elem {elem:.2e} norm {norm:.2e}")
        assert elem <= TOL and norm <= TOL


# Shapes of 12 MiB and more take the large-matrix kernels.  Rows of one or two chunks (k = 2048, 4096) with at most
# eight tasks per wave go to the kernel whose waves own whole rows (6001 x 4096, 12001 x 2048, 32767 x 2048: ragged row
# counts, so the last workgroup and its waves are short); more rows than that (20000 x 4096, 40001 x 2048) and every
# other row length go to the chunk-owner kernel: 32-lane teams (k / 256 = 12), a row count below the number of compute
# units times the waves, and a row of 16 chunks (k = 32768).
BIG_CASES = [(6001, 4096), (7301, 3072), (3001, 8192), (16385, 1536), (800, 32768), (12001, 2048), (32767, 2048),
             (20000, 4096), (40001, 2048),
             # rows of 43, 54, 74, 17 and 34 super-blocks: whole-wave teams with a short last chunk
             (4096, 11008), (3001, 13824), (2500, 18944), (5003, 4352), (3001, 8704)]


@pytest.mark.parametrize("n,k", BIG_CASES)
@pytest.mark.parametrize("x_dtype", [pm.DTYPE_BF16, pm.DTYPE_F32])
def test_qgemv_q4k_large_ragged_shapes(oracle, n, k, x_dtype):
    # quantized bytes generated directly (every byte pattern is a valid block; d and dmin kept small and finite)
    rng = np.random.default_rng(n + k)
    raw = rng.integers(0, 256, size=(n * (k // 256), 144), dtype=np.uint8)
    raw[:, 0:4] = np.frombuffer(np.array([0.01, 0.02], np.float16).tobytes(), np.uint8)
    raw = raw.reshape(-1)
    x_dev, x_ref = activations(oracle, n, k, x_dtype)
    for order in (0, 1):
        want = oracle.qmatvec(Q4K, raw, n, k, x_ref, order=order)
        got = gpu_qgemv(Q4K, raw, n, k, x_dev, x_dtype, order)
        elem, norm = rel_errors(got, want)
        print(f"Q4_K {n}x{k} x_dtype {x_dtype} order {order}: elem {elem:.2e} norm {norm:.2e}")
        assert elem <= TOL and norm <= TOL


# Q6_K matrices of 12 MiB and more take the kernel that stages rows through LDS: ragged row counts, rows of 1 to 8 chunks, fewer rows than compute units times
# waves; activations with large and tiny outliers and a run of zeros (the fixed-point scale is per 16 elements).
Q6K_BIG_CASES = [(6001, 4096), (14336, 4096), (4096, 14336), (30001, 2048), (500, 16384), (1900, 6144),
                 # rows that are not whole chunks: 14, 43, 9 and 25 super-blocks (even and odd: rows start at any even address)
                 (6001, 3584), (3001, 11008), (7001, 2304), (2049, 6400),
                 # rows shorter than a chunk (1 to 7 super-blocks): several whole rows are one task of a wave; row counts
                 # that leave the last task short
                 # (from 24 MiB on; rows of 5 or 6 super-blocks and smaller matrices stay with the general kernel)
                 (32001, 1024), (151936, 1024), (62003, 512), (121003, 256), (40002, 768), (18002, 1792), (24001, 1280),
                 (20001, 1536), (15001, 1024)]


@pytest.mark.parametrize("n,k", Q6K_BIG_CASES)
@pytest.mark.parametrize("x_dtype", [pm.DTYPE_BF16, pm.DTYPE_F32])
def test_qgemv_q6k_large_shapes(oracle, n, k, x_dtype):
    rng = np.random.default_rng(n + k)
    raw = rng.integers(0, 256, size=(n * (k // 256), 210), dtype=np.uint8)
    raw[:, 208:210] = np.frombuffer(np.array([0.001], np.float16).tobytes(), np.uint8)
    raw = raw.reshape(-1)
    x = rng.standard_normal(k).astype(np.float32)
    x[rng.integers(0, k, k // 300)] *= 1000.0
    x[rng.integers(0, k, k // 300)] *= 1e-6
    x[5:21] = 0.0
    if x_dtype == pm.DTYPE_BF16:
        x_dev = oracle.f32_to_bf16_bits(x)
        x_ref = oracle.bf16_bits_to_f32(x_dev)
    else:
        x_dev = x_ref = x
    want = oracle.qmatvec(Q6K, raw, n, k, x_ref)
    got = gpu_qgemv(Q6K, raw, n, k, x_dev, x_dtype, 0)
    elem, norm = rel_errors(got, want)
    print(f"Q6_K {n}x{k} x_dtype {x_dtype}: elem {elem:.2e} norm {norm:.2e}")
    assert elem <= TOL and norm <= TOL


def test_qgemv_q6k_large_quantized_weights_and_linearity(oracle):
    n, k = 7000, 4096
    wq = pm.quantize(weights(21, n * k, outliers=1e-3), Q6K)
    rng = np.random.default_rng(22)
    xa, xb = rng.standard_normal(k).astype(np.float32), rng.standard_normal(k).astype(np.float32)
    want = oracle.qmatvec(Q6K, wq, n, k, xa)
    ya = gpu_qgemv(Q6K, wq, n, k, xa, pm.DTYPE_F32, 0)
    elem, norm = rel_errors(ya, want)
    assert elem <= TOL and norm <= TOL
    yb = gpu_qgemv(Q6K, wq, n, k, xb, pm.DTYPE_F32, 0)
    yab = gpu_qgemv(Q6K, wq, n, k, (xa + xb).astype(np.float32), pm.DTYPE_F32, 0)
    assert np.abs(yab - (ya + yb)).max() <= 1e-4 * np.abs(yab).max()
    assert not gpu_qgemv(Q6K, wq, n, k, np.zeros(k, np.float32), pm.DTYPE_F32, 0).any()
    # an infinity among the activations reaches every output
    xa[100] = np.inf
    assert np.isnan(gpu_qgemv(Q6K, wq, n, k, xa, pm.DTYPE_F32, 0)).all()


# Q8_0 matrices of 12 MiB and more with rows of at least 64 blocks (k >= 2048, a multiple of 256) take the kernel that
# stages rows through LDS: ragged row counts, rows of 1, 2, 7 and 16 chunks, fewer rows than compute units times waves;
# activations with large and tiny outliers and a run of zeros; quants over the whole int8 range.
Q8_0_BIG_CASES = [(6001, 4096), (14336, 4096), (4096, 14336), (30001, 2048), (500, 32768), (1900, 6144),
                  # rows whose last chunk is short: 112, 344, 72 and 200 blocks
                  (6001, 3584), (3001, 11008), (7001, 2304), (2049, 6400),
                 # rows shorter than a chunk (1 to 7 super-blocks): several whole rows are one task of a wave; row counts
                 # that leave the last task short
                 # (from 24 MiB on; rows of 5 or 6 super-blocks and smaller matrices stay with the general kernel)
                 (32001, 1024), (151936, 1024), (62003, 512), (121003, 256), (40002, 768), (18002, 1792), (24001, 1280),
                 (20001, 1536), (15001, 1024)]


@pytest.mark.parametrize("n,k", Q8_0_BIG_CASES)
@pytest.mark.parametrize("x_dtype", [pm.DTYPE_BF16, pm.DTYPE_F32])
def test_qgemv_q8_0_large_shapes(oracle, n, k, x_dtype):
    rng = np.random.default_rng(n + k + 1)
    raw = rng.integers(0, 256, size=(n * (k // 32), 34), dtype=np.uint8)
    scales = (rng.uniform(0.5, 2.0, n * (k // 32)) * 1e-3 * rng.choice([-1.0, 1.0], n * (k // 32))).astype(np.float16)
    raw[:, 0:2] = scales.view(np.uint8).reshape(-1, 2)
    raw = raw.reshape(-1)
    x = rng.standard_normal(k).astype(np.float32)
    x[rng.integers(0, k, k // 300)] *= 1000.0
    x[rng.integers(0, k, k // 300)] *= 1e-6
    x[5:40] = 0.0
    if x_dtype == pm.DTYPE_BF16:
        x_dev = oracle.f32_to_bf16_bits(x)
        x_ref = oracle.bf16_bits_to_f32(x_dev)
    else:
        x_dev = x_ref = x
    want = oracle.qmatvec(Q8_0, raw, n, k, x_ref)
    got = gpu_qgemv(Q8_0, raw, n, k, x_dev, x_dtype, 0)
    elem, norm = rel_errors(got, want)
    print(f"Q8_0 {n}x{k} x_dtype {x_dtype}: elem {elem:.2e} norm {norm:.2e}")
    assert elem <= TOL and norm <= TOL


def test_qgemv_q8_0_large_unit_vectors_and_special_values(oracle):
    """Every position of a block, in an even and in an odd block, reaches the right activation; zero input gives zero;
    an infinity among the activations reaches every output."""
    n, k = 7000, 4096
    wq = pm.quantize(weights(23, n * k, outliers=1e-3), Q8_0)
    w = oracle.dequantize(Q8_0, wq, [n, k]).reshape(n, k)
    for j in list(range(0, 70)) + [2047, 2048, 2049, 4062, 4063, 4095]:
        x = np.zeros(k, np.float32)
        x[j] = 1.0
        got = gpu_qgemv(Q8_0, wq, n, k, x, pm.DTYPE_F32, 0)
        assert np.array_equal(got, w[:, j]), j
    assert not gpu_qgemv(Q8_0, wq, n, k, np.zeros(k, np.float32), pm.DTYPE_F32, 0).any()
    x = np.random.default_rng(5).standard_normal(k).astype(np.float32)
    x[100] = np.inf
    assert np.isnan(gpu_qgemv(Q8_0, wq, n, k, x, pm.DTYPE_F32, 0)).all()


def test_qgemv_config0_q8_0_round_trip_and_gemv(oracle):
    # BASELINE config 0: 3072x1024 N(0, 0.02), Q8_0 round trip, then y = W x with f32 x ~ N(0, 1)
    n, k = 3072, 1024
    w = weights(0, n * k)
    x = np.random.default_rng(1).standard_normal(k).astype(np.float32)
    raw = pm.quantize(w, Q8_0)
    assert np.array_equal(raw, oracle.quantize(Q8_0, w))
    deq = pm.dequantize(raw, Q8_0, [n, k])
    assert np.array_equal(deq.view(np.uint32), oracle.dequantize(Q8_0, raw, [n, k]).view(np.uint32))
    want = (deq.reshape(n, k).astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
    got = gpu_qgemv(Q8_0, raw, n, k, x, pm.DTYPE_F32)
    elem, norm = rel_errors(got, want)
    assert elem <= TOL and norm <= TOL


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
def test_qgemv_config1_full_size(oracle, n, k):
    # BASELINE config 1 at full size; weights quantized by the GPU quantizer (itself checked bit-exact
    # against the oracle on a slice), GEMV checked against the oracle on every output.
    w = weights(11, n * k)
    raw = pm.quantize(w, Q4K)
    sl = 256 * 4096
    assert np.array_equal(raw[: 144 * 4096], oracle.quantize(Q4K, w[:sl]))
    bits = oracle.f32_to_bf16_bits(np.random.default_rng(12).standard_normal(k).astype(np.float32))
    want = oracle.qmatvec(Q4K, raw, n, k, oracle.bf16_bits_to_f32(bits))
    got = gpu_qgemv(Q4K, raw, n, k, bits, pm.DTYPE_BF16)
    elem, norm = rel_errors(got, want)
    print(f"Q4_K {n}x{k}: elem {elem:.2e} norm {norm:.2e}")
    assert elem <= TOL and norm <= TOL


def test_qgemv_linearity_and_zero_input(oracle):
    # size-independent properties: W(ax) = a W x for a power of two (exact), W 0 = 0
    n, k = 256, 4096
    wq = oracle.quantize(Q4K, weights(21, n * k))
    x = np.random.default_rng(22).standard_normal(k).astype(np.float32)
    b = oracle.f32_to_bf16_bits(x)
    b4 = oracle.f32_to_bf16_bits(oracle.bf16_bits_to_f32(b) * np.float32(4.0))
    y1 = gpu_qgemv(Q4K, wq, n, k, b, pm.DTYPE_BF16)
    y4 = gpu_qgemv(Q4K, wq, n, k, b4, pm.DTYPE_BF16)
    assert np.array_equal(y4, y1 * np.float32(4.0))
    y0 = gpu_qgemv(Q4K, wq, n, k, np.zeros(k, np.uint16), pm.DTYPE_BF16)
    assert not y0.any()


def test_qgemv_batch_runs_a_decode_step(oracle):
    from pmetal_amd import _lib
    lib = _lib.load()
    shapes = [(Q4K, 2048, 1024), (Q6K, 1024, 1024), (Q4K, 1024, 2048), (Q6K, 1024, 3072)]
    descs = (_lib.LinearDesc * len(shapes))()
    keep, wants = [], []
    for i, (t, n, k) in enumerate(shapes):
        wq = oracle.quantize(t, weights(40 + i, n * k))
        bits = oracle.f32_to_bf16_bits(np.random.default_rng(50 + i).standard_normal(k).astype(np.float32))
        dw, dx, dy = pm.DeviceBuffer.from_host(wq), pm.DeviceBuffer.from_host(bits), pm.DeviceBuffer(4 * n)
        keep.append((dw, dx, dy))
        descs[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, dw.ptr, dx.ptr, dy.ptr)
        wants.append(oracle.qmatvec(t, wq, n, k, oracle.bf16_bits_to_f32(bits)))
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(shapes), None))
    pm.check(lib.pmetal_hip_sync(None))
    for (dw, dx, dy), want in zip(keep, wants):
        elem, norm = rel_errors(dy.to_host(np.float32), want)
        assert elem <= TOL and norm <= TOL


@pytest.mark.parametrize("order", [0, 1])
def test_qgemv_batch_groups_projections_of_one_activation(oracle, order):
    """q / k / v-like projections that share x go through one grouped launch; the rows must come out exactly as
    from separate launches (and a fifth matrix starts a new group, a different x ends one)."""
    from pmetal_amd import _lib
    lib = _lib.load()
    k = 1024
    bits = oracle.f32_to_bf16_bits(np.random.default_rng(70).standard_normal(k).astype(np.float32))
    other = oracle.f32_to_bf16_bits(np.random.default_rng(71).standard_normal(k).astype(np.float32))
    dx, dx2 = pm.DeviceBuffer.from_host(bits), pm.DeviceBuffer.from_host(other)
    rows = [2048, 1024, 1000, 37, 515, 96]
    xs_of = [dx, dx, dx, dx, dx, dx2]
    descs = (_lib.LinearDesc * len(rows))()
    keep, singles = [], []
    for i, n in enumerate(rows):
        wq = oracle.quantize(Q4K, weights(80 + i, n * k))
        dw, dy = pm.DeviceBuffer.from_host(wq), pm.DeviceBuffer(4 * n)
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, 4 * n, None))
        keep.append((dw, dy))
        descs[i] = _lib.LinearDesc(Q4K, pm.DTYPE_BF16, order, 0, n, k, dw.ptr, xs_of[i].ptr, dy.ptr)
        x_bits = bits if xs_of[i] is dx else other
        singles.append(gpu_qgemv(Q4K, wq, n, k, x_bits, pm.DTYPE_BF16, order))
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(rows), None))
    pm.check(lib.pmetal_hip_sync(None))
    for (dw, dy), single in zip(keep, singles):
        assert np.array_equal(dy.to_host(np.float32), single)


@pytest.mark.parametrize("k,x_dtype", [(4096, pm.DTYPE_BF16), (2048, pm.DTYPE_F32)])
@pytest.mark.parametrize("order", [0, 1])
def test_qgemv_batch_groups_that_are_large_as_a_whole(oracle, order, k, x_dtype):
    """q / k / v of an 8B-class model: each below the large-matrix threshold, 14 MB together.  The group streams through
    the row-owner kernel as one launch; every member against the oracle and against its own launch (ragged row counts,
    a fourth small member, then a matrix with another x)."""
    from pmetal_amd import _lib
    lib = _lib.load()
    rows = [4096, 1024, 1031, 517, 700]
    rng = np.random.default_rng(k + order)
    xa, xa_ref = activations(oracle, 5, k, x_dtype)
    xb, xb_ref = activations(oracle, 6, k, x_dtype)
    dx, dx2 = pm.DeviceBuffer.from_host(xa), pm.DeviceBuffer.from_host(xb)
    xs_of = [dx, dx, dx, dx, dx2]
    descs = (_lib.LinearDesc * len(rows))()
    keep = []
    for i, n in enumerate(rows):
        raw = rng.integers(0, 256, size=(n * (k // 256), 144), dtype=np.uint8)
        raw[:, 0:4] = np.frombuffer(np.array([0.01, 0.02], np.float16).tobytes(), np.uint8)
        raw = raw.reshape(-1)
        dw, dy = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer(4 * n)
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, 4 * n, None))
        x_dev, x_ref = (xa, xa_ref) if xs_of[i] is dx else (xb, xb_ref)
        keep.append((dw, dy, raw, n, x_dev, x_ref))
        descs[i] = _lib.LinearDesc(Q4K, x_dtype, order, 0, n, k, dw.ptr, xs_of[i].ptr, dy.ptr)
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(rows), None))
    pm.check(lib.pmetal_hip_sync(None))
    for dw, dy, raw, n, x_dev, x_ref in keep:
        got = dy.to_host(np.float32)
        want = oracle.qmatvec(Q4K, raw, n, k, x_ref, order=order)
        elem, norm = rel_errors(got, want)
        assert elem <= TOL and norm <= TOL, (n, elem, norm)
        single = gpu_qgemv(Q4K, raw, n, k, x_dev, x_dtype, order)
        assert np.abs(got - single).max() <= 2e-6 * np.abs(single).max()


@pytest.mark.parametrize("k,x_dtype", [(1024, pm.DTYPE_BF16), (2048, pm.DTYPE_F32), (768, pm.DTYPE_BF16)])
@pytest.mark.parametrize("rows", [[2048, 1024, 1024], [517, 300], [1024, 1000, 37, 96], [2048, 1024, 1024, 1024]])
@pytest.mark.parametrize("order", [0, 1])
def test_qgemv_batch_takes_a_q6k_projection_into_a_q4k_group(oracle, order, rows, k, x_dtype):
    """q and k in Q4_K followed by v in Q6_K over the same x (a Q4_K_M layer): one launch.  The last of `rows` is the
    Q6_K matrix; every member against the oracle and against its own launch.  With four Q4_K members before it the
    Q6_K matrix does not fit the group and runs on its own."""
    mixed_group_case(oracle, order, rows, k, x_dtype)


@pytest.mark.parametrize("rows,k,x_dtype", [([4096, 1024, 1024], 4096, pm.DTYPE_BF16), ([4096, 1024, 1024], 4096, pm.DTYPE_F32),
                                            ([8192, 2100, 517], 2048, pm.DTYPE_BF16), ([5120, 3001], 4096, pm.DTYPE_BF16),
                                            ([3000, 1000, 1000, 4100], 4096, pm.DTYPE_BF16)])
@pytest.mark.parametrize("order", [0, 1])
def test_qgemv_batch_takes_a_q6k_projection_into_a_large_q4k_group(oracle, order, rows, k, x_dtype):
    """The same with the shapes of an 8B-class model (q 4096 x 4096, k and a Q6_K v 1024 x 4096: the group streams
    through the kernel for large matrices, the Q6_K member as its fourth), with ragged row counts, with rows of one
    chunk, and with a Q6_K member that is larger than any Q4_K member."""
    mixed_group_case(oracle, order, rows, k, x_dtype)


def mixed_group_case(oracle, order, rows, k, x_dtype):
    from pmetal_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(k + order + len(rows))
    xa, xa_ref = activations(oracle, 9, k, x_dtype)
    dx = pm.DeviceBuffer.from_host(xa)
    if len(rows) == 4 and rows[0] == 2048:
        rows = rows + [600]
    descs = (_lib.LinearDesc * len(rows))()
    keep = []
    for i, n in enumerate(rows):
        t = Q6K if i == len(rows) - 1 else Q4K
        bs = 210 if t == Q6K else 144
        raw = rng.integers(0, 256, size=(n * (k // 256), bs), dtype=np.uint8)
        half = np.frombuffer(np.array([0.01, 0.02], np.float16).tobytes(), np.uint8)
        if t == Q6K:
            raw[:, 208:210] = half[:2]
        else:
            raw[:, 0:4] = half
        raw = raw.reshape(-1)
        # y needs 4-byte alignment only, in a shared launch as in a launch of its own: every other member sits one float in
        shift = i % 2
        dw, dy = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer(4 * (n + 4))
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, 4 * (n + 4), None))
        keep.append((t, dw, dy, raw, n, shift))
        descs[i] = _lib.LinearDesc(t, x_dtype, order, 0, n, k, dw.ptr, dx.ptr, dy.ptr + 4 * shift)
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(rows), None))
    pm.check(lib.pmetal_hip_sync(None))
    for t, dw, dy, raw, n, shift in keep:
        whole = dy.to_host(np.float32)
        got = whole[shift:shift + n]
        assert np.isnan(whole[shift + n:]).all() and np.isnan(whole[:shift]).all()  # nothing written outside
        want = oracle.qmatvec(t, raw, n, k, xa_ref, order=order)
        elem, norm = rel_errors(got, want)
        assert elem <= TOL and norm <= TOL, (t, n, elem, norm)
        single = gpu_qgemv(t, raw, n, k, xa, x_dtype, order)
        assert np.abs(got - single).max() <= 2e-6 * np.abs(single).max()


@pytest.mark.parametrize("order", [0, 1])
def test_qgemv_batch_pairs_large_projections_of_one_activation(oracle, order):
    """Two consecutive large Q4_K matrices that share x (gate / up) go through one launch of the large-matrix kernel:
    the results of one by one launches, also with different and ragged row counts, followed by an unrelated third matrix."""
    from pmetal_amd import _lib
    lib = _lib.load()
    k = 4096
    rows = [6001, 7301, 6500]
    rng = np.random.default_rng(17)
    bits = oracle.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32))
    other = oracle.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32))
    dx, dx2 = pm.DeviceBuffer.from_host(bits), pm.DeviceBuffer.from_host(other)
    xs_of = [dx, dx, dx2]
    descs = (_lib.LinearDesc * len(rows))()
    keep, singles = [], []
    for i, n in enumerate(rows):
        raw = rng.integers(0, 256, size=(n * (k // 256), 144), dtype=np.uint8)
        raw[:, 0:4] = np.frombuffer(np.array([0.01, 0.02], np.float16).tobytes(), np.uint8)
        raw = raw.reshape(-1)
        dw, dy = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer(4 * n)
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, 4 * n, None))
        keep.append((dw, dy))
        descs[i] = _lib.LinearDesc(Q4K, pm.DTYPE_BF16, order, 0, n, k, dw.ptr, xs_of[i].ptr, dy.ptr)
        singles.append(gpu_qgemv(Q4K, raw, n, k, bits if xs_of[i] is dx else other, pm.DTYPE_BF16, order))
        if i == 0:
            want = oracle.qmatvec(Q4K, raw, n, k, oracle.bf16_bits_to_f32(bits), order=order)
            elem, norm = rel_errors(singles[0], want)
            assert elem <= TOL and norm <= TOL
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(rows), None))
    pm.check(lib.pmetal_hip_sync(None))
    for (dw, dy), single in zip(keep, singles):
        # the shared launch divides the rows among workgroups differently, so the lanes that add up a row differ: equal up
        # to the order of the f32 partial sums
        got = dy.to_host(np.float32)
        assert np.abs(got - single).max() <= 2e-6 * np.abs(single).max()


def test_qgemv_argument_errors():
    from pmetal_amd import _lib
    lib = _lib.load()
    buf = pm.DeviceBuffer(4096)
    assert lib.pmetal_hip_qgemv(Q4K, buf.ptr, 4, 100, buf.ptr, 1, buf.ptr, 0, None) == 6  # k % 256
    assert lib.pmetal_hip_qgemv(Q4K, buf.ptr, 0, 256, buf.ptr, 1, buf.ptr, 0, None) == 6
    assert lib.pmetal_hip_qgemv(Q4K, None, 4, 256, buf.ptr, 1, buf.ptr, 0, None) == 1
    assert lib.pmetal_hip_qgemv(Q4K, buf.ptr + 2, 4, 256, buf.ptr, 1, buf.ptr, 0, None) == 1
    assert lib.pmetal_hip_qgemv(2, buf.ptr, 4, 256, buf.ptr, 1, buf.ptr, 0, None) == 2
    assert b"16-byte" in lib.pmetal_hip_last_error_message() or lib.pmetal_hip_last_error_code() == 2
