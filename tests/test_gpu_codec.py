"""GPU parity: quantize / dequantize through the C ABI must equal the CPU oracle bit for bit."""
import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import Q4K, Q6K, Q8_0, first_mismatch, gpu_dequantize_dev, gpu_quantize_dev, weights

pytestmark = pytest.mark.gpu
BLOCK = {Q8_0: 34, Q4K: 144, Q6K: 210}


@pytest.fixture(scope="module", autouse=True)
def _device():
    pm.init(0)


def edge_inputs(block_elems):
    """Inputs the reference tests and the format's corner cases call for."""
    rng = np.random.default_rng(99)
    ramp = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    cases = {
        "ramp": ramp,
        "zeros": np.zeros(512, np.float32),
        "constant": np.full(512, 0.37, np.float32),
        "all_positive": np.abs(weights(1, 1024)) + np.float32(0.01),
        "all_negative": -np.abs(weights(2, 1024)) - np.float32(0.01),
        "tiny": weights(3, 1024, std=1e-30),
        "denormal": (rng.standard_normal(512) * 1e-41).astype(np.float32),
        "huge": weights(4, 1024, std=1e30),
        "mixed_scale": (weights(5, 2048) * np.repeat(10.0 ** rng.integers(-6, 6, 2048 // 16), 16)).astype(np.float32),
        "one_hot": np.eye(1, 768, 300, dtype=np.float32).reshape(-1) * 3.0,
        "signed_zero": np.where(np.arange(512) % 2 == 0, np.float32(0.0), np.float32(-0.0)).astype(np.float32),
        "half_ties": (np.arange(512) % 31 - 15).astype(np.float32) * np.float32(0.5),
        "ragged": weights(6, 256 * 3 + 77),
        "short": weights(7, 5),
        "one_block_plus_one": weights(8, block_elems + 1),
        # quotients that sit exactly on rounding ties, and scales spread over 35 orders of magnitude
        "tie_grid": ((rng.integers(-63, 64, 1 << 16) * 0.5) * np.repeat(rng.uniform(0.001, 1, 1 << 8), 256)).astype(np.float32),
        "scale_spread": (rng.standard_normal(1 << 16) * np.repeat(np.exp(rng.uniform(-40, 40, 1 << 11)), 32)).astype(np.float32),
    }
    for name, bad in (("with_inf", np.inf), ("with_nan", np.nan)):
        x = weights(9, 1 << 14)
        x[rng.integers(0, x.size, 40)] = bad
        x[rng.integers(0, x.size, 40)] = -bad
        cases[name] = x
    return cases


@pytest.mark.parametrize("t", [Q8_0, Q4K, Q6K])
def test_quantize_edge_cases_bit_exact(oracle, t):
    for name, x in edge_inputs(32 if t == Q8_0 else 256).items():
        want = oracle.quantize(t, x)
        got = gpu_quantize_dev(t, x)
        assert np.array_equal(got, want), f"{name}: {first_mismatch(got, want, BLOCK[t])}"


def test_quantize_q4k_corner_cases_inside_a_large_tensor(oracle):
    """The corner cases above, Gaussian data with outliers and runs of constants, laid end to end to 32768 + 5
    super-blocks and a ragged tail: sub-blocks that need one, two or all five passes of the search side by side in one
    wave, in a tensor of many workgroups."""
    rng = np.random.default_rng(4)
    parts, total, want_n = [], 0, (32768 + 5) * 256 + 77
    cases = list(edge_inputs(256).values())
    i = 0
    while total < want_n:
        c = cases[i % len(cases)] if i % 3 == 0 else weights(500 + i, int(rng.integers(1, 40)) * 1024 + int(rng.integers(0, 256)), outliers=1e-3 * (i % 2))
        if i % 7 == 3:
            c = np.full(int(rng.integers(1, 9)) * 32, np.float32(rng.standard_normal()), np.float32)
        parts.append(c)
        total += c.size
        i += 1
    x = np.concatenate(parts)[:want_n].astype(np.float32)
    want = oracle.quantize(Q4K, x)
    got = gpu_quantize_dev(Q4K, x)
    assert np.array_equal(got, want), first_mismatch(got, want, BLOCK[Q4K])


def _batch_case(seed):
    """Tensors of a model-like mix: types, sizes from a few blocks to millions of elements, ragged tails, an empty one."""
    rng = np.random.default_rng(seed)
    specs = [(Q4K, 3 << 20), (Q6K, (1 << 20) + 77), (Q4K, 1000), (Q8_0, 0), (Q8_0, 3072 * 1024), (13, 2 << 20), (Q4K, 4 << 20),
             (10, (1 << 19) + 5), (11, 1 << 19), (Q6K, 5 << 19), (2, 4096), (Q4K, 256), (Q4K, 1 << 22)]
    order = rng.permutation(len(specs))
    return [(specs[i][0], weights(900 + seed * 31 + int(i), specs[i][1], outliers=1e-3 * (int(i) % 2))) for i in order]


@pytest.mark.parametrize("stream_kind", ["default", "created"])
def test_quantize_batch_equals_separate_calls(oracle, stream_kind):
    """pmetal_hip_quantize_batch_dev: the bytes of one pmetal_hip_quantize_dev per tensor (and of the oracle), with the
    batch spread over two streams inside the library; what the caller's stream held before the batch (here: the fill of
    one source tensor) is done before any tensor is read, and what it is given afterwards (a dequantize of the last
    output) runs after every tensor."""
    from pmetal_amd import _lib
    lib = _lib.load()
    stream = lib.pmetal_hip_stream_create() if stream_kind == "created" else None
    for seed in (1, 2):
        case = _batch_case(seed)
        src = [pm.DeviceBuffer.from_host(x) if x.size else pm.DeviceBuffer(16) for _, x in case]
        sizes = [lib.pmetal_hip_tensor_size(t, x.size) for t, x in case]
        dst = [pm.DeviceBuffer(max(b, 16)) for b in sizes]
        for d, b in zip(dst, sizes):
            pm.check(lib.pmetal_hip_memset(d.ptr, 0xA5, max(b, 16), None))
        pm.check(lib.pmetal_hip_sync(None))
        # one source is produced on the caller's stream right before the batch
        big = max(range(len(case)), key=lambda i: case[i][1].size)
        pm.check(lib.pmetal_hip_fill_normal_f32(src[big].ptr, case[big][1].size, 4242 + seed, 0.02, 1e-3, 0.5, stream))
        descs = (_lib.QuantizeDesc * len(case))()
        for i, (t, x) in enumerate(case):
            descs[i] = _lib.QuantizeDesc(t, 0, src[i].ptr, x.size, dst[i].ptr, sizes[i])
        pm.check(lib.pmetal_hip_quantize_batch_dev(descs, len(case), stream))
        last = len(case) - 1 if case[-1][1].size else len(case) - 2
        back = pm.DeviceBuffer(4 * case[last][1].size)
        pm.check(lib.pmetal_hip_dequantize_dev(case[last][0], dst[last].ptr, sizes[last], back.ptr, case[last][1].size, 0, stream))
        pm.check(lib.pmetal_hip_sync(stream))
        filled = src[big].to_host(np.float32, case[big][1].size)
        for i, (t, x) in enumerate(case):
            want = oracle.quantize(t, filled if i == big else x)
            got = dst[i].to_host(np.uint8, sizes[i])
            assert np.array_equal(got, want), (seed, i, t, x.size)
        want_back = oracle.dequantize(case[last][0], dst[last].to_host(np.uint8, sizes[last]), [case[last][1].size])
        assert np.array_equal(back.to_host(np.float32, case[last][1].size).view(np.uint32), want_back.view(np.uint32))
    if stream:
        pm.check(lib.pmetal_hip_stream_destroy(stream))


def test_mirror_quantize_tensors_dev(oracle):
    """pmetal_amd.gguf.quantize_tensors_dev: a list of device-resident tensors, one buffer of blocks each (an empty one included)."""
    xs = [(Q4K, weights(41, 5 << 18)), (Q6K, weights(42, (3 << 18) + 100)), (Q8_0, weights(43, 0)), (13, weights(44, 1 << 18))]
    src = [pm.DeviceBuffer.from_host(x) if x.size else pm.DeviceBuffer(16) for _, x in xs]
    outs = pm.gguf.quantize_tensors_dev([(t, b, x.size) for (t, x), b in zip(xs, src)])
    pm.check(_lib_sync())
    for (t, x), out in zip(xs, outs):
        want = oracle.quantize(t, x)
        assert np.array_equal(out.to_host(np.uint8, want.size), want), t


def _lib_sync():
    from pmetal_amd import _lib
    return _lib.load().pmetal_hip_sync(None)


@pytest.mark.parametrize("t", [Q4K, Q6K])
def test_quantize_batch_of_one_large_tensor(oracle, t):
    """A batch of a single large tensor is cut in two inside the library: the bytes of the whole tensor, ragged tail included."""
    from pmetal_amd import _lib
    lib = _lib.load()
    x = weights(333 + t, (1 << 24) + 3 * 2048 + 77, outliers=1e-3)
    nbytes = lib.pmetal_hip_tensor_size(t, x.size)
    dx, dq = pm.DeviceBuffer.from_host(x), pm.DeviceBuffer(nbytes)
    pm.check(lib.pmetal_hip_memset(dq.ptr, 0xA5, nbytes, None))
    descs = (_lib.QuantizeDesc * 1)(_lib.QuantizeDesc(t, 0, dx.ptr, x.size, dq.ptr, nbytes))
    pm.check(lib.pmetal_hip_quantize_batch_dev(descs, 1, None))
    pm.check(lib.pmetal_hip_sync(None))
    want = oracle.quantize(t, x)
    got = dq.to_host(np.uint8, nbytes)
    assert np.array_equal(got, want), first_mismatch(got, want, BLOCK[t])


def test_quantize_batch_checks_every_descriptor_first_and_can_be_recorded(oracle):
    from pmetal_amd import _lib
    lib = _lib.load()
    xs = [weights(70 + i, n) for i, n in enumerate((1 << 20, 1 << 19, 3 << 18))]
    types = [Q4K, Q6K, Q4K]
    src = [pm.DeviceBuffer.from_host(x) for x in xs]
    sizes = [lib.pmetal_hip_tensor_size(t, x.size) for t, x in zip(types, xs)]
    dst = [pm.DeviceBuffer(b) for b in sizes]
    for d, b in zip(dst, sizes):
        pm.check(lib.pmetal_hip_memset(d.ptr, 0xA5, b, None))
    descs = (_lib.QuantizeDesc * 3)()
    for i in range(3):
        descs[i] = _lib.QuantizeDesc(types[i], 0, src[i].ptr, xs[i].size, dst[i].ptr, sizes[i])
    # a wrong size in the last descriptor: nothing is launched
    descs[2].dst_len = sizes[2] - 144
    assert lib.pmetal_hip_quantize_batch_dev(descs, 3, None) == 3
    assert b"tensor 2" in lib.pmetal_hip_last_error_message()
    descs[2].dst_len = sizes[2]
    descs[1].ggml_type = 16
    assert lib.pmetal_hip_quantize_batch_dev(descs, 3, None) == 2
    descs[1].ggml_type = Q6K
    assert lib.pmetal_hip_quantize_batch_dev(None, 3, None) == 1
    lib.pmetal_hip_clear_error()
    pm.check(lib.pmetal_hip_sync(None))
    assert all(np.all(d.to_host(np.uint8, b) == 0xA5) for d, b in zip(dst, sizes))
    assert lib.pmetal_hip_quantize_batch_dev(descs, 0, None) == 0
    # recorded on a created stream and replayed twice
    stream = lib.pmetal_hip_stream_create()
    pm.check(lib.pmetal_hip_quantize_batch_dev(descs, 3, stream))
    pm.check(lib.pmetal_hip_sync(stream))
    want = [oracle.quantize(t, x) for t, x in zip(types, xs)]
    pm.check(lib.pmetal_hip_record_begin(stream))
    pm.check(lib.pmetal_hip_quantize_batch_dev(descs, 3, stream))
    # (a recorded batch stays on its stream; the library's second stream is free for a batch run on another stream meanwhile)
    other = lib.pmetal_hip_stream_create()
    for d, b in zip(dst, sizes):
        pm.check(lib.pmetal_hip_memset(d.ptr, 0x33, b, other))
    pm.check(lib.pmetal_hip_quantize_batch_dev(descs, 3, other))
    rec = lib.pmetal_hip_record_end(stream)
    assert rec, lib.pmetal_hip_last_error_message()
    pm.check(lib.pmetal_hip_sync(other))  # (the thread that records may not wait for a stream before the recording ends)
    for i in range(3):
        assert np.array_equal(dst[i].to_host(np.uint8, sizes[i]), want[i]), i
    pm.check(lib.pmetal_hip_stream_destroy(other))
    for rep in range(2):
        for d, b in zip(dst, sizes):
            pm.check(lib.pmetal_hip_memset(d.ptr, 0x5A, b, None))
        pm.check(lib.pmetal_hip_sync(None))
        pm.check(lib.pmetal_hip_replay(rec, stream))
        pm.check(lib.pmetal_hip_sync(stream))
        for i in range(3):
            assert np.array_equal(dst[i].to_host(np.uint8, sizes[i]), want[i]), (rep, i)
    pm.check(lib.pmetal_hip_recording_destroy(rec))
    pm.check(lib.pmetal_hip_stream_destroy(stream))


@pytest.mark.parametrize("t", [Q8_0, Q4K, Q6K])
def test_quantize_empty(oracle, t):
    assert gpu_quantize_dev(t, np.zeros(0, np.float32)).size == 0
    assert pm.quantize(np.zeros(0, np.float32), t).size == 0


@pytest.mark.parametrize("t,n,outl", [(Q8_0, 3072 * 1024, 0.0), (Q4K, 1 << 21, 0.0), (Q4K, 1 << 21, 1e-3),
                                      (Q6K, 1 << 21, 0.0), (Q6K, 1 << 21, 1e-3)])
def test_quantize_random_bit_exact(oracle, t, n, outl):
    x = weights(100 + t, n, outliers=outl)
    want = oracle.quantize(t, x)
    got = gpu_quantize_dev(t, x)
    assert np.array_equal(got, want), first_mismatch(got, want, BLOCK[t])


@pytest.mark.parametrize("t", [Q8_0, Q4K, Q6K])
def test_quantize_host_pointer_entry_point(oracle, t):
    x = weights(7 + t, 256 * 40 + (13 if t == Q8_0 else 0))
    assert np.array_equal(pm.quantize(x, t), oracle.quantize(t, x))


@pytest.mark.parametrize("n", [11_000_000 + 123, 20_000_000 + 7, 1_500_000 + 31, 262_144])
@pytest.mark.parametrize("t", [Q8_0, Q4K, Q6K, 13, 11, 10, 15])
def test_host_pointer_entry_points_on_a_tensor_of_several_staging_chunks(oracle, t, n):
    """Host tensors of 256 Ki elements or more go through pinned staging chunks (a quarter of the tensor rounded up to
    8192 elements, between 256 Ki and 4 Mi elements).  Ragged tails: the bytes equal those of the one-launch device
    path, and the super-blocks on both sides of chunk boundaries, the first and the last ones equal the oracle's; the
    same for the way back."""
    x = weights(500 + t, n)
    got = pm.quantize(x, t)
    assert np.array_equal(got, gpu_quantize_dev(t, x))
    bs, ts = (32, 34) if t == Q8_0 else (256, {Q4K: 144, Q6K: 210, 13: 176, 11: 110, 10: 84, 15: 292}[t])
    chunk = min(max((n // 4 + 8191) // 8192 * 8192, 256 << 10), 4 << 20)
    spots = [0] + [c * chunk - 2 * bs for c in (1, 2) if c * chunk + 2 * bs < n] + [(n // bs - 3) * bs]
    for e0 in spots:
        e1 = min(n, e0 + 4 * bs)
        want = oracle.quantize(t, x[e0:e1])
        assert np.array_equal(got[e0 // bs * ts:e0 // bs * ts + want.size], want), e0
    n_out = (n // bs) * bs - 13  # dequantize truncates to the shape's element count
    whole = got[:n // bs * ts]
    back = pm.dequantize(whole, t, (n_out,))
    assert back.size == n_out
    assert np.array_equal(back.view(np.uint32), gpu_dequantize_dev(t, whole, n // bs * bs)[:n_out].view(np.uint32))
    for e0 in spots[:-1]:
        want = oracle.dequantize(t, got[e0 // bs * ts:(e0 // bs + 4) * ts], (4 * bs,))
        assert np.array_equal(back[e0:e0 + 4 * bs].view(np.uint32), want.view(np.uint32)), e0


@pytest.mark.parametrize("t", [Q8_0, Q4K, Q6K])
def test_dequantize_quantized_weights_bit_exact(oracle, t):
    x = weights(200 + t, 1 << 20, outliers=1e-3)
    raw = oracle.quantize(t, x)
    orders = (0, 1) if t == Q4K else (0,)
    for order in orders:
        want = oracle.dequantize(t, raw, [x.size], order=order)
        got = gpu_dequantize_dev(t, raw, x.size, order)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"order {order}"
    # host-pointer entry point with a 2-D shape, as load_gguf calls it
    got = pm.dequantize(raw, t, [1 << 10, 1 << 10])
    assert np.array_equal(got.view(np.uint32), oracle.dequantize(t, raw, [1 << 10, 1 << 10]).view(np.uint32))


@pytest.mark.parametrize("t", [Q8_0, Q4K, Q6K])
def test_dequantize_arbitrary_bytes_and_ragged_tail(oracle, t):
    # every bit pattern of scales / quants, including f16 subnormals, infinities and NaNs in d
    rng = np.random.default_rng(300 + t)
    be = 32 if t == Q8_0 else 256
    nblocks = 4096
    raw = rng.integers(0, 256, nblocks * BLOCK[t], dtype=np.uint8)
    for n in (nblocks * be, nblocks * be - 3, nblocks * be - be + 1):
        r = raw[: pm.GgmlType(t).tensor_size(n)]
        for order in ((0, 1) if t == Q4K else (0,)):
            want = oracle.dequantize(t, r, [n], order=order)
            got = gpu_dequantize_dev(t, r, n, order)
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(got), nan)
            assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_reference_roundtrip_bounds_on_gpu(oracle):
    # the reference's own round-trip tests (k_quants.rs:1446-1509), run through the GPU path
    ramp = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    for t, rmse_max, err_max in ((Q4K, 0.15, 0.5), (Q6K, 0.1, 0.3)):
        back = pm.dequantize(pm.quantize(ramp, t), t, [256])
        assert np.sqrt(np.mean((back - ramp) ** 2)) < rmse_max and np.max(np.abs(back - ramp)) < err_max
    back = pm.dequantize(pm.quantize(ramp, Q8_0), Q8_0, [256])
    assert np.max(np.abs(back - ramp)) < 0.01


def test_errors_match_reference_classes():
    with pytest.raises(pm.DequantError) as e:
        pm.dequantize(np.zeros(10, np.uint8), Q4K, [256])
    assert e.value.kind == "InvalidSize"
    with pytest.raises(pm.DequantError) as e:
        pm.dequantize(np.zeros(0, np.uint8), Q4K, [-1])
    assert e.value.kind == "InvalidShape"
    with pytest.raises(pm.DequantError) as e:
        pm.dequantize(np.zeros(0, np.uint8), 99, [0])
    assert e.value.kind == "UnsupportedType"
    with pytest.raises(pm.QuantizationError):
        pm.quantize(np.zeros(256, np.float32), 16)  # IQ2_XXS: outside this path
    assert pm.dequantize(np.zeros(0, np.uint8), Q6K, [0, 7]).size == 0
