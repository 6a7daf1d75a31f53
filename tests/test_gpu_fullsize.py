"""GPU parity at the full sizes of the measured configurations: the Llama-3-8B-shaped quantizer input (every distinct
tensor shape and type of the Q4_K_M recipe, generated on the device, every super-block compared bit for bit with the
oracle run on all host threads) and the Qwen3-0.6B-shaped decode step (one layer of every recipe variant plus the output
projection against dequantize-then-matmul)."""
import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import Q4K, Q6K, first_mismatch, rel_errors
from pmetal_amd import _lib

pytestmark = pytest.mark.gpu
BLOCK = {Q4K: 144, Q6K: 210, 13: 176, 11: 110, 10: 84, 15: 292}
TOL = 1e-3


@pytest.fixture(scope="module", autouse=True)
def _device():
    pm.init(0)


def _d2h(lib, ptr, offset, nbytes, dtype):
    out = np.empty(nbytes // np.dtype(dtype).itemsize, dtype)
    pm.check(lib.pmetal_hip_d2h(out.ctypes.data, ptr + offset, nbytes))
    return out


# (name, rows, cols, type) of the distinct tensors of a Llama-3-8B-shaped model under the Q4_K_M recipe
# (crates/pmetal/src/commands/quantize.rs:999-1137 with n_layers = 32)
LLAMA3_8B = [("blk.4.attn_q", 4096, 4096, Q4K), ("blk.4.attn_k", 1024, 4096, Q4K), ("blk.0.attn_v", 1024, 4096, Q6K),
             ("blk.4.ffn_gate", 14336, 4096, Q4K), ("blk.4.ffn_down", 4096, 14336, Q4K),
             ("blk.0.ffn_down", 4096, 14336, Q6K), ("output", 128256, 4096, Q6K)]


# the fused attn_qkv tensor of the recipe (Q5_K) and the other candidate types of the KL calibration on the 14336 x 4096
# tensor it is measured on (dynamic.rs:958-965)
OTHER_TYPES = [("blk.4.attn_qkv", 6144, 4096, 13), ("calibrate.q8k", 14336, 4096, 15), ("calibrate.q5k", 14336, 4096, 13),
               ("calibrate.q3k", 14336, 4096, 11), ("calibrate.q2k", 14336, 4096, 10)]


def _oracle_dequantize_threads(oracle, t, raw, n, threads):
    """The oracle's dequantizer over ranges of super-blocks on several host threads (ctypes releases the GIL)."""
    from concurrent.futures import ThreadPoolExecutor
    sbs = n // 256
    out = np.empty(n, np.float32)
    edges = [sbs * i // threads for i in range(threads + 1)]

    def work(i):
        a, b = edges[i], edges[i + 1]
        if b > a:
            out[a * 256:b * 256] = oracle.dequantize(t, raw[a * BLOCK[t]:b * BLOCK[t]], [(b - a) * 256])

    with ThreadPoolExecutor(threads) as pool:
        list(pool.map(work, range(threads)))
    return out


@pytest.mark.parametrize("name,rows,cols,t", LLAMA3_8B + OTHER_TYPES, ids=[x[0] for x in LLAMA3_8B + OTHER_TYPES])
def test_quantize_full_size_tensor_whole(oracle, name, rows, cols, t):
    """Every super-block of the tensor: the device's bytes against the oracle's (run on all host threads), then the device's
    dequantized values of those bytes against the oracle's, bit for bit."""
    lib = _lib.load()
    n = rows * cols
    threads = min(oracle.host_threads(), 16)
    if not name.startswith("calibrate"):
        assert int(pm.q4km_tensor_type(name + ".weight", 2, 32)) == t
    x = pm.DeviceBuffer(4 * n)
    # N(0, 0.02^2) with 0.1 % of +-0.5 outliers, generated on the device
    pm.check(lib.pmetal_hip_fill_normal_f32(x.ptr, n, 1234 + rows, 0.02, 1e-3, 0.5, None))
    nbytes = lib.pmetal_hip_tensor_size(t, n)
    q = pm.DeviceBuffer(nbytes)
    pm.check(lib.pmetal_hip_memset(q.ptr, 0xA5, nbytes, None))
    pm.check(lib.pmetal_hip_quantize_dev(t, x.ptr, n, q.ptr, nbytes, None), "quantize")
    pm.check(lib.pmetal_hip_sync(None))
    xin = _d2h(lib, x.ptr, 0, 4 * n, np.float32)
    got = _d2h(lib, q.ptr, 0, nbytes, np.uint8)
    want = oracle.quantize(t, xin, threads=threads)
    assert np.array_equal(got, want), f"{name}: {first_mismatch(got, want, BLOCK[t])}"
    del xin, want
    # dequantize the whole tensor in place of x
    pm.check(lib.pmetal_hip_dequantize_dev(t, q.ptr, nbytes, x.ptr, n, 0, None))
    pm.check(lib.pmetal_hip_sync(None))
    deq = _d2h(lib, x.ptr, 0, 4 * n, np.float32)
    want = _oracle_dequantize_threads(oracle, t, got, n, threads)
    assert np.array_equal(deq.view(np.uint32), want.view(np.uint32)), name


def test_decode_step_projections_against_oracle(oracle):
    """One layer of each recipe variant of a Qwen3-0.6B-shaped decoder (layer 0: attn_v and ffn_down in Q6_K,
    layer 3: all Q4_K) and the output projection, through the grouped batch entry point."""
    lib = _lib.load()
    shapes = []
    for layer in (0, 3):
        for nm, n, k in (("attn_q", 2048, 1024), ("attn_k", 1024, 1024), ("attn_v", 1024, 1024), ("attn_output", 1024, 2048),
                         ("ffn_gate", 3072, 1024), ("ffn_up", 3072, 1024), ("ffn_down", 1024, 3072)):
            shapes.append((n, k, int(pm.q4km_tensor_type(f"blk.{layer}.{nm}.weight", 2, 28))))
    shapes.append((151936, 1024, int(pm.q4km_tensor_type("output.weight", 2, 28))))
    assert [s[2] for s in shapes[:7]] == [Q4K, Q4K, Q6K, Q4K, Q4K, Q4K, Q6K] and shapes[-1][2] == Q6K
    xs = {}
    for k in (1024, 2048, 3072):
        bits = oracle.f32_to_bf16_bits(np.random.default_rng(k).standard_normal(k).astype(np.float32))
        xs[k] = (bits, pm.DeviceBuffer.from_host(bits))
    descs = (_lib.LinearDesc * len(shapes))()
    keep = []
    for i, (n, k, t) in enumerate(shapes):
        w = pm.DeviceBuffer(4 * n * k)
        pm.check(lib.pmetal_hip_fill_normal_f32(w.ptr, n * k, 77 + i, 0.02, 0.0, 0.0, None))
        nbytes = lib.pmetal_hip_tensor_size(t, n * k)
        q = pm.DeviceBuffer(nbytes)
        pm.check(lib.pmetal_hip_quantize_dev(t, w.ptr, n * k, q.ptr, nbytes, None), "quantize")
        y = pm.DeviceBuffer(4 * n)
        pm.check(lib.pmetal_hip_memset(y.ptr, 0xFF, 4 * n, None))
        keep.append((q, y, nbytes))
        descs[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, q.ptr, xs[k][1].ptr, y.ptr)
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(shapes), None))
    pm.check(lib.pmetal_hip_sync(None))
    for (n, k, t), (q, y, nbytes) in zip(shapes, keep):
        raw = q.to_host(np.uint8, nbytes)
        want = oracle.qmatvec(t, raw, n, k, oracle.bf16_bits_to_f32(xs[k][0]))
        elem, norm = rel_errors(y.to_host(np.float32, n), want)
        assert elem <= TOL and norm <= TOL, (n, k, t, elem, norm)
