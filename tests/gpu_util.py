"""Helpers shared by the GPU parity tests (everything goes through the C ABI of libpmetal_hip.so)."""
import ctypes as C

import numpy as np

import pmetal_amd as pm
from pmetal_amd import _lib

Q8_0, Q4K, Q6K = 8, 12, 14


def weights(seed, n, std=0.02, outliers=0.0):
    """N(0, std^2) with an optional fraction of +-0.5 outliers (the quantizer benchmark's distribution)."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal(n) * std).astype(np.float32)
    if outliers:
        idx = rng.random(n) < outliers
        w[idx] = np.where(rng.random(int(idx.sum())) < 0.5, np.float32(0.5), np.float32(-0.5))
    return w


def gpu_quantize_dev(t, x):
    """Device-resident entry point: upload f32, quantize on the stream, download the bytes."""
    lib = _lib.load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    nbytes = lib.pmetal_hip_tensor_size(t, x.size)
    dx = pm.DeviceBuffer.from_host(x) if x.size else pm.DeviceBuffer(16)
    dq = pm.DeviceBuffer(max(nbytes, 16))
    pm.check(lib.pmetal_hip_memset(dq.ptr, 0xA5, max(nbytes, 16), None))  # poison: every byte must be written
    pm.check(lib.pmetal_hip_quantize_dev(t, dx.ptr, x.size, dq.ptr, nbytes, None), "quantize")
    pm.check(lib.pmetal_hip_sync(None))
    return dq.to_host(np.uint8, nbytes)


def gpu_dequantize_dev(t, raw, n, order=0):
    lib = _lib.load()
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    dq = pm.DeviceBuffer.from_host(raw) if raw.size else pm.DeviceBuffer(16)
    dy = pm.DeviceBuffer(max(4 * n, 16))
    pm.check(lib.pmetal_hip_memset(dy.ptr, 0xA5, max(4 * n, 16), None))
    pm.check(lib.pmetal_hip_dequantize_dev(t, dq.ptr, raw.size, dy.ptr, n, order, None))
    pm.check(lib.pmetal_hip_sync(None))
    return dy.to_host(np.float32, n)


def gpu_qgemv(t, wq, n, k, x, x_dtype, order=0):
    """x: float32 array (x_dtype 0) or uint16 bf16 bit patterns (x_dtype 1)."""
    lib = _lib.load()
    dw = pm.DeviceBuffer.from_host(np.ascontiguousarray(wq, dtype=np.uint8))
    dx = pm.DeviceBuffer.from_host(x)
    dy = pm.DeviceBuffer(4 * n)
    pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, 4 * n, None))  # NaN poison
    pm.check(lib.pmetal_hip_qgemv(t, dw.ptr, n, k, dx.ptr, x_dtype, dy.ptr, order, None))
    pm.check(lib.pmetal_hip_sync(None))
    return dy.to_host(np.float32, n)


def rel_errors(got, want):
    """(element-wise max relative error over |want| > 1e-3*max|want|, normwise max error)."""
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    scale = np.max(np.abs(want))
    diff = np.abs(got - want)
    big = np.abs(want) > 1e-3 * scale
    elem = float(np.max(diff[big] / np.abs(want[big]))) if big.any() else 0.0
    return elem, float(np.max(diff) / scale) if scale > 0 else float(np.max(diff))


def first_mismatch(a, b, block):
    bad = np.nonzero(a != b)[0]
    if bad.size == 0:
        return "identical"
    i = int(bad[0])
    return (f"{bad.size} differing bytes in {np.unique(bad // block).size} blocks; first at byte {i} "
            f"(block {i // block}, offset {i % block}): got {a[i]} want {b[i]}")
