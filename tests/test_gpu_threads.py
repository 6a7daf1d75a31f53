"""Several host threads in the library at once (ctypes releases the GIL for the duration of a call): the error slot and
the GEMM workspace are per thread, the staging buffers of the host entry points are shared behind a lock.  Every thread's
results must be what a single thread gets."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import Q4K, Q6K, Q8_0, gpu_qgemv, rel_errors, weights

pytestmark = pytest.mark.gpu


def test_four_threads_quantize_dequantize_and_multiply(oracle):
    pm.init(0)
    lib = pm._lib.load()
    n, k, m = 700, 1024, 24
    jobs = []
    for i, t in enumerate([Q4K, Q6K, Q8_0, Q4K]):
        w = weights(300 + i, n * k, outliers=1e-3)
        x = np.random.default_rng(400 + i).standard_normal((m, k)).astype(np.float32)
        bits = oracle.f32_to_bf16_bits(x.reshape(-1))
        jobs.append((t, w, bits, oracle.bf16_bits_to_f32(bits).reshape(m, k)))

    def work(job):
        t, w, bits, xr = job
        pm.init(0)  # the current device is a per-thread setting
        out = []
        for _ in range(3):
            wq = pm.quantize(w, t)  # 700 Ki elements: the staged path of the host entry points
            back = pm.dequantize(wq, t, (n * k,))
            y1 = gpu_qgemv(t, wq, n, k, bits[:k], pm.DTYPE_BF16, 0)
            dw, dx = pm.DeviceBuffer.from_host(wq), pm.DeviceBuffer.from_host(bits)
            dy = pm.DeviceBuffer(4 * m * n)
            pm.check(lib.pmetal_hip_qgemm(t, dw.ptr, n, k, dx.ptr, pm.DTYPE_BF16, m, dy.ptr, pm.DTYPE_F32, 0, None))
            pm.check(lib.pmetal_hip_sync(None))
            out.append((wq, back, y1, dy.to_host(np.float32, m * n).reshape(m, n)))
            # an error in this thread lands in this thread's slot
            assert lib.pmetal_hip_qgemv(99, dw.ptr, n, k, dx.ptr, pm.DTYPE_BF16, dy.ptr, 0, None) != 0
            assert lib.pmetal_hip_last_error_code() != 0
            lib.pmetal_hip_clear_error()
        return out

    with ThreadPoolExecutor(4) as pool:
        results = list(pool.map(work, jobs))
    for (t, w, bits, xr), outs in zip(jobs, results):
        want_q = oracle.quantize(t, w, threads=8)
        want_back = oracle.dequantize(t, want_q, [n * k])
        want_y = oracle.qmatmul(t, want_q, n, k, xr, threads=8)
        for wq, back, y1, ym in outs:
            assert np.array_equal(wq, want_q)
            assert np.array_equal(back.view(np.uint32), want_back.view(np.uint32))
            for got, want in ((y1, want_y[0]), (ym.reshape(-1), want_y.reshape(-1))):
                elem, norm = rel_errors(got, want)
                assert elem <= 1e-3 and norm <= 1e-3, (t, elem, norm)
