"""The entry point that allocates nothing (pmetal_hip_qgemm_noalloc) against pmetal_hip_qgemm, through the C ABI.

Both run the same kernels with the same launch plan, one on the library's grown-on-demand workspace, the other on the
fixed scratch array in the code object, so the outputs must agree bit for bit (which also satisfies the 1e-3 bound of the
quantized linear).  Two calls in a row share the array: the second, smaller call must not see anything of the first."""
import numpy as np
import pytest

import pmetal_amd as pm
from pmetal_amd import _lib

pytestmark = pytest.mark.gpu
Q8_0, Q4K, Q6K = 8, 12, 14


def _bind(lib):
    return lib.pmetal_hip_qgemm_noalloc


def _both(lib, fn, t, n, k, m, seed, y_dtype=0, order=0, x_dtype=1):
    rng = np.random.default_rng(seed)
    nbytes = lib.pmetal_hip_tensor_size(t, n * k)
    w = rng.integers(0, 256, nbytes, dtype=np.uint8)
    # keep every f16 scale field finite: clear the top exponent bit of d (and dmin)
    ts = lib.pmetal_hip_type_size(t)
    blocks = w.reshape(-1, ts)
    for off in {Q4K: (1, 3), Q6K: (209,), Q8_0: (1,)}[t]:
        blocks[:, off] &= 0x3F
    x = rng.standard_normal(m * k).astype(np.float32)
    if x_dtype == 1:
        xb = ((x.view(np.uint32) + 0x7FFF + ((x.view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16)
    else:
        xb = x
    dw, dx = pm.DeviceBuffer.from_host(w), pm.DeviceBuffer.from_host(xb)
    ysz = m * n * (4 if y_dtype == 0 else 2)
    outs = []
    for f in (lib.pmetal_hip_qgemm, fn):
        dy = pm.DeviceBuffer(ysz)
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, ysz, None))
        pm.check(f(t, dw.ptr, n, k, dx.ptr, x_dtype, m, dy.ptr, y_dtype, order, None))
        pm.check(lib.pmetal_hip_sync(None))
        outs.append(dy.to_host(np.uint8, ysz))
    return outs


def test_noalloc_equals_qgemm_two_calls_in_a_row():
    lib = _lib.load()
    pm.init(0)
    fn = _bind(lib)
    # first a call with a K split (partial tiles in the scratch), then a smaller one over the same array
    for (t, n, k, m, y_dtype, order, x_dtype) in ((Q4K, 1024, 4096, 48, 0, 0, 1), (Q4K, 512, 1024, 5, 1, 1, 1),
                                                  (Q6K, 768, 2048, 33, 0, 0, 0), (Q6K, 256, 512, 1, 1, 0, 1),
                                                  (Q8_0, 512, 2048, 130, 0, 0, 1), (Q8_0, 256, 256, 7, 0, 0, 0)):
        print("case", t, n, k, m, y_dtype, order, x_dtype, flush=True)
        a, b = _both(lib, fn, t, n, k, m, seed=n + m, y_dtype=y_dtype, order=order, x_dtype=x_dtype)
        assert np.array_equal(a, b), (t, n, k, m)
        assert not np.all(a == 0xFF)


def test_noalloc_rejects_what_does_not_fit():
    lib = _lib.load()
    pm.init(0)
    fn = _bind(lib)
    d = pm.DeviceBuffer(4096)
    # 2048 activation rows of k = 8192 need 75 MB of converted activations: refused before anything is launched
    assert fn(Q4K, d.ptr, 14336, 8192, d.ptr, 1, 2048, d.ptr, 0, 0, None) == 7
    assert b"scratch" in lib.pmetal_hip_last_error_message()
    assert fn(13, d.ptr, 256, 256, d.ptr, 1, 16, d.ptr, 0, 0, None) == 2  # Q5_K goes through re-blocking
    assert fn(Q4K, d.ptr, 256, 256, None, 1, 16, d.ptr, 0, 0, None) == 1
