"""The entry point that allocates nothing (pmetal_hip_qgemm_noalloc) against pmetal_hip_qgemm, through the C ABI.

Both run the same kernels with the same launch plan, one on the library's grown-on-demand workspace, the other on the
fixed scratch array in the code object, so the outputs must agree bit for bit (which also satisfies the 1e-3 bound of the
quantized linear).  Two calls in a row share the array: the second, smaller call must not see anything of the first."""
import ctypes as C

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
    for off in {Q4K: (1, 3), Q6K: (209,), Q8_0: (1,), 13: (1, 3), 11: (109,), 10: (81, 83)}[t]:
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
                                                  (Q8_0, 512, 2048, 130, 0, 0, 1), (Q8_0, 256, 256, 7, 0, 0, 0),
                                                  # Q5_K, Q3_K, Q2_K: the matrix kernels with a K split, then the short-batch
                                                  # kernels (rows of 32 and 24 super-blocks go in runs with partial tiles)
                                                  (Q4K, 900, 4096, 27, 0, 1, 1), (13, 640, 8192, 20, 0, 0, 1),
                                                  (13, 1024, 4096, 48, 0, 0, 1), (13, 512, 8192, 9, 1, 1, 1),
                                                  (11, 640, 2048, 40, 0, 0, 1), (11, 333, 6144, 4, 0, 0, 0),
                                                  (10, 512, 2048, 100, 1, 0, 1), (10, 250, 4096, 16, 0, 0, 1)):
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
    assert fn(15, d.ptr, 256, 256, d.ptr, 1, 16, d.ptr, 0, 0, None) == 2  # Q8_K: activations only, no GEMM
    assert fn(Q4K, d.ptr, 256, 256, None, 1, 16, d.ptr, 0, 0, None) == 1


def test_noalloc_records_on_a_stream_that_has_no_workspace():
    """What the entry point is for: on a fresh stream, where no call has grown a workspace yet, pmetal_hip_qgemm cannot be
    recorded (it would have to allocate) and pmetal_hip_qgemm_noalloc can; the replays give the bits of the eager call."""
    lib = _lib.load()
    pm.init(0)
    fn = _bind(lib)
    t, n, k, m = Q4K, 768, 2048, 40
    rng = np.random.default_rng(99)
    w = rng.integers(0, 256, lib.pmetal_hip_tensor_size(t, n * k), dtype=np.uint8)
    w.reshape(-1, 144)[:, (1, 3)] &= 0x3F
    x = rng.standard_normal(m * k).astype(np.float32)
    dw, dx = pm.DeviceBuffer.from_host(w), pm.DeviceBuffer.from_host(x)
    eager = pm.DeviceBuffer(m * n * 4)
    pm.check(lib.pmetal_hip_qgemm(t, dw.ptr, n, k, dx.ptr, 0, m, eager.ptr, 0, 0, None))
    pm.check(lib.pmetal_hip_sync(None))
    want = eager.to_host(np.uint8)
    lib.pmetal_hip_stream_create.restype = C.c_void_p
    lib.pmetal_hip_record_end.restype = C.c_void_p
    st = C.c_void_p(lib.pmetal_hip_stream_create())
    assert st.value
    dy = pm.DeviceBuffer(m * n * 4)
    pm.check(lib.pmetal_hip_record_begin(st))
    refused = lib.pmetal_hip_qgemm(t, dw.ptr, n, k, dx.ptr, 0, m, dy.ptr, 0, 0, st)
    rc = fn(t, dw.ptr, n, k, dx.ptr, 0, m, dy.ptr, 0, 0, st)
    rec = C.c_void_p(lib.pmetal_hip_record_end(st))
    assert refused == 1, "pmetal_hip_qgemm must refuse to allocate while the stream is being recorded"
    assert rc == 0 and rec.value
    for _ in range(3):
        pm.check(lib.pmetal_hip_memset(dy.ptr, 0xFF, m * n * 4, None))
        pm.check(lib.pmetal_hip_sync(None))
        pm.check(lib.pmetal_hip_replay(rec, st))
        pm.check(lib.pmetal_hip_sync(st))
        assert np.array_equal(dy.to_host(np.uint8), want)
    pm.check(lib.pmetal_hip_recording_destroy(rec))
    pm.check(lib.pmetal_hip_stream_destroy(st))


def test_noalloc_refuses_a_call_that_would_overlap_on_another_stream():
    """All calls on a device share one scratch array.  A second call on another stream while the first one's kernels may
    still run is refused (class 8) instead of racing; once the first stream has been waited for, it goes through."""
    lib = _lib.load()
    pm.init(0)
    fn = _bind(lib)
    t, n, k, m = Q4K, 14336, 4096, 512
    rng = np.random.default_rng(7)
    w = rng.integers(0, 256, lib.pmetal_hip_tensor_size(t, n * k), dtype=np.uint8)
    w.reshape(-1, 144)[:, (1, 3)] &= 0x3F
    x = rng.standard_normal(m * k).astype(np.float32)
    dw, dx = pm.DeviceBuffer.from_host(w), pm.DeviceBuffer.from_host(x)
    dy, dy2 = pm.DeviceBuffer(m * n * 4), pm.DeviceBuffer(m * n * 4)
    lib.pmetal_hip_stream_create.restype = C.c_void_p
    s1, s2 = C.c_void_p(lib.pmetal_hip_stream_create()), C.c_void_p(lib.pmetal_hip_stream_create())
    pm.check(lib.pmetal_hip_sync(None))
    seen_busy = False
    for _ in range(8):  # a queue of calls on one stream is fine ...
        pm.check(fn(t, dw.ptr, n, k, dx.ptr, 0, m, dy.ptr, 0, 0, s1))
    rc = fn(t, dw.ptr, n, k, dx.ptr, 0, m, dy2.ptr, 0, 0, s2)  # ... another stream behind it is not, while they run
    seen_busy = rc == 8
    if seen_busy:
        assert b"scratch" in lib.pmetal_hip_last_error_message()
    lib.pmetal_hip_clear_error()
    pm.check(lib.pmetal_hip_sync(s1))
    pm.check(fn(t, dw.ptr, n, k, dx.ptr, 0, m, dy2.ptr, 0, 0, s2))
    pm.check(lib.pmetal_hip_sync(s2))
    assert np.array_equal(dy.to_host(np.uint8), dy2.to_host(np.uint8))
    assert seen_busy or rc == 0  # eight 90 us calls were still queued unless the machine drained them first
    pm.check(lib.pmetal_hip_stream_destroy(s1))
    pm.check(lib.pmetal_hip_stream_destroy(s2))
