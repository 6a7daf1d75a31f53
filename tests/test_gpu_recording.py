"""GPU: a recorded launch sequence (HIP graph) replays to the same bits as the eager launches.

A recording is replayed several times with eager work and synchronisations of the program between the replays,
and every replay is checked against the eager result."""
import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import Q4K, Q6K, Q8_0, weights
from pmetal_amd import _lib

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    pm.init(0)


def test_recorded_decode_projections_replay_bit_exact(oracle):
    lib = _lib.load()
    shapes = [(Q4K, 1024, 1024), (Q4K, 1024, 1024), (Q4K, 2048, 1024), (Q6K, 1024, 1024), (Q4K, 3072, 1024),
              (Q4K, 3072, 1024), (Q8_0, 512, 1024), (Q4K, 1024, 3072), (Q6K, 4096, 1024), (Q4K, 16384, 4096)]
    xs = {k: pm.DeviceBuffer.from_host(oracle.f32_to_bf16_bits(np.random.default_rng(k).standard_normal(k).astype(np.float32)))
          for k in (1024, 3072, 4096)}
    descs = (_lib.LinearDesc * len(shapes))()
    keep = []
    for i, (t, n, k) in enumerate(shapes):
        w = pm.DeviceBuffer.from_host(oracle.quantize(t, weights(500 + i, n * k)))
        y = pm.DeviceBuffer(4 * n)
        keep.append((w, y, n))
        descs[i] = _lib.LinearDesc(t, pm.DTYPE_BF16, 0, 0, n, k, w.ptr, xs[k].ptr, y.ptr)

    def clear():
        for _, y, n in keep:
            pm.check(lib.pmetal_hip_memset(y.ptr, 0xFF, 4 * n, None))
        pm.check(lib.pmetal_hip_sync(None))

    clear()
    pm.check(lib.pmetal_hip_qgemv_batch(descs, len(shapes), None))
    pm.check(lib.pmetal_hip_sync(None))
    eager = [y.to_host(np.float32).copy() for _, y, _ in keep]
    assert all(np.isfinite(e).all() for e in eager)

    stream = lib.pmetal_hip_stream_create()
    assert stream
    try:
        pm.check(lib.pmetal_hip_record_begin(stream))
        assert lib.pmetal_hip_memset(keep[0][1].ptr, 0, 16, stream) != 0  # refuses to be recorded
        lib.pmetal_hip_clear_error()
        pm.check(lib.pmetal_hip_qgemv_batch(descs, len(shapes), stream))
        rec = lib.pmetal_hip_record_end(stream)
        assert rec, lib.pmetal_hip_last_error_message()
        try:
            for rep in range(4):
                clear()  # eager work of the program between replays
                pm.check(lib.pmetal_hip_replay(rec, stream))
                pm.check(lib.pmetal_hip_sync(stream))
                for (w, y, n), want in zip(keep, eager):
                    assert np.array_equal(y.to_host(np.float32), want), rep
        finally:
            pm.check(lib.pmetal_hip_recording_destroy(rec))
    finally:
        pm.check(lib.pmetal_hip_stream_destroy(stream))


def test_record_argument_errors():
    lib = _lib.load()
    assert lib.pmetal_hip_record_begin(None) != 0
    assert not lib.pmetal_hip_record_end(None)
    assert lib.pmetal_hip_replay(None, None) != 0
    assert lib.pmetal_hip_recording_destroy(None) == 0
    assert lib.pmetal_hip_stream_destroy(None) == 0
    lib.pmetal_hip_clear_error()


def test_recorded_qgemm_survives_a_larger_call_on_the_same_stream(oracle):
    """A recording of the fused GEMM names the library's scratch buffer.  A larger call on the same stream afterwards
    gets a new buffer, the recorded one stays alive, and the replay reproduces the eager bits; a shape the stream's
    buffer cannot hold is refused while the stream is being recorded."""
    lib = _lib.load()
    n, k, m = 512, 1024, 24
    w = pm.DeviceBuffer.from_host(oracle.quantize(Q4K, weights(900, n * k)))
    xb = oracle.f32_to_bf16_bits(np.random.default_rng(901).standard_normal(m * k).astype(np.float32))
    x = pm.DeviceBuffer.from_host(xb)
    y = pm.DeviceBuffer(4 * m * n)
    n2, k2, m2 = 768, 2048, 200
    w2 = pm.DeviceBuffer.from_host(oracle.quantize(Q4K, weights(902, n2 * k2)))
    x2 = pm.DeviceBuffer.from_host(oracle.f32_to_bf16_bits(np.random.default_rng(903).standard_normal(m2 * k2).astype(np.float32)))
    y2 = pm.DeviceBuffer(4 * m2 * n2)
    stream = lib.pmetal_hip_stream_create()
    assert stream
    try:
        # nothing has run on this stream yet: a recording cannot allocate the scratch
        pm.check(lib.pmetal_hip_record_begin(stream))
        rc = lib.pmetal_hip_qgemm(Q4K, w.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_F32, 0, stream)
        assert rc == 1 and b"recorded" in lib.pmetal_hip_last_error_message()
        lib.pmetal_hip_clear_error()
        dead = lib.pmetal_hip_record_end(stream)
        if dead:
            pm.check(lib.pmetal_hip_recording_destroy(dead))
        lib.pmetal_hip_clear_error()
        # eager run (allocates the stream's scratch), then the recording
        pm.check(lib.pmetal_hip_qgemm(Q4K, w.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_F32, 0, stream))
        pm.check(lib.pmetal_hip_sync(stream))
        eager = y.to_host(np.float32).copy()
        assert np.isfinite(eager).all()
        pm.check(lib.pmetal_hip_record_begin(stream))
        pm.check(lib.pmetal_hip_qgemm(Q4K, w.ptr, n, k, x.ptr, pm.DTYPE_BF16, m, y.ptr, pm.DTYPE_F32, 0, stream))
        rec = lib.pmetal_hip_record_end(stream)
        assert rec, lib.pmetal_hip_last_error_message()
        try:
            for rep in range(3):
                # a larger product on the same stream between replays: its scratch must not replace the recorded one
                pm.check(lib.pmetal_hip_qgemm(Q4K, w2.ptr, n2, k2, x2.ptr, pm.DTYPE_BF16, m2, y2.ptr, pm.DTYPE_F32, 0, stream))
                pm.check(lib.pmetal_hip_memset(y.ptr, 0xFF, 4 * m * n, None))
                pm.check(lib.pmetal_hip_sync(None))
                pm.check(lib.pmetal_hip_replay(rec, stream))
                pm.check(lib.pmetal_hip_sync(stream))
                assert np.array_equal(y.to_host(np.float32), eager), rep
        finally:
            pm.check(lib.pmetal_hip_recording_destroy(rec))
    finally:
        pm.check(lib.pmetal_hip_stream_destroy(stream))
