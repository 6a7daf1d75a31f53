"""KL-calibration metric and per-tensor calibration (crates/pmetal-gguf/src/dynamic.rs:140-180, :420-502): the oracle
against what pins it, then the device metric and the GPU round trips against the oracle."""
import math

import numpy as np
import pytest

Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K, Q8K = 8, 10, 11, 12, 13, 14, 15


def test_kl_divergence_known_answers(oracle):
    kl = oracle.kl_divergence
    # the reference's own tests (dynamic.rs:934-956)
    data = np.array([1, 2, 3, 4, 5], np.float32)
    assert kl(data, data) < 1e-10
    assert 0.0 < kl(data, np.array([1.1, 2.1, 2.9, 4.2, 4.8], np.float32)) < 1.0
    assert kl(np.zeros(8, np.float32), np.zeros(8, np.float32)) == 0.0
    assert kl(np.zeros(0, np.float32), np.zeros(0, np.float32)) == 0.0
    # by hand: orthogonal unit vectors: rmse = sqrt(2/2) = 1 over rms(original) = sqrt(1/2); cosine distance 1
    assert kl(np.array([1, 0], np.float32), np.array([0, 1], np.float32)) == pytest.approx(math.sqrt(2) + 1, rel=1e-15)
    # a doubled vector: error equals the original (nrmse 1), direction kept (cosine distance 0)
    assert kl(data, 2 * data) == pytest.approx(1.0, abs=1e-15)
    # a flipped vector: error twice the original, cosine similarity -1
    assert kl(data, -data) == pytest.approx(4.0, abs=1e-15)
    # zero original, non-zero reconstruction: both terms fall back (nrmse 0, cosine similarity 1)
    assert kl(np.zeros(4, np.float32), np.ones(4, np.float32)) == 0.0
    # non-zero original, zero reconstruction: nrmse 1, cosine similarity falls back to 1
    assert kl(data, np.zeros(5, np.float32)) == pytest.approx(1.0, abs=1e-15)
    # against numpy in f64 (the difference is taken in f32 first, as the reference takes it)
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal(5000).astype(np.float32), rng.standard_normal(5000).astype(np.float32)
    d = (a - b).astype(np.float64)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    want = math.sqrt((d * d).mean()) / math.sqrt((a64 * a64).mean()) + 1 - (a64 @ b64) / math.sqrt((a64 @ a64) * (b64 @ b64))
    assert kl(a, b) == pytest.approx(want, rel=1e-12)


def test_critical_layers_and_calibration_logic(oracle):
    # dynamic.rs:789-800
    assert all(oracle.is_critical_layer(n) for n in ("lm_head.weight", "model.output.weight", "model.embed_tokens.weight", "token_embd.weight"))
    assert not oracle.is_critical_layer("model.layers.0.mlp.weight")
    # dynamic.rs:968-985: a critical layer gets the fallback type whatever the data
    t, score, scores = oracle.calibrate_tensor("model.lm_head.weight", np.ones(1024, np.float32), [32, 32])
    assert (t, score, scores) == (Q8K, 0.0, [(Q8K, 0.0)])
    # dynamic.rs:987-1018: the ramp; the selected type is a candidate, at least one candidate was scored
    data = (np.arange(256) * 0.01 - 1.28).astype(np.float32)
    t, score, scores = oracle.calibrate_tensor("model.layers.0.mlp.gate_proj.weight", data, [1, 256])
    assert t in oracle.DEFAULT_CANDIDATES and scores and [s[0] for s in scores] == [Q8K, Q6K, Q5K, Q4K, Q3K, Q2K]
    assert scores[0][1] < 0.01 and t == max((s for s in scores if s[1] <= 0.01), key=lambda s: [Q8K, Q6K, Q5K, Q4K, Q3K, Q2K].index(s[0]))[0]
    # the most compressed candidate under the threshold wins; none under it -> the first (highest quality) one
    x = (np.random.default_rng(1).standard_normal(4096) * 0.02).astype(np.float32)
    _, _, scores = oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 256], order=oracle.ORDER_GGML)
    by = dict(scores)
    assert by[Q8K] < by[Q6K] < by[Q5K] < by[Q4K] < by[Q3K] < by[Q2K]  # fewer bits, more loss (in the order that inverts the quantizer)
    assert oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 256], kl_threshold=by[Q5K] * 1.01, order=oracle.ORDER_GGML)[0] == Q5K
    assert oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 256], kl_threshold=by[Q4K] * 1.01, order=oracle.ORDER_GGML)[0] == Q4K
    assert oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 256], kl_threshold=1e-9, order=oracle.ORDER_GGML)[0] == Q8K
    # in the reference dequantizer's own order Q4_K and Q5_K come back scrambled: their scores are of order one
    _, _, ref_scores = oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 256])
    ref_by = dict(ref_scores)
    assert ref_by[Q4K] > 1.0 and ref_by[Q5K] > 1.0 and ref_by[Q6K] == by[Q6K] and ref_by[Q8K] == by[Q8K]
    # a shape whose byte size is not the data's: every dequantize fails, the fallback with f64::MAX comes back (:468-475)
    t, score, scores = oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 200])
    assert t == Q8K and score == np.finfo(np.float64).max and len(scores) == 1
    # a shape a few elements short of the data still has the data's byte size: it is scored on the elements it names
    t, score, scores = oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 255])
    assert len(scores) == 6 and score < 0.01
    # no candidate that the quantizer implements (here and in the reference: the i-quants, quantize.rs:82-85)
    assert oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [16, 256], candidates=(16, 17))[1] == np.finfo(np.float64).max


def test_q8k_dequantize_known_answers(oracle):
    # k_quants.rs:1345-1365: d = 0.5, qs[i] = i % 128
    import struct
    q = (np.arange(256) % 128).astype(np.int8)
    blk = np.frombuffer(struct.pack("<f", 0.5) + q.tobytes() + bytes(32), np.uint8)
    out = oracle.dequantize(Q8K, blk, [256])
    assert out[0] == 0.0 and out[1] == 0.5 and out[2] == 1.0 and out[10] == 5.0 and out[255] == 63.5
    x = ((np.arange(256) - 128.0) * 0.01).astype(np.float32)
    back = oracle.dequantize(Q8K, oracle.quantize(Q8K, x), [256])
    assert np.sqrt(np.mean((back - x) ** 2)) < 0.01 and np.abs(back - x).max() < 0.02  # k_quants.rs:1421-1443


@pytest.mark.gpu
def test_gpu_kl_divergence_and_q8k_round_trip(oracle):
    import pmetal_amd as pm
    from pmetal_amd import gguf
    pm.init(0)
    rng = np.random.default_rng(5)
    for n in (1, 3, 5, 257, 4096, 100003, 1 << 22):
        a = rng.standard_normal(n).astype(np.float32)
        b = (a + rng.standard_normal(n).astype(np.float32) * np.float32(0.05)).astype(np.float32)
        da, db = pm.DeviceBuffer.from_host(np.concatenate([a, np.zeros(4, np.float32)])), pm.DeviceBuffer.from_host(np.concatenate([b, np.zeros(4, np.float32)]))
        got, want = gguf.kl_divergence_dev(da, db, n), oracle.kl_divergence(a, b)
        assert got == pytest.approx(want, rel=1e-11), n
    z = pm.DeviceBuffer.from_host(np.zeros(64, np.float32))
    one = pm.DeviceBuffer.from_host(np.ones(64, np.float32))
    assert gguf.kl_divergence_dev(z, z, 64) == 0.0 and gguf.kl_divergence_dev(z, one, 64) == 0.0 and gguf.kl_divergence_dev(one, z, 64) == 1.0
    assert gguf.kl_divergence_dev(z, z, 0) == 0.0
    # Q8_K through the generic quantize / dequantize entry points, ragged length included
    for n in (256, 1000, 1 << 16):
        x = rng.standard_normal(n).astype(np.float32)
        q = pm.quantize(x, Q8K)
        assert np.array_equal(q, oracle.quantize(Q8K, x))
        assert np.array_equal(pm.dequantize(q, Q8K, [n]).view(np.uint32), oracle.dequantize(Q8K, q, [n]).view(np.uint32))


@pytest.mark.gpu
def test_gpu_calibrate_tensor_matches_oracle(oracle):
    import pmetal_amd as pm
    from pmetal_amd import gguf
    pm.init(0)
    rng = np.random.default_rng(6)
    tensors = {
        "blk.0.ffn_up.weight": ((rng.standard_normal(64 * 1024) * 0.02).astype(np.float32), [64, 1024]),
        "model.layers.3.self_attn.q_proj.weight": ((rng.standard_normal(32 * 512) * np.repeat(np.exp(rng.uniform(-2, 2, 64)), 256)).astype(np.float32), [32, 512]),
        "model.layers.0.mlp.gate_proj.weight": ((np.arange(256) * 0.01 - 1.28).astype(np.float32), [1, 256]),
        "model.lm_head.weight": (np.ones(1024, np.float32), [32, 32]),
        "blk.1.attn_k.weight": (np.zeros(512, np.float32), [2, 256]),
    }
    for name, (x, shape) in tensors.items():
        for kwargs in ({}, {"order": 1}, {"sample_size": 300}, {"kl_threshold": 0.05, "order": 1}, {"kl_threshold": 1e-9},
                       {"candidates": (Q6K, Q4K), "fallback_type": Q6K, "order": 1}, {"candidates": (Q3K, Q2K), "kl_threshold": 0.5}, {"candidates": (16, 17)}):
            wt, ws, wall = oracle.calibrate_tensor(name, x, shape, **kwargs)
            gt, gs, gall = gguf.calibrate_tensor(name, x, shape, **kwargs)
            assert gt == wt and [t for t, _ in gall] == [t for t, _ in wall], (name, kwargs)
            # the score is nrmse + (1 - cos): the f64 sums differ in their last bits with the summation order, which the
            # subtraction from 1 turns into an absolute error of a few 1e-16
            assert gs == pytest.approx(ws, rel=1e-10, abs=1e-14), (name, kwargs)
            for (_, a), (_, b) in zip(gall, wall):
                assert a == pytest.approx(b, rel=1e-10, abs=1e-14), (name, kwargs)
    x = tensors["blk.0.ffn_up.weight"][0]
    t, score, _ = gguf.calibrate_tensor("blk.0.ffn_up.weight", x, [64, 1000])
    assert t == Q8K and score == np.finfo(np.float64).max
    got, want = gguf.calibrate_tensor("blk.0.ffn_up.weight", x, [64, 1023]), oracle.calibrate_tensor("blk.0.ffn_up.weight", x, [64, 1023])
    assert got[0] == want[0] and got[1] == pytest.approx(want[1], rel=1e-10, abs=1e-14) and len(got[2]) == len(want[2]) == 6


@pytest.mark.gpu
def test_gpu_fused_dequantize_and_score_equals_the_two_steps(oracle):
    """pmetal_hip_kl_divergence_quantized_dev against dequantize_dev + kl_divergence_dev and against the oracle, for every
    k-quant type, both element orders, lengths that end inside a block and inside a float4, random block bytes."""
    import pmetal_amd as pm
    from pmetal_amd import _lib, gguf
    pm.init(0)
    lib = _lib.load()
    rng = np.random.default_rng(31)
    n_full = 256 * 700
    x = (rng.standard_normal(n_full) * 0.02).astype(np.float32)
    dx = pm.DeviceBuffer.from_host(x)
    ddeq = pm.DeviceBuffer(4 * n_full)
    for t in (Q8K, Q6K, Q5K, Q4K, Q3K, Q2K):
        q = oracle.quantize(t, x)
        dq = pm.DeviceBuffer.from_host(q)
        for order in (0, 1):
            for n in (n_full, n_full - 1, n_full - 255, 256 * 300 + 7, 5, 1):
                got = gguf.kl_divergence_quantized_dev(t, dq, q.size, dx, n, order)
                pm.check(lib.pmetal_hip_dequantize_dev(t, dq.ptr, q.size, ddeq.ptr, n_full, order, None))
                two = gguf.kl_divergence_dev(dx, ddeq, n)
                want = oracle.kl_divergence(x[:n], oracle.dequantize(t, q, [n_full], order=order)[:n])
                assert got == pytest.approx(two, rel=1e-10, abs=1e-14), (t, order, n)
                assert got == pytest.approx(want, rel=1e-10, abs=1e-14), (t, order, n)
        # zero elements: 0.0 without touching the device; more elements than the blocks hold: invalid size
        assert gguf.kl_divergence_quantized_dev(t, dq, q.size, dx, 0) == 0.0
        sc = __import__("ctypes").c_double()
        assert lib.pmetal_hip_kl_divergence_quantized_dev(t, dq.ptr, q.size, dx.ptr, n_full + 1, 0, sc, None) == 3
        assert lib.pmetal_hip_kl_divergence_quantized_dev(t, dq.ptr, q.size - 2, dx.ptr, 16, 0, sc, None) == 3
        lib.pmetal_hip_clear_error()
    # a type with 32-element blocks has no fused comparison: the reference's unsupported-type class
    sc = __import__("ctypes").c_double()
    assert lib.pmetal_hip_kl_divergence_quantized_dev(Q8_0, dx.ptr, 34, dx.ptr, 32, 0, sc, None) == 2
    assert lib.pmetal_hip_kl_divergence_quantized_dev(Q4K, dx.ptr, 144, dx.ptr, 32, 7, sc, None) == 1
    lib.pmetal_hip_clear_error()
    # NaNs and infinities in random block bytes propagate as in the two-step path
    raw = rng.integers(0, 256, 176 * 64, dtype=np.uint8)
    draw = pm.DeviceBuffer.from_host(raw)
    got = gguf.kl_divergence_quantized_dev(Q5K, draw, raw.size, dx, 64 * 256, 1)
    pm.check(lib.pmetal_hip_dequantize_dev(Q5K, draw.ptr, raw.size, ddeq.ptr, 64 * 256, 1, None))
    two = gguf.kl_divergence_dev(dx, ddeq, 64 * 256)
    assert (np.isnan(got) and np.isnan(two)) or got == pytest.approx(two, rel=1e-10)
