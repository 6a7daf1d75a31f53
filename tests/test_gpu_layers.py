"""GPU: two decoder-layer-shaped stacks of GGUF-typed projections through ``GgufLinear`` (the GGUF counterpart of
``LayerWeight::matmul_from``, crates/pmetal-bridge/src/qwen3_native/weights.rs:29-84) against the oracle.

Layer A has the Q4_K_M recipe's types for a layer that gets more bits (attn_v and ffn_down in Q6_K), layer B a fused
attn_qkv tensor (Q5_K by the recipe) and, as a KL calibration may choose, a Q3_K up- and a Q2_K gate-projection.  The glue
between the projections (an elementwise mix in place of attention, SiLU gating, residuals, rounding of the activations to
bf16) is host code shared by both paths, so what is compared is the chain of quantized linears: every projection against the
oracle's dequantize-then-matmul on the same input, and the stack's output against a run that never touches the GPU."""
import numpy as np
import pytest

import pmetal_amd as pm
from gpu_util import weights

pytestmark = pytest.mark.gpu
H, KV, FF = 1024, 256, 2816
TOL = 1e-3


@pytest.fixture(scope="module", autouse=True)
def _device():
    pm.init(0)


def _layers(oracle):
    n_layers = 8
    spec = []
    # layer A: blk.0 of an 8-layer model (use_more_bits -> Q6_K for attn_v and ffn_down)
    a = {nm: int(pm.q4km_tensor_type(f"blk.0.{nm}.weight", 2, n_layers)) for nm in
         ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")}
    assert [a["attn_v"], a["ffn_down"], a["attn_q"]] == [14, 14, 12]
    spec.append(a)
    # layer B: blk.1 with a fused attn_qkv (Q5_K by the recipe); up / gate as a calibration might pick them
    b = {nm: int(pm.q4km_tensor_type(f"blk.1.{nm}.weight", 2, n_layers)) for nm in ("attn_qkv", "attn_output", "ffn_down")}
    assert b["attn_qkv"] == 13 and b["ffn_down"] == 12
    b["ffn_up"], b["ffn_gate"] = 11, 10
    spec.append(b)
    shapes = {"attn_q": (H, H), "attn_k": (KV, H), "attn_v": (KV, H), "attn_qkv": (H + 2 * KV, H), "attn_output": (H, H),
              "ffn_gate": (FF, H), "ffn_up": (FF, H), "ffn_down": (H, FF)}
    out = []
    for li, types in enumerate(spec):
        layer = {}
        for j, (nm, t) in enumerate(sorted(types.items())):
            n, k = shapes[nm]
            raw = oracle.quantize(t, weights(7000 + 10 * li + j, n * k, std=0.03))
            layer[nm] = (t, n, k, raw)
        out.append(layer)
    return out


def _errors(got, want):
    """(element-wise max relative error over |want| > 1e-2 * max|want|, max error relative to max|want|).  The activations
    between the projections are products (gated, mixed): heavy-tailed, so that an f32 dot product over them is itself only
    good to about 1e-6 of the row's scale; outputs a thousand times smaller than the largest cannot then hold 1e-3, whatever
    computes them, and the element-wise bound is taken over outputs within a hundredth of the largest."""
    got, want = got.astype(np.float64), want.astype(np.float64)
    scale = np.max(np.abs(want))
    diff = np.abs(got - want)
    big = np.abs(want) > 1e-2 * scale
    return (float(np.max(diff[big] / np.abs(want[big]))) if big.any() else 0.0), float(np.max(diff) / scale)


def _bf16(oracle, a):
    bits = oracle.f32_to_bf16_bits(np.ascontiguousarray(a, dtype=np.float32).reshape(-1))
    return bits.reshape(a.shape), oracle.bf16_bits_to_f32(bits).reshape(a.shape)


def _forward(oracle, layers, x, project):
    """x: [m, H] f32.  project(layer_index, name, bits [m, k], values [m, k]) -> [m, n] f32."""
    m = x.shape[0]
    for li, layer in enumerate(layers):
        xb, xr = _bf16(oracle, x)
        if "attn_qkv" in layer:
            qkv = project(li, "attn_qkv", xb, xr)
            q, kk, v = qkv[:, :H], qkv[:, H:H + KV], qkv[:, H + KV:]
        else:
            q, kk, v = project(li, "attn_q", xb, xr), project(li, "attn_k", xb, xr), project(li, "attn_v", xb, xr)
        a = q.copy()
        a[:, :KV] += kk * v  # stands in for attention: every projection's output reaches the next one
        ab, ar = _bf16(oracle, a)
        h = x + project(li, "attn_output", ab, ar)
        hb, hr = _bf16(oracle, h)
        g, u = project(li, "ffn_gate", hb, hr), project(li, "ffn_up", hb, hr)
        f = g / (1.0 + np.exp(-g.astype(np.float64))).astype(np.float32) * u
        fb, fr = _bf16(oracle, f)
        x = h + project(li, "ffn_down", fb, fr)
        assert x.shape == (m, H)
    return x


@pytest.mark.parametrize("m", [1, 5, 24])
def test_two_layer_stack_of_gguf_linears(oracle, m):
    layers = _layers(oracle)
    lin = [{nm: pm.GgufLinear(t, n, k, raw, prepare_gemm=True) for nm, (t, n, k, raw) in layer.items()} for layer in layers]
    # (every type multiplies its blocks as they are: nothing is prepared)
    assert all(l.reblocked is None for layer in lin for l in layer.values())
    threads = min(oracle.host_threads(), 16)
    worst = [0.0]

    def on_cpu(li, nm, bits, vals):
        t, n, k, raw = layers[li][nm]
        return oracle.qmatmul(t, raw, n, k, vals, threads=threads)

    def on_gpu(li, nm, bits, vals):
        t, n, k, raw = layers[li][nm]
        y = lin[li][nm].forward(pm.DeviceBuffer.from_host(bits), m=bits.shape[0], x_dtype=pm.DTYPE_BF16)
        got = y.to_host(np.float32).reshape(bits.shape[0], n)
        want = on_cpu(li, nm, bits, vals)  # the same input: this projection alone
        for row in range(bits.shape[0]):
            elem, norm = _errors(got[row], want[row])
            worst[0] = max(worst[0], elem, norm)
            assert elem <= TOL and norm <= TOL, (li, nm, row, elem, norm)
        return got

    x = np.random.default_rng(123 + m).standard_normal((m, H)).astype(np.float32)
    y_gpu = _forward(oracle, layers, x, on_gpu)
    y_cpu = _forward(oracle, layers, x, on_cpu)
    assert np.isfinite(y_gpu).all()
    # The two chains round their activations to bf16 between projections; where a last-bit difference of a projection lands
    # on a rounding boundary one activation moves by 2^-9 of its value, and later projections spread that (the gated
    # activations are heavy-tailed: one dominant element that flips moves the whole output by about 2^-9): the outputs agree to
    # a few bf16 steps, in the aggregate (relative L2) and element by element.
    l2 = float(np.linalg.norm(y_gpu - y_cpu) / np.linalg.norm(y_cpu))
    worst_el = float(np.max(np.abs(y_gpu - y_cpu)) / np.max(np.abs(y_cpu)))
    print(f"m={m}: worst single-projection error {worst[0]:.2e}, stack difference L2 {l2:.2e}, max {worst_el:.2e}")
    assert l2 <= 1e-2 and worst_el <= 2e-2, (l2, worst_el)


@pytest.mark.parametrize("t", [13, 11, 10])
def test_reblocked_gemm_equals_qgemm_and_rejects_bad_sizes(oracle, t):
    """pmetal_hip_qgemm_reblocked over weights re-blocked once gives what pmetal_hip_qgemm gives on the original blocks (a
    matrix kernel of the type's own), to the f32 summation order."""
    from pmetal_amd import _lib
    lib = _lib.load()
    n, k, m = 384, 2048, 40
    raw = oracle.quantize(t, weights(60 + t, n * k))
    xb = oracle.f32_to_bf16_bits(np.random.default_rng(61).standard_normal(m * k).astype(np.float32))
    dw, dx = pm.DeviceBuffer.from_host(raw), pm.DeviceBuffer.from_host(xb)
    size = lib.pmetal_hip_reblock_size(t, n, k)
    assert size == (2 if t in (13, 10) else 1) * n * (k // 256) * 210 and lib.pmetal_hip_reblock_size(12, n, k) == 0
    rb = pm.DeviceBuffer(size)
    pm.check(lib.pmetal_hip_reblock_dev(t, dw.ptr, n, k, 0, rb.ptr, size, None))
    for y_dtype, ysz in ((pm.DTYPE_F32, 4), (pm.DTYPE_BF16, 2)):
        y1, y2 = pm.DeviceBuffer(m * n * ysz), pm.DeviceBuffer(m * n * ysz)
        pm.check(lib.pmetal_hip_qgemm(t, dw.ptr, n, k, dx.ptr, pm.DTYPE_BF16, m, y1.ptr, y_dtype, 0, None))
        pm.check(lib.pmetal_hip_qgemm_reblocked(t, rb.ptr, size, n, k, dx.ptr, pm.DTYPE_BF16, m, y2.ptr, y_dtype, None))
        pm.check(lib.pmetal_hip_sync(None))
        if y_dtype == pm.DTYPE_F32:
            a, b = y1.to_host(np.float32), y2.to_host(np.float32)
            assert np.max(np.abs(a - b)) <= 1e-5 * np.max(np.abs(b))
        else:
            a, b = ((y.to_host(np.uint16).astype(np.uint32) << 16).view(np.float32) for y in (y1, y2))
            assert np.max(np.abs(a - b)) <= 2.0 ** -7 * np.max(np.abs(b))
    assert lib.pmetal_hip_reblock_dev(t, dw.ptr, n, k, 0, rb.ptr, size - 16, None) == 3
    assert lib.pmetal_hip_qgemm_reblocked(t, rb.ptr, size + 16, n, k, dx.ptr, pm.DTYPE_BF16, m, y1.ptr, 0, None) == 3
    assert lib.pmetal_hip_reblock_dev(12, dw.ptr, n, k, 0, rb.ptr, size, None) == 2
    lib.pmetal_hip_clear_error()
