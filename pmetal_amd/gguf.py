"""Host-side mirror of the reference's quantize / dequantize / quantized-linear API over the C ABI.

Names, argument meaning and error behaviour follow the Rust interface the kernels stand in for:

* ``GgmlType``        -- crates/pmetal-gguf/src/types.rs:16-187
* ``quantize``        -- crates/pmetal-gguf/src/quantize.rs:17 ``quantize(data, dtype) -> Vec<u8>``
* ``dequantize``      -- crates/pmetal-gguf/src/dequant.rs:92 ``dequantize(data, dtype, shape) -> Vec<f32>``
* ``DequantError``    -- crates/pmetal-gguf/src/dequant.rs:37-70
* ``GgufLinear``      -- the GGUF-typed counterpart of ``LayerWeight::matmul_from``
  (crates/pmetal-bridge/src/qwen3_native/weights.rs:66-84)
* ``use_more_bits`` / ``q4km_tensor_type`` -- crates/pmetal/src/commands/quantize.rs:988-1137

Everything computes on the GPU through ``libpmetal_hip.so``; nothing here falls back to the CPU.
"""
from __future__ import annotations

import ctypes as C
import enum

import numpy as np

from . import _lib


class GgmlType(enum.IntEnum):
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q8_1 = 9
    Q4K = 12
    Q5K = 13
    Q6K = 14
    Q8K = 15
    Q3K = 11
    Q2K = 10

    def type_size(self) -> int:
        return _lib.load().pmetal_hip_type_size(int(self))

    def block_size(self) -> int:
        return _lib.load().pmetal_hip_block_size(int(self))

    def tensor_size(self, n_elements: int) -> int:
        return _lib.load().pmetal_hip_tensor_size(int(self), n_elements)


ORDER_REF, ORDER_GGML = 0, 1
DTYPE_F32, DTYPE_BF16 = 0, 1


class PMetalHipError(RuntimeError):
    """A failed call; ``code`` is the PMETAL_HIP_ERR_* class."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[pmetal_hip {code}] {message}")
        self.code = code
        self.message = message


class QuantizationError(PMetalHipError):
    """PMetalError::Quantization (crates/pmetal-core/src/error.rs:50-52)."""


class DequantError(PMetalHipError):
    """DequantError (dequant.rs:37-70); ``kind`` names the variant."""
    KINDS = {2: "UnsupportedType", 3: "InvalidSize", 6: "InvalidShape", 7: "ShapeTooLarge"}

    @property
    def kind(self) -> str:
        return self.KINDS.get(self.code, "Other")


class NoDeviceError(PMetalHipError):
    pass


def check(rc: int, ctx: str = "") -> None:
    if rc == 0:
        return
    msg = _lib.load().pmetal_hip_last_error_message().decode("utf-8", "replace")
    if rc == 5:
        raise NoDeviceError(rc, msg)
    if ctx == "quantize" and rc in (2, 3):
        raise QuantizationError(rc, msg)
    if rc in DequantError.KINDS:
        raise DequantError(rc, msg)
    raise PMetalHipError(rc, msg)


def init(device: int = 0) -> None:
    check(_lib.load().pmetal_hip_init(device))


def device_count() -> int:
    return _lib.load().pmetal_hip_device_count()


def quantize(data, dtype: int) -> np.ndarray:
    """``quantize(data: &[f32], dtype) -> Vec<u8>``; bytes bit-identical to the reference CPU path."""
    lib = _lib.load()
    x = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
    out = np.empty(lib.pmetal_hip_tensor_size(int(dtype), x.size), dtype=np.uint8)
    check(lib.pmetal_hip_quantize(int(dtype), x.ctypes.data, x.size, out.ctypes.data, out.size), "quantize")
    return out


def dequantize(data, dtype: int, shape, order: int = ORDER_REF) -> np.ndarray:
    """``dequantize(data: &[u8], dtype, shape: &[i32]) -> Vec<f32>`` (flat, row-major)."""
    lib = _lib.load()
    raw = np.ascontiguousarray(data, dtype=np.uint8).reshape(-1)
    shp = (C.c_int32 * max(len(shape), 1))(*[int(d) for d in shape])
    nbytes, nelem = C.c_size_t(), C.c_size_t()
    check(lib.pmetal_hip_expected_byte_size(int(dtype), shp, len(shape), C.byref(nbytes), C.byref(nelem)))
    if raw.size != nbytes.value:  # reported by the library itself, before any allocation here
        check(lib.pmetal_hip_dequantize(int(dtype), raw.ctypes.data, raw.size, shp, len(shape), None, 0, order))
    out = np.empty(nelem.value, dtype=np.float32)
    check(lib.pmetal_hip_dequantize(int(dtype), raw.ctypes.data, raw.size, shp, len(shape), out.ctypes.data, out.size,
                                    order))
    return out


def use_more_bits(layer: int, n_layers: int) -> bool:
    return bool(_lib.load().pmetal_hip_use_more_bits(layer, n_layers))


def q4km_tensor_type(gguf_name: str, ndim: int, n_layers: int) -> GgmlType:
    return GgmlType(_lib.load().pmetal_hip_q4km_tensor_type(gguf_name.encode(), ndim, n_layers))


class DeviceBuffer:
    """A device allocation owned by the caller (freed on ``free()`` / garbage collection)."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = _lib.load().pmetal_hip_alloc(self.nbytes)
        if not self.ptr:
            check(_lib.load().pmetal_hip_last_error_code() or 4)

    @classmethod
    def from_host(cls, arr: np.ndarray) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        check(_lib.load().pmetal_hip_h2d(buf.ptr, arr.ctypes.data, arr.nbytes))
        return buf

    def to_host(self, dtype, count: int | None = None) -> np.ndarray:
        dt = np.dtype(dtype)
        n = self.nbytes // dt.itemsize if count is None else count
        out = np.empty(n, dtype=dt)
        check(_lib.load().pmetal_hip_d2h(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self) -> None:
        if getattr(self, "ptr", None):
            _lib.load().pmetal_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _dev_ptr(obj) -> int:
    if isinstance(obj, DeviceBuffer):
        return obj.ptr
    if hasattr(obj, "data_ptr"):  # a torch tensor on the GPU
        return int(obj.data_ptr())
    return int(obj)


def quantize_tensors_dev(tensors, stream=None):
    """The tensor loop of ``run_quantization`` (crates/pmetal/src/commands/quantize.rs:1378-1428) over tensors that are
    already on the device: ``tensors`` is a sequence of ``(dtype, src, n)`` (``src`` a device buffer or torch tensor of
    ``n`` f32 values); returns one ``DeviceBuffer`` of blocks per tensor.  One ``pmetal_hip_quantize_batch_dev`` call: the
    bytes of one ``quantize`` per tensor, the independent tensors spread over two streams inside the library."""
    lib = _lib.load()
    tensors = [(int(t), src, int(n)) for t, src, n in tensors]
    sizes = [lib.pmetal_hip_tensor_size(t, n) for t, _, n in tensors]
    outs = [DeviceBuffer(max(b, 16)) for b in sizes]
    descs = (_lib.QuantizeDesc * max(len(tensors), 1))()
    for i, (t, src, n) in enumerate(tensors):
        descs[i] = _lib.QuantizeDesc(t, 0, _dev_ptr(src) if n else None, n, outs[i].ptr, sizes[i])
    check(lib.pmetal_hip_quantize_batch_dev(descs, len(tensors), stream), "quantize")
    return outs


def q8k_size(n_elements: int) -> int:
    """Bytes of ``n_elements`` quantized to Q8_K (292 per 256, crates/pmetal-gguf/src/k_quants.rs:140-155)."""
    return _lib.load().pmetal_hip_q8k_size(n_elements)


def quantize_q8k_dev(x, n: int, out=None, stream=None) -> DeviceBuffer:
    """``quantize_q8k`` (crates/pmetal-gguf/src/k_quants.rs:815-871) of ``n`` f32 values on the device."""
    lib = _lib.load()
    if out is None:
        out = DeviceBuffer(max(q8k_size(n), 16))
    check(lib.pmetal_hip_quantize_q8k_dev(_dev_ptr(x), n, _dev_ptr(out), q8k_size(n), stream), "quantize")
    return out


def qgemv_q8k(dtype: int, w, n: int, k: int, xq, y=None, stream=None) -> DeviceBuffer:
    """``y[r] = vec_dot_<dtype>_q8k(row r of w, xq)`` (crates/pmetal-gguf/src/vec_dot.rs:617-810; Q4_K, Q6_K, Q5_K, Q3_K, Q2_K), bit for bit."""
    lib = _lib.load()
    if y is None:
        y = DeviceBuffer(max(4 * n, 16))
    check(lib.pmetal_hip_qgemv_q8k(int(dtype), _dev_ptr(w), n, k, _dev_ptr(xq), _dev_ptr(y), stream))
    return y


def kl_divergence_dev(original, dequantized, n: int, stream=None) -> float:
    """``compute_kl_divergence`` (crates/pmetal-gguf/src/dynamic.rs:140-180) of two device arrays of ``n`` f32."""
    score = C.c_double()
    check(_lib.load().pmetal_hip_kl_divergence_dev(_dev_ptr(original), _dev_ptr(dequantized), n, C.byref(score), stream))
    return score.value


def kl_divergence_quantized_dev(dtype, quantized, nbytes: int, original, n: int, order: int = ORDER_REF, stream=None) -> float:
    """Dequantize-and-score in one pass for the k-quant types: the first ``n`` elements of the blocks against ``original``."""
    score = C.c_double()
    check(_lib.load().pmetal_hip_kl_divergence_quantized_dev(int(dtype), _dev_ptr(quantized), nbytes, _dev_ptr(original), n, order,
                                                             C.byref(score), stream))
    return score.value


def is_critical_layer(name: str) -> bool:
    """``DynamicQuantizer::is_critical_layer`` (crates/pmetal-gguf/src/dynamic.rs:254-268)."""
    return any(s in name for s in ("lm_head", "output", "token_embd", "embed_tokens", "wte", "final_norm", "ln_f"))


#: ``KlCalibrationConfig::default().candidates`` (crates/pmetal-gguf/src/dynamic.rs:104-121), best quality first
DEFAULT_KL_CANDIDATES = (GgmlType.Q8K, GgmlType.Q6K, GgmlType.Q5K, GgmlType.Q4K, GgmlType.Q3K, GgmlType.Q2K)


def calibrate_tensor(name: str, data, shape, candidates=DEFAULT_KL_CANDIDATES, kl_threshold: float = 0.01,
                     fallback_type: int = GgmlType.Q8K, sample_size: int = 0, order: int = ORDER_REF):
    """``DynamicQuantizer::calibrate_tensor`` (crates/pmetal-gguf/src/dynamic.rs:420-502) with the round trips on the GPU:
    the tensor is uploaded once, every candidate is quantized and scored on the device against its dequantized values (in
    the reference dequantizer's element order unless ``order`` says otherwise; the k-quants without storing them).  Returns ``(quant_type, kl_score, all_scores)``.  As in
    the reference, a candidate the quantizer does not implement is skipped."""
    lib = _lib.load()
    x = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
    if is_critical_layer(name):
        return int(fallback_type), 0.0, [(int(fallback_type), 0.0)]
    n = x.size
    n_shape = int(np.prod([int(d) for d in shape], dtype=np.int64)) if len(shape) else 1
    sample = sample_size if 0 < sample_size < n else n
    scores = []
    if n:
        dx, ddeq = DeviceBuffer.from_host(x), None
    for t in candidates:
        t = int(t)
        # quantize the whole tensor, dequantize what the shape asks for; a type without kernels, or a shape whose byte
        # size is not that of the quantized tensor, is an `Err(_) => continue` (dynamic.rs:456-464)
        nbytes = lib.pmetal_hip_tensor_size(t, n)
        if not lib.pmetal_hip_is_supported(t) or n_shape > n or lib.pmetal_hip_tensor_size(t, n_shape) != nbytes:
            continue
        if n_shape == 0:
            scores.append((t, 0.0))
            continue
        dq = DeviceBuffer(max(nbytes, 16))
        check(lib.pmetal_hip_quantize_dev(t, dx.ptr, n, dq.ptr, nbytes, None), "quantize")
        if lib.pmetal_hip_block_size(t) == 256:  # k-quants: decoded and compared in one pass, nothing stored
            scores.append((t, kl_divergence_quantized_dev(t, dq, nbytes, dx, min(sample, n_shape), order)))
        else:
            ddeq = ddeq or DeviceBuffer(4 * max(n, 4))
            check(lib.pmetal_hip_dequantize_dev(t, dq.ptr, nbytes, ddeq.ptr, n_shape, order, None))
            scores.append((t, kl_divergence_dev(dx, ddeq, min(sample, n_shape))))
        dq.free()
    if not scores:
        big = float(np.finfo(np.float64).max)
        return int(fallback_type), big, [(int(fallback_type), big)]
    best_type, best_score = scores[0]
    for t, sc in reversed(scores):
        if sc <= kl_threshold:
            best_type, best_score = t, sc
            break
    return best_type, best_score, scores


class GgufLinear:
    """A GGUF-quantized weight ``[n, k]`` resident on the device; ``forward`` is ``x @ W^T``.

    Mirrors ``LayerWeight::matmul_from`` (crates/pmetal-bridge/src/qwen3_native/weights.rs:66-84): one token goes through
    the fused GEMV, several through the fused GEMM.  ``w`` are the packed block bytes (host array or device buffer).
    As the reference brings a weight into its matmul's layout when the model is loaded (weights.rs:29-45),
    Every type has matrix kernels that read its blocks as they are, so nothing is prepared at load time; ``prepare_gemm``
    is accepted and ignored (it used to re-block Q5_K / Q3_K / Q2_K weights into the Q6_K form their GEMM then multiplied
    with: ``pmetal_hip_reblock_dev`` / ``pmetal_hip_qgemm_reblocked`` still do that for callers who ask)."""

    def __init__(self, dtype: int, n: int, k: int, w, order: int = ORDER_REF, prepare_gemm: bool = False):
        self.dtype, self.n, self.k, self.order = GgmlType(dtype), int(n), int(k), order
        expected = self.dtype.tensor_size(self.n * self.k)
        if isinstance(w, np.ndarray):
            if w.size != expected:
                raise DequantError(3, f"Invalid data size: expected {expected} bytes, got {w.size}")
            w = DeviceBuffer.from_host(np.ascontiguousarray(w, dtype=np.uint8))
        self.w = w
        self.reblocked, self.reblocked_len = None, 0  # (kept for callers that look at them)

    def forward(self, x, m: int = 1, x_dtype: int = DTYPE_BF16, y=None, y_dtype: int = DTYPE_F32, stream=None):
        """``x``: device buffer of ``[m, k]`` activations; returns the device buffer of ``[m, n]`` outputs."""
        lib = _lib.load()
        if y is None:
            y = DeviceBuffer(m * self.n * (4 if y_dtype == DTYPE_F32 else 2))
        check(lib.pmetal_hip_qlinear(int(self.dtype), _dev_ptr(self.w), self.n, self.k, _dev_ptr(x), x_dtype, m,
                                     _dev_ptr(y), y_dtype, self.order, stream))
        return y
