"""ctypes binding of the CPU oracle (``libpmetal_oracle.so``).

Test infrastructure only: the test-suite, the smoke check and the benchmark's
CPU-baseline leg import this; the product package never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpmetal_oracle.so")

TYPE_F32, TYPE_F16, TYPE_Q8_0, TYPE_Q4K, TYPE_Q6K = 0, 1, 8, 12, 14
TYPE_Q5K, TYPE_Q8K = 13, 15
TYPE_Q2K, TYPE_Q3K = 10, 11
ORDER_REF, ORDER_GGML = 0, 1
OK, ERR_UNSUPPORTED_TYPE, ERR_INVALID_SIZE, ERR_INVALID_SHAPE, ERR_SHAPE_TOO_LARGE = 0, 2, 3, 6, 7


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a no-op when the library is newer than its sources)."""
    srcs = [os.path.join(HERE, f) for f in ("pmetal_oracle.c", "pmetal_oracle.h", "Makefile")]
    stale = force or not os.path.exists(LIB_PATH) or any(
        os.path.getmtime(s) > os.path.getmtime(LIB_PATH) for s in srcs
    )
    if stale:
        subprocess.run(["make", "-C", HERE, "-B", "libpmetal_oracle.so"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        f32p, u8p, i8p, i32p = (C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_int8),
                                C.POINTER(C.c_int32))
        L.pmo_f32_to_f16.argtypes, L.pmo_f32_to_f16.restype = [C.c_float], C.c_uint16
        L.pmo_f16_to_f32.argtypes, L.pmo_f16_to_f32.restype = [C.c_uint16], C.c_float
        L.pmo_f32_to_bf16.argtypes, L.pmo_f32_to_bf16.restype = [C.c_float], C.c_uint16
        L.pmo_bf16_to_f32.argtypes, L.pmo_bf16_to_f32.restype = [C.c_uint16], C.c_float
        L.pmo_nearest_int.argtypes, L.pmo_nearest_int.restype = [C.c_float], C.c_int32
        L.pmo_make_qkx1_quants.argtypes = [C.c_int32, C.c_int32, f32p, C.c_int32, f32p, f32p]
        L.pmo_make_qkx1_quants.restype = None
        L.pmo_make_qx_quants.argtypes = [C.c_int32, C.c_int32, f32p, C.c_int32, i8p]
        L.pmo_make_qx_quants.restype = C.c_float
        L.pmo_make_q3_quants.argtypes = [f32p, C.c_int32, C.c_int32, C.c_int32, i8p]
        L.pmo_make_q3_quants.restype = C.c_float
        L.pmo_get_scale_min_k4.argtypes = [C.c_int32, u8p, u8p, u8p]
        L.pmo_get_scale_min_k4.restype = None
        for name in ("pmo_type_size", "pmo_block_size"):
            getattr(L, name).argtypes, getattr(L, name).restype = [C.c_uint32], C.c_size_t
        L.pmo_tensor_size.argtypes, L.pmo_tensor_size.restype = [C.c_uint32, C.c_size_t], C.c_size_t
        for name in ("pmo_quantize_q8_0", "pmo_quantize_q4k", "pmo_quantize_q6k"):
            getattr(L, name).argtypes, getattr(L, name).restype = [f32p, C.c_size_t, u8p], None
        L.pmo_dequantize_q8_0.argtypes, L.pmo_dequantize_q8_0.restype = [u8p, C.c_size_t, f32p], None
        L.pmo_dequantize_q6k.argtypes, L.pmo_dequantize_q6k.restype = [u8p, C.c_size_t, f32p], None
        L.pmo_dequantize_q4k.argtypes = [u8p, C.c_size_t, f32p, C.c_uint32]
        L.pmo_dequantize_q4k.restype = None
        L.pmo_quantize.argtypes = [C.c_uint32, f32p, C.c_size_t, u8p, C.c_size_t]
        L.pmo_quantize.restype = C.c_int32
        L.pmo_dequantize.argtypes = [C.c_uint32, u8p, C.c_size_t, i32p, C.c_size_t, f32p, C.c_size_t,
                                     C.c_uint32]
        L.pmo_dequantize.restype = C.c_int32
        L.pmo_use_more_bits.argtypes, L.pmo_use_more_bits.restype = [C.c_size_t, C.c_size_t], C.c_int32
        L.pmo_is_quantizable_gguf_tensor.argtypes = [C.c_char_p, C.c_size_t]
        L.pmo_is_quantizable_gguf_tensor.restype = C.c_int32
        L.pmo_q4km_tensor_type.argtypes = [C.c_char_p, C.c_size_t, C.c_size_t]
        L.pmo_q4km_tensor_type.restype = C.c_uint32
        for name in ("pmo_qmatvec_f64", "pmo_qmatvec_f32"):
            getattr(L, name).argtypes = [C.c_uint32, u8p, C.c_size_t, C.c_size_t, f32p, f32p, C.c_uint32]
            getattr(L, name).restype = C.c_int32
        L.pmo_qmatmul_f64.argtypes = [C.c_uint32, u8p, C.c_size_t, C.c_size_t, f32p, C.c_size_t, f32p,
                                      C.c_uint32]
        L.pmo_qmatmul_f64.restype = C.c_int32
        L.pmo_kl_divergence.argtypes, L.pmo_kl_divergence.restype = [f32p, f32p, C.c_size_t], C.c_double
        L.pmo_q8k_size.argtypes, L.pmo_q8k_size.restype = [C.c_size_t], C.c_size_t
        L.pmo_quantize_q8k.argtypes, L.pmo_quantize_q8k.restype = [f32p, C.c_size_t, u8p], None
        for name in ("pmo_vec_dot_q4k_q8k", "pmo_vec_dot_q6k_q8k", "pmo_vec_dot_q5k_q8k", "pmo_vec_dot_q3k_q8k", "pmo_vec_dot_q2k_q8k"):
            getattr(L, name).argtypes, getattr(L, name).restype = [u8p, u8p, C.c_size_t], C.c_float
        L.pmo_qmatvec_q8k.argtypes = [C.c_uint32, u8p, C.c_size_t, C.c_size_t, u8p, f32p]
        L.pmo_qmatvec_q8k.restype = C.c_int32
        L.pmo_quantize_mt.argtypes = [C.c_uint32, f32p, C.c_size_t, u8p, C.c_size_t, C.c_int32]
        L.pmo_quantize_mt.restype = C.c_int32
        L.pmo_qmatvec_mt.argtypes = [C.c_uint32, u8p, C.c_size_t, C.c_size_t, f32p, f32p, C.c_uint32, C.c_int32, C.c_int32]
        L.pmo_qmatvec_mt.restype = C.c_int32
        L.pmo_qmatmul_f64_mt.argtypes = [C.c_uint32, u8p, C.c_size_t, C.c_size_t, f32p, C.c_size_t, f32p, C.c_uint32,
                                         C.c_int32]
        L.pmo_qmatmul_f64_mt.restype = C.c_int32
        _lib = L
    return _lib


def host_threads() -> int:
    """Threads worth starting on this host: the CPUs this process may run on."""
    try:
        return max(1, len(os.sched_getaffinity(0)))
    except AttributeError:
        return max(1, os.cpu_count() or 1)


def _f32p(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u8p(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def tensor_size(t: int, n: int) -> int:
    return lib().pmo_tensor_size(t, n)


def quantize(t: int, x: np.ndarray, threads: int = 1) -> np.ndarray:
    """quantize.rs:17 ``quantize(data, dtype)``: flat f32 -> block bytes (``threads`` > 1: the same bytes, block ranges
    spread over host threads)."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.zeros(tensor_size(t, x.size), dtype=np.uint8)
    if threads > 1:
        rc = lib().pmo_quantize_mt(t, _f32p(x), x.size, _u8p(out), out.size, threads)
    else:
        rc = lib().pmo_quantize(t, _f32p(x), x.size, _u8p(out), out.size)
    if rc != OK:
        raise ValueError(f"oracle quantize failed with code {rc}")
    return out


def dequantize(t: int, data: np.ndarray, shape, order: int = ORDER_REF) -> np.ndarray:
    """dequant.rs:92 ``dequantize(data, dtype, shape)``; raises ValueError(code) like DequantError."""
    data = np.ascontiguousarray(data, dtype=np.uint8).reshape(-1)
    shp = np.asarray(list(shape), dtype=np.int32)
    n = 1
    for d in shape:
        n *= max(int(d), 0)
    # an absurd shape is rejected by the validation before dst is touched; do not try to allocate it
    out = np.empty(n if n < (1 << 40) else 0, dtype=np.float32)
    rc = lib().pmo_dequantize(t, _u8p(data), data.size, shp.ctypes.data_as(C.POINTER(C.c_int32)), shp.size,
                              _f32p(out), out.size, order)
    if rc != OK:
        raise ValueError(rc)
    return out


def make_qkx1_quants(nmax: int, ntry: int, x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    s, m = C.c_float(), C.c_float()
    lib().pmo_make_qkx1_quants(nmax, ntry, _f32p(x), x.size, C.byref(s), C.byref(m))
    return np.float32(s.value), np.float32(m.value)


def make_qx_quants(n: int, nmax: int, x: np.ndarray, rmse_type: int):
    x = np.ascontiguousarray(x, dtype=np.float32)
    ls = np.zeros(n, dtype=np.int8)
    s = lib().pmo_make_qx_quants(n, nmax, _f32p(x), rmse_type, ls.ctypes.data_as(C.POINTER(C.c_int8)))
    return np.float32(s), ls


def make_q3_quants(x: np.ndarray, nmax: int, do_rmse: bool):
    """quantize.rs:655 ``make_q3_quants``: (scale, quants offset by nmax)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    ls = np.zeros(x.size, dtype=np.int8)
    s = lib().pmo_make_q3_quants(_f32p(x), x.size, nmax, int(do_rmse), ls.ctypes.data_as(C.POINTER(C.c_int8)))
    return np.float32(s), ls


def get_scale_min_k4(j: int, q: np.ndarray):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    sc, m = C.c_uint8(), C.c_uint8()
    lib().pmo_get_scale_min_k4(j, _u8p(q), C.byref(sc), C.byref(m))
    return sc.value, m.value


def qmatvec(t: int, w: np.ndarray, n_rows: int, k: int, x: np.ndarray, order: int = ORDER_REF,
            acc: str = "f64", threads: int = 1) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.uint8).reshape(-1)
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert w.size == n_rows * tensor_size(t, k) and x.size == k
    y = np.empty(n_rows, dtype=np.float32)
    if threads > 1:
        rc = lib().pmo_qmatvec_mt(t, _u8p(w), n_rows, k, _f32p(x), _f32p(y), order, 1 if acc == "f64" else 0, threads)
    else:
        fn = lib().pmo_qmatvec_f64 if acc == "f64" else lib().pmo_qmatvec_f32
        rc = fn(t, _u8p(w), n_rows, k, _f32p(x), _f32p(y), order)
    if rc != OK:
        raise ValueError(rc)
    return y


def qmatmul(t: int, w: np.ndarray, n_rows: int, k: int, x: np.ndarray, order: int = ORDER_REF,
            threads: int = 1) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.uint8).reshape(-1)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    y = np.empty((x.shape[0], n_rows), dtype=np.float32)
    if threads > 1:
        rc = lib().pmo_qmatmul_f64_mt(t, _u8p(w), n_rows, k, _f32p(x), x.shape[0], _f32p(y), order, threads)
    else:
        rc = lib().pmo_qmatmul_f64(t, _u8p(w), n_rows, k, _f32p(x), x.shape[0], _f32p(y), order)
    if rc != OK:
        raise ValueError(rc)
    return y


def quantize_q8k(x: np.ndarray) -> np.ndarray:
    """k_quants.rs:815-871 ``quantize_q8k``: flat f32 -> 292-byte blocks."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.zeros(lib().pmo_q8k_size(x.size), dtype=np.uint8)
    if x.size:
        lib().pmo_quantize_q8k(_f32p(x), x.size, _u8p(out))
    return out


def vec_dot_q8k(t: int, xs: np.ndarray, ys: np.ndarray, n_blocks: int) -> float:
    """vec_dot.rs:617-810 (scalar): one row of Q4_K / Q6_K / Q5_K / Q3_K / Q2_K blocks against Q8_K blocks."""
    xs = np.ascontiguousarray(xs, dtype=np.uint8).reshape(-1)
    ys = np.ascontiguousarray(ys, dtype=np.uint8).reshape(-1)
    assert xs.size == n_blocks * tensor_size(t, 256) and ys.size == n_blocks * 292
    fn = {TYPE_Q4K: lib().pmo_vec_dot_q4k_q8k, TYPE_Q6K: lib().pmo_vec_dot_q6k_q8k, TYPE_Q5K: lib().pmo_vec_dot_q5k_q8k,
          TYPE_Q3K: lib().pmo_vec_dot_q3k_q8k, TYPE_Q2K: lib().pmo_vec_dot_q2k_q8k}[t]
    return float(fn(_u8p(xs), _u8p(ys), n_blocks))


def qmatvec_q8k(t: int, w: np.ndarray, n_rows: int, k: int, xq: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.uint8).reshape(-1)
    xq = np.ascontiguousarray(xq, dtype=np.uint8).reshape(-1)
    assert w.size == n_rows * tensor_size(t, k) and xq.size == (k // 256) * 292
    y = np.empty(n_rows, dtype=np.float32)
    rc = lib().pmo_qmatvec_q8k(t, _u8p(w), n_rows, k, _u8p(xq), _f32p(y))
    if rc != OK:
        raise ValueError(rc)
    return y


def kl_divergence(original: np.ndarray, dequantized: np.ndarray) -> float:
    """dynamic.rs:140-180 ``compute_kl_divergence``."""
    a = np.ascontiguousarray(original, dtype=np.float32).reshape(-1)
    b = np.ascontiguousarray(dequantized, dtype=np.float32).reshape(-1)
    assert a.size == b.size
    return float(lib().pmo_kl_divergence(_f32p(a), _f32p(b), a.size))


def is_critical_layer(name: str) -> bool:
    """dynamic.rs:254-268"""
    return any(s in name for s in ("lm_head", "output", "token_embd", "embed_tokens", "wte", "final_norm", "ln_f"))


DEFAULT_CANDIDATES = (15, 14, 13, 12, 11, 10)  # Q8K, Q6K, Q5K, Q4K, Q3K, Q2K (dynamic.rs:104-121)


def calibrate_tensor(name: str, data: np.ndarray, shape, candidates=DEFAULT_CANDIDATES, kl_threshold: float = 0.01,
                     fallback_type: int = 15, sample_size: int = 0, order: int = ORDER_REF):
    """dynamic.rs:420-502 ``calibrate_tensor``: (quant_type, kl_score, all_scores).  A candidate whose quantizer or
    dequantizer fails is skipped (:456-464), which here is every type the oracle does not restate."""
    data = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
    if is_critical_layer(name):
        return fallback_type, 0.0, [(fallback_type, 0.0)]
    sample = data[:sample_size] if 0 < sample_size < data.size else data
    scores = []
    for t in candidates:
        try:
            deq = dequantize(t, quantize(t, data), shape, order)
        except ValueError:
            continue
        n = min(sample.size, deq.size)
        scores.append((t, kl_divergence(sample[:n], deq[:n])))
    if not scores:
        return fallback_type, float(np.finfo(np.float64).max), [(fallback_type, float(np.finfo(np.float64).max))]
    best_type, best_score = scores[0]
    for t, sc in reversed(scores):
        if sc <= kl_threshold:
            best_type, best_score = t, sc
            break
    return best_type, best_score, scores


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """half::bf16::from_f32 (RNE) on an array, vectorised; returns uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), rounded)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
