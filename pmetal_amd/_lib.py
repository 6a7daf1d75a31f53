"""ctypes loader for ``libpmetal_hip.so``; fails loudly when the library is missing or unusable."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpmetal_hip.so")

# every symbol include/pmetal_hip.h declares: (name, restype, argtypes)
_vp, _sz, _i32, _u32, _i64, _u64, _f32 = (C.c_void_p, C.c_size_t, C.c_int32, C.c_uint32, C.c_int64, C.c_uint64,
                                          C.c_float)


class LinearDesc(C.Structure):
    """``pmetal_hip_linear_desc``"""
    _fields_ = [("ggml_type", _u32), ("x_dtype", _u32), ("order", _u32), ("reserved", _u32), ("n", _i64),
                ("k", _i64), ("w_dev", _vp), ("x_dev", _vp), ("y_dev", _vp)]


class GemmDesc(C.Structure):
    """``pmetal_hip_gemm_desc``"""
    _fields_ = [("ggml_type", _u32), ("y_dtype", _u32), ("order", _u32), ("reserved", _u32), ("n", _i64), ("w_dev", _vp),
                ("y_dev", _vp)]


class QuantizeDesc(C.Structure):
    """``pmetal_hip_quantize_desc``"""
    _fields_ = [("ggml_type", _u32), ("reserved", _u32), ("src_dev", _vp), ("n", _sz), ("dst_dev", _vp), ("dst_len", _sz)]


SYMBOLS = [
    ("pmetal_hip_device_count", _i32, []),
    ("pmetal_hip_init", _i32, [_i32]),
    ("pmetal_hip_last_error_code", _i32, []),
    ("pmetal_hip_last_error_message", C.c_char_p, []),
    ("pmetal_hip_clear_error", None, []),
    ("pmetal_hip_type_size", _sz, [_u32]),
    ("pmetal_hip_block_size", _sz, [_u32]),
    ("pmetal_hip_tensor_size", _sz, [_u32, _sz]),
    ("pmetal_hip_expected_byte_size", _i32, [_u32, C.POINTER(_i32), _sz, C.POINTER(_sz), C.POINTER(_sz)]),
    ("pmetal_hip_is_supported", _i32, [_u32]),
    ("pmetal_hip_alloc", _vp, [_sz]),
    ("pmetal_hip_free", _i32, [_vp]),
    ("pmetal_hip_h2d", _i32, [_vp, _vp, _sz]),
    ("pmetal_hip_d2h", _i32, [_vp, _vp, _sz]),
    ("pmetal_hip_memset", _i32, [_vp, C.c_int, _sz, _vp]),
    ("pmetal_hip_sync", _i32, [_vp]),
    ("pmetal_hip_stream_create", _vp, []),
    ("pmetal_hip_stream_destroy", _i32, [_vp]),
    ("pmetal_hip_record_begin", _i32, [_vp]),
    ("pmetal_hip_record_end", _vp, [_vp]),
    ("pmetal_hip_replay", _i32, [_vp, _vp]),
    ("pmetal_hip_recording_destroy", _i32, [_vp]),
    ("pmetal_hip_event_create", _vp, []),
    ("pmetal_hip_event_record", _i32, [_vp, _vp]),
    ("pmetal_hip_event_elapsed_ms", _i32, [_vp, _vp, C.POINTER(_f32)]),
    ("pmetal_hip_event_destroy", _i32, [_vp]),
    ("pmetal_hip_quantize", _i32, [_u32, _vp, _sz, _vp, _sz]),
    ("pmetal_hip_quantize_dev", _i32, [_u32, _vp, _sz, _vp, _sz, _vp]),
    ("pmetal_hip_quantize_batch_dev", _i32, [C.POINTER(QuantizeDesc), _sz, _vp]),
    ("pmetal_hip_dequantize", _i32, [_u32, _vp, _sz, C.POINTER(_i32), _sz, _vp, _sz, _u32]),
    ("pmetal_hip_dequantize_dev", _i32, [_u32, _vp, _sz, _vp, _sz, _u32, _vp]),
    ("pmetal_hip_qgemv", _i32, [_u32, _vp, _i64, _i64, _vp, _u32, _vp, _u32, _vp]),
    ("pmetal_hip_qgemm", _i32, [_u32, _vp, _i64, _i64, _vp, _u32, _i64, _vp, _u32, _u32, _vp]),
    ("pmetal_hip_qgemm_noalloc", _i32, [_u32, _vp, _i64, _i64, _vp, _u32, _i64, _vp, _u32, _u32, _vp]),
    ("pmetal_hip_qgemm_batch", _i32, [C.POINTER(GemmDesc), _sz, _i64, _vp, _u32, _i64, _vp]),
    ("pmetal_hip_reblock_size", _sz, [_u32, _i64, _i64]),
    ("pmetal_hip_reblock_dev", _i32, [_u32, _vp, _i64, _i64, _u32, _vp, _sz, _vp]),
    ("pmetal_hip_qgemm_reblocked", _i32, [_u32, _vp, _sz, _i64, _i64, _vp, _u32, _i64, _vp, _u32, _vp]),
    ("pmetal_hip_qlinear", _i32, [_u32, _vp, _i64, _i64, _vp, _u32, _i64, _vp, _u32, _u32, _vp]),
    ("pmetal_hip_qgemv_batch", _i32, [C.POINTER(LinearDesc), _sz, _vp]),
    ("pmetal_hip_q8k_size", _sz, [_sz]),
    ("pmetal_hip_quantize_q8k_dev", _i32, [_vp, _sz, _vp, _sz, _vp]),
    ("pmetal_hip_qgemv_q8k", _i32, [_u32, _vp, _i64, _i64, _vp, _vp, _vp]),
    ("pmetal_hip_kl_divergence_dev", _i32, [_vp, _vp, _sz, C.POINTER(C.c_double), _vp]),
    ("pmetal_hip_kl_divergence_quantized_dev", _i32, [_u32, _vp, _sz, _vp, _sz, _u32, C.POINTER(C.c_double), _vp]),
    ("pmetal_hip_use_more_bits", _i32, [_sz, _sz]),
    ("pmetal_hip_is_quantizable_gguf_tensor", _i32, [C.c_char_p, _sz]),
    ("pmetal_hip_q4km_tensor_type", _u32, [C.c_char_p, _sz, _sz]),
    ("pmetal_hip_fill_normal_f32", _i32, [_vp, _sz, _u64, _f32, _f32, _f32, _vp]),
    ("pmetal_hip_f32_to_bf16_dev", _i32, [_vp, _vp, _sz, _vp]),
    ("pmetal_hip_mfma_probe_f16", _i32, [_i32, _i32, _i32, _vp, _vp]),
    ("pmetal_hip_read_probe", _i32, [_vp, _sz, _vp, _vp]),
]

_lib = None


def load() -> C.CDLL:
    """Load the HIP library.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m pmetal_amd.build` (needs hipcc, targets gfx950)")
        lib = C.CDLL(LIB_PATH)
        for name, restype, argtypes in SYMBOLS:
            fn = getattr(lib, name)  # AttributeError if the library does not export it
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib
