"""MI355X-native implementation of PMetal's GGUF block-quantized weight path (Q8_0 / Q4_K / Q6_K).

The product is ``libpmetal_hip.so`` (hand-written HIP for gfx950 behind a C ABI, ``include/pmetal_hip.h``);
this package is the thin host-side mirror of the reference's Rust API used by tests and benchmarks.
"""
from .gguf import (DTYPE_BF16, DTYPE_F32, ORDER_GGML, ORDER_REF, DequantError, DeviceBuffer, GgmlType, GgufLinear,
                   NoDeviceError, PMetalHipError, QuantizationError, check, dequantize, device_count, init,
                   q4km_tensor_type, quantize, use_more_bits)

__all__ = ["DTYPE_BF16", "DTYPE_F32", "ORDER_GGML", "ORDER_REF", "DequantError", "DeviceBuffer", "GgmlType",
           "GgufLinear", "NoDeviceError", "PMetalHipError", "QuantizationError", "check", "dequantize",
           "device_count", "init", "q4km_tensor_type", "quantize", "use_more_bits"]
