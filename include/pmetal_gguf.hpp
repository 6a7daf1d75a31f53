// pmetal_gguf.hpp -- C++ host-side mirror of the reference's quantize / dequantize / quantized-linear
// API over the C ABI of libpmetal_hip.so (include/pmetal_hip.h).  Header-only; link with -lpmetal_hip.
//
// The reference is Rust; this mirror keeps its names, argument meaning and error behaviour so that a
// caller (or a test) reads like the reference's own:
//   pmetal_gguf::quantize(data, dtype)            crates/pmetal-gguf/src/quantize.rs:17
//   pmetal_gguf::dequantize(data, dtype, shape)   crates/pmetal-gguf/src/dequant.rs:92
//   pmetal_gguf::DequantError{kind}               crates/pmetal-gguf/src/dequant.rs:37-70
//   pmetal_gguf::QuantizationError                PMetalError::Quantization, crates/pmetal-core/src/error.rs:50-52
//   pmetal_gguf::GgmlType::{type_size, block_size, tensor_size}   crates/pmetal-gguf/src/types.rs:102-187
//   pmetal_gguf::GgufLinear::matmul_from(x, m)    LayerWeight::matmul_from,
//                                                 crates/pmetal-bridge/src/qwen3_native/weights.rs:66-84
// A Rust `Result::Err` becomes a thrown exception carrying the library's message.  Everything computes on
// the GPU; there is no CPU fallback (a missing device throws NoDeviceError).
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "pmetal_hip.h"

namespace pmetal_gguf {

enum class GgmlType : uint32_t { F32 = 0, F16 = 1, Q8_0 = 8, Q4K = 12, Q5K = 13, Q6K = 14 };

inline size_t type_size(GgmlType t) { return pmetal_hip_type_size((uint32_t)t); }
inline size_t block_size(GgmlType t) { return pmetal_hip_block_size((uint32_t)t); }
inline size_t tensor_size(GgmlType t, size_t n_elements) { return pmetal_hip_tensor_size((uint32_t)t, n_elements); }

struct Error : std::runtime_error {
    int32_t code;
    Error(int32_t c, const std::string &msg) : std::runtime_error(msg), code(c) {}
};
struct QuantizationError : Error {
    using Error::Error;
};
struct NoDeviceError : Error {
    using Error::Error;
};
struct DequantError : Error {
    enum class Kind { UnsupportedType, InvalidSize, ShapeMismatch, InvalidShape, ShapeTooLarge, Other };
    Kind kind;
    DequantError(int32_t c, const std::string &msg) : Error(c, msg), kind(kind_of(c)) {}
    static Kind kind_of(int32_t c) {
        switch (c) {
        case PMETAL_HIP_ERR_UNSUPPORTED_TYPE: return Kind::UnsupportedType;
        case PMETAL_HIP_ERR_INVALID_SIZE: return Kind::InvalidSize;
        case PMETAL_HIP_ERR_INVALID_SHAPE: return Kind::InvalidShape;
        case PMETAL_HIP_ERR_SHAPE_TOO_LARGE: return Kind::ShapeTooLarge;
        default: return Kind::Other;
        }
    }
};

namespace detail {
inline void check(int32_t rc, bool quantizing = false) {
    if (rc == PMETAL_HIP_OK) return;
    const std::string msg = pmetal_hip_last_error_message();
    if (rc == PMETAL_HIP_ERR_NO_DEVICE) throw NoDeviceError(rc, msg);
    if (quantizing && (rc == PMETAL_HIP_ERR_UNSUPPORTED_TYPE || rc == PMETAL_HIP_ERR_INVALID_SIZE))
        throw QuantizationError(rc, msg);
    if (rc == PMETAL_HIP_ERR_UNSUPPORTED_TYPE || rc == PMETAL_HIP_ERR_INVALID_SIZE ||
        rc == PMETAL_HIP_ERR_INVALID_SHAPE || rc == PMETAL_HIP_ERR_SHAPE_TOO_LARGE)
        throw DequantError(rc, msg);
    throw Error(rc, msg);
}
}  // namespace detail

// quantize(data: &[f32], dtype) -> Result<Vec<u8>>; bytes bit-identical to the reference CPU quantizer.
inline std::vector<uint8_t> quantize(const float *data, size_t n, GgmlType dtype) {
    std::vector<uint8_t> out(tensor_size(dtype, n));
    detail::check(pmetal_hip_quantize((uint32_t)dtype, data, n, out.data(), out.size()), true);
    return out;
}
inline std::vector<uint8_t> quantize(const std::vector<float> &data, GgmlType dtype) {
    return quantize(data.data(), data.size(), dtype);
}

// dequantize(data: &[u8], dtype, shape: &[i32]) -> Result<Vec<f32>, DequantError>; row-major values.
// `order` selects the Q4_K element order (PMETAL_HIP_ORDER_REF reproduces the reference bit for bit).
inline std::vector<float> dequantize(const uint8_t *data, size_t len, GgmlType dtype, const std::vector<int32_t> &shape,
                                     uint32_t order = PMETAL_HIP_ORDER_REF) {
    size_t bytes = 0, elems = 0;
    detail::check(pmetal_hip_expected_byte_size((uint32_t)dtype, shape.data(), shape.size(), &bytes, &elems));
    if (len != bytes)  // let the library word the InvalidSize error
        detail::check(pmetal_hip_dequantize((uint32_t)dtype, data, len, shape.data(), shape.size(), nullptr, 0, order));
    std::vector<float> out(elems);
    detail::check(pmetal_hip_dequantize((uint32_t)dtype, data, len, shape.data(), shape.size(), out.data(), out.size(),
                                        order));
    return out;
}
inline std::vector<float> dequantize(const std::vector<uint8_t> &data, GgmlType dtype, const std::vector<int32_t> &shape,
                                     uint32_t order = PMETAL_HIP_ORDER_REF) {
    return dequantize(data.data(), data.size(), dtype, shape, order);
}

// A device allocation owned by the caller.
class DeviceBuffer {
   public:
    explicit DeviceBuffer(size_t bytes) : bytes_(bytes), ptr_(pmetal_hip_alloc(bytes)) {
        if (!ptr_) detail::check(pmetal_hip_last_error_code() ? pmetal_hip_last_error_code() : PMETAL_HIP_ERR_HIP_RUNTIME);
    }
    DeviceBuffer(const void *host, size_t bytes) : DeviceBuffer(bytes) { detail::check(pmetal_hip_h2d(ptr_, host, bytes)); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : bytes_(o.bytes_), ptr_(o.ptr_) { o.ptr_ = nullptr; }
    ~DeviceBuffer() {
        if (ptr_) pmetal_hip_free(ptr_);
    }
    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }
    void to_host(void *dst, size_t bytes) const { detail::check(pmetal_hip_d2h(dst, ptr_, bytes)); }

   private:
    size_t bytes_;
    void *ptr_;
};

// A GGUF-quantized weight [n, k] resident on the device; the counterpart of LayerWeight for GGUF types.
class GgufLinear {
   public:
    GgufLinear(GgmlType dtype, int64_t n, int64_t k, const std::vector<uint8_t> &packed,
               uint32_t order = PMETAL_HIP_ORDER_REF)
        : dtype_(dtype), n_(n), k_(k), order_(order), w_(check_size(dtype, n, k, packed), packed.size()) {}

    // x: [m, k] activations on the device (bf16 unless x_dtype says f32); returns [m, n] f32 on the device.
    // m == 1 runs the fused GEMV, m > 1 the fused GEMM (LayerWeight::matmul_from makes the same split).
    DeviceBuffer matmul_from(const DeviceBuffer &x, int64_t m = 1, uint32_t x_dtype = PMETAL_HIP_DTYPE_BF16,
                             void *stream = nullptr) const {
        DeviceBuffer y((size_t)m * (size_t)n_ * sizeof(float));
        detail::check(pmetal_hip_qlinear((uint32_t)dtype_, (const uint8_t *)w_.ptr(), n_, k_, x.ptr(), x_dtype, m, y.ptr(),
                                         PMETAL_HIP_DTYPE_F32, order_, stream));
        return y;
    }
    int64_t n() const { return n_; }
    int64_t k() const { return k_; }

   private:
    static const void *check_size(GgmlType dtype, int64_t n, int64_t k, const std::vector<uint8_t> &packed) {
        const size_t expected = tensor_size(dtype, (size_t)n * (size_t)k);
        if (packed.size() != expected)
            throw DequantError(PMETAL_HIP_ERR_INVALID_SIZE, "Invalid data size: expected " + std::to_string(expected) +
                                                                " bytes, got " + std::to_string(packed.size()));
        return packed.data();
    }
    GgmlType dtype_;
    int64_t n_, k_;
    uint32_t order_;
    DeviceBuffer w_;
};

// Q4_K_M recipe: crates/pmetal/src/commands/quantize.rs:988-1137
inline bool use_more_bits(size_t layer, size_t n_layers) { return pmetal_hip_use_more_bits(layer, n_layers) != 0; }
inline GgmlType q4km_tensor_type(const std::string &gguf_name, size_t ndim, size_t n_layers) {
    return (GgmlType)pmetal_hip_q4km_tensor_type(gguf_name.c_str(), ndim, n_layers);
}

}  // namespace pmetal_gguf
