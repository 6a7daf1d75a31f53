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
//   pmetal_gguf::quantize_model_q4_k_m(...)       the quantize-and-write loop of run_quantization,
//                                                 crates/pmetal/src/commands/quantize.rs:1339-1433
//   pmetal_gguf::hf_to_gguf_name                  crates/pmetal-models/src/weight_format.rs:389-435
//   pmetal_gguf::gguf_to_hf_name, load_gguf       WeightLoader::gguf_to_hf_name / load_gguf,
//                                                 crates/pmetal-models/src/weight_format.rs:332-386, :258-313
// A Rust `Result::Err` becomes a thrown exception carrying the library's message.  Everything computes on
// the GPU; there is no CPU fallback (a missing device throws NoDeviceError).
#pragma once

#include <cstdint>
#include <stdexcept>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "pmetal_gguf_file.hpp"
#include "pmetal_hip.h"

namespace pmetal_gguf {

// GgmlType (all ids of crates/pmetal-gguf/src/types.rs:16-97) comes from pmetal_gguf_file.hpp; the sizes below are the
// library's own answers for the types it computes with.
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
    // prepare_gemm: accepted and ignored.  Every type has matrix kernels that read its blocks as they are, so nothing is
    // laid out again at load time (the reference does that for its matmul, weights.rs:29-45).
    GgufLinear(GgmlType dtype, int64_t n, int64_t k, const std::vector<uint8_t> &packed,
               uint32_t order = PMETAL_HIP_ORDER_REF, bool prepare_gemm = false)
        : dtype_(dtype), n_(n), k_(k), order_(order), w_(check_size(dtype, n, k, packed), packed.size()) {
        (void)prepare_gemm;
    }

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

// The tensor loop of run_quantization (crates/pmetal/src/commands/quantize.rs:1378-1428) over tensors that are already on
// the device: one DeviceBuffer of blocks per (dtype, src, n), the bytes of one quantize() per tensor, through one
// pmetal_hip_quantize_batch_dev call (the independent tensors spread over two streams inside the library).
struct DeviceTensorF32 {
    GgmlType dtype;
    const float *src_dev;
    size_t n;
};
inline std::vector<DeviceBuffer> quantize_tensors_dev(const std::vector<DeviceTensorF32> &tensors, void *stream = nullptr) {
    std::vector<DeviceBuffer> outs;
    std::vector<pmetal_hip_quantize_desc> descs;
    outs.reserve(tensors.size());
    for (const DeviceTensorF32 &t : tensors) {
        const size_t bytes = pmetal_hip_tensor_size((uint32_t)t.dtype, t.n);
        outs.emplace_back(bytes ? bytes : 16);
        descs.push_back(pmetal_hip_quantize_desc{(uint32_t)t.dtype, 0u, t.src_dev, t.n, (uint8_t *)outs.back().ptr(), bytes});
    }
    detail::check(pmetal_hip_quantize_batch_dev(descs.data(), descs.size(), stream), true);
    return outs;
}

// quantize_q8k (crates/pmetal-gguf/src/k_quants.rs:815-871) of n f32 values on the device: 292-byte BlockQ8K blocks.
inline DeviceBuffer quantize_q8k(const DeviceBuffer &x, size_t n, void *stream = nullptr) {
    DeviceBuffer out(pmetal_hip_q8k_size(n) ? pmetal_hip_q8k_size(n) : 16);
    detail::check(pmetal_hip_quantize_q8k_dev((const float *)x.ptr(), n, (uint8_t *)out.ptr(), pmetal_hip_q8k_size(n), stream), true);
    return out;
}
// y[r] = vec_dot_q4k_q8k / vec_dot_q6k_q8k (row r of w, xq), crates/pmetal-gguf/src/vec_dot.rs:829-851, as the scalar
// definitions (:617-692) compute them, bit for bit.  w: [n, k] Q4K or Q6K blocks, xq: k / 256 Q8_K blocks, all on the device.
inline DeviceBuffer qgemv_q8k(GgmlType dtype, const DeviceBuffer &w, int64_t n, int64_t k, const DeviceBuffer &xq,
                              void *stream = nullptr) {
    DeviceBuffer y((size_t)(n > 0 ? n : 1) * sizeof(float));
    detail::check(pmetal_hip_qgemv_q8k((uint32_t)dtype, (const uint8_t *)w.ptr(), n, k, (const uint8_t *)xq.ptr(), (float *)y.ptr(), stream));
    return y;
}

// DynamicQuantizer::is_critical_layer (crates/pmetal-gguf/src/dynamic.rs:254-268)
inline bool is_critical_layer(const std::string &name) {
    for (const char *s : {"lm_head", "output", "token_embd", "embed_tokens", "wte", "final_norm", "ln_f"})
        if (name.find(s) != std::string::npos) return true;
    return false;
}

// KlCalibrationConfig and CalibratedTensor (crates/pmetal-gguf/src/dynamic.rs:80-123, :186-196)
struct KlCalibrationConfig {
    std::vector<GgmlType> candidates{GgmlType::Q8K, GgmlType::Q6K, GgmlType::Q5K, GgmlType::Q4K, GgmlType::Q3K, GgmlType::Q2K};
    double kl_threshold = 0.01;
    GgmlType fallback_type = GgmlType::Q8K;
    size_t sample_size = 0;
    uint32_t order = PMETAL_HIP_ORDER_REF;  // element order of the dequantizer in the round trip (the reference: REF)
};
struct CalibratedTensor {
    GgmlType quant_type;
    double kl_score;
    std::vector<std::pair<GgmlType, double>> all_scores;
};

// DynamicQuantizer::calibrate_tensor (crates/pmetal-gguf/src/dynamic.rs:420-502) with the round trips on the GPU: the
// tensor is uploaded once; every candidate is quantized and scored on the device (the k-quants without storing the dequantized tensor).  A candidate without
// kernels here, or a shape whose byte size is not the quantized tensor's, is skipped, as the reference
// skips a candidate whose quantize or dequantize fails.
inline CalibratedTensor calibrate_tensor(const std::string &name, const float *data, size_t n, const std::vector<int32_t> &shape,
                                         const KlCalibrationConfig &cfg = KlCalibrationConfig()) {
    const double kMax = 1.7976931348623157e308;  // f64::MAX
    if (is_critical_layer(name)) return {cfg.fallback_type, 0.0, {{cfg.fallback_type, 0.0}}};
    size_t n_shape = 1;
    for (int32_t d : shape) n_shape *= (size_t)(d > 0 ? d : 0);
    const size_t sample = cfg.sample_size > 0 && n > cfg.sample_size ? cfg.sample_size : n;
    std::vector<std::pair<GgmlType, double>> scores;
    DeviceBuffer dx((n ? n : 4) * sizeof(float));
    std::unique_ptr<DeviceBuffer> ddeq;  // only for a type that has no fused comparison
    if (n) detail::check(pmetal_hip_h2d(dx.ptr(), data, n * sizeof(float)));
    for (GgmlType t : cfg.candidates) {
        const size_t nbytes = pmetal_hip_tensor_size((uint32_t)t, n);
        if (!pmetal_hip_is_supported((uint32_t)t) || n_shape > n || pmetal_hip_tensor_size((uint32_t)t, n_shape) != nbytes) continue;
        if (n_shape == 0) {
            scores.emplace_back(t, 0.0);
            continue;
        }
        DeviceBuffer dq(nbytes ? nbytes : 16);
        detail::check(pmetal_hip_quantize_dev((uint32_t)t, (const float *)dx.ptr(), n, (uint8_t *)dq.ptr(), nbytes, nullptr), true);
        const size_t cmp_len = sample < n_shape ? sample : n_shape;
        double score = 0.0;
        if (pmetal_hip_block_size((uint32_t)t) == 256) {  // k-quants: decoded and compared in one pass, nothing stored
            detail::check(pmetal_hip_kl_divergence_quantized_dev((uint32_t)t, (const uint8_t *)dq.ptr(), nbytes, (const float *)dx.ptr(), cmp_len,
                                                                 cfg.order, &score, nullptr));
        } else {
            if (!ddeq) ddeq.reset(new DeviceBuffer(n * sizeof(float)));
            detail::check(pmetal_hip_dequantize_dev((uint32_t)t, (const uint8_t *)dq.ptr(), nbytes, (float *)ddeq->ptr(), n_shape, cfg.order, nullptr));
            detail::check(pmetal_hip_kl_divergence_dev((const float *)dx.ptr(), (const float *)ddeq->ptr(), cmp_len, &score, nullptr));
        }
        scores.emplace_back(t, score);
    }
    if (scores.empty()) return {cfg.fallback_type, kMax, {{cfg.fallback_type, kMax}}};
    CalibratedTensor out{scores[0].first, scores[0].second, scores};
    for (auto it = scores.rbegin(); it != scores.rend(); ++it)
        if (it->second <= cfg.kl_threshold) {
            out.quant_type = it->first, out.kl_score = it->second;
            break;
        }
    return out;
}

// Q4_K_M recipe: crates/pmetal/src/commands/quantize.rs:988-1137
inline bool use_more_bits(size_t layer, size_t n_layers) { return pmetal_hip_use_more_bits(layer, n_layers) != 0; }
inline GgmlType q4km_tensor_type(const std::string &gguf_name, size_t ndim, size_t n_layers) {
    return (GgmlType)pmetal_hip_q4km_tensor_type(gguf_name.c_str(), ndim, n_layers);
}


// quantize(data, dtype) for every type the Q4_K_M recipe yields: F32 and F16 are conversions on the host
// (crates/pmetal-gguf/src/quantize.rs:19-30), the 32-element formats and the k-quants run on the GPU, anything else is the
// reference's "not yet implemented" error.
inline std::vector<uint8_t> quantize_any(const float *data, size_t n, GgmlType dtype) {
    if (dtype == GgmlType::F32) {
        std::vector<uint8_t> out(n * 4);
        if (n) std::memcpy(out.data(), data, n * 4);
        return out;
    }
    if (dtype == GgmlType::F16) {
        std::vector<uint8_t> out(n * 2);
        for (size_t i = 0; i < n; i++) {
            const uint16_t h = f32_to_f16_bits(data[i]);
            std::memcpy(out.data() + 2 * i, &h, 2);
        }
        return out;
    }
    return quantize(data, n, dtype);
}

// WeightLoader::hf_to_gguf_name (crates/pmetal-models/src/weight_format.rs:389-435)
inline std::string hf_to_gguf_name(const std::string &hf_name) {
    if (hf_name == "model.embed_tokens.weight") return "token_embd.weight";
    if (hf_name == "model.norm.weight") return "output_norm.weight";
    if (hf_name == "lm_head.weight") return "output.weight";
    static const std::string prefix = "model.layers.";
    if (hf_name.compare(0, prefix.size(), prefix) != 0) return hf_name;
    const std::string rest = hf_name.substr(prefix.size());
    const size_t dot = rest.find('.');
    if (dot == std::string::npos) return hf_name;
    const std::string layer = rest.substr(0, dot), suffix = rest.substr(dot + 1);
    {  // usize::from_str: decimal digits behind an optional '+', value below 2^64
        const size_t first = !layer.empty() && layer[0] == '+' ? 1 : 0;
        if (layer.size() == first) return hf_name;
        unsigned long long v = 0;
        for (size_t i = first; i < layer.size(); i++) {
            if (layer[i] < '0' || layer[i] > '9') return hf_name;
            const unsigned d = (unsigned)(layer[i] - '0');
            if (v > (UINT64_MAX - d) / 10) return hf_name;
            v = v * 10 + d;
        }
    }
    static const std::pair<const char *, const char *> table[] = {
        {"input_layernorm.weight", "attn_norm.weight"},
        {"self_attn.q_proj.weight", "attn_q.weight"},
        {"self_attn.k_proj.weight", "attn_k.weight"},
        {"self_attn.v_proj.weight", "attn_v.weight"},
        {"self_attn.o_proj.weight", "attn_output.weight"},
        {"post_attention_layernorm.weight", "ffn_norm.weight"},
        {"mlp.gate.weight", "ffn_gate_inp.weight"},
        {"mlp.router.weight", "ffn_gate_inp.weight"},
        {"mlp.gate_proj.weight", "ffn_gate.weight"},
        {"mlp.up_proj.weight", "ffn_up.weight"},
        {"mlp.down_proj.weight", "ffn_down.weight"},
        {"mlp.experts.gate_proj.weight", "ffn_gate_exps.weight"},
        {"mlp.experts.up_proj.weight", "ffn_up_exps.weight"},
        {"mlp.experts.down_proj.weight", "ffn_down_exps.weight"},
        {"mlp.shared_expert.gate_proj.weight", "ffn_gate_shexp.weight"},
        {"mlp.shared_expert.up_proj.weight", "ffn_up_shexp.weight"},
        {"mlp.shared_expert.down_proj.weight", "ffn_down_shexp.weight"},
        {"mlp.shared_experts.gate_proj.weight", "ffn_gate_shexp.weight"},
        {"mlp.shared_experts.up_proj.weight", "ffn_up_shexp.weight"},
        {"mlp.shared_experts.down_proj.weight", "ffn_down_shexp.weight"},
        {"mlp.shared_expert_gate.weight", "ffn_gate_inp_shexp.weight"},
        {"self_attn.q_norm.weight", "attn_q_norm.weight"},
        {"self_attn.k_norm.weight", "attn_k_norm.weight"},
    };
    std::string mapped = suffix;
    for (const auto &row : table)
        if (suffix == row.first) mapped = row.second;
    return "blk." + layer + "." + mapped;
}

// WeightLoader::gguf_to_hf_name (crates/pmetal-models/src/weight_format.rs:332-386): the three top-level tensors, then
// blk.N.<tensor> -> model.layers.N.<tensor>; N is taken as written (it is not parsed), unknown names pass through.
inline std::string gguf_to_hf_name(const std::string &gguf_name) {
    if (gguf_name == "token_embd.weight") return "model.embed_tokens.weight";
    if (gguf_name == "output_norm.weight") return "model.norm.weight";
    if (gguf_name == "output.weight") return "lm_head.weight";
    if (gguf_name.compare(0, 4, "blk.") != 0) return gguf_name;
    // splitn(3, '.'): "blk", the block number, the rest; fewer than three parts pass through
    const size_t d1 = gguf_name.find('.', 4);
    if (d1 == std::string::npos) return gguf_name;
    const std::string block = gguf_name.substr(4, d1 - 4), rest = gguf_name.substr(d1 + 1);
    static const std::pair<const char *, const char *> table[] = {
        {"attn_norm.weight", "input_layernorm.weight"},
        {"attn_q.weight", "self_attn.q_proj.weight"},
        {"attn_k.weight", "self_attn.k_proj.weight"},
        {"attn_v.weight", "self_attn.v_proj.weight"},
        {"attn_output.weight", "self_attn.o_proj.weight"},
        {"ffn_norm.weight", "post_attention_layernorm.weight"},
        {"ffn_gate.weight", "mlp.gate_proj.weight"},
        {"ffn_up.weight", "mlp.up_proj.weight"},
        {"ffn_down.weight", "mlp.down_proj.weight"},
        {"ffn_gate_inp.weight", "mlp.gate.weight"},
        {"ffn_gate_exps.weight", "mlp.experts.gate_proj.weight"},
        {"ffn_up_exps.weight", "mlp.experts.up_proj.weight"},
        {"ffn_down_exps.weight", "mlp.experts.down_proj.weight"},
        {"ffn_gate_shexp.weight", "mlp.shared_expert.gate_proj.weight"},
        {"ffn_up_shexp.weight", "mlp.shared_expert.up_proj.weight"},
        {"ffn_down_shexp.weight", "mlp.shared_expert.down_proj.weight"},
        {"ffn_gate_inp_shexp.weight", "mlp.shared_expert_gate.weight"},
        {"attn_q_norm.weight", "self_attn.q_norm.weight"},
        {"attn_k_norm.weight", "self_attn.k_norm.weight"},
    };
    std::string mapped = rest;
    for (const auto &row : table)
        if (rest == row.first) mapped = row.second;
    return "model.layers." + block + "." + mapped;
}

// dequantize(data, dtype, shape) for every type this build decodes: F32 / F16 / BF16 are conversions on the host
// (crates/pmetal-gguf/src/dequant.rs:219-258, sizes validated as there), the 32-element formats and the k-quants run on the GPU.
inline bool load_supported(GgmlType dtype) {
    return dtype == GgmlType::F32 || dtype == GgmlType::F16 || dtype == GgmlType::Bf16 || pmetal_hip_is_supported((uint32_t)dtype) != 0;
}
inline std::vector<float> dequantize_any(const uint8_t *data, size_t len, GgmlType dtype, const std::vector<int32_t> &shape) {
    if (dtype != GgmlType::F32 && dtype != GgmlType::F16 && dtype != GgmlType::Bf16) return dequantize(data, len, dtype, shape);
    size_t n = 1;
    for (int32_t d : shape) {
        if (d < 0) throw DequantError(PMETAL_HIP_ERR_INVALID_SHAPE, "dimensions must be non-negative");
        if (d != 0 && n > SIZE_MAX / (size_t)d) throw DequantError(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "shape is too large");
        n *= (size_t)d;
    }
    const size_t width = dtype == GgmlType::F32 ? 4 : 2;
    if (n > SIZE_MAX / width) throw DequantError(PMETAL_HIP_ERR_SHAPE_TOO_LARGE, "shape is too large");
    if (len != n * width)
        throw DequantError(PMETAL_HIP_ERR_INVALID_SIZE,
                           "Invalid data size: expected " + std::to_string(n * width) + " bytes, got " + std::to_string(len));
    std::vector<float> out(n);
    for (size_t i = 0; i < n; i++) {
        if (dtype == GgmlType::F32) {
            std::memcpy(&out[i], data + 4 * i, 4);
        } else {
            uint16_t h;
            std::memcpy(&h, data + 2 * i, 2);
            if (dtype == GgmlType::F16) {
                out[i] = f16_bits_to_f32(h);
            } else {
                const uint32_t u = (uint32_t)h << 16;
                std::memcpy(&out[i], &u, 4);
            }
        }
    }
    return out;
}

// One tensor as WeightLoader::load_gguf returns it: f32 values, row-major, with the shape the file gives.
struct LoadedTensor {
    std::vector<int32_t> shape;
    std::vector<float> data;
};

// WeightLoader::load_gguf (crates/pmetal-models/src/weight_format.rs:258-313): every tensor of the file whose type can be
// decoded, dequantized to f32 under its Hugging Face name; tensors of other types are skipped (the reference logs a
// warning), a dimension beyond i32 is an error (:142-153).  Here "can be decoded" means load_supported(): the plain
// types and the block types with kernels in this library; `skipped`, when given, receives the names left out.
inline std::map<std::string, LoadedTensor> load_gguf(const std::string &path, std::vector<std::string> *skipped = nullptr) {
    const GgufContent content = GgufContent::from_file(path);
    std::map<std::string, LoadedTensor> weights;
    for (const std::string &name : content.tensor_order) {
        const TensorInfo *info = content.get_tensor_info(name);
        if (!info) throw Error(PMETAL_HIP_ERR_INVALID_ARG, "Tensor not found: " + name);
        if (!load_supported(info->dtype)) {
            if (skipped) skipped->push_back(name);
            continue;
        }
        LoadedTensor t;
        for (uint64_t d : info->dimensions) {
            if (d > (uint64_t)INT32_MAX)
                throw Error(PMETAL_HIP_ERR_SHAPE_TOO_LARGE,
                            "Tensor " + name + " dimension " + std::to_string(d) + " exceeds MLX i32 shape limits");
            t.shape.push_back((int32_t)d);
        }
        const std::vector<uint8_t> raw = content.read_tensor_data_from_file(path, name);
        t.data = dequantize_any(raw.data(), raw.size(), info->dtype, t.shape);
        weights[gguf_to_hf_name(name)] = std::move(t);
    }
    return weights;
}

// One f32 tensor of the model to quantize: its Hugging Face name, row-major shape and values (not owned).
struct SourceTensor {
    std::string name;
    std::vector<uint64_t> shape;
    const float *data;
};

// The quantize-and-write loop of run_quantization for `--method q4_k_m` over dense tensors
// (crates/pmetal/src/commands/quantize.rs:1339-1433): tensors in the order of their Hugging Face names, each under
// its GGUF name, with the type the recipe gives it (norms and 1-D tensors F16, attn_v / ffn_down of the layers that get
// more bits and the embedding / output matrices Q6_K, a fused attn_qkv Q5_K, the rest Q4_K), quantized by quantize_any.  The builder starts as
// GgufBuilder::with_model(architecture, "quantized-model"); the caller adds the model's own metadata and writes it.
inline GgufBuilder quantize_model_q4_k_m(const std::string &architecture, const std::vector<SourceTensor> &weights,
                                         size_t n_layers) {
    GgufBuilder builder = GgufBuilder::with_model(architecture, "quantized-model");
    std::vector<const SourceTensor *> order;
    for (const SourceTensor &t : weights) order.push_back(&t);
    std::sort(order.begin(), order.end(), [](const SourceTensor *a, const SourceTensor *b) { return a->name < b->name; });
    for (const SourceTensor *t : order) {
        const std::string gguf_name = hf_to_gguf_name(t->name);
        const GgmlType target = q4km_tensor_type(gguf_name, t->shape.size(), n_layers);
        size_t n = 1;
        for (uint64_t d : t->shape) n *= (size_t)d;
        try {
            builder.add_raw_tensor(gguf_name, t->shape, target, quantize_any(t->data, n, target));
        } catch (const Error &e) {
            throw QuantizationError(e.code, "Quantization error for " + t->name + ": " + e.what());
        }
    }
    return builder;
}

}  // namespace pmetal_gguf
