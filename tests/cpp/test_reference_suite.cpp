// The reference's own unit tests for this path, restated against the C++ host mirror
// (include/pmetal_gguf.hpp) so that they read like the originals:
//   crates/pmetal-gguf/src/k_quants.rs:1334-1342 (block sizes), :1368-1383 (Q4K dequantize range),
//   :1446-1465, :1490-1509, :1512-1553 (Q4K / Q6K / Q3K / Q2K round trips), crates/pmetal-gguf/src/dequant.rs:1016-1036 (Q8_0
//   block structure), :1139-1150 (invalid size / shape), crates/pmetal/src/commands/quantize.rs:1561-1608
//   (Q4_K_M recipe), crates/pmetal-gguf/src/dynamic.rs:789-800, :934-1018 (critical layers, KL metric, calibration).
// Usage: test_reference_suite [--host-only]   (--host-only skips everything that needs a GPU)
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "pmetal_gguf.hpp"

using namespace pmetal_gguf;

static int failures = 0;
#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            failures++;                                                    \
        }                                                                  \
    } while (0)

static float rmse(const std::vector<float> &a, const std::vector<float> &b) {
    double s = 0;
    for (size_t i = 0; i < a.size(); i++) s += (double)(a[i] - b[i]) * (a[i] - b[i]);
    return (float)std::sqrt(s / a.size());
}
static float max_err(const std::vector<float> &a, const std::vector<float> &b) {
    float m = 0;
    for (size_t i = 0; i < a.size(); i++) m = std::fmax(m, std::fabs(a[i] - b[i]));
    return m;
}
static uint16_t f16_bits(float f) {  // only for the exactly representable constants used below
    if (f == 0.0f) return 0;
    int e;
    float m = std::frexp(f, &e);  // f = m * 2^e, m in [0.5, 1)
    return (uint16_t)(((e - 1 + 15) << 10) | (uint16_t)((m * 2 - 1) * 1024));
}

static void test_block_sizes() {  // k_quants.rs:1334-1342
    CHECK(type_size(GgmlType::Q4K) == 144);
    CHECK(type_size(GgmlType::Q6K) == 210);
    CHECK(type_size(GgmlType::Q8_0) == 34);
    CHECK(block_size(GgmlType::Q4K) == 256 && block_size(GgmlType::Q8_0) == 32);
    CHECK(tensor_size(GgmlType::Q4K, 14336ull * 4096) == 33030144);
}

static void test_recipe() {  // commands/quantize.rs:1561-1608
    CHECK(q4km_tensor_type("blk.0.ffn_down.weight", 2, 32) == GgmlType::Q6K);
    CHECK(q4km_tensor_type("blk.0.attn_norm.weight", 1, 32) == GgmlType::F16);
    CHECK(q4km_tensor_type("output.weight", 2, 32) == GgmlType::Q6K);
    CHECK(q4km_tensor_type("blk.4.ffn_down.weight", 2, 32) == GgmlType::Q4K);
    CHECK(use_more_bits(0, 32) && !use_more_bits(4, 32) && use_more_bits(31, 32));
}

static void test_invalid_size_and_shape() {  // dequant.rs:1139-1150
    bool caught = false;
    try {
        dequantize(std::vector<uint8_t>(10), GgmlType::Q4K, {256});
    } catch (const DequantError &e) {
        caught = e.kind == DequantError::Kind::InvalidSize;
    }
    CHECK(caught);
    caught = false;
    try {
        dequantize(std::vector<uint8_t>(), GgmlType::Q4K, {-1});
    } catch (const DequantError &e) {
        caught = e.kind == DequantError::Kind::InvalidShape;
    }
    CHECK(caught);
    caught = false;
    try {
        quantize(std::vector<float>(256), (GgmlType)16);  // IQ2_XXS is outside this path
    } catch (const QuantizationError &) {
        caught = true;
    }
    CHECK(caught);
}

static void test_q8_0_block_structure() {  // dequant.rs:1016-1036
    std::vector<uint8_t> data(34);
    const uint16_t h = f16_bits(0.5f);
    std::memcpy(data.data(), &h, 2);
    for (int i = 0; i < 32; i++) data[2 + i] = (uint8_t)i;
    const auto r = dequantize(data, GgmlType::Q8_0, {32});
    CHECK(r.size() == 32);
    CHECK(std::fabs(r[0] - 0.0f) < 0.01f && std::fabs(r[2] - 1.0f) < 0.01f && std::fabs(r[4] - 2.0f) < 0.01f);
}

static void test_q4k_dequantize_simple() {  // k_quants.rs:1368-1383
    std::vector<uint8_t> blk(144, 0x21);
    const uint16_t one = f16_bits(1.0f), zero = 0;
    std::memcpy(&blk[0], &one, 2);
    std::memcpy(&blk[2], &zero, 2);
    const uint8_t scales[12] = {1, 1, 1, 1, 0, 0, 0, 0, 0, 0, 0, 0};
    std::memcpy(&blk[4], scales, 12);
    const auto out = dequantize(blk, GgmlType::Q4K, {256});
    bool in_range = true;
    for (float v : out) in_range = in_range && v >= 0.0f && v <= 15.0f;
    CHECK(in_range);
    CHECK(out[0] == 1.0f && out[16] == 2.0f && out[32] == 1.0f && out[48] == 2.0f && out[128] == 0.0f);
}

static void test_roundtrips() {  // k_quants.rs:1446-1465, :1490-1509
    std::vector<float> original(256);
    for (int i = 0; i < 256; i++) original[i] = ((float)i - 128.0f) * 0.01f;
    {
        const auto bytes = quantize(original, GgmlType::Q4K);
        CHECK(bytes.size() == 144);
        const auto restored = dequantize(bytes, GgmlType::Q4K, {256});
        CHECK(rmse(original, restored) < 0.15f && max_err(original, restored) < 0.5f);
        const auto ggml = dequantize(bytes, GgmlType::Q4K, {256}, PMETAL_HIP_ORDER_GGML);
        CHECK(rmse(original, ggml) < 0.02f);
    }
    {
        const auto bytes = quantize(original, GgmlType::Q6K);
        CHECK(bytes.size() == 210);
        const auto restored = dequantize(bytes, GgmlType::Q6K, {256});
        CHECK(rmse(original, restored) < 0.1f && max_err(original, restored) < 0.3f);
    }
    {  // k_quants.rs:1512-1531
        const auto bytes = quantize(original, GgmlType::Q3K);
        CHECK(bytes.size() == 110);
        const auto restored = dequantize(bytes, GgmlType::Q3K, {256});
        CHECK(rmse(original, restored) < 1.5f && max_err(original, restored) < 4.0f);
        CHECK(rmse(original, restored) < 0.2f);  // what the format actually achieves on the ramp
    }
    {  // k_quants.rs:1534-1553
        const auto bytes = quantize(original, GgmlType::Q2K);
        CHECK(bytes.size() == 84);
        const auto restored = dequantize(bytes, GgmlType::Q2K, {256});
        CHECK(rmse(original, restored) < 1.0f && max_err(original, restored) < 2.0f);
        CHECK(rmse(original, restored) < 0.3f);
    }
    {  // the Q5_K sibling of :1446-1465, in the order that inverts the quantizer's packing
        const auto bytes = quantize(original, GgmlType::Q5K);
        CHECK(bytes.size() == 176);
        const auto restored = dequantize(bytes, GgmlType::Q5K, {256}, PMETAL_HIP_ORDER_GGML);
        CHECK(rmse(original, restored) < 0.05f && max_err(original, restored) < 0.15f);
    }
    {
        const auto bytes = quantize(original, GgmlType::Q8_0);
        CHECK(bytes.size() == 8 * 34);
        const auto restored = dequantize(bytes, GgmlType::Q8_0, {256});
        CHECK(max_err(original, restored) < 0.01f);
    }
}

static void test_linear_matmul_from() {
    const int64_t n = 64, k = 512;
    std::vector<float> w((size_t)n * k);
    for (size_t i = 0; i < w.size(); i++) w[i] = 0.02f * std::sin(0.37f * (float)i);
    const auto packed = quantize(w, GgmlType::Q4K);
    const auto deq = dequantize(packed, GgmlType::Q4K, {(int32_t)n, (int32_t)k});
    std::vector<uint16_t> x(k);  // bf16 bit patterns of small integers (exact)
    std::vector<float> xf(k);
    for (int64_t i = 0; i < k; i++) {
        xf[i] = (float)((i % 7) - 3);
        uint32_t u;
        std::memcpy(&u, &xf[i], 4);
        x[i] = (uint16_t)(u >> 16);
    }
    GgufLinear lin(GgmlType::Q4K, n, k, packed);
    DeviceBuffer dx(x.data(), x.size() * 2);
    std::vector<float> y(n);
    lin.matmul_from(dx, 1).to_host(y.data(), n * sizeof(float));
    double worst = 0, scale = 0;
    for (int64_t r = 0; r < n; r++) {
        double want = 0;
        for (int64_t i = 0; i < k; i++) want += (double)deq[r * k + i] * xf[i];
        worst = std::fmax(worst, std::fabs(want - y[r]));
        scale = std::fmax(scale, std::fabs(want));
    }
    CHECK(worst <= 1e-3 * scale);
}

static void test_critical_layers() {  // dynamic.rs:789-800
    CHECK(is_critical_layer("lm_head.weight") && is_critical_layer("model.output.weight"));
    CHECK(is_critical_layer("model.embed_tokens.weight") && is_critical_layer("token_embd.weight"));
    CHECK(!is_critical_layer("model.layers.0.mlp.weight"));
    const KlCalibrationConfig cfg;  // dynamic.rs:958-965
    CHECK(cfg.candidates.size() == 6 && cfg.candidates.front() == GgmlType::Q8K && cfg.candidates.back() == GgmlType::Q2K);
    CHECK(cfg.sample_size == 0 && std::fabs(cfg.kl_threshold - 0.01) < 1e-9);
}

static void test_calibration() {  // dynamic.rs:968-1018, :934-956 through the device metric
    const KlCalibrationConfig cfg;
    const std::vector<float> ones(1024, 1.0f);
    const CalibratedTensor crit = calibrate_tensor("model.lm_head.weight", ones.data(), ones.size(), {32, 32}, cfg);
    CHECK(crit.quant_type == cfg.fallback_type && crit.kl_score == 0.0);
    std::vector<float> ramp(256);
    for (int i = 0; i < 256; i++) ramp[i] = (float)i * 0.01f - 1.28f;
    const CalibratedTensor r = calibrate_tensor("model.layers.0.mlp.gate_proj.weight", ramp.data(), ramp.size(), {1, 256}, cfg);
    bool member = r.quant_type == cfg.fallback_type;
    for (GgmlType t : cfg.candidates) member = member || t == r.quant_type;
    CHECK(member && !r.all_scores.empty());
    CHECK(r.all_scores.size() == 6 && r.all_scores[0].first == GgmlType::Q8K && r.all_scores[0].second < 0.01);
    // compute_kl_divergence: identical -> ~0, perturbed -> small positive, zeros -> 0
    const float a[8] = {1, 2, 3, 4, 5, 0, 0, 0}, b[8] = {1.1f, 2.1f, 2.9f, 4.2f, 4.8f, 0, 0, 0}, z[8] = {0};
    DeviceBuffer da(a, sizeof a), db(b, sizeof b), dz(z, sizeof z);
    double s = -1;
    detail::check(pmetal_hip_kl_divergence_dev((const float *)da.ptr(), (const float *)da.ptr(), 5, &s, nullptr));
    CHECK(s >= 0 && s < 1e-10);
    detail::check(pmetal_hip_kl_divergence_dev((const float *)da.ptr(), (const float *)db.ptr(), 5, &s, nullptr));
    CHECK(s > 0 && s < 1.0);
    detail::check(pmetal_hip_kl_divergence_dev((const float *)dz.ptr(), (const float *)dz.ptr(), 8, &s, nullptr));
    CHECK(s == 0.0);
}

// the tensor loop of run_quantization (commands/quantize.rs:1378-1428) over device-resident tensors: the bytes of quantize()
static void test_quantize_tensors_dev() {
    const GgmlType types[3] = {GgmlType::Q4K, GgmlType::Q6K, GgmlType::Q8_0};
    const size_t sizes[3] = {256 * 900, 256 * 500 + 17, 32 * 1000};
    std::vector<std::vector<float>> host(3);
    std::vector<DeviceBuffer> src;
    std::vector<DeviceTensorF32> list;
    for (int i = 0; i < 3; i++) {
        host[i].resize(sizes[i]);
        for (size_t j = 0; j < sizes[i]; j++) host[i][j] = 0.02f * std::sin(0.37f * (float)j + (float)i) + (j % 97 == 0 ? 0.4f : 0.0f);
        src.emplace_back(host[i].data(), sizes[i] * sizeof(float));
        list.push_back(DeviceTensorF32{types[i], (const float *)src.back().ptr(), sizes[i]});
    }
    std::vector<DeviceBuffer> outs = quantize_tensors_dev(list);
    detail::check(pmetal_hip_sync(nullptr));
    for (int i = 0; i < 3; i++) {
        const std::vector<uint8_t> want = quantize(host[i].data(), sizes[i], types[i]);
        std::vector<uint8_t> got(want.size());
        outs[i].to_host(got.data(), got.size());
        CHECK(got == want);
    }
}

int main(int argc, char **argv) {
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host-only") == 0;
    test_block_sizes();
    test_recipe();
    test_invalid_size_and_shape();
    test_critical_layers();
    if (!host_only) {
        CHECK(pmetal_hip_init(0) == 0);
        test_q8_0_block_structure();
        test_q4k_dequantize_simple();
        test_roundtrips();
        test_linear_matmul_from();
        test_calibration();
        test_quantize_tensors_dev();
    }
    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
