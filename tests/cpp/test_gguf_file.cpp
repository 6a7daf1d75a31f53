// Test driver for the GGUF container mirror (include/pmetal_gguf_file.hpp) and the Q4_K_M model driver
// (include/pmetal_gguf.hpp).
//
//   test_gguf_file                              the reference's own unit tests, restated:
//                                               crates/pmetal-gguf/src/writer.rs:617-723, reader.rs:614-671
//   test_gguf_file --build SPEC OUT             build the file a spec describes (grammar below) and write it
//   test_gguf_file --dump IN                    read a file and print what the reader found, canonically
//   test_gguf_file --read-error IN              print the kind of GgufReadError reading IN raises ("none" if none)
//   test_gguf_file --f16 IN OUT                 raw f32 values -> raw f16 bit patterns (f32_to_f16_bits)
//   test_gguf_file --quantize-model SPEC OUT    (GPU) synthetic f32 model -> quantize_model_q4_k_m -> OUT
//   test_gguf_file --f16-to-f32 IN OUT          raw f16 bit patterns -> raw f32 values (f16_bits_to_f32)
//   test_gguf_file --load-model IN OUT          (GPU) load_gguf: tensor names and shapes to stdout, f32 values to OUT
//   test_gguf_file --names IN                   (GPU build) gguf_to_hf_name and hf_to_gguf_name of every hex-encoded name in IN
//
// Spec grammar (whitespace-separated tokens; strings are hex-encoded so that they may hold anything):
//   align N | meta KEYHEX VALUE | tensor NAMEHEX DTYPE NDIMS DIM... SEED
//   VALUE := u8 N | i8 N | u16 N | i16 N | u32 N | i32 N | u64 N | i64 N | bool N | f32 BITS | f64 BITS | str HEX
//          | arr COUNT VALUE...
//   tensor data: byte i of the tensor is (SEED * 131 + i * 7 + (i >> 8)) & 0xFF
// Model spec: arch HEX | layers N | tensor NAMEHEX NDIMS DIM... SEED, values from the generator in synth_value().
#include <chrono>
#include <cinttypes>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <iterator>
#include <sstream>

#include "pmetal_gguf_file.hpp"
#ifndef PMETAL_TEST_HOST_ONLY
#include "pmetal_gguf.hpp"
#endif

using namespace pmetal_gguf;

static int failures = 0;
#define CHECK(cond)                                                      \
    do {                                                                 \
        if (!(cond)) {                                                   \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            failures++;                                                  \
        }                                                                \
    } while (0)

template <typename F>
static bool throws_invalid_argument(F f) {
    try {
        f();
    } catch (const InvalidArgument &) {
        return true;
    }
    return false;
}
template <typename F>
static std::string read_error_kind(F f) {
    static const char *const names[] = {"Io", "InvalidMagic", "UnsupportedVersion", "InvalidValueType", "InvalidDtype",
                                        "InvalidAlignment", "TensorNotFound", "InvalidUtf8", "StringTooLarge", "ArrayTooLarge",
                                        "TooManyTensors", "TooManyMetadata", "TooManyTensorDimensions", "DuplicateMetadataKey",
                                        "DuplicateTensorName", "ArrayNestingTooDeep", "IntegerOverflow"};
    try {
        f();
    } catch (const GgufReadError &e) {
        return names[(int)e.kind];
    }
    return "none";
}

static std::string unhex(const std::string &h) {
    std::string out;
    for (size_t i = 0; i + 1 < h.size(); i += 2) out.push_back((char)std::stoi(h.substr(i, 2), nullptr, 16));
    return out;
}
static std::string hex(const std::string &s) {
    static const char *d = "0123456789abcdef";
    std::string out;
    for (unsigned char c : s) out.push_back(d[c >> 4]), out.push_back(d[c & 15]);
    return out.empty() ? "-" : out;
}
static std::vector<uint8_t> slurp(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    return std::vector<uint8_t>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

static MetadataValue parse_value(std::istream &in) {
    std::string kind, tok;
    in >> kind;
    if (kind == "arr") {
        size_t n;
        in >> n;
        std::vector<MetadataValue> a;
        for (size_t i = 0; i < n; i++) a.push_back(parse_value(in));
        return MetadataValue::Array(std::move(a));
    }
    in >> tok;
    if (kind == "str") return MetadataValue::String(tok == "-" ? std::string() : unhex(tok));
    if (kind == "f32") {
        const uint32_t b = (uint32_t)std::stoull(tok);
        float f;
        std::memcpy(&f, &b, 4);
        return MetadataValue::Float32(f);
    }
    if (kind == "f64") {
        const uint64_t b = std::stoull(tok);
        double f;
        std::memcpy(&f, &b, 8);
        return MetadataValue::Float64(f);
    }
    if (kind == "u8") return MetadataValue::Uint8((uint8_t)std::stoull(tok));
    if (kind == "i8") return MetadataValue::Int8((int8_t)std::stoll(tok));
    if (kind == "u16") return MetadataValue::Uint16((uint16_t)std::stoull(tok));
    if (kind == "i16") return MetadataValue::Int16((int16_t)std::stoll(tok));
    if (kind == "u32") return MetadataValue::Uint32((uint32_t)std::stoull(tok));
    if (kind == "i32") return MetadataValue::Int32((int32_t)std::stoll(tok));
    if (kind == "u64") return MetadataValue::Uint64(std::stoull(tok));
    if (kind == "i64") return MetadataValue::Int64(std::stoll(tok));
    if (kind == "bool") return MetadataValue::Bool(tok != "0");
    throw std::runtime_error("bad value kind " + kind);
}

static void print_value(const MetadataValue &v) {
    switch (v.type) {
    case MetadataValueType::Uint8: std::printf("u8 %" PRIu64, v.u); break;
    case MetadataValueType::Int8: std::printf("i8 %" PRId64, v.i); break;
    case MetadataValueType::Uint16: std::printf("u16 %" PRIu64, v.u); break;
    case MetadataValueType::Int16: std::printf("i16 %" PRId64, v.i); break;
    case MetadataValueType::Uint32: std::printf("u32 %" PRIu64, v.u); break;
    case MetadataValueType::Int32: std::printf("i32 %" PRId64, v.i); break;
    case MetadataValueType::Uint64: std::printf("u64 %" PRIu64, v.u); break;
    case MetadataValueType::Int64: std::printf("i64 %" PRId64, v.i); break;
    case MetadataValueType::Bool: std::printf("bool %" PRIu64, v.u); break;
    case MetadataValueType::Float32: {
        uint32_t b;
        std::memcpy(&b, &v.f32, 4);
        std::printf("f32 %u", b);
        break;
    }
    case MetadataValueType::Float64: {
        uint64_t b;
        std::memcpy(&b, &v.f64, 8);
        std::printf("f64 %" PRIu64, b);
        break;
    }
    case MetadataValueType::String: std::printf("str %s", hex(v.str).c_str()); break;
    case MetadataValueType::Array:
        std::printf("arr %zu", v.arr.size());
        for (const MetadataValue &e : v.arr) {
            std::printf(" ");
            print_value(e);
        }
        break;
    }
}

static uint64_t fnv1a(const std::vector<uint8_t> &b) {
    uint64_t h = 1469598103934665603ull;
    for (uint8_t c : b) h = (h ^ c) * 1099511628211ull;
    return h;
}

static int cmd_build(const std::string &spec, const std::string &out) {
    std::ifstream in(spec);
    GgufBuilder b;
    std::string word;
    try {
        while (in >> word) {
            if (word == "align") {
                uint32_t a;
                in >> a;
                b.alignment(a);
            } else if (word == "meta") {
                std::string key;
                in >> key;
                b.add_metadata(key == "-" ? std::string() : unhex(key), parse_value(in));
            } else if (word == "tensor") {
                std::string name;
                uint32_t dtype;
                size_t nd;
                in >> name >> dtype >> nd;
                std::vector<uint64_t> dims(nd);
                uint64_t n = 1;
                for (uint64_t &d : dims) in >> d, n *= d;
                uint64_t seed;
                in >> seed;
                GgmlType t;
                if (!ggml_type_from_u32(dtype, t)) throw std::runtime_error("bad dtype");
                uint64_t bytes;
                if (!ggml_tensor_size_checked(t, n, bytes)) throw std::runtime_error("overflow");
                std::vector<uint8_t> data((size_t)bytes);
                for (size_t i = 0; i < data.size(); i++) data[i] = (uint8_t)((seed * 131 + i * 7 + (i >> 8)) & 0xFF);
                b.add_raw_tensor(unhex(name), dims, t, std::move(data));
            }
        }
        b.write_file(out);
    } catch (const InvalidArgument &e) {
        std::printf("InvalidArgument\n");
        return 3;
    }
    std::printf("ok\n");
    return 0;
}

static int cmd_dump(const std::string &path) {
    const std::vector<uint8_t> file = slurp(path);
    const GgufContent c = GgufContent::read(file);
    const GgufContent from_disk = GgufContent::from_file(path);
    std::printf("version %u\ndata_offset %" PRIu64 "\n", c.version, c.tensor_data_offset);
    std::vector<std::string> keys;
    for (const auto &kv : c.metadata) keys.push_back(kv.first);
    std::sort(keys.begin(), keys.end());
    for (const std::string &k : keys) {
        std::printf("meta %s ", hex(k).c_str());
        print_value(c.metadata.at(k));
        std::printf("\n");
    }
    for (const std::string &name : c.tensor_order) {
        const TensorInfo &t = c.tensor_infos.at(name);
        std::printf("tensor %s %u %u", hex(name).c_str(), (uint32_t)t.dtype, t.n_dimensions);
        for (uint64_t d : t.dimensions) std::printf(" %" PRIu64, d);
        const std::vector<uint8_t> data = c.read_tensor_data(file, name);
        if (data != from_disk.read_tensor_data_from_file(path, name)) std::printf(" MISMATCH-between-memory-and-file");
        std::printf(" offset %" PRIu64 " bytes %zu fnv %" PRIu64 "\n", t.offset, data.size(), fnv1a(data));
    }
    return 0;
}

#ifndef PMETAL_TEST_HOST_ONLY
// value i of a synthetic tensor: exact in double, so that every language computes the same float
static float synth_value(uint64_t seed, uint64_t i) {
    uint64_t z = seed * 0x9E3779B97F4A7C15ull + i * 0xBF58476D1CE4E5B9ull + 0x94D049BB133111EBull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const double u = (double)(z >> 40) / 16777216.0 - 0.5;  // 24 bits -> [-0.5, 0.5)
    return (float)(u * 0.125);
}

static int cmd_quantize_model(const std::string &spec, const std::string &out) {
    std::ifstream in(spec);
    std::string word, arch = "llama";
    size_t layers = 0;
    std::vector<std::vector<float>> storage;
    std::vector<SourceTensor> weights;
    while (in >> word) {
        if (word == "arch") {
            in >> word;
            arch = unhex(word);
        } else if (word == "layers") {
            in >> layers;
        } else if (word == "tensor") {
            std::string name;
            size_t nd;
            in >> name >> nd;
            std::vector<uint64_t> dims(nd);
            uint64_t n = 1;
            for (uint64_t &d : dims) in >> d, n *= d;
            uint64_t seed;
            in >> seed;
            storage.emplace_back((size_t)n);
            for (uint64_t i = 0; i < n; i++) storage.back()[(size_t)i] = synth_value(seed, i);
            weights.push_back(SourceTensor{unhex(name), dims, nullptr});
        }
    }
    for (size_t i = 0; i < weights.size(); i++) weights[i].data = storage[i].data();
    double f32_bytes = 0;
    for (const auto &v : storage) f32_bytes += 4.0 * (double)v.size();
    const auto t0 = std::chrono::steady_clock::now();
    GgufBuilder b = quantize_model_q4_k_m(arch, weights, layers);
    const auto t1 = std::chrono::steady_clock::now();
    b.add_u32(arch + ".block_count", (uint32_t)layers);
    b.write_file(out);
    const auto t2 = std::chrono::steady_clock::now();
    const double q = std::chrono::duration<double>(t1 - t0).count(), w = std::chrono::duration<double>(t2 - t1).count();
    std::printf("ok %zu tensors; %.3f GB of f32 quantized from host memory in %.3f s (%.2f GB/s), file written in %.3f s\n",
                b.num_tensors(), f32_bytes / 1e9, q, f32_bytes / 1e9 / q, w);
    return 0;
}

// load_gguf: per tensor, in the order of the Hugging Face names, a line `hexname ndim dims... dtype-independent count`;
// the f32 values of all tensors follow each other in OUT in the same order.
static int cmd_load_model(const std::string &file, const std::string &out) {
    std::vector<std::string> skipped;
    const auto weights = load_gguf(file, &skipped);
    std::ofstream o(out, std::ios::binary);
    for (const auto &kv : weights) {
        std::printf("%s %zu", hex(kv.first).c_str(), kv.second.shape.size());
        for (int32_t d : kv.second.shape) std::printf(" %d", d);
        std::printf(" %zu\n", kv.second.data.size());
        o.write(reinterpret_cast<const char *>(kv.second.data.data()), (std::streamsize)(kv.second.data.size() * 4));
    }
    for (const std::string &s : skipped) std::printf("skipped %s\n", hex(s).c_str());
    return 0;
}
#endif

static void put32(std::vector<uint8_t> &b, uint32_t v) { detail::put_le<uint32_t>(b, v); }
static void put64(std::vector<uint8_t> &b, uint64_t v) { detail::put_le<uint64_t>(b, v); }
static void put_str(std::vector<uint8_t> &b, const std::string &s) {
    put64(b, s.size());
    b.insert(b.end(), s.begin(), s.end());
}

static int reference_tests() {
    {  // writer.rs:617-626 test_gguf_header
        const std::vector<uint8_t> bytes = GgufBuilder::with_model("llama", "test-model").build_to_bytes();
        const uint32_t magic = GGUF_MAGIC, version = GGUF_VERSION;
        CHECK(std::memcmp(bytes.data(), &magic, 4) == 0);
        CHECK(std::memcmp(bytes.data() + 4, &version, 4) == 0);
    }
    {  // :629-636 test_gguf_metadata
        GgufBuilder b = GgufBuilder::with_model("llama", "test-model");
        b.add_u32("test.value", 42).add_string("test.string", "hello");
        CHECK(!b.build_to_bytes().empty());
    }
    {  // :639-653 test_gguf_tensor, :656-669 tensor_dimensions_round_trip_in_row_major_order
        GgufBuilder b = GgufBuilder::with_model("llama", "test-model");
        b.add_f32_tensor("test.weight", {2, 3}, {1.0f, 2.0f, 3.0f, 4.0f, 5.0f, 6.0f});
        const std::vector<uint8_t> bytes = b.build_to_bytes();
        uint64_t count;
        std::memcpy(&count, bytes.data() + 8, 8);
        CHECK(count == 1);
        const GgufContent c = GgufContent::read(bytes);
        const TensorInfo *info = c.get_tensor_info("test.weight");
        CHECK(info && info->dimensions == (std::vector<uint64_t>{2, 3}));
        const std::vector<uint8_t> data = c.read_tensor_data(bytes, "test.weight");
        float back[6];
        CHECK(data.size() == 24);
        std::memcpy(back, data.data(), 24);
        CHECK(back[0] == 1.0f && back[5] == 6.0f);
        CHECK(c.architecture() && *c.architecture() == "llama");
        CHECK(c.tensor_data_offset % 32 == 0 && c.version == 3);
    }
    // :672-677 test_alignment
    CHECK(align_offset(0, 32) == 0 && align_offset(1, 32) == 32 && align_offset(32, 32) == 32 && align_offset(33, 32) == 64);
    {  // :680-689 test_string_array
        GgufBuilder b = GgufBuilder::with_model("llama", "test-model");
        b.add_string_array("tokenizer.ggml.tokens", {"hello", "world"});
        const GgufContent c = GgufContent::read(b.build_to_bytes());
        const MetadataValue *v = c.get_metadata("tokenizer.ggml.tokens");
        CHECK(v && v->type == MetadataValueType::Array && v->arr.size() == 2 && v->arr[1].str == "world");
    }
    // :692-695 zero_alignment_is_rejected
    CHECK(throws_invalid_argument([] { GgufBuilder::with_model("llama", "test-model").alignment(0).build_to_bytes(); }));
    // :698-708 heterogeneous_metadata_array_is_rejected
    CHECK(throws_invalid_argument([] {
        GgufBuilder b = GgufBuilder::with_model("llama", "test-model");
        b.add_metadata("bad.array", MetadataValue::Array({MetadataValue::Uint32(1), MetadataValue::String("two")}));
        b.build_to_bytes();
    }));
    // :711-715 tensor_byte_size_mismatch_is_rejected
    CHECK(throws_invalid_argument([] {
        GgufBuilder b = GgufBuilder::with_model("llama", "test-model");
        b.add_raw_tensor("bad.weight", {2}, GgmlType::F32, std::vector<uint8_t>(4, 0));
        b.build_to_bytes();
    }));
    // :718-723 duplicate_tensor_names_are_rejected
    CHECK(throws_invalid_argument([] {
        GgufBuilder b = GgufBuilder::with_model("llama", "test-model");
        b.add_f32_tensor("dup.weight", {1}, {1.0f}).add_f32_tensor("dup.weight", {1}, {2.0f});
        b.build_to_bytes();
    }));
    {  // reader.rs:614-625 test_ggml_type_conversion
        GgmlType t;
        CHECK(ggml_type_from_u32(0, t) && t == GgmlType::F32);
        CHECK(ggml_type_from_u32(1, t) && t == GgmlType::F16);
        CHECK(ggml_type_from_u32(2, t) && t == GgmlType::Q4_0);
        CHECK(ggml_type_from_u32(8, t) && t == GgmlType::Q8_0);
        CHECK(ggml_type_from_u32(30, t) && t == GgmlType::Bf16);
        CHECK(ggml_type_from_u32(39, t) && t == GgmlType::Mxfp4);
        CHECK(ggml_type_from_u32(40, t) && t == GgmlType::Nvfp4);
        CHECK(ggml_type_from_u32(41, t) && t == GgmlType::Q1_0);
        CHECK(!ggml_type_from_u32(255, t) && !ggml_type_from_u32(4, t) && !ggml_type_from_u32(5, t));
    }
    {  // reader.rs:634-650 duplicate_metadata_keys_are_rejected
        std::vector<uint8_t> b;
        put32(b, GGUF_MAGIC), put32(b, 3), put64(b, 0), put64(b, 2);
        put_str(b, "dup"), put32(b, 4), put32(b, 1);
        put_str(b, "dup"), put32(b, 4), put32(b, 2);
        bool hit = false;
        try {
            GgufContent::read(b);
        } catch (const GgufReadError &e) {
            hit = e.kind == GgufReadError::Kind::DuplicateMetadataKey && e.subject == "dup";
        }
        CHECK(hit);
    }
    {  // reader.rs:653-669 excessive_tensor_rank_is_rejected_before_dimension_allocation
        std::vector<uint8_t> b;
        put32(b, GGUF_MAGIC), put32(b, 3), put64(b, 1), put64(b, 0);
        put_str(b, "bad.weight"), put32(b, MAX_TENSOR_DIMS + 1);
        bool hit = false;
        try {
            GgufContent::read(b);
        } catch (const GgufReadError &e) {
            hit = e.kind == GgufReadError::Kind::TooManyTensorDimensions && e.subject == "bad.weight";
        }
        CHECK(hit);
    }
    {  // the k-quant block sizes the container relies on (k_quants.rs:1334-1342)
        uint64_t bytes;
        CHECK(ggml_tensor_size_checked(GgmlType::Q4K, 256, bytes) && bytes == 144);
        CHECK(ggml_tensor_size_checked(GgmlType::Q6K, 257, bytes) && bytes == 420);
        CHECK(ggml_tensor_size_checked(GgmlType::Q8_0, 33, bytes) && bytes == 68);
        CHECK(!ggml_tensor_size_checked(GgmlType::F64, UINT64_MAX / 4, bytes));
    }
    if (failures == 0) std::printf("all reference container tests passed\n");
    return failures ? 1 : 0;
}

int main(int argc, char **argv) {
    try {
        if (argc == 1) return reference_tests();
        const std::string cmd = argv[1];
        if (cmd == "--build" && argc == 4) return cmd_build(argv[2], argv[3]);
        if (cmd == "--dump" && argc == 3) return cmd_dump(argv[2]);
        if (cmd == "--read-error" && argc == 3) {
            const std::vector<uint8_t> file = slurp(argv[2]);
            std::printf("%s\n", read_error_kind([&] { GgufContent::read(file); }).c_str());
            return 0;
        }
        if (cmd == "--f16" && argc == 4) {
            const std::vector<uint8_t> in = slurp(argv[2]);
            std::vector<uint16_t> out(in.size() / 4);
            for (size_t i = 0; i < out.size(); i++) {
                float f;
                std::memcpy(&f, in.data() + 4 * i, 4);
                out[i] = f32_to_f16_bits(f);
            }
            std::ofstream(argv[3], std::ios::binary).write(reinterpret_cast<const char *>(out.data()), (std::streamsize)(out.size() * 2));
            return 0;
        }
        if (cmd == "--f16-to-f32" && argc == 4) {
            const std::vector<uint8_t> in = slurp(argv[2]);
            std::vector<float> out(in.size() / 2);
            for (size_t i = 0; i < out.size(); i++) {
                uint16_t h;
                std::memcpy(&h, in.data() + 2 * i, 2);
                out[i] = f16_bits_to_f32(h);
            }
            std::ofstream(argv[3], std::ios::binary).write(reinterpret_cast<const char *>(out.data()), (std::streamsize)(out.size() * 4));
            return 0;
        }
#ifndef PMETAL_TEST_HOST_ONLY
        if (cmd == "--quantize-model" && argc == 4) return cmd_quantize_model(argv[2], argv[3]);
        if (cmd == "--load-model" && argc == 4) return cmd_load_model(argv[2], argv[3]);
        if (cmd == "--names" && argc == 3) {  // one hex-encoded name per line: both mappings of it
            std::ifstream in(argv[2]);
            std::string word;
            while (in >> word) {
                const std::string name = unhex(word);
                std::printf("%s %s\n", hex(gguf_to_hf_name(name)).c_str(), hex(hf_to_gguf_name(name)).c_str());
            }
            return 0;
        }
#endif
    } catch (const std::exception &e) {
        std::printf("exception: %s\n", e.what());
        return 2;
    }
    std::printf("usage: see the head of tests/cpp/test_gguf_file.cpp\n");
    return 64;
}
