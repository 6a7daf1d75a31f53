// pmetal_gguf_file.hpp -- the GGUF container (version 3 writer, version 1-3 reader) beside the quantizer, as a
// header-only C++ mirror of the reference's builder and reader.  Host code only: nothing here needs the GPU or
// libpmetal_hip.so; include/pmetal_gguf.hpp puts the GPU quantizer in front of it.
//
// Names, argument meaning, limits and error behaviour follow
//   GgufBuilder            crates/pmetal-gguf/src/writer.rs:14-538   (metadata in key order, tensor data aligned,
//                                                                    dimensions reversed on disk)
//   GgufContent            crates/pmetal-gguf/src/reader.rs:176-444  (header, metadata, tensor infos; data on demand)
//   GgufReadError          crates/pmetal-gguf/src/reader.rs:80-170
//   GgmlType, TensorInfo, MetadataValue, keys   crates/pmetal-gguf/src/types.rs:4-390
// A Rust `Err` becomes a thrown exception: InvalidArgument for the builder (PMetalError::InvalidArgument),
// GgufReadError{kind} for the reader.
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace pmetal_gguf {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;  // "GGUF", little endian (types.rs:4)
constexpr uint32_t GGUF_VERSION = 3;          // types.rs:7
constexpr uint32_t GGUF_DEFAULT_ALIGNMENT = 32;  // types.rs:10

// reader.rs:58-77
constexpr size_t MAX_STRING_LENGTH = 10u * 1024u * 1024u;
constexpr size_t MAX_ARRAY_LENGTH = 1000000;
constexpr size_t MAX_TENSOR_COUNT = 100000;
constexpr size_t MAX_METADATA_COUNT = 100000;
constexpr uint32_t MAX_TENSOR_DIMS = 16;
constexpr uint8_t MAX_ARRAY_DEPTH = 8;  // reader.rs:485

namespace keys {  // types.rs:370-390
constexpr const char *GENERAL_ARCHITECTURE = "general.architecture";
constexpr const char *GENERAL_QUANTIZATION_VERSION = "general.quantization_version";
constexpr const char *GENERAL_ALIGNMENT = "general.alignment";
constexpr const char *GENERAL_NAME = "general.name";
constexpr const char *GENERAL_FILE_TYPE = "general.file_type";
}  // namespace keys

// types.rs:16-97 (ids), :102-187 (sizes)
enum class GgmlType : uint32_t {
    F32 = 0, F16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9, Q2K = 10, Q3K = 11, Q4K = 12, Q5K = 13,
    Q6K = 14, Q8K = 15, Iq2Xxs = 16, Iq2Xs = 17, Iq3Xxs = 18, Iq1S = 19, Iq4Nl = 20, Iq3S = 21, Iq2S = 22, Iq4Xs = 23,
    I8 = 24, I16 = 25, I32 = 26, I64 = 27, F64 = 28, Iq1M = 29, Bf16 = 30, Q4_0_4_4 = 31, Q4_0_4_8 = 32, Q4_0_8_8 = 33,
    Tq1_0 = 34, Tq2_0 = 35, Iq4Nl_4_4 = 36, Iq4Nl_4_8 = 37, Iq4Nl_8_8 = 38, Mxfp4 = 39, Nvfp4 = 40, Q1_0 = 41,
};

namespace detail {
struct TypeRow {
    uint32_t id, bytes, elems;
};
// (id, bytes per block, elements per block)
constexpr TypeRow kTypeTable[] = {
    {0, 4, 1},     {1, 2, 1},     {2, 18, 32},   {3, 20, 32},   {6, 22, 32},    {7, 24, 32},   {8, 34, 32},   {9, 36, 32},
    {10, 84, 256}, {11, 110, 256}, {12, 144, 256}, {13, 176, 256}, {14, 210, 256}, {15, 292, 256}, {16, 66, 256}, {17, 74, 256},
    {18, 98, 256}, {19, 50, 256}, {20, 18, 32},  {21, 110, 256}, {22, 82, 256},  {23, 136, 256}, {24, 1, 1},    {25, 2, 1},
    {26, 4, 1},    {27, 8, 1},    {28, 8, 1},    {29, 56, 256}, {30, 2, 1},     {31, 18, 32},  {32, 18, 32},  {33, 18, 32},
    {34, 54, 256}, {35, 66, 256}, {36, 18, 32},  {37, 18, 32},  {38, 18, 32},   {39, 17, 32},  {40, 36, 64},  {41, 18, 128},
};
inline const TypeRow *type_row(uint32_t id) {
    for (const TypeRow &r : kTypeTable)
        if (r.id == id) return &r;
    return nullptr;
}
}  // namespace detail

// GgmlType::try_from (reader.rs:563-612)
inline bool ggml_type_from_u32(uint32_t v, GgmlType &out) {
    if (!detail::type_row(v)) return false;
    out = (GgmlType)v;
    return true;
}
inline size_t ggml_type_size(GgmlType t) { return detail::type_row((uint32_t)t)->bytes; }
inline size_t ggml_block_size(GgmlType t) { return detail::type_row((uint32_t)t)->elems; }
// tensor_size_checked (types.rs:181-186): false on overflow
inline bool ggml_tensor_size_checked(GgmlType t, uint64_t n_elements, uint64_t &bytes) {
    const uint64_t bs = ggml_block_size(t), ts = ggml_type_size(t);
    if (n_elements > UINT64_MAX - (bs - 1)) return false;
    const uint64_t blocks = (n_elements + bs - 1) / bs;
    if (blocks != 0 && ts > UINT64_MAX / blocks) return false;
    bytes = blocks * ts;
    return true;
}

// types.rs:193-220
enum class MetadataValueType : uint32_t {
    Uint8 = 0, Int8 = 1, Uint16 = 2, Int16 = 3, Uint32 = 4, Int32 = 5, Float32 = 6, Bool = 7, String = 8, Array = 9,
    Uint64 = 10, Int64 = 11, Float64 = 12,
};

// types.rs:224-251.  One of: an integer (u: unsigned kinds and Bool, i: signed kinds), a float (f32 / f64), a string, or
// an array of values.
struct MetadataValue {
    MetadataValueType type = MetadataValueType::Uint8;
    uint64_t u = 0;
    int64_t i = 0;
    float f32 = 0.0f;
    double f64 = 0.0;
    std::string str;
    std::vector<MetadataValue> arr;

    MetadataValueType value_type() const { return type; }
    static MetadataValue Uint8(uint8_t v) { return unsigned_(MetadataValueType::Uint8, v); }
    static MetadataValue Int8(int8_t v) { return signed_(MetadataValueType::Int8, v); }
    static MetadataValue Uint16(uint16_t v) { return unsigned_(MetadataValueType::Uint16, v); }
    static MetadataValue Int16(int16_t v) { return signed_(MetadataValueType::Int16, v); }
    static MetadataValue Uint32(uint32_t v) { return unsigned_(MetadataValueType::Uint32, v); }
    static MetadataValue Int32(int32_t v) { return signed_(MetadataValueType::Int32, v); }
    static MetadataValue Uint64(uint64_t v) { return unsigned_(MetadataValueType::Uint64, v); }
    static MetadataValue Int64(int64_t v) { return signed_(MetadataValueType::Int64, v); }
    static MetadataValue Bool(bool v) { return unsigned_(MetadataValueType::Bool, v ? 1 : 0); }
    static MetadataValue Float32(float v) {
        MetadataValue m;
        m.type = MetadataValueType::Float32, m.f32 = v;
        return m;
    }
    static MetadataValue Float64(double v) {
        MetadataValue m;
        m.type = MetadataValueType::Float64, m.f64 = v;
        return m;
    }
    static MetadataValue String(std::string v) {
        MetadataValue m;
        m.type = MetadataValueType::String, m.str = std::move(v);
        return m;
    }
    static MetadataValue Array(std::vector<MetadataValue> v) {
        MetadataValue m;
        m.type = MetadataValueType::Array, m.arr = std::move(v);
        return m;
    }

   private:
    static MetadataValue unsigned_(MetadataValueType t, uint64_t v) {
        MetadataValue m;
        m.type = t, m.u = v;
        return m;
    }
    static MetadataValue signed_(MetadataValueType t, int64_t v) {
        MetadataValue m;
        m.type = t, m.i = v;
        return m;
    }
};

struct InvalidArgument : std::invalid_argument {  // PMetalError::InvalidArgument
    using std::invalid_argument::invalid_argument;
};

// types.rs:284-366.  `dimensions` is row-major (outermost first), as the reference's public API has it.
struct TensorInfo {
    std::string name;
    uint32_t n_dimensions = 0;
    std::vector<uint64_t> dimensions;
    GgmlType dtype = GgmlType::F32;
    uint64_t offset = 0;  // relative to the tensor data section; set by the writer

    TensorInfo() = default;
    TensorInfo(std::string n, std::vector<uint64_t> dims, GgmlType t)
        : name(std::move(n)), n_dimensions((uint32_t)dims.size()), dimensions(std::move(dims)), dtype(t) {}

    // n_elements_checked / byte_size_checked: false on overflow
    bool n_elements_checked(uint64_t &n) const {
        uint64_t total = 1;
        for (uint64_t d : dimensions) {
            if (d != 0 && total > UINT64_MAX / d) return false;
            total *= d;
        }
        n = total;
        return true;
    }
    bool byte_size_checked(uint64_t &bytes) const {
        uint64_t n;
        return n_elements_checked(n) && ggml_tensor_size_checked(dtype, n, bytes);
    }
};

namespace detail {
inline bool align_offset_checked(uint64_t offset, uint64_t alignment, uint64_t &out) {  // writer.rs:591-606
    const uint64_t rem = offset % alignment;
    if (rem == 0) {
        out = offset;
        return true;
    }
    if (offset > UINT64_MAX - (alignment - rem)) return false;
    out = offset + (alignment - rem);
    return true;
}
template <typename T>
inline void put_le(std::vector<uint8_t> &out, T v) {  // the build targets little-endian hosts only
    uint8_t b[sizeof(T)];
    std::memcpy(b, &v, sizeof(T));
    out.insert(out.end(), b, b + sizeof(T));
}
}  // namespace detail

// half::f16::from_f32 on the host (IEEE round to nearest even, subnormals kept, NaN quieted with its top payload bits):
// the F16 tensors of a quantized model (norms, 1-D tensors) are small, they do not go to the GPU.
inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, exp = (x >> 23) & 0xFFu, man = x & 0x7FFFFFu;
    if (exp == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? (0x0200u | (man >> 13)) : 0u));
    const int e = (int)exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);  // overflow to infinity
    if (e <= 0) {                                       // subnormal half or zero
        if (e < -10) return (uint16_t)sign;
        const uint32_t m = man | 0x800000u;
        const int shift = 14 - e;  // 14 .. 24
        uint32_t half_man = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);  // a carry into the exponent field gives the smallest normal, as it should
    }
    uint32_t out = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (out & 1u))) out++;  // may carry up to infinity, as it should
    return (uint16_t)(sign | out);
}

// half::f16::to_f32 on the host: exact (every f16 value, subnormals included, is an f32 value; NaN keeps its payload).
inline float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0x1F) {
        x = sign | 0x7F800000u | (man << 13);
    } else if (exp != 0) {
        x = sign | ((exp + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        x = sign;
    } else {  // subnormal half: man * 2^-24, normalised
        int shift = 0;
        uint32_t m = man;
        while (!(m & 0x400u)) m <<= 1, shift++;
        x = sign | ((uint32_t)(113 - shift) << 23) | ((m & 0x3FFu) << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// align_offset (writer.rs:609-611, test helper in the reference)
inline uint64_t align_offset(uint64_t offset, uint64_t alignment) {
    uint64_t out;
    if (alignment == 0) throw InvalidArgument("GGUF alignment must be greater than zero");
    if (!detail::align_offset_checked(offset, alignment, out)) throw InvalidArgument("GGUF aligned offset overflows u64");
    return out;
}

// writer.rs:14-538
class GgufBuilder {
   public:
    GgufBuilder() {  // :33-50
        add_metadata(keys::GENERAL_ALIGNMENT, MetadataValue::Uint32(GGUF_DEFAULT_ALIGNMENT));
        add_metadata(keys::GENERAL_QUANTIZATION_VERSION, MetadataValue::Uint32(2));
    }
    static GgufBuilder with_model(const std::string &architecture, const std::string &name) {  // :53-64
        GgufBuilder b;
        b.add_metadata(keys::GENERAL_ARCHITECTURE, MetadataValue::String(architecture));
        b.add_metadata(keys::GENERAL_NAME, MetadataValue::String(name));
        return b;
    }
    GgufBuilder &alignment(uint32_t a) {  // :67-74
        alignment_ = a;
        metadata_[keys::GENERAL_ALIGNMENT] = MetadataValue::Uint32(a);
        return *this;
    }
    GgufBuilder &add_metadata(const std::string &key, MetadataValue v) {  // :77-80 (a later value replaces an earlier one)
        metadata_[key] = std::move(v);
        return *this;
    }
    GgufBuilder &add_string(const std::string &key, const std::string &v) { return add_metadata(key, MetadataValue::String(v)); }
    GgufBuilder &add_u32(const std::string &key, uint32_t v) { return add_metadata(key, MetadataValue::Uint32(v)); }
    GgufBuilder &add_u64(const std::string &key, uint64_t v) { return add_metadata(key, MetadataValue::Uint64(v)); }
    GgufBuilder &add_f32(const std::string &key, float v) { return add_metadata(key, MetadataValue::Float32(v)); }
    GgufBuilder &add_bool(const std::string &key, bool v) { return add_metadata(key, MetadataValue::Bool(v)); }
    GgufBuilder &add_string_array(const std::string &key, const std::vector<std::string> &values) {
        std::vector<MetadataValue> a;
        for (const std::string &s : values) a.push_back(MetadataValue::String(s));
        return add_metadata(key, MetadataValue::Array(std::move(a)));
    }
    GgufBuilder &add_f32_array(const std::string &key, const std::vector<float> &values) {
        std::vector<MetadataValue> a;
        for (float v : values) a.push_back(MetadataValue::Float32(v));
        return add_metadata(key, MetadataValue::Array(std::move(a)));
    }
    GgufBuilder &add_i32_array(const std::string &key, const std::vector<int32_t> &values) {
        std::vector<MetadataValue> a;
        for (int32_t v : values) a.push_back(MetadataValue::Int32(v));
        return add_metadata(key, MetadataValue::Array(std::move(a)));
    }
    GgufBuilder &add_f32_tensor(const std::string &name, std::vector<uint64_t> dims, const std::vector<float> &data) {  // :126-137
        std::vector<uint8_t> bytes(data.size() * 4);
        if (!data.empty()) std::memcpy(bytes.data(), data.data(), bytes.size());
        return add_raw_tensor(name, std::move(dims), GgmlType::F32, std::move(bytes));
    }
    // f16 / bf16 tensors are handed over as their 16-bit patterns (:140-164)
    GgufBuilder &add_f16_tensor(const std::string &name, std::vector<uint64_t> dims, const std::vector<uint16_t> &bits) {
        return add_16bit(name, std::move(dims), GgmlType::F16, bits);
    }
    GgufBuilder &add_bf16_tensor(const std::string &name, std::vector<uint64_t> dims, const std::vector<uint16_t> &bits) {
        return add_16bit(name, std::move(dims), GgmlType::Bf16, bits);
    }
    GgufBuilder &add_raw_tensor(const std::string &name, std::vector<uint64_t> dims, GgmlType dtype, std::vector<uint8_t> data) {  // :167-177
        tensors_.emplace_back(TensorInfo(name, std::move(dims), dtype), std::move(data));
        return *this;
    }

    size_t num_tensors() const { return tensors_.size(); }
    const std::vector<std::pair<TensorInfo, std::vector<uint8_t>>> &tensors() const { return tensors_; }

    // write (:180-224) into memory
    std::vector<uint8_t> build_to_bytes() const {
        validate();
        std::vector<uint8_t> out;
        uint64_t total = 0;
        for (const auto &t : tensors_) total += t.second.size() + alignment_;
        out.reserve((size_t)total + 4096);
        detail::put_le<uint32_t>(out, GGUF_MAGIC);  // write_header :303-327
        detail::put_le<uint32_t>(out, GGUF_VERSION);
        detail::put_le<uint64_t>(out, tensors_.size());
        detail::put_le<uint64_t>(out, metadata_.size());
        for (const auto &kv : metadata_) {  // BTreeMap order = byte-wise key order = std::map<std::string>
            write_string(out, kv.first);
            write_value(out, kv.second);
        }
        for (const TensorInfo &info : calculate_tensor_offsets()) write_tensor_info(out, info);
        pad_to_alignment(out);
        for (size_t i = 0; i < tensors_.size(); i++) {
            out.insert(out.end(), tensors_[i].second.begin(), tensors_[i].second.end());
            if (i + 1 < tensors_.size()) pad_to_alignment(out);  // no padding behind the last tensor (:213-220)
        }
        return out;
    }
    void write_file(const std::string &path) const {
        const std::vector<uint8_t> bytes = build_to_bytes();
        std::ofstream f(path, std::ios::binary | std::ios::trunc);
        if (!f) throw std::runtime_error("cannot open " + path + " for writing");
        f.write(reinterpret_cast<const char *>(bytes.data()), (std::streamsize)bytes.size());
        if (!f) throw std::runtime_error("write to " + path + " failed");
    }

   private:
    GgufBuilder &add_16bit(const std::string &name, std::vector<uint64_t> dims, GgmlType t, const std::vector<uint16_t> &bits) {
        std::vector<uint8_t> bytes(bits.size() * 2);
        if (!bits.empty()) std::memcpy(bytes.data(), bits.data(), bytes.size());
        return add_raw_tensor(name, std::move(dims), t, std::move(bytes));
    }
    void validate() const {  // :226-293
        if (alignment_ == 0 || alignment_ > 1048576)
            throw InvalidArgument("GGUF alignment must be in 1..=1048576, got " + std::to_string(alignment_));
        for (const auto &kv : metadata_) {
            if (kv.first.size() > MAX_STRING_LENGTH)
                throw InvalidArgument("GGUF metadata key " + kv.first + " exceeds " + std::to_string(MAX_STRING_LENGTH) + " bytes");
            validate_value(kv.second);
        }
        std::set<std::string> names;
        for (const auto &t : tensors_) {
            const TensorInfo &info = t.first;
            if (!names.insert(info.name).second) throw InvalidArgument("Duplicate GGUF tensor name: " + info.name);
            if (info.name.size() > MAX_STRING_LENGTH)
                throw InvalidArgument("GGUF tensor name " + info.name + " exceeds " + std::to_string(MAX_STRING_LENGTH) + " bytes");
            if (info.n_dimensions != info.dimensions.size())
                throw InvalidArgument("GGUF tensor " + info.name + " declares " + std::to_string(info.n_dimensions) +
                                      " dimensions but stores " + std::to_string(info.dimensions.size()));
            if (info.n_dimensions > MAX_TENSOR_DIMS)
                throw InvalidArgument("GGUF tensor " + info.name + " has " + std::to_string(info.n_dimensions) +
                                      " dimensions, exceeding maximum of " + std::to_string(MAX_TENSOR_DIMS));
            uint64_t expected;
            if (!info.byte_size_checked(expected))
                throw InvalidArgument("GGUF tensor " + info.name + " has invalid dimensions or dtype: integer overflow");
            if (expected != t.second.size())
                throw InvalidArgument("GGUF tensor " + info.name + " has " + std::to_string(t.second.size()) + " bytes but its shape requires " +
                                      std::to_string(expected) + " bytes");
        }
    }
    static void validate_array_elements(const std::vector<MetadataValue> &arr) {  // :559-576
        if (arr.size() > MAX_ARRAY_LENGTH)
            throw InvalidArgument("GGUF metadata array has " + std::to_string(arr.size()) + " elements, exceeding " + std::to_string(MAX_ARRAY_LENGTH));
        for (const MetadataValue &e : arr)
            if (e.type != arr.front().type) throw InvalidArgument("GGUF metadata arrays must contain a single value type");
    }
    static void validate_value(const MetadataValue &v) {  // :540-557
        if (v.type == MetadataValueType::String && v.str.size() > MAX_STRING_LENGTH)
            throw InvalidArgument("GGUF string metadata value exceeds " + std::to_string(MAX_STRING_LENGTH) + " bytes");
        if (v.type == MetadataValueType::Array) {
            validate_array_elements(v.arr);
            for (const MetadataValue &e : v.arr) validate_value(e);
        }
    }
    static void write_string(std::vector<uint8_t> &out, const std::string &s) {  // :330-341
        detail::put_le<uint64_t>(out, s.size());
        out.insert(out.end(), s.begin(), s.end());
    }
    static void write_value(std::vector<uint8_t> &out, const MetadataValue &v) {  // :344-415: type, then the data
        detail::put_le<uint32_t>(out, (uint32_t)v.type);
        write_value_data(out, v);
    }
    static void write_value_data(std::vector<uint8_t> &out, const MetadataValue &v) {  // :418-480
        switch (v.type) {
        case MetadataValueType::Uint8: detail::put_le<uint8_t>(out, (uint8_t)v.u); break;
        case MetadataValueType::Int8: detail::put_le<int8_t>(out, (int8_t)v.i); break;
        case MetadataValueType::Uint16: detail::put_le<uint16_t>(out, (uint16_t)v.u); break;
        case MetadataValueType::Int16: detail::put_le<int16_t>(out, (int16_t)v.i); break;
        case MetadataValueType::Uint32: detail::put_le<uint32_t>(out, (uint32_t)v.u); break;
        case MetadataValueType::Int32: detail::put_le<int32_t>(out, (int32_t)v.i); break;
        case MetadataValueType::Float32: detail::put_le<float>(out, v.f32); break;
        case MetadataValueType::Bool: detail::put_le<uint8_t>(out, v.u ? 1 : 0); break;
        case MetadataValueType::String: write_string(out, v.str); break;
        case MetadataValueType::Uint64: detail::put_le<uint64_t>(out, v.u); break;
        case MetadataValueType::Int64: detail::put_le<int64_t>(out, v.i); break;
        case MetadataValueType::Float64: detail::put_le<double>(out, v.f64); break;
        case MetadataValueType::Array: {
            // element type once (Uint8 for an empty array), the length, then the elements without type codes; a
            // nested array writes its own header the same way
            validate_array_elements(v.arr);
            detail::put_le<uint32_t>(out, v.arr.empty() ? 0u : (uint32_t)v.arr.front().type);
            detail::put_le<uint64_t>(out, v.arr.size());
            for (const MetadataValue &e : v.arr) write_value_data(out, e);
            break;
        }
        }
    }
    static void write_tensor_info(std::vector<uint8_t> &out, const TensorInfo &info) {  // :483-511
        write_string(out, info.name);
        detail::put_le<uint32_t>(out, info.n_dimensions);
        for (auto it = info.dimensions.rbegin(); it != info.dimensions.rend(); ++it) detail::put_le<uint64_t>(out, *it);
        detail::put_le<uint32_t>(out, (uint32_t)info.dtype);
        detail::put_le<uint64_t>(out, info.offset);
    }
    std::vector<TensorInfo> calculate_tensor_offsets() const {  // :514-537
        std::vector<TensorInfo> infos;
        uint64_t offset = 0;
        for (const auto &t : tensors_) {
            TensorInfo info = t.first;
            info.offset = offset;
            infos.push_back(std::move(info));
            const uint64_t len = t.second.size();
            if (offset > UINT64_MAX - len) throw InvalidArgument("GGUF tensor offsets overflow u64");
            if (!detail::align_offset_checked(offset + len, alignment_, offset))
                throw InvalidArgument("GGUF aligned offset overflows u64");
        }
        return infos;
    }
    void pad_to_alignment(std::vector<uint8_t> &out) const {
        uint64_t aligned;
        if (!detail::align_offset_checked(out.size(), alignment_, aligned)) throw InvalidArgument("GGUF aligned offset overflows u64");
        out.resize((size_t)aligned, 0);
    }

    std::map<std::string, MetadataValue> metadata_;
    std::vector<std::pair<TensorInfo, std::vector<uint8_t>>> tensors_;
    uint32_t alignment_ = GGUF_DEFAULT_ALIGNMENT;
};

// reader.rs:80-170
struct GgufReadError : std::runtime_error {
    enum class Kind {
        Io, InvalidMagic, UnsupportedVersion, InvalidValueType, InvalidDtype, InvalidAlignment, TensorNotFound, InvalidUtf8,
        StringTooLarge, ArrayTooLarge, TooManyTensors, TooManyMetadata, TooManyTensorDimensions, DuplicateMetadataKey,
        DuplicateTensorName, ArrayNestingTooDeep, IntegerOverflow,
    };
    Kind kind;
    std::string subject;  // the key / tensor name the error is about, where the reference carries one
    GgufReadError(Kind k, const std::string &msg, std::string subj = std::string())
        : std::runtime_error(msg), kind(k), subject(std::move(subj)) {}
};

// reader.rs:176-444: header, metadata and tensor infos of a GGUF file held in memory; tensor data are ranges of it.
class GgufContent {
   public:
    uint32_t version = 0;  // 1, 2 or 3
    std::unordered_map<std::string, MetadataValue> metadata;
    std::unordered_map<std::string, TensorInfo> tensor_infos;
    std::vector<std::string> tensor_order;  // names in file order (the reference keeps a map only)
    uint64_t tensor_data_offset = 0;

    static GgufContent read(const uint8_t *data, size_t len) {  // :189-333
        Cursor c{data, len, 0};
        GgufContent g;
        const uint32_t magic = c.get<uint32_t>();
        if (magic != GGUF_MAGIC) throw GgufReadError(GgufReadError::Kind::InvalidMagic, "Invalid GGUF magic: expected 0x46554747, got " + hex8(magic));
        g.version = c.get<uint32_t>();
        if (g.version < 1 || g.version > 3)
            throw GgufReadError(GgufReadError::Kind::UnsupportedVersion, "Unsupported GGUF version: " + std::to_string(g.version));
        const bool v1 = g.version == 1;
        const uint64_t tensor_count = v1 ? c.get<uint32_t>() : c.get<uint64_t>();
        const uint64_t kv_count = v1 ? c.get<uint32_t>() : c.get<uint64_t>();
        if (tensor_count > MAX_TENSOR_COUNT)
            throw GgufReadError(GgufReadError::Kind::TooManyTensors, "Too many tensors: " + std::to_string(tensor_count) + " exceeds maximum of " + std::to_string(MAX_TENSOR_COUNT));
        if (kv_count > MAX_METADATA_COUNT)
            throw GgufReadError(GgufReadError::Kind::TooManyMetadata, "Too many metadata entries: " + std::to_string(kv_count) + " exceeds maximum of " + std::to_string(MAX_METADATA_COUNT));
        for (uint64_t k = 0; k < kv_count; k++) {
            std::string key = read_string(c, v1);
            const uint32_t vt = c.get<uint32_t>();
            MetadataValue v = read_value(c, vt, v1, 0);
            if (!g.metadata.emplace(key, std::move(v)).second)
                throw GgufReadError(GgufReadError::Kind::DuplicateMetadataKey, "Duplicate GGUF metadata key: " + key, key);
        }
        for (uint64_t t = 0; t < tensor_count; t++) {
            TensorInfo info;
            info.name = read_string(c, v1);
            info.n_dimensions = c.get<uint32_t>();
            if (info.n_dimensions > MAX_TENSOR_DIMS)
                throw GgufReadError(GgufReadError::Kind::TooManyTensorDimensions,
                                    "Tensor " + info.name + " has " + std::to_string(info.n_dimensions) + " dimensions, exceeding maximum of " + std::to_string(MAX_TENSOR_DIMS), info.name);
            for (uint32_t d = 0; d < info.n_dimensions; d++) info.dimensions.push_back(v1 ? c.get<uint32_t>() : c.get<uint64_t>());
            std::reverse(info.dimensions.begin(), info.dimensions.end());  // fastest axis first on disk, row-major here
            const uint32_t dt = c.get<uint32_t>();
            if (!ggml_type_from_u32(dt, info.dtype)) throw GgufReadError(GgufReadError::Kind::InvalidDtype, "Invalid tensor dtype: " + std::to_string(dt));
            info.offset = c.get<uint64_t>();
            uint64_t bytes;
            if (!info.byte_size_checked(bytes)) throw GgufReadError(GgufReadError::Kind::IntegerOverflow, "Integer overflow in tensor size calculation");
            const std::string name = info.name;
            if (!g.tensor_infos.emplace(name, std::move(info)).second)
                throw GgufReadError(GgufReadError::Kind::DuplicateTensorName, "Duplicate GGUF tensor name: " + name, name);
            g.tensor_order.push_back(name);
        }
        uint64_t alignment = GGUF_DEFAULT_ALIGNMENT;  // :305-312: general.alignment as u32 or u64, else the default
        const auto a = g.metadata.find(keys::GENERAL_ALIGNMENT);
        if (a != g.metadata.end() && (a->second.type == MetadataValueType::Uint32 || a->second.type == MetadataValueType::Uint64))
            alignment = a->second.u;
        if (alignment == 0 || alignment > 1048576)
            throw GgufReadError(GgufReadError::Kind::InvalidAlignment, "Invalid alignment: " + std::to_string(alignment) + " (must be 1..=1048576)");
        if (!detail::align_offset_checked(c.pos, alignment, g.tensor_data_offset))
            throw GgufReadError(GgufReadError::Kind::IntegerOverflow, "Integer overflow in tensor size calculation");
        return g;
    }
    static GgufContent read(const std::vector<uint8_t> &bytes) { return read(bytes.data(), bytes.size()); }
    // from_file (:336-340): header, metadata and tensor infos of a file; the tensor data stay on disk.  The header part
    // is read in growing pieces, so a multi-gigabyte model costs a few megabytes here.
    static GgufContent from_file(const std::string &path) {
        std::ifstream f(path, std::ios::binary);
        if (!f) throw GgufReadError(GgufReadError::Kind::Io, "IO error: cannot open " + path);
        f.seekg(0, std::ios::end);
        const uint64_t size = (uint64_t)f.tellg();
        std::vector<uint8_t> head;
        for (uint64_t want = 1u << 20;; want *= 4) {
            const uint64_t take = want < size ? want : size;
            head.resize((size_t)take);
            f.seekg(0);
            f.read(reinterpret_cast<char *>(head.data()), (std::streamsize)take);
            if (!f) throw GgufReadError(GgufReadError::Kind::Io, "IO error: read of " + path + " failed");
            try {
                return read(head.data(), head.size());
            } catch (const GgufReadError &e) {
                if (e.kind != GgufReadError::Kind::Io || take == size) throw;
            }
        }
    }
    // read_tensor_data (:371-407) from the file itself
    std::vector<uint8_t> read_tensor_data_from_file(const std::string &path, const std::string &name) const {
        const TensorInfo *info = get_tensor_info(name);
        if (!info) throw GgufReadError(GgufReadError::Kind::TensorNotFound, "Tensor not found: " + name, name);
        uint64_t bytes;
        if (!info->byte_size_checked(bytes) || tensor_data_offset > UINT64_MAX - info->offset)
            throw GgufReadError(GgufReadError::Kind::IntegerOverflow, "Integer overflow in tensor size calculation");
        std::ifstream f(path, std::ios::binary);
        if (!f) throw GgufReadError(GgufReadError::Kind::Io, "IO error: cannot open " + path);
        std::vector<uint8_t> out((size_t)bytes);
        f.seekg((std::streamoff)(tensor_data_offset + info->offset));
        f.read(reinterpret_cast<char *>(out.data()), (std::streamsize)bytes);
        if (!f) throw GgufReadError(GgufReadError::Kind::Io, "IO error: failed to fill whole buffer");
        return out;
    }

    const MetadataValue *get_metadata(const std::string &key) const {
        const auto it = metadata.find(key);
        return it == metadata.end() ? nullptr : &it->second;
    }
    const TensorInfo *get_tensor_info(const std::string &name) const {
        const auto it = tensor_infos.find(name);
        return it == tensor_infos.end() ? nullptr : &it->second;
    }
    const std::string *architecture() const {
        const MetadataValue *v = get_metadata(keys::GENERAL_ARCHITECTURE);
        return v && v->type == MetadataValueType::String ? &v->str : nullptr;
    }
    size_t num_tensors() const { return tensor_infos.size(); }

    // read_tensor_data (:371-407): the bytes of one tensor out of the file image
    std::vector<uint8_t> read_tensor_data(const uint8_t *file, size_t file_len, const std::string &name) const {
        const TensorInfo *info = get_tensor_info(name);
        if (!info) throw GgufReadError(GgufReadError::Kind::TensorNotFound, "Tensor not found: " + name, name);
        uint64_t bytes;
        if (!info->byte_size_checked(bytes)) throw GgufReadError(GgufReadError::Kind::IntegerOverflow, "Integer overflow in tensor size calculation");
        if (tensor_data_offset > UINT64_MAX - info->offset || tensor_data_offset + info->offset > UINT64_MAX - bytes)
            throw GgufReadError(GgufReadError::Kind::IntegerOverflow, "Integer overflow in tensor size calculation");
        const uint64_t begin = tensor_data_offset + info->offset;
        if (begin + bytes > file_len) throw GgufReadError(GgufReadError::Kind::Io, "IO error: failed to fill whole buffer");
        return std::vector<uint8_t>(file + begin, file + begin + bytes);
    }
    std::vector<uint8_t> read_tensor_data(const std::vector<uint8_t> &file, const std::string &name) const {
        return read_tensor_data(file.data(), file.size(), name);
    }

   private:
    struct Cursor {
        const uint8_t *p;
        size_t len, pos;
        void need(size_t n) const {
            if (n > len - pos) throw GgufReadError(GgufReadError::Kind::Io, "IO error: failed to fill whole buffer");
        }
        template <typename T>
        T get() {
            need(sizeof(T));
            T v;
            std::memcpy(&v, p + pos, sizeof(T));
            pos += sizeof(T);
            return v;
        }
    };
    static std::string hex8(uint32_t v) {
        char b[16];
        std::snprintf(b, sizeof b, "0x%08X", v);
        return b;
    }
    static bool valid_utf8(const std::string &s) {
        const unsigned char *p = reinterpret_cast<const unsigned char *>(s.data());
        size_t i = 0, n = s.size();
        while (i < n) {
            const unsigned char c = p[i];
            size_t extra;
            uint32_t cp;
            if (c < 0x80) { i++; continue; }
            if (c >= 0xC2 && c <= 0xDF) extra = 1, cp = c & 0x1F;
            else if (c >= 0xE0 && c <= 0xEF) extra = 2, cp = c & 0x0F;
            else if (c >= 0xF0 && c <= 0xF4) extra = 3, cp = c & 0x07;
            else return false;
            if (i + extra >= n) return false;
            for (size_t k = 1; k <= extra; k++) {
                if ((p[i + k] & 0xC0) != 0x80) return false;
                cp = (cp << 6) | (p[i + k] & 0x3F);
            }
            if ((extra == 2 && (cp < 0x800 || (cp >= 0xD800 && cp <= 0xDFFF))) || (extra == 3 && (cp < 0x10000 || cp > 0x10FFFF))) return false;
            i += extra + 1;
        }
        return true;
    }
    static std::string read_string(Cursor &c, bool v1) {  // :446-479
        const uint64_t len = v1 ? c.get<uint32_t>() : c.get<uint64_t>();
        if (len > MAX_STRING_LENGTH)
            throw GgufReadError(GgufReadError::Kind::StringTooLarge, "String too large: " + std::to_string(len) + " bytes exceeds maximum of " + std::to_string(MAX_STRING_LENGTH) + " bytes");
        c.need((size_t)len);
        std::string s(reinterpret_cast<const char *>(c.p + c.pos), (size_t)len);
        c.pos += (size_t)len;
        while (!s.empty() && s.back() == '\0') s.pop_back();  // some files carry trailing nulls
        if (!valid_utf8(s)) throw GgufReadError(GgufReadError::Kind::InvalidUtf8, "Invalid UTF-8 in string");
        return s;
    }
    static MetadataValue read_value(Cursor &c, uint32_t vt, bool v1, uint8_t depth) {  // :493-560
        switch (vt) {
        case 0: return MetadataValue::Uint8(c.get<uint8_t>());
        case 1: return MetadataValue::Int8(c.get<int8_t>());
        case 2: return MetadataValue::Uint16(c.get<uint16_t>());
        case 3: return MetadataValue::Int16(c.get<int16_t>());
        case 4: return MetadataValue::Uint32(c.get<uint32_t>());
        case 5: return MetadataValue::Int32(c.get<int32_t>());
        case 6: return MetadataValue::Float32(c.get<float>());
        case 7: return MetadataValue::Bool(c.get<uint8_t>() != 0);
        case 8: return MetadataValue::String(read_string(c, v1));
        case 9: {
            if (depth >= MAX_ARRAY_DEPTH)
                throw GgufReadError(GgufReadError::Kind::ArrayNestingTooDeep, "Metadata array nesting depth exceeded limit of " + std::to_string(MAX_ARRAY_DEPTH));
            const uint32_t et = c.get<uint32_t>();
            const uint64_t len = v1 ? c.get<uint32_t>() : c.get<uint64_t>();
            if (len > MAX_ARRAY_LENGTH)
                throw GgufReadError(GgufReadError::Kind::ArrayTooLarge, "Array too large: " + std::to_string(len) + " elements exceeds maximum of " + std::to_string(MAX_ARRAY_LENGTH) + " elements");
            std::vector<MetadataValue> elems;
            elems.reserve((size_t)len);
            for (uint64_t k = 0; k < len; k++) elems.push_back(read_value(c, et, v1, (uint8_t)(depth + 1)));
            return MetadataValue::Array(std::move(elems));
        }
        case 10: return MetadataValue::Uint64(c.get<uint64_t>());
        case 11: return MetadataValue::Int64(c.get<int64_t>());
        case 12: return MetadataValue::Float64(c.get<double>());
        default: throw GgufReadError(GgufReadError::Kind::InvalidValueType, "Invalid metadata value type: " + std::to_string(vt));
        }
    }
};

}  // namespace pmetal_gguf
