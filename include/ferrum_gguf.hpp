// ferrum_gguf.hpp -- bounds-checked GGUF v2/v3 index and tensor reads (C++17,
// header only), and the hand-over of K-quant tensors to the device.
//
// Mirrors GgufReader of the reference (src/loader/gguf.rs:162-530): the block
// table of block_layout (:91-121), the descriptor limits (:9-21), alignment
// from general.alignment (default 32), the validation order of
// GgufReader::read (:197-391), logical_matrix_shape / logical_expert_shape
// (:133-157), read_tensor_into (:474-493), stream_tensor (:498-529) and
// tensors_equal_payload (:419-441).  Every failure is ferrum::Error of kind
// Gguf.  load_quantized_matrix / load_quantized_expert_matrix pass the packed
// blocks to Device::quantized_matrix unchanged (src/quantization.rs:86-111).
#ifndef FERRUM_GGUF_HPP
#define FERRUM_GGUF_HPP

#include <algorithm>
#include <array>
#include <fstream>
#include <istream>
#include <map>
#include <sstream>
#include <variant>

#include "ferrum_hip.hpp"

namespace ferrum {
namespace gguf {

constexpr uint64_t kMaxTensors = 1000000, kMaxMetadata = 1000000, kMaxArrayItems = 4000000;
constexpr uint64_t kMaxStringBytes = 16ull * 1024 * 1024;
constexpr size_t kMaxTensorNameBytes = 64, kMaxUntaggedTensorNameBytes = 256;

[[noreturn]] inline void fail(const std::string& message) { throw Error(ErrorKind::Gguf, message); }

struct BlockLayout {
    size_t elements, bytes;
    bool operator==(const BlockLayout& o) const { return elements == o.elements && bytes == o.bytes; }
};

inline BlockLayout block_layout(uint32_t type_id) {
    switch (type_id) {
        case 0: return {1, 4};        // F32
        case 1: return {1, 2};        // F16
        case 30: return {1, 2};       // BF16
        case 2: return {32, 18};      // Q4_0
        case 3: return {32, 20};      // Q4_1
        case 6: return {32, 22};      // Q5_0
        case 7: return {32, 24};      // Q5_1
        case 8: return {32, 34};      // Q8_0
        case 9: return {32, 36};      // Q8_1
        case 10: return {256, 84};    // Q2_K
        case 11: return {256, 110};   // Q3_K
        case 12: return {256, 144};   // Q4_K
        case 13: return {256, 176};   // Q5_K
        case 14: return {256, 210};   // Q6_K
        case 15: return {256, 292};   // Q8_K
        case 18: return {256, 98};    // IQ3_XXS
        case 20: return {32, 18};     // IQ4_NL
        case 21: return {256, 110};   // IQ3_S
        case 22: return {256, 82};    // IQ2_S
        case 23: return {256, 136};   // IQ4_XS
        case 42: return {64, 18};
        default: fail("unsupported GGML tensor type " + std::to_string(type_id));
    }
}

enum class MetadataType : uint32_t {
    Uint8 = 0, Int8, Uint16, Int16, Uint32, Int32, Float32, Bool, String, Array, Uint64, Int64, Float64
};

struct MetadataValue;
struct MetadataArray {
    MetadataType element_type;
    std::vector<MetadataValue> values;   // empty when the array was skipped
};
struct MetadataValue {
    MetadataType type;
    std::variant<uint64_t, int64_t, double, bool, std::string, MetadataArray> value;
    uint64_t as_u64() const { return std::get<uint64_t>(value); }
    int64_t as_i64() const { return std::get<int64_t>(value); }
    double as_f64() const { return std::get<double>(value); }
    bool as_bool() const { return std::get<bool>(value); }
    const std::string& as_string() const { return std::get<std::string>(value); }
    const MetadataArray& as_array() const { return std::get<MetadataArray>(value); }
};

struct TensorInfo {
    std::string name;
    std::vector<uint64_t> dimensions;   // GGUF order: dimension zero is contiguous
    uint32_t type_id = 0;
    uint64_t offset = 0;                // relative to the aligned tensor-data section
    size_t byte_len = 0;

    std::array<size_t, 2> logical_matrix_shape() const {
        if (dimensions.size() != 2)
            fail("tensor " + name + " is rank " + std::to_string(dimensions.size()) + ", expected a matrix");
        return {(size_t)dimensions[1], (size_t)dimensions[0]};
    }
    std::array<size_t, 3> logical_expert_shape() const {
        if (dimensions.size() != 3)
            fail("tensor " + name + " is rank " + std::to_string(dimensions.size()) + ", expected an expert matrix");
        return {(size_t)dimensions[2], (size_t)dimensions[1], (size_t)dimensions[0]};
    }
};

class Reader {
public:
    // The stream must be seekable and outlive the reader.
    explicit Reader(std::istream& stream, uint64_t max_array_items = UINT64_MAX, bool require_architecture = true)
        : in_(&stream) {
        parse(max_array_items, require_architecture);
    }
    static Reader open(const std::string& path, uint64_t max_array_items = UINT64_MAX,
                       bool require_architecture = true) {
        auto file = std::make_unique<std::ifstream>(path, std::ios::binary);
        if (!*file) fail("open " + path + ": cannot read the file");
        return Reader(std::move(file), max_array_items, require_architecture);
    }

    uint32_t version() const { return version_; }
    uint64_t alignment() const { return alignment_; }
    uint64_t tensor_data_offset() const { return tensor_data_offset_; }
    const std::map<std::string, MetadataValue>& metadata() const { return metadata_; }
    const std::map<std::string, TensorInfo>& tensors() const { return tensors_; }
    const MetadataValue* metadata_value(const std::string& key) const {
        auto it = metadata_.find(key);
        return it == metadata_.end() ? nullptr : &it->second;
    }
    const TensorInfo& tensor(const std::string& name) const {
        auto it = tensors_.find(name);
        if (it == tensors_.end()) fail("missing tensor " + name);
        return it->second;
    }

    void read_tensor_into(const std::string& name, uint8_t* destination, size_t length) {
        const TensorInfo& t = tensor(name);
        if (length != t.byte_len)
            fail("tensor " + name + " has " + std::to_string(t.byte_len) + " bytes, destination has " +
                 std::to_string(length));
        read_range(t, 0, destination, length);
    }
    void stream_tensor(const std::string& name, size_t chunk_bytes,
                       const std::function<void(const uint8_t*, size_t)>& consume) {
        if (chunk_bytes == 0) fail("tensor stream chunk size must be positive");
        const TensorInfo& t = tensor(name);
        std::vector<uint8_t> scratch(std::min(chunk_bytes, t.byte_len));
        for (size_t done = 0; done < t.byte_len;) {
            const size_t length = std::min(scratch.size(), t.byte_len - done);
            read_range(t, done, scratch.data(), length);
            consume(scratch.data(), length);
            done += length;
        }
    }
    bool tensors_equal_payload(const std::string& left, const std::string& right) {
        const TensorInfo &a = tensor(left), &b = tensor(right);
        if (a.dimensions != b.dimensions || a.type_id != b.type_id || a.byte_len != b.byte_len) return false;
        std::vector<uint8_t> x(256 * 1024), y(256 * 1024);
        for (size_t done = 0; done < a.byte_len;) {
            const size_t length = std::min(x.size(), a.byte_len - done);
            read_range(a, done, x.data(), length);
            read_range(b, done, y.data(), length);
            if (!std::equal(x.begin(), x.begin() + length, y.begin())) return false;
            done += length;
        }
        return true;
    }

private:
    Reader(std::unique_ptr<std::istream> owned, uint64_t max_array_items, bool require_architecture)
        : owned_(std::move(owned)), in_(owned_.get()) {
        parse(max_array_items, require_architecture);
    }

    void take(void* out, size_t n, const char* what) {
        in_->read(static_cast<char*>(out), (std::streamsize)n);
        if ((size_t)in_->gcount() != n) fail(std::string("unexpected end of file while reading ") + what);
    }
    template <class T> T scalar(const char* what) {
        T v;
        take(&v, sizeof v, what);   // GGUF and gfx950 hosts are both little-endian
        return v;
    }
    std::string string(const char* what) {
        const uint64_t n = scalar<uint64_t>(what);
        if (n > kMaxStringBytes || n > file_len_) fail(std::string(what) + " length " + std::to_string(n) + " is unreasonable");
        std::string s(n, '\0');
        take(s.data(), n, what);
        for (size_t i = 0; i < s.size();) {   // well-formed UTF-8, as String::from_utf8 requires
            const unsigned char c = (unsigned char)s[i];
            const int extra = c < 0x80 ? 0 : (c >> 5) == 6 ? 1 : (c >> 4) == 14 ? 2 : (c >> 3) == 30 ? 3 : -1;
            if (extra < 0 || i + extra >= s.size() + (extra == 0)) fail(std::string(what) + " is not valid UTF-8");
            for (int j = 1; j <= extra; ++j)
                if (((unsigned char)s[i + j] >> 6) != 2) fail(std::string(what) + " is not valid UTF-8");
            i += extra + 1;
        }
        return s;
    }
    static MetadataType metadata_type(uint32_t id) {
        if (id > 12) fail("unsupported metadata type " + std::to_string(id));
        return static_cast<MetadataType>(id);
    }
    MetadataValue value(MetadataType type, uint64_t max_items) {
        switch (type) {
            case MetadataType::Uint8: return {type, (uint64_t)scalar<uint8_t>("uint8 metadata")};
            case MetadataType::Int8: return {type, (int64_t)scalar<int8_t>("int8 metadata")};
            case MetadataType::Uint16: return {type, (uint64_t)scalar<uint16_t>("uint16 metadata")};
            case MetadataType::Int16: return {type, (int64_t)scalar<int16_t>("int16 metadata")};
            case MetadataType::Uint32: return {type, (uint64_t)scalar<uint32_t>("uint32 metadata")};
            case MetadataType::Int32: return {type, (int64_t)scalar<int32_t>("int32 metadata")};
            case MetadataType::Float32: return {type, (double)scalar<float>("float32 metadata")};
            case MetadataType::Uint64: return {type, scalar<uint64_t>("uint64 metadata")};
            case MetadataType::Int64: return {type, scalar<int64_t>("int64 metadata")};
            case MetadataType::Float64: return {type, scalar<double>("float64 metadata")};
            case MetadataType::Bool: {
                const int8_t v = scalar<int8_t>("bool metadata");
                if (v != 0 && v != 1) fail("invalid bool value " + std::to_string(v));
                return {type, v == 1};
            }
            case MetadataType::String: return {type, string("string metadata")};
            case MetadataType::Array: {
                const MetadataType element = metadata_type(scalar<uint32_t>("array element type"));
                if (element == MetadataType::Array) fail("nested metadata arrays are unsupported");
                const uint64_t count = scalar<uint64_t>("array element count");
                if (count > kMaxArrayItems || count > file_len_)
                    fail("unreasonable metadata array length " + std::to_string(count));
                MetadataArray array{element, {}};
                const bool keep = count <= max_items;
                if (keep) array.values.reserve(count);
                for (uint64_t i = 0; i < count; ++i) {
                    MetadataValue v = value(element, UINT64_MAX);
                    if (keep) array.values.push_back(std::move(v));
                }
                return {type, std::move(array)};
            }
        }
        fail("unsupported metadata type");
    }

    void parse(uint64_t max_array_items, bool require_architecture) {
        in_->seekg(0, std::ios::end);
        file_len_ = (uint64_t)in_->tellg();
        in_->seekg(0);
        char magic[4];
        take(magic, 4, "magic");
        if (std::memcmp(magic, "GGUF", 4) != 0) fail("invalid magic; expected GGUF");
        version_ = scalar<uint32_t>("version");
        if (version_ != 2 && version_ != 3) fail("unsupported version " + std::to_string(version_));
        const uint64_t tensor_count = scalar<uint64_t>("tensor count");
        const uint64_t metadata_count = scalar<uint64_t>("metadata count");
        if (tensor_count > kMaxTensors || metadata_count > kMaxMetadata)
            fail("unreasonable descriptor counts: " + std::to_string(tensor_count) + " tensors, " +
                 std::to_string(metadata_count) + " metadata entries");

        for (uint64_t i = 0; i < metadata_count; ++i) {
            std::string key = string("metadata key");
            MetadataValue v = value(metadata_type(scalar<uint32_t>("metadata value type")), max_array_items);
            if (!metadata_.emplace(key, std::move(v)).second) fail("duplicate metadata key " + key);
        }
        alignment_ = 32;
        if (const MetadataValue* a = metadata_value("general.alignment")) {
            if (a->type != MetadataType::Uint32) fail("general.alignment must have uint32 type");
            alignment_ = a->as_u64();
        }
        if (alignment_ < 8 || alignment_ % 8)
            fail("general.alignment must be a positive multiple of 8, got " + std::to_string(alignment_));
        if (require_architecture) {
            const MetadataValue* arch = metadata_value("general.architecture");
            if (!arch || arch->type != MetadataType::String) fail("missing or invalid general.architecture metadata");
        }

        bool quantized = false;
        const size_t max_name = require_architecture ? kMaxTensorNameBytes : kMaxUntaggedTensorNameBytes;
        for (uint64_t i = 0; i < tensor_count; ++i) {
            TensorInfo t;
            t.name = string("tensor name");
            if (t.name.size() > max_name) fail("tensor name exceeds " + std::to_string(max_name) + " bytes");
            const uint32_t rank = scalar<uint32_t>("tensor rank");
            if (rank < 1 || rank > 4) fail("tensor " + t.name + " has unsupported rank " + std::to_string(rank));
            uint64_t elements = 1;
            for (uint32_t r = 0; r < rank; ++r) {
                const uint64_t dim = scalar<uint64_t>("tensor dimension");
                if (dim == 0) fail("tensor " + t.name + " has an empty dimension");
                if (elements > (UINT64_MAX >> 1) / dim) fail("tensor " + t.name + " element count overflow");
                elements *= dim;
                t.dimensions.push_back(dim);
            }
            t.type_id = scalar<uint32_t>("tensor type");
            t.offset = scalar<uint64_t>("tensor data offset");
            BlockLayout layout{};
            try {
                layout = block_layout(t.type_id);
            } catch (const Error& e) {
                fail("tensor " + t.name + ": " + e.what());
            }
            if (t.dimensions[0] % layout.elements)
                fail("tensor " + t.name + " fastest dimension " + std::to_string(t.dimensions[0]) +
                     " is not divisible by block size " + std::to_string(layout.elements) + " for type " +
                     std::to_string(t.type_id));
            const uint64_t blocks = elements / layout.elements;
            if (blocks > (UINT64_MAX >> 1) / layout.bytes) fail("tensor " + t.name + " byte length overflow");
            t.byte_len = (size_t)(blocks * layout.bytes);
            if (t.offset % alignment_)
                fail("tensor " + t.name + " offset " + std::to_string(t.offset) + " is not aligned to " +
                     std::to_string(alignment_));
            quantized |= !(t.type_id == 0 || t.type_id == 1 || t.type_id == 30);
            std::string name = t.name;
            if (!tensors_.emplace(name, std::move(t)).second) fail("duplicate tensor name " + name);
        }

        const uint64_t end = (uint64_t)in_->tellg();
        tensor_data_offset_ = (end + alignment_ - 1) / alignment_ * alignment_;
        struct Range { uint64_t start, stop; const std::string* name; };
        std::vector<Range> ranges;
        for (const auto& [name, t] : tensors_) {
            if (t.offset > UINT64_MAX - tensor_data_offset_ || t.byte_len > UINT64_MAX - tensor_data_offset_ - t.offset)
                fail("tensor " + name + " range overflow");
            const uint64_t start = tensor_data_offset_ + t.offset, stop = start + t.byte_len;
            if (stop > file_len_)
                fail("tensor " + name + " range " + std::to_string(start) + ".." + std::to_string(stop) +
                     " exceeds file length " + std::to_string(file_len_));
            ranges.push_back({start, stop, &name});
        }
        std::sort(ranges.begin(), ranges.end(), [](const Range& a, const Range& b) { return a.start < b.start; });
        for (size_t i = 1; i < ranges.size(); ++i)
            if (ranges[i - 1].stop > ranges[i].start)
                fail("tensor ranges overlap: " + *ranges[i - 1].name + " and " + *ranges[i].name);
        if (require_architecture && quantized) {
            const MetadataValue* v = metadata_value("general.quantization_version");
            if (!v || v->type != MetadataType::Uint32)
                fail("quantized tensor file is missing uint32 general.quantization_version");
        }
    }

    void read_range(const TensorInfo& t, size_t relative, uint8_t* out, size_t length) {
        if (relative > t.byte_len || length > t.byte_len - relative) fail("tensor " + t.name + " range exceeds payload");
        in_->clear();
        in_->seekg((std::streamoff)(tensor_data_offset_ + t.offset + relative));
        in_->read(reinterpret_cast<char*>(out), (std::streamsize)length);
        if ((size_t)in_->gcount() != length) fail("read tensor " + t.name + ": short read");
    }

    std::unique_ptr<std::istream> owned_;
    std::istream* in_ = nullptr;
    uint64_t file_len_ = 0, alignment_ = 32, tensor_data_offset_ = 0;
    uint32_t version_ = 0;
    std::map<std::string, MetadataValue> metadata_;
    std::map<std::string, TensorInfo> tensors_;
};

// A rank-2 Q4_K / Q6_K tensor as a device matrix of [dims[1], dims[0]].
inline QuantizedMatrix load_quantized_matrix(const Device& device, Reader& reader, const std::string& name) {
    const TensorInfo& t = reader.tensor(name);
    const auto shape = t.logical_matrix_shape();
    return device.quantized_matrix(shape[0], shape[1], format_from_ggml_type(t.type_id),
                                   [&](uint8_t* dst, size_t n) { reader.read_tensor_into(name, dst, n); });
}

// A rank-3 tensor as [experts, rows, columns] = [dims[2], dims[1], dims[0]].
inline QuantizedExpertMatrix load_quantized_expert_matrix(const Device& device, Reader& reader,
                                                          const std::string& name) {
    const TensorInfo& t = reader.tensor(name);
    const auto shape = t.logical_expert_shape();
    return device.quantized_expert_matrix(shape[0], shape[1], shape[2], format_from_ggml_type(t.type_id),
                                          [&](uint8_t* dst, size_t n) { reader.read_tensor_into(name, dst, n); });
}

// The gate and up expert tensors ([experts, I, H] each) interleaved per expert into
// [experts, 2I, H] rows, gate first, streamed 64 rows at a time
// (load_quantized_input_experts, src/model/lfm2_moe/gguf.rs:466-534).
inline void read_stacked_experts(Reader& reader, const std::string& gate_name, const std::string& up_name,
                                 uint8_t* destination, size_t length) {
    const TensorInfo gate = reader.tensor(gate_name), up = reader.tensor(up_name);
    const auto shape = gate.logical_expert_shape();
    if (up.logical_expert_shape() != shape || up.type_id != gate.type_id)
        throw Error(ErrorKind::Weight, up_name + ": gate and up expert tensors differ in shape or type");
    const QuantizationFormat format = format_from_ggml_type(gate.type_id);
    const size_t experts = shape[0], intermediate = shape[1], hidden = shape[2];
    const size_t row_bytes = hidden / block_elements(format) * block_bytes(format);
    const size_t component_bytes = experts * intermediate * row_bytes;
    if (length != 2 * component_bytes) fail("stacked expert destination has " + std::to_string(length) + " bytes");
    const std::string* names[2] = {&gate_name, &up_name};
    for (size_t component = 0; component < 2; ++component) {
        const std::string& name = *names[component];
        if (reader.tensor(name).byte_len != component_bytes)
            throw Error(ErrorKind::Weight, name + ": expected " + std::to_string(component_bytes) + " packed expert bytes");
        size_t written = 0;
        reader.stream_tensor(name, row_bytes * 64, [&](const uint8_t* chunk, size_t n) {
            if (n % row_bytes) fail("tensor " + name + " stream ended inside an expert row");
            for (size_t i = 0; i < n / row_bytes; ++i) {
                const size_t source_row = written / row_bytes + i;
                const size_t expert = source_row / intermediate, within = source_row % intermediate;
                if (expert >= experts) fail("tensor " + name + " contains too many expert rows");
                std::memcpy(destination + ((expert * 2 + component) * intermediate + within) * row_bytes,
                            chunk + i * row_bytes, row_bytes);
            }
            written += n;
        });
        if (written != component_bytes)
            fail("tensor " + name + " streamed " + std::to_string(written) + " bytes, expected " +
                 std::to_string(component_bytes));
    }
}

inline QuantizedExpertMatrix load_quantized_input_experts(const Device& device, Reader& reader,
                                                          const std::string& gate_name, const std::string& up_name) {
    const TensorInfo& gate = reader.tensor(gate_name);
    const auto shape = gate.logical_expert_shape();
    return device.quantized_expert_matrix(shape[0], 2 * shape[1], shape[2], format_from_ggml_type(gate.type_id),
                                          [&](uint8_t* dst, size_t n) { read_stacked_experts(reader, gate_name, up_name, dst, n); });
}

}  // namespace gguf
}  // namespace ferrum

#endif  // FERRUM_GGUF_HPP
