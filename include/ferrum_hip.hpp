// ferrum_hip.hpp -- C++17 host side over the C ABI of ferrum_hip.h.
//
// It mirrors the operator interface of the reference's device type for the
// quantized-matmul path: the same names, argument meaning and error variants
// as MetalDevice::project_quantized (src/ops/transformer.rs:96-297), the
// routed-expert operators (src/ops/mod.rs:23-551), QuantizedMatrix /
// QuantizedExpertMatrix (src/quantization.rs:76-194), Tensor and DType
// (src/tensor/mod.rs), Execution (src/metal/mod.rs:263-278) and
// SparseMoe::forward (src/nn/moe.rs:222-390).  Header only; link
// libferrum_hip.so.  Errors are thrown as ferrum::Error carrying the variant
// of src/error.rs:3-51.  Like the reference's Rc handles, nothing here is
// thread-safe.
#ifndef FERRUM_HIP_HPP
#define FERRUM_HIP_HPP

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "ferrum_hip.h"

namespace ferrum {

enum class ErrorKind {
    Shape = FH_ERR_SHAPE, DType = FH_ERR_DTYPE, DeviceMismatch = FH_ERR_DEVICE_MISMATCH,
    Range = FH_ERR_RANGE, Dispatch = FH_ERR_DISPATCH, Synchronization = FH_ERR_SYNCHRONIZATION,
    Allocation = FH_ERR_ALLOCATION, Gguf = FH_ERR_GGUF, Weight = FH_ERR_WEIGHT,
    Parameter = FH_ERR_PARAMETER, Token = FH_ERR_TOKEN, Validation = FH_ERR_VALIDATION,
    Config = 100  // host-side only
};

class Error : public std::runtime_error {
public:
    Error(ErrorKind kind, const std::string& message) : std::runtime_error(message), kind_(kind) {}
    ErrorKind kind() const { return kind_; }
private:
    ErrorKind kind_;
};

inline void check(fh_status status) {
    if (status != FH_OK) throw Error(static_cast<ErrorKind>(status), fh_last_error());
}

enum class DType : uint32_t { F32 = FH_F32, F16 = FH_F16, BF16 = FH_BF16 };
inline size_t size_bytes(DType d) { return d == DType::F32 ? 4 : 2; }

// ---- storage rounding, as DType::round / Tensor::from_f32 (src/tensor/mod.rs:19-25) ----
inline uint16_t f32_to_bf16_bits(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
inline float bf16_bits_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float v;
    std::memcpy(&v, &u, 4);
    return v;
}
inline uint16_t f32_to_f16_bits(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    u &= 0x7fffffffu;
    if (u > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((u >> 13) & 0x1ffu));
    if (u >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);  // >= 65536 (or inf)
    if (u < 0x33000001u) return (uint16_t)sign;                // rounds to zero
    int32_t exp = (int32_t)(u >> 23) - 127;
    uint32_t man = (u & 0x7fffffu) | 0x800000u;
    int shift = exp < -14 ? 13 + (-14 - exp) : 13;              // subnormal results lose more bits
    uint32_t half = man >> shift, rest = man & ((1u << shift) - 1), mid = 1u << (shift - 1);
    if (rest > mid || (rest == mid && (half & 1u))) ++half;
    uint32_t bits = exp < -14 ? half : ((uint32_t)(exp + 15) << 10) + (half - 0x400u);
    if (bits >= 0x7c00u) bits = 0x7c00u;
    return (uint16_t)(sign | bits);
}
inline float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 0x3ffu;
    float v;
    if (exp == 0) {
        v = std::ldexp((float)man, -24);
    } else if (exp == 31) {
        uint32_t u = 0x7f800000u | (man << 13);
        std::memcpy(&v, &u, 4);
    } else {
        v = std::ldexp((float)(man | 0x400u), (int)exp - 25);
    }
    uint32_t u;
    std::memcpy(&u, &v, 4);
    u |= sign;
    std::memcpy(&v, &u, 4);
    return v;
}

// IQ4_XS and Q8_0 are the hybrid engine's Format::Iq4Xs / Format::Q8_0 (src/hybrid/weights.rs:29-60).
// A row is a whole number of blocks: 256 weights, or for Q8_0 the 32 weights of a 34-byte GGML block
// (src/loader/gguf.rs:99).
enum class QuantizationFormat : uint32_t {
    Q8_0 = FH_GGML_Q8_0, Q4_K = FH_GGML_Q4_K, Q5_K = FH_GGML_Q5_K, Q6_K = FH_GGML_Q6_K, IQ4_XS = FH_GGML_IQ4_XS
};
inline size_t block_elements(QuantizationFormat f) { return f == QuantizationFormat::Q8_0 ? 32 : 256; }
inline size_t block_bytes(QuantizationFormat f) {
    switch (f) {
        case QuantizationFormat::Q8_0: return 34;
        case QuantizationFormat::Q4_K: return 144;
        case QuantizationFormat::Q5_K: return 176;
        case QuantizationFormat::Q6_K: return 210;
        case QuantizationFormat::IQ4_XS: return 136;
    }
    return 0;
}
inline QuantizationFormat format_from_ggml_type(uint32_t id) {
    if (id == FH_GGML_Q4_K) return QuantizationFormat::Q4_K;
    if (id == FH_GGML_Q5_K) return QuantizationFormat::Q5_K;
    if (id == FH_GGML_Q6_K) return QuantizationFormat::Q6_K;
    if (id == FH_GGML_IQ4_XS) return QuantizationFormat::IQ4_XS;
    if (id == FH_GGML_Q8_0) return QuantizationFormat::Q8_0;
    throw Error(ErrorKind::Gguf, "unsupported GGML type " + std::to_string(id));
}

class Device;

namespace detail {
struct DeviceHandle {
    fh_device* raw = nullptr;
    ~DeviceHandle() { if (raw) fh_device_destroy(raw); }
};
struct BufferHandle {
    fh_buffer* raw = nullptr;
    std::shared_ptr<DeviceHandle> owner;
    size_t bytes = 0;
    ~BufferHandle() { if (raw) fh_buffer_free(raw); }
};
struct MatrixHandle {
    fh_qmatrix* raw = nullptr;
    std::shared_ptr<DeviceHandle> owner;
    ~MatrixHandle() { if (raw) fh_qmatrix_destroy(raw); }
};
}  // namespace detail

// A dense row-major view into a device buffer (src/tensor/mod.rs).
class Tensor {
public:
    Tensor() = default;
    const std::vector<size_t>& shape() const { return shape_; }
    DType dtype() const { return dtype_; }
    size_t numel() const {
        size_t n = 1;
        for (size_t d : shape_) n *= d;
        return n;
    }
    size_t byte_size() const { return numel() * size_bytes(dtype_); }
    Tensor view(size_t element_offset, std::vector<size_t> shape) const {
        Tensor t = *this;
        t.shape_ = std::move(shape);
        t.offset_ = offset_ + element_offset * size_bytes(dtype_);
        if (t.offset_ + t.byte_size() > buffer_->bytes) throw Error(ErrorKind::Range, "tensor view is out of range");
        return t;
    }
    // Waits for the device, then widens to f32.
    std::vector<float> to_f32() const {
        const size_t n = numel();
        std::vector<float> out(n);
        if (dtype_ == DType::F32) {
            check(fh_buffer_download(buffer_->raw, offset_, out.data(), n * 4));
            return out;
        }
        std::vector<uint16_t> raw(n);
        check(fh_buffer_download(buffer_->raw, offset_, raw.data(), n * 2));
        for (size_t i = 0; i < n; ++i)
            out[i] = dtype_ == DType::F16 ? f16_bits_to_f32(raw[i]) : bf16_bits_to_f32(raw[i]);
        return out;
    }
    fh_view c_view() const { return fh_view{buffer_->raw, offset_, static_cast<uint32_t>(dtype_)}; }
    const std::shared_ptr<detail::DeviceHandle>& owner() const { return buffer_->owner; }

private:
    friend class Device;
    std::shared_ptr<detail::BufferHandle> buffer_;
    size_t offset_ = 0;
    std::vector<size_t> shape_;
    DType dtype_ = DType::F32;
};

struct Metrics {
    std::string operation;
    size_t bytes_read = 0, bytes_written = 0;
};
struct Output {
    Tensor tensor;
    Metrics metrics;
};

class QuantizedMatrix {
public:
    size_t rows() const { return rows_; }
    size_t columns() const { return columns_; }
    QuantizationFormat format() const { return format_; }
    size_t byte_size() const { return fh_qmatrix_byte_size(handle_->raw); }
    fh_qmatrix* raw() const { return handle_->raw; }
    const std::shared_ptr<detail::DeviceHandle>& owner() const { return handle_->owner; }

private:
    friend class Device;
    friend class QuantizedExpertMatrix;
    std::shared_ptr<detail::MatrixHandle> handle_;
    size_t rows_ = 0, columns_ = 0;
    QuantizationFormat format_ = QuantizationFormat::Q4_K;
};

class QuantizedExpertMatrix {
public:
    size_t experts() const { return experts_; }
    size_t rows_per_expert() const { return matrix_.rows_ / experts_; }
    size_t columns() const { return matrix_.columns_; }
    QuantizationFormat format() const { return matrix_.format_; }
    size_t byte_size() const { return matrix_.byte_size(); }
    const QuantizedMatrix& matrix() const { return matrix_; }

private:
    friend class Device;
    QuantizedMatrix matrix_;
    size_t experts_ = 0;
};

enum class MoeScoringFunction { Softmax, Sigmoid };
struct MoeRoutingPolicy {
    size_t experts = 0, top_k = 0;
    MoeScoringFunction scoring_function = MoeScoringFunction::Softmax;
    bool normalize_top_k_prob = true;
    float normalization_epsilon = 0.f;
    float routed_scaling_factor = 1.f;
    bool use_expert_bias = false;
    fh_routing_policy c() const {
        return fh_routing_policy{(uint32_t)experts, (uint32_t)top_k,
                                 scoring_function == MoeScoringFunction::Sigmoid ? 1u : 0u,
                                 normalize_top_k_prob ? 1u : 0u, normalization_epsilon, routed_scaling_factor};
    }
};

// Recorded operator calls, replayed as one HIP graph (Execution of the reference).
class Graph {
public:
    explicit Graph(fh_graph* raw) : raw_(raw, fh_graph_destroy) {}
    void launch() const { check(fh_graph_launch(raw_.get())); }
private:
    std::shared_ptr<fh_graph> raw_;
};

class Device {
public:
    explicit Device(int ordinal = 0) : handle_(std::make_shared<detail::DeviceHandle>()) {
        check(fh_device_create(ordinal, &handle_->raw));
    }
    fh_device* raw() const { return handle_->raw; }
    void synchronize() const { check(fh_synchronize(handle_->raw)); }
    std::string last_operation() const { return fh_last_operation(handle_->raw); }
    void set_k_quant_gemv_ksplit(int64_t simds) const { check(fh_set_tuning(handle_->raw, "k_quant_gemv_ksplit", simds)); }
    void set_tuning(const char* key, int64_t value) const { check(fh_set_tuning(handle_->raw, key, value)); }
    int64_t get_tuning(const char* key) const {
        int64_t value = 0;
        check(fh_get_tuning(handle_->raw, key, &value));
        return value;
    }
    // Bound on the routing temporaries of one SparseMoe chunk (set_moe_routing_temporary_limit,
    // src/metal/legacy.rs:520-534; 128 MiB at first).
    void set_moe_routing_temporary_limit(size_t bytes) const { set_tuning("moe_routing_temporary_limit", (int64_t)bytes); }
    size_t moe_routing_temporary_limit() const { return (size_t)get_tuning("moe_routing_temporary_limit"); }
    bool owns(const Tensor& t) const { return t.buffer_ && t.buffer_->owner == handle_; }

    // ---- tensors ----
    Tensor zeros(std::vector<size_t> shape, DType dtype) const {
        Tensor t;
        t.shape_ = std::move(shape);
        t.dtype_ = dtype;
        auto buffer = std::make_shared<detail::BufferHandle>();
        buffer->owner = handle_;
        buffer->bytes = t.byte_size() ? t.byte_size() : 1;
        check(fh_buffer_alloc(handle_->raw, buffer->bytes, &buffer->raw));
        t.buffer_ = std::move(buffer);
        return t;
    }
    Tensor from_f32(std::vector<size_t> shape, DType dtype, const std::vector<float>& values) const {
        Tensor t = zeros(std::move(shape), dtype);
        if (values.size() != t.numel()) throw Error(ErrorKind::Shape, "value count does not match the shape");
        if (dtype == DType::F32) {
            check(fh_buffer_upload(t.buffer_->raw, 0, values.data(), values.size() * 4));
        } else {
            std::vector<uint16_t> raw(values.size());
            for (size_t i = 0; i < raw.size(); ++i)
                raw[i] = dtype == DType::F16 ? f32_to_f16_bits(values[i]) : f32_to_bf16_bits(values[i]);
            check(fh_buffer_upload(t.buffer_->raw, 0, raw.data(), raw.size() * 2));
        }
        return t;
    }
    Tensor from_bits(std::vector<size_t> shape, const std::vector<uint32_t>& words) const {
        Tensor t = zeros(std::move(shape), DType::F32);
        if (words.size() != t.numel()) throw Error(ErrorKind::Shape, "value count does not match the shape");
        check(fh_buffer_upload(t.buffer_->raw, 0, words.data(), words.size() * 4));
        return t;
    }

    // ---- weights ----
    // QuantizedMatrix::from_reader: `fill` writes the packed GGUF bytes.
    QuantizedMatrix quantized_matrix(size_t rows, size_t columns, QuantizationFormat format,
                                     const std::function<void(uint8_t*, size_t)>& fill,
                                     size_t experts = 1) const {
        if (rows == 0 || columns == 0 || columns % block_elements(format) != 0 || experts == 0 || rows % experts)
            throw Error(ErrorKind::Shape, "quantized matrix requires nonempty rows and whole blocks");
        std::vector<uint8_t> host(rows * (columns / block_elements(format)) * block_bytes(format));
        fill(host.data(), host.size());
        QuantizedMatrix m;
        m.handle_ = std::make_shared<detail::MatrixHandle>();
        m.handle_->owner = handle_;
        check(fh_qmatrix_create(handle_->raw, static_cast<uint32_t>(format), rows / experts, columns, experts,
                                host.data(), host.size(), &m.handle_->raw));
        m.rows_ = rows;
        m.columns_ = columns;
        m.format_ = format;
        return m;
    }
    QuantizedExpertMatrix quantized_expert_matrix(size_t experts, size_t rows_per_expert, size_t columns,
                                                  QuantizationFormat format,
                                                  const std::function<void(uint8_t*, size_t)>& fill) const {
        if (experts == 0 || rows_per_expert == 0) throw Error(ErrorKind::Shape, "invalid quantized expert geometry");
        QuantizedExpertMatrix e;
        e.matrix_ = quantized_matrix(experts * rows_per_expert, columns, format, fill, experts);
        e.experts_ = experts;
        return e;
    }

    // ---- operators ----
    Tensor dequantize(const QuantizedMatrix& w, DType dtype = DType::F32) const {
        Tensor out = zeros({w.rows(), w.columns()}, dtype);
        fh_view v = out.c_view();
        check(fh_dequantize(handle_->raw, w.raw(), &v));
        return out;
    }
    Output embedding_gather_quantized(const QuantizedMatrix& w, const std::vector<uint32_t>& tokens,
                                      DType dtype) const {
        if (tokens.empty()) throw Error(ErrorKind::Shape, "embedding gather requires tokens");
        Tensor out = zeros({tokens.size(), w.columns()}, dtype);
        fh_view v = out.c_view();
        check(fh_embedding_gather_quantized(handle_->raw, w.raw(), tokens.data(), tokens.size(), &v));
        return {out, {last_operation(), 0, out.byte_size()}};
    }
    // Y[M,N] = X[M,K] . W[N,K]^T; the output takes the activation dtype unless told otherwise.
    Output project_quantized(const Tensor& a, const QuantizedMatrix& w, const Tensor* out = nullptr,
                             const DType* out_dtype = nullptr) const {
        const auto& dims = a.shape();
        if (dims.size() != 2 || dims[1] != w.columns() || dims[0] == 0)
            throw Error(ErrorKind::Shape, "quantized projection requires [M,K] matching [N,K]");
        if (!owns(a) || w.owner() != handle_) throw Error(ErrorKind::DeviceMismatch, "tensor or weight belongs to another device");
        Tensor y = out ? *out : zeros({dims[0], w.rows()}, out_dtype ? *out_dtype : a.dtype());
        fh_view xv = a.c_view(), yv = y.c_view();
        check(fh_project_quantized(handle_->raw, w.raw(), &xv, (uint32_t)dims[0], &yv));
        return {y, {last_operation(), a.byte_size() + w.byte_size(), y.byte_size()}};
    }
    // [rows, 2] F32 carrier of u32 bits: first maximal index and a non-finite flag.
    Tensor argmax_rows(const Tensor& logits) const {
        const auto& dims = logits.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] == 0 || dims[1] > 0xffffffffull)
            throw Error(ErrorKind::Shape, "argmax requires nonempty [rows,width]");
        if (!owns(logits)) throw Error(ErrorKind::DeviceMismatch, "tensor belongs to another device");
        Tensor out = zeros({dims[0], 2}, DType::F32);
        fh_view lv = logits.c_view(), ov = out.c_view();
        check(fh_argmax_rows(handle_->raw, &lv, (uint32_t)dims[0], (uint32_t)dims[1], &ov));
        return out;
    }
    // (residual, normed): residual = a + b in the operands' dtype, normed = rmsnorm(residual) * weight
    // (MetalDevice::add_rmsnorm, src/ops/mod.rs:762-820).  Outputs may be passed in to reuse buffers.
    std::pair<Tensor, Tensor> add_rmsnorm(const Tensor& a, const Tensor& b, const Tensor& weight, float epsilon,
                                          const Tensor* residual_out = nullptr,
                                          const Tensor* normed_out = nullptr) const {
        const auto& dims = a.shape();
        if (dims.empty() || dims.back() == 0 || a.numel() == 0)
            throw Error(ErrorKind::Shape, "last dimension must be nonzero");
        const uint64_t width = dims.back();
        if (a.shape() != b.shape() || a.dtype() != b.dtype() || weight.dtype() != a.dtype())
            throw Error(ErrorKind::Shape, "fused add+RMSNorm operands must match");
        if (weight.shape().size() != 1 || weight.shape()[0] != width || width > 0xffffffffull - 256)
            throw Error(ErrorKind::Shape, "RMSNorm weight must match the last dimension");
        if (!std::isfinite(epsilon) || epsilon <= 0.f)
            throw Error(ErrorKind::Parameter, "epsilon must be finite and positive");
        if (!owns(a) || !owns(b) || !owns(weight)) throw Error(ErrorKind::DeviceMismatch, "tensor belongs to another device");
        Tensor residual = residual_out ? *residual_out : zeros(dims, a.dtype());
        Tensor normed = normed_out ? *normed_out : zeros(dims, a.dtype());
        fh_view av = a.c_view(), bv = b.c_view(), wv = weight.c_view(), rv = residual.c_view(), nv = normed.c_view();
        check(fh_add_rmsnorm(handle_->raw, &av, &bv, &wv, (uint32_t)(a.numel() / width), (uint32_t)width, epsilon, &rv,
                             &nv));
        return {residual, normed};
    }
    Tensor moe_route(const Tensor& logits, const Tensor* selection_bias, const MoeRoutingPolicy& policy,
                     const Tensor* out = nullptr) const {
        const auto& dims = logits.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] != policy.experts)
            throw Error(ErrorKind::Shape, "invalid sparse routing geometry");
        Tensor meta = out ? *out : zeros({dims[0] * policy.top_k, 3}, DType::F32);
        fh_view lv = logits.c_view(), mv = meta.c_view(), bv{};
        if (selection_bias) bv = selection_bias->c_view();
        fh_routing_policy pc = policy.c();
        check(fh_moe_route(handle_->raw, &lv, (uint32_t)dims[0], selection_bias ? &bv : nullptr, &pc, &mv));
        return meta;
    }
    // The hybrid engine's router (h_moe_route): metadata rows in selection order; when
    // `shared_gate` is given it receives sigmoid(dot(x[t], gate_vector)) per token, or ones
    // without a vector.
    Tensor moe_route_ranked(const Tensor& logits, const MoeRoutingPolicy& policy, const Tensor* x = nullptr,
                            const Tensor* gate_vector = nullptr, const Tensor* shared_gate = nullptr) const {
        const auto& dims = logits.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] != policy.experts)
            throw Error(ErrorKind::Shape, "invalid sparse routing geometry");
        Tensor meta = zeros({dims[0] * policy.top_k, 3}, DType::F32);
        fh_view lv = logits.c_view(), mv = meta.c_view(), xv{}, wv{}, gv{};
        if (x) xv = x->c_view();
        if (gate_vector) wv = gate_vector->c_view();
        if (shared_gate) gv = shared_gate->c_view();
        fh_routing_policy pc = policy.c();
        check(fh_moe_route_ranked(handle_->raw, &lv, (uint32_t)dims[0], &pc, x ? &xv : nullptr,
                                  gate_vector ? &wv : nullptr, gate_vector ? (uint32_t)gate_vector->numel() : 0, &mv,
                                  shared_gate ? &gv : nullptr));
        return meta;
    }
    // h_moe_combine: the weighted sum of the routed rows plus shared_gate[t] * shared[t].
    Tensor expert_combine_shared(const Tensor& input, const Tensor& metadata, size_t tokens, size_t hidden,
                                 size_t top_k, const Tensor& shared, const Tensor* shared_gate = nullptr,
                                 const Tensor* out = nullptr) const {
        Tensor y = out ? *out : zeros({tokens, hidden}, input.dtype());
        fh_view iv = input.c_view(), mv = metadata.c_view(), sv = shared.c_view(), yv = y.c_view(), gv{};
        if (shared_gate) gv = shared_gate->c_view();
        check(fh_expert_combine_shared(handle_->raw, &iv, &mv, (uint32_t)tokens, (uint32_t)hidden, (uint32_t)top_k,
                                       &sv, shared_gate ? &gv : nullptr, &yv));
        return y;
    }
    // ---- the hybrid engine's routed FFN in its own layout: ids / weights as plain arrays
    // (HybridModel::moe_ffn, src/hybrid/engine.rs:2881-3080); u32 values ride in F32 carriers ----
    struct HybridRoutes {
        Tensor ids, weights, shared_gate;
    };
    // h_moe_route: ids and weights [tokens * top_k] in selection order, and the shared-expert gate
    HybridRoutes hybrid_moe_route(const Tensor& logits, const MoeRoutingPolicy& policy, const Tensor* x = nullptr,
                                  const Tensor* gate_vector = nullptr) const {
        const auto& dims = logits.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] != policy.experts)
            throw Error(ErrorKind::Shape, "invalid sparse routing geometry");
        HybridRoutes r{zeros({dims[0] * policy.top_k}, DType::F32), zeros({dims[0] * policy.top_k}, DType::F32),
                       zeros({dims[0]}, DType::F32)};
        fh_view lv = logits.c_view(), iv = r.ids.c_view(), wtv = r.weights.c_view(), gv = r.shared_gate.c_view(), xv{}, wv{};
        if (x) xv = x->c_view();
        if (gate_vector) wv = gate_vector->c_view();
        fh_routing_policy pc = policy.c();
        check(fh_hybrid_moe_route(handle_->raw, &lv, (uint32_t)dims[0], &pc, x ? &xv : nullptr,
                                  gate_vector ? &wv : nullptr, gate_vector ? (uint32_t)gate_vector->numel() : 0, &iv,
                                  &wtv, &gv));
        return r;
    }
    // HybridModel::project: exact f32 weights for 1..4 rows (or always with `exact`), f16 tiles from 5 rows on
    Output hybrid_project(const QuantizedMatrix& w, const Tensor& a, bool exact = false) const {
        const auto& dims = a.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] != w.columns())
            throw Error(ErrorKind::Shape, "quantized projection requires [M,K] matching [N,K]");
        Tensor y = zeros({dims[0], w.rows()}, a.dtype());
        fh_view xv = a.c_view(), yv = y.c_view();
        check(fh_hybrid_project(handle_->raw, w.raw(), &xv, (uint32_t)dims[0], &yv, exact ? 1u : 0u));
        return {y, {last_operation(), a.byte_size() + w.byte_size(), y.byte_size()}};
    }
    // HybridModel::project_id: route r multiplies activation row r / x_div by expert ids[r]
    Tensor hybrid_project_id(const QuantizedExpertMatrix& w, const Tensor& x, const Tensor& ids, size_t routes,
                             size_t x_div) const {
        if (routes == 0 || x_div == 0 || routes % x_div != 0 || ids.numel() != routes)
            throw Error(ErrorKind::Shape, "expert projection geometry");
        Tensor y = zeros({routes, w.rows_per_expert()}, x.dtype());
        fh_view xv = x.c_view(), iv = ids.c_view(), yv = y.c_view();
        check(fh_hybrid_project_id(handle_->raw, w.matrix().raw(), &xv, &iv, (uint32_t)routes, (uint32_t)x_div, &yv));
        return y;
    }
    // project_id with the shared expert's projection in the same launch: its `tokens` rows read
    // shared_x [tokens, K] when given (down), else the token rows x (gate, up).
    // Returns {y [routes, N], shared_y [tokens, N]}.
    std::pair<Tensor, Tensor> hybrid_project_id_with_shared(const QuantizedExpertMatrix& w, const QuantizedMatrix& shared_w,
                                                            const Tensor& x, const Tensor& ids, size_t routes,
                                                            size_t x_div, size_t tokens,
                                                            const Tensor* shared_x = nullptr) const {
        if (routes == 0 || x_div == 0 || routes % x_div != 0 || ids.numel() != routes || tokens == 0 ||
            (!shared_x && tokens != routes / x_div) || shared_w.rows() != w.rows_per_expert() ||
            shared_w.columns() != w.columns() || shared_w.format() != w.format())
            throw Error(ErrorKind::Shape, "expert projection geometry");
        Tensor y = zeros({routes, w.rows_per_expert()}, x.dtype());
        Tensor ys = zeros({tokens, w.rows_per_expert()}, x.dtype());
        fh_view xv = x.c_view(), iv = ids.c_view(), yv = y.c_view(), ysv = ys.c_view(), sxv{};
        if (shared_x) sxv = shared_x->c_view();
        check(fh_hybrid_project_id_with_shared(handle_->raw, w.matrix().raw(), shared_w.raw(), &xv, &iv, (uint32_t)routes,
                                               (uint32_t)x_div, (uint32_t)tokens, shared_x ? &sxv : nullptr, &yv, &ysv));
        return {y, ys};
    }
    struct HybridMap {
        Tensor offsets, sorted, position;
    };
    // h_moe_map: expert-major order of the routes, stable inside an expert
    HybridMap hybrid_moe_map(const Tensor& ids, size_t experts) const {
        const size_t routes = ids.numel();
        HybridMap m{zeros({experts + 1}, DType::F32), zeros({routes}, DType::F32), zeros({routes}, DType::F32)};
        fh_view iv = ids.c_view(), ov = m.offsets.c_view(), sv = m.sorted.c_view(), pv = m.position.c_view();
        check(fh_hybrid_moe_map(handle_->raw, &iv, (uint32_t)experts, (uint32_t)routes, &ov, &sv, &pv));
        return m;
    }
    // h_moe_gather: out[p] = x[sorted[p] / used]
    Tensor hybrid_moe_gather(const Tensor& x, const Tensor& sorted, size_t used) const {
        const auto& dims = x.shape();
        if (dims.size() != 2 || used == 0 || sorted.numel() != dims[0] * used)
            throw Error(ErrorKind::Shape, "route gather needs [tokens, hidden] and tokens * used routes");
        Tensor out = zeros({sorted.numel(), dims[1]}, x.dtype());
        fh_view xv = x.c_view(), sv = sorted.c_view(), ov = out.c_view();
        check(fh_hybrid_moe_gather(handle_->raw, &xv, &sv, (uint32_t)dims[1], (uint32_t)used, (uint32_t)sorted.numel(), &ov));
        return out;
    }
    // HybridModel::project_mm_id: rows offsets[e] .. offsets[e + 1] of the expert-sorted x times expert e
    Tensor hybrid_project_mm_id(const QuantizedExpertMatrix& w, const Tensor& x, const Tensor& offsets) const {
        const auto& dims = x.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] != w.columns() || offsets.numel() != w.experts() + 1)
            throw Error(ErrorKind::Shape, "expert projection geometry");
        Tensor y = zeros({dims[0], w.rows_per_expert()}, x.dtype());
        fh_view xv = x.c_view(), fv = offsets.c_view(), yv = y.c_view();
        check(fh_hybrid_project_mm_id(handle_->raw, w.matrix().raw(), &xv, &fv, (uint32_t)dims[0], &yv));
        return y;
    }
    // project_mm_id with the shared expert's dense projection of shared_x [tokens, K] in the same launch.
    // Returns {y [routes, N], shared_y [tokens, N]}.
    std::pair<Tensor, Tensor> hybrid_project_mm_id_with_shared(const QuantizedExpertMatrix& w, const QuantizedMatrix& shared_w,
                                                               const Tensor& x, const Tensor& offsets,
                                                               const Tensor& shared_x) const {
        const auto& dims = x.shape();
        const auto& sd = shared_x.shape();
        if (dims.size() != 2 || dims[0] == 0 || dims[1] != w.columns() || offsets.numel() != w.experts() + 1 ||
            sd.size() != 2 || sd[0] == 0 || sd[1] != dims[1] || shared_x.dtype() != x.dtype() ||
            shared_w.rows() != w.rows_per_expert() || shared_w.columns() != w.columns() || shared_w.format() != w.format())
            throw Error(ErrorKind::Shape, "expert projection geometry");
        Tensor y = zeros({dims[0], w.rows_per_expert()}, x.dtype());
        Tensor ys = zeros({sd[0], w.rows_per_expert()}, x.dtype());
        fh_view xv = x.c_view(), fv = offsets.c_view(), sxv = shared_x.c_view(), yv = y.c_view(), ysv = ys.c_view();
        check(fh_hybrid_project_mm_id_with_shared(handle_->raw, w.matrix().raw(), shared_w.raw(), &xv, &fv, (uint32_t)dims[0],
                                                  (uint32_t)sd[0], &sxv, &yv, &ysv));
        return {y, ys};
    }
    // h_moe_combine (f32): weighted sum of each token's routed rows through `position` (or the routes
    // themselves when null) plus shared_gate[t] * shared[t]
    Tensor hybrid_moe_combine(const Tensor& down, const Tensor& weights, const Tensor* position, const Tensor& shared,
                              const Tensor& shared_gate, size_t used) const {
        const auto& dims = shared.shape();
        if (dims.size() != 2 || used == 0) throw Error(ErrorKind::Shape, "expert combine geometry mismatch");
        Tensor out = zeros({dims[0], dims[1]}, DType::F32);
        fh_view dv = down.c_view(), wv = weights.c_view(), sv = shared.c_view(), gv = shared_gate.c_view(), ov = out.c_view(), pv{};
        if (position) pv = position->c_view();
        check(fh_hybrid_moe_combine(handle_->raw, &dv, &wv, position ? &pv : nullptr, &sv, &gv, (uint32_t)dims[1],
                                    (uint32_t)used, (uint32_t)dims[0], &ov));
        return out;
    }
    Tensor expert_assign(const Tensor& hidden, const Tensor& metadata, size_t top_k, const Tensor* out = nullptr) const {
        const auto& x = hidden.shape();
        const auto& m = metadata.shape();
        if (x.size() != 2 || m.size() != 2 || m[1] != 3 || top_k == 0 || x[0] * top_k != m[0])
            throw Error(ErrorKind::Shape, "expert assignments require [S,H] and [S*top_k,3]");
        Tensor y = out ? *out : zeros({m[0], x[1]}, hidden.dtype());
        fh_view hv = hidden.c_view(), mv = metadata.c_view(), yv = y.c_view();
        check(fh_expert_assign(handle_->raw, &hv, (uint32_t)x[0], (uint32_t)x[1], &mv, (uint32_t)top_k, &yv));
        return y;
    }
    Tensor expert_project_quantized(const Tensor& input, const Tensor& metadata, const QuantizedExpertMatrix& w,
                                    size_t features, size_t experts, const Tensor* out = nullptr) const {
        const auto& x = input.shape();
        if (x.size() != 2 || x[0] == 0 || x[1] != features || metadata.shape() != std::vector<size_t>{x[0], 3} ||
            w.experts() != experts || w.columns() != features)
            throw Error(ErrorKind::Shape, "quantized expert projection geometry mismatch");
        Tensor y = out ? *out : zeros({x[0], w.rows_per_expert()}, input.dtype());
        fh_view xv = input.c_view(), mv = metadata.c_view(), yv = y.c_view();
        check(fh_expert_project_quantized(handle_->raw, w.matrix().raw(), &xv, (uint32_t)x[0], &mv, &yv));
        return y;
    }
    // Decode-sized fusions (see ferrum_hip.h): the same bits as the separate calls in one launch.
    // Gather: input is hidden [tokens, K], row a uses hidden[token(a), :].
    Tensor expert_project_gathered(const Tensor& hidden, const Tensor& metadata, const QuantizedExpertMatrix& w,
                                   const Tensor* out = nullptr) const {
        return expert_project_fused(hidden, metadata, w, FH_INPUT_GATHER, out);
    }
    // SiLU: input is [A, 2K], gate first; expert_silu_mul is applied on the way in.
    Tensor expert_project_silu_mul(const Tensor& packed, const Tensor& metadata, const QuantizedExpertMatrix& w,
                                   const Tensor* out = nullptr) const {
        return expert_project_fused(packed, metadata, w, FH_INPUT_SILU_MUL, out);
    }
    // The routed projection and, in the same launch, the shared expert's dense projection of
    // every token (fh_expert_project_with_shared): form FH_INPUT_GATHER reads both from
    // input [tokens, K]; FH_INPUT_SILU_MUL reads the routed rows from input [A, 2K] and the
    // shared ones from shared_input [tokens, 2K].  Returns {routed [A, N], shared [tokens, N]}.
    std::pair<Tensor, Tensor> expert_project_with_shared(const Tensor& input, const Tensor& metadata,
                                                         const QuantizedExpertMatrix& w, const QuantizedMatrix& shared_w,
                                                         size_t tokens, uint32_t form,
                                                         const Tensor* shared_input = nullptr) const {
        const auto& x = input.shape();
        const auto& m = metadata.shape();
        const size_t k = w.columns();
        const bool silu = form == FH_INPUT_SILU_MUL;
        if ((form != FH_INPUT_GATHER && !silu) || x.size() != 2 || m.size() != 2 || m[0] == 0 || m[1] != 3 || tokens == 0 ||
            x[0] != (silu ? m[0] : tokens) || x[1] != (silu ? 2 * k : k) || silu != (shared_input != nullptr) ||
            (shared_input && (shared_input->shape() != std::vector<size_t>{tokens, 2 * k} ||
                              shared_input->dtype() != input.dtype())) ||
            shared_w.rows() != w.rows_per_expert() || shared_w.columns() != k || shared_w.format() != w.format())
            throw Error(ErrorKind::Shape, "quantized expert projection geometry mismatch");
        if (!owns(input) || !owns(metadata) || shared_w.owner() != handle_)
            throw Error(ErrorKind::DeviceMismatch, "tensor or weight belongs to another device");
        Tensor y = zeros({m[0], w.rows_per_expert()}, input.dtype());
        Tensor ys = zeros({tokens, w.rows_per_expert()}, input.dtype());
        fh_view xv = input.c_view(), mv = metadata.c_view(), yv = y.c_view(), ysv = ys.c_view(), sxv{};
        if (shared_input) sxv = shared_input->c_view();
        check(fh_expert_project_with_shared(handle_->raw, w.matrix().raw(), shared_w.raw(), &xv, (uint32_t)tokens, form,
                                            (uint32_t)m[0], &mv, shared_input ? &sxv : nullptr, &yv, &ysv));
        return {y, ys};
    }
    Output project_silu_mul_quantized(const Tensor& packed, const QuantizedMatrix& w, const Tensor* out = nullptr) const {
        const auto& dims = packed.shape();
        if (dims.size() != 2 || dims[1] != 2 * w.columns() || dims[0] == 0)
            throw Error(ErrorKind::Shape, "quantized projection requires [M,2K] matching [N,K]");
        if (!owns(packed) || w.owner() != handle_) throw Error(ErrorKind::DeviceMismatch, "tensor or weight belongs to another device");
        Tensor y = out ? *out : zeros({dims[0], w.rows()}, packed.dtype());
        fh_view xv = packed.c_view(), yv = y.c_view();
        check(fh_project_silu_mul_quantized(handle_->raw, w.raw(), &xv, (uint32_t)dims[0], &yv));
        return {y, {last_operation(), packed.byte_size() + w.byte_size(), y.byte_size()}};
    }
    Tensor expert_silu_mul(const Tensor& input, size_t intermediate, const Tensor* out = nullptr) const {
        const auto& x = input.shape();
        if (x.size() != 2 || intermediate == 0 || intermediate * 2 != x[1])
            throw Error(ErrorKind::Shape, "packed expert activation geometry mismatch");
        Tensor y = out ? *out : zeros({x[0], intermediate}, input.dtype());
        fh_view iv = input.c_view(), yv = y.c_view();
        check(fh_expert_silu_mul(handle_->raw, &iv, (uint32_t)x[0], (uint32_t)intermediate, &yv));
        return y;
    }
    Tensor expert_combine(const Tensor& input, const Tensor& metadata, size_t tokens, size_t hidden, size_t top_k,
                          const Tensor* out = nullptr) const {
        if (top_k == 0 || hidden == 0 || input.shape() != std::vector<size_t>{tokens * top_k, hidden})
            throw Error(ErrorKind::Shape, "expert combine geometry mismatch");
        Tensor y = out ? *out : zeros({tokens, hidden}, input.dtype());
        fh_view iv = input.c_view(), mv = metadata.c_view(), yv = y.c_view();
        check(fh_expert_combine(handle_->raw, &iv, &mv, (uint32_t)tokens, (uint32_t)hidden, (uint32_t)top_k, &yv));
        return y;
    }

    // Records the operator calls made by `body` and returns them as a graph.
    Graph execution(const std::function<void()>& body) const {
        check(fh_execution_begin(handle_->raw));
        fh_graph* raw = nullptr;
        try {
            body();
        } catch (...) {
            (void)fh_execution_end(handle_->raw, &raw);
            if (raw) fh_graph_destroy(raw);
            throw;
        }
        check(fh_execution_end(handle_->raw, &raw));
        return Graph(raw);
    }

private:
    Tensor expert_project_fused(const Tensor& input, const Tensor& metadata, const QuantizedExpertMatrix& w,
                                uint32_t form, const Tensor* out) const {
        const auto& x = input.shape();
        const auto& m = metadata.shape();
        const size_t width = w.columns() * (form == FH_INPUT_SILU_MUL ? 2 : 1);
        if (x.size() != 2 || x[0] == 0 || x[1] != width || m.size() != 2 || m[0] == 0 || m[1] != 3 ||
            (form != FH_INPUT_GATHER && m[0] != x[0]))
            throw Error(ErrorKind::Shape, "quantized expert projection geometry mismatch");
        Tensor y = out ? *out : zeros({m[0], w.rows_per_expert()}, input.dtype());
        fh_view xv = input.c_view(), mv = metadata.c_view(), yv = y.c_view();
        check(fh_expert_project_fused(handle_->raw, w.matrix().raw(), &xv, (uint32_t)x[0], form, (uint32_t)m[0], &mv, &yv));
        return y;
    }
    std::shared_ptr<detail::DeviceHandle> handle_;
};

// What SparseMoe::forward did since the last take_stats (MoeStats, src/nn/moe.rs:75-116).
// Durations are host seconds spent enqueueing.  Routing runs on the device, so the set of
// active experts is never read back and active_experts_known turns false with the first pass.
struct MoeStats {
    double router_projection_enqueue = 0, routing = 0, routing_boundary_wait = 0, expert_dispatch = 0,
           combine_dispatch = 0;
    size_t active_experts = 0;
    bool active_experts_known = true;
    size_t assignments = 0;
    size_t peak_temporary_bytes = 0;
    void merge(const MoeStats& other) {
        router_projection_enqueue += other.router_projection_enqueue;
        routing += other.routing;
        routing_boundary_wait += other.routing_boundary_wait;
        expert_dispatch += other.expert_dispatch;
        combine_dispatch += other.combine_dispatch;
        active_experts += other.active_experts;
        active_experts_known = active_experts_known && other.active_experts_known;
        assignments += other.assignments;
        peak_temporary_bytes = std::max(peak_temporary_bytes, other.peak_temporary_bytes);
    }
};

// SparseMoe::forward without the router's own dense layer: the caller passes
// the router logits (that layer is outside the quantized path).
class SparseMoe {
public:
    SparseMoe(const Device& device, QuantizedExpertMatrix input_experts, QuantizedExpertMatrix output_experts,
              MoeRoutingPolicy routing)
        : device_(device), input_(std::move(input_experts)), output_(std::move(output_experts)), routing_(routing) {
        const size_t two_i = input_.rows_per_expert();
        if (two_i == 0 || two_i % 2 || output_.experts() != input_.experts() ||
            output_.rows_per_expert() != input_.columns() || output_.columns() * 2 != two_i ||
            routing_.experts != input_.experts() || routing_.top_k == 0 || routing_.top_k > routing_.experts)
            throw Error(ErrorKind::Config, "invalid sparse expert weight geometry");
    }
    // A shared expert that every token runs next to its routed ones, as the hybrid engine's
    // moe_ffn does (src/hybrid/engine.rs:2925): input [2*I_s, H] with the gate rows first,
    // output [H, I_s].  Its result is added in the combine, scaled by forward's shared_gate.
    void set_shared_expert(QuantizedMatrix input, QuantizedMatrix output) {
        if (input.columns() != input_.columns() || output.rows() != input_.columns() || input.rows() == 0 ||
            input.rows() != 2 * output.columns())
            throw Error(ErrorKind::Config, "invalid shared expert weight geometry");
        shared_rides_ = input.rows() == input_.rows_per_expert() && input.format() == input_.format() &&
                        output.format() == output_.format();
        shared_input_ = std::move(input);
        shared_output_ = std::move(output);
    }
    // Routing temporaries of `tokens` tokens as the reference counts them (src/nn/moe.rs:232-249,
    // :306-316): per assignment the assigned, gate|up, activated and output rows plus one routing
    // record; per token its logits and its combined row.
    size_t temporary_bytes(size_t tokens, DType dtype) const {
        const size_t h = input_.columns(), i = input_.rows_per_expert() / 2, e = input_.experts();
        const size_t per_assignment = (2 * h + 3 * i) * size_bytes(dtype) + 3 * sizeof(float);
        return tokens * (per_assignment * routing_.top_k + (e + h) * size_bytes(dtype));
    }
    // The statistics gathered since the last call, which start afresh (take_stats, src/nn/moe.rs:218-220).
    MoeStats take_stats() const {
        MoeStats taken = stats_;
        stats_ = MoeStats{};
        return taken;
    }
    // Tokens are taken in chunks whose routing temporaries stay under the device's
    // moe_routing_temporary_limit (src/nn/moe.rs:250-256); every chunk's combine writes its rows of
    // one output tensor, so nothing is read back between chunks.
    Tensor forward(const Tensor& hidden, const Tensor& router_logits, const Tensor* selection_bias = nullptr,
                   const Tensor* shared_gate = nullptr) const {
        const auto& dims = hidden.shape();
        const size_t h = input_.columns(), e = input_.experts();
        if (dims.size() != 2 || dims[1] != h || dims[0] == 0)
            throw Error(ErrorKind::Shape, "sparse expert input requires [tokens,hidden]");
        if (router_logits.shape() != std::vector<size_t>{dims[0], e})
            throw Error(ErrorKind::Shape, "router logits require [tokens,experts]");
        const size_t tokens = dims[0];
        const size_t per_token = temporary_bytes(1, hidden.dtype());
        const size_t limit = (size_t)device_.get_tuning("moe_routing_temporary_limit");
        const size_t chunk = std::min(tokens, std::max<size_t>(1, limit / per_token));
        MoeStats stats;
        stats.active_experts_known = false;
        Tensor out = chunk == tokens ? forward_chunk(hidden, router_logits, selection_bias, shared_gate, nullptr, stats)
                                     : device_.zeros({tokens, h}, hidden.dtype());
        for (size_t start = 0; chunk != tokens && start < tokens; start += chunk) {
            const size_t count = std::min(chunk, tokens - start);
            Tensor rows = out.view(start * h, {count, h});
            Tensor gate;
            if (shared_gate) gate = shared_gate->view(start, {count});
            forward_chunk(hidden.view(start * h, {count, h}), router_logits.view(start * e, {count, e}), selection_bias,
                          shared_gate ? &gate : nullptr, &rows, stats);
        }
        stats_.merge(stats);
        return out;
    }

    // fh_moe_ffn: the steps of forward() with the inputs folded into the projections, enqueued by one
    // library call with its temporaries in the library's workspace; the same bits.
    Tensor forward_in_one_call(const Tensor& hidden, const Tensor& router_logits, const Tensor* selection_bias = nullptr,
                               const Tensor* shared_gate = nullptr) const {
        const auto& dims = hidden.shape();
        const size_t h = input_.columns(), e = input_.experts();
        if (dims.size() != 2 || dims[1] != h || dims[0] == 0)
            throw Error(ErrorKind::Shape, "sparse expert input requires [tokens,hidden]");
        if (router_logits.shape() != std::vector<size_t>{dims[0], e})
            throw Error(ErrorKind::Shape, "router logits require [tokens,experts]");
        Tensor out = device_.zeros({dims[0], h}, hidden.dtype());
        fh_view hv = hidden.c_view(), lv = router_logits.c_view(), ov = out.c_view(), bv{}, gv{};
        if (selection_bias) bv = selection_bias->c_view();
        if (shared_gate) gv = shared_gate->c_view();
        const fh_routing_policy pc = routing_.c();
        check(fh_moe_ffn(device_.raw(), &hv, &lv, (uint32_t)dims[0], selection_bias ? &bv : nullptr, &pc,
                                        input_.matrix().raw(), output_.matrix().raw(),
                                        shared_input_ ? shared_input_->raw() : nullptr,
                                        shared_output_ ? shared_output_->raw() : nullptr,
                                        shared_gate ? &gv : nullptr, &ov));
        return out;
    }

    // most f32 assignments that take the fused per-assignment kernels (f32 rows have no
    // grouped form by default, and the per-assignment SiLU is recomputed by every workgroup);
    // also the most assignments whose shared expert rides in the routed launches
    size_t fused_max_assignments = 31;
    // false: expert_assign and expert_silu_mul always run as launches of their own
    bool fuse_inputs = true;

private:
    Tensor forward_chunk(const Tensor& hidden, const Tensor& router_logits, const Tensor* selection_bias,
                         const Tensor* shared_gate, const Tensor* out, MoeStats& stats) const {
        using clock = std::chrono::steady_clock;
        const auto seconds = [](clock::time_point a, clock::time_point b) {
            return std::chrono::duration<double>(b - a).count();
        };
        const auto& dims = hidden.shape();
        const size_t h = input_.columns(), i = input_.rows_per_expert() / 2, e = input_.experts();
        const size_t tokens = dims[0], a = tokens * routing_.top_k;
        stats.assignments += a;
        stats.peak_temporary_bytes = std::max(stats.peak_temporary_bytes, temporary_bytes(tokens, hidden.dtype()));
        const auto t0 = clock::now();
        Tensor meta = device_.moe_route(router_logits, selection_bias, routing_);
        const auto t1 = clock::now();
        stats.routing += seconds(t0, t1);
        Tensor expert_output, shared_output;
        if (shared_input_) {
            if (fuse_inputs && shared_rides_ && (a <= fused_max_assignments || hidden.dtype() != DType::F32)) {
                // four launches: the shared expert's rows are batch entries of the routed ones in
                // decode and further token groups of the grouped kernel beyond it
                auto up = device_.expert_project_with_shared(hidden, meta, input_, *shared_input_, tokens, FH_INPUT_GATHER);
                auto down = device_.expert_project_with_shared(up.first, meta, output_, *shared_output_, tokens,
                                                               FH_INPUT_SILU_MUL, &up.second);
                expert_output = down.first;
                shared_output = down.second;
            } else {
                expert_output = routed(hidden, meta, h, i, e);
                Tensor shared_projected = device_.project_quantized(hidden, *shared_input_).tensor;
                shared_output =
                    fuse_inputs && tokens <= fused_max_assignments
                        ? device_.project_silu_mul_quantized(shared_projected, *shared_output_).tensor
                        : device_.project_quantized(device_.expert_silu_mul(shared_projected, shared_output_->columns()),
                                                    *shared_output_).tensor;
            }
        } else {
            expert_output = routed(hidden, meta, h, i, e);
        }
        const auto t2 = clock::now();
        stats.expert_dispatch += seconds(t1, t2);
        Tensor combined = shared_input_ ? device_.expert_combine_shared(expert_output, meta, tokens, h, routing_.top_k,
                                                                        shared_output, shared_gate, out)
                                        : device_.expert_combine(expert_output, meta, tokens, h, routing_.top_k, out);
        stats.combine_dispatch += seconds(t2, clock::now());
        return combined;
    }

    // the routed experts' outputs [A, H], before the combine
    Tensor routed(const Tensor& hidden, const Tensor& meta, size_t h, size_t i, size_t e) const {
        const auto& dims = hidden.shape();
        if (fuse_inputs && (dims[0] * routing_.top_k <= fused_max_assignments || hidden.dtype() != DType::F32)) {
            // the copy and the activation ride inside the projections: per assignment in
            // decode, and in the grouped kernel's gather of an expert's rows beyond it
            Tensor projected = device_.expert_project_gathered(hidden, meta, input_);
            return device_.expert_project_silu_mul(projected, meta, output_);
        }
        Tensor assigned = device_.expert_assign(hidden, meta, routing_.top_k);
        Tensor projected = device_.expert_project_quantized(assigned, meta, input_, h, e);
        Tensor activated = device_.expert_silu_mul(projected, i);
        return device_.expert_project_quantized(activated, meta, output_, i, e);
    }

    const Device& device_;
    QuantizedExpertMatrix input_, output_;
    MoeRoutingPolicy routing_;
    std::optional<QuantizedMatrix> shared_input_, shared_output_;
    bool shared_rides_ = false;
    mutable MoeStats stats_;
};

}  // namespace ferrum

#endif  // FERRUM_HIP_HPP
