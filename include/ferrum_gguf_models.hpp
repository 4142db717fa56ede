// ferrum_gguf_models.hpp -- which tensor of a GGUF file is which weight of the model
// (C++17, header only), for the reference's two GGUF model families.
//
// The reader (ferrum_gguf.hpp) knows tensors by their GGUF names, the operators know
// packed matrices; this is the step between:
//   specifications        canonical weights and logical shapes of a model
//                         (specifications_with_policy, src/model/weights.rs:170-268)
//   qwen_source_name      canonical -> GGUF name (gguf_weight_name, src/model/qwen_gguf.rs:304-342)
//   lfm2_moe_source_names canonical -> GGUF name(s) (source_names, src/model/lfm2_moe/gguf.rs:322-366)
//   plan_qwen             metadata -> ModelShape, and the file checked against the contract
//                         (src/model/qwen_gguf.rs:32-222)
//   lfm2_moe_shape / plan_lfm2_moe   the same for LFM2-MoE (src/model/lfm2_moe/gguf.rs:93-320)
//   bind_quantized        the plan's quantized tensors on the device, blocks verbatim, gate and
//                         up experts interleaved (qwen_gguf.rs:236-268, lfm2_moe/gguf.rs:434-574)
// Dense tensors (norms, biases, unquantized embeddings) are named and checked but not
// uploaded: they do not take the quantized-matmul path.  Failures are ferrum::Error of the
// kind the reference's variant maps to (Weight, Config, Gguf).
#ifndef FERRUM_GGUF_MODELS_HPP
#define FERRUM_GGUF_MODELS_HPP

#include <optional>
#include <set>

#include "ferrum_gguf.hpp"

namespace ferrum {
namespace gguf {
namespace models {

struct SparseFeedForward {
    size_t experts = 0, intermediate_size = 0;
    bool use_expert_bias = false;
};

struct LayerShape {
    size_t intermediate_size = 0;
    std::optional<size_t> short_conv_kernel;    // attention when empty
    std::optional<SparseFeedForward> sparse;    // a dense feed-forward when empty
};

enum class QkNorm { None, PerHead, Projection };

// The part of ModelConfig + ArchitecturePolicy the tensor contract depends on.
struct ModelShape {
    size_t vocab_size = 0, hidden_size = 0, num_attention_heads = 0, num_key_value_heads = 0, head_dim = 0;
    bool tie_word_embeddings = true;
    std::vector<LayerShape> layers;
    QkNorm qk_norm = QkNorm::None;
    bool qkv_bias = false;
    std::string architecture;
};

using Specification = std::pair<std::string, std::vector<size_t>>;

inline std::vector<Specification> specifications(const ModelShape& m) {
    const size_t h = m.hidden_size, q = m.num_attention_heads * m.head_dim, k = m.num_key_value_heads * m.head_dim;
    std::vector<Specification> specs = {{"embedding.weight", {m.vocab_size, h}}, {"final_norm.weight", {h}}};
    if (!m.tie_word_embeddings) specs.push_back({"lm_head.weight", {m.vocab_size, h}});
    for (size_t l = 0; l < m.layers.size(); ++l) {
        const LayerShape& layer = m.layers[l];
        const std::string at = "layers." + std::to_string(l) + ".";
        specs.push_back({at + "input_norm.weight", {h}});
        specs.push_back({at + "post_norm.weight", {h}});
        if (!layer.short_conv_kernel) {
            specs.push_back({at + "q.weight", {q, h}});
            specs.push_back({at + "k.weight", {k, h}});
            specs.push_back({at + "v.weight", {k, h}});
            specs.push_back({at + "o.weight", {h, q}});
        } else {
            specs.push_back({at + "conv.in_proj.weight", {3 * h, h}});
            specs.push_back({at + "conv.depthwise.weight", {h, 1, *layer.short_conv_kernel}});
            specs.push_back({at + "conv.out_proj.weight", {h, h}});
        }
        if (!layer.sparse) {
            const size_t i = layer.intermediate_size;
            specs.push_back({at + "gate.weight", {i, h}});
            specs.push_back({at + "up.weight", {i, h}});
            specs.push_back({at + "down.weight", {h, i}});
        } else {
            const SparseFeedForward& s = *layer.sparse;
            specs.push_back({at + "moe.router.weight", {s.experts, h}});
            specs.push_back({at + "moe.input.weight", {s.experts, 2 * s.intermediate_size, h}});
            specs.push_back({at + "moe.output.weight", {s.experts, h, s.intermediate_size}});
            if (s.use_expert_bias) specs.push_back({at + "moe.router_bias.weight", {s.experts}});
        }
        if (!layer.short_conv_kernel && m.qk_norm != QkNorm::None) {
            const bool per_head = m.qk_norm == QkNorm::PerHead;
            specs.push_back({at + "q_norm.weight", {per_head ? m.head_dim : m.num_attention_heads * m.head_dim}});
            specs.push_back({at + "k_norm.weight", {per_head ? m.head_dim : m.num_key_value_heads * m.head_dim}});
        }
    }
    return specs;
}

namespace detail {

inline std::vector<std::string> split(const std::string& s) {
    std::vector<std::string> parts;
    size_t from = 0;
    for (size_t dot; (dot = s.find('.', from)) != std::string::npos; from = dot + 1) parts.push_back(s.substr(from, dot - from));
    parts.push_back(s.substr(from));
    return parts;
}

inline const char* component(const std::string& name) {
    static const std::pair<const char*, const char*> table[] = {
        {"input_norm", "attn_norm"}, {"post_norm", "ffn_norm"}, {"q", "attn_q"}, {"k", "attn_k"}, {"v", "attn_v"},
        {"o", "attn_output"}, {"q_norm", "attn_q_norm"}, {"k_norm", "attn_k_norm"}, {"gate", "ffn_gate"},
        {"up", "ffn_up"}, {"down", "ffn_down"}};
    for (const auto& [canonical, source] : table)
        if (name == canonical) return source;
    return nullptr;
}

[[noreturn]] inline void weight_error(const std::string& name, const std::string& message) {
    throw Error(ErrorKind::Weight, name + ": " + message);
}

inline std::string show(const std::vector<size_t>& shape) {
    std::string out = "[";
    for (size_t i = 0; i < shape.size(); ++i) out += (i ? ", " : "") + std::to_string(shape[i]);
    return out + "]";
}

inline const MetadataValue& meta(const Reader& reader, const std::string& key) {
    const MetadataValue* v = reader.metadata_value(key);
    if (v == nullptr) fail("missing metadata key " + key);
    return *v;
}

inline const std::string& meta_string(const Reader& reader, const std::string& key) {
    const MetadataValue& v = meta(reader, key);
    if (v.type != MetadataType::String) fail("metadata key " + key + " is not a string");
    return v.as_string();
}

inline bool integer_value(const MetadataValue& v, int64_t* out) {
    switch (v.type) {
        case MetadataType::Uint8: case MetadataType::Uint16: case MetadataType::Uint32: case MetadataType::Uint64:
            *out = (int64_t)v.as_u64();
            return v.as_u64() <= (uint64_t)INT64_MAX;
        case MetadataType::Int8: case MetadataType::Int16: case MetadataType::Int32: case MetadataType::Int64:
            *out = v.as_i64();
            return true;
        default: return false;
    }
}

inline size_t meta_usize(const Reader& reader, const std::string& key) {
    int64_t value = 0;
    if (!integer_value(meta(reader, key), &value) || value < 0) fail("metadata key " + key + " is not a non-negative integer");
    return (size_t)value;
}

inline std::vector<size_t> logical_shape(const TensorInfo& t, bool depthwise = false) {
    const auto& d = t.dimensions;
    if (d.size() == 1) return {(size_t)d[0]};
    if (d.size() == 2) return depthwise ? std::vector<size_t>{(size_t)d[1], 1, (size_t)d[0]} : std::vector<size_t>{(size_t)d[1], (size_t)d[0]};
    if (d.size() == 3) return {(size_t)d[2], (size_t)d[1], (size_t)d[0]};
    weight_error(t.name, "unsupported GGUF tensor rank " + std::to_string(d.size()));
}

inline bool dense_type(uint32_t id) { return id == 0 || id == 1 || id == 30; }
inline bool matrix_quantized_type(uint32_t id) {   // src/model/qwen_gguf.rs:238
    return id == 2 || id == 6 || id == 7 || id == 8 || id == 12 || id == 13 || id == 14;
}

inline bool ends_with(const std::string& s, const std::string& tail) {
    return s.size() >= tail.size() && s.compare(s.size() - tail.size(), tail.size(), tail) == 0;
}

}  // namespace detail

inline std::string qwen_source_name(const std::string& canonical) {
    if (canonical == "embedding.weight") return "token_embd.weight";
    if (canonical == "final_norm.weight") return "output_norm.weight";
    if (canonical == "lm_head.weight") return "output.weight";
    const auto parts = detail::split(canonical);
    if (parts.size() != 4 || parts[0] != "layers") detail::weight_error(canonical, "cannot map canonical Qwen weight");
    const char* component = detail::component(parts[2]);
    if (component == nullptr) detail::weight_error(canonical, "unsupported Qwen weight component");
    return "blk." + parts[1] + "." + component + "." + parts[3];
}

inline std::vector<std::string> lfm2_moe_source_names(const std::string& canonical) {
    if (canonical == "embedding.weight") return {"token_embd.weight"};
    if (canonical == "final_norm.weight") return {"token_embd_norm.weight"};
    const auto parts = detail::split(canonical);
    const auto unmapped = [&]() { detail::weight_error(canonical, "unmapped LFM2-MoE GGUF tensor"); };
    if (parts.size() == 5 && parts[0] == "layers" && parts[2] == "moe") {
        const std::string at = "blk." + parts[1] + ".";
        if (parts[3] == "router") return {at + "ffn_gate_inp.weight"};
        if (parts[3] == "router_bias") return {at + "exp_probs_b.bias"};
        if (parts[3] == "input") return {at + "ffn_gate_exps.weight", at + "ffn_up_exps.weight"};
        if (parts[3] == "output") return {at + "ffn_down_exps.weight"};
        unmapped();
    }
    if (parts.size() < 2 || parts[0] != "layers") unmapped();
    std::string component;
    if (parts.size() == 4 && parts[3] == "weight" && detail::component(parts[2]) != nullptr) {
        component = detail::component(parts[2]);
    } else if (parts.size() == 5 && parts[2] == "conv" && parts[4] == "weight" &&
               (parts[3] == "in_proj" || parts[3] == "depthwise" || parts[3] == "out_proj")) {
        component = parts[3] == "depthwise" ? "shortconv.conv" : "shortconv." + parts[3];
    } else {
        unmapped();
    }
    return {"blk." + parts[1] + "." + component + ".weight"};
}

enum class BindingKind { Dense, Quantized, Experts, StackedExperts };

// One canonical weight of the model and the tensor(s) of the file that hold it.
struct Binding {
    std::string canonical;
    std::vector<std::string> sources;
    std::vector<size_t> shape;   // logical: [rows, cols], [experts, rows, cols], [n] ...
    BindingKind kind = BindingKind::Dense;
    uint32_t type_id = 0;
};

struct TensorPlan {
    std::vector<Binding> bindings;
    bool redundant_output = false;   // a tied model whose file also carries output.weight
    size_t tensor_count = 0, source_tensor_bytes = 0, parameter_count = 0;

    const Binding& binding(const std::string& canonical) const {
        for (const Binding& b : bindings)
            if (b.canonical == canonical) return b;
        detail::weight_error(canonical, "missing mapped tensor");
    }
};

namespace detail {
template <class Skip>
inline void totals(const Reader& reader, TensorPlan* plan, Skip skip) {
    for (const auto& [name, t] : reader.tensors()) {
        plan->tensor_count += 1;
        plan->source_tensor_bytes += t.byte_len;
        if (skip(name)) continue;
        size_t elements = 1;
        for (uint64_t d : t.dimensions) elements *= (size_t)d;
        plan->parameter_count += elements;
    }
}
}  // namespace detail

inline std::pair<ModelShape, TensorPlan> plan_qwen(Reader& reader) {
    using namespace detail;
    const std::string arch = meta_string(reader, "general.architecture");
    if (arch != "qwen2" && arch != "qwen3")
        throw Error(ErrorKind::Config, "GGUF architecture \"" + arch + "\" is unsupported; expected qwen2 or qwen3");
    const bool qwen3 = arch == "qwen3";
    const bool has_output = reader.tensors().count("output.weight") != 0;
    ModelShape m;
    m.architecture = arch;
    m.tie_word_embeddings = has_output ? reader.tensors_equal_payload("token_embd.weight", "output.weight") : true;
    const auto embedding = reader.tensor("token_embd.weight").logical_matrix_shape();
    m.vocab_size = embedding[0];
    m.hidden_size = meta_usize(reader, arch + ".embedding_length");
    if (embedding[1] != m.hidden_size)
        throw Error(ErrorKind::Config, "token_embd.weight hidden dimension " + std::to_string(embedding[1]) +
                                           " differs from metadata " + std::to_string(m.hidden_size));
    m.num_attention_heads = meta_usize(reader, arch + ".attention.head_count");
    m.num_key_value_heads = meta_usize(reader, arch + ".attention.head_count_kv");
    if (qwen3) {
        m.head_dim = meta_usize(reader, "qwen3.attention.key_length");
        if (meta_usize(reader, "qwen3.attention.value_length") != m.head_dim)
            throw Error(ErrorKind::Config, "Qwen3 K/V head dimensions must match");
    } else if (reader.metadata_value("qwen2.rope.dimension_count") != nullptr) {
        m.head_dim = meta_usize(reader, "qwen2.rope.dimension_count");
    } else if (m.num_attention_heads != 0 && m.hidden_size % m.num_attention_heads == 0) {
        m.head_dim = m.hidden_size / m.num_attention_heads;
    } else {
        throw Error(ErrorKind::Config, "cannot infer head dimension from Qwen2 metadata");
    }
    const size_t intermediate = meta_usize(reader, arch + ".feed_forward_length");
    const size_t layers = meta_usize(reader, arch + ".block_count");
    if (m.vocab_size == 0 || m.hidden_size == 0 || m.num_attention_heads == 0 || m.num_key_value_heads == 0 ||
        m.head_dim == 0 || intermediate == 0 || layers == 0 || m.num_attention_heads % m.num_key_value_heads != 0)
        throw Error(ErrorKind::Config, "invalid Qwen model geometry");
    m.layers.assign(layers, LayerShape{intermediate, std::nullopt, std::nullopt});
    m.qk_norm = qwen3 ? QkNorm::PerHead : QkNorm::None;
    m.qkv_bias = !qwen3;

    struct Expected { std::string source, canonical; std::vector<size_t> shape; };
    std::vector<Expected> expected;
    for (const auto& [canonical, shape] : specifications(m)) expected.push_back({qwen_source_name(canonical), canonical, shape});
    TensorPlan plan;
    plan.redundant_output = m.tie_word_embeddings && has_output;
    if (m.qkv_bias)
        for (size_t l = 0; l < layers; ++l) {
            const std::pair<const char*, size_t> biases[] = {{"q", m.num_attention_heads * m.head_dim},
                                                             {"k", m.num_key_value_heads * m.head_dim},
                                                             {"v", m.num_key_value_heads * m.head_dim}};
            for (const auto& [name, length] : biases)
                expected.push_back({"blk." + std::to_string(l) + ".attn_" + name + ".bias",
                                    "layers." + std::to_string(l) + "." + name + ".bias", {length}});
        }
    if (reader.tensors().count("output.bias") != 0) {
        if (qwen3) weight_error("output.bias", "Qwen3 output projection has no bias");
        expected.push_back({"output.bias", "lm_head.bias", {m.vocab_size}});
    }
    std::set<std::string> names;
    for (const Expected& e : expected) {
        names.insert(e.source);
        const TensorInfo& t = reader.tensor(e.source);
        if (t.dimensions.size() > 2) weight_error(e.source, "unsupported Qwen tensor rank " + std::to_string(t.dimensions.size()));
        const auto found = logical_shape(t);
        if (found != e.shape) weight_error(e.source, "expected shape " + show(e.shape) + ", found " + show(found));
        BindingKind kind;
        if (dense_type(t.type_id)) kind = BindingKind::Dense;
        else if (matrix_quantized_type(t.type_id) && e.shape.size() == 2) kind = BindingKind::Quantized;
        else weight_error(e.source, "unsupported GGML type " + std::to_string(t.type_id) + " for Qwen tensor");
        plan.bindings.push_back({e.canonical, {e.source}, e.shape, kind, t.type_id});
    }
    for (const auto& [name, t] : reader.tensors())
        if (names.count(name) == 0 && !(plan.redundant_output && name == "output.weight"))
            weight_error(name, "unexpected tensor for supported Qwen GGUF contract");
    totals(reader, &plan, [&](const std::string& n) { return plan.redundant_output && n == "output.weight"; });
    return {m, plan};
}

// Layers whose entry in the per-layer KV-head schedule is zero are short convolutions; the
// first leading_dense_block_count layers are dense, the rest sparse.  Whether the router has
// a selection bias and whether the output projection is tied come from the model's
// companion config in the reference, hence the two arguments.
inline ModelShape lfm2_moe_shape(const Reader& reader, bool use_expert_bias = true, bool tie_word_embeddings = true) {
    using namespace detail;
    const char* differs = "LFM2-MoE GGUF metadata differs from the companion official config";
    const char* schedule_differs = "LFM2-MoE GGUF per-layer KV-head schedule differs from config";
    if (meta_string(reader, "general.architecture") != "lfm2moe") throw Error(ErrorKind::Config, differs);
    if (meta_usize(reader, "lfm2moe.expert_gating_func") != 2) throw Error(ErrorKind::Config, differs);
    ModelShape m;
    m.architecture = "lfm2moe";
    m.hidden_size = meta_usize(reader, "lfm2moe.embedding_length");
    m.num_attention_heads = meta_usize(reader, "lfm2moe.attention.head_count");
    const size_t layers = meta_usize(reader, "lfm2moe.block_count");
    const MetadataValue& schedule = meta(reader, "lfm2moe.attention.head_count_kv");
    if (schedule.type != MetadataType::Array || schedule.as_array().values.size() != layers)
        throw Error(ErrorKind::Config, schedule_differs);
    std::vector<int64_t> kv(layers, 0);
    std::set<int64_t> live;
    for (size_t l = 0; l < layers; ++l) {
        if (!integer_value(schedule.as_array().values[l], &kv[l])) throw Error(ErrorKind::Config, schedule_differs);
        if (kv[l] != 0) live.insert(kv[l]);
    }
    if (live.size() != 1 || *live.begin() < 0 || m.num_attention_heads == 0 || m.hidden_size % m.num_attention_heads != 0)
        throw Error(ErrorKind::Config, schedule_differs);
    const size_t dense_layers = meta_usize(reader, "lfm2moe.leading_dense_block_count");
    const SparseFeedForward sparse{meta_usize(reader, "lfm2moe.expert_count"),
                                   meta_usize(reader, "lfm2moe.expert_feed_forward_length"), use_expert_bias};
    const size_t intermediate = meta_usize(reader, "lfm2moe.feed_forward_length");
    const size_t taps = meta_usize(reader, "lfm2moe.shortconv.l_cache");
    m.vocab_size = meta_usize(reader, "lfm2moe.vocab_size");
    m.num_key_value_heads = (size_t)*live.begin();
    m.head_dim = m.hidden_size / m.num_attention_heads;
    m.tie_word_embeddings = tie_word_embeddings;
    m.qk_norm = QkNorm::PerHead;
    for (size_t l = 0; l < layers; ++l) {
        LayerShape layer;
        layer.intermediate_size = intermediate;
        if (kv[l] == 0) layer.short_conv_kernel = taps;
        if (l >= dense_layers) layer.sparse = sparse;
        m.layers.push_back(layer);
    }
    return m;
}

inline TensorPlan plan_lfm2_moe(Reader& reader, const ModelShape& m) {
    using namespace detail;
    TensorPlan plan;
    plan.redundant_output = m.tie_word_embeddings && reader.tensors().count("output.weight") != 0;
    if (plan.redundant_output && !reader.tensors_equal_payload("token_embd.weight", "output.weight"))
        weight_error("output.weight", "tied GGUF output weights differ from token embeddings");
    const auto specs = specifications(m);
    std::set<std::string> expected;
    for (const auto& [canonical, shape] : specs)
        for (const std::string& source : lfm2_moe_source_names(canonical)) expected.insert(source);
    if (plan.redundant_output) expected.insert("output.weight");
    for (const auto& [name, t] : reader.tensors())
        if (expected.count(name) == 0) weight_error(name, "unexpected tensor for the supported LFM2-MoE GGUF contract");

    const auto expert_component = [&](const std::string& name, const std::vector<size_t>& want) -> const TensorInfo& {
        const TensorInfo& t = reader.tensor(name);
        const auto shape = t.logical_expert_shape();
        const std::vector<size_t> found(shape.begin(), shape.end());
        if (found != want) weight_error(name, "expected logical expert shape " + show(want) + ", found " + show(found));
        if (t.type_id < 12 || t.type_id > 14) weight_error(name, "LFM2-MoE GGUF expert projections must use Q4_K, Q5_K, or Q6_K");
        return t;
    };
    for (const auto& [canonical, shape] : specs) {
        const auto sources = lfm2_moe_source_names(canonical);
        const bool input = ends_with(canonical, ".moe.input.weight"), output = ends_with(canonical, ".moe.output.weight");
        if (input || output) {
            const size_t layer = std::stoul(split(canonical)[1]);
            if (!m.layers[layer].sparse) throw Error(ErrorKind::Config, "GGUF expert tensor targets a dense layer");
            const SparseFeedForward& s = *m.layers[layer].sparse;
            if (input) {
                const std::vector<size_t> want = {s.experts, s.intermediate_size, m.hidden_size};
                const TensorInfo& gate = expert_component(sources[0], want);
                const TensorInfo& up = expert_component(sources[1], want);
                if (gate.type_id != up.type_id) weight_error(canonical, "gate/up expert tensors use different quantization formats");
                plan.bindings.push_back({canonical, sources, shape, BindingKind::StackedExperts, gate.type_id});
            } else {
                const TensorInfo& t = expert_component(sources[0], {s.experts, m.hidden_size, s.intermediate_size});
                plan.bindings.push_back({canonical, sources, shape, BindingKind::Experts, t.type_id});
            }
            continue;
        }
        const TensorInfo& t = reader.tensor(sources[0]);
        const auto found = logical_shape(t, ends_with(canonical, ".conv.depthwise.weight"));
        if (found != shape) weight_error(sources[0], "expected logical shape " + show(shape) + ", found " + show(found));
        BindingKind kind = BindingKind::Dense;
        if (matrix_quantized_type(t.type_id)) {
            if (shape.size() != 2) weight_error(sources[0], "quantized non-expert GGUF tensors must be matrices");
            kind = BindingKind::Quantized;
        } else if (!dense_type(t.type_id)) {
            weight_error(sources[0], "unsupported GGML tensor type " + std::to_string(t.type_id));
        }
        plan.bindings.push_back({canonical, sources, shape, kind, t.type_id});
    }
    totals(reader, &plan, [&](const std::string& n) {
        return ends_with(n, ".exp_probs_b.bias") || (plan.redundant_output && n == "output.weight");
    });
    return plan;
}

// The plan's quantized tensors on the device under their canonical names.
struct BoundWeights {
    std::map<std::string, QuantizedMatrix> matrices;
    std::map<std::string, QuantizedExpertMatrix> experts;
    size_t quantized_tensor_bytes = 0;
};

inline BoundWeights bind_quantized(const Device& device, Reader& reader, const TensorPlan& plan) {
    BoundWeights bound;
    for (const Binding& b : plan.bindings) {
        if (b.kind == BindingKind::Dense) continue;
        if (b.kind == BindingKind::Quantized) {
            QuantizedMatrix w = load_quantized_matrix(device, reader, b.sources[0]);
            if (std::vector<size_t>{w.rows(), w.columns()} != b.shape)
                detail::weight_error(b.canonical, "packed matrix shape differs from model policy");
            bound.quantized_tensor_bytes += w.byte_size();
            bound.matrices.emplace(b.canonical, std::move(w));
            continue;
        }
        QuantizedExpertMatrix w = b.kind == BindingKind::Experts
                                      ? load_quantized_expert_matrix(device, reader, b.sources[0])
                                      : load_quantized_input_experts(device, reader, b.sources[0], b.sources[1]);
        if (std::vector<size_t>{w.experts(), w.rows_per_expert(), w.columns()} != b.shape)
            detail::weight_error(b.canonical, "packed gate/up expert shape differs from model policy");
        bound.quantized_tensor_bytes += w.byte_size();
        bound.experts.emplace(b.canonical, std::move(w));
    }
    return bound;
}

}  // namespace models
}  // namespace gguf
}  // namespace ferrum

#endif  // FERRUM_GGUF_MODELS_HPP
