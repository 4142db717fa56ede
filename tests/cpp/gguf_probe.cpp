// Prints what ferrum::gguf::Reader finds in the file named by argv[1], one item a
// line, for the CPU tests to compare with the Python reader; a rejected file
// prints "error: <message>" and exits with 2.  argv[2], when given, is the
// array-skipping limit; argv[3] == "untagged" drops the architecture rule.
// "<file> plan qwen" and "<file> plan lfm2moe [nobias]" print the model-level binding of the
// file's tensors instead (exit 3 for a rejection that is not of the Gguf kind).
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "ferrum_gguf_models.hpp"

using namespace ferrum;

static void print(const gguf::MetadataValue& v) {
    switch (v.type) {
        case gguf::MetadataType::String: std::printf("%s", v.as_string().c_str()); break;
        case gguf::MetadataType::Bool: std::printf("%s", v.as_bool() ? "True" : "False"); break;
        case gguf::MetadataType::Float32:
        case gguf::MetadataType::Float64: std::printf("%.17g", v.as_f64()); break;
        case gguf::MetadataType::Uint8: case gguf::MetadataType::Uint16: case gguf::MetadataType::Uint32:
        case gguf::MetadataType::Uint64: std::printf("%" PRIu64, v.as_u64()); break;
        case gguf::MetadataType::Array:
            std::printf("[");
            for (const auto& item : v.as_array().values) { print(item); std::printf(","); }
            std::printf("]");
            break;
        default: std::printf("%" PRId64, v.as_i64());
    }
}

static void print_plan(const gguf::models::ModelShape& m, const gguf::models::TensorPlan& plan) {
    std::printf("shape %s vocab %zu hidden %zu heads %zu kv %zu head_dim %zu layers %zu tied %d bias %d qk_norm %d\n",
                m.architecture.c_str(), m.vocab_size, m.hidden_size, m.num_attention_heads, m.num_key_value_heads,
                m.head_dim, m.layers.size(), (int)m.tie_word_embeddings, (int)m.qkv_bias, (int)m.qk_norm);
    for (const auto& b : plan.bindings) {
        std::printf("bind %s <-", b.canonical.c_str());
        for (const auto& source : b.sources) std::printf(" %s", source.c_str());
        std::printf(" shape");
        for (size_t d : b.shape) std::printf(" %zu", d);
        std::printf(" kind %d type %u\n", (int)b.kind, b.type_id);
    }
    std::printf("totals %zu tensors %zu bytes %zu parameters redundant %d\n", plan.tensor_count, plan.source_tensor_bytes,
                plan.parameter_count, (int)plan.redundant_output);
}

int main(int argc, char** argv) {
    if (argc < 2) return 64;
    try {
        if (argc >= 4 && !std::strcmp(argv[2], "plan")) {
            gguf::Reader file = gguf::Reader::open(argv[1]);
            if (!std::strcmp(argv[3], "qwen")) {
                const auto [shape, plan] = gguf::models::plan_qwen(file);
                print_plan(shape, plan);
            } else {
                const auto shape = gguf::models::lfm2_moe_shape(file, !(argc > 4 && !std::strcmp(argv[4], "nobias")));
                print_plan(shape, gguf::models::plan_lfm2_moe(file, shape));
            }
            return 0;
        }
        if (argc == 5 && !std::strcmp(argv[2], "stack")) {   // <file> stack <gate> <up>: FNV-1a of the interleaved rows
            gguf::Reader file = gguf::Reader::open(argv[1]);
            const auto shape = file.tensor(argv[3]).logical_expert_shape();
            std::vector<uint8_t> payload(2 * file.tensor(argv[3]).byte_len);
            gguf::read_stacked_experts(file, argv[3], argv[4], payload.data(), payload.size());
            uint64_t h = 1469598103934665603ull;
            for (uint8_t b : payload) h = (h ^ b) * 1099511628211ull;
            std::printf("stacked %zu %zu %zu fnv %016" PRIx64 "\n", shape[0], 2 * shape[1], shape[2], h);
            return 0;
        }
        const uint64_t limit = argc > 2 ? std::strtoull(argv[2], nullptr, 10) : UINT64_MAX;
        gguf::Reader file = gguf::Reader::open(argv[1], limit, !(argc > 3 && !std::strcmp(argv[3], "untagged")));
        std::printf("version %u alignment %" PRIu64 " data %" PRIu64 "\n", file.version(), file.alignment(),
                    file.tensor_data_offset());
        for (const auto& [key, value] : file.metadata()) {
            std::printf("meta %s %u ", key.c_str(), static_cast<uint32_t>(value.type));
            print(value);
            std::printf("\n");
        }
        for (const auto& [name, t] : file.tensors()) {
            std::vector<uint8_t> payload(t.byte_len);
            file.read_tensor_into(name, payload.data(), payload.size());
            uint64_t streamed = 1469598103934665603ull, whole = streamed;   // FNV-1a over both read paths
            for (uint8_t b : payload) whole = (whole ^ b) * 1099511628211ull;
            file.stream_tensor(name, 1000, [&](const uint8_t* p, size_t n) {
                for (size_t i = 0; i < n; ++i) streamed = (streamed ^ p[i]) * 1099511628211ull;
            });
            std::printf("tensor %s type %u offset %" PRIu64 " bytes %zu dims", name.c_str(), t.type_id, t.offset,
                        t.byte_len);
            for (uint64_t dim : t.dimensions) std::printf(" %" PRIu64, dim);
            std::printf(" fnv %016" PRIx64 " %s\n", whole, whole == streamed ? "stream-ok" : "stream-differs");
        }
    } catch (const Error& e) {
        std::printf("error: %s\n", e.what());
        return e.kind() == ErrorKind::Gguf ? 2 : 3;
    }
    return 0;
}
