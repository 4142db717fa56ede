// Exercises the C++ host side (include/ferrum_hip.hpp) on the GPU and checks
// it against the CPU oracle.  The cases follow the reference's operator tests:
// embedding gather bitwise (src/ops/transformer.rs:3307-3329), GEMV / GEMM
// against the CPU dequant (src/diffusion/tests.rs:718-761), shape and ownership
// errors (src/ops/mod.rs:553-609), and the routed FFN against a host evaluation
// (src/nn/moe.rs:602-651).  Prints one line per case; exit status 0 = all passed.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "ferrum_gguf_models.hpp"
#include "ferrum_hip.hpp"

extern "C" {
int fo_dequantize(uint32_t ggml_type, const uint8_t* packed, size_t rows, size_t cols, float* out);
int fo_project_f64(uint32_t ggml_type, const uint8_t* packed, size_t n, size_t k, const float* x,
                   size_t m, float* y, int weight_round, int threads);
int fo_select_routes(const float* logits, size_t tokens, size_t experts, size_t top_k, int sigmoid,
                     int normalize, float eps, float scaling, const float* bias, float* metadata);
void fo_expert_assign(const float* hidden, const float* metadata, size_t assignments, size_t width, float* out);
int fo_expert_project(uint32_t ggml_type, const uint8_t* packed, size_t experts, size_t rows, size_t k,
                      const float* x, const float* metadata, size_t assignments, float* y, int weight_round,
                      int out_round, int f64);
void fo_expert_silu_mul(const float* in, size_t assignments, size_t intermediate, uint32_t dtype, float* out);
void fo_expert_combine(const float* in, const float* metadata, size_t tokens, size_t hidden, size_t top_k,
                       uint32_t dtype, float* out);
void fo_round_storage_array(const float* in, size_t n, uint32_t dtype, float* out);
void fo_moe_map(const uint32_t* ids, size_t experts, size_t routes, uint32_t* offsets, uint32_t* sorted,
                uint32_t* position);
void fo_add_rmsnorm(const float* a, const float* b, const float* weight, size_t rows, size_t width, float eps,
                    uint32_t dtype, float* residual, float* normed);
}

using namespace ferrum;

static int failures = 0;
static void report(const char* name, bool ok, double figure = 0) {
    std::printf("%-58s %s  %.3g\n", name, ok ? "ok" : "FAILED", figure);
    std::fflush(stdout);
    if (!ok) ++failures;
}

struct Rng {  // splitmix64
    uint64_t s;
    uint64_t next() {
        uint64_t z = (s += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    double uniform() { return (double)(next() >> 11) / 9007199254740992.0; }
    float normal() { return (float)(std::sqrt(-2.0 * std::log(uniform() + 1e-300)) * std::cos(6.283185307179586 * uniform())); }
};

// Random super-blocks with small finite f16 scales.
static std::vector<uint8_t> blocks(QuantizationFormat f, size_t rows, size_t cols, uint64_t seed) {
    Rng rng{seed};
    const size_t bb = block_bytes(f), n = rows * (cols / 256);
    std::vector<uint8_t> out(n * bb);
    for (auto& b : out) b = (uint8_t)rng.next();
    for (size_t i = 0; i < n; ++i) {
        uint8_t* blk = out.data() + i * bb;
        const uint16_t d = f32_to_f16_bits((float)(std::fabs(rng.normal()) * (f == QuantizationFormat::Q4_K ? 0.01 : 0.002)));
        if (f == QuantizationFormat::Q4_K) {
            const uint16_t dmin = f32_to_f16_bits((float)(std::fabs(rng.normal()) * 0.005));
            std::memcpy(blk, &d, 2);
            std::memcpy(blk + 2, &dmin, 2);
        } else {
            std::memcpy(blk + 208, &d, 2);
        }
    }
    return out;
}

static double rel_l2(const std::vector<float>& a, const std::vector<float>& b) {
    double num = 0, den = 0;
    for (size_t i = 0; i < a.size(); ++i) {
        num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]);
        den += (double)b[i] * b[i];
    }
    return std::sqrt(num / den);
}

static QuantizedMatrix upload(const Device& d, QuantizationFormat f, size_t rows, size_t cols,
                              const std::vector<uint8_t>& bytes) {
    return d.quantized_matrix(rows, cols, f, [&](uint8_t* dst, size_t n) { std::memcpy(dst, bytes.data(), n); });
}

// A GGUF v3 file holding the given K-quant tensors back to back at 32-byte
// aligned offsets (the layout src/loader/gguf.rs:709-748 builds for its tests).
struct FileTensor {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t type;
    const std::vector<uint8_t>* payload;
};
static std::string gguf_file(const std::vector<FileTensor>& tensors, const std::string& architecture = "qwen3moe",
                             const std::vector<std::pair<std::string, uint32_t>>& numbers = {}) {
    std::string out("GGUF");
    auto put = [&out](const void* p, size_t n) { out.append(static_cast<const char*>(p), n); };
    auto u32 = [&](uint32_t v) { put(&v, 4); };
    auto u64 = [&](uint64_t v) { put(&v, 8); };
    auto str = [&](const std::string& v) { u64(v.size()); out += v; };
    u32(3);
    u64(tensors.size());
    u64(2 + numbers.size());
    str("general.architecture"); u32(8); str(architecture);
    str("general.quantization_version"); u32(4); u32(2);
    for (const auto& [key, value] : numbers) { str(key); u32(4); u32(value); }
    uint64_t cursor = 0;
    std::vector<uint64_t> offsets;
    for (const auto& t : tensors) {
        str(t.name);
        u32((uint32_t)t.dims.size());
        for (uint64_t dim : t.dims) u64(dim);
        u32(t.type);
        u64(cursor);
        offsets.push_back(cursor);
        cursor = (cursor + t.payload->size() + 31) / 32 * 32;
    }
    out.resize((out.size() + 31) / 32 * 32, '\0');
    const size_t base = out.size();
    out.resize(base + cursor, '\0');
    for (size_t i = 0; i < tensors.size(); ++i)
        std::memcpy(&out[base + offsets[i]], tensors[i].payload->data(), tensors[i].payload->size());
    return out;
}

int main() {
    Device d(0);
    const uint32_t kF16 = 1;
    for (QuantizationFormat f : {QuantizationFormat::Q4_K, QuantizationFormat::Q6_K}) {
        const uint32_t type = static_cast<uint32_t>(f);
        const size_t n = 200, k = 1024;
        const auto packed = blocks(f, n, k, 11 + type);
        QuantizedMatrix w = upload(d, f, n, k, packed);

        std::vector<float> want(n * k);
        fo_dequantize(type, packed.data(), n, k, want.data());
        const auto dense = d.dequantize(w).to_f32();
        report(f == QuantizationFormat::Q4_K ? "q4_k dequantize is bit-exact" : "q6_k dequantize is bit-exact",
               std::memcmp(dense.data(), want.data(), want.size() * 4) == 0);

        const std::vector<uint32_t> tokens = {3, 0, 199, 3};
        const auto gathered = d.embedding_gather_quantized(w, tokens, DType::BF16).tensor.to_f32();
        bool same = true;
        for (size_t t = 0; t < tokens.size(); ++t)
            for (size_t c = 0; c < k; ++c)
                same &= gathered[t * k + c] == bf16_bits_to_f32(f32_to_bf16_bits(want[tokens[t] * k + c]));
        report("embedding gather matches the rounded dequant bitwise", same);

        Rng rng{5};
        std::vector<float> x(k);
        for (auto& v : x) v = rng.normal();
        std::vector<float> ref(n);
        fo_project_f64(type, packed.data(), n, k, x.data(), 1, ref.data(), 0, 4);
        Output y = d.project_quantized(d.from_f32({1, k}, DType::F32, x), w);
        report(("gemv vs f64 oracle: " + y.metrics.operation).c_str(), rel_l2(y.tensor.to_f32(), ref) <= 1e-5,
               rel_l2(y.tensor.to_f32(), ref));

        const size_t m = 8;
        std::vector<float> xm(m * k);
        for (auto& v : xm) v = f16_bits_to_f32(f32_to_f16_bits(rng.normal()));
        std::vector<float> refm(m * n);
        fo_project_f64(type, packed.data(), n, k, xm.data(), m, refm.data(), kF16, 4);
        const DType f32 = DType::F32;
        Output ym = d.project_quantized(d.from_f32({m, k}, DType::F16, xm), w, nullptr, &f32);
        report(("small-M gemm vs f16-tile oracle: " + ym.metrics.operation).c_str(),
               rel_l2(ym.tensor.to_f32(), refm) <= 1e-5, rel_l2(ym.tensor.to_f32(), refm));

        bool threw = false;
        try {
            d.project_quantized(d.from_f32({1, k / 2}, DType::F32, std::vector<float>(k / 2, 1.f)), w);
        } catch (const Error& e) {
            threw = e.kind() == ErrorKind::Shape;
        }
        report("mismatched K is Error::Shape", threw);
    }
    {
        bool threw = false;
        try {
            d.quantized_matrix(4, 256, QuantizationFormat::Q4_K, [](uint8_t* dst, size_t n) {
                std::memset(dst, 0, n);
                dst[1] = 0x7c;  // d = +inf
            });
        } catch (const Error& e) {
            threw = e.kind() == ErrorKind::Weight;
        }
        report("non-finite block scale is Error::Weight", threw);
    }
    {
        // routed FFN: 8 experts, hidden 512, intermediate 256, top-2, 40 tokens, f32 activations
        const size_t experts = 8, hidden = 512, inter = 256, top_k = 2, tokens = 40;
        const auto win = blocks(QuantizationFormat::Q4_K, experts * 2 * inter, hidden, 21);
        const auto wout = blocks(QuantizationFormat::Q4_K, experts * hidden, inter, 22);
        Rng rng{23};
        std::vector<float> x(tokens * hidden), logits(tokens * experts);
        for (auto& v : x) v = rng.normal();
        for (auto& v : logits) v = rng.normal();
        auto copy_from = [](const std::vector<uint8_t>& src) {
            return [&src](uint8_t* dst, size_t n) { std::memcpy(dst, src.data(), n); };
        };
        SparseMoe moe(d, d.quantized_expert_matrix(experts, 2 * inter, hidden, QuantizationFormat::Q4_K, copy_from(win)),
                      d.quantized_expert_matrix(experts, hidden, inter, QuantizationFormat::Q4_K, copy_from(wout)),
                      MoeRoutingPolicy{experts, top_k});
        const auto got = moe.forward(d.from_f32({tokens, hidden}, DType::F32, x),
                                     d.from_f32({tokens, experts}, DType::F32, logits)).to_f32();
        const size_t a = tokens * top_k;
        std::vector<float> meta(a * 3), assigned(a * hidden), up(a * 2 * inter), act(a * inter), down(a * hidden),
            want(tokens * hidden);
        fo_select_routes(logits.data(), tokens, experts, top_k, 0, 1, 0.f, 1.f, nullptr, meta.data());
        fo_expert_assign(x.data(), meta.data(), a, hidden, assigned.data());
        fo_expert_project(FH_GGML_Q4_K, win.data(), experts, 2 * inter, hidden, assigned.data(), meta.data(), a,
                          up.data(), 0, 0, 1);
        fo_expert_silu_mul(up.data(), a, inter, 0, act.data());
        fo_expert_project(FH_GGML_Q4_K, wout.data(), experts, hidden, inter, act.data(), meta.data(), a, down.data(),
                          0, 0, 1);
        fo_expert_combine(down.data(), meta.data(), tokens, hidden, top_k, 0, want.data());
        report("SparseMoe::forward vs host evaluation", rel_l2(got, want) <= 2e-5, rel_l2(got, want));

        // decode-sized batch: the fused projections give the bits of the separate steps
        const size_t few = 3;
        Tensor xs = d.from_f32({few, hidden}, DType::F16, std::vector<float>(x.begin(), x.begin() + few * hidden));
        Tensor ls = d.from_f32({few, experts}, DType::F32, std::vector<float>(logits.begin(), logits.begin() + few * experts));
        const auto fused = moe.forward(xs, ls).to_f32();
        moe.fuse_inputs = false;
        const auto separate = moe.forward(xs, ls).to_f32();
        report("SparseMoe::forward decode path equals the separate steps bitwise",
               std::memcmp(fused.data(), separate.data(), fused.size() * 4) == 0);

        // a shared expert: with one token it rides in the routed launches, and every launch is the
        // per-row kernel either way, so the two orchestrations give the same bits
        const auto sin = blocks(QuantizationFormat::Q4_K, 2 * inter, hidden, 25);
        const auto sout = blocks(QuantizationFormat::Q4_K, hidden, inter, 26);
        moe.set_shared_expert(upload(d, QuantizationFormat::Q4_K, 2 * inter, hidden, sin),
                              upload(d, QuantizationFormat::Q4_K, hidden, inter, sout));
        Tensor x1 = d.from_f32({1, hidden}, DType::F16, std::vector<float>(x.begin(), x.begin() + hidden));
        Tensor l1 = d.from_f32({1, experts}, DType::F32, std::vector<float>(logits.begin(), logits.begin() + experts));
        Tensor gate1 = d.from_f32({1}, DType::F32, std::vector<float>{0.625f});
        moe.fuse_inputs = true;
        const auto riding = moe.forward(x1, l1, nullptr, &gate1).to_f32();
        const bool rode = d.last_operation() == std::string("h_moe_combine");
        moe.fuse_inputs = false;
        const auto apart = moe.forward(x1, l1, nullptr, &gate1).to_f32();
        float peak = 0.f;
        for (float v : riding) peak = std::max(peak, std::fabs(v));
        report("SparseMoe with a shared expert: riding in the routed launches equals the separate calls bitwise",
               rode && peak > 1e-4f && std::memcmp(riding.data(), apart.data(), riding.size() * 4) == 0, peak);
        bool refused = false;
        try {
            moe.set_shared_expert(upload(d, QuantizationFormat::Q4_K, 2 * inter, hidden, sin),
                                  upload(d, QuantizationFormat::Q4_K, 2 * inter, hidden, sin));
        } catch (const Error& e) {
            refused = e.kind() == ErrorKind::Config;
        }
        report("a shared expert whose output matrix does not fit is Error::Config", refused);

        // chunks: 80 f16 tokens, twenty to a chunk (enough assignments for the grouped kernels), against the pass that is not cut (src/nn/moe.rs:467-520)
        {
            const size_t many = 80;
            std::vector<float> xm(many * hidden), lm(many * experts);
            for (size_t t = 0; t < many; ++t) {
                std::copy(x.begin() + (t % tokens) * hidden, x.begin() + (t % tokens + 1) * hidden, xm.begin() + t * hidden);
                for (size_t j = 0; j < experts; ++j) lm[t * experts + j] = logits[(t % tokens) * experts + (j + t) % experts];
            }
            Tensor xt = d.from_f32({many, hidden}, DType::F16, xm), lt = d.from_f32({many, experts}, DType::F32, lm);
            std::vector<float> gates(many);
            for (size_t t = 0; t < many; ++t) gates[t] = 0.25f + 0.01f * (float)t;
            Tensor gt = d.from_f32({many}, DType::F32, gates);
            moe.fuse_inputs = true;
            (void)moe.take_stats();
            const auto whole = moe.forward(xt, lt, nullptr, &gt).to_f32();
            const MoeStats ws = moe.take_stats();
            const size_t before = d.moe_routing_temporary_limit(), per_token = moe.temporary_bytes(1, DType::F16);
            d.set_moe_routing_temporary_limit(20 * per_token + 1);
            const auto cut = moe.forward(xt, lt, nullptr, &gt).to_f32();
            const MoeStats cs = moe.take_stats();
            d.set_moe_routing_temporary_limit(before);
            const auto one_call = moe.forward_in_one_call(xt, lt, nullptr, &gt).to_f32();
            report("fh_moe_ffn gives the bits of SparseMoe::forward", std::memcmp(one_call.data(), whole.data(), whole.size() * 4) == 0);
            report("SparseMoe::forward in chunks gives the bits of the whole pass",
                   before == (size_t(128) << 20) && std::memcmp(cut.data(), whole.data(), cut.size() * 4) == 0 &&
                       ws.assignments == many * top_k && cs.assignments == many * top_k && !cs.active_experts_known &&
                       ws.peak_temporary_bytes == many * per_token && cs.peak_temporary_bytes == 20 * per_token &&
                       moe.take_stats().assignments == 0);
        }

        Device other(0);
        bool threw = false;
        try {
            d.project_quantized(other.from_f32({1, 256}, DType::F32, std::vector<float>(256, 1.f)),
                                upload(d, QuantizationFormat::Q4_K, 4, 256, blocks(QuantizationFormat::Q4_K, 4, 256, 3)));
        } catch (const Error& e) {
            threw = e.kind() == ErrorKind::DeviceMismatch;
        }
        report("a tensor of another device is Error::DeviceMismatch", threw);

        // Q8_0 rows of 2880 weights: ninety 34-byte blocks, which is not whole runs of eight (src/loader/gguf.rs:99)
        {
            const size_t qn = 96, qk = 2880, qblocks = qn * (qk / 32);
            Rng qr{77};
            std::vector<uint8_t> q8(qblocks * 34);
            for (auto& b : q8) b = (uint8_t)qr.next();
            for (size_t i = 0; i < qblocks; ++i) {
                const uint16_t scale = f32_to_f16_bits((float)(std::fabs(qr.normal()) * 0.002));
                std::memcpy(q8.data() + i * 34, &scale, 2);
            }
            QuantizedMatrix qw = upload(d, QuantizationFormat::Q8_0, qn, qk, q8);
            std::vector<float> dense(qn * qk), qx(2 * qk), qref(2 * qn);
            fo_dequantize(FH_GGML_Q8_0, q8.data(), qn, qk, dense.data());
            const auto on_device = d.dequantize(qw, DType::F32).to_f32();
            for (auto& v : qx) v = qr.normal();
            fo_project_f64(FH_GGML_Q8_0, q8.data(), qn, qk, qx.data(), 2, qref.data(), 0, 1);
            const auto qy = d.project_quantized(d.from_f32({2, qk}, DType::F32, qx), qw);
            report("Q8_0 rows of ninety blocks: dequantize bit-exact, projection vs f64 oracle",
                   qw.byte_size() == q8.size() && std::memcmp(on_device.data(), dense.data(), dense.size() * 4) == 0 &&
                       rel_l2(qy.tensor.to_f32(), qref) <= 1e-5,
                   rel_l2(qy.tensor.to_f32(), qref));
        }
    }
    {
        // an execution records the calls and replays them
        const size_t n = 256, k = 512;
        const auto packed = blocks(QuantizationFormat::Q4_K, n, k, 31);
        QuantizedMatrix w = upload(d, QuantizationFormat::Q4_K, n, k, packed);
        Tensor x = d.from_f32({1, k}, DType::F32, std::vector<float>(k, 0.5f));
        Tensor y = d.zeros({1, n}, DType::F32);
        const auto eager = d.project_quantized(x, w).tensor.to_f32();
        Graph graph = d.execution([&] { d.project_quantized(x, w, &y); });
        graph.launch();
        graph.launch();
        const auto replayed = y.to_f32();
        report("a recorded execution replays the projection bitwise",
               std::memcmp(eager.data(), replayed.data(), eager.size() * 4) == 0);
    }
    {
        // tensors read from a GGUF stream reach the device unchanged
        const size_t n = 96, k = 768, experts = 3, rows = 32;
        const auto q4 = blocks(QuantizationFormat::Q4_K, n, k, 41);
        const auto q6 = blocks(QuantizationFormat::Q6_K, n, k, 42);
        const auto ex = blocks(QuantizationFormat::Q4_K, experts * rows, k, 43);
        std::istringstream stream(gguf_file({{"blk.0.attn_q.weight", {k, n}, FH_GGML_Q4_K, &q4},
                                             {"output.weight", {k, n}, FH_GGML_Q6_K, &q6},
                                             {"blk.0.ffn_down_exps.weight", {k, rows, experts}, FH_GGML_Q4_K, &ex}}));
        gguf::Reader file(stream);
        bool exact = true;
        for (const auto& [name, packed] : {std::pair<const char*, const std::vector<uint8_t>*>{"blk.0.attn_q.weight", &q4},
                                           {"output.weight", &q6}}) {
            QuantizedMatrix w = gguf::load_quantized_matrix(d, file, name);
            std::vector<float> want(n * k);
            fo_dequantize(static_cast<uint32_t>(w.format()), packed->data(), n, k, want.data());
            const auto dense = d.dequantize(w).to_f32();
            exact &= w.rows() == n && w.columns() == k && std::memcmp(dense.data(), want.data(), want.size() * 4) == 0;
        }
        report("matrices loaded from GGUF dequantize bit-exactly", exact);
        QuantizedExpertMatrix e = gguf::load_quantized_expert_matrix(d, file, "blk.0.ffn_down_exps.weight");
        std::vector<float> want(experts * rows * k);
        fo_dequantize(FH_GGML_Q4_K, ex.data(), experts * rows, k, want.data());
        const auto dense = d.dequantize(e.matrix()).to_f32();
        report("expert tensor loaded from GGUF keeps [experts, rows, columns]",
               e.experts() == experts && e.rows_per_expert() == rows && e.columns() == k &&
                   std::memcmp(dense.data(), want.data(), want.size() * 4) == 0);
        bool threw = false;
        try {
            gguf::load_quantized_matrix(d, file, "blk.0.ffn_down_exps.weight");
        } catch (const Error& err) {
            threw = err.kind() == ErrorKind::Gguf;
        }
        report("a rank-3 tensor is not a matrix: Error::Gguf", threw);
    }
    {
        // a whole Qwen3 file bound by canonical name (src/model/qwen_gguf.rs:32-268): the plan names every
        // tensor, the quantized ones reach the device verbatim under the model's own names
        const size_t h = 256, heads = 2, kv = 1, hd = 128, inter = 512, vocab = 512;
        auto dense = [](size_t count) { return std::vector<uint8_t>(count * 4, 0); };
        const auto embd = blocks(QuantizationFormat::Q6_K, vocab, h, 51), norm = dense(h), head_norm = dense(hd);
        const auto wq = blocks(QuantizationFormat::Q4_K, heads * hd, h, 52), wk = blocks(QuantizationFormat::Q4_K, kv * hd, h, 53);
        const auto wv = blocks(QuantizationFormat::Q6_K, kv * hd, h, 54), wo = blocks(QuantizationFormat::Q4_K, h, heads * hd, 55);
        const auto wg = blocks(QuantizationFormat::Q4_K, inter, h, 56), wu = blocks(QuantizationFormat::Q4_K, inter, h, 57);
        const auto wd = blocks(QuantizationFormat::Q6_K, h, inter, 58);
        std::istringstream stream(gguf_file(
            {{"token_embd.weight", {h, vocab}, FH_GGML_Q6_K, &embd}, {"output_norm.weight", {h}, 0, &norm},
             {"blk.0.attn_norm.weight", {h}, 0, &norm}, {"blk.0.ffn_norm.weight", {h}, 0, &norm},
             {"blk.0.attn_q.weight", {h, heads * hd}, FH_GGML_Q4_K, &wq}, {"blk.0.attn_k.weight", {h, kv * hd}, FH_GGML_Q4_K, &wk},
             {"blk.0.attn_v.weight", {h, kv * hd}, FH_GGML_Q6_K, &wv}, {"blk.0.attn_output.weight", {heads * hd, h}, FH_GGML_Q4_K, &wo},
             {"blk.0.attn_q_norm.weight", {hd}, 0, &head_norm}, {"blk.0.attn_k_norm.weight", {hd}, 0, &head_norm},
             {"blk.0.ffn_gate.weight", {h, inter}, FH_GGML_Q4_K, &wg}, {"blk.0.ffn_up.weight", {h, inter}, FH_GGML_Q4_K, &wu},
             {"blk.0.ffn_down.weight", {inter, h}, FH_GGML_Q6_K, &wd}},
            "qwen3",
            {{"qwen3.embedding_length", (uint32_t)h}, {"qwen3.attention.head_count", (uint32_t)heads},
             {"qwen3.attention.head_count_kv", (uint32_t)kv}, {"qwen3.attention.key_length", (uint32_t)hd},
             {"qwen3.attention.value_length", (uint32_t)hd}, {"qwen3.feed_forward_length", (uint32_t)inter},
             {"qwen3.block_count", 1u}}));
        gguf::Reader file(stream);
        const auto [shape, plan] = gguf::models::plan_qwen(file);
        report("the Qwen3 plan reads the model shape and names all thirteen tensors",
               shape.vocab_size == vocab && shape.hidden_size == h && shape.head_dim == hd && shape.tie_word_embeddings &&
                   shape.layers.size() == 1 && plan.bindings.size() == 13 && plan.tensor_count == 13 &&
                   plan.binding("layers.0.down.weight").sources[0] == "blk.0.ffn_down.weight");
        const gguf::models::BoundWeights bound = gguf::models::bind_quantized(d, file, plan);
        size_t packed_bytes = embd.size() + wq.size() + wk.size() + wv.size() + wo.size() + wg.size() + wu.size() + wd.size();
        bool exact = bound.matrices.size() == 8 && bound.experts.empty() && bound.quantized_tensor_bytes == packed_bytes;
        if (exact) {
            const QuantizedMatrix& down = bound.matrices.at("layers.0.down.weight");
            std::vector<float> want(h * inter);
            fo_dequantize(FH_GGML_Q6_K, wd.data(), h, inter, want.data());
            const auto got = d.dequantize(down).to_f32();
            exact = down.rows() == h && down.columns() == inter && std::memcmp(got.data(), want.data(), want.size() * 4) == 0;
        }
        report("its quantized tensors are on the device under their canonical names, bit for bit", exact);
        bool threw = false;
        try {
            plan.binding("lm_head.weight");   // tied: the file has no output.weight
        } catch (const Error& err) {
            threw = err.kind() == ErrorKind::Weight;
        }
        report("a tied model has no lm_head binding: Error::Weight", threw);
    }
    {
        // residual add + RMSNorm (add_rmsnorm, src/ops/mod.rs:762-820): bit-exact residual, normalised
        // rows against the float64 CPU reference
        const size_t rows = 3, width = 1000;
        std::vector<float> a(rows * width), b(rows * width), w(width);
        for (size_t i = 0; i < a.size(); ++i) {
            a[i] = (float)((double)((i * 73 + 19) % 257) - 128.0) / 73.f;
            b[i] = (float)((double)(((i + 11) * 73 + 19) % 257) - 128.0) / 73.f;
        }
        for (size_t j = 0; j < width; ++j) w[j] = 1.f + (float)((double)(((j + 3) * 73 + 19) % 257) - 128.0) / 73.f;
        std::vector<float> want_residual(a.size()), want_normed(a.size());
        fo_add_rmsnorm(a.data(), b.data(), w.data(), rows, width, 1e-6f, 0, want_residual.data(), want_normed.data());
        auto [residual, normed] = d.add_rmsnorm(d.from_f32({rows, width}, DType::F32, a),
                                                d.from_f32({rows, width}, DType::F32, b),
                                                d.from_f32({width}, DType::F32, w), 1e-6f);
        const auto got_residual = residual.to_f32();
        report("add_rmsnorm residual is the f32 sum, bit for bit",
               std::memcmp(got_residual.data(), want_residual.data(), a.size() * 4) == 0);
        const double err = rel_l2(normed.to_f32(), want_normed);
        report("add_rmsnorm rows match the float64 CPU reference", err <= 1e-6, err);
        bool threw = false;
        try {
            d.add_rmsnorm(residual, normed, d.from_f32({width}, DType::F32, w), 0.f);
        } catch (const Error& err) {
            threw = err.kind() == ErrorKind::Parameter;
        }
        report("a zero epsilon is refused: Error::Parameter", threw);
    }
    {
        // the hybrid engine's layout: route map (h_moe_map) and per-route expert GEMV (project_id)
        const size_t experts = 6, routes = 300, rows = 24, k = 512;
        std::vector<uint32_t> ids(routes);
        for (size_t r = 0; r < routes; ++r) ids[r] = (uint32_t)((r * 7 + r / 5) % experts);
        std::vector<uint32_t> want_offsets(experts + 1), want_sorted(routes), want_position(routes);
        fo_moe_map(ids.data(), experts, routes, want_offsets.data(), want_sorted.data(), want_position.data());
        Tensor id_tensor = d.from_bits({routes}, ids);
        auto map = d.hybrid_moe_map(id_tensor, experts);
        auto words = [](const Tensor& t) {
            const std::vector<float> f = t.to_f32();
            std::vector<uint32_t> u(f.size());
            std::memcpy(u.data(), f.data(), f.size() * 4);
            return u;
        };
        report("hybrid route map equals the h_moe_map restatement",
               words(map.offsets) == want_offsets && words(map.sorted) == want_sorted &&
                   words(map.position) == want_position);
        const auto packed = blocks(QuantizationFormat::Q4_K, experts * rows, k, 77);
        QuantizedExpertMatrix w = d.quantized_expert_matrix(
            experts, rows, k, QuantizationFormat::Q4_K,
            [&packed](uint8_t* dst, size_t bytes) { std::memcpy(dst, packed.data(), bytes); });
        std::vector<float> x(routes / 3 * k);
        for (size_t i = 0; i < x.size(); ++i) x[i] = (float)((double)((i * 41 + 11) % 127) / 113.0 - 0.55);
        Tensor y = d.hybrid_project_id(w, d.from_f32({routes / 3, k}, DType::F32, x), id_tensor, routes, 3);
        std::vector<float> xr(routes * k), meta(routes * 3, 0.f), want(routes * rows);
        for (size_t r = 0; r < routes; ++r) {
            std::memcpy(&xr[r * k], &x[(r / 3) * k], k * 4);
            std::memcpy(&meta[r * 3], &ids[r], 4);
        }
        fo_expert_project(FH_GGML_Q4_K, packed.data(), experts, rows, k, xr.data(), meta.data(), routes, want.data(), 0, 0, 1);
        const double err = rel_l2(y.to_f32(), want);
        report("hybrid project_id: each route times its expert", err <= 1e-5, err);
    }
    std::printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
