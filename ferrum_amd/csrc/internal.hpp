// Shared definitions of the gfx950 backend: device objects, error plumbing and
// the host-side launchers each kernel file exports.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <map>
#include <utility>
#include <vector>
#include <string>

#include "../../include/ferrum_hip.h"
#include "../../include/ferrum_hip_probe.h"

struct fh_device {
    // The device object lives until fh_device_destroy has been called and the last buffer,
    // matrix, graph or event created on it is gone: their release functions read it.
    int handles = 1;       // the caller's own handle, plus one per live object
    bool closed = false;   // fh_device_destroy has run: the stream is gone, memory is freed directly
    int ordinal = 0;
    hipStream_t stream = nullptr;
    hipDeviceProp_t props{};
    const char* last_operation = "";
    bool capturing = false;
    std::map<std::string, int64_t> tuning;
    // scratch owned by the device: [counter words | floats / ids]
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    // this device's copy of the library's fixed scratch array (fh_project_quantized_no_alloc)
    void* fixed_scratch = nullptr;
    static constexpr size_t kCounterWords = 1u << 16;
    // Releases asked for while an execution is being recorded wait for its end:
    // freeing or synchronizing inside a stream capture would invalidate it.
    // scratch blocks that were outgrown while recorded executions (which carry their address)
    // were alive: freed with the last of those
    std::vector<void*> retired_scratch;
    // temporaries of fh_moe_ffn: one block, grown like the scratch and retired with it
    fh_buffer* workspace = nullptr;
    // activations rewritten to the width of a matrix whose rows are stored padded: grown the same way
    fh_buffer* padded_rows = nullptr;
    int live_graphs = 0;
    std::vector<void*> deferred_frees;
    std::vector<std::pair<hipGraphExec_t, hipGraph_t>> deferred_graphs;
};

struct fh_buffer {
    fh_device* device = nullptr;
    void* ptr = nullptr;
    size_t bytes = 0;
};

struct fh_qmatrix {
    fh_device* device = nullptr;
    void* ptr = nullptr;
    size_t bytes = 0;
    uint32_t ggml_type = 0;
    uint64_t rows = 0;     // per expert
    uint64_t cols = 0;
    uint64_t experts = 1;
    // Width of a stored row, a multiple of 256: `cols` except for a Q8_0 matrix whose rows are 32 n
    // weights with n not a multiple of 8, which is kept with every row padded by empty blocks
    // (scale and quants zero) so that the kernels see runs of eight blocks.
    uint64_t stored_cols = 0;
    bool padded() const { return stored_cols != cols; }
};

struct fh_graph {
    fh_device* device = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

struct fh_event {
    fh_device* device = nullptr;
    hipEvent_t event = nullptr;
};

namespace fh {

fh_status fail(fh_status code, const char* fmt, ...);
fh_status hip_fail(hipError_t err, const char* what);

constexpr uint32_t kQ4K = FH_GGML_Q4_K;
constexpr uint32_t kQ5K = FH_GGML_Q5_K;
constexpr uint32_t kQ6K = FH_GGML_Q6_K;
constexpr uint32_t kIQ4XS = FH_GGML_IQ4_XS;
constexpr uint32_t kQ8_0 = FH_GGML_Q8_0;

// bytes of 256 weights: one super-block, or eight 34-byte blocks of Q8_0
constexpr uint32_t block_bytes_of(uint32_t ggml_type) {
    return ggml_type == kQ4K     ? 144u
           : ggml_type == kQ5K   ? 176u
           : ggml_type == kQ6K   ? 210u
           : ggml_type == kIQ4XS ? 136u
           : ggml_type == kQ8_0  ? 272u
                                 : 0u;
}

inline size_t block_bytes(uint32_t ggml_type) {
    return block_bytes_of(ggml_type);
}
inline size_t dtype_bytes(uint32_t dtype) { return dtype == FH_F32 ? 4 : 2; }

// ---- launchers (one per kernel family); each returns the kernel name ----

// dequant.hip
// f32 -> f16 (round to nearest even), `count` a multiple of 8: activations on their way to the tile kernels
const char* launch_argmax_rows(hipStream_t s, const void* logits, uint32_t dtype, uint32_t rows, uint32_t width,
                               uint32_t* out);
void launch_round_to_f16(hipStream_t s, const float* in, uint16_t* out, size_t count);
// rows are stored `cols` wide (a multiple of 256) and written `out_cols` wide
const char* launch_dequantize(hipStream_t s, uint32_t ggml_type, const void* w, size_t rows,
                              size_t cols, size_t out_cols, void* out, uint32_t out_dtype);
// pieces of `cols` elements (a multiple of 32) -> pieces of `padded` elements, zero beyond `cols`
void launch_pad_rows(hipStream_t s, const void* in, void* out, size_t pieces, size_t cols, size_t padded,
                     size_t element_bytes);
const char* launch_embedding_gather(hipStream_t s, uint32_t ggml_type, const void* w, size_t cols, size_t out_cols,
                                    const uint32_t* ids_dev, size_t count, void* out,
                                    uint32_t out_dtype);

// probe.hip: measurement kernels (a plain 128-bit read of a buffer; an MFMA issue loop)
const char* launch_read_probe(hipStream_t s, const void* data, size_t bytes, uint32_t* sink, int64_t form);
const char* launch_mfma_probe(hipStream_t s, int shape, uint32_t groups, uint32_t iterations, float* sink,
                              double* flops);
const char* launch_coissue_probe(hipStream_t s, uint32_t groups, uint32_t iterations, uint32_t mfma,
                                 uint32_t valu_rounds, float* sink);

// norm.hip
// residual = round(a + b), normed = rmsnorm(residual) * weight; all operands of one dtype,
// no output overlapping an operand or the other output.
const char* launch_add_rmsnorm(hipStream_t s, const void* a, const void* b, const void* weight, void* residual,
                               void* normed, uint32_t rows, uint32_t width, uint32_t dtype, float eps);

// gemv.hip
// how a GEMV launch reads its activations
enum : uint32_t {
    kXPlain = 0,    // row m of x
    kXGather = 1,   // row token(m) of x, the token id from the routing metadata (expert_assign fused)
    kXSiluMul = 2,  // x is [m, 2K]: silu(x[:, :K]) * x[:, K:] with expert_silu_mul's rounding
    kXDivide = 3,   // row m / x_div of x: the hybrid engine's project_id, whose routes share a token's row
};

// what route_token (route_device.hpp) takes: one token's routing by one wave
struct RouteTokenArgs {
    const void* logits;
    uint32_t logits_dtype;
    const float* bias;
    float* metadata;
    uint32_t experts, top_k, sigmoid, normalize;
    float eps, scaling;
    uint32_t rank_order;
    const void* gate_x;
    uint32_t gate_x_dtype;
    const float* gate_w;
    uint32_t hidden;
    float* shared_gate;
    float* ids_out;
    float* weights_out;
};

struct GemvArgs {
    uint32_t ggml_type;
    const void* w;        // packed [n, k] (per expert when metadata is set)
    const void* x;        // [m, k]
    void* y;              // [m, n]
    uint32_t n, k, m;
    uint32_t x_dtype, y_dtype;
    // expert form: when metadata != nullptr, row m of x uses expert
    // bits(metadata[3*m]) and weight rows [expert*n, expert*n + n)
    const float* metadata;
    uint32_t experts;
    int ksplit;           // 0 = automatic, else at least this many K segments
    uint32_t x_mode;      // kXPlain, kXGather or kXSiluMul
    uint32_t x_rows;      // rows of x (kXGather clamps the token id to it)
    uint32_t meta_stride; // floats per entry of `metadata`: 0 or 3 = {id, token, weight}, 1 = ids only
    uint32_t x_div;       // kXDivide: batch entries per row of x (0 = 1)
    // A shared expert riding in the same launch: the last shared_rows of the m batch entries
    // are tokens 0 .. shared_rows - 1 on the dense matrix shared_w [n, k], writing shared_y
    // [shared_rows, n]; they read row t of shared_x when set, else row t of x.  Null = none.
    const void* shared_w;
    uint32_t shared_rows;
    const void* shared_x;
    void* shared_y;
    // the streamed matrix-core kernel may take the launch (dense Q4_K or Q6_K, plain rows, rows that fit LDS)
    int stream;           // 0 never, 1 where it is the faster kernel, 2 wherever it can run
    bool stream_own;      // the streamed Q4_K kernel's waves load their own super-blocks where tiles are <= 14 rows
    int cu_count;
    float* partials;      // scratch for K segments (gemv_plan says how much)
    uint32_t* counters;   // zeroed scratch, one word per (row tile, m)
    // One token whose routing has not run yet: every workgroup routes it first (one wave, the
    // bits of moe_route), takes its entry's expert from that, and workgroup 0 writes the records
    // to route->metadata for the launches that follow.  `metadata` is then only a non-null marker.
    const RouteTokenArgs* route;
};
struct GemvPlan {
    int bs, it;           // block slots per wave step, steps
    uint32_t segments, seg_len, rows_per_wg, tiles;
};
GemvPlan gemv_plan(uint32_t n, uint32_t k, uint32_t m, int forced_segments);
const char* launch_gemv(hipStream_t s, const GemvArgs& a);
// whether a launch with GemvArgs::route set exists for these rows and this router
bool gemv_routes(uint32_t n, uint32_t k, uint32_t experts, uint32_t top_k);

// gemv.hip: the down projection of a token's routed entries (and its shared expert) with
// expert_combine's weighted sum in the same launch; the bits of the two separate launches
struct ExpertDownCombineArgs {
    uint32_t ggml_type;
    const void* w;          // routed experts [experts][n, k]
    const void* w_shared;   // [n, k] or null
    const void* x;          // [tokens * top_k][2k] packed gate|up rows
    const void* x_shared;   // [tokens][2k]
    const float* metadata;  // [tokens * top_k][3]
    const float* shared_gate;
    void* y;                // [tokens][n]
    uint32_t n, k, tokens, top_k, experts, dtype;
};
bool expert_down_combine_fits(uint32_t ggml_type, uint32_t n, uint32_t k, uint32_t top_k, bool shared);
const char* launch_expert_down_combine(hipStream_t s, const ExpertDownCombineArgs& a);

// gemv_stream.hip: the Q4_K and Q6_K GEMV with LDS-direct weight loads and matrix-core dot products
struct StreamPlan {
    bool ok;              // the row length fits the kernel (LDS and per-wave block budget)
    uint32_t tile_rows;   // weight rows per workgroup (1..16)
    uint32_t tiles;
    uint32_t waves;       // waves per workgroup
    uint32_t row_stride;  // bytes between a tile's rows in LDS
    uint32_t lds_bytes;
    // rows too long for one tile are cut into K segments (grid.y), met through the scratch
    // partials and counters exactly as the FMA kernel's segments are
    uint32_t segments, seg_blocks;
};
// any_size: also matrices so small that the FMA kernel is the faster one
StreamPlan gemv_stream_plan(uint32_t ggml_type, uint32_t n, uint32_t k, uint32_t m, int cu_count, bool any_size,
                            int forced_segments);
const char* launch_gemv_stream(hipStream_t s, const GemvArgs& a, const StreamPlan& plan);
// whether launch_gemv hands this launch to the streamed kernel, and its plan
bool gemv_takes_stream(const GemvArgs& a, StreamPlan* plan);
// K segments and row tiles of the kernel launch_gemv will run: what sizes the scratch
struct GemvScratch {
    uint32_t segments, tiles;
};
GemvScratch gemv_scratch(const GemvArgs& a);

// gemm.hip
struct GemmArgs {
    uint32_t ggml_type;
    const void* w;
    const void* x;        // [m, k] f16 or bf16
    void* y;              // [m, n]
    uint32_t n, k, m;
    uint32_t x_dtype, y_dtype;
    int cu_count;
    int wide_min_rows;   // smallest M that takes the 256-row tile
    int wide_shape;      // matrix instruction of the 256-row tile: 0 = 16x16x32, 1 = 32x32x16 where it wins, 2 = always
    int wide32_tile;     // 0 = chosen by shape; else 10 x (row tiles per wave) + column tiles of the 32x32x16 form
    int skinny_max_rows; // largest M that takes the register-dequant kernel
    // routed-expert form of the register-dequant kernel: w is [experts, n, k],
    // x and y rows are assignments, m is their count; tokens of expert e are
    // expert_order[expert_offsets[e] .. expert_offsets[e + 1])
    uint32_t experts;
    const uint32_t* expert_offsets;
    const uint32_t* expert_order;
    // routed form with the expert's rows resident in LDS (expert_rows_fit_lds): when set,
    // x is [x_rows, k] token rows and assignment a reads the row of its token,
    // gather_metadata[3a + 1], as expert_assign would have copied it
    const float* gather_metadata;
    uint32_t x_rows;
    // that kernel can carry a shared expert: tokens 0 .. shared_rows - 1 on the dense matrix
    // shared_w [n, k], reading row t of shared_x (null: row t of x, which then holds token
    // rows) and writing row t of shared_y
    const void* shared_w;
    uint32_t shared_rows;
    const void* shared_x;
    void* shared_y;
    // dense product: the rows are short enough to stay in LDS for the whole K (launch_gemm
    // then weighs launch_gemm_resident against the other kernels)
    bool rows_resident;
    bool use_resident;    // set by launch_gemm_resident only
    bool few_tiles_split; // up to 16 rows, few weight tiles per workgroup: the tiles' super-blocks are dealt over the waves
    bool weight_ring;     // routed form, rows resident: Q4_K and Q6_K weights through LDS rings where they fit beside the rows
};
const char* launch_gemm(hipStream_t s, const GemmArgs& a);

// gemm_skinny.hip
const char* launch_gemm_skinny(hipStream_t s, const GemmArgs& a);
// dense [m, k] x [n, k]^T with 16 or 32 rows at a time resident in LDS; needs expert_rows_fit_lds(k, 1, 1)
const char* launch_gemm_resident(hipStream_t s, const GemmArgs& a);
// whether the routed form keeps an expert's activation rows of width k in LDS,
// which is the kernel that takes the gathered input form
bool expert_rows_fit_lds(uint32_t k, uint32_t m, uint32_t experts);

// moe.hip
// what the hybrid engine's router adds: selection order kept, shared-expert gate
struct RouteExtras {
    uint32_t rank_order = 0;
    const void* gate_x = nullptr;      // [tokens, hidden] activations the gate vector is dotted with
    uint32_t gate_x_dtype = 0;
    const float* gate_w = nullptr;     // [hidden], or null: the gate is 1
    uint32_t hidden = 0;
    float* shared_gate = nullptr;      // [tokens], or null: no gate output
    float* ids_out = nullptr;          // [tokens, top_k] expert ids as u32 bits, or null
    float* weights_out = nullptr;      // [tokens, top_k] route weights, or null
};
const char* launch_moe_route(hipStream_t s, const void* logits, uint32_t logits_dtype,
                             const float* bias, float* metadata, uint32_t tokens,
                             const fh_routing_policy& policy, const RouteExtras& extras);
// the hybrid engine's stages over plain id / weight arrays (h_moe_map, h_moe_gather, h_moe_combine)
const char* launch_moe_map(hipStream_t s, const uint32_t* ids, uint32_t experts, uint32_t routes, uint32_t* offsets,
                           uint32_t* sorted, uint32_t* position);
const char* launch_moe_gather_sorted(hipStream_t s, const void* x, const uint32_t* sorted, void* out, uint32_t routes,
                                     uint32_t used, uint32_t tokens, uint32_t row_bytes);
const char* launch_hybrid_combine(hipStream_t s, const float* down, const float* weights, const uint32_t* position,
                                  const float* shared, const float* shared_gate, float* out, uint32_t hidden,
                                  uint32_t used, uint32_t tokens, uint32_t rows);
const char* launch_expert_group(hipStream_t s, const float* metadata, uint32_t assignments,
                                uint32_t experts, uint32_t* offsets, uint32_t* order, void* y,
                                uint32_t row_bytes);
const char* launch_expert_assign(hipStream_t s, const void* hidden, const float* metadata,
                                 void* out, uint32_t assignments, uint32_t row_bytes, uint32_t tokens);
const char* launch_expert_silu_mul(hipStream_t s, const void* in, void* out, uint32_t assignments,
                                   uint32_t intermediate, uint32_t in_dtype, uint32_t out_dtype);
void launch_expert_silu_mul_pair(hipStream_t s, const void* in, const void* in2, void* out, uint32_t rows,
                                 uint32_t rows2, uint32_t intermediate, uint32_t dtype);
const char* launch_expert_combine(hipStream_t s, const void* in, const float* metadata, void* out,
                                  uint32_t tokens, uint32_t hidden, uint32_t top_k,
                                  uint32_t in_dtype, uint32_t out_dtype, const void* shared,
                                  const float* shared_gate);

}  // namespace fh
