// Mixture-of-experts helper stages on gfx950: routing, row gather, SiLU*up and
// the weighted combine.  They stand in for moe_route, expert_assign,
// expert_silu_mul and expert_combine of the reference
// (src/metal/shaders/ops.metal:1894-1967, 2223-2246) and keep their rounding
// points.  The routed projections themselves live in gemv.hip / gemm.hip.
#include "device_utils.hpp"
#include "internal.hpp"
#include "route_device.hpp"

namespace fh {
namespace {

// One wave per token: route_token of route_device.hpp.
template <int kPerLane>   // experts <= 64 * kPerLane
__global__ __launch_bounds__(64) void moe_route_kernel(const RouteTokenArgs a, uint32_t tokens) {
    extern __shared__ float scores_lds[];  // experts floats
    const uint32_t token = blockIdx.x;
    if (token >= tokens) return;
    route_token<kPerLane>(a, token, threadIdx.x, scores_lds);
}

// out[a, :] = hidden[token(a), :]; rows are copied in pieces of sizeof(V).
template <typename V>
__global__ __launch_bounds__(256) void expert_assign_kernel(const V* __restrict__ hidden,
                                                            const float* __restrict__ metadata,
                                                            V* __restrict__ out,
                                                            uint32_t assignments,
                                                            uint32_t row_pieces, uint32_t tokens) {
    const uint32_t a = blockIdx.x;
    if (a >= assignments) return;
    uint32_t token = __float_as_uint(metadata[3 * (size_t)a + 1]);
    token = token < tokens ? token : tokens - 1;  // a damaged triple reads a wrong row, never outside
    const V* src = hidden + (size_t)token * row_pieces;
    V* dst = out + (size_t)a * row_pieces;
    for (uint32_t i = threadIdx.x; i < row_pieces; i += blockDim.x) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void expert_silu_mul_kernel(const void* __restrict__ in,
                                                              void* __restrict__ out,
                                                              uint32_t assignments,
                                                              uint32_t intermediate,
                                                              uint32_t in_dtype,
                                                              uint32_t out_dtype) {
    size_t total = (size_t)assignments * intermediate;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t a = i / intermediate, column = i % intermediate;
        size_t base = a * 2 * intermediate;
        float gate = load_as_f32(in, base + column, in_dtype);
        float up = load_as_f32(in, base + intermediate + column, in_dtype);
        float activated = round_storage(silu_stable(gate), out_dtype);
        store_from_f32(out, i, out_dtype, activated * up);
    }
}

__global__ __launch_bounds__(256) void expert_combine_kernel(const void* __restrict__ in,
                                                             const float* __restrict__ metadata,
                                                             void* __restrict__ out,
                                                             uint32_t tokens, uint32_t hidden,
                                                             uint32_t top_k, uint32_t in_dtype,
                                                             uint32_t out_dtype,
                                                             const void* __restrict__ shared,
                                                             const float* __restrict__ shared_gate) {
    size_t total = (size_t)tokens * hidden;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t token = i / hidden, column = i % hidden;
        float sum = 0.f;
        for (uint32_t rank = 0; rank < top_k; ++rank) {
            size_t a = token * top_k + rank;
            float gate = round_storage(metadata[a * 3 + 2], out_dtype);
            float value = load_as_f32(in, a * hidden + column, in_dtype);
            sum += round_storage(gate * value, out_dtype);
        }
        if (shared != nullptr) {
            const float gate = round_storage(shared_gate != nullptr ? shared_gate[token] : 1.f, out_dtype);
            sum += round_storage(gate * load_as_f32(shared, i, in_dtype), out_dtype);
        }
        store_from_f32(out, i, out_dtype, sum);
    }
}

// Eight consecutive elements of a row at a time (one 128-bit access for the
// 16-bit types), for rows whose length is a multiple of 8 and 16-byte aligned.
__device__ __forceinline__ void load8(const void* p, size_t i, uint32_t dtype, float (&v)[8]) {
    if (dtype == FH_F32) {
        const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i);
        const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p) + i);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = dtype == FH_F16 ? f16_bits_to_f32(w[j] & 0xffffu) : bf16_bits_to_f32(w[j] & 0xffffu);
            v[2 * j + 1] = dtype == FH_F16 ? f16_bits_to_f32(w[j] >> 16) : bf16_bits_to_f32(w[j] >> 16);
        }
    }
}
__device__ __forceinline__ void store8(void* p, size_t i, uint32_t dtype, const float (&v)[8]) {
    if (dtype == FH_F32) {
        *reinterpret_cast<float4*>(static_cast<float*>(p) + i) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(static_cast<float*>(p) + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            w[j] = dtype == FH_F16 ? (f32_to_f16_bits(v[2 * j]) | (f32_to_f16_bits(v[2 * j + 1]) << 16))
                                   : (f32_to_bf16_bits(v[2 * j]) | (f32_to_bf16_bits(v[2 * j + 1]) << 16));
        *reinterpret_cast<uint4*>(static_cast<uint16_t*>(p) + i) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

__global__ __launch_bounds__(256) void expert_silu_mul8_kernel(const void* __restrict__ in,
                                                               void* __restrict__ out,
                                                               uint32_t assignments, uint32_t intermediate,
                                                               uint32_t in_dtype, uint32_t out_dtype) {
    const size_t total = (size_t)assignments * intermediate / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const size_t a = (i * 8) / intermediate, column = (i * 8) % intermediate;
        float gate[8], up[8], result[8];
        load8(in, a * 2 * intermediate + column, in_dtype, gate);
        load8(in, a * 2 * intermediate + intermediate + column, in_dtype, up);
#pragma unroll
        for (int j = 0; j < 8; ++j) result[j] = round_storage(silu_stable(gate[j]), out_dtype) * up[j];
        store8(out, i * 8, out_dtype, result);
    }
}

// expert_silu_mul8_kernel over two inputs whose outputs follow one another: rows of `in`
// first, then rows of `in2` (a shared expert's rows behind the routed ones), in one launch.
__global__ __launch_bounds__(256) void expert_silu_mul8_pair_kernel(const void* __restrict__ in,
                                                                    const void* __restrict__ in2,
                                                                    void* __restrict__ out, uint32_t rows,
                                                                    uint32_t rows2, uint32_t intermediate,
                                                                    uint32_t dtype) {
    const size_t total = (size_t)(rows + rows2) * intermediate / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t a = (i * 8) / intermediate;
        const size_t column = (i * 8) % intermediate;
        const void* src = in;
        if (a >= rows) {
            a -= rows;
            src = in2;
        }
        float gate[8], up[8], result[8];
        load8(src, a * 2 * intermediate + column, dtype, gate);
        load8(src, a * 2 * intermediate + intermediate + column, dtype, up);
#pragma unroll
        for (int j = 0; j < 8; ++j) result[j] = round_storage(silu_stable(gate[j]), dtype) * up[j];
        store8(out, i * 8, dtype, result);
    }
}

// The dtypes are template parameters: with one token the kernel is a single short
// dependent instruction stream, and every runtime dtype switch lengthens it.
template <uint32_t in_dtype, uint32_t out_dtype>
__global__ __launch_bounds__(256) void expert_combine8_kernel(const void* __restrict__ in,
                                                              const float* __restrict__ metadata,
                                                              void* __restrict__ out, uint32_t tokens,
                                                              uint32_t hidden, uint32_t top_k,
                                                              const void* __restrict__ shared,
                                                              const float* __restrict__ shared_gate) {
    // each product is rounded before it is added: with f32 storage round_storage is the
    // identity and would not keep the compiler from fusing the two into an fma
#pragma clang fp contract(off)
    const size_t total = (size_t)tokens * hidden / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const size_t token = (i * 8) / hidden, column = (i * 8) % hidden;
        float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // eight ranks at a time: their loads are issued together (one memory
        // latency instead of eight), the additions stay in rank order
        for (uint32_t rank0 = 0; rank0 < top_k; rank0 += 8) {
            float gate[8], value[8][8];
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint32_t rank = rank0 + r < top_k ? rank0 + r : top_k - 1;
                const size_t a = token * top_k + rank;
                gate[r] = metadata[a * 3 + 2];
                load8(in, a * hidden + column, in_dtype, value[r]);
            }
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                if (rank0 + r < top_k) {
                    const float weight = round_storage(gate[r], out_dtype);
#pragma unroll
                    for (int j = 0; j < 8; ++j) sum[j] += round_storage(weight * value[r][j], out_dtype);
                }
            }
        }
        if (shared != nullptr) {
            const float weight = round_storage(shared_gate != nullptr ? shared_gate[token] : 1.f, out_dtype);
            float value[8];
            load8(shared, i * 8, in_dtype, value);
#pragma unroll
            for (int j = 0; j < 8; ++j) sum[j] += round_storage(weight * value[j], out_dtype);
        }
        store8(out, i * 8, out_dtype, sum);
    }
}

unsigned grid_for(size_t threads) {
    size_t blocks = (threads + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (blocks == 0) blocks = 1;
    return (unsigned)blocks;
}

// Groups assignments by expert for the grouped projection: offsets[e] is the
// first slot of expert e in `order` (offsets[experts] = number of valid
// assignments) and order[] lists assignment ids expert by expert.  The order
// inside an expert is whatever the LDS atomics give; every output row depends
// on its own assignment only, so results do not depend on it.  Rows whose
// expert id is out of range are zero-filled here, as the per-assignment form
// leaves them.  One workgroup; experts <= 1024.
constexpr int kGroupThreads = 1024;

// Inclusive sum over the 1024 threads of a workgroup, in thread order: each wave scans its
// own 64 values through lane shuffles and adds the totals of the waves before it, so two
// barriers replace the twenty of a step-doubling scan through LDS.  wave_total: 16 words.
__device__ __forceinline__ uint32_t block_inclusive_scan_1024(uint32_t v, uint32_t* wave_total) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t sum = v;
#pragma unroll
    for (uint32_t step = 1; step < 64; step <<= 1) {
        const uint32_t below = (uint32_t)__shfl_up((int)sum, step, 64);
        if (lane >= step) sum += below;
    }
    __syncthreads();  // wave_total may still be read from an earlier scan
    if (lane == 63) wave_total[wave] = sum;
    __syncthreads();
    for (uint32_t w = 0; w < wave; ++w) sum += wave_total[w];
    return sum;
}

__global__ __launch_bounds__(kGroupThreads) void expert_group_kernel(const float* __restrict__ metadata,
                                                                     uint32_t assignments, uint32_t experts,
                                                                     uint32_t* __restrict__ offsets,
                                                                     uint32_t* __restrict__ order,
                                                                     uint32_t* __restrict__ y_words,
                                                                     uint32_t row_words) {
    __shared__ uint32_t count[kGroupThreads];
    __shared__ uint32_t wave_total[kGroupThreads / 64];
    const uint32_t tid = threadIdx.x;
    count[tid] = 0;
    __syncthreads();
    // eight ids per thread are requested together: one memory latency per 8192 assignments
    for (uint32_t base = 0; base < assignments; base += 8 * kGroupThreads) {
        uint32_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t a = base + i * kGroupThreads + tid;
            e[i] = a < assignments ? __float_as_uint(metadata[3 * (size_t)a]) : 0xffffffffu;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (e[i] < experts) atomicAdd(&count[e[i]], 1u);
    }
    __syncthreads();
    // inclusive scan over the expert counts
    const uint32_t v = count[tid];
    const uint32_t upto = block_inclusive_scan_1024(v, wave_total);
    const uint32_t first = upto - v;
    if (tid < experts) offsets[tid] = first;
    if (tid == experts - 1) offsets[experts] = upto;
    count[tid] = first;  // now the next free slot of each expert
    __syncthreads();
    for (uint32_t base = 0; base < assignments; base += 8 * kGroupThreads) {
        uint32_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t a = base + i * kGroupThreads + tid;
            e[i] = a < assignments ? __float_as_uint(metadata[3 * (size_t)a]) : 0u;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t a = base + i * kGroupThreads + tid;
            if (a >= assignments) continue;
            if (e[i] < experts) {
                order[atomicAdd(&count[e[i]], 1u)] = a;
            } else {
                for (uint32_t j = 0; j < row_words; ++j) y_words[(size_t)a * row_words + j] = 0u;
            }
        }
    }
}

// h_moe_map (src/metal/shaders/hybrid.metal:2321-2358): the deterministic expert-major
// order of routes.  offsets[e] .. offsets[e + 1] are expert e's rows, sorted[p] is the route
// at row p, position[r] the row of route r; inside an expert routes keep their order.
// Routes whose id is not an expert are left out, as there.  One workgroup; experts <= 1024.
// Routes are placed 1024 at a time: a wave ranks its 64 routes among themselves by ballot
// and leaves one count per expert, and a route's row is its expert's next free row plus the
// counts of the waves before its own plus its rank.
constexpr int kMapThreads = 1024;
constexpr int kMapWaves = kMapThreads / 64;
static_assert(kMapThreads == 1024 && kGroupThreads == 1024, "block_inclusive_scan_1024 covers 1024 threads");

__global__ __launch_bounds__(kMapThreads) void moe_map_kernel(const uint32_t* __restrict__ ids, uint32_t experts,
                                                              uint32_t routes, uint32_t* __restrict__ offsets,
                                                              uint32_t* __restrict__ sorted,
                                                              uint32_t* __restrict__ position) {
    __shared__ uint32_t next[kMapThreads];                 // counts, then the next free row of each expert
    __shared__ uint32_t wave_total[kMapWaves];
    __shared__ uint8_t wave_count[kMapWaves][kMapThreads];  // routes of expert e in wave w of this round
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    next[tid] = 0;
    __syncthreads();
    for (uint32_t base = 0; base < routes; base += 8 * kMapThreads) {
        uint32_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t r = base + i * kMapThreads + tid;
            e[i] = r < routes ? ids[r] : 0xffffffffu;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (e[i] < experts) atomicAdd(&next[e[i]], 1u);
    }
    __syncthreads();
    const uint32_t mine = next[tid];
    const uint32_t upto = block_inclusive_scan_1024(mine, wave_total);
    const uint32_t first = upto - mine;
    if (tid < experts) offsets[tid] = first;
    if (tid == experts - 1) offsets[experts] = upto;
    next[tid] = first;

    uint32_t id_bits = 0;
    while ((1u << id_bits) < experts) ++id_bits;
    for (uint32_t r0 = 0; r0 < routes; r0 += kMapThreads) {
#pragma unroll
        for (int w = 0; w < kMapWaves; ++w) wave_count[w][tid] = 0;
        __syncthreads();
        const uint32_t r = r0 + tid;
        const uint32_t e = r < routes ? ids[r] : 0xffffffffu;
        const bool valid = e < experts;
        // lanes of this wave that hold the same expert
        unsigned long long peers = __ballot(valid);
        for (uint32_t b = 0; b < id_bits; ++b) {
            const bool bit = (e >> b) & 1u;
            const unsigned long long with_bit = __ballot(bit);
            peers &= bit ? with_bit : ~with_bit;
        }
        const uint32_t rank = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
        if (valid && rank == 0) wave_count[wave][e] = (uint8_t)__popcll(peers);
        __syncthreads();
        if (valid) {
            uint32_t row = next[e] + rank;
            for (uint32_t w = 0; w < wave; ++w) row += wave_count[w][e];
            sorted[row] = r;
            position[r] = row;
        }
        __syncthreads();
        uint32_t total = 0;
#pragma unroll
        for (int w = 0; w < kMapWaves; ++w) total += wave_count[w][tid];
        next[tid] += total;
        __syncthreads();
    }
}

// h_moe_gather (src/metal/shaders/hybrid.metal:2360-2370): row p of the output is the
// activation row of the token that route sorted[p] belongs to.  Rows move in pieces of sizeof(V).
template <typename V>
__global__ __launch_bounds__(256) void moe_gather_sorted_kernel(const V* __restrict__ x,
                                                                const uint32_t* __restrict__ sorted,
                                                                V* __restrict__ out, uint32_t used,
                                                                uint32_t tokens, uint32_t pieces) {
    const uint32_t row = blockIdx.x;
    uint32_t token = sorted[row] / used;
    token = token < tokens ? token : tokens - 1;
    for (uint32_t i = threadIdx.x; i < pieces; i += blockDim.x) out[(size_t)row * pieces + i] = x[(size_t)token * pieces + i];
}

// h_moe_combine (src/metal/shaders/hybrid.metal:2372-2388), f32:
// out[t] = sum_s weights[t, s] * down[row(t, s)] + shared_gate[t] * shared[t], the sum in
// rank order; row(t, s) is the route itself or position[route].
template <int VEC>
__global__ __launch_bounds__(256) void hybrid_combine_kernel(const float* __restrict__ down,
                                                             const float* __restrict__ weights,
                                                             const uint32_t* __restrict__ position,
                                                             const float* __restrict__ shared,
                                                             const float* __restrict__ shared_gate,
                                                             float* __restrict__ out, uint32_t hidden,
                                                             uint32_t used, uint32_t tokens, uint32_t rows) {
    const size_t total = (size_t)tokens * hidden / VEC;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = (i * VEC) / hidden, column = (i * VEC) % hidden;
        float acc[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
        for (uint32_t s = 0; s < used; ++s) {
            const size_t r = t * used + s;
            uint32_t row = position != nullptr ? position[r] : (uint32_t)r;
            row = row < rows ? row : rows - 1;
            const float w = weights[r];
            const float* src = down + (size_t)row * hidden + column;
            if constexpr (VEC == 4) {
                const float4 v = *reinterpret_cast<const float4*>(src);
                acc[0] += w * v.x;
                acc[1] += w * v.y;
                acc[2] += w * v.z;
                acc[3] += w * v.w;
            } else {
                acc[0] += w * src[0];
            }
        }
        const float g = shared_gate[t];
        if constexpr (VEC == 4) {
            const float4 sv = *reinterpret_cast<const float4*>(shared + i * 4);
            *reinterpret_cast<float4*>(out + i * 4) =
                make_float4(acc[0] + g * sv.x, acc[1] + g * sv.y, acc[2] + g * sv.z, acc[3] + g * sv.w);
        } else {
            out[i] = acc[0] + g * shared[i];
        }
    }
}

}  // namespace

const char* launch_moe_route(hipStream_t s, const void* logits, uint32_t logits_dtype,
                             const float* bias, float* metadata, uint32_t tokens,
                             const fh_routing_policy& p, const RouteExtras& x) {
    const size_t lds = ((p.experts + 3u) & ~3u) * sizeof(float);
    RouteTokenArgs args{};
    args.logits = logits;
    args.logits_dtype = logits_dtype;
    args.bias = bias;
    args.metadata = metadata;
    args.experts = p.experts;
    args.top_k = p.top_k;
    args.sigmoid = p.sigmoid;
    args.normalize = p.normalize_top_k_prob;
    args.eps = p.normalization_epsilon;
    args.scaling = p.routed_scaling_factor;
    args.rank_order = x.rank_order;
    args.gate_x = x.gate_x;
    args.gate_x_dtype = x.gate_x_dtype;
    args.gate_w = x.gate_w;
    args.hidden = x.hidden;
    args.shared_gate = x.shared_gate;
    args.ids_out = x.ids_out;
    args.weights_out = x.weights_out;
#define FH_ROUTE(PL) hipLaunchKernelGGL(moe_route_kernel<PL>, dim3(tokens), dim3(64), lds, s, args, tokens)
    if (p.experts <= 64) FH_ROUTE(1);
    else if (p.experts <= 128) FH_ROUTE(2);
    else if (p.experts <= 256) FH_ROUTE(4);
    else if (p.experts <= 512) FH_ROUTE(8);
    else FH_ROUTE(kMaxPerLane);
#undef FH_ROUTE
    return x.rank_order ? "h_moe_route" : "moe_route";
}

const char* launch_expert_group(hipStream_t s, const float* metadata, uint32_t assignments,
                                uint32_t experts, uint32_t* offsets, uint32_t* order, void* y,
                                uint32_t row_bytes) {
    hipLaunchKernelGGL(expert_group_kernel, dim3(1), dim3(kGroupThreads), 0, s, metadata, assignments,
                       experts, offsets, order, static_cast<uint32_t*>(y), row_bytes / 4);
    return "expert_group";
}

const char* launch_expert_assign(hipStream_t s, const void* hidden, const float* metadata,
                                 void* out, uint32_t assignments, uint32_t row_bytes, uint32_t tokens) {
    if (row_bytes % 16 == 0) {
        hipLaunchKernelGGL(expert_assign_kernel<uint4>, dim3(assignments), dim3(256), 0, s,
                           static_cast<const uint4*>(hidden), metadata, static_cast<uint4*>(out),
                           assignments, row_bytes / 16, tokens);
    } else if (row_bytes % 4 == 0) {
        hipLaunchKernelGGL(expert_assign_kernel<uint32_t>, dim3(assignments), dim3(256), 0, s,
                           static_cast<const uint32_t*>(hidden), metadata,
                           static_cast<uint32_t*>(out), assignments, row_bytes / 4, tokens);
    } else {
        hipLaunchKernelGGL(expert_assign_kernel<uint16_t>, dim3(assignments), dim3(256), 0, s,
                           static_cast<const uint16_t*>(hidden), metadata,
                           static_cast<uint16_t*>(out), assignments, row_bytes / 2, tokens);
    }
    return "expert_assign";
}

const char* launch_expert_silu_mul(hipStream_t s, const void* in, void* out, uint32_t assignments,
                                   uint32_t intermediate, uint32_t in_dtype, uint32_t out_dtype) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    if (intermediate % 8 == 0 && aligned) {
        hipLaunchKernelGGL(expert_silu_mul8_kernel, dim3(grid_for((size_t)assignments * intermediate / 8)),
                           dim3(256), 0, s, in, out, assignments, intermediate, in_dtype, out_dtype);
    } else {
        hipLaunchKernelGGL(expert_silu_mul_kernel, dim3(grid_for((size_t)assignments * intermediate)),
                           dim3(256), 0, s, in, out, assignments, intermediate, in_dtype, out_dtype);
    }
    return "expert_silu_mul";
}

// rows of `in` then rows2 of `in2`, [.., 2 * intermediate] each, into out [rows + rows2, intermediate]
void launch_expert_silu_mul_pair(hipStream_t s, const void* in, const void* in2, void* out, uint32_t rows,
                                 uint32_t rows2, uint32_t intermediate, uint32_t dtype) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(in2) |
                           reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    if (intermediate % 8 == 0 && aligned) {
        hipLaunchKernelGGL(expert_silu_mul8_pair_kernel, dim3(grid_for((size_t)(rows + rows2) * intermediate / 8)),
                           dim3(256), 0, s, in, in2, out, rows, rows2, intermediate, dtype);
        return;
    }
    launch_expert_silu_mul(s, in, out, rows, intermediate, dtype, dtype);
    launch_expert_silu_mul(s, in2, static_cast<uint8_t*>(out) + (size_t)rows * intermediate * 2, rows2, intermediate,
                           dtype, dtype);
}

const char* launch_expert_combine(hipStream_t s, const void* in, const float* metadata, void* out,
                                  uint32_t tokens, uint32_t hidden, uint32_t top_k,
                                  uint32_t in_dtype, uint32_t out_dtype, const void* shared,
                                  const float* shared_gate) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out) |
                           reinterpret_cast<uintptr_t>(shared)) & 15u) == 0;
    if (hidden % 8 == 0 && aligned) {
        const dim3 grid(grid_for((size_t)tokens * hidden / 8));
#define FH_COMBINE(I, O)                                                                                       \
    if (in_dtype == I && out_dtype == O)                                                                       \
        hipLaunchKernelGGL((expert_combine8_kernel<I, O>), grid, dim3(256), 0, s, in, metadata, out, tokens,   \
                           hidden, top_k, shared, shared_gate);
        FH_COMBINE(0, 0) FH_COMBINE(0, 1) FH_COMBINE(0, 2)
        FH_COMBINE(1, 0) FH_COMBINE(1, 1) FH_COMBINE(1, 2)
        FH_COMBINE(2, 0) FH_COMBINE(2, 1) FH_COMBINE(2, 2)
#undef FH_COMBINE
    } else {
        hipLaunchKernelGGL(expert_combine_kernel, dim3(grid_for((size_t)tokens * hidden)), dim3(256), 0,
                           s, in, metadata, out, tokens, hidden, top_k, in_dtype, out_dtype, shared, shared_gate);
    }
    return shared != nullptr ? "h_moe_combine" : "expert_combine";
}

const char* launch_moe_map(hipStream_t s, const uint32_t* ids, uint32_t experts, uint32_t routes, uint32_t* offsets,
                           uint32_t* sorted, uint32_t* position) {
    hipLaunchKernelGGL(moe_map_kernel, dim3(1), dim3(kMapThreads), 0, s, ids, experts, routes, offsets, sorted,
                       position);
    return "h_moe_map";
}

const char* launch_moe_gather_sorted(hipStream_t s, const void* x, const uint32_t* sorted, void* out, uint32_t routes,
                                     uint32_t used, uint32_t tokens, uint32_t row_bytes) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    if (row_bytes % 16 == 0 && aligned) {
        hipLaunchKernelGGL(moe_gather_sorted_kernel<uint4>, dim3(routes), dim3(256), 0, s, static_cast<const uint4*>(x),
                           sorted, static_cast<uint4*>(out), used, tokens, row_bytes / 16);
    } else {
        hipLaunchKernelGGL(moe_gather_sorted_kernel<uint16_t>, dim3(routes), dim3(256), 0, s,
                           static_cast<const uint16_t*>(x), sorted, static_cast<uint16_t*>(out), used, tokens,
                           row_bytes / 2);
    }
    return "h_moe_gather";
}

const char* launch_hybrid_combine(hipStream_t s, const float* down, const float* weights, const uint32_t* position,
                                  const float* shared, const float* shared_gate, float* out, uint32_t hidden,
                                  uint32_t used, uint32_t tokens, uint32_t rows) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(down) | reinterpret_cast<uintptr_t>(shared) |
                           reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    if (hidden % 4 == 0 && aligned) {
        hipLaunchKernelGGL(hybrid_combine_kernel<4>, dim3(grid_for((size_t)tokens * hidden / 4)), dim3(256), 0, s, down,
                           weights, position, shared, shared_gate, out, hidden, used, tokens, rows);
    } else {
        hipLaunchKernelGGL(hybrid_combine_kernel<1>, dim3(grid_for((size_t)tokens * hidden)), dim3(256), 0, s, down,
                           weights, position, shared, shared_gate, out, hidden, used, tokens, rows);
    }
    return "h_moe_combine";
}

}  // namespace fh
