// Streamed Q4_K GEMV for gfx950: y[n] = sum_k W[n,k] x[k], one activation row per grid.z entry.
//
// Same product as q4_k_gemv_factored / q4_k_gemv_ksplit of the reference
// (src/metal/shaders/ops.metal:983-1070) in a form built around what limits a
// GEMV of this size on this chip: how the bytes are requested, and how few vector
// instructions are spent per weight.
//
// Bytes.  A workgroup owns up to 16 consecutive weight rows for the whole K.  Its
// waves copy those rows into LDS with LDS-direct loads (global_load_lds_dwordx4):
// every instruction moves one contiguous kilobyte of one row, nothing passes through
// registers, and all of a tile's loads are in flight before anything else happens.
//
// Arithmetic.  The nibbles never become floats on the vector ALU.  Masked in place
// inside a 16-bit half a nibble is the f16 subnormal q * 2^-24 (q * 2^-20 for a high
// nibble), which is a legal matrix-core operand, so the integer dot products
// sum q*x of every 32-weight group run on v_mfma_f32_16x16x32_f16:
//   * B operand (columns n = the tile's 16 weight rows): lane (n, g) holds eight
//     weights of chunk g (64 weights, two groups) of row n's super-block.
//   * A operand (rows j): the activations, as f16 "hi" and "lo" parts of x * s (s a
//     power of two that brings the largest magnitude of its 64-weight chunk to
//     [2^14, 2^15); hi + lo carries 22 bits; the scale is per 64-weight chunk).  Row j = 4g + i is non-zero only in
//     the k slots lane group g covers, so D[4g + i][n] is the dot product of chunk g
//     alone: i = 0 / 1 the hi / lo part against the low nibbles' group, i = 2 / 3
//     against the high nibbles' group.  Low- and high-nibble steps accumulate into
//     two D tiles; each lane (n, g) then finds the four sums of its own chunk in its
//     own registers.
//   * Per super-block a lane applies the two 6-bit scales and minimums of its chunk
//     and the block's d and dmin once.
//
// Activations.  A super-block of a tile is multiplied by exactly one wave, so that wave
// also turns the block's activations into A operands: it requests them before the
// tile's loads (loads complete in issue order, so they can be waited for with the tile
// still in flight), and passes each block through a 1 KB slot of its own in LDS, which
// re-orders the values from "four consecutive per lane" to operand order.
#include <type_traits>

#include "device_utils.hpp"
#include "internal.hpp"

namespace fh {
namespace {

constexpr uint32_t kQ4Bytes = 144;
constexpr uint32_t kSlotBytes = 1024u + 64u + 16u;   // A operands, {group sum, group sum, 1/s, -} per chunk, 16 zero bytes

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct StreamParams {
    const uint8_t* w;     // [n, nb] super-blocks
    const void* x;        // [m, 256 nb]
    void* y;              // [m, n]
    uint32_t n, nb;
    uint32_t tile_rows;   // rows per workgroup, 1..16
    uint32_t row_stride;  // bytes between rows of the tile in LDS
    uint32_t x_dtype, y_dtype;
    // rows longer than a tile can hold: grid.y K segments of seg_blocks super-blocks each
    uint32_t segments, seg_blocks, m;
    float* partials;      // [segments][m][n]
    uint32_t* counters;   // one per (row tile, batch row), zero between launches
};

// LDS-direct load: 16 bytes per lane from `g` to LDS address `lds_addr` + 16 * lane.
__device__ __forceinline__ void lds_load16(const void* g, uint32_t lds_addr) {
    const uint32_t a = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(a) : "memory");
}

// s_waitcnt vmcnt(n), n a wave-uniform run-time value up to 15 (0 beyond)
__device__ __forceinline__ void wait_vmcnt(uint32_t n) {
#define FH_VM(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        FH_VM(1) FH_VM(2) FH_VM(3) FH_VM(4) FH_VM(5) FH_VM(6) FH_VM(7) FH_VM(8)
        FH_VM(9) FH_VM(10) FH_VM(11) FH_VM(12) FH_VM(13) FH_VM(14) FH_VM(15)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef FH_VM
}

__device__ __forceinline__ uint32_t pack_halves(_Float16 lo, _Float16 hi) {
    typedef _Float16 half2t __attribute__((ext_vector_type(2)));
    half2t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, v);
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// One wave writes a super-block's activations (lane = float4 number inside the block) into its
// slot in operand order.  The 16 lanes of a DPP row hold one chunk (64 weights), which is what a
// lane group of the A operand covers, so the power-of-two scale is chosen per chunk and never
// leaves the row.
__device__ __forceinline__ void stage_block(float4 v, uint8_t* slot, uint32_t lane) {
    float top = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    top = dpp_max<0xB1>(top);
    top = dpp_max<0x4E>(top);
    top = dpp_max<0x141>(top);
    top = dpp_max<0x140>(top);
    uint32_t e = __float_as_uint(top) >> 23;
    e = e < 15u ? 15u : e > 254u ? 254u : e;
    const float s = __uint_as_float((268u - e) << 23);   // 2^(14 - exponent of the chunk's largest)
    // hi = f16(x s), lo = f16(x s - hi): each one fused multiply-add that rounds to a half
    half2v h02, h13, l02, l13;
    h02.x = (_Float16)(v.x * s);
    h02.y = (_Float16)(v.z * s);
    h13.x = (_Float16)(v.y * s);
    h13.y = (_Float16)(v.w * s);
    l02.x = (_Float16)fmaf(v.x, s, -(float)h02.x);
    l02.y = (_Float16)fmaf(v.z, s, -(float)h02.y);
    l13.x = (_Float16)fmaf(v.y, s, -(float)h13.x);
    l13.y = (_Float16)fmaf(v.w, s, -(float)h13.y);
    // chunk g, group parity hbit, step u, half of the step
    const uint32_t g = lane >> 4, hbit = (lane >> 3) & 1u, u = (lane >> 1) & 3u;
    uint8_t* const dst = slot + ((u * 4u + g) * 4u + 2u * hbit) * 16u + 8u * (lane & 1u);
    // k slots of an operand dword pair are weights {0, 2} and {1, 3} of four consecutive ones
    *reinterpret_cast<uint2*>(dst) = make_uint2(__builtin_bit_cast(uint32_t, h02), __builtin_bit_cast(uint32_t, h13));
    *reinterpret_cast<uint2*>(dst + 16) = make_uint2(__builtin_bit_cast(uint32_t, l02), __builtin_bit_cast(uint32_t, l13));
    float sum = (v.x + v.y) + (v.z + v.w);
    sum = dpp_add<0xB1>(sum);
    sum = dpp_add<0x4E>(sum);
    sum = dpp_add<0x141>(sum);   // the eight lanes of a 32-weight group now all hold its sum
    // every lane writes (same value, same address within its group): {sum of x in the group, 1 / s}
    float* const aux = reinterpret_cast<float*>(slot + 1024u) + 4u * g;
    aux[hbit] = sum;
    aux[2] = __uint_as_float((e - 14u) << 23);
}

// LDS map (bytes): [tile: tile_rows x row_stride][a slot per wave][row sums: waves x 16 f32]
// DT: activation dtype; WAVES: waves per workgroup; MAXB: super-blocks a wave may own (row length
// <= WAVES * MAXB * 256).  Three workgroups of eight waves share a compute unit: six waves per
// SIMD (ten-wave workgroups were tried for 20-block rows, two blocks per wave; only two of them
// fit a compute unit's wave slots, and the launch took a third longer).
template <int DT, int WAVES, int MAXB>
__global__ __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(6, 6)))
void gemv_stream_q4k(const StreamParams p) {
    constexpr uint32_t kSWaves = WAVES;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this workgroup's K segment: super-blocks first .. first + nb - 1 of the rows
    const uint32_t first = blockIdx.y * p.seg_blocks;
    const uint32_t nb = min(p.seg_blocks, p.nb - first);
    const uint32_t row_bytes = nb * kQ4Bytes;          // of the segment
    const uint32_t full_row_bytes = p.nb * kQ4Bytes;
    const uint32_t row0 = blockIdx.x * p.tile_rows;
    const uint32_t rows = min(p.tile_rows, p.n - row0);

    uint8_t* const tile = lds;
    uint8_t* const slot = tile + p.tile_rows * p.row_stride + wave * kSlotBytes;
    float* const rsum = reinterpret_cast<float*>(tile + p.tile_rows * p.row_stride + kSWaves * kSlotBytes);

    // 1. this wave's activation blocks are requested first
    const size_t xrow = ((size_t)blockIdx.z * p.nb + first) * 256u;
    typename std::conditional<DT == FH_F32, u32x4, u32x2>::type xraw[MAXB];
#pragma unroll
    for (int i = 0; i < MAXB; ++i) {
        // a wave with fewer blocks repeats its last one: the register is then defined by the
        // load alone, and nothing can touch it before the wait below
        const uint32_t b = min(wave + kSWaves * i, nb - 1u);
        if constexpr (DT == FH_F32) {
            const float* src = static_cast<const float*>(p.x) + xrow + b * 256u + lane * 4u;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xraw[i]) : "v"(src) : "memory");
        } else {
            const uint16_t* src = static_cast<const uint16_t*>(p.x) + xrow + b * 256u + lane * 4u;
            asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(xraw[i]) : "v"(src) : "memory");
        }
    }

    // 2. the tile: instruction i covers kilobyte (i % per_row) of row (i / per_row)
    const uint32_t per_row = (row_bytes + 1023u) >> 10;
    const uint32_t total = rows * per_row;
    const uint8_t* const wbase = p.w + (size_t)row0 * full_row_bytes + (size_t)first * kQ4Bytes + lane * 16u;
    const uint32_t tile_addr = (uint32_t)(uintptr_t)tile;
    uint32_t issued = 0;
    for (uint32_t i = wave; i < total; i += kSWaves) {
        const uint32_t r = i / per_row, c = i - r * per_row;
        if (c * 1024u + lane * 16u < row_bytes)
            lds_load16(wbase + (size_t)r * full_row_bytes + c * 1024u, tile_addr + r * p.row_stride + c * 1024u);
        ++issued;
    }
    if (lane < 4u) reinterpret_cast<uint32_t*>(slot + 1024u + 64u)[lane] = 0u;

    // 3. the activations have arrived (the tile's loads may still be in flight)
    wait_vmcnt(issued);
    float4 xv[MAXB];
#pragma unroll
    for (int i = 0; i < MAXB; ++i) {
        asm volatile("" : "+v"(xraw[i])::"memory");
        if constexpr (DT == FH_F32) {
            xv[i] = make_float4(__uint_as_float(xraw[i].x), __uint_as_float(xraw[i].y), __uint_as_float(xraw[i].z),
                                __uint_as_float(xraw[i].w));
        } else if constexpr (DT == FH_F16) {
            xv[i] = make_float4(f16_bits_to_f32(xraw[i].x & 0xffffu), f16_bits_to_f32(xraw[i].x >> 16),
                                f16_bits_to_f32(xraw[i].y & 0xffffu), f16_bits_to_f32(xraw[i].y >> 16));
        } else {
            xv[i] = make_float4(bf16_bits_to_f32(xraw[i].x & 0xffffu), bf16_bits_to_f32(xraw[i].x >> 16),
                                bf16_bits_to_f32(xraw[i].y & 0xffffu), bf16_bits_to_f32(xraw[i].y >> 16));
        }
    }
    stage_block(xv[0], slot, lane);   // the first block while the tile is on its way
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // 4. multiply this wave's super-blocks
    const uint32_t n = lane & 15u, g = lane >> 4;
    const uint32_t nc = n < rows ? n : rows - 1u;
    const bool active = (n >> 2) == g;
    const uint8_t* const wrow = tile + nc * p.row_stride;
    const uint8_t* const xlane = active ? slot + (g * 4u + (n & 3u)) * 16u : slot + 1024u + 64u;
    const uint32_t xstep = active ? 256u : 0u;
    const float* const auxp = reinterpret_cast<const float*>(slot + 1024u) + 4u * g;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < MAXB; ++i) {
        const uint32_t b = wave + kSWaves * i;
        if (b < nb) {
            // this block's operands leave the slot first, so the next block can move in while
            // this one is multiplied
            u32x4 xa[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) xa[u] = *reinterpret_cast<const u32x4*>(xlane + u * xstep);
            const float4 aux = *reinterpret_cast<const float4*>(auxp);
            const uint8_t* const blk = wrow + b * kQ4Bytes;
            const uint4 hdr = *reinterpret_cast<const uint4*>(blk);
            const uint4 qa = *reinterpret_cast<const uint4*>(blk + 16u + 32u * g);
            const uint4 qb = *reinterpret_cast<const uint4*>(blk + 32u + 32u * g);
            if (i + 1 < MAXB && b + kSWaves < nb) {
                asm volatile("s_waitcnt lgkmcnt(3)" ::: "memory");   // the five slot reads are the oldest
                stage_block(xv[i + 1], slot, lane);
            }
            const uint32_t raw[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
            floatx4 dl = {0.f, 0.f, 0.f, 0.f}, dh = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t q0 = raw[2 * u], q1 = raw[2 * u + 1];
                const uint32_t s0 = q0 >> 8, s1 = q1 >> 8;
                const u32x4 lo = {q0 & 0x000f000fu, s0 & 0x000f000fu, q1 & 0x000f000fu, s1 & 0x000f000fu};
                const u32x4 hi = {q0 & 0x00f000f0u, s0 & 0x00f000f0u, q1 & 0x00f000f0u, s1 & 0x00f000f0u};
                const half8 a = __builtin_bit_cast(half8, xa[u]);
                dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8, lo), dl, 0, 0, 0);
                dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8, hi), dh, 0, 0, 0);
            }
            float sc_lo, sc_hi, mn_lo, mn_hi;
            q4k_chunk_scales(hdr.y, hdr.z, hdr.w, g, sc_lo, sc_hi, mn_lo, mn_hi);
            const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
            // low nibbles were q * 2^-24, high nibbles 16 q * 2^-24
            const float dots = fmaf(sc_lo * 16777216.f, dl[0] + dl[1], (sc_hi * 1048576.f) * (dh[2] + dh[3]));
            const float mins = fmaf(mn_lo, aux.x, mn_hi * aux.y);
            acc = fmaf(d * aux.z, dots, fmaf(-dmin, mins, acc));
        }
    }

    // 5. chunks of a row (lanes n, n + 16, n + 32, n + 48), then the waves, in a fixed order
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (lane < 16u) rsum[wave * 16u + lane] = acc;
    __syncthreads();
    float total_sum = 0.f;
    if (tid < rows) {
#pragma unroll
        for (int w = 0; w < kSWaves; ++w) total_sum += rsum[w * 16 + tid];
    }
    if (p.segments == 1) {
        if (tid < rows) store_from_f32(p.y, (size_t)blockIdx.z * p.n + row0 + tid, p.y_dtype, total_sum);
        return;
    }
    // 6. K segments meet in the scratch buffer and the last workgroup of a tile adds them in segment
    // order (device-scope relaxed atomics, coherent across the L2 slices; src/metal/shaders/ops.metal:1031-1070
    // has the same two-stage shape)
    const uint32_t mrow = blockIdx.z;
    if (tid < rows)
        __hip_atomic_store(&p.partials[((size_t)blockIdx.y * p.m + mrow) * p.n + row0 + tid], total_sum, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the stores above have completed
    __syncthreads();
    uint32_t* const flag = reinterpret_cast<uint32_t*>(rsum);   // the row sums have been read
    if (tid == 0) {
        uint32_t* counter = p.counters + (size_t)mrow * gridDim.x + blockIdx.x;
        const uint32_t ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t last = ticket == p.segments - 1 ? 1u : 0u;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last;
    }
    __syncthreads();
    if (*flag == 0) return;
    if (tid < rows) {
        float total = 0.f;
        for (uint32_t sg = 0; sg < p.segments; ++sg)
            total += __hip_atomic_load(&p.partials[((size_t)sg * p.m + mrow) * p.n + row0 + tid], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        store_from_f32(p.y, (size_t)mrow * p.n + row0 + tid, p.y_dtype, total);
    }
}

}  // namespace

// Tile height that spreads the rows evenly: the fewest 16-row rounds per compute unit, then the
// smallest height that still fits them.
StreamPlan gemv_stream_plan(uint32_t n, uint32_t k, uint32_t m, int cu_count, bool any_size, int forced_segments) {
    StreamPlan plan{};
    const uint32_t nb = k / 256u;
    const uint32_t cus = cu_count > 0 ? (uint32_t)cu_count : 256u;
    const uint32_t rounds = ((n + 15u) / 16u + cus - 1u) / cus;
    uint32_t h = (n + cus * rounds - 1u) / (cus * rounds);
    if (h > 16u) h = 16u;
    if (h < 1u) h = 1u;
    // An LDS-direct load names its LDS address in 16 bits of M0, so a tile stays below 64 KB, and
    // a wave owns at most six super-blocks: longer rows are cut into K segments of equal length.
    auto stride_of = [](uint32_t blocks) {
        uint32_t units = 9u * blocks;      // bytes / 16
        if ((units & 1u) == 0) ++units;    // odd number of 16-byte units: 16 rows start in 16 different bank groups
        return units * 16u;
    };
    // ... and, where it must be cut anyway, short enough that three workgroups share a compute
    // unit's LDS (the headline's uncut 14 x 2896 bytes do)
    const uint32_t budget = (160u * 1024u) / 3u - 8u * kSlotBytes - 8u * 64u;
    // (the segments then spread the work, so the tiles are as tall as the matrix instruction)
    // the reference's K-split switch asks for at least that many segments, as far as whole blocks go
    const uint32_t wanted = forced_segments > 1 ? ((uint32_t)forced_segments < nb ? (uint32_t)forced_segments : nb) : 1u;
    if (wanted > 1u || nb > 48u || h * stride_of(nb) > 65536u) h = n < 16u ? n : 16u;
    uint32_t segments = wanted, seg = (nb + wanted - 1u) / wanted;
    while (seg > 48u || h * stride_of(seg) > (segments == 1 ? 65536u : budget)) {
        ++segments;
        seg = (nb + segments - 1u) / segments;
        if (seg <= 1u) break;
    }
    segments = (nb + seg - 1u) / seg;
    plan.segments = segments;
    plan.seg_blocks = seg;
    plan.row_stride = stride_of(seg);
    if (h * plan.row_stride > 65536u) h = 65536u / plan.row_stride;
    plan.tile_rows = h;
    plan.tiles = (n + h - 1u) / h;
    plan.waves = 8u;
    plan.lds_bytes = h * plan.row_stride + plan.waves * kSlotBytes + plan.waves * 64u;
    // matrices of a megabyte or two finish sooner on the FMA kernel's smaller workgroups
    plan.ok = nb >= 1 && seg >= 1u && seg <= 48u && segments <= 65535u && h >= 1u && (any_size || (uint64_t)n * nb >= 16384u) &&
              plan.lds_bytes <= 160u * 1024u && m >= 1 && m <= 65535u;
    return plan;
}

const char* launch_gemv_stream(hipStream_t s, const GemvArgs& a, const StreamPlan& plan) {
    StreamParams p{};
    p.w = static_cast<const uint8_t*>(a.w);
    p.x = a.x;
    p.y = a.y;
    p.n = a.n;
    p.nb = a.k / 256u;
    p.tile_rows = plan.tile_rows;
    p.row_stride = plan.row_stride;
    p.x_dtype = a.x_dtype;
    p.y_dtype = a.y_dtype;
    p.segments = plan.segments;
    p.seg_blocks = plan.seg_blocks;
    p.m = a.m;
    p.partials = a.partials;
    p.counters = a.counters;
    typedef void (*Kernel)(const StreamParams);
    // [dtype][blocks per wave: 2, 3, 6]
    static const Kernel kernels[3][3] = {
        {gemv_stream_q4k<FH_F32, 8, 2>, gemv_stream_q4k<FH_F32, 8, 3>, gemv_stream_q4k<FH_F32, 8, 6>},
        {gemv_stream_q4k<FH_F16, 8, 2>, gemv_stream_q4k<FH_F16, 8, 3>, gemv_stream_q4k<FH_F16, 8, 6>},
        {gemv_stream_q4k<FH_BF16, 8, 2>, gemv_stream_q4k<FH_BF16, 8, 3>, gemv_stream_q4k<FH_BF16, 8, 6>},
    };
    static bool raised = false;
    if (!raised) {
        for (const auto& row : kernels)
            for (Kernel kernel : row)
                (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          160 * 1024);
        raised = true;
    }
    const int shape = plan.seg_blocks <= 16u ? 0 : plan.seg_blocks <= 24u ? 1 : 2;
    hipLaunchKernelGGL(kernels[a.x_dtype][shape], dim3(plan.tiles, plan.segments, a.m), dim3(plan.waves * kWave), plan.lds_bytes, s, p);
    return plan.segments > 1 ? "q4_k_gemv_ksplit" : "q4_k_gemv_factored";
}

}  // namespace fh
