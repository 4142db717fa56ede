// Streamed Q4_K and Q6_K GEMV for gfx950: y[n] = sum_k W[n,k] x[k], one activation row per grid.z entry.
//
// Same product as q4_k_gemv_factored / q4_k_gemv_ksplit of the reference
// (src/metal/shaders/ops.metal:983-1070; Q6_K: q6_k_factored_rows, q6_k_gemv_ksplit and
// q6_k_gemv_factored, :1393-1439) in a form built around what limits a
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
#include "lds_direct.hpp"

namespace fh {
namespace {

constexpr uint32_t kQ4Bytes = 144;
constexpr uint32_t kQ6Bytes = 210;
constexpr uint32_t kSlotBytes = 1024u + 64u + 16u;   // A operands, {group sum, group sum, 1/s, -} per chunk, 16 zero bytes
// Q6_K: A operands, {four group sums, four 1/s} per lane group, 16 zero bytes
constexpr uint32_t kSlot6Bytes = 1024u + 128u + 16u;
template <uint32_t TYPE> struct StreamFormat;
template <> struct StreamFormat<kQ4K> { static constexpr uint32_t kBytes = kQ4Bytes, kSlot = kSlotBytes, kAux = 64u; };
template <> struct StreamFormat<kQ6K> { static constexpr uint32_t kBytes = kQ6Bytes, kSlot = kSlot6Bytes, kAux = 128u; };

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
    uint32_t tile_bytes;  // of the tile region in LDS
    uint32_t x_dtype, y_dtype;
    // rows longer than a tile can hold: grid.y K segments of seg_blocks super-blocks each
    uint32_t segments, seg_blocks, m;
    float* partials;      // [segments][m][n]
    uint32_t* counters;   // one per (row tile, batch row), zero between launches
};

__device__ __forceinline__ uint32_t pack_halves(_Float16 lo, _Float16 hi) {
    typedef _Float16 half2t __attribute__((ext_vector_type(2)));
    half2t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, v);
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// f16(a s) and f16(b s) in the two halves of a dword, and f16(a s - hi) and f16(b s - hi) against such
// a pair: one v_fma_mix per value, written straight into its half (s is a power of two, so a s is
// exact and the first is the plain rounding of the product).
__device__ __forceinline__ uint32_t hi_pair(float a, float b, float s) {
    uint32_t r;
    asm("v_fma_mixlo_f16 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(s));
    asm("v_fma_mixhi_f16 %0, %1, %2, 0" : "+v"(r) : "v"(b), "v"(s));
    return r;
}
__device__ __forceinline__ uint32_t lo_pair(float a, float b, float s, uint32_t hi) {
    uint32_t r;
    asm("v_fma_mixlo_f16 %0, %1, %2, -%3 op_sel_hi:[0,0,1]" : "=v"(r) : "v"(a), "v"(s), "v"(hi));
    asm("v_fma_mixhi_f16 %0, %1, %2, -%3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "+v"(r) : "v"(b), "v"(s), "v"(hi));
    return r;
}

// One wave writes a super-block's activations (lane = float4 number inside the block) into its
// slot in operand order.  The 16 lanes of a DPP row hold one chunk (64 weights), which is what a
// lane group of the A operand covers, so the power-of-two scale is chosen per chunk and never
// leaves the row.
__device__ __forceinline__ void stage_block(float4 v, uint8_t* slot, uint32_t lane) {
    // the largest magnitude's exponent: magnitudes order like their bit patterns, and an unsigned
    // maximum folds into the DPP instruction itself
    uint32_t top = __float_as_uint(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    top = dpp_umax<0xB1>(top);
    top = dpp_umax<0x4E>(top);
    top = dpp_umax<0x141>(top);
    top = dpp_umax<0x140>(top);
    uint32_t e = top >> 23;
    e = e < 15u ? 15u : e > 254u ? 254u : e;
    const float s = __uint_as_float((268u - e) << 23);   // 2^(14 - exponent of the chunk's largest)
    // hi = f16(x s), lo = f16(x s - hi): each one fused multiply-add that rounds to a half
    const uint32_t h02 = hi_pair(v.x, v.z, s), h13 = hi_pair(v.y, v.w, s);
    const uint32_t l02 = lo_pair(v.x, v.z, s, h02), l13 = lo_pair(v.y, v.w, s, h13);
    // chunk g, group parity hbit, step u, half of the step
    const uint32_t g = lane >> 4, hbit = (lane >> 3) & 1u, u = (lane >> 1) & 3u;
    uint8_t* const dst = slot + ((u * 4u + g) * 4u + 2u * hbit) * 16u + 8u * (lane & 1u);
    // k slots of an operand dword pair are weights {0, 2} and {1, 3} of four consecutive ones
    *reinterpret_cast<uint2*>(dst) = make_uint2(h02, h13);
    *reinterpret_cast<uint2*>(dst + 16) = make_uint2(l02, l13);
    float sum = (v.x + v.y) + (v.z + v.w);
    sum = dpp_add<0xB1>(sum);
    sum = dpp_add<0x4E>(sum);
    sum = dpp_add<0x141>(sum);   // the eight lanes of a 32-weight group now all hold its sum
    // every lane writes (same value, same address within its group): {sum of x in the group, 1 / s}
    float* const aux = reinterpret_cast<float*>(slot + 1024u) + 4u * g;
    aux[hbit] = sum;
    aux[2] = __uint_as_float((e - 14u) << 23);
}

// The same for a Q6_K super-block (the layout src/metal/shaders/ops.metal:1397-1425 indexes).
// Weight 128 h + 32 s + 16 e + j (half h, slice s, j < 16) has its low four bits in
// nibble s / 2 of ql[64 h + 32 (s & 1) + 16 e + j] and its high two in bits 2 s of
// qh[32 h + 16 e + j]; lane group g = 2 h + e of the B operand holds those three 16-byte pieces,
// four scale groups of 16 weights.  Step u = 2 (s & 1) + j / 8 multiplies eight bytes of a ql
// piece: rows 4 g + 0 / 1 of A carry the hi / lo parts of the activations under the low nibbles
// (slice s & 1), rows 4 g + 2 / 3 those under the high nibbles (slice 2 + (s & 1)), and the same
// operand serves the two bit planes of qh that belong to those slices.  Lane L holds activations
// 4 L .. 4 L + 3, so L = 32 h + 8 s + 4 e + j / 4: a quad of lanes is one scale group, which gets
// a power-of-two scale of its own.
__device__ __forceinline__ void stage_block_q6k(float4 v, uint8_t* slot, uint32_t lane) {
    uint32_t top = __float_as_uint(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    top = dpp_umax<0xB1>(top);
    top = dpp_umax<0x4E>(top);
    uint32_t ex = top >> 23;
    ex = ex < 15u ? 15u : ex > 254u ? 254u : ex;
    const float s = __uint_as_float((268u - ex) << 23);
    const uint32_t h02 = hi_pair(v.x, v.z, s), h13 = hi_pair(v.y, v.w, s);
    const uint32_t l02 = lo_pair(v.x, v.z, s, h02), l13 = lo_pair(v.y, v.w, s, h13);
    const uint32_t h = lane >> 5, sl = (lane >> 3) & 3u, e = (lane >> 2) & 1u, up = (lane >> 1) & 1u;
    const uint32_t g = 2u * h + e, u = 2u * (sl & 1u) + up, i = 2u * (sl >> 1);
    uint8_t* const dst = slot + ((u * 4u + g) * 4u + i) * 16u + 8u * (lane & 1u);
    *reinterpret_cast<uint2*>(dst) = make_uint2(h02, h13);
    *reinterpret_cast<uint2*>(dst + 16) = make_uint2(l02, l13);
    float sum = (v.x + v.y) + (v.z + v.w);
    sum = dpp_add<0xB1>(sum);
    sum = dpp_add<0x4E>(sum);   // the four lanes of a scale group now all hold its sum
    float* const aux = reinterpret_cast<float*>(slot + 1024u) + 8u * g;
    aux[sl] = sum;
    aux[4u + sl] = __uint_as_float((ex - 14u) << 23);
}

// 16 or 8 bytes of a tile in LDS that are only 2-byte aligned (Q6_K blocks are 210 bytes long)
__device__ __forceinline__ uint4 lds_u4_unaligned(const uint8_t* p) {
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
__device__ __forceinline__ uint2 lds_u2_unaligned(const uint8_t* p) {
    uint2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

// LDS map (bytes): [tile: tile_rows x row_stride][a slot per wave][row sums: waves x 16 f32]
// DT: activation dtype; WAVES: waves per workgroup; MAXB: super-blocks a wave may own (row length
// <= WAVES * MAXB * 256).  Three workgroups of eight waves share a compute unit: six waves per
// SIMD (ten-wave workgroups were tried for 20-block rows, two blocks per wave; only two of them
// fit a compute unit's wave slots, and the launch took a third longer).
// OWN: a wave requests exactly the super-blocks it multiplies -- a block of all the tile's
// rows is tile_rows x 9 pieces of 16 bytes, 64 pieces per instruction -- and waits for its own
// loads only; the tile in LDS is then [block][row][144 bytes] (rows 36 words apart: sixteen rows
// read sixteen different groups of four banks).
template <uint32_t TYPE, int DT, int WAVES, int MAXB, bool OWN = false>
__device__ __forceinline__ void gemv_stream_body(const StreamParams& p) {
    constexpr uint32_t kSWaves = WAVES;
    constexpr uint32_t kBlock = StreamFormat<TYPE>::kBytes;    // bytes of a super-block
    constexpr uint32_t kSlotBytes = StreamFormat<TYPE>::kSlot;
    constexpr uint32_t kAuxBytes = StreamFormat<TYPE>::kAux;
    auto stage = [](float4 v, uint8_t* slot, uint32_t lane) {
        if constexpr (TYPE == kQ4K) stage_block(v, slot, lane);
        else stage_block_q6k(v, slot, lane);
    };
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // this workgroup's K segment: super-blocks first .. first + nb - 1 of the rows
    const uint32_t first = blockIdx.y * p.seg_blocks;
    const uint32_t nb = min(p.seg_blocks, p.nb - first);
    const uint32_t row_bytes = nb * kBlock;          // of the segment
    const uint32_t full_row_bytes = p.nb * kBlock;
    const uint32_t row0 = blockIdx.x * p.tile_rows;
    const uint32_t rows = min(p.tile_rows, p.n - row0);

    uint8_t* const tile = lds;
    uint8_t* const slot = tile + p.tile_bytes + wave * kSlotBytes;
    float* const rsum = reinterpret_cast<float*>(tile + p.tile_bytes + kSWaves * kSlotBytes);

    // 1. this wave's activation blocks are requested first.  These are register loads the
    // compiler cannot see the latency of: xraw[i] holds the data only after wait_vmcnt(issued)
    // under 3., which lets exactly the `issued` later LDS-direct loads stay in flight (vmcnt
    // retires in order, so "at most `issued` outstanding" means every load before them is done).
    // Until then nothing may read, copy or spill xraw: the empty asm with "+v"(xraw[i]) after the
    // wait is the first use the compiler is shown, the kernel has no scratch, and the build's
    // check of the generated text fails if any instruction between a load and the wait names a
    // destination register.
    const size_t xrow = ((size_t)blockIdx.z * p.nb + first) * 256u;
    typename std::conditional<DT == FH_F32, u32x4, u32x2>::type xraw[MAXB];
#pragma unroll
    for (int i = 0; i < MAXB; ++i) {
        // a wave with fewer blocks repeats its last one: the register is then defined by the
        // load alone, and nothing can touch it before the wait below
        const uint32_t b = min(wave + kSWaves * i, nb - 1u);
        // (with a scalar base and a lane offset instead of these 64-bit addresses the launch measured
        // 0.3 us slower on the 17408 x 5120 matrix, three rounds in turn on one device)
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
    const uint8_t* const wbase = p.w + (size_t)row0 * full_row_bytes + (size_t)first * kBlock;
    const uint32_t tile_addr = (uint32_t)(uintptr_t)tile;
    uint32_t issued = 0;
    // OWN: a super-block of the tile is tile_rows x 9 pieces of 16 bytes, piece 64 j + lane by instruction j
    const uint32_t block_pieces = p.tile_rows * (kBlock / 16u), groups = (block_pieces + 63u) / 64u;
    const uint32_t block_pitch = block_pieces * 16u;
    if constexpr (OWN) {
        // where a lane's piece of a block lies from the block's first row on: the same for every block
        uint32_t lane_offset[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t piece = 64u * j + lane, rl = piece / (kBlock / 16u), pc = piece - rl * (kBlock / 16u);
            lane_offset[j] = min(rl, rows - 1u) * full_row_bytes + 16u * pc;
        }
        const uint8_t* const first_row = p.w + (size_t)row0 * full_row_bytes + (size_t)first * kBlock;
#pragma unroll
        for (int i = 0; i < MAXB; ++i) {
            const uint32_t b = wave + kSWaves * i;
            if (b < nb) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if ((uint32_t)j < groups) {
                        if (64u * j + lane < block_pieces)
                            lds_load16_at(first_row + b * kBlock, lane_offset[j], tile_addr + b * block_pitch + 1024u * j);
                        ++issued;
                    }
                }
            }
        }
    } else {
        for (uint32_t i = wave; i < total; i += kSWaves) {
            const uint32_t r = i / per_row, c = i - r * per_row;
            if (c * 1024u + lane * 16u < row_bytes)
                lds_load16_at(wbase + (size_t)r * full_row_bytes + c * 1024u, lane * 16u,
                              tile_addr + r * p.row_stride + c * 1024u);
            ++issued;
        }
    }
    if (lane < 4u) reinterpret_cast<uint32_t*>(slot + 1024u + kAuxBytes)[lane] = 0u;

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
    stage(xv[0], slot, lane);   // the first block while the tile is on its way
    if constexpr (!OWN) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // 4. multiply this wave's super-blocks
    const uint32_t n = lane & 15u, g = lane >> 4;
    const uint32_t nc = n < rows ? n : rows - 1u;
    const bool active = (n >> 2) == g;
    const uint8_t* const wrow = tile + nc * p.row_stride;
    const uint8_t* const xlane = active ? slot + (g * 4u + (n & 3u)) * 16u : slot + 1024u + kAuxBytes;
    const uint32_t xstep = active ? 256u : 0u;
    const float* const auxp = reinterpret_cast<const float*>(slot + 1024u) + (kAuxBytes / 16u) * g;
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
            if constexpr (OWN) {
                // this block's loads have landed when only the later blocks' are outstanding
                wait_vmcnt(issued - (uint32_t)(i + 1) * groups);
            }
            if constexpr (TYPE == kQ4K) {
                const float4 aux = *reinterpret_cast<const float4*>(auxp);
                const uint8_t* const blk = OWN ? tile + b * block_pitch + nc * kBlock : wrow + b * kBlock;
                const uint4 hdr = *reinterpret_cast<const uint4*>(blk);
                const uint4 qa = *reinterpret_cast<const uint4*>(blk + 16u + 32u * g);
                const uint4 qb = *reinterpret_cast<const uint4*>(blk + 32u + 32u * g);
                if (i + 1 < MAXB && b + kSWaves < nb) {
                    asm volatile("s_waitcnt lgkmcnt(3)" ::: "memory");   // the five slot reads are the oldest
                    stage(xv[i + 1], slot, lane);
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
            } else {
                const float4 sums = *reinterpret_cast<const float4*>(auxp);
                const float4 inv = *reinterpret_cast<const float4*>(auxp + 4);
                asm volatile("" ::: "memory");   // the slot reads are issued before the tile reads
                const uint8_t* const blk = wrow + b * kBlock;
                const uint32_t h = g >> 1, e = g & 1u;
                const uint4 qa = lds_u4_unaligned(blk + 64u * h + 16u * e);
                const uint4 qb = lds_u4_unaligned(blk + 64u * h + 32u + 16u * e);
                const uint4 qh = lds_u4_unaligned(blk + 128u + 32u * h + 16u * e);
                const uint2 sc8 = lds_u2_unaligned(blk + 192u + 8u * h);
                uint16_t dbits;
                __builtin_memcpy(&dbits, blk + 208u, 2);
                if (i + 1 < MAXB && b + kSWaves < nb) {
                    // the six slot reads are the oldest; at least five instructions read the tile
                    asm volatile("s_waitcnt lgkmcnt(5)" ::: "memory");
                    stage(xv[i + 1], slot, lane);
                }
                const uint32_t ql[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
                const uint32_t ph[4] = {qh.x, qh.y, qh.z, qh.w};
                // [piece][low nibbles, high nibbles, their bit planes]
                floatx4 dn[2][4];
#pragma unroll
                for (int pc = 0; pc < 2; ++pc)
#pragma unroll
                    for (int t = 0; t < 4; ++t) dn[pc][t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int up = 0; up < 2; ++up) {
                    const uint32_t p0 = ph[2 * up], p1 = ph[2 * up + 1];
                    const uint32_t t0 = p0 >> 8, t1 = p1 >> 8;
#pragma unroll
                    for (int pc = 0; pc < 2; ++pc) {
                        const uint32_t q0 = ql[4 * pc + 2 * up], q1 = ql[4 * pc + 2 * up + 1];
                        const uint32_t s0 = q0 >> 8, s1 = q1 >> 8;
                        // Bit planes 0 and 2 belong to the first ql piece, 1 and 3 to the second.  The matrix
                        // core's sum keeps a fixed number of bits below the operands' exponent field, which is
                        // the same for every subnormal, so what a dot product loses does not depend on where
                        // in the field the bits sit, while the factor that undoes the position does: planes 0
                        // and 1, whose values count sixteenfold, move to the top of the field (bits 8..9).
                        const uint32_t mh = pc == 0 ? 0x00300030u : 0x00c000c0u;
                        const u32x4 nl = {q0 & 0x000f000fu, s0 & 0x000f000fu, q1 & 0x000f000fu, s1 & 0x000f000fu};
                        const u32x4 nh = {q0 & 0x00f000f0u, s0 & 0x00f000f0u, q1 & 0x00f000f0u, s1 & 0x00f000f0u};
                        const u32x4 pl = pc == 0 ? u32x4{(p0 << 8) & 0x03000300u, p0 & 0x03000300u, (p1 << 8) & 0x03000300u,
                                                         p1 & 0x03000300u}
                                                 : u32x4{(p0 << 6) & 0x03000300u, (p0 >> 2) & 0x03000300u,
                                                         (p1 << 6) & 0x03000300u, (p1 >> 2) & 0x03000300u};
                        const u32x4 pw = {p0 & mh, t0 & mh, p1 & mh, t1 & mh};
                        const half8 a = __builtin_bit_cast(half8, xa[2 * pc + up]);
                        dn[pc][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8, nl), dn[pc][0], 0, 0, 0);
                        dn[pc][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8, nh), dn[pc][1], 0, 0, 0);
                        dn[pc][2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8, pl), dn[pc][2], 0, 0, 0);
                        dn[pc][3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(half8, pw), dn[pc][3], 0, 0, 0);
                    }
                }
                // The operands were (times 2^-24): low nibble q, high nibble 16 q, planes 0 and 1 256 v, plane 2
                // 16 v, plane 3 64 v; a weight is q + 16 v - 32.  Slices 0 and 2 come from the first piece.
                const float s0q = fmaf(16.f, dn[0][0][0] + dn[0][0][1], dn[0][2][0] + dn[0][2][1]) * 1048576.f;
                const float s2q = fmaf(16.f, dn[0][3][2] + dn[0][3][3], dn[0][1][2] + dn[0][1][3]) * 1048576.f;
                const float s1q = fmaf(16.f, dn[1][0][0] + dn[1][0][1], dn[1][2][0] + dn[1][2][1]) * 1048576.f;
                const float s3q = fmaf(4.f, dn[1][3][2] + dn[1][3][3], dn[1][1][2] + dn[1][1][3]) * 1048576.f;
                // the lane group's int8 scales: bytes e, e + 2, e + 4, e + 6 of its half's eight
                const uint32_t lo = sc8.x >> (8u * e), hi = sc8.y >> (8u * e);
                const float c0 = (float)(int)(int8_t)lo, c1 = (float)(int)(int8_t)(lo >> 16);
                const float c2 = (float)(int)(int8_t)hi, c3 = (float)(int)(int8_t)(hi >> 16);
                const float r0 = fmaf(s0q, inv.x, -32.f * sums.x), r1 = fmaf(s1q, inv.y, -32.f * sums.y);
                const float r2 = fmaf(s2q, inv.z, -32.f * sums.z), r3 = fmaf(s3q, inv.w, -32.f * sums.w);
                const float total = fmaf(c0, r0, c1 * r1) + fmaf(c2, r2, c3 * r3);
                acc = fmaf(f16_bits_to_f32(dbits), total, acc);
            }
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

template <int DT, int WAVES, int MAXB>
__global__ __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(6, 6)))
void gemv_stream_q4k(const StreamParams p) {
    gemv_stream_body<kQ4K, DT, WAVES, MAXB>(p);
}

template <int DT, int WAVES, int MAXB>
__global__ __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(6, 6)))
void gemv_stream_q4k_own(const StreamParams p) {
    gemv_stream_body<kQ4K, DT, WAVES, MAXB, true>(p);
}

// Q6_K rows are 46% longer: two workgroups share a compute unit, four waves per SIMD.
template <int DT, int WAVES, int MAXB>
__global__ __launch_bounds__(WAVES * kWave) void gemv_stream_q6k(const StreamParams p) {
    gemv_stream_body<kQ6K, DT, WAVES, MAXB>(p);
}

}  // namespace

// Tile height that spreads the rows evenly: the fewest 16-row rounds per compute unit, then the
// smallest height that still fits them.
StreamPlan gemv_stream_plan(uint32_t ggml_type, uint32_t n, uint32_t k, uint32_t m, int cu_count, bool any_size,
                            int forced_segments) {
    StreamPlan plan{};
    const bool q6 = ggml_type == kQ6K;
    const uint32_t block = q6 ? kQ6Bytes : kQ4Bytes, slot = q6 ? kSlot6Bytes : kSlotBytes;
    const uint32_t nb = k / 256u;
    const uint32_t cus = cu_count > 0 ? (uint32_t)cu_count : 256u;
    const uint32_t rounds = ((n + 15u) / 16u + cus - 1u) / cus;
    uint32_t h = (n + cus * rounds - 1u) / (cus * rounds);
    if (h > 16u) h = 16u;
    if (h < 1u) h = 1u;
    // A tile stays below 64 KB -- 70 KB for Q6_K, whose workgroups share a compute unit in twos and
    // whose sixteen rows of 5120 weights are 67 KB -- so that two or three workgroups share a compute
    // unit's LDS (the LDS-direct loads themselves reach every LDS address: M0 values of 69632, 135168
    // and 150000 were written to and read back on this device), and a wave owns at most six
    // super-blocks: longer rows are cut into K segments of equal length.
    const uint32_t tile_cap = q6 ? 70u * 1024u : 65536u;
    auto stride_of = [block](uint32_t blocks) {
        uint32_t units = (block * blocks + 15u) / 16u;   // bytes / 16
        if ((units & 1u) == 0) ++units;    // odd number of 16-byte units: 16 rows start in 16 different bank groups
        return units * 16u;
    };
    // ... and, where it must be cut anyway, short enough that three workgroups share a compute
    // unit's LDS (the headline's uncut 14 x 2896 bytes do)
    const uint32_t budget = (160u * 1024u) / 3u - 8u * slot - 8u * 64u;
    // (the segments then spread the work, so the tiles are as tall as the matrix instruction)
    // the reference's K-split switch asks for at least that many segments, as far as whole blocks go
    const uint32_t wanted = forced_segments > 1 ? ((uint32_t)forced_segments < nb ? (uint32_t)forced_segments : nb) : 1u;
    if (wanted > 1u || nb > 48u || h * stride_of(nb) > tile_cap) h = n < 16u ? n : 16u;
    uint32_t segments = wanted, seg = (nb + wanted - 1u) / wanted;
    // LDS-direct loads want dword-aligned addresses: a Q6_K segment starts on an even block
    auto even_up = [q6](uint32_t blocks) { return q6 ? (blocks + 1u) & ~1u : blocks; };
    if (segments > 1u) seg = even_up(seg);
    while (seg > 48u || h * stride_of(seg) > (segments == 1 ? tile_cap : budget)) {
        ++segments;
        seg = even_up((nb + segments - 1u) / segments);
        if (seg <= (q6 ? 2u : 1u)) break;
    }
    segments = (nb + seg - 1u) / seg;
    plan.segments = segments;
    plan.seg_blocks = seg;
    plan.row_stride = stride_of(seg);
    if (h * plan.row_stride > tile_cap) h = tile_cap / plan.row_stride;
    plan.tile_rows = h;
    plan.tiles = (n + h - 1u) / h;
    plan.waves = 8u;
    plan.lds_bytes = h * plan.row_stride + plan.waves * slot + plan.waves * 64u;
    // Matrices of a megabyte or two finish sooner on the FMA kernel's smaller workgroups.  Q6_K costs
    // twice the matrix instructions and half again the vector work of Q4_K per super-block, which
    // tiles of rows of 5120 do not hide (17408 x 5120 in fourteen-row tiles: 22.6 against 21.3 us on
    // the FMA kernel; 151936 x 5120 in fifteen-row tiles 142 - 147 against 141 - 142 us, in two K
    // segments 168 us); rows that must be cut into segments in any case gain (5120 x 17408: 22.7
    // against 25.0 us).  Output matrices of a million super-blocks or more whose rows the FMA kernel
    // cannot cut evenly over its eight block slots gain too, in uncut sixteen-row tiles (us, FMA
    // against this kernel: 151936 x 5120 139.7 / 134.5, 65536 x 5120 63.2 / 62.2, 262144 x 2560 131.7 /
    // 116.1; but 151936 x 4096 112.9 / 117.8, 128256 x 4096 95.9 / 100.4, 151936 x 2048 58.8 / 60.2,
    // 32000 x 5120 33.3 / 33.8).
    const bool big_head = q6 && segments == 1u && h == 16u && (nb & 7u) != 0 && (uint64_t)n * nb >= 1000000u;
    const bool wins = q6 ? nb > 48u || big_head : (uint64_t)n * nb >= 16384u;
    plan.ok = nb >= 1 && seg >= 1u && seg <= 48u && segments <= 65535u && h >= 1u && (any_size || wins) &&
              plan.lds_bytes <= 160u * 1024u && m >= 1 && m <= 65535u && (!q6 || (nb & 1u) == 0);
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
    p.tile_bytes = plan.tile_rows * plan.row_stride;
    p.x_dtype = a.x_dtype;
    p.y_dtype = a.y_dtype;
    p.segments = plan.segments;
    p.seg_blocks = plan.seg_blocks;
    p.m = a.m;
    p.partials = a.partials;
    p.counters = a.counters;
    typedef void (*Kernel)(const StreamParams);
    // [format][dtype][blocks per wave: 2, 3, 6]
    static const Kernel kernels[2][3][3] = {
        {{gemv_stream_q4k<FH_F32, 8, 2>, gemv_stream_q4k<FH_F32, 8, 3>, gemv_stream_q4k<FH_F32, 8, 6>},
         {gemv_stream_q4k<FH_F16, 8, 2>, gemv_stream_q4k<FH_F16, 8, 3>, gemv_stream_q4k<FH_F16, 8, 6>},
         {gemv_stream_q4k<FH_BF16, 8, 2>, gemv_stream_q4k<FH_BF16, 8, 3>, gemv_stream_q4k<FH_BF16, 8, 6>}},
        {{gemv_stream_q6k<FH_F32, 8, 2>, gemv_stream_q6k<FH_F32, 8, 3>, gemv_stream_q6k<FH_F32, 8, 6>},
         {gemv_stream_q6k<FH_F16, 8, 2>, gemv_stream_q6k<FH_F16, 8, 3>, gemv_stream_q6k<FH_F16, 8, 6>},
         {gemv_stream_q6k<FH_BF16, 8, 2>, gemv_stream_q6k<FH_BF16, 8, 3>, gemv_stream_q6k<FH_BF16, 8, 6>}},
    };
    static bool raised = false;
    if (!raised) {
        for (const auto& format : kernels)
            for (const auto& row : format)
                for (Kernel kernel : row)
                    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        raised = true;
    }
    const int shape = plan.seg_blocks <= 16u ? 0 : plan.seg_blocks <= 24u ? 1 : 2;
    const int format = a.ggml_type == kQ6K ? 1 : 0;
    // Q4_K tiles of up to 14 rows (two load instructions per super-block): every wave loads what it
    // multiplies and no workgroup barrier stands between the loads and the arithmetic.  Same box,
    // 17408 x 5120: 12.15 against 13.2 us and 12.3 against 12.4 us on two boxes (f16 activations 12.1
    // against 12.4); 5120 x 5120 6.5 either way.  Taller tiles need a third, nearly empty instruction
    // per block and lose (4096 x 4096: 4.54 against 4.40 us, 18992 x 5120: 14.0 against 13.8).
    const uint32_t own_bytes = plan.seg_blocks * plan.tile_rows * kQ4Bytes;
    if (a.stream_own && format == 0 && plan.tile_rows * (kQ4Bytes / 16u) <= 128u && own_bytes <= 65536u) {
        static const Kernel own_kernels[3][3] = {
            {gemv_stream_q4k_own<FH_F32, 8, 2>, gemv_stream_q4k_own<FH_F32, 8, 3>, gemv_stream_q4k_own<FH_F32, 8, 6>},
            {gemv_stream_q4k_own<FH_F16, 8, 2>, gemv_stream_q4k_own<FH_F16, 8, 3>, gemv_stream_q4k_own<FH_F16, 8, 6>},
            {gemv_stream_q4k_own<FH_BF16, 8, 2>, gemv_stream_q4k_own<FH_BF16, 8, 3>, gemv_stream_q4k_own<FH_BF16, 8, 6>},
        };
        Kernel kernel = own_kernels[a.x_dtype][shape];
        static bool once = false;
        if (!once) {
            for (const auto& row : own_kernels)
                for (Kernel k : row)
                    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            once = true;
        }
        p.tile_bytes = own_bytes;
        const uint32_t lds = own_bytes + plan.waves * kSlotBytes + plan.waves * 64u;
        hipLaunchKernelGGL(kernel, dim3(plan.tiles, plan.segments, a.m), dim3(plan.waves * kWave), lds, s, p);
        return plan.segments > 1 ? "q4_k_gemv_ksplit" : "q4_k_gemv_factored";
    }
    hipLaunchKernelGGL(kernels[format][a.x_dtype][shape], dim3(plan.tiles, plan.segments, a.m), dim3(plan.waves * kWave),
                       plan.lds_bytes, s, p);
    if (format == 1) return plan.segments > 1 ? "q6_k_gemv_ksplit" : "q6_k_gemv_factored";
    return plan.segments > 1 ? "q4_k_gemv_ksplit" : "q4_k_gemv_factored";
}

}  // namespace fh
