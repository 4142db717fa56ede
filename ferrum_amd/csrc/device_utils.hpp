// Device-side helpers shared by the kernels: storage dtypes, GGUF K-quant field
// extraction and 64-lane wave reductions.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace fh {

constexpr int kWave = 64;

// ---- storage dtypes (0 f32, 1 f16, 2 bf16) ------------------------------------

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(bits)));
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) {
    return __uint_as_float(bits << 16);
}

// Round to nearest even; NaN keeps its payload with the quiet bit set
// (the reference's store(), src/metal/shaders/ops.metal:11-20).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float x) {
    uint32_t bits = __float_as_uint(x);
    if (x != x) return (bits >> 16) | 0x40u;
    return (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float x) {
    return __half_as_ushort(__float2half_rn(x));
}

template <int DT>
__device__ __forceinline__ float load_as_f32(const void* p, size_t i) {
    if constexpr (DT == 0) {
        return static_cast<const float*>(p)[i];
    } else if constexpr (DT == 1) {
        return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    } else {
        return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    }
}

__device__ __forceinline__ float load_as_f32(const void* p, size_t i, uint32_t dtype) {
    if (dtype == 0) return static_cast<const float*>(p)[i];
    uint32_t bits = static_cast<const uint16_t*>(p)[i];
    return dtype == 1 ? f16_bits_to_f32(bits) : bf16_bits_to_f32(bits);
}

__device__ __forceinline__ void store_from_f32(void* p, size_t i, uint32_t dtype, float v) {
    if (dtype == 0) {
        static_cast<float*>(p)[i] = v;
    } else if (dtype == 1) {
        static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_f16_bits(v));
    } else {
        static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    }
}

__device__ __forceinline__ float round_storage(float v, uint32_t dtype) {
    if (dtype == 1) return f16_bits_to_f32(f32_to_f16_bits(v));
    if (dtype == 2) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    return v;
}

// SiLU in the branch-stable form of expert_silu_mul (src/metal/shaders/ops.metal:2223-2232):
// 1 / (1 + exp(-g)) for g >= 0 and exp(g) / (1 + exp(g)) below.  Both sides are one
// exponential of -|g| and one division, so they are written as that: the same values with
// half the work of evaluating the two sides.
__device__ __forceinline__ float silu_stable(float gate) {
    const float e = expf(-fabsf(gate));
    return gate * ((gate >= 0.f ? 1.f : e) / (1.f + e));
}

// 16-byte and 2-byte loads from addresses that are only 2-byte aligned (Q6_K
// blocks are 210 bytes); gfx950 global loads accept unaligned addresses.
__device__ __forceinline__ uint4 load_u4_unaligned(const uint8_t* p) {
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}
__device__ __forceinline__ uint32_t load_u16_unaligned(const uint8_t* p) {
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}

// ---- Q4_K (144 B: f16 d, f16 dmin, 12 B scales, 128 B nibbles) ----------------

// 6-bit scale and minimum of 32-weight group `group` (0..7).
__device__ __forceinline__ void q4k_scale_min(const uint8_t* s, uint32_t group, uint32_t& sc,
                                              uint32_t& mn) {
    if (group < 4) {
        sc = s[group] & 63u;
        mn = s[group + 4] & 63u;
    } else {
        sc = (s[group + 4] & 15u) | ((uint32_t)(s[group - 4] >> 6) << 4);
        mn = (uint32_t)(s[group + 4] >> 4) | ((uint32_t)(s[group] >> 6) << 4);
    }
}

// Scales and minimums of the two 32-weight groups 2c and 2c+1 that share the
// 32 quant bytes of chunk c (0..3), from the header words {bytes 4..7, 8..11,
// 12..15 of the block}.  Groups 4..7 keep their low nibbles in bytes 8..11
// and their top two bits in bits 6..7 of bytes 0..7.
__device__ __forceinline__ void q4k_chunk_scales(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t c,
                                                 float& sc_lo, float& sc_hi, float& mn_lo,
                                                 float& mn_hi) {
    // blended with a mask rather than selected: c differs between lanes and a
    // select of two computed values tends to come back as a divergent branch
    const uint32_t upper = 0u - (c >> 1);
    uint32_t scw = (((s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)) & upper) | (s0 & 0x3f3f3f3fu & ~upper);
    uint32_t mnw = ((((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)) & upper) |
                   (s1 & 0x3f3f3f3fu & ~upper);
    uint32_t shift = (c & 1u) << 4;
    scw >>= shift;
    mnw >>= shift;
    sc_lo = (float)(scw & 0xffu);
    sc_hi = (float)((scw >> 8) & 0xffu);
    mn_lo = (float)(mnw & 0xffu);
    mn_hi = (float)((mnw >> 8) & 0xffu);
}

// One dequantised weight, ((d*sc)*q) - (dmin*m) with each step rounded to f32.
// d and dmin carry 11 significant bits, so both products are exact and only
// the subtraction rounds; the value is therefore independent of contraction.
__device__ __forceinline__ float q4k_weight(const uint8_t* w, size_t row, uint32_t column,
                                            uint32_t blocks) {
    const uint8_t* block = w + (row * blocks + (column >> 8)) * 144;
    uint32_t within = column & 255u, group = within >> 5, lane = within & 31u, chunk = within >> 6;
    uint32_t byte = block[16 + chunk * 32 + lane];
    uint32_t q = (group & 1u) ? (byte >> 4) : (byte & 15u);
    float d = f16_bits_to_f32(block[0] | (block[1] << 8));
    float dmin = f16_bits_to_f32(block[2] | (block[3] << 8));
    uint32_t sc, mn;
    q4k_scale_min(block + 4, group, sc, mn);
    float a = d * (float)sc;
    float b = a * (float)q;
    float c = dmin * (float)mn;
    return b - c;
}

// ---- Q5_K (176 B: f16 d, f16 dmin, scales[12], qh[32], qs[128]) -----------------

// q5_k_weight (src/metal/shaders/ops.metal:846-857): the Q4_K value with bit
// `group` of qh[lane] as the quant's fifth bit.
__device__ __forceinline__ float q5k_weight(const uint8_t* w, size_t row, uint32_t column,
                                            uint32_t blocks) {
    const uint8_t* block = w + (row * blocks + (column >> 8)) * 176;
    uint32_t within = column & 255u, group = within >> 5, lane = within & 31u, chunk = within >> 6;
    uint32_t byte = block[48 + chunk * 32 + lane];
    uint32_t q = (group & 1u) ? (byte >> 4) : (byte & 15u);
    q |= (((uint32_t)block[16 + lane] >> group) & 1u) << 4;
    float d = f16_bits_to_f32(block[0] | (block[1] << 8));
    float dmin = f16_bits_to_f32(block[2] | (block[3] << 8));
    uint32_t sc, mn;
    q4k_scale_min(block + 4, group, sc, mn);
    float a = d * (float)sc;
    float b = a * (float)q;
    float c = dmin * (float)mn;
    return b - c;
}

// ---- Q6_K (210 B: ql[128], qh[64], int8 scales[16], f16 d) ---------------------

__device__ __forceinline__ float q6k_weight(const uint8_t* w, size_t row, uint32_t column,
                                            uint32_t blocks) {
    const uint8_t* block = w + (row * blocks + (column >> 8)) * 210;
    uint32_t within = column & 255u, group = within >> 5, lane = within & 31u;
    uint32_t half_block = group >> 2, slice = group & 3u;
    uint32_t byte = block[half_block * 64 + (slice & 1u) * 32 + lane];
    uint32_t low = slice < 2 ? (byte & 15u) : (byte >> 4);
    uint32_t high = ((uint32_t)block[128 + half_block * 32 + lane] >> (slice * 2)) & 3u;
    int q = (int)(low | (high << 4)) - 32;
    int scale = (int8_t)block[192 + half_block * 8 + slice * 2 + (lane >> 4)];
    float d = f16_bits_to_f32(block[208] | (block[209] << 8));
    float a = d * (float)scale;
    return a * (float)q;
}

// ---- IQ4_XS (136 B: f16 d, u16 scales_h, scales_l[4], qs[128]) ------------------
//
// block_iq4_xs / dequantize_iq4_xs (src/metal/shaders/hybrid.metal:27, 580-596):
// eight 32-weight sub-blocks.  Sub-block i owns qs[16i .. 16i + 15]: the low
// nibble of byte j is its weight j, the high nibble its weight 16 + j.  A
// nibble indexes a 16-entry codebook (kvalues_iq4nl_f, hybrid.metal:34-37);
// the sub-block scale is d * (ls - 32) with the 6-bit ls = nibble i of
// scales_l | bits 2i, 2i + 1 of scales_h << 4.  d * (ls - 32) has at most 17
// significant bits and the codebook 7, so the f32 weight is exact.

// codebook value + 128 (1 .. 241) as unsigned bytes, four per word
constexpr uint32_t kIq4Table0 = 0x3f2d1801u;  //  -127 -104  -83  -65
constexpr uint32_t kIq4Table1 = 0x766a5d4fu;  //   -49  -35  -22  -10
constexpr uint32_t kIq4Table2 = 0xa6998d81u;  //     1   13   25   38
constexpr uint32_t kIq4Table3 = 0xf1d9c5b5u;  //    53   69   89  113

// The low nibble of each byte of q, looked up: four bytes of codebook + 128.
// v_perm_b32 picks from eight table bytes by the nibble's low three bits; a
// third one picks between the two halves of the table by its top bit.
__device__ __forceinline__ uint32_t iq4_lookup4(uint32_t q) {
    const uint32_t low3 = q & 0x07070707u;
    const uint32_t a = __builtin_amdgcn_perm(kIq4Table1, kIq4Table0, low3);
    const uint32_t b = __builtin_amdgcn_perm(kIq4Table3, kIq4Table2, low3);
    const uint32_t pick = ((q >> 1) & 0x04040404u) | 0x03020100u;
    return __builtin_amdgcn_perm(b, a, pick);
}

// Bytes 0, 1 (or 2, 3) of v, each widened to a 16-bit field: read as f16 these
// are the subnormals byte * 2^-24.
__device__ __forceinline__ uint32_t bytes01_as_halves(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c010c00u); }
__device__ __forceinline__ uint32_t bytes23_as_halves(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c030c02u); }

// d * (ls - 32) of sub-block i from the header words {d | scales_h << 16, scales_l}
__device__ __forceinline__ float iq4xs_scale(uint32_t h0, uint32_t h1, uint32_t i) {
    const uint32_t ls = ((h1 >> (4u * i)) & 15u) | (((h0 >> (16u + 2u * i)) & 3u) << 4);
    return f16_bits_to_f32(h0 & 0xffffu) * (float)((int)ls - 32);
}

__device__ __forceinline__ float iq4xs_weight(const uint8_t* w, size_t row, uint32_t column, uint32_t blocks) {
    const uint8_t* block = w + (row * blocks + (column >> 8)) * 136;
    const uint32_t within = column & 255u, sub = within >> 5, j = within & 31u;
    const uint32_t byte = block[8 + 16 * sub + (j & 15u)];
    const uint32_t index = j < 16 ? (byte & 15u) : (byte >> 4);
    const uint32_t h0 = block[0] | (block[1] << 8) | (block[2] << 16) | ((uint32_t)block[3] << 24);
    const uint32_t h1 = block[4] | (block[5] << 8) | (block[6] << 16) | ((uint32_t)block[7] << 24);
    const uint32_t word = index < 8 ? (index < 4 ? kIq4Table0 : kIq4Table1) : (index < 12 ? kIq4Table2 : kIq4Table3);
    const int value = (int)((word >> (8u * (index & 3u))) & 0xffu) - 128;
    return iq4xs_scale(h0, h1, sub) * (float)value;
}

// ---- Q8_0 (34 B: f16 d, int8 qs[32]; eight blocks per 256 weights) ---------------
//
// block_q8_0 / dequantize_q8_0 (src/metal/shaders/hybrid.metal:23, 499-508; CPU
// twin src/hybrid/draft/gguf.rs:331-338): weight = d * q, exact in f32.

__device__ __forceinline__ float q8_0_weight(const uint8_t* w, size_t row, uint32_t column, uint32_t blocks) {
    const uint8_t* block = w + (row * blocks + (column >> 8)) * 272 + 34 * ((column & 255u) >> 5);
    const float d = f16_bits_to_f32(block[0] | (block[1] << 8));
    return d * (float)(int)(int8_t)block[2 + (column & 31u)];
}

// 4-byte aligned 16-byte and 4-byte loads
__device__ __forceinline__ uint32_t load_u32_unaligned(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}

// One lane's 64 weights of a 256-weight run: blocks 2c and 2c + 1, 68 bytes at 68c,
// [d0][q0 x 32][d1][q1 x 32].  The quants of the first block straddle dwords by two
// bytes; v_alignbyte_b32 puts them back.  q + 128 (a byte xor) is then widened like
// the other formats' quants.
struct Q8Pair {
    uint32_t w[17];
    __device__ __forceinline__ void load(const uint8_t* p) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 v;
            __builtin_memcpy(&v, p + 16 * i, 16);
            w[4 * i] = v.x;
            w[4 * i + 1] = v.y;
            w[4 * i + 2] = v.z;
            w[4 * i + 3] = v.w;
        }
        w[16] = load_u32_unaligned(p + 64);
    }
    __device__ __forceinline__ float d(int block) const {
        return f16_bits_to_f32(block == 0 ? (w[0] & 0xffffu) : (w[8] >> 16));
    }
    // quant dword j (0..7) of block `block`, four bytes of q + 128
    __device__ __forceinline__ uint32_t biased(int block, int j) const {
        const uint32_t q = block == 0 ? __builtin_amdgcn_alignbyte(w[j + 1], w[j], 2) : w[9 + j];
        return q ^ 0x80808080u;
    }
};

// ---- wave reductions -----------------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(moved);
}

// Sum over the 64 lanes; every lane of the wave must be active.  The total is
// returned in all lanes.
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror: the other quad of each 8
    v = dpp_add<0x140>(v);  // row_mirror: the other half of each 16
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    // lanes the pattern leaves unwritten keep the old value (the first operand): their own v
    int moved = __builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, false);
    return fmaxf(v, __int_as_float(moved));
}

// The same on unsigned integers (and so on the bit patterns of non-negative floats): lanes the
// pattern leaves unwritten read 0, the identity, which lets the move fold into v_max_u32_dpp.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_umax(uint32_t v) {
    const uint32_t moved = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
    return moved > v ? moved : v;
}

// Maximum over the 64 lanes, returned in all lanes; every lane of the wave must be active.
__device__ __forceinline__ float wave_max(float v) {
    v = dpp_max<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_max<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_max<0x141>(v);  // row_half_mirror
    v = dpp_max<0x140>(v);  // row_mirror
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

}  // namespace fh
