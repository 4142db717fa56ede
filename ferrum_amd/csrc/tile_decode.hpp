// Pieces shared by the MFMA tile kernels: the 16x16x32 matrix instruction and
// the one-rounding decode of quants into f16 / bf16 tile values.
#pragma once

#include "device_utils.hpp"

namespace fh {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ float4v mfma16(uint4 a, uint4 b, float4v c) {
    if constexpr (DT == 1) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a),
                                                      __builtin_bit_cast(half8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// exact widening of an f16 (sub)normal held in one half of a dword
__device__ __forceinline__ float lo_half(uint32_t v) { return (float)__builtin_bit_cast(half2v, v).x; }
__device__ __forceinline__ float hi_half(uint32_t v) { return (float)__builtin_bit_cast(half2v, v).y; }

// Two tile values fma(q, scale, offset), each rounded once to the tile dtype,
// packed into a dword.  q arrives as an f16 subnormal (an integer quant masked
// in place, i.e. q * 2^-24 or 16q * 2^-24) and `scale` carries the inverse
// power of two, so the f32 product is the exact integer multiple and the
// result has the bits of the reference's (d*sc)*q - dmin*m.  For f16 the
// compiler emits v_fma_mixlo/mixhi_f16: no conversion or pack instructions.
template <int DT>
__device__ __forceinline__ uint32_t fma_pair(float qa, float qb, float scale, float offset) {
    if constexpr (DT == 1) {
        half2v r;
        r.x = (_Float16)fmaf(qa, scale, offset);
        r.y = (_Float16)fmaf(qb, scale, offset);
        return __builtin_bit_cast(uint32_t, r);
    } else {
        return f32_to_bf16_bits(fmaf(qa, scale, offset)) | (f32_to_bf16_bits(fmaf(qb, scale, offset)) << 16);
    }
}

}  // namespace fh
