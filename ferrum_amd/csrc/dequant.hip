// Whole-matrix dequantisation and embedding gather for GGUF Q4_K / Q5_K / Q6_K / IQ4_XS / Q8_0.
//
// Values follow the reference's per-element decoders (q4_k_weight,
// src/metal/shaders/ops.metal:834-845; q6_k_weight, :1316-1329); the gather
// kernels stand in for embedding_gather_q4_k / _q6_k (:1122-1127, 1486-1491).
// One thread produces four consecutive columns, so stores are 16 bytes (f32)
// or 8 bytes (f16 / bf16) and each 144- or 210-byte block is read by 64
// neighbouring threads.  Rows are stored `cols` wide (a multiple of 256) and written
// `out_cols` wide: a Q8_0 row of 32 n weights is kept padded with empty blocks.
#include "device_utils.hpp"
#include "internal.hpp"

namespace fh {
namespace {

template <uint32_t TYPE>
__device__ __forceinline__ float weight_at(const uint8_t* w, size_t row, uint32_t column,
                                           uint32_t blocks) {
    if constexpr (TYPE == kQ4K) {
        return q4k_weight(w, row, column, blocks);
    } else if constexpr (TYPE == kQ5K) {
        return q5k_weight(w, row, column, blocks);
    } else if constexpr (TYPE == kIQ4XS) {
        return iq4xs_weight(w, row, column, blocks);
    } else if constexpr (TYPE == kQ8_0) {
        return q8_0_weight(w, row, column, blocks);
    } else {
        return q6k_weight(w, row, column, blocks);
    }
}

template <uint32_t TYPE>
__device__ __forceinline__ void emit4(const uint8_t* w, size_t src_row, size_t dst_row,
                                      uint32_t column, uint32_t cols, uint32_t out_cols, void* out, uint32_t dtype) {
    uint32_t blocks = cols >> 8;
    float v0 = weight_at<TYPE>(w, src_row, column, blocks);
    float v1 = weight_at<TYPE>(w, src_row, column + 1, blocks);
    float v2 = weight_at<TYPE>(w, src_row, column + 2, blocks);
    float v3 = weight_at<TYPE>(w, src_row, column + 3, blocks);
    size_t base = dst_row * out_cols + column;
    if (dtype == 0) {
        *reinterpret_cast<float4*>(static_cast<float*>(out) + base) = make_float4(v0, v1, v2, v3);
    } else {
        uint32_t lo, hi;
        if (dtype == 1) {
            lo = f32_to_f16_bits(v0) | (f32_to_f16_bits(v1) << 16);
            hi = f32_to_f16_bits(v2) | (f32_to_f16_bits(v3) << 16);
        } else {
            lo = f32_to_bf16_bits(v0) | (f32_to_bf16_bits(v1) << 16);
            hi = f32_to_bf16_bits(v2) | (f32_to_bf16_bits(v3) << 16);
        }
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(out) + base) = make_uint2(lo, hi);
    }
}

template <uint32_t TYPE>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ w,
                                                         size_t rows, uint32_t cols, uint32_t out_cols,
                                                         void* __restrict__ out, uint32_t dtype) {
    uint32_t quads_per_row = out_cols >> 2;
    size_t total = rows * quads_per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t row = i / quads_per_row;
        uint32_t column = (uint32_t)(i % quads_per_row) << 2;
        emit4<TYPE>(w, row, row, column, cols, out_cols, out, dtype);
    }
}

template <uint32_t TYPE>
__global__ __launch_bounds__(256) void embedding_gather_kernel(const uint8_t* __restrict__ w,
                                                               uint32_t cols, uint32_t out_cols,
                                                               const uint32_t* __restrict__ ids,
                                                               size_t count,
                                                               void* __restrict__ out,
                                                               uint32_t dtype) {
    uint32_t quads_per_row = out_cols >> 2;
    size_t total = count * quads_per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        size_t token = i / quads_per_row;
        uint32_t column = (uint32_t)(i % quads_per_row) << 2;
        emit4<TYPE>(w, ids[token], token, column, cols, out_cols, out, dtype);
    }
}

unsigned grid_for(size_t threads) {
    size_t blocks = (threads + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks == 0) blocks = 1;
    return (unsigned)blocks;
}

}  // namespace

const char* launch_dequantize(hipStream_t s, uint32_t ggml_type, const void* w, size_t rows,
                              size_t cols, size_t out_cols, void* out, uint32_t out_dtype) {
    unsigned grid = grid_for(rows * (out_cols / 4));
    if (ggml_type == kQ4K) {
        hipLaunchKernelGGL(dequantize_kernel<kQ4K>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), rows, (uint32_t)cols, (uint32_t)out_cols, out, out_dtype);
        return "dequantize_q4_k";
    }
    if (ggml_type == kQ5K) {
        hipLaunchKernelGGL(dequantize_kernel<kQ5K>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), rows, (uint32_t)cols, (uint32_t)out_cols, out, out_dtype);
        return "dequantize_q5_k";
    }
    if (ggml_type == kIQ4XS) {
        hipLaunchKernelGGL(dequantize_kernel<kIQ4XS>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), rows, (uint32_t)cols, (uint32_t)out_cols, out, out_dtype);
        return "dequantize_iq4_xs";
    }
    if (ggml_type == kQ8_0) {
        hipLaunchKernelGGL(dequantize_kernel<kQ8_0>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), rows, (uint32_t)cols, (uint32_t)out_cols, out, out_dtype);
        return "dequantize_q8_0";
    }
    hipLaunchKernelGGL(dequantize_kernel<kQ6K>, dim3(grid), dim3(256), 0, s,
                       static_cast<const uint8_t*>(w), rows, (uint32_t)cols, (uint32_t)out_cols, out, out_dtype);
    return "dequantize_q6_k";
}

const char* launch_embedding_gather(hipStream_t s, uint32_t ggml_type, const void* w, size_t cols, size_t out_cols,
                                    const uint32_t* ids_dev, size_t count, void* out,
                                    uint32_t out_dtype) {
    unsigned grid = grid_for(count * (out_cols / 4));
    if (ggml_type == kQ4K) {
        hipLaunchKernelGGL(embedding_gather_kernel<kQ4K>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), (uint32_t)cols, (uint32_t)out_cols, ids_dev, count, out,
                           out_dtype);
        return "embedding_gather_q4_k";
    }
    if (ggml_type == kQ5K) {
        hipLaunchKernelGGL(embedding_gather_kernel<kQ5K>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), (uint32_t)cols, (uint32_t)out_cols, ids_dev, count, out,
                           out_dtype);
        return "embedding_gather_q5_k";
    }
    if (ggml_type == kIQ4XS) {
        hipLaunchKernelGGL(embedding_gather_kernel<kIQ4XS>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), (uint32_t)cols, (uint32_t)out_cols, ids_dev, count, out,
                           out_dtype);
        return "embedding_gather_iq4_xs";
    }
    if (ggml_type == kQ8_0) {
        hipLaunchKernelGGL(embedding_gather_kernel<kQ8_0>, dim3(grid), dim3(256), 0, s,
                           static_cast<const uint8_t*>(w), (uint32_t)cols, (uint32_t)out_cols, ids_dev, count, out,
                           out_dtype);
        return "embedding_gather_q8_0";
    }
    hipLaunchKernelGGL(embedding_gather_kernel<kQ6K>, dim3(grid), dim3(256), 0, s,
                       static_cast<const uint8_t*>(w), (uint32_t)cols, (uint32_t)out_cols, ids_dev, count, out,
                       out_dtype);
    return "embedding_gather_q6_k";
}

namespace {

__global__ __launch_bounds__(256) void round_to_f16_kernel(const float4* __restrict__ in, uint4* __restrict__ out,
                                                           size_t groups) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < groups;
         i += (size_t)gridDim.x * blockDim.x) {
        const float4 a = in[2 * i], b = in[2 * i + 1];
        uint4 v;
        v.x = f32_to_f16_bits(a.x) | (f32_to_f16_bits(a.y) << 16);
        v.y = f32_to_f16_bits(a.z) | (f32_to_f16_bits(a.w) << 16);
        v.z = f32_to_f16_bits(b.x) | (f32_to_f16_bits(b.y) << 16);
        v.w = f32_to_f16_bits(b.z) | (f32_to_f16_bits(b.w) << 16);
        out[i] = v;
    }
}

// Rows of `parts` pieces of `cols` elements each, rewritten with every piece `padded` elements long and
// zero beyond `cols`: activations on their way to a matrix whose rows are stored padded.  One thread
// moves eight bytes (cols and padded are multiples of 32 elements of two or four bytes).
__global__ __launch_bounds__(256) void pad_rows_kernel(const uint2* __restrict__ in, uint2* __restrict__ out,
                                                       size_t pieces, uint32_t cols8, uint32_t padded8) {
    const size_t total = pieces * padded8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const size_t piece = i / padded8;
        const uint32_t at = (uint32_t)(i % padded8);
        out[i] = at < cols8 ? in[piece * cols8 + at] : make_uint2(0u, 0u);
    }
}

}  // namespace

namespace {

// argmax_rows (src/metal/shaders/ops.metal:2438-2464) with the reference's own
// schedule, so rows that hold NaN report the same (flagged) index: 1024
// threads per row scan columns tid, tid + 1024, ...; groups of 32 lanes merge
// by a shuffle-down tree; thread 0 folds the 32 group results in order.
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const void* __restrict__ logits, uint32_t dtype,
                                                           uint32_t width, uint32_t* __restrict__ out) {
    __shared__ float best_value[32];
    __shared__ uint32_t best_index[32], bad_any[32];
    const uint32_t tid = threadIdx.x, row = blockIdx.x;
    const size_t base = (size_t)row * width;
    float best = -INFINITY;
    uint32_t index = 0xffffffffu, bad = 0;
    for (uint32_t j = tid; j < width; j += 1024) {
        const float x = load_as_f32(logits, base + j, dtype);
        bad |= (uint32_t)!isfinite(x);
        if (x > best || index == 0xffffffffu) {
            best = x;
            index = j;
        }
    }
    for (uint32_t offset = 16; offset > 0; offset /= 2) {
        const float other = __shfl_down(best, offset, 32);
        const uint32_t other_index = __shfl_down(index, offset, 32);
        if (other > best || (other == best && other_index < index)) {
            best = other;
            index = other_index;
        }
    }
    for (uint32_t offset = 16; offset > 0; offset /= 2) bad |= __shfl_xor(bad, offset, 32);
    if ((tid & 31u) == 0) {
        best_value[tid >> 5] = best;
        best_index[tid >> 5] = index;
        bad_any[tid >> 5] = bad;
    }
    __syncthreads();
    if (tid == 0) {
        for (uint32_t s = 1; s < 32; ++s) {
            if (best_value[s] > best || (best_value[s] == best && best_index[s] < index)) {
                best = best_value[s];
                index = best_index[s];
            }
            bad |= bad_any[s];
        }
        out[2 * (size_t)row] = index;
        out[2 * (size_t)row + 1] = bad;
    }
}

}  // namespace

const char* launch_argmax_rows(hipStream_t s, const void* logits, uint32_t dtype, uint32_t rows, uint32_t width,
                               uint32_t* out) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(1024), 0, s, logits, dtype, width, out);
    return "argmax_rows";
}

void launch_round_to_f16(hipStream_t s, const float* in, uint16_t* out, size_t count) {
    const size_t groups = count / 8;
    size_t blocks = (groups + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(round_to_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, s,
                       reinterpret_cast<const float4*>(in), reinterpret_cast<uint4*>(out), groups);
}

void launch_pad_rows(hipStream_t s, const void* in, void* out, size_t pieces, size_t cols, size_t padded,
                     size_t element_bytes) {
    const uint32_t cols8 = (uint32_t)(cols * element_bytes / 8), padded8 = (uint32_t)(padded * element_bytes / 8);
    hipLaunchKernelGGL(pad_rows_kernel, dim3(grid_for(pieces * padded8)), dim3(256), 0, s,
                       static_cast<const uint2*>(in), static_cast<uint2*>(out), pieces, cols8, padded8);
}

}  // namespace fh
