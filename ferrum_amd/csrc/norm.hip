// Residual add fused with the RMSNorm that follows it: the step between two
// projections of a decoder layer.
//
//   residual = round_storage(a + b)
//   normed   = residual * rsqrt(mean(residual^2) + eps) * weight
//
// add_rmsnorm (src/metal/shaders/ops.metal:99-124; host side
// MetalDevice::add_rmsnorm, src/ops/mod.rs:762-820) and, for f32 rows, the
// hybrid engine's h_add_rmsnorm (src/metal/shaders/hybrid.metal:1576-1595).
// The residual is the storage-rounded sum, so it equals a separate `add`; the
// mean runs over the rounded values in f32 and the product is taken as
// (x * inv) * weight, as the reference's kernels do.
//
// One workgroup of 256 threads per row.  Rows whose width is a multiple of 4
// move as 16-byte (f32) or 8-byte (f16 / bf16) groups and stay in registers
// between the two passes up to 16384 columns; other rows take the element loop
// and read a and b twice.
#include "device_utils.hpp"
#include "internal.hpp"

namespace fh {
namespace {

constexpr int kNormThreads = 256;
constexpr int kNormMaxCache = 16;  // most groups of 4 a thread keeps between the passes

// sum over the workgroup, returned in every thread
__device__ __forceinline__ float block_sum(float v, float* partial) {
    v = wave_sum(v);
    if ((threadIdx.x & 63u) == 0) partial[threadIdx.x >> 6] = v;
    __syncthreads();
    return (partial[0] + partial[1]) + (partial[2] + partial[3]);
}

template <int DT>
__device__ __forceinline__ float4 load4(const void* p, size_t group) {
    if constexpr (DT == 0) {
        return static_cast<const float4*>(p)[group];
    } else {
        const uint2 raw = static_cast<const uint2*>(p)[group];
        if constexpr (DT == 1) {
            return make_float4(f16_bits_to_f32(raw.x & 0xffffu), f16_bits_to_f32(raw.x >> 16),
                               f16_bits_to_f32(raw.y & 0xffffu), f16_bits_to_f32(raw.y >> 16));
        } else {
            return make_float4(bf16_bits_to_f32(raw.x & 0xffffu), bf16_bits_to_f32(raw.x >> 16),
                               bf16_bits_to_f32(raw.y & 0xffffu), bf16_bits_to_f32(raw.y >> 16));
        }
    }
}

template <int DT>
__device__ __forceinline__ void store4(void* p, size_t group, float4 v) {
    if constexpr (DT == 0) {
        static_cast<float4*>(p)[group] = v;
    } else if constexpr (DT == 1) {
        static_cast<uint2*>(p)[group] = make_uint2(f32_to_f16_bits(v.x) | (f32_to_f16_bits(v.y) << 16),
                                                   f32_to_f16_bits(v.z) | (f32_to_f16_bits(v.w) << 16));
    } else {
        static_cast<uint2*>(p)[group] = make_uint2(f32_to_bf16_bits(v.x) | (f32_to_bf16_bits(v.y) << 16),
                                                   f32_to_bf16_bits(v.z) | (f32_to_bf16_bits(v.w) << 16));
    }
}

template <int DT>
__device__ __forceinline__ float4 rounded_sum(float4 x, float4 y) {
    return make_float4(round_storage(x.x + y.x, DT), round_storage(x.y + y.y, DT),
                       round_storage(x.z + y.z, DT), round_storage(x.w + y.w, DT));
}

// width % 4 == 0 and width <= 4 * kNormThreads * kNormCache
template <int DT, int kNormCache>
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_rows_kernel(
    const void* __restrict__ a, const void* __restrict__ b, const void* __restrict__ weight,
    void* __restrict__ residual, void* __restrict__ normed, uint32_t width, float eps) {
    __shared__ float partial[4];
    const uint32_t tid = threadIdx.x, groups = width >> 2;
    const size_t base = (size_t)blockIdx.x * groups;
    float4 x[kNormCache], w[kNormCache];
    float sum = 0.f;
#pragma unroll
    for (int s = 0; s < kNormCache; ++s) {
        const uint32_t g = tid + s * kNormThreads;
        if (g < groups) {
            x[s] = rounded_sum<DT>(load4<DT>(a, base + g), load4<DT>(b, base + g));
            w[s] = load4<DT>(weight, g);
        } else {
            x[s] = w[s] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
#pragma unroll
    for (int s = 0; s < kNormCache; ++s) {
        const uint32_t g = tid + s * kNormThreads;
        if (g < groups) store4<DT>(residual, base + g, x[s]);
        // the reference adds one element at a time into its running sum
        sum += x[s].x * x[s].x;
        sum += x[s].y * x[s].y;
        sum += x[s].z * x[s].z;
        sum += x[s].w * x[s].w;
    }
    sum = block_sum(sum, partial);
    const float inv = rsqrtf(sum / (float)width + eps);
#pragma unroll
    for (int s = 0; s < kNormCache; ++s) {
        const uint32_t g = tid + s * kNormThreads;
        if (g < groups)
            store4<DT>(normed, base + g,
                       make_float4(x[s].x * inv * w[s].x, x[s].y * inv * w[s].y, x[s].z * inv * w[s].z,
                                   x[s].w * inv * w[s].w));
    }
}

// any width: the element loop of the reference
template <int dtype>
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_any_kernel(
    const void* __restrict__ a, const void* __restrict__ b, const void* __restrict__ weight,
    void* __restrict__ residual, void* __restrict__ normed, uint32_t width, float eps) {
    __shared__ float partial[4];
    const uint32_t tid = threadIdx.x;
    const size_t base = (size_t)blockIdx.x * width;
    float sum = 0.f;
    for (uint32_t j = tid; j < width; j += kNormThreads) {
        const float x = round_storage(load_as_f32(a, base + j, dtype) + load_as_f32(b, base + j, dtype), dtype);
        store_from_f32(residual, base + j, dtype, x);
        sum += x * x;
    }
    sum = block_sum(sum, partial);
    const float inv = rsqrtf(sum / (float)width + eps);
    for (uint32_t j = tid; j < width; j += kNormThreads) {
        const float x = round_storage(load_as_f32(a, base + j, dtype) + load_as_f32(b, base + j, dtype), dtype);
        store_from_f32(normed, base + j, dtype, x * inv * load_as_f32(weight, j, dtype));
    }
}

template <int DT>
void launch_dtype(hipStream_t s, const void* a, const void* b, const void* weight, void* residual, void* normed,
                  uint32_t rows, uint32_t width, float eps) {
    const dim3 grid(rows), block(kNormThreads);
    const uint32_t per_thread = (width / 4 + kNormThreads - 1) / kNormThreads;
    if (width % 4 != 0 || per_thread > (uint32_t)kNormMaxCache) {
        hipLaunchKernelGGL(add_rmsnorm_any_kernel<DT>, grid, block, 0, s, a, b, weight, residual, normed, width, eps);
    } else if (per_thread <= 2) {
        hipLaunchKernelGGL((add_rmsnorm_rows_kernel<DT, 2>), grid, block, 0, s, a, b, weight, residual, normed, width, eps);
    } else if (per_thread <= 5) {
        hipLaunchKernelGGL((add_rmsnorm_rows_kernel<DT, 5>), grid, block, 0, s, a, b, weight, residual, normed, width, eps);
    } else if (per_thread <= 8) {
        hipLaunchKernelGGL((add_rmsnorm_rows_kernel<DT, 8>), grid, block, 0, s, a, b, weight, residual, normed, width, eps);
    } else {
        hipLaunchKernelGGL((add_rmsnorm_rows_kernel<DT, kNormMaxCache>), grid, block, 0, s, a, b, weight, residual,
                           normed, width, eps);
    }
}

}  // namespace

const char* launch_add_rmsnorm(hipStream_t s, const void* a, const void* b, const void* weight, void* residual,
                               void* normed, uint32_t rows, uint32_t width, uint32_t dtype, float eps) {
    if (dtype == FH_F32) {
        launch_dtype<0>(s, a, b, weight, residual, normed, rows, width, eps);
    } else if (dtype == FH_F16) {
        launch_dtype<1>(s, a, b, weight, residual, normed, rows, width, eps);
    } else {
        launch_dtype<2>(s, a, b, weight, residual, normed, rows, width, eps);
    }
    return "add_rmsnorm";
}

}  // namespace fh
