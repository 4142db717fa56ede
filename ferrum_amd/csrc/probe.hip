// Measurement kernels: what the device does with no operator attached.
//
//  * read_probe: every lane loads 8 x 16 bytes that its wave covers contiguously and
//    xors them; nothing is written.  Its time over a buffer is what HBM delivers to a
//    kernel that does nothing with the bytes, the figure a streaming GEMV is read
//    against.
//  * mfma_probe: every wave issues `iterations` rounds of eight independent MFMA
//    chains on register operands and stores one float at the end.  Its rate is what the
//    matrix cores sustain for one instruction shape, the figure a tile GEMM is read
//    against.  With RANDOM set the operands are pseudo-random f16 values instead of small
//    integers: the matrix cores then draw more power and, with every compute unit
//    multiplying, the chip lowers its clock.
//  * coissue_probe: workgroups of eight waves, two per SIMD.  Waves 0..3 issue
//    v_mfma_f32_32x32x16_f16 (when `mfma` is set), waves 4..7 issue rounds of eight
//    independent v_fma_f32 (when `valu_rounds` is not zero).  Timed alone and
//    together, it shows whether matrix and vector arithmetic of two waves on one
//    SIMD overlap: what a kernel that decodes weights next to its multiplications
//    can hope for.
//
// None has a counterpart in the reference; all are launched by the benchmark only.
#include "internal.hpp"

namespace fh {
namespace {

// THREADS per workgroup, UNROLL 128-bit loads per lane (a wave's loads of one round are contiguous);
// DIRECT: the loads go to LDS (LDS-direct, no register written) instead of registers.
template <int THREADS, int UNROLL, bool DIRECT>
__global__ __launch_bounds__(THREADS) void read_probe(const uint4* __restrict__ p, size_t n16,
                                                      uint32_t* __restrict__ sink) {
    const size_t base = (size_t)blockIdx.x * THREADS * UNROLL + threadIdx.x;
    if constexpr (DIRECT) {
        // every wave has UNROLL KB of LDS of its own; lanes past the end re-read the last 16 bytes
        extern __shared__ __attribute__((aligned(16))) uint8_t probe_lds[];
        const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            const size_t idx = base + (size_t)i * THREADS;
            const uint4* src = p + (idx < n16 ? idx : n16 - 1);
            const uint32_t at = (wave * UNROLL + i) * 1024u;
            // M0 carries the LDS address of an LDS-direct load; nothing else in this kernel uses M0
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(at) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const uint32_t a = *reinterpret_cast<const uint32_t*>(probe_lds + threadIdx.x * 16u);
        if (a == 0x9e3779b9u && p[0].x == 0x12345678u) sink[0] = a;
    } else {
        uint4 v[UNROLL];
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            const size_t idx = base + (size_t)i * THREADS;
            v[i] = idx < n16 ? p[idx] : make_uint4(0, 0, 0, 0);
        }
        uint32_t a = 0;
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) a ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
        // the store keeps the loads alive; one lane in 2^32 takes it on random data, into scratch
        if (a == 0x9e3779b9u) sink[0] = a;
    }
}

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kChains = 8;

// SHAPE 0: v_mfma_f32_16x16x32_f16 (16384 flop), SHAPE 1: v_mfma_f32_32x32x16_f16 (32768 flop)
template <int SHAPE, bool RANDOM = false>
__global__ __launch_bounds__(256) void mfma_probe(uint32_t iterations, float seed, float* __restrict__ sink) {
    half8 a, b;
    if constexpr (RANDOM) {
        // sign and mantissa from a linear congruential sequence per lane, exponent 0.5 .. 2
        uint32_t h = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
        uint32_t w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            h = h * 1664525u + 1013904223u;
            w[i] = (h & 0x83ff83ffu) | (((h >> 10) & 1u) ? 0x3c003c00u : 0x38003800u);
        }
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        a = __builtin_bit_cast(half8, u32x4{w[0], w[1], w[2], w[3]});
        b = __builtin_bit_cast(half8, u32x4{w[4], w[5], w[6], w[7]});
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = (_Float16)(seed * (float)((threadIdx.x + i) & 7));
            b[i] = (_Float16)(seed * (float)((threadIdx.x * 3 + i) & 7));
        }
    }
    float total = 0.0f;
    if constexpr (SHAPE == 0) {
        float4v acc[kChains];
#pragma unroll
        for (int c = 0; c < kChains; ++c) acc[c] = float4v{0, 0, 0, 0};
        for (uint32_t it = 0; it < iterations; ++it) {
#pragma unroll
            for (int c = 0; c < kChains; ++c)
                acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < kChains; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
    } else {
        float16v acc[kChains];
#pragma unroll
        for (int c = 0; c < kChains; ++c)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[c][j] = 0.0f;
        for (uint32_t it = 0; it < iterations; ++it) {
#pragma unroll
            for (int c = 0; c < kChains; ++c)
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < kChains; ++c)
#pragma unroll
            for (int j = 0; j < 16; ++j) total += acc[c][j];
    }
    sink[blockIdx.x * 256 + threadIdx.x] = total;
}

__global__ __launch_bounds__(512) void coissue_probe(uint32_t iterations, uint32_t mfma, uint32_t valu_rounds,
                                                     float* __restrict__ sink) {
    const uint32_t wave = threadIdx.x >> 6;
    float total = 0.0f;
    if (wave < 4) {
        if (mfma == 0) return;
        half8 a, b;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = (_Float16)(0x1p-10f * (float)((threadIdx.x + i) & 7));
            b[i] = (_Float16)(0x1p-10f * (float)((threadIdx.x * 3 + i) & 7));
        }
        float16v acc[kChains];
#pragma unroll
        for (int c = 0; c < kChains; ++c)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[c][j] = 0.0f;
        for (uint32_t it = 0; it < iterations; ++it) {
#pragma unroll
            for (int c = 0; c < kChains; ++c)
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[c], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < kChains; ++c)
#pragma unroll
            for (int j = 0; j < 16; ++j) total += acc[c][j];
    } else {
        if (valu_rounds == 0) return;
        float x[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = 0x1p-10f * (float)(threadIdx.x + i);
        const float scale = 1.0001f, step = 0.5f;
        for (uint32_t it = 0; it < iterations; ++it)
            for (uint32_t r = 0; r < valu_rounds; ++r) {
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = __builtin_fmaf(x[i], scale, step);
            }
#pragma unroll
        for (int i = 0; i < 8; ++i) total += x[i];
    }
    sink[blockIdx.x * 512 + threadIdx.x] = total;
}

}  // namespace

const char* launch_coissue_probe(hipStream_t stream, uint32_t groups, uint32_t iterations, uint32_t mfma,
                                 uint32_t valu_rounds, float* sink) {
    coissue_probe<<<dim3(groups), dim3(512), 0, stream>>>(iterations, mfma, valu_rounds, sink);
    return mfma != 0 && valu_rounds != 0 ? "coissue_probe_mfma_and_valu" : mfma != 0 ? "coissue_probe_mfma" : "coissue_probe_valu";
}

template <int THREADS, int UNROLL, bool DIRECT>
void launch_read_form(hipStream_t stream, const void* data, size_t n16, uint32_t* sink) {
    const size_t per_group = (size_t)THREADS * UNROLL;
    const unsigned groups = (unsigned)((n16 + per_group - 1) / per_group);
    const size_t lds = DIRECT ? (size_t)(THREADS / 64) * UNROLL * 1024 : 0;
    read_probe<THREADS, UNROLL, DIRECT><<<dim3(groups), dim3(THREADS), lds, stream>>>(static_cast<const uint4*>(data), n16, sink);
}

// form = 100 x threads per workgroup + loads per lane, + 1000000 for LDS-direct loads; 0 = 256 threads x 8 loads
const char* launch_read_probe(hipStream_t stream, const void* data, size_t bytes, uint32_t* sink, int64_t form) {
    const size_t n16 = bytes / 16;
    switch (form) {
        case 25604: launch_read_form<256, 4, false>(stream, data, n16, sink); return "read_probe_256x4";
        case 25616: launch_read_form<256, 16, false>(stream, data, n16, sink); return "read_probe_256x16";
        case 51204: launch_read_form<512, 4, false>(stream, data, n16, sink); return "read_probe_512x4";
        case 51208: launch_read_form<512, 8, false>(stream, data, n16, sink); return "read_probe_512x8";
        case 102404: launch_read_form<1024, 4, false>(stream, data, n16, sink); return "read_probe_1024x4";
        case 102408: launch_read_form<1024, 8, false>(stream, data, n16, sink); return "read_probe_1024x8";
        case 1025608: launch_read_form<256, 8, true>(stream, data, n16, sink); return "read_probe_256x8_lds_direct";
        case 1025616: launch_read_form<256, 16, true>(stream, data, n16, sink); return "read_probe_256x16_lds_direct";
        case 1051208: launch_read_form<512, 8, true>(stream, data, n16, sink); return "read_probe_512x8_lds_direct";
        default: launch_read_form<256, 8, false>(stream, data, n16, sink); return "read_probe";
    }
}

const char* launch_mfma_probe(hipStream_t stream, int shape, uint32_t groups, uint32_t iterations,
                              float* sink, double* flops) {
    const double per = shape == 0 ? 2.0 * 16 * 16 * 32 : 2.0 * 32 * 32 * 16;
    *flops = per * kChains * (double)iterations * 4.0 * groups;
    if (shape == 0) {
        mfma_probe<0><<<dim3(groups), dim3(256), 0, stream>>>(iterations, 0x1p-10f, sink);
        return "mfma_probe_16x16x32_f16";
    }
    if (shape == 2) {
        mfma_probe<1, true><<<dim3(groups), dim3(256), 0, stream>>>(iterations, 0x1p-10f, sink);
        return "mfma_probe_32x32x16_f16_random_operands";
    }
    mfma_probe<1><<<dim3(groups), dim3(256), 0, stream>>>(iterations, 0x1p-10f, sink);
    return "mfma_probe_32x32x16_f16";
}

}  // namespace fh
