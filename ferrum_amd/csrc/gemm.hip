// Dequant-fused tile GEMM for GGUF Q4_K / Q6_K on gfx950:
// Y[M,N] = X[M,K] * W[N,K]^T, f16 or bf16 activations, f32 accumulation.
//
// Stands in for the reference's tile kernels q4_k_gemm_mpp / q6_k_gemm_mpp
// (src/metal/shaders/project_mpp.metal:474-729, 1098-1214) and, for F16
// activations, i_mm_q4_k / i_mm_q6_k (src/metal/shaders/diffusion.metal:230-291).
// As there, a K slab of the weight tile is decoded once per workgroup into LDS
// in the activation dtype (each value is the f32 dequantised weight rounded to
// nearest even) and fed to the matrix cores.
//
// Tile: 128 (M) x 128 (N) x 64 (K) per 256-thread workgroup; four waves in a
// 2 x 2 arrangement, each owning 64 x 64 outputs as 2 x 2 MFMA 32x32x16 tiles.
// LDS rows are padded to 72 halfs so 128-bit fragment reads are conflict free.
#include "device_utils.hpp"
#include "internal.hpp"

namespace fh {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLd = kBK + 8;  // halfs per LDS row
constexpr int kThreads = 256;

template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (DT == 1) {
        return f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
    } else {
        return f32_to_bf16_bits(a) | (f32_to_bf16_bits(b) << 16);
    }
}

// Raw bytes one thread needs to decode 32 weights (two runs of 16) of one row.
template <uint32_t TYPE>
struct RawW;

template <>
struct RawW<kQ4K> {
    uint4 hdr, qs;
    // chunk c (0..3) of the block, half h (0..1) of its 32 bytes
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c, uint32_t h) {
        hdr = *reinterpret_cast<const uint4*>(block);
        qs = *reinterpret_cast<const uint4*>(block + 16 + 32 * c + 16 * h);
    }
    // out_lo: 16 weights at k = 16h + i; out_hi: 16 weights at k = 32 + 16h + i
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t c, uint32_t (&out_lo)[8],
                                           uint32_t (&out_hi)[8]) const {
        float d = f16_bits_to_f32(hdr.x & 0xffffu);
        float dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc0, sc1, mn0, mn1;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, c, sc0, sc1, mn0, mn1);
        float a0 = d * sc0, b0 = dmin * mn0;
        float a1 = d * sc1, b1 = dmin * mn1;
        const uint32_t q[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t lo = q[t] & 0x0f0f0f0fu, hi = (q[t] >> 4) & 0x0f0f0f0fu;
            // a*q and b are exact in f32, so the fused form rounds once, like
            // the reference's (a*q) - b.
            float l0 = fmaf(a0, (float)(lo & 0xffu), -b0), l1 = fmaf(a0, (float)((lo >> 8) & 0xffu), -b0);
            float l2 = fmaf(a0, (float)((lo >> 16) & 0xffu), -b0), l3 = fmaf(a0, (float)(lo >> 24), -b0);
            float h0 = fmaf(a1, (float)(hi & 0xffu), -b1), h1 = fmaf(a1, (float)((hi >> 8) & 0xffu), -b1);
            float h2 = fmaf(a1, (float)((hi >> 16) & 0xffu), -b1), h3 = fmaf(a1, (float)(hi >> 24), -b1);
            out_lo[2 * t] = pack2<DT>(l0, l1);
            out_lo[2 * t + 1] = pack2<DT>(l2, l3);
            out_hi[2 * t] = pack2<DT>(h0, h1);
            out_hi[2 * t + 1] = pack2<DT>(h2, h3);
        }
    }
};

// Q6_K: the 64-wide K slab c (0..3) of a block, weights 64c .. 64c+63, is
// slices 2(c&1) and 2(c&1)+1 of half c>>1: the low nibbles (c even) or the
// high nibbles (c odd) of all 64 ql bytes of that half.  Thread half h covers
// 32 weights: slice 2(c&1)+h, positions 0..31.
template <>
struct RawW<kQ6K> {
    uint4 ql0, ql1, qh0, qh1;
    uint32_t tail;  // d | scale(l<16) << 16 | scale(l>=16) << 24

    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c, uint32_t h) {
        uint32_t half = c >> 1;
        const uint8_t* ql = block + 64 * half + 32 * h;      // slice&1 == h
        const uint8_t* qh = block + 128 + 32 * half;
        ql0 = load_u4_unaligned(ql);
        ql1 = load_u4_unaligned(ql + 16);
        qh0 = load_u4_unaligned(qh);
        qh1 = load_u4_unaligned(qh + 16);
        uint32_t slice = 2 * (c & 1u) + h;
        uint32_t si = 192 + 8 * half + 2 * slice;
        uint32_t d = load_u16_unaligned(block + 208);
        tail = d | ((uint32_t)block[si] << 16) | ((uint32_t)block[si + 1] << 24);
    }
    // out_lo: positions 0..15, out_hi: positions 16..31 of k = 32h + l
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t c, uint32_t (&out_lo)[8],
                                           uint32_t (&out_hi)[8], uint32_t h) const {
        float d = f16_bits_to_f32(tail & 0xffffu);
        float s_lo = d * (float)(int)(int8_t)(tail >> 16);
        float s_hi = d * (float)(int)(int8_t)(tail >> 24);
        uint32_t slice = 2 * (c & 1u) + h;
        uint32_t nib_shift = (c & 1u) * 4, plane_shift = 2 * slice;
        const uint32_t l[8] = {ql0.x, ql0.y, ql0.z, ql0.w, ql1.x, ql1.y, ql1.z, ql1.w};
        const uint32_t p[8] = {qh0.x, qh0.y, qh0.z, qh0.w, qh1.x, qh1.y, qh1.z, qh1.w};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            uint32_t q = ((l[t] >> nib_shift) & 0x0f0f0f0fu) | (((p[t] >> plane_shift) & 0x03030303u) << 4);
            float s = t < 4 ? s_lo : s_hi;
            float v0 = s * (float)((int)(q & 0xffu) - 32), v1 = s * (float)((int)((q >> 8) & 0xffu) - 32);
            float v2 = s * (float)((int)((q >> 16) & 0xffu) - 32), v3 = s * (float)((int)(q >> 24) - 32);
            uint32_t* out = t < 4 ? out_lo : out_hi;
            out[2 * (t & 3)] = pack2<DT>(v0, v1);
            out[2 * (t & 3) + 1] = pack2<DT>(v2, v3);
        }
    }
};

template <int DT>
__device__ __forceinline__ float16v mfma(uint4 a, uint4 b, float16v c) {
    if constexpr (DT == 1) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                      __builtin_bit_cast(half8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

template <uint32_t TYPE, int DT>
__global__ __launch_bounds__(kThreads) void gemm_tile_kernel(const uint8_t* __restrict__ w,
                                                             const uint16_t* __restrict__ x,
                                                             void* __restrict__ y, uint32_t m,
                                                             uint32_t n, uint32_t nb,
                                                             uint32_t y_dtype) {
    __shared__ __attribute__((aligned(16))) uint16_t xs[kBM * kLd];
    __shared__ __attribute__((aligned(16))) uint16_t ws[kBN * kLd];
    constexpr uint32_t kBlockBytes = TYPE == kQ4K ? 144 : 210;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n0 = blockIdx.x * kBN, m0 = blockIdx.y * kBM;
    const uint32_t k = nb << 8;

    // loader roles: one tile row per thread pair
    const uint32_t lrow = tid >> 1, lh = tid & 1u;
    const uint32_t wrow = n0 + lrow < n ? n0 + lrow : n - 1;
    const uint8_t* wsrc = w + (size_t)wrow * nb * kBlockBytes;
    const bool xlive = m0 + lrow < m;
    const uint16_t* xsrc = x + (size_t)(xlive ? m0 + lrow : 0) * k + 32 * lh;

    const uint32_t wm = (wave >> 1) * 64, wn = (wave & 1u) * 64;
    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const uint32_t steps = nb * 4;
    RawW<TYPE> raw;
    uint4 xr[4];
    raw.load(wsrc, 0, lh);
#pragma unroll
    for (int i = 0; i < 4; ++i)
        xr[i] = xlive ? reinterpret_cast<const uint4*>(xsrc)[i] : make_uint4(0, 0, 0, 0);

    for (uint32_t step = 0; step < steps; ++step) {
        const uint32_t c = step & 3u;
        uint32_t lo[8], hi[8];
        if constexpr (TYPE == kQ4K) {
            raw.template decode<DT>(c, lo, hi);
        } else {
            raw.template decode<DT>(c, lo, hi, lh);
        }
        __syncthreads();  // previous step's fragment reads are done
        {
            // Q4_K: lo -> k 16h.., hi -> k 32+16h..;  Q6_K: lo -> k 32h.., hi -> k 32h+16..
            uint32_t k_lo = TYPE == kQ4K ? 16 * lh : 32 * lh;
            uint32_t k_hi = TYPE == kQ4K ? 32 + 16 * lh : 32 * lh + 16;
            uint4* dst_lo = reinterpret_cast<uint4*>(&ws[lrow * kLd + k_lo]);
            uint4* dst_hi = reinterpret_cast<uint4*>(&ws[lrow * kLd + k_hi]);
            dst_lo[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            dst_lo[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
            dst_hi[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            dst_hi[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
            uint4* xdst = reinterpret_cast<uint4*>(&xs[lrow * kLd + 32 * lh]);
#pragma unroll
            for (int i = 0; i < 4; ++i) xdst[i] = xr[i];
        }
        if (step + 1 < steps) {
            uint32_t nstep = step + 1;
            raw.load(wsrc + (size_t)(nstep >> 2) * kBlockBytes, nstep & 3u, lh);
            const uint4* xp = reinterpret_cast<const uint4*>(xsrc + (size_t)nstep * kBK);
#pragma unroll
            for (int i = 0; i < 4; ++i) xr[i] = xlive ? xp[i] : make_uint4(0, 0, 0, 0);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            uint32_t koff = kk * 16 + 8 * (lane >> 5);
            uint4 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i] = *reinterpret_cast<const uint4*>(&xs[(wm + 32 * i + (lane & 31u)) * kLd + koff]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                b[j] = *reinterpret_cast<const uint4*>(&ws[(wn + 32 * j + (lane & 31u)) * kLd + koff]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = mfma<DT>(a[i], b[j], acc[i][j]);
        }
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t col = n0 + wn + 32 * j + (lane & 31u);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                uint32_t row = m0 + wm + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < m && col < n) store_from_f32(y, (size_t)row * n + col, y_dtype, acc[i][j][v]);
            }
        }
}

}  // namespace

const char* launch_gemm(hipStream_t s, const GemmArgs& a) {
    dim3 grid((a.n + kBN - 1) / kBN, (a.m + kBM - 1) / kBM);
    const uint32_t nb = a.k / 256;
    const uint8_t* w = static_cast<const uint8_t*>(a.w);
    const uint16_t* x = static_cast<const uint16_t*>(a.x);
    if (a.ggml_type == kQ4K) {
        if (a.x_dtype == FH_F16) {
            hipLaunchKernelGGL((gemm_tile_kernel<kQ4K, 1>), grid, dim3(kThreads), 0, s, w, x, a.y, a.m,
                               a.n, nb, a.y_dtype);
        } else {
            hipLaunchKernelGGL((gemm_tile_kernel<kQ4K, 2>), grid, dim3(kThreads), 0, s, w, x, a.y, a.m,
                               a.n, nb, a.y_dtype);
        }
        return "q4_k_gemm_mfma";
    }
    if (a.x_dtype == FH_F16) {
        hipLaunchKernelGGL((gemm_tile_kernel<kQ6K, 1>), grid, dim3(kThreads), 0, s, w, x, a.y, a.m, a.n,
                           nb, a.y_dtype);
    } else {
        hipLaunchKernelGGL((gemm_tile_kernel<kQ6K, 2>), grid, dim3(kThreads), 0, s, w, x, a.y, a.m, a.n,
                           nb, a.y_dtype);
    }
    return "q6_k_gemm_mfma";
}

}  // namespace fh
