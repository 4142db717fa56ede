// Dequant-fused tile GEMM for GGUF Q4_K / Q5_K / Q6_K / IQ4_XS / Q8_0 on gfx950:
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
#include <type_traits>

#include "device_utils.hpp"
#include "tile_decode.hpp"
#include "internal.hpp"

namespace fh {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLd = kBK + 8;  // halfs per LDS row

template <int DT>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (DT == 1) {
        return f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
    } else {
        return f32_to_bf16_bits(a) | (f32_to_bf16_bits(b) << 16);
    }
}

// How a loader thread's half h (0..1) of a 64-weight K slab maps to K offsets:
// Q4_K / Q5_K decode 16 low-nibble weights at 16h and 16 high-nibble weights at
// 32 + 16h; Q6_K and IQ4_XS decode 32 consecutive weights at 32h.
template <uint32_t TYPE>
constexpr bool kNibblePlanes = TYPE == kQ4K || TYPE == kQ5K;
// a producer's task reads eight input dwords (one value per byte) instead of four (two nibbles per byte)
template <uint32_t TYPE>
constexpr bool kEightDwords = TYPE == kQ6K || TYPE == kQ8_0;
template <uint32_t TYPE>
__device__ __forceinline__ constexpr uint32_t k_lo_of(uint32_t h) { return kNibblePlanes<TYPE> ? 16 * h : 32 * h; }
template <uint32_t TYPE>
__device__ __forceinline__ constexpr uint32_t k_hi_of(uint32_t h) { return kNibblePlanes<TYPE> ? 32 + 16 * h : 32 * h + 16; }

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

// Q5_K: Q4_K's walk with the fifth bits: bit 2c (low nibbles) and 2c + 1 (high
// nibbles) of qh[l], l the position inside the chunk.
template <>
struct RawW<kQ5K> {
    uint4 hdr, qs, qh;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c, uint32_t h) {
        hdr = *reinterpret_cast<const uint4*>(block);
        qh = *reinterpret_cast<const uint4*>(block + 16 + 16 * h);
        qs = *reinterpret_cast<const uint4*>(block + 48 + 32 * c + 16 * h);
    }
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
        const uint32_t p[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t bits = p[t] >> (2 * c);
            uint32_t lo = (q[t] & 0x0f0f0f0fu) | ((bits & 0x01010101u) << 4);
            uint32_t hi = ((q[t] >> 4) & 0x0f0f0f0fu) | ((bits & 0x02020202u) << 3);
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

// IQ4_XS: K slab c is sub-blocks 2c and 2c + 1; thread half h decodes sub-block
// 2c + h from its 16 qs bytes: low nibbles are weights 0..15, high nibbles 16..31.
template <>
struct RawW<kIQ4XS> {
    uint2 hdr;
    uint4 qs;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c, uint32_t h) {
        hdr = *reinterpret_cast<const uint2*>(block);
        qs = load_u4_unaligned(block + 8 + 32 * c + 16 * h);
    }
    // out_lo: 16 weights at k = 32h + i; out_hi: 16 weights at k = 32h + 16 + i
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t c, uint32_t (&out_lo)[8], uint32_t (&out_hi)[8],
                                           uint32_t h) const {
        const float dl = iq4xs_scale(hdr.x, hdr.y, 2 * c + h);
        const float scale = dl * 16777216.f, offset = -128.f * dl;
        const uint32_t q[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t l = iq4_lookup4(q[t]), u = iq4_lookup4(q[t] >> 4);
            const uint32_t l01 = bytes01_as_halves(l), l23 = bytes23_as_halves(l);
            const uint32_t u01 = bytes01_as_halves(u), u23 = bytes23_as_halves(u);
            out_lo[2 * t] = fma_pair<DT>(lo_half(l01), hi_half(l01), scale, offset);
            out_lo[2 * t + 1] = fma_pair<DT>(lo_half(l23), hi_half(l23), scale, offset);
            out_hi[2 * t] = fma_pair<DT>(lo_half(u01), hi_half(u01), scale, offset);
            out_hi[2 * t + 1] = fma_pair<DT>(lo_half(u23), hi_half(u23), scale, offset);
        }
    }
};

// Q8_0: K slab c is blocks 2c and 2c + 1 of the 256-weight run; thread half h decodes
// block 2c + h: 34 bytes at 34 (2c + h), two-byte aligned.
template <>
struct RawW<kQ8_0> {
    uint4 qa, qb;
    uint32_t dh;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c, uint32_t h) {
        const uint8_t* b = block + 34 * (2 * c + h);
        dh = load_u16_unaligned(b);
        qa = load_u4_unaligned(b + 2);
        qb = load_u4_unaligned(b + 18);
    }
    // out_lo: 16 weights at k = 32h + i; out_hi: 16 weights at k = 32h + 16 + i
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t, uint32_t (&out_lo)[8], uint32_t (&out_hi)[8], uint32_t) const {
        const float d = f16_bits_to_f32(dh);
        const float scale = d * 16777216.f, offset = -128.f * d;
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t u = q[t] ^ 0x80808080u;
            const uint32_t u01 = bytes01_as_halves(u), u23 = bytes23_as_halves(u);
            uint32_t* out = t < 4 ? out_lo : out_hi;
            out[2 * (t & 3)] = fma_pair<DT>(lo_half(u01), hi_half(u01), scale, offset);
            out[2 * (t & 3) + 1] = fma_pair<DT>(lo_half(u23), hi_half(u23), scale, offset);
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

// TS = 128: four waves, 64 x 64 each; TS = 64: two waves, 32 x 64 each (four times the
// workgroups, for matrices too small to fill the chip with 128 x 128 tiles); TS = 32: one
// wave and one 32 x 32 tile, when even 64 x 64 tiles number fewer than the compute units.
template <uint32_t TYPE, int DT, int TS>
__global__ __launch_bounds__(2 * TS) void gemm_tile_kernel(const uint8_t* __restrict__ w,
                                                             const uint16_t* __restrict__ x,
                                                             void* __restrict__ y, uint32_t m,
                                                             uint32_t n, uint32_t nb,
                                                             uint32_t y_dtype) {
    constexpr int WI = TS == 128 ? 2 : 1;  // 32-row tiles per wave
    constexpr int WJ = TS == 32 ? 1 : 2;   // 32-column tiles per wave
    __shared__ __attribute__((aligned(16))) uint16_t xs[TS * kLd];
    __shared__ __attribute__((aligned(16))) uint16_t ws[TS * kLd];
    constexpr uint32_t kBlockBytes = block_bytes_of(TYPE);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n0 = blockIdx.x * TS, m0 = blockIdx.y * TS;
    const uint32_t k = nb << 8;

    // loader roles: one tile row per thread pair
    const uint32_t lrow = tid >> 1, lh = tid & 1u;
    const uint32_t wrow = n0 + lrow < n ? n0 + lrow : n - 1;
    const uint8_t* wsrc = w + (size_t)wrow * nb * kBlockBytes;
    const bool xlive = m0 + lrow < m;
    const uint16_t* xsrc = x + (size_t)(xlive ? m0 + lrow : 0) * k + 32 * lh;

    const uint32_t wm = TS == 128 ? (wave >> 1) * 64 : TS == 64 ? wave * 32 : 0, wn = TS == 128 ? (wave & 1u) * 64 : 0;
    float16v acc[WI][WJ];
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
        for (int j = 0; j < WJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // One register stage per K slab of a super-block: the loads of a slab are issued a whole
    // block (four slabs) before it is decoded, so a memory round trip is spread over four steps.
    RawW<TYPE> raw[4];
    uint4 xr[4][4];
    auto fetch = [&](int c, uint32_t block) {
        raw[c].load(wsrc + (size_t)block * kBlockBytes, (uint32_t)c, lh);
        const uint4* xp = reinterpret_cast<const uint4*>(xsrc + ((size_t)block * 4 + c) * kBK);
#pragma unroll
        for (int i = 0; i < 4; ++i) xr[c][i] = xlive ? xp[i] : make_uint4(0, 0, 0, 0);
    };
#pragma unroll
    for (int c = 0; c < 4; ++c) fetch(c, 0);

    for (uint32_t block = 0; block < nb; ++block) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t lo[8], hi[8];
            if constexpr (kNibblePlanes<TYPE>) {
                raw[c].template decode<DT>((uint32_t)c, lo, hi);
            } else {
                raw[c].template decode<DT>((uint32_t)c, lo, hi, lh);
            }
            __syncthreads();  // previous step's fragment reads are done
            {
                const uint32_t k_lo = k_lo_of<TYPE>(lh), k_hi = k_hi_of<TYPE>(lh);
                uint4* dst_lo = reinterpret_cast<uint4*>(&ws[lrow * kLd + k_lo]);
                uint4* dst_hi = reinterpret_cast<uint4*>(&ws[lrow * kLd + k_hi]);
                dst_lo[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                dst_lo[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
                dst_hi[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                dst_hi[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
                uint4* xdst = reinterpret_cast<uint4*>(&xs[lrow * kLd + 32 * lh]);
#pragma unroll
                for (int i = 0; i < 4; ++i) xdst[i] = xr[c][i];
            }
            if (block + 1 < nb) fetch(c, block + 1);
            __syncthreads();
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                uint32_t koff = kk * 16 + 8 * (lane >> 5);
                uint4 a[WI], b[WJ];
#pragma unroll
                for (int i = 0; i < WI; ++i)
                    a[i] = *reinterpret_cast<const uint4*>(&xs[(wm + 32 * i + (lane & 31u)) * kLd + koff]);
#pragma unroll
                for (int j = 0; j < WJ; ++j)
                    b[j] = *reinterpret_cast<const uint4*>(&ws[(wn + 32 * j + (lane & 31u)) * kLd + koff]);
#pragma unroll
                for (int i = 0; i < WI; ++i)
#pragma unroll
                    for (int j = 0; j < WJ; ++j) acc[i][j] = mfma<DT>(a[i], b[j], acc[i][j]);
            }
        }
    }

#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
        for (int j = 0; j < WJ; ++j) {
            uint32_t col = n0 + wn + 32 * j + (lane & 31u);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                uint32_t row = m0 + wm + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < m && col < n) store_from_f32(y, (size_t)row * n + col, y_dtype, acc[i][j][v]);
            }
        }
}


// ---- wide tile: 256 (M) x 16*NT (N) x 64 (K) ---------------------------------------
//
// For prefill-sized M.  One workgroup owns `cols` (<= 16*NT) output columns and
// 256 rows, so the grid can be sized to the chip (e.g. 17408 columns = 128
// tiles of 136, times two M tiles = 256 workgroups on 256 CUs) and every
// weight is decoded once per 256 rows.  Eight waves: four consumers, each 64
// rows x 16*NT columns as 4 x NT MFMA 16x16x32 tiles with their activation
// fragments loaded straight from global memory, and four producers that
// decode the weight slab into LDS.  A SIMD therefore
// holds one wave issuing MFMAs and one issuing VALU / memory work, which the
// hardware overlaps.  LDS is double buffered: while slab s feeds the matrix
// cores, slab s+1 is decoded into the other buffer and the global loads of
// slabs s+2 and s+3 are in flight; one barrier per slab.
//
// Workgroup ids are mapped so that the M tiles of one weight tile sit on the
// same XCD (ids that are equal mod 8) and share it through that XCD's L2.
constexpr int kWM = 256;

template <uint32_t TYPE, int DT>
__device__ __forceinline__ void decode_to_lds(const RawW<TYPE>& raw, uint32_t c, uint32_t h,
                                              uint16_t* wrow_lds) {
    uint32_t lo[8], hi[8];
    if constexpr (kNibblePlanes<TYPE>) {
        raw.template decode<DT>(c, lo, hi);
    } else {
        raw.template decode<DT>(c, lo, hi, h);
    }
    const uint32_t k_lo = k_lo_of<TYPE>(h), k_hi = k_hi_of<TYPE>(h);
    uint4* dst_lo = reinterpret_cast<uint4*>(wrow_lds + k_lo);
    uint4* dst_hi = reinterpret_cast<uint4*>(wrow_lds + k_hi);
    dst_lo[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    dst_lo[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
    dst_hi[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    dst_hi[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
}


// Raw bytes one producer thread needs from a whole super-block: its half h of
// each of the four 64-weight K slabs.  Loading by block (not by slab) issues
// the global loads four slabs or more ahead of their use.  decode() turns one
// input dword (4 quant bytes) of slab c into tile values: Q4_K gives two
// dwords for k = 16h + 4t .. (low nibbles) and two for k = 32 + 16h + 4t ..
// (high nibbles); Q6_K gives two dwords for k = 32h + 4t ...
// component t of a register quad; t may differ between lanes (two selects), and folds away
// when it is a constant
__device__ __forceinline__ uint32_t pick4(const uint4& q, int t) {
    const uint32_t lo = (t & 1) ? q.y : q.x, hi = (t & 1) ? q.w : q.z;
    return (t & 2) ? hi : lo;
}

template <uint32_t TYPE>
struct BlockW;

template <>
struct BlockW<kQ4K> {
    uint4 hdr, q[4];
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t h) {
        hdr = *reinterpret_cast<const uint4*>(block);
#pragma unroll
        for (int c = 0; c < 4; ++c) q[c] = *reinterpret_cast<const uint4*>(block + 16 + 32 * c + 16 * h);
    }
    struct Scales {
        float a_lo, a_hi, b_lo, b_hi;
    };
    __device__ __forceinline__ Scales scales(int c, uint32_t) const {
        float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc0, sc1, mn0, mn1;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, (uint32_t)c, sc0, sc1, mn0, mn1);
        // d*sc and dmin*m are exact in f32; the powers of two undo the subnormal encoding
        return {(d * sc0) * 16777216.f, (d * sc1) * 1048576.f, -(dmin * mn0), -(dmin * mn1)};
    }
    __device__ __forceinline__ uint32_t dword(int c, int t) const { return pick4(q[c], t); }
    // out[0..1]: low-nibble pair dwords, out[2..3]: high-nibble pair dwords
    template <int DT>
    __device__ __forceinline__ void decode(int c, uint32_t, int t, const Scales& s, uint32_t (&out)[4]) const {
        const uint32_t w0 = dword(c, t), w1 = w0 >> 8;
        const uint32_t l02 = w0 & 0x000f000fu, h02 = w0 & 0x00f000f0u;
        const uint32_t l13 = w1 & 0x000f000fu, h13 = w1 & 0x00f000f0u;
        out[0] = fma_pair<DT>(lo_half(l02), lo_half(l13), s.a_lo, s.b_lo);
        out[1] = fma_pair<DT>(hi_half(l02), hi_half(l13), s.a_lo, s.b_lo);
        out[2] = fma_pair<DT>(lo_half(h02), lo_half(h13), s.a_hi, s.b_hi);
        out[3] = fma_pair<DT>(hi_half(h02), hi_half(h13), s.a_hi, s.b_hi);
    }
};

template <>
struct BlockW<kQ5K> {
    uint4 hdr, qh, q[4];
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t h) {
        hdr = *reinterpret_cast<const uint4*>(block);
        qh = *reinterpret_cast<const uint4*>(block + 16 + 16 * h);
#pragma unroll
        for (int c = 0; c < 4; ++c) q[c] = *reinterpret_cast<const uint4*>(block + 48 + 32 * c + 16 * h);
    }
    using Scales = BlockW<kQ4K>::Scales;
    __device__ __forceinline__ Scales scales(int c, uint32_t) const {
        float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc0, sc1, mn0, mn1;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, (uint32_t)c, sc0, sc1, mn0, mn1);
        return {(d * sc0) * 16777216.f, (d * sc1) * 1048576.f, -(dmin * mn0), -(dmin * mn1)};
    }
    // low nibble | fifth bit << 4 reads as q * 2^-24; high nibble in place | fifth bit << 8 as 16q * 2^-24
    template <int DT>
    __device__ __forceinline__ void decode(int c, uint32_t, int t, const Scales& s, uint32_t (&out)[4]) const {
        const uint32_t w0 = pick4(q[c], t), w1 = w0 >> 8;
        const uint32_t p0 = pick4(qh, t) >> (2 * c), p1 = p0 >> 8;
        const uint32_t l02 = (w0 & 0x000f000fu) | ((p0 & 0x00010001u) << 4);
        const uint32_t l13 = (w1 & 0x000f000fu) | ((p1 & 0x00010001u) << 4);
        const uint32_t h02 = (w0 & 0x00f000f0u) | ((p0 & 0x00020002u) << 7);
        const uint32_t h13 = (w1 & 0x00f000f0u) | ((p1 & 0x00020002u) << 7);
        out[0] = fma_pair<DT>(lo_half(l02), lo_half(l13), s.a_lo, s.b_lo);
        out[1] = fma_pair<DT>(hi_half(l02), hi_half(l13), s.a_lo, s.b_lo);
        out[2] = fma_pair<DT>(lo_half(h02), lo_half(h13), s.a_hi, s.b_hi);
        out[3] = fma_pair<DT>(hi_half(h02), hi_half(h13), s.a_hi, s.b_hi);
    }
};

// IQ4_XS: half h of slab c is sub-block 2c + h; input dword t gives the pair dwords of its
// weights 4t .. 4t + 3 (low nibbles, out[0..1]) and 16 + 4t .. (high nibbles, out[2..3]).
template <>
struct BlockW<kIQ4XS> {
    uint2 hdr;
    uint4 q[4];
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t h) {
        hdr = *reinterpret_cast<const uint2*>(block);
#pragma unroll
        for (int c = 0; c < 4; ++c) q[c] = load_u4_unaligned(block + 8 + 32 * c + 16 * h);
    }
    using Scales = BlockW<kQ4K>::Scales;
    __device__ __forceinline__ Scales scales(int c, uint32_t h) const {
        const float dl = iq4xs_scale(hdr.x, hdr.y, 2u * (uint32_t)c + h);
        return {dl * 16777216.f, dl * 16777216.f, -128.f * dl, -128.f * dl};
    }
    template <int DT>
    __device__ __forceinline__ void decode(int c, uint32_t, int t, const Scales& s, uint32_t (&out)[4]) const {
        const uint32_t v = pick4(q[c], t);
        const uint32_t l = iq4_lookup4(v), u = iq4_lookup4(v >> 4);
        const uint32_t l01 = bytes01_as_halves(l), l23 = bytes23_as_halves(l);
        const uint32_t u01 = bytes01_as_halves(u), u23 = bytes23_as_halves(u);
        out[0] = fma_pair<DT>(lo_half(l01), hi_half(l01), s.a_lo, s.b_lo);
        out[1] = fma_pair<DT>(lo_half(l23), hi_half(l23), s.a_lo, s.b_lo);
        out[2] = fma_pair<DT>(lo_half(u01), hi_half(u01), s.a_hi, s.b_hi);
        out[3] = fma_pair<DT>(lo_half(u23), hi_half(u23), s.a_hi, s.b_hi);
    }
};

// Q8_0: half h of slab c is block 2c + h; input dword t (0..7) gives the pair dwords of its
// weights 4t .. 4t + 3.
template <>
struct BlockW<kQ8_0> {
    uint4 q[4][2];
    uint32_t dh[4];
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t h) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint8_t* b = block + 34 * (2 * c + h);
            dh[c] = load_u16_unaligned(b);
            q[c][0] = load_u4_unaligned(b + 2);
            q[c][1] = load_u4_unaligned(b + 18);
        }
    }
    struct Scales {
        float scale, offset;
    };
    __device__ __forceinline__ Scales scales(int c, uint32_t) const {
        const float d = f16_bits_to_f32(dh[c]);
        return {d * 16777216.f, -128.f * d};
    }
    template <int DT>
    __device__ __forceinline__ void decode(int c, uint32_t, int t, const Scales& s, uint32_t (&out)[4]) const {
        const uint32_t v[8] = {q[c][0].x, q[c][0].y, q[c][0].z, q[c][0].w, q[c][1].x, q[c][1].y, q[c][1].z, q[c][1].w};
        const uint32_t u = v[t] ^ 0x80808080u;
        const uint32_t u01 = bytes01_as_halves(u), u23 = bytes23_as_halves(u);
        out[0] = fma_pair<DT>(lo_half(u01), hi_half(u01), s.scale, s.offset);
        out[1] = fma_pair<DT>(lo_half(u23), hi_half(u23), s.scale, s.offset);
        out[2] = 0;
        out[3] = 0;
    }
};

template <>
struct BlockW<kQ6K> {
    uint4 l[2][2], p[2][2], sc;  // ql / qh of both halves, the 16 scales
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t h) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            l[half][0] = load_u4_unaligned(block + 64 * half + 32 * h);
            l[half][1] = load_u4_unaligned(block + 64 * half + 32 * h + 16);
            p[half][0] = load_u4_unaligned(block + 128 + 32 * half);
            p[half][1] = load_u4_unaligned(block + 128 + 32 * half + 16);
        }
        sc = load_u4_unaligned(block + 192);
        d = load_u16_unaligned(block + 208);
    }
    struct Scales {
        float s[2], off[2];   // scale (with the power of two) and -32*scale of positions 0..15 / 16..31
        uint32_t plane_shift;
    };
    __device__ __forceinline__ Scales scales(int c, uint32_t h) const {
        const int half = c >> 1;
        // scales 8*half + 2*slice (+1), slice = 2(c&1) + h: a 16-bit pair of word 2*half + (c&1)
        const uint32_t words[4] = {sc.x, sc.y, sc.z, sc.w};
        const uint32_t pair = words[2 * half + (c & 1)] >> (16 * h);
        const float df = f16_bits_to_f32(d);
        const float s0 = df * (float)(int)(int8_t)pair, s1 = df * (float)(int)(int8_t)(pair >> 8);
        const float pow2 = (c & 1) ? 1048576.f : 16777216.f;  // high nibbles sit four bits up
        return {{s0 * pow2, s1 * pow2}, {-32.f * s0, -32.f * s1}, 2u * (2u * (c & 1) + h)};
    }
    // out[0..1]: the two pair dwords of positions 4t .. 4t+3
    template <int DT>
    __device__ __forceinline__ void decode(int c, uint32_t, int t, const Scales& s, uint32_t (&out)[4]) const {
        const int half = c >> 1;
        const uint32_t lw[8] = {l[half][0].x, l[half][0].y, l[half][0].z, l[half][0].w,
                                l[half][1].x, l[half][1].y, l[half][1].z, l[half][1].w};
        const uint32_t pw[8] = {p[half][0].x, p[half][0].y, p[half][0].z, p[half][0].w,
                                p[half][1].x, p[half][1].y, p[half][1].z, p[half][1].w};
        const uint32_t w0 = lw[t], w1 = w0 >> 8;
        const uint32_t p0 = pw[t] >> s.plane_shift, p1 = p0 >> 8;
        uint32_t q02, q13;
        if ((c & 1) == 0) {   // low nibbles | plane bits << 4 : q * 2^-24
            q02 = (w0 & 0x000f000fu) | ((p0 & 0x00030003u) << 4);
            q13 = (w1 & 0x000f000fu) | ((p1 & 0x00030003u) << 4);
        } else {              // high nibbles in place | plane bits << 8 : 16q * 2^-24
            q02 = (w0 & 0x00f000f0u) | ((p0 & 0x00030003u) << 8);
            q13 = (w1 & 0x00f000f0u) | ((p1 & 0x00030003u) << 8);
        }
        const float sv = s.s[t >> 2], ov = s.off[t >> 2];
        out[0] = fma_pair<DT>(lo_half(q02), lo_half(q13), sv, ov);
        out[1] = fma_pair<DT>(hi_half(q02), hi_half(q13), sv, ov);
        out[2] = 0;
        out[3] = 0;
    }
};

// Decode one (slab c, half h) task of a row into its LDS row.
template <uint32_t TYPE, int DT>
__device__ __forceinline__ void decode_block_slab(const BlockW<TYPE>& blk, int c, uint32_t h,
                                                  uint16_t* wrow_lds) {
    const auto s = blk.scales(c, h);
    if constexpr (!kEightDwords<TYPE>) {
        uint32_t lo[8], hi[8];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t out[4];
            blk.template decode<DT>(c, h, t, s, out);
            lo[2 * t] = out[0];
            lo[2 * t + 1] = out[1];
            hi[2 * t] = out[2];
            hi[2 * t + 1] = out[3];
        }
        uint4* dst_lo = reinterpret_cast<uint4*>(wrow_lds + k_lo_of<TYPE>(h));
        uint4* dst_hi = reinterpret_cast<uint4*>(wrow_lds + k_hi_of<TYPE>(h));
        dst_lo[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        dst_lo[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        dst_hi[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        dst_hi[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
    } else {
        uint32_t v[16];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            uint32_t out[4];
            blk.template decode<DT>(c, h, t, s, out);
            v[2 * t] = out[0];
            v[2 * t + 1] = out[1];
        }
        uint4* dst = reinterpret_cast<uint4*>(wrow_lds + 32 * h);           // k = 32h ..
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = make_uint4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
    }
}

// A quarter of a task: input dword t of Q4_K, or dwords t and t + 4 of Q6_K.
template <uint32_t TYPE, int DT>
__device__ __forceinline__ void decode_block_piece(const BlockW<TYPE>& blk, int c, uint32_t h, int t,
                                                   uint16_t* wrow_lds) {
    const auto s = blk.scales(c, h);
    if constexpr (!kEightDwords<TYPE>) {
        uint32_t out[4];
        blk.template decode<DT>(c, h, t, s, out);   // the dword is selected, the arithmetic runs once
        *reinterpret_cast<uint2*>(wrow_lds + k_lo_of<TYPE>(h) + 4 * t) = make_uint2(out[0], out[1]);
        *reinterpret_cast<uint2*>(wrow_lds + k_hi_of<TYPE>(h) + 4 * t) = make_uint2(out[2], out[3]);
    } else {
        uint32_t a[4] = {0, 0, 0, 0}, b[4] = {0, 0, 0, 0};
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
            if (tt == t) {
                blk.template decode<DT>(c, h, tt, s, a);
                blk.template decode<DT>(c, h, tt + 4, s, b);
            }
        *reinterpret_cast<uint2*>(wrow_lds + 32 * h + 4 * t) = make_uint2(a[0], a[1]);
        *reinterpret_cast<uint2*>(wrow_lds + 32 * h + 16 + 4 * t) = make_uint2(b[0], b[1]);
    }
}

// Waves that multiply: each owns 16 * kWideRowTiles rows of the 256-row tile; four more waves decode.
constexpr int kWideConsumers = 4;   // eight (two multiplying waves per SIMD) measured the same at M = 512 and slower for the heavier decoders
constexpr int kWideRowTiles = 16 / kWideConsumers;
constexpr int kWideThreads = (kWideConsumers + 4) * 64;

template <uint32_t TYPE, int DT, int NT>
__global__ __launch_bounds__(kWideThreads) void gemm_wide_kernel(const uint8_t* __restrict__ w,
                                                                 const uint16_t* __restrict__ x,
                                                                 void* __restrict__ y, uint32_t m,
                                                                 uint32_t n, uint32_t nb,
                                                                 uint32_t y_dtype, uint32_t cols,
                                                                 uint32_t tiles_m, uint32_t tiles_n) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    constexpr uint32_t kBlockBytes = block_bytes_of(TYPE);
    constexpr uint32_t kRowsW = 16 * NT;
    constexpr uint32_t kStage = kRowsW * kLd;  // halfs per buffer
    constexpr bool kExtra = NT > 8;                    // rows 128.. need a second decode task

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    // XCD-aware tile order: ids r, r+8, r+16, .. of a group share the XCD (id mod 8)
    uint32_t tile_m, tile_n;
    {
        const uint32_t group_ids = 8 * tiles_m, id = blockIdx.x;
        const uint32_t g = id / group_ids, r = id % group_ids;
        tile_n = g * 8 + (r & 7u);
        tile_m = r >> 3;
        if (tile_n >= tiles_n) return;
    }
    const uint32_t n0 = tile_n * cols, m0 = tile_m * kWM;
    const uint32_t ncols = n - n0 < cols ? n - n0 : cols;
    const uint32_t k = nb << 8;
    const uint32_t steps = nb * 4;

    if (wave >= kWideConsumers) {
        // ---- producers: global -> registers -> (decode) -> LDS, two slabs ahead ----
        const uint32_t pt = tid - kWideConsumers * 64, pw = wave - kWideConsumers;
        const uint32_t wr = pt >> 1, wh = pt & 1u;
        const uint8_t* wsrc = w + (size_t)(n0 + (wr < ncols ? wr : ncols - 1)) * nb * kBlockBytes;
        // rows 128.. of a 136-column tile: 8 rows x 2 halves x 4 quarter pieces, one per lane
        const uint32_t er = 128 + (lane >> 3), eh = (lane >> 2) & 1u, et = lane & 3u;
        const uint8_t* esrc = w + (size_t)(n0 + (er < ncols ? er : ncols - 1)) * nb * kBlockBytes;
        // register sets: the block being decoded and the next one or two in flight
        constexpr bool kDeep = !kEightDwords<TYPE>;   // Q6_K and Q8_0 sets are twice as large: one block ahead
        BlockW<TYPE> cur, n1, n2, ecur, en1, en2;
        auto load_block = [&](BlockW<TYPE>& main, BlockW<TYPE>& extra, uint32_t b) {
            main.load(wsrc + (size_t)b * kBlockBytes, wh);
            if (kExtra) extra.load(esrc + (size_t)b * kBlockBytes, eh);
        };
        auto store_slab = [&](int c) {
            uint16_t* ws = lds + (c & 1) * kStage;
            decode_block_slab<TYPE, DT>(cur, c, wh, ws + wr * kLd);
            if (kExtra && pw == (uint32_t)c && er < ncols)
                decode_block_piece<TYPE, DT>(ecur, c, eh, (int)et, ws + er * kLd);
        };
        load_block(cur, ecur, 0);
        if (nb > 1) load_block(n1, en1, 1);
        if (kDeep && nb > 2) load_block(n2, en2, 2);
        store_slab(0);
        for (uint32_t b = 0; b < nb; ++b) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                __syncthreads();  // slab 4b + c is visible; the other buffer is free
                if (c < 3) {
                    store_slab(c + 1);
                } else if (b + 1 < nb) {
                    cur = n1;
                    ecur = en1;
                    if (kDeep) {
                        n1 = n2;
                        en1 = en2;
                        if (b + 3 < nb) load_block(n2, en2, b + 3);
                    } else if (b + 2 < nb) {
                        load_block(n1, en1, b + 2);
                    }
                    store_slab(0);
                }
            }
        }
        return;
    }

    // ---- consumers: LDS fragments -> MFMA ----
    float4v acc[kWideRowTiles][NT];
#pragma unroll
    for (int i = 0; i < kWideRowTiles; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

    // A fragments come straight from global memory (the activation tile is
    // L2 resident and each wave owns its 64 rows): lane (row = lane & 15,
    // g = lane >> 4) holds k = 8g .. 8g+7 of a 32-wide K half.  They run
    // through a ring of three register sets, loaded two K halves ahead.
    const uint32_t g = lane >> 4;
    // rows past m are clamped: they only feed outputs that are never stored
    const uint16_t* asrc[kWideRowTiles];
#pragma unroll
    for (int i = 0; i < kWideRowTiles; ++i) {
        uint32_t row = m0 + wave * (16 * kWideRowTiles) + 16 * i + (lane & 15u);
        asrc[i] = x + (size_t)(row < m ? row : m - 1) * k + 8 * g;
    }
    auto load_a = [&](uint4 (&a)[kWideRowTiles], uint32_t u) {
#pragma unroll
        for (int i = 0; i < kWideRowTiles; ++i) a[i] = *reinterpret_cast<const uint4*>(asrc[i] + (size_t)u * 32);
    };
    const uint32_t frag_off = (lane & 15u) * kLd + 8 * g;
    auto mma_half = [&](const uint4 (&a)[kWideRowTiles], uint32_t u) {
        const uint16_t* ws = lds + ((u >> 1) & 1u) * kStage + frag_off + (u & 1u) * 32;
        // B fragments through a ring of four so three LDS reads stay in flight
        uint4 b[4];
#pragma unroll
        for (int j = 0; j < 3; ++j) b[j] = *reinterpret_cast<const uint4*>(ws + 16 * j * kLd);
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            if (j + 3 < NT) b[(j + 3) % 4] = *reinterpret_cast<const uint4*>(ws + 16 * (j + 3) * kLd);
#pragma unroll
            for (int i = 0; i < kWideRowTiles; ++i) acc[i][j] = mfma16<DT>(a[i], b[j % 4], acc[i][j]);
        }
        // issue order for the scheduler (0x100 = DS read, 0x008 = MFMA)
        __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
#pragma unroll
        for (int j = 0; j < NT - 3; ++j) {
            __builtin_amdgcn_sched_group_barrier(0x008, kWideRowTiles, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 3 * kWideRowTiles, 0);
    };
    const uint32_t halves = steps * 2;
    constexpr int kRing = 4;               // A register sets: loads run kRing - 1 halves ahead
    static_assert(kRing % 2 == 0, "the slab barrier falls on even halves of the ring");
    uint4 a[kRing][kWideRowTiles];
#pragma unroll
    for (int i = 0; i < kRing - 1; ++i)
        if ((uint32_t)i < halves) load_a(a[i], i);
    __builtin_amdgcn_s_setprio(2);  // the MFMA wave goes first when both waves of a SIMD can issue
    // Main loop: kRing K halves of straight-line code, so the outstanding-load
    // counts are exact and the A loads stay ahead; the last halves run through
    // a guarded tail.
    uint32_t u = 0;
    for (; u + 2 * kRing - 1 <= halves; u += kRing) {
#pragma unroll
        for (int ph = 0; ph < kRing; ++ph) {
            if ((ph & 1) == 0) __syncthreads();  // a new slab
            load_a(a[(ph + kRing - 1) % kRing], u + ph + kRing - 1);
            mma_half(a[ph], u + ph);
        }
    }
    for (; u < halves; u += kRing) {
#pragma unroll
        for (int ph = 0; ph < kRing; ++ph) {
            const uint32_t uu = u + ph;
            if (uu < halves) {
                if ((uu & 1u) == 0) __syncthreads();  // a new slab
                if (uu + kRing - 1 < halves) load_a(a[(ph + kRing - 1) % kRing], uu + kRing - 1);
                mma_half(a[ph], uu);
            }
        }
    }
    __builtin_amdgcn_s_setprio(0);

#pragma unroll
    for (int i = 0; i < kWideRowTiles; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const uint32_t lc = 16 * j + (lane & 15u);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t row = m0 + wave * (16 * kWideRowTiles) + 16 * i + 4 * (lane >> 4) + v;
                if (row < m && lc < ncols)
                    store_from_f32(y, (size_t)row * n + n0 + lc, y_dtype, acc[i][j][v]);
            }
        }
}

// ---- the 256-row tile on the 32x32x16 matrix instruction --------------------------------
// Same division of labour as gemm_wide_kernel (four waves decode weight rows into a double
// buffered LDS slab of 64 K, four waves multiply, each owning 64 of the tile's 256 activation
// rows), but the multiplying waves issue v_mfma_f32_32x32x16, which does twice the work per
// issue slot of the 16x16x32 form.  A wave's tile is 2 x NT blocks of 32 x 32 (NT = 4 or 5:
// 128 or 160 weight rows per workgroup).  Within a slab lane group kg = lane / 32 multiplies
// K 32 kg .. 32 kg + 31, eight at a step, so a lane's activations for one slab are 64
// contiguous bytes of its row.
template <int DT>
__device__ __forceinline__ float16v mfma32(uint4 a, uint4 b, float16v c) {
    if constexpr (DT == 1) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                      __builtin_bit_cast(half8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

// LDS of the 32x32x16 form: four activation rings of 16 KB (one per multiplying wave, two
// stages of 64 rows x 64 K), then the two weight slabs.  (The rings come first; M0, which carries an
// LDS-direct load's LDS address, also reaches the addresses above 64 KB: 69632, 135168 and 150000
// were written and read back on this device.)
// (RT = row tiles of 32 per multiplying wave: 2 for the 256-row tile, 1 for a 128-row tile)
template <int RT>
struct Wide32 {
    static constexpr uint32_t kWaveRows = 32 * RT;
    static constexpr uint32_t kTileRows = 4 * kWaveRows;
    static constexpr uint32_t kHalfBytes = kWaveRows * 64;          // a wave's rows x 32 K
    static constexpr uint32_t kStageBytes = 2 * kHalfBytes;         // one slab
    static constexpr uint32_t kRingBytes = 2 * kStageBytes;         // two stages
    static constexpr uint32_t kWeightsAt = 4 * kRingBytes;
    static constexpr int kDmaPieces = 4 * RT;                       // load instructions per slab and wave
};

// LDS-direct load: 16 bytes per lane from `g` to LDS address `lds_addr` + 16 * lane.
// The statement writes M0 without being able to declare it (M0 is refused in a clobber list):
// sound while the compiler keeps nothing of its own in M0 in this kernel, which has no other
// client of it.  The load returns no register and is covered only by the hand-placed
// `s_waitcnt vmcnt(0)` statements of the main loop; those wait for everything, so loads of the
// compiler's own in between cannot make them wrong.  The build checks the generated text for
// the M0 rule and for scratch (ferrum_amd/isa_check.py).
__device__ __forceinline__ void lds_direct16(const void* g, uint32_t lds_addr) {
    const uint32_t a = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(a) : "memory");
}

template <uint32_t TYPE, int DT, int NT, int RT>
__global__ __launch_bounds__(512) void gemm_wide32_kernel(const uint8_t* __restrict__ w,
                                                          const uint16_t* __restrict__ x,
                                                          void* __restrict__ y, uint32_t m, uint32_t n,
                                                          uint32_t nb, uint32_t y_dtype, uint32_t cols,
                                                          uint32_t tiles_m, uint32_t tiles_n) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    constexpr uint32_t kBlockBytes = block_bytes_of(TYPE);
    using Geo = Wide32<RT>;
    constexpr uint32_t kRowsW = 32 * NT;
    constexpr uint32_t kStage = kRowsW * kLd;  // halfs per buffer
    constexpr bool kExtra = NT > 4;            // rows 128 .. 159 are a second decode task

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    // XCD-aware tile order: ids r, r+8, r+16, .. of a group share the XCD (id mod 8)
    uint32_t tile_m, tile_n;
    {
        const uint32_t group_ids = 8 * tiles_m, id = blockIdx.x;
        const uint32_t g = id / group_ids, r = id % group_ids;
        tile_n = g * 8 + (r & 7u);
        tile_m = r >> 3;
        if (tile_n >= tiles_n) return;
    }
    const uint32_t n0 = tile_n * cols, m0 = tile_m * Geo::kTileRows;
    const uint32_t ncols = n - n0 < cols ? n - n0 : cols;
    const uint32_t k = nb << 8;

    if (wave >= 4) {
        // ---- producers: global -> registers -> (decode) -> LDS, blocks ahead ----
        const uint32_t pt = tid - 256, pw = wave - 4;
        const uint32_t wr = pt >> 1, wh = pt & 1u;
        const uint8_t* wsrc = w + (size_t)(n0 + (wr < ncols ? wr : ncols - 1)) * nb * kBlockBytes;
        // rows 128 .. 159: every wave takes eight of them, a lane one quarter of a (row, half) task
        // of every slab, so all slabs cost the same
        const uint32_t er = 128 + 8 * pw + (lane >> 3), eh = (lane >> 2) & 1u, et = lane & 3u;
        const uint8_t* esrc = w + (size_t)(n0 + (er < ncols ? er : ncols - 1)) * nb * kBlockBytes;
        constexpr bool kDeep = !kEightDwords<TYPE>;   // Q6_K and Q8_0 sets are twice as large: one block ahead
        BlockW<TYPE> cur, n1, n2, ecur, en1, en2;
        const bool has_row = kRowsW >= 128 || wr < kRowsW;   // narrow tiles leave some decoding lanes without a row
        auto store_slab = [&](int c) {
            uint16_t* ws = lds + Geo::kWeightsAt / 2 + (c & 1) * kStage;
            if (has_row) decode_block_slab<TYPE, DT>(cur, c, wh, ws + wr * kLd);
            if (kExtra) decode_block_piece<TYPE, DT>(ecur, c, eh, (int)et, ws + er * kLd);
        };
        auto load_main = [&](BlockW<TYPE>& set, uint32_t b) {
            if (has_row) set.load(wsrc + (size_t)b * kBlockBytes, wh);
        };
        load_main(cur, 0);
        if (kExtra) ecur.load(esrc, eh);
        if (nb > 1) {
            load_main(n1, 1);
            if (kExtra) en1.load(esrc + kBlockBytes, eh);
        }
        if (kDeep && nb > 2) {
            load_main(n2, 2);
            if (kExtra) en2.load(esrc + 2 * (size_t)kBlockBytes, eh);
        }
        store_slab(0);
        // The register set that the shift after a block's last slab frees is loaded with the block
        // `ahead` blocks on: rows 0 .. 127 at once, rows 128 .. two slabs later, so the load
        // instructions are spread over the slabs.
        constexpr uint32_t ahead = kDeep ? 3 : 2;
        for (uint32_t b = 0; b < nb; ++b) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                __syncthreads();  // slab 4b + c is visible; the other buffer is free
                if (c < 3) {
                    store_slab(c + 1);
                    if (c == 1 && kExtra && b >= 1 && b + ahead - 1 < nb) {
                        if (kDeep) en2.load(esrc + (size_t)(b + ahead - 1) * kBlockBytes, eh);
                        else en1.load(esrc + (size_t)(b + ahead - 1) * kBlockBytes, eh);
                    }
                } else if (b + 1 < nb) {
                    cur = n1;
                    if (kDeep) {
                        ecur = en1;
                        n1 = n2;
                        en1 = en2;
                        if (b + 3 < nb) load_main(n2, b + 3);
                    } else {
                        ecur = en1;
                        if (b + 2 < nb) load_main(n1, b + 2);
                    }
                    store_slab(0);
                }
            }
        }
        return;
    }

    // ---- consumers: own activation rows by LDS-direct loads, weights from LDS -> MFMA ----
    float16v acc[RT][NT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const uint32_t r32 = lane & 31u, kg = lane >> 5;
    // The wave's 64 activation rows travel through a ring of its own in LDS, one slab (64 K,
    // 8 KB) per stage, two stages: no other wave reads them, so no barrier is involved, only the
    // wave's own count of outstanding loads.  A stage is two halves of 32 K; in a half the
    // 16-byte piece q of local row r sits at unit 4 r + (q ^ ((r >> 2) & 3)), which spreads
    // the sixteen rows a fragment read touches over all banks.  One load instruction fills
    // 1 KB: 16 rows x 4 pieces, lane l = (row 16 t + l / 4, unit l % 4).
    const uint32_t a_ring = wave * Geo::kRingBytes;   // stage s of the ring is a_ring + kStageBytes (s & 1)
    const uint16_t* adma[2 * RT];
#pragma unroll
    for (int t = 0; t < 2 * RT; ++t) {
        const uint32_t r = 16 * t + (lane >> 2);
        const uint32_t q = (lane & 3u) ^ ((r >> 2) & 3u);
        const uint32_t row = m0 + wave * Geo::kWaveRows + r;
        // rows past m are clamped: they only feed outputs that are never stored
        adma[t] = x + (size_t)(row < m ? row : m - 1) * k + 8 * q;
    }
    // load instruction i of a slab: half i / (2 RT), rows 16 (i % (2 RT)) ..
    auto dma_piece = [&](uint32_t slab, int i) {
        lds_direct16(adma[i % (2 * RT)] + (size_t)slab * 64 + 32 * (i / (2 * RT)),
                     a_ring + (slab & 1u) * Geo::kStageBytes + (uint32_t)(i / (2 * RT)) * Geo::kHalfBytes +
                         (uint32_t)(i % (2 * RT)) * 1024u);
    };
    auto dma_slab = [&](uint32_t slab) {
#pragma unroll
        for (int i = 0; i < Geo::kDmaPieces; ++i) dma_piece(slab, i);
    };
    // fragment addresses: activations of row tile i at step s (0..3) of the slab, weights of column tile j
    const uint32_t sw = (r32 >> 2) & 3u;
    const uint32_t a_off0 = (4 * r32 + ((2 * kg) ^ sw)) * 16, a_off1 = (4 * r32 + ((2 * kg + 1) ^ sw)) * 16;
    const uint8_t* const lds_bytes = reinterpret_cast<const uint8_t*>(lds);
    const uint32_t b_off = Geo::kWeightsAt + (r32 * kLd + 16 * kg) * 2;
    constexpr int kFrags = RT + NT;   // fragments of a step: RT of activations, NT of weights
    struct Frags {
        uint4 v[kFrags];
    };
    auto read_frag = [&](Frags& f, uint32_t slab, int s, int t) {
        if (t < RT) {
            f.v[t] = *reinterpret_cast<const uint4*>(lds_bytes + a_ring + (slab & 1u) * Geo::kStageBytes +
                                                      (s >> 1) * Geo::kHalfBytes + ((s & 1) ? a_off1 : a_off0) + t * 2048);
        } else {
            f.v[t] = *reinterpret_cast<const uint4*>(lds_bytes + b_off + (slab & 1u) * (kStage * 2) + (s >> 1) * 64 +
                                                      (s & 1) * 16 + (t - RT) * (32 * kLd * 2));
        }
    };
    // One step: 2 NT multiplications on `cur`, and between them, one at a time so that each
    // hides behind a multiplication in flight, the reads of step (slab, s)'s fragments into
    // `next` and, with DMA set, the eight load instructions of activation slab `dma`.
    auto step = [&](const Frags& cur, Frags& next, uint32_t slab, int s, auto with_reads, auto with_dma, uint32_t dma) {
        constexpr int kMul = RT * NT;
        constexpr int kSlots = kMul > kFrags ? (kMul > Geo::kDmaPieces ? kMul : Geo::kDmaPieces)
                                             : (kFrags > Geo::kDmaPieces ? kFrags : Geo::kDmaPieces);
#pragma unroll
        for (int idx = 0; idx < kSlots; ++idx) {
            if constexpr (decltype(with_reads)::value)
                if (idx < kFrags) read_frag(next, slab, s, idx);
            if constexpr (decltype(with_dma)::value)
                if (idx < Geo::kDmaPieces) dma_piece(dma, idx);
            if (idx < kMul)
                acc[idx % RT][idx / RT] = mfma32<DT>(cur.v[idx % RT], cur.v[RT + idx / RT], acc[idx % RT][idx / RT]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    constexpr std::true_type yes{};
    constexpr std::false_type no{};
    // Software pipeline, one step deep: the fragments of step s + 1 are read while step s
    // multiplies, also across the slab boundary.  The barrier that opens slab c + 1 therefore
    // sits before the last step of slab c, whose fragments are in registers by then.
    const uint32_t slabs = nb * 4;   // at least four
    Frags f0, f1;
    dma_slab(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();               // the weights of slab 0 are visible
    dma_slab(1);
#pragma unroll
    for (int t = 0; t < kFrags; ++t) read_frag(f0, 0, 0, t);
    __builtin_amdgcn_s_setprio(2);  // the MFMA wave goes first when both waves of a SIMD can issue
    // the loop body is one straight run of code, so the counts of outstanding LDS reads are exact
    for (uint32_t c = 0; c + 1 < slabs; ++c) {
        step(f0, f1, c, 1, yes, no, 0u);
        step(f1, f0, c, 2, yes, no, 0u);
        step(f0, f1, c, 3, yes, no, 0u);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the activations of slab c + 1 have landed
        __syncthreads();           // its weights are visible; slab c is in registers, its buffers are free
        __builtin_amdgcn_sched_barrier(0);
        // On the last pass (c + 2 == slabs) there is no further slab, and the clamp loads slab
        // slabs - 1 a second time: into the stage it already occupies, the one this step and the
        // tail below read.  The bytes written are the bytes already there, so the readers see
        // the same values whichever copy they meet; the straight-line body stays one code path.
        // This holds only while the clamp names the slab that stage holds: a deeper ring or
        // another stage index must peel this pass and drop its loads instead.
        static_assert(Geo::kRingBytes == 2 * Geo::kStageBytes, "the clamped reload below relies on a two-stage activation ring");
        step(f1, f0, c + 1, 0, yes, yes, c + 2 < slabs ? c + 2 : slabs - 1);
    }
    {
        const uint32_t c = slabs - 1;
        step(f0, f1, c, 1, yes, no, 0u);
        step(f1, f0, c, 2, yes, no, 0u);
        step(f0, f1, c, 3, yes, no, 0u);
        step(f1, f0, c, 0, no, no, 0u);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the spare load of the last slab
    }
    __builtin_amdgcn_s_setprio(0);

    // element v of a lane's block: row 8 (v / 4) + 4 kg + v % 4, column r32
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const uint32_t lc = 32 * j + r32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = m0 + wave * Geo::kWaveRows + 32 * i + 8 * (v >> 2) + 4 * kg + (v & 3);
                if (row < m && lc < ncols)
                    store_from_f32(y, (size_t)row * n + n0 + lc, y_dtype, acc[i][j][v]);
            }
        }
}

struct WidePlan {
    int nt;
    uint32_t cols, tiles_m, tiles_n;
    int rt;   // 32x32x16 form: row tiles of 32 per multiplying wave (2: 256-row tile, 1: 128-row tile)
};

// Columns per workgroup: 128 or 136, whichever wastes the least of the chip's `cus`
// compute units (whole rounds of workgroups) and of the MFMA tile.  The ninth column
// tile is decoded eight rows deep (LDS rows 128..135), so 136 is the widest.
WidePlan wide_plan(uint32_t m, uint32_t n, int cus) {
    WidePlan best{};
    double best_cost = 1e300;
    const uint32_t tiles_m = (m + kWM - 1) / kWM;
    for (uint32_t cols : {128u, 136u}) {
        const int nt = cols > 128 ? 9 : 8;
        const uint32_t tiles_n = (n + cols - 1) / cols;
        const uint64_t wgs = (uint64_t)tiles_m * tiles_n;
        const uint64_t rounds = (wgs + cus - 1) / cus;
        const double cost = (double)rounds * nt;   // time ~ rounds x MFMA tiles per slab
        if (cost < best_cost) {
            best_cost = cost;
            best = {nt, cols, tiles_m, tiles_n};
        }
    }
    return best;
}

// What a round of workgroups of one 32x32x16 tile takes over rows of 5120, in us: one workgroup per
// compute unit (`alone`), or two where LDS and registers hold two, from the first pair
// (`pair_first`) to a pair everywhere (`pair_all`; 0 = the tile runs alone).  Measured on
// 17408 / 34816 / 8192 / 5120 columns at 48 - 2048 rows; two 128 x 128 tiles on a compute unit take
// 88 - 108 us where one takes 64, so a pair does a fifth to a half more per microsecond.
struct Wide32Tile {
    int rt, nt;
    double alone, pair_first, pair_all;
};
constexpr Wide32Tile kWide32Tiles[] = {
    {1, 2, 49.0, 61.0, 71.0}, {1, 3, 58.6, 0.0, 0.0}, {1, 4, 64.0, 88.0, 108.0}, {1, 5, 79.0, 0.0, 0.0},
    {2, 4, 90.0, 0.0, 0.0},   {2, 5, 108.0, 0.0, 0.0},
};
// an eighth of a tile's time is its prologue and its stores, the rest goes with the length of a row
inline double wide_row_length_factor(uint32_t k) { return 0.125 + 0.875 * (double)k / 5120.0; }

// The 128 x 96 tile is there for one case: a few columns more than 64 per workgroup make one
// workgroup per compute unit where 128 x 64 tiles would number a few more than the compute units and
// the units with two set the time (17408 columns on 256 units: 68 columns each, 128 rows in 58.6 -
// 60.9 against 61.1 us, 96 rows in 56.6 - 58.6 against 60.0 on two boxes; the same bits).  Its width is the fewest columns,
// a multiple of four, that make at most `cus` workgroups; 0 tiles when that is not in 65 .. 96.
WidePlan wide32_make(uint32_t m, uint32_t n, int rt, int nt, int cus = 256) {
    const uint32_t rows = 128u * (uint32_t)rt, tiles_m = (m + rows - 1) / rows;
    uint32_t cols = 32u * (uint32_t)nt;
    if (nt == 3) {
        const uint32_t per_row_tile = (uint32_t)cus / tiles_m;
        cols = per_row_tile == 0 ? 0 : ((n + per_row_tile - 1) / per_row_tile + 3u) & ~3u;
        if (cols <= 64u || cols > 96u) return WidePlan{3, 96, tiles_m, 0, rt};
    }
    return WidePlan{nt, cols, tiles_m, (n + cols - 1) / cols, rt};
}

double wide32_estimate(const Wide32Tile& t, uint64_t wgs, uint64_t cus) {
    if (wgs <= cus) return t.alone;
    if (t.pair_first == 0.0) return (double)((wgs + cus - 1) / cus) * t.alone;
    const uint64_t full = wgs / (2 * cus), rest = wgs % (2 * cus);
    double us = (double)full * t.pair_all;
    if (rest > cus) {
        us += t.pair_first + (t.pair_all - t.pair_first) * (double)(rest - cus) / (double)cus;
    } else if (rest > 0) {
        us += full > 0 ? 0.66 * t.alone : t.alone;  // a last round of single workgroups starts while pairs still run
    }
    return us;
}

// The tile of the 32x32x16 form with the smallest estimate for this shape.  Tiles whose workgroups
// would leave more than half the chip idle are left to the kernels made for few columns (nt = 0
// when that holds for all of them).  At 17408 x 5120 that gives 128 x 64 up to 128 rows (61 us),
// 128 x 160 up to 256 (78), 128 x 128 up to 384 (97), 256 x 160 beyond (111 at 512 rows), each
// against the 16x16x32 form's 85 / 106 / 108 / 115 us; at 8192 x 4096 and 512 rows 128 x 128, 52
// against 83 us.  Over 38 measured shapes the estimate picked the fastest tile every time.
WidePlan wide32_plan(uint32_t m, uint32_t n, uint32_t k, int cus, double* estimate) {
    WidePlan best{};
    double best_us = 1e300;
    for (const Wide32Tile& t : kWide32Tiles) {
        const WidePlan p = wide32_make(m, n, t.rt, t.nt, cus);
        const uint64_t wgs = (uint64_t)p.tiles_m * p.tiles_n;
        if (wgs * 2 < (uint64_t)cus) continue;
        const double us = wide32_estimate(t, wgs, (uint64_t)cus);
        if (us < best_us) {
            best_us = us;
            best = p;
        }
    }
    *estimate = best_us * wide_row_length_factor(k);
    return best;
}

// The 16x16x32 form keeps two workgroups on a compute unit, one storing while the other
// multiplies, so its rounds need not be whole: 2048 x 17408 x 5120 takes 442 us in 4.25 rounds.
double wide16_estimate(uint32_t m, uint32_t n, uint32_t k, int cus) {
    const uint64_t wgs = (uint64_t)((m + kWM - 1) / kWM) * ((n + 127) / 128);
    const double rounds = (double)wgs / (double)cus;
    return (rounds < 1.0 ? 1.0 : rounds) * 105.0 * wide_row_length_factor(k);
}

// The rows-resident kernel: a start that grows with the matrix, then a cost per group of rows that
// LDS holds at once (32 rows of up to 2560, 16 of up to 5120), since every weight is decoded once
// per group.  Measured at 48 - 512 rows on the shapes above and 151936 x 2048; within a sixth of each.
double resident_estimate(uint32_t m, uint32_t n, uint32_t k) {
    const double weights = (double)n * (double)k;
    if ((size_t)32 * k * 2 <= 160u * 1024) return 12.0 + weights * 0.68e-7 + weights * 1.25e-7 * ((m + 31) / 32);
    const double start = weights * 1.5e-7;
    return 12.0 + (start < 14.0 ? start : 14.0) + weights * 8.3e-8 * ((m + 15) / 16);
}

template <uint32_t TYPE, int DT, int NT, int RT>
void launch_wide32(hipStream_t s, const GemmArgs& a, const WidePlan& plan) {
    const size_t lds = Wide32<RT>::kWeightsAt + 2 * (size_t)(32 * NT) * kLd * sizeof(uint16_t);
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_wide32_kernel<TYPE, DT, NT, RT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        configured = true;
    }
    const uint32_t groups = (plan.tiles_n + 7) / 8;
    dim3 grid(groups * 8 * plan.tiles_m);
    hipLaunchKernelGGL((gemm_wide32_kernel<TYPE, DT, NT, RT>), grid, dim3(512), lds, s,
                       static_cast<const uint8_t*>(a.w), static_cast<const uint16_t*>(a.x), a.y, a.m, a.n,
                       a.k / 256, a.y_dtype, plan.cols, plan.tiles_m, plan.tiles_n);
}

template <uint32_t TYPE, int DT, int NT>
void launch_wide(hipStream_t s, const GemmArgs& a, const WidePlan& plan) {
    const size_t lds = 2 * (size_t)(16 * NT) * kLd * sizeof(uint16_t);
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_wide_kernel<TYPE, DT, NT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        configured = true;
    }
    const uint32_t groups = (plan.tiles_n + 7) / 8;
    dim3 grid(groups * 8 * plan.tiles_m);
    hipLaunchKernelGGL((gemm_wide_kernel<TYPE, DT, NT>), grid, dim3(kWideThreads), lds, s,
                       static_cast<const uint8_t*>(a.w), static_cast<const uint16_t*>(a.x), a.y, a.m, a.n,
                       a.k / 256, a.y_dtype, plan.cols, plan.tiles_m, plan.tiles_n);
}

template <uint32_t TYPE, int DT>
void launch_wide_nt(hipStream_t s, const GemmArgs& a, const WidePlan& plan, const WidePlan& p32) {
    if (p32.nt != 0) {
        if (p32.rt == 1) {
            if (p32.nt == 3) launch_wide32<TYPE, DT, 3, 1>(s, a, p32);
            else if (p32.nt == 2) launch_wide32<TYPE, DT, 2, 1>(s, a, p32);
            else if (p32.nt == 5) launch_wide32<TYPE, DT, 5, 1>(s, a, p32);
            else launch_wide32<TYPE, DT, 4, 1>(s, a, p32);
        } else {
            if (p32.nt == 5) launch_wide32<TYPE, DT, 5, 2>(s, a, p32);
            else launch_wide32<TYPE, DT, 4, 2>(s, a, p32);
        }
        return;
    }
    if (plan.nt == 9) {
        launch_wide<TYPE, DT, 9>(s, a, plan);
    } else {
        launch_wide<TYPE, DT, 8>(s, a, plan);
    }
}

}  // namespace

const char* launch_gemm(hipStream_t s, const GemmArgs& a) {
    // the 256-row tile pays off only when its workgroups cover at least half the chip
    const uint64_t wide_wgs = (uint64_t)((a.m + kWM - 1) / kWM) * ((a.n + 127) / 128);
    const bool wide_pays = a.m >= (uint32_t)a.wide_min_rows && wide_wgs * 2 >= (uint64_t)a.cu_count;
    // Rows that fit LDS for their whole length take the kernel that keeps them there and streams
    // the weights past them through registers.  Against the register-dequant kernel that stages
    // the rows slab by slab (up to 64 rows) it is 15% faster at 2 - 16 rows and up to twice at 64
    // (64 x 4096 x 4096: 14.1 against 29.7 us; 64 x 17408 x 5120: 52.8 against 74.0 us, the same
    // bits), except for 512-long rows in 16-row batches or
    // less, where a launch is 4 us either way; against the square tiles 1.4 - 2.2 times
    // (512 x 1024 x 2048: 11.5 against 22.8 us).
    // Rows longer than 2560 fit only 16 at a time, and every weight is then decoded M / 16 times:
    // that still wins up to 256 rows (256 x 5120 x 5120: 51 against 86 us) and loses at 512 (95
    // against 84 us).
    // From wide_min_rows rows on, the tiles of the 32x32x16 form compete: the smallest estimate
    // among them, the 16x16x32 form and the rows-resident kernel takes the call.
    WidePlan p32{};
    double us32 = 1e300;
    if (a.wide_shape != 0 && a.m >= (uint32_t)a.wide_min_rows) {
        if (a.wide32_tile != 0) {
            p32 = wide32_make(a.m, a.n, a.wide32_tile / 10, a.wide32_tile % 10, a.cu_count);
            if (p32.tiles_n == 0) p32 = wide32_make(a.m, a.n, 1, 4);   // no width of the 96-column tile fits this shape
            us32 = 0.0;
        } else {
            p32 = wide32_plan(a.m, a.n, a.k, a.cu_count, &us32);
            if (p32.nt == 0 && a.wide_shape == 2 && wide_pays) {
                p32 = wide32_make(a.m, a.n, 2, 5);
                us32 = 0.0;
            }
        }
    }
    const double us16 = wide_pays && a.wide_shape != 2 ? wide16_estimate(a.m, a.n, a.k, a.cu_count) : 1e300;
    if (a.rows_resident) {
        const bool few = a.m <= (uint32_t)a.skinny_max_rows;
        const bool groups_of_32 = (size_t)32 * a.k * 2 <= 160u * 1024;
        // Where the 256-row tile would pay, it is mostly empty below 256 rows while this kernel's
        // cost grows with the row count: 65 x 17408 x 5120 takes 67 against 82 us and 128 rows
        // 87 against 87; with groups of 32 (K = 2048) 128 rows take 30 against 41 us and 256
        // rows 49 against 49.
        bool take = few          ? !(a.k <= 512 && a.m <= 16)
                    : wide_pays ? a.m <= (groups_of_32 ? 192u : 96u)
                                : groups_of_32 || a.m <= 256;
        // (the estimates were measured on rows of 2048 and more; shorter ones keep the rule above)
        if (p32.nt != 0 && (a.k >= 1024 || a.wide32_tile != 0))
            take = resident_estimate(a.m, a.n, a.k) < (us32 < us16 ? us32 : us16);
        if (take) return launch_gemm_resident(s, a);
    }
    if (p32.nt != 0 && us16 < us32) p32.nt = 0;
    if (p32.nt == 0 && a.m <= (uint32_t)a.skinny_max_rows) return launch_gemm_skinny(s, a);
    if (wide_pays || p32.nt != 0) {
        const WidePlan plan = wide_plan(a.m, a.n, a.cu_count);
        if (a.ggml_type == kQ4K) {
            if (a.x_dtype == FH_F16) launch_wide_nt<kQ4K, 1>(s, a, plan, p32); else launch_wide_nt<kQ4K, 2>(s, a, plan, p32);
            return "q4_k_gemm_mfma_m256";
        }
        if (a.ggml_type == kQ5K) {
            if (a.x_dtype == FH_F16) launch_wide_nt<kQ5K, 1>(s, a, plan, p32); else launch_wide_nt<kQ5K, 2>(s, a, plan, p32);
            return "q5_k_gemm_mfma_m256";
        }
        if (a.ggml_type == kIQ4XS) {
            if (a.x_dtype == FH_F16) launch_wide_nt<kIQ4XS, 1>(s, a, plan, p32); else launch_wide_nt<kIQ4XS, 2>(s, a, plan, p32);
            return "iq4_xs_gemm_mfma_m256";
        }
        if (a.ggml_type == kQ8_0) {
            if (a.x_dtype == FH_F16) launch_wide_nt<kQ8_0, 1>(s, a, plan, p32); else launch_wide_nt<kQ8_0, 2>(s, a, plan, p32);
            return "q8_0_gemm_mfma_m256";
        }
        if (a.x_dtype == FH_F16) launch_wide_nt<kQ6K, 1>(s, a, plan, p32); else launch_wide_nt<kQ6K, 2>(s, a, plan, p32);
        return "q6_k_gemm_mfma_m256";
    }
    // 128 x 128 tiles, or 64 x 64 when those would leave most of the chip idle
    const uint64_t big_wgs = (uint64_t)((a.n + kBN - 1) / kBN) * ((a.m + kBM - 1) / kBM);
    const bool small = big_wgs * 2 < (uint64_t)a.cu_count;
    const uint64_t mid_wgs = (uint64_t)((a.n + 63) / 64) * ((a.m + 63) / 64);
    const bool tiny = small && mid_wgs < (uint64_t)a.cu_count;
    const uint32_t ts = tiny ? 32 : small ? 64 : 128;
    dim3 grid((a.n + ts - 1) / ts, (a.m + ts - 1) / ts);
    const uint32_t nb = a.k / 256;
    const uint8_t* w = static_cast<const uint8_t*>(a.w);
    const uint16_t* x = static_cast<const uint16_t*>(a.x);
    auto run = [&](auto big, auto little, auto least) {
        if (tiny) {
            hipLaunchKernelGGL(least, grid, dim3(64), 0, s, w, x, a.y, a.m, a.n, nb, a.y_dtype);
        } else if (small) {
            hipLaunchKernelGGL(little, grid, dim3(128), 0, s, w, x, a.y, a.m, a.n, nb, a.y_dtype);
        } else {
            hipLaunchKernelGGL(big, grid, dim3(256), 0, s, w, x, a.y, a.m, a.n, nb, a.y_dtype);
        }
    };
    if (a.ggml_type == kQ4K) {
        if (a.x_dtype == FH_F16) {
            run(gemm_tile_kernel<kQ4K, 1, 128>, gemm_tile_kernel<kQ4K, 1, 64>, gemm_tile_kernel<kQ4K, 1, 32>);
        } else {
            run(gemm_tile_kernel<kQ4K, 2, 128>, gemm_tile_kernel<kQ4K, 2, 64>, gemm_tile_kernel<kQ4K, 2, 32>);
        }
        return "q4_k_gemm_mfma";
    }
    if (a.ggml_type == kQ5K) {
        if (a.x_dtype == FH_F16) {
            run(gemm_tile_kernel<kQ5K, 1, 128>, gemm_tile_kernel<kQ5K, 1, 64>, gemm_tile_kernel<kQ5K, 1, 32>);
        } else {
            run(gemm_tile_kernel<kQ5K, 2, 128>, gemm_tile_kernel<kQ5K, 2, 64>, gemm_tile_kernel<kQ5K, 2, 32>);
        }
        return "q5_k_gemm_mfma";
    }
    if (a.ggml_type == kIQ4XS) {
        if (a.x_dtype == FH_F16) {
            run(gemm_tile_kernel<kIQ4XS, 1, 128>, gemm_tile_kernel<kIQ4XS, 1, 64>, gemm_tile_kernel<kIQ4XS, 1, 32>);
        } else {
            run(gemm_tile_kernel<kIQ4XS, 2, 128>, gemm_tile_kernel<kIQ4XS, 2, 64>, gemm_tile_kernel<kIQ4XS, 2, 32>);
        }
        return "iq4_xs_gemm_mfma";
    }
    if (a.ggml_type == kQ8_0) {
        if (a.x_dtype == FH_F16) {
            run(gemm_tile_kernel<kQ8_0, 1, 128>, gemm_tile_kernel<kQ8_0, 1, 64>, gemm_tile_kernel<kQ8_0, 1, 32>);
        } else {
            run(gemm_tile_kernel<kQ8_0, 2, 128>, gemm_tile_kernel<kQ8_0, 2, 64>, gemm_tile_kernel<kQ8_0, 2, 32>);
        }
        return "q8_0_gemm_mfma";
    }
    if (a.x_dtype == FH_F16) {
        run(gemm_tile_kernel<kQ6K, 1, 128>, gemm_tile_kernel<kQ6K, 1, 64>, gemm_tile_kernel<kQ6K, 1, 32>);
    } else {
        run(gemm_tile_kernel<kQ6K, 2, 128>, gemm_tile_kernel<kQ6K, 2, 64>, gemm_tile_kernel<kQ6K, 2, 32>);
    }
    return "q6_k_gemm_mfma";
}

}  // namespace fh
