// Skinny-M projection (2 <= M <= 64 tokens, f16 / bf16 activations) on the
// matrix cores: Y[M,N] = X[M,K] . W[N,K]^T for Q4_K / Q5_K / Q6_K / IQ4_XS / Q8_0 weights.
//
// With this few tokens the job is a weight stream (HBM bound), so nothing of
// the weights goes through LDS.  A wave owns 16 weight rows.  Its 64 lanes are
// 16 rows x 4 lane groups, and a lane group owns one quarter of every
// super-block of its row (Q4_K: one 64-weight chunk, 32 contiguous bytes;
// Q6_K: 16 positions of one 128-weight half).  The lane decodes its 64 weights
// in registers straight into eight A operands of v_mfma_f32_16x16x32 (rows =
// weight rows): an MFMA only needs A and B to agree on which 32 K indices a
// step covers, so step s simply takes "the s-th run of 8 weights of every lane
// group's quarter", and the activations are read from LDS in the same order.
// Decoding is the one-rounding fma of tile_decode.hpp, so tile values carry the
// bits of the reference's dequantisation rounded once to the tile type.
//
// The four waves of a workgroup cover 64 rows and share the activation slab
// (16*TT tokens x 256 K) of the current super-block through a double-buffered
// LDS tile; one barrier per super-block.  Every lane keeps kRing super-blocks
// and kRing activation slabs in flight in registers: loads return in order, so
// both rings must run equally far ahead or the nearer one would drain the
// farther.
#include <hip/hip_runtime.h>

#include "device_utils.hpp"
#include "lds_direct.hpp"
#include "tile_decode.hpp"
#include "internal.hpp"

namespace fh {
namespace {

constexpr int kSkThreads = 256;
constexpr int kSkRows = 64;         // weight rows per workgroup
constexpr int kSlabLd = 256 + 8;    // halfs per token row of the LDS slab (16-byte skew)
constexpr int kRing = 5;

// One lane's quarter of a super-block, raw, and its decode into 8 A operands.
// klocal(g, s): K offset inside the super-block of the 8 weights of operand s.
template <uint32_t TYPE>
struct Quarter;

template <>
struct Quarter<kQ4K> {
    static constexpr uint32_t kBlockBytes = 144;
    uint4 hdr, qa, qb;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t g) {
        hdr = *reinterpret_cast<const uint4*>(block);
        qa = *reinterpret_cast<const uint4*>(block + 16 + 32 * g);
        qb = *reinterpret_cast<const uint4*>(block + 32 + 32 * g);
    }
    // operands 0..3: low nibbles (weights 64g + 8s ..), 4..7: high nibbles (64g + 32 + 8(s-4) ..)
    static __device__ __forceinline__ uint32_t klocal(uint32_t g, int s) { return 64 * g + 8 * s; }
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t g, uint4 (&a)[8]) const {
        const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc0, sc1, mn0, mn1;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, g, sc0, sc1, mn0, mn1);
        // d*sc and dmin*m are exact in f32; the powers of two undo the subnormal encoding
        const float a_lo = (d * sc0) * 16777216.f, a_hi = (d * sc1) * 1048576.f;
        const float b_lo = -(dmin * mn0), b_hi = -(dmin * mn1);
        const uint32_t v[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        uint32_t lo[16], hi[16];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t w0 = v[t], w1 = w0 >> 8;
            const uint32_t l02 = w0 & 0x000f000fu, h02 = w0 & 0x00f000f0u;
            const uint32_t l13 = w1 & 0x000f000fu, h13 = w1 & 0x00f000f0u;
            lo[2 * t] = fma_pair<DT>(lo_half(l02), lo_half(l13), a_lo, b_lo);
            lo[2 * t + 1] = fma_pair<DT>(hi_half(l02), hi_half(l13), a_lo, b_lo);
            hi[2 * t] = fma_pair<DT>(lo_half(h02), lo_half(h13), a_hi, b_hi);
            hi[2 * t + 1] = fma_pair<DT>(hi_half(h02), hi_half(h13), a_hi, b_hi);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            a[s] = make_uint4(lo[4 * s], lo[4 * s + 1], lo[4 * s + 2], lo[4 * s + 3]);
            a[4 + s] = make_uint4(hi[4 * s], hi[4 * s + 1], hi[4 * s + 2], hi[4 * s + 3]);
        }
    }
};

template <>
struct Quarter<kQ5K> {
    static constexpr uint32_t kBlockBytes = 176;
    uint4 hdr, ha, hb, qa, qb;   // ha, hb: the block's 32 qh bytes (fifth bits, bit 2g low / 2g + 1 high nibbles)
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t g) {
        hdr = *reinterpret_cast<const uint4*>(block);
        ha = *reinterpret_cast<const uint4*>(block + 16);
        hb = *reinterpret_cast<const uint4*>(block + 32);
        qa = *reinterpret_cast<const uint4*>(block + 48 + 32 * g);
        qb = *reinterpret_cast<const uint4*>(block + 64 + 32 * g);
    }
    static __device__ __forceinline__ uint32_t klocal(uint32_t g, int s) { return 64 * g + 8 * s; }
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t g, uint4 (&a)[8]) const {
        const float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc0, sc1, mn0, mn1;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, g, sc0, sc1, mn0, mn1);
        const float a_lo = (d * sc0) * 16777216.f, a_hi = (d * sc1) * 1048576.f;
        const float b_lo = -(dmin * mn0), b_hi = -(dmin * mn1);
        const uint32_t v[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const uint32_t p[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        uint32_t lo[16], hi[16];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t w0 = v[t], w1 = w0 >> 8;
            const uint32_t p0 = p[t] >> (2 * g), p1 = p0 >> 8;
            const uint32_t l02 = (w0 & 0x000f000fu) | ((p0 & 0x00010001u) << 4);
            const uint32_t l13 = (w1 & 0x000f000fu) | ((p1 & 0x00010001u) << 4);
            const uint32_t h02 = (w0 & 0x00f000f0u) | ((p0 & 0x00020002u) << 7);
            const uint32_t h13 = (w1 & 0x00f000f0u) | ((p1 & 0x00020002u) << 7);
            lo[2 * t] = fma_pair<DT>(lo_half(l02), lo_half(l13), a_lo, b_lo);
            lo[2 * t + 1] = fma_pair<DT>(hi_half(l02), hi_half(l13), a_lo, b_lo);
            hi[2 * t] = fma_pair<DT>(lo_half(h02), lo_half(h13), a_hi, b_hi);
            hi[2 * t + 1] = fma_pair<DT>(hi_half(h02), hi_half(h13), a_hi, b_hi);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            a[s] = make_uint4(lo[4 * s], lo[4 * s + 1], lo[4 * s + 2], lo[4 * s + 3]);
            a[4 + s] = make_uint4(hi[4 * s], hi[4 * s + 1], hi[4 * s + 2], hi[4 * s + 3]);
        }
    }
};

// IQ4_XS: lane group g owns sub-blocks 2g and 2g + 1 (qs bytes [32g, +32)).  Low
// nibbles are a sub-block's weights 0..15, high nibbles 16..31, so operand s
// covers weights 64g + 8s .. as for Q4_K.  Codebook bytes (value + 128) become
// f16 subnormals; fma(byte, scale, -128 scale) is the exact weight.
template <>
struct Quarter<kIQ4XS> {
    static constexpr uint32_t kBlockBytes = 136;
    uint2 hdr;
    uint4 qa, qb;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t g) {
        hdr = *reinterpret_cast<const uint2*>(block);
        qa = load_u4_unaligned(block + 8 + 32 * g);
        qb = load_u4_unaligned(block + 24 + 32 * g);
    }
    static __device__ __forceinline__ uint32_t klocal(uint32_t g, int s) { return 64 * g + 8 * s; }
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t g, uint4 (&a)[8]) const {
        const uint32_t v[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            const float dl = iq4xs_scale(hdr.x, hdr.y, 2 * g + sub);
            const float scale = dl * 16777216.f, offset = -128.f * dl;
            uint32_t lo[8], hi[8];   // pair dwords of weights 0..15 and 16..31 of the sub-block
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t l = iq4_lookup4(v[4 * sub + t]), h = iq4_lookup4(v[4 * sub + t] >> 4);
                const uint32_t l01 = bytes01_as_halves(l), l23 = bytes23_as_halves(l);
                const uint32_t h01 = bytes01_as_halves(h), h23 = bytes23_as_halves(h);
                lo[2 * t] = fma_pair<DT>(lo_half(l01), hi_half(l01), scale, offset);
                lo[2 * t + 1] = fma_pair<DT>(lo_half(l23), hi_half(l23), scale, offset);
                hi[2 * t] = fma_pair<DT>(lo_half(h01), hi_half(h01), scale, offset);
                hi[2 * t + 1] = fma_pair<DT>(lo_half(h23), hi_half(h23), scale, offset);
            }
            a[4 * sub] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            a[4 * sub + 1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
            a[4 * sub + 2] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            a[4 * sub + 3] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        }
    }
};

// Q8_0: lane group g owns blocks 2g and 2g + 1 of the 256-weight run; operand s covers
// weights 64g + 8s .., two quant dwords of one block.
template <>
struct Quarter<kQ8_0> {
    static constexpr uint32_t kBlockBytes = 272;
    Q8Pair p;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t g) { p.load(block + 68 * g); }
    static __device__ __forceinline__ uint32_t klocal(uint32_t g, int s) { return 64 * g + 8 * s; }
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t, uint4 (&a)[8]) const {
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const float d = p.d(blk);
            const float scale = d * 16777216.f, offset = -128.f * d;   // fma(q + 128, d, -128 d) = d q, exact
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const uint32_t u0 = p.biased(blk, 2 * s), u1 = p.biased(blk, 2 * s + 1);
                const uint32_t a01 = bytes01_as_halves(u0), a23 = bytes23_as_halves(u0);
                const uint32_t b01 = bytes01_as_halves(u1), b23 = bytes23_as_halves(u1);
                a[4 * blk + s] = make_uint4(fma_pair<DT>(lo_half(a01), hi_half(a01), scale, offset),
                                            fma_pair<DT>(lo_half(a23), hi_half(a23), scale, offset),
                                            fma_pair<DT>(lo_half(b01), hi_half(b01), scale, offset),
                                            fma_pair<DT>(lo_half(b23), hi_half(b23), scale, offset));
            }
        }
    }
};

template <>
struct Quarter<kQ6K> {
    static constexpr uint32_t kBlockBytes = 210;
    uint4 la, lb, ph, sc;
    uint32_t d;
    // lane group g: half h = g / 2 of the block, positions j0 = 16 (g & 1) .. j0 + 15
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t g) {
        const uint32_t h = g >> 1, j0 = (g & 1u) * 16;
        la = load_u4_unaligned(block + 64 * h + j0);
        lb = load_u4_unaligned(block + 64 * h + 32 + j0);
        ph = load_u4_unaligned(block + 128 + 32 * h + j0);
        sc = load_u4_unaligned(block + 192);
        d = load_u16_unaligned(block + 208);
    }
    // operand s: slice s / 2 (32 weights each), positions j0 + 8 (s & 1) ..
    static __device__ __forceinline__ uint32_t klocal(uint32_t g, int s) {
        return 128 * (g >> 1) + 32 * (s >> 1) + 16 * (g & 1u) + 8 * (s & 1);
    }
    template <int DT>
    __device__ __forceinline__ void decode(uint32_t g, uint4 (&a)[8]) const {
        const float df = f16_bits_to_f32(d);
        const uint32_t h = g >> 1;
        const uint32_t scw[4] = {sc.x, sc.y, sc.z, sc.w};
        const uint32_t lav[4] = {la.x, la.y, la.z, la.w}, lbv[4] = {lb.x, lb.y, lb.z, lb.w};
        const uint32_t phv[4] = {ph.x, ph.y, ph.z, ph.w};
        // scales 8h + 2*slice + (g & 1): slices 0,1 in word 2h, slices 2,3 in word 2h + 1
        const uint32_t w_lo = (h ? scw[2] : scw[0]) >> (8 * (g & 1u));
        const uint32_t w_hi = (h ? scw[3] : scw[1]) >> (8 * (g & 1u));
#pragma unroll
        for (int slice = 0; slice < 4; ++slice) {
            const uint32_t word = slice < 2 ? w_lo : w_hi;
            const float s = df * (float)(int)(int8_t)(word >> (16 * (slice & 1)));
            const float scale = s * ((slice < 2) ? 16777216.f : 1048576.f);  // high nibbles sit 4 bits up
            const float offset = -32.f * s;
            uint32_t out[8];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t w0 = (slice & 1) ? lbv[t] : lav[t], w1 = w0 >> 8;
                const uint32_t p0 = phv[t] >> (2 * slice), p1 = p0 >> 8;
                uint32_t q02, q13;
                if (slice < 2) {  // low nibble | plane bits << 4 : q * 2^-24
                    q02 = (w0 & 0x000f000fu) | ((p0 & 0x00030003u) << 4);
                    q13 = (w1 & 0x000f000fu) | ((p1 & 0x00030003u) << 4);
                } else {          // high nibble in place | plane bits << 8 : 16 q * 2^-24
                    q02 = (w0 & 0x00f000f0u) | ((p0 & 0x00030003u) << 8);
                    q13 = (w1 & 0x00f000f0u) | ((p1 & 0x00030003u) << 8);
                }
                out[2 * t] = fma_pair<DT>(lo_half(q02), lo_half(q13), scale, offset);
                out[2 * t + 1] = fma_pair<DT>(hi_half(q02), hi_half(q13), scale, offset);
            }
            a[2 * slice] = make_uint4(out[0], out[1], out[2], out[3]);
            a[2 * slice + 1] = make_uint4(out[4], out[5], out[6], out[7]);
        }
    }
};

// One thread's share of an activation slab (16*TT tokens x 256 K) on its way
// from global memory to LDS.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // a native vector: copies stay in registers

template <int XP>
struct SlabRows {
    const uint16_t* row[XP];  // activation row of the token each piece belongs to, at this thread's column
};

template <int XP>
struct SlabRegs {
    u32x4 v[XP];
    __device__ __forceinline__ void load(const SlabRows<XP>& rows, size_t col) {
#pragma unroll
        for (int p = 0; p < XP; ++p) v[p] = *reinterpret_cast<const u32x4*>(rows.row[p] + col);
    }
    __device__ __forceinline__ void store(uint16_t* dst) const {
#pragma unroll
        for (int p = 0; p < XP; ++p) *reinterpret_cast<u32x4*>(dst + p * 8 * kSlabLd) = v[p];
    }
};

// GROUPED = false: the dense projection, tokens 0 .. m-1 of x, one weight matrix.
// GROUPED = true: the routed-expert projection.  blockIdx.y is an expert; its
// tokens are the assignments order[offsets[e]] .. order[offsets[e+1] - 1], or rows
// offsets[e] .. offsets[e+1] - 1 themselves when order is null (rows
// of x and of y), its weights rows [e*n, e*n + n), and the workgroup makes as
// many passes of 16*TT tokens as the expert's count needs (the weights of the
// later passes come from L2).
template <uint32_t TYPE, int DT, int TT, bool GROUPED>
__global__ __launch_bounds__(kSkThreads) void gemm_skinny_kernel(const uint8_t* __restrict__ w,
                                                                 const uint16_t* __restrict__ x,
                                                                 void* __restrict__ y, uint32_t m,
                                                                 uint32_t n, uint32_t nb,
                                                                 uint32_t y_dtype,
                                                                 const uint32_t* __restrict__ offsets,
                                                                 const uint32_t* __restrict__ order) {
    constexpr uint32_t kBB = Quarter<TYPE>::kBlockBytes;
    constexpr int kTokens = 16 * TT;
    constexpr int kSlab = kTokens * kSlabLd;      // halfs per LDS buffer
    constexpr int kXP = 2 * TT;                   // 16-byte pieces of a slab per thread
    __shared__ __attribute__((aligned(16))) uint16_t slab[2 * kSlab];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint32_t row0 = blockIdx.x * kSkRows + wave * 16;
    const uint32_t row = min(row0 + r, n - 1);
    const size_t k = (size_t)nb * 256;

    uint32_t first_token = 0, count = m;
    size_t expert_row = 0;
    if constexpr (GROUPED) {
        // a damaged offsets table reads wrong rows, never rows outside the m assignments
        first_token = min(offsets[blockIdx.y], m);
        const uint32_t upto = min(offsets[blockIdx.y + 1], m);
        count = upto > first_token ? upto - first_token : 0;
        expert_row = (size_t)blockIdx.y * n;
    }
    const uint8_t* wrow = w + (expert_row + row) * nb * kBB;

    // activation slab pieces of this thread: piece p covers token 8p + tid / 32, halfs
    // 8 (tid % 32) ..
    const uint32_t xtok = tid >> 5, xcol = 8 * (tid & 31u);
    const uint32_t xdst = xtok * kSlabLd + xcol;

    // B operand address of (token r of tile tt, step s) inside a slab
    uint32_t boff[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) boff[s] = r * kSlabLd + Quarter<TYPE>::klocal(g, s);
    const uint32_t last = nb - 1;

    for (uint32_t t0 = 0; t0 < count; t0 += kTokens) {
        const uint32_t mt = min((uint32_t)kTokens, count - t0);
        if (t0 != 0) __syncthreads();  // the previous pass is done with the slabs
        // tokens past the count repeat the last one (their output columns are never
        // stored), which keeps the loop free of branches
        SlabRows<kXP> rows;
#pragma unroll
        for (int p = 0; p < kXP; ++p) {
            uint32_t token = first_token + t0 + min(xtok + 8 * p, mt - 1);
            if constexpr (GROUPED) token = order != nullptr ? order[token] : token;
            rows.row[p] = x + (size_t)token * k + xcol;
        }

        SlabRegs<kXP> xr[kRing];
        Quarter<TYPE> ring[kRing];
        // ring[i] holds super-block j with j % kRing == i; xr[i] holds activation slab j + 1
        {
            SlabRegs<kXP> first;
            first.load(rows, 0);
#pragma unroll
            for (int i = 0; i < kRing; ++i) {
                ring[i].load(wrow + (size_t)min((uint32_t)i, last) * kBB, g);
                xr[i].load(rows, 256 * (size_t)min((uint32_t)i + 1, last));
                // issue order matters: the loop waits by count, oldest first
                __builtin_amdgcn_sched_barrier(0);
            }
            first.store(slab + xdst);
        }

        float4v acc[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};

        auto multiply = [&](const uint4 (&a)[8], uint32_t buf) {
            const uint16_t* sl = slab + buf * kSlab;
#pragma unroll
            for (int s = 0; s < 8; ++s) {
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const uint4 bfrag = *reinterpret_cast<const uint4*>(sl + boff[s] + t * 16 * kSlabLd);
                    acc[t] = mfma16<DT>(a[s], bfrag, acc[t]);
                }
            }
        };

        uint32_t b = 0;
        // Full rings, straight-line: a load that would run past the row re-reads the
        // last super-block / slab instead (a cache hit that is never used), so the
        // loop body has no branch and the outstanding-load counts stay exact.
        for (; b + kRing <= nb; b += kRing) {
#pragma unroll
            for (int i = 0; i < kRing; ++i) {
                const uint32_t j = b + i;
                __syncthreads();
                // keep the scheduler from pulling a later super-block's decode up to here:
                // it would have to wait for that block's loads and drain the ring
                __builtin_amdgcn_sched_barrier(0);
                xr[i].store(slab + ((j + 1) & 1u) * kSlab + xdst);
                xr[i].load(rows, 256 * (size_t)min(j + 1 + kRing, last));
                uint4 a[8];
                ring[i].template decode<DT>(g, a);
                ring[i].load(wrow + (size_t)min(j + kRing, last) * kBB, g);
                multiply(a, j & 1u);
            }
        }
        // the nb % kRing super-blocks left over are already in registers
#pragma unroll
        for (int i = 0; i < kRing - 1; ++i) {
            const uint32_t j = b + i;
            if (j < nb) {
                __syncthreads();
                xr[i].store(slab + ((j + 1) & 1u) * kSlab + xdst);
                uint4 a[8];
                ring[i].template decode<DT>(g, a);
                multiply(a, j & 1u);
            }
        }

        // C layout of 16x16x32: acc[t][v] = (weight row 4g + v, token 16t + r)
        const uint32_t out_row = row0 + 4 * g;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            const uint32_t tok = 16 * t + r;
            if (tok >= mt) continue;
            uint32_t token = first_token + t0 + tok;
            if constexpr (GROUPED) token = order != nullptr ? order[token] : token;
            const size_t base = (size_t)token * n + out_row;
            if (y_dtype == FH_F32 && (n & 3u) == 0 && out_row + 3 < n) {
                *reinterpret_cast<float4*>(static_cast<float*>(y) + base) =
                    make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (out_row + v < n) store_from_f32(y, base + v, y_dtype, acc[t][v]);
            }
        }
    }
}

// Routed-expert projection with the expert's activations resident in LDS.
// When an expert's tokens (16*TT of them at a time) fit LDS for the whole K, a
// workgroup gathers them once and then streams weight rows past them with no
// further barrier: wave w takes row tiles w, w+4, ... of the workgroup's share
// and walks (tile, super-block) units through a register ring, so the prefetch
// runs across tile boundaries.  blockIdx.y = expert, blockIdx.x = which share
// of the expert's rows.  Dynamic LDS: 16*TT rows of K halfs.
//
// The rows are [A, K] rows or, with metadata given, the row of the assignment's
// token in [tokens, K]: expert_assign folded into the gather.  (SiLU * up is not
// folded in: it is bound by its exponentials and divisions, and one workgroup
// per compute unit doing them ahead of its first MFMA costs more than the
// launch that spreads them over the whole chip: +11 us against -5 us.)
constexpr size_t kResLdsBytes = 160u * 1024;   // a workgroup may take all of a compute unit's LDS
constexpr int kResRing = 6;
constexpr int kResWaves = 8;                    // two waves per SIMD hide each other's decode and MFMA waits
constexpr int kResThreads = 64 * kResWaves;

// A shared expert in the same launch: every token also runs the dense matrix w [n, k];
// token t reads row t of x (null: row t of the routed x, which then holds token rows) and
// writes row t of y.  Its work is cut into pieces of 16*TT consecutive tokens times
// tiles_per_slice row tiles, `slices` of them per token group, and the workgroups share the
// pieces out after their own expert, so the grid and its one round of workgroups stay as
// they are.
struct ResidentShared {
    const uint8_t* w;
    const uint16_t* x;
    void* y;
    uint32_t tokens;
    uint32_t slices;
    uint32_t tiles_per_slice;
};

// Copies `mt` activation rows into LDS for the resident kernels: row `tok` of the item to
// xs[tok * ld ..], its 16-byte pieces swizzled by the row's low four bits; eight pieces per thread
// in flight at a time.  The row behind a slot is found through up to two tables (the expert-sorted
// order, then the assignment's token).  All eight pieces look their rows up together, table by
// table, before any row is read: a round trip per table and one for the rows, where piece after
// piece would chain up to twenty-four.
__device__ __forceinline__ void gather_rows(uint16_t* xs, const uint16_t* __restrict__ xsrc, uint32_t mt,
                                            uint32_t pieces, uint32_t k, uint32_t ld, uint32_t first_token,
                                            const uint32_t* __restrict__ order, const float* __restrict__ metadata,
                                            uint32_t x_rows, uint32_t tid) {
    const uint32_t total = mt * pieces;
    for (uint32_t base = 0; base < total; base += 8 * kResThreads) {
        u32x4 v[8];
        uint32_t dst[8], row[8], pc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t idx = min(base + j * kResThreads + tid, total - 1);
            const uint32_t tok = idx / pieces;
            pc[j] = idx - tok * pieces;
            dst[j] = tok * ld + 8 * (pc[j] ^ (tok & 15u));
            row[j] = first_token + tok;  // without tables a slot is its row
        }
        if (order != nullptr) {
#pragma unroll
            for (int j = 0; j < 8; ++j) row[j] = order[row[j]];
        }
        if (metadata != nullptr) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t token = __float_as_uint(metadata[3 * (size_t)row[j] + 1]);
                row[j] = token < x_rows ? token : x_rows - 1;
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const u32x4*>(xsrc + (size_t)row[j] * k + 8 * (size_t)pc[j]);
#pragma unroll
        for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(xs + dst[j]) = v[j];
    }
}

template <uint32_t TYPE, int DT, int TT>
__global__ __launch_bounds__(kResThreads) void expert_resident_kernel(const uint8_t* __restrict__ w,
                                                                     const uint16_t* __restrict__ x,
                                                                     void* __restrict__ y, uint32_t n,
                                                                     uint32_t nb, uint32_t y_dtype,
                                                                     const uint32_t* __restrict__ offsets,
                                                                     const uint32_t* __restrict__ order,
                                                                     uint32_t tiles_per_wg,
                                                                     const float* __restrict__ metadata,
                                                                     uint32_t x_rows, uint32_t routes,
                                                                     const ResidentShared sh) {
    constexpr uint32_t kBB = Quarter<TYPE>::kBlockBytes;
    constexpr int kTokens = 16 * TT;
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t r = lane & 15u, g = lane >> 4;
    // Rows are not padded: 16 rows of 5120 halves are all of LDS.  The 16-byte piece p of row t
    // sits at piece p ^ (t & 15) instead, so the sixteen rows a B-operand read touches at one k
    // (and the sixteen consecutive pieces a gather write covers) fall on different banks.
    const uint32_t k = nb * 256, ld = k;
    // no offsets: a dense product, all of it shared-expert pieces
    // a damaged offsets table reads wrong rows, never rows outside the `routes` assignments
    const uint32_t expert_first = offsets != nullptr ? min(offsets[blockIdx.y], routes) : 0;
    const uint32_t expert_upto = offsets != nullptr ? min(offsets[blockIdx.y + 1], routes) : 0;
    const uint32_t count = expert_upto > expert_first ? expert_upto - expert_first : 0;
    const uint32_t tiles = (n + 15) / 16;
    const uint32_t pieces = k / 8;  // 16-byte pieces per activation row

    // work items of this workgroup: its expert's tokens, 16*TT at a time, then its part of
    // the shared expert's pieces
    const uint32_t passes = (count + kTokens - 1) / kTokens;
    const uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x, wgs = gridDim.x * gridDim.y;
    const uint32_t shared_pieces = sh.w != nullptr ? (sh.tokens + kTokens - 1) / kTokens * sh.slices : 0;
    const uint32_t my_pieces = shared_pieces > wg ? (shared_pieces - wg + wgs - 1) / wgs : 0;
    for (uint32_t item = 0; item < passes + my_pieces; ++item) {
        const bool shared = item >= passes;  // uniform over the workgroup
        uint32_t first_token, mt, tile_begin, tile_end;
        if (!shared) {
            first_token = expert_first + item * kTokens;
            mt = min((uint32_t)kTokens, count - item * kTokens);
            tile_begin = blockIdx.x * tiles_per_wg + wave;
            tile_end = min(tiles, (blockIdx.x + 1) * tiles_per_wg);
        } else {
            const uint32_t piece = wg + (item - passes) * wgs;
            const uint32_t group = piece / sh.slices, slice = piece - group * sh.slices;
            first_token = group * kTokens;
            mt = min((uint32_t)kTokens, sh.tokens - first_token);
            tile_begin = slice * sh.tiles_per_slice + wave;
            tile_end = min(tiles, (slice + 1) * sh.tiles_per_slice);
        }
        const uint8_t* wexpert = shared ? sh.w : w + (size_t)blockIdx.y * n * nb * kBB;
        const uint16_t* xsrc = shared && sh.x != nullptr ? sh.x : x;
        void* ydst = shared ? sh.y : y;
        if (item != 0) __syncthreads();  // the previous item is done with the rows
        gather_rows(xs, xsrc, mt, pieces, k, ld, first_token, shared ? nullptr : order, shared ? nullptr : metadata,
                    x_rows, tid);
        __syncthreads();
        if (tile_begin >= tile_end) continue;  // uniform per wave; no barrier follows in this item

        // B operand rows: token 16t + r, clamped (columns past mt are never stored)
        uint32_t boff[TT];
        uint32_t out_token[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            const uint32_t tok = min(16u * t + r, mt - 1);
            boff[t] = tok * ld;
            out_token[t] = order != nullptr && !shared ? order[first_token + tok] : first_token + tok;
        }
        uint32_t kl[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) kl[s] = (((Quarter<TYPE>::klocal(g, s) >> 3) ^ r) << 3);  // row 16t + r: swizzle r

        // units = (tile, super-block) pairs of this wave, in order
        const uint32_t my_tiles = (tile_end - tile_begin + kResWaves - 1) / kResWaves;
        const uint32_t units = my_tiles * nb;
        auto unit_ptr = [&](uint32_t tile, uint32_t b) {
            const uint32_t row = min(tile * 16 + r, n - 1);
            return wexpert + ((size_t)row * nb + b) * kBB;
        };
        Quarter<TYPE> ring[kResRing];
        uint32_t ptile = tile_begin, pb = 0;  // next unit to prefetch
        auto prefetch = [&](Quarter<TYPE>& slot) {
            slot.load(unit_ptr(min(ptile, tile_end - 1), pb), g);
            if (++pb == nb) {
                pb = 0;
                ptile += kResWaves;
            }
        };
#pragma unroll
        for (int i = 0; i < kResRing; ++i) {
            prefetch(ring[i]);
            __builtin_amdgcn_sched_barrier(0);
        }

        float4v acc[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
        uint32_t tile = tile_begin, b = 0;
        auto consume = [&](Quarter<TYPE>& slot) {
            uint4 a[8];
            slot.template decode<DT>(g, a);
            prefetch(slot);
            const uint16_t* xb = xs + 256 * b;
#pragma unroll
            for (int s = 0; s < 8; ++s) {
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const uint4 bfrag = *reinterpret_cast<const uint4*>(xb + boff[t] + kl[s]);
                    acc[t] = mfma16<DT>(a[s], bfrag, acc[t]);
                }
            }
            if (++b == nb) {
                // C layout of 16x16x32: acc[t][v] = (weight row 4g + v, token 16t + r)
                const uint32_t out_row = tile * 16 + 4 * g;
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    if (16u * t + r < mt) {
                        const size_t base = (size_t)out_token[t] * n + out_row;
                        if (y_dtype == FH_F32 && (n & 3u) == 0 && out_row + 3 < n) {
                            *reinterpret_cast<float4*>(static_cast<float*>(ydst) + base) =
                                make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
                        } else if (y_dtype != FH_F32 && (n & 3u) == 0 && out_row + 3 < n) {
                            uint2 packed;
                            if (y_dtype == FH_F16) {
                                packed.x = f32_to_f16_bits(acc[t][0]) | (f32_to_f16_bits(acc[t][1]) << 16);
                                packed.y = f32_to_f16_bits(acc[t][2]) | (f32_to_f16_bits(acc[t][3]) << 16);
                            } else {
                                packed.x = f32_to_bf16_bits(acc[t][0]) | (f32_to_bf16_bits(acc[t][1]) << 16);
                                packed.y = f32_to_bf16_bits(acc[t][2]) | (f32_to_bf16_bits(acc[t][3]) << 16);
                            }
                            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(ydst) + base) = packed;
                        } else {
#pragma unroll
                            for (int v = 0; v < 4; ++v)
                                if (out_row + v < n) store_from_f32(ydst, base + v, y_dtype, acc[t][v]);
                        }
                    }
                    acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
                }
                b = 0;
                tile += kResWaves;
            }
        };
        uint32_t u = 0;
        for (; u + kResRing <= units; u += kResRing) {
#pragma unroll
            for (int i = 0; i < kResRing; ++i) {
                __builtin_amdgcn_sched_barrier(0);
                consume(ring[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < kResRing - 1; ++i)
            if (u + i < units) consume(ring[i]);
    }
}

// expert_resident_kernel with the weights going through LDS.  Loading weights straight into the
// MFMA operand layout puts sixteen different rows under sixteen neighbouring lanes, and the vector
// L1 then looks up one line per lane: the weight stream of that kernel stops at 3.4 TB/s.  A 16-row
// tile of weights is one contiguous run of 16 x nb x 144 bytes, so here every wave copies its tiles
// into a ring of LDS slots of its own with LDS-direct loads -- whole kilobytes per instruction, the
// next tiles on their way while this one is multiplied -- and the lanes pick their header and their
// chunk's quants out of LDS.  It needs room for the rings beside the token rows (rows of up to
// ~1024 weights for 32 tokens), and n a multiple of 16 (a tile is read whole).  Q4_K and Q6_K (a
// tile of either is a whole number of 16-byte pieces at a 16-byte aligned address).
template <uint32_t TYPE, int DT, int TT, int NB>
__global__ __launch_bounds__(kResThreads) void expert_ring_kernel(const uint8_t* __restrict__ w,
                                                                 const uint16_t* __restrict__ x,
                                                                 void* __restrict__ y, uint32_t n,
                                                                 uint32_t nb, uint32_t y_dtype,
                                                                 const uint32_t* __restrict__ offsets,
                                                                 const uint32_t* __restrict__ order,
                                                                 uint32_t tiles_per_wg,
                                                                 const float* __restrict__ metadata,
                                                                 uint32_t x_rows, uint32_t routes,
                                                                 const ResidentShared sh, uint32_t ring_tiles) {
    constexpr uint32_t kBB = Quarter<TYPE>::kBlockBytes;
    constexpr int kTokens = 16 * TT;
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint32_t k = nb * 256, ld = k;
    const uint32_t expert_first = offsets != nullptr ? min(offsets[blockIdx.y], routes) : 0;
    const uint32_t expert_upto = offsets != nullptr ? min(offsets[blockIdx.y + 1], routes) : 0;
    const uint32_t count = expert_upto > expert_first ? expert_upto - expert_first : 0;
    const uint32_t tiles = n / 16;
    const uint32_t pieces = k / 8;  // 16-byte pieces per activation row
    // a tile of weights: 16 rows x nb super-blocks, contiguous; its ring slot, in whole kilobytes of requests
    const uint32_t tile_bytes = 16u * nb * kBB, per_tile = (tile_bytes + 1023u) >> 10;
    uint8_t* const ring = reinterpret_cast<uint8_t*>(xs) + (size_t)kTokens * k * 2 + (size_t)wave * ring_tiles * tile_bytes;
    const uint32_t ring_addr = (uint32_t)(uintptr_t)ring;

    const uint32_t passes = (count + kTokens - 1) / kTokens;
    const uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x, wgs = gridDim.x * gridDim.y;
    const uint32_t shared_pieces = sh.w != nullptr ? (sh.tokens + kTokens - 1) / kTokens * sh.slices : 0;
    const uint32_t my_pieces = shared_pieces > wg ? (shared_pieces - wg + wgs - 1) / wgs : 0;
    for (uint32_t item = 0; item < passes + my_pieces; ++item) {
        const bool shared = item >= passes;  // uniform over the workgroup
        uint32_t first_token, mt, tile_begin, tile_end;
        if (!shared) {
            first_token = expert_first + item * kTokens;
            mt = min((uint32_t)kTokens, count - item * kTokens);
            tile_begin = blockIdx.x * tiles_per_wg + wave;
            tile_end = min(tiles, (blockIdx.x + 1) * tiles_per_wg);
        } else {
            const uint32_t piece = wg + (item - passes) * wgs;
            const uint32_t group = piece / sh.slices, slice = piece - group * sh.slices;
            first_token = group * kTokens;
            mt = min((uint32_t)kTokens, sh.tokens - first_token);
            tile_begin = slice * sh.tiles_per_slice + wave;
            tile_end = min(tiles, (slice + 1) * sh.tiles_per_slice);
        }
        const uint8_t* wexpert = shared ? sh.w : w + (size_t)blockIdx.y * n * nb * kBB;
        const uint16_t* xsrc = shared && sh.x != nullptr ? sh.x : x;
        void* ydst = shared ? sh.y : y;
        if (item != 0) __syncthreads();  // the previous item is done with the rows
        // this wave's tiles: tile_begin, tile_begin + 8, ..; the first ones are requested once the rows are
        // in LDS (the gather's own loads are the compiler's, and nothing of its may stand between a
        // request and the wait that counts it)
        const uint32_t my_tiles = tile_begin < tile_end ? (tile_end - tile_begin + kResWaves - 1) / kResWaves : 0;
        uint32_t requested = 0;
        auto request_tile = [&]() {
            const uint8_t* const base = wexpert + (size_t)(tile_begin + requested * kResWaves) * tile_bytes;
            const uint32_t slot_addr = ring_addr + (requested % ring_tiles) * tile_bytes;
            for (uint32_t c = 0; c < per_tile; ++c) {
                if (c * 1024u + lane * 16u < tile_bytes) lds_load16_at(base + c * 1024u, lane * 16u, slot_addr + c * 1024u);
            }
            ++requested;
        };
        gather_rows(xs, xsrc, mt, pieces, k, ld, first_token, shared ? nullptr : order, shared ? nullptr : metadata,
                    x_rows, tid);
        __syncthreads();
        if (my_tiles == 0) continue;  // uniform per wave; no barrier follows in this item

        // B operand rows: token 16t + r, clamped (columns past mt are never stored)
        uint32_t boff[TT];
        uint32_t out_token[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) {
            const uint32_t tok = min(16u * t + r, mt - 1);
            boff[t] = tok * ld;
            out_token[t] = order != nullptr && !shared ? order[first_token + tok] : first_token + tok;
        }
        // (the loads above are the last of the compiler's before the requests: it waits for them here,
        // where nothing of this wave's is in flight)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int t = 0; t < TT; ++t) asm volatile("" : "+v"(out_token[t]));
        while (requested < my_tiles && requested < ring_tiles) request_tile();
        uint32_t kl[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) kl[s] = (((Quarter<TYPE>::klocal(g, s) >> 3) ^ r) << 3);  // row 16t + r: swizzle r

        // Every tile multiplies the same token rows.  Where they fit the wave's registers (two waves a
        // SIMD leave each 256) the B operands are read out of LDS once per item and not once per tile:
        // read per tile they are 16 KB per wave and super-block, more LDS traffic than the weights
        // (32 registers per super-block and 16 tokens)
        constexpr bool kRowsInRegisters = NB * TT <= 4 && TYPE == kQ4K;
        uint4 brow[kRowsInRegisters ? NB * 8 * TT : 1];
        if constexpr (kRowsInRegisters) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int s = 0; s < 8; ++s)
#pragma unroll
                    for (int t = 0; t < TT; ++t)
                        brow[(b * 8 + s) * TT + t] = *reinterpret_cast<const uint4*>(xs + 256 * b + boff[t] + kl[s]);
        }

        float4v acc[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
        // lane (r, g) finds row r of a slot at r x nb x 144
        const uint32_t lane_row = r * nb * kBB;
        for (uint32_t i = 0; i < my_tiles; ++i) {
            const uint32_t tile = tile_begin + i * kResWaves;
            // requests retire in issue order: behind tile i's stand those of the tiles asked for since
            wait_vmcnt((requested - 1u - i) * per_tile);
            const uint8_t* const slot = ring + (i % ring_tiles) * tile_bytes + lane_row;
            // the whole tile (NB super-blocks of the lane's row) leaves its slot at once, and the slot
            // is asked for the tile `ring_tiles` places ahead before anything is multiplied: a slot is
            // out of flight for one LDS round trip, not for a tile's arithmetic.  (Reading tile i + 1
            // out of LDS while tile i is multiplied takes that round trip out of the wave's way too and
            // changes nothing: the kernel is bound by its decode arithmetic.)
            Quarter<TYPE> q[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) q[b].load(slot + b * kBB, g);
            if (requested < my_tiles) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                request_tile();
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                uint4 a[8];
                q[b].template decode<DT>(g, a);
                const uint16_t* xb = xs + 256 * b;
#pragma unroll
                for (int s = 0; s < 8; ++s) {
#pragma unroll
                    for (int t = 0; t < TT; ++t) {
                        uint4 bfrag;
                        if constexpr (kRowsInRegisters) bfrag = brow[(b * 8 + s) * TT + t];
                        else bfrag = *reinterpret_cast<const uint4*>(xb + boff[t] + kl[s]);
                        acc[t] = mfma16<DT>(a[s], bfrag, acc[t]);
                    }
                }
            }
            // C layout of 16x16x32: acc[t][v] = (weight row 4g + v, token 16t + r)
            const uint32_t out_row = tile * 16 + 4 * g;
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                if (16u * t + r < mt) {
                    const size_t base = (size_t)out_token[t] * n + out_row;
                    if (y_dtype == FH_F32) {
                        *reinterpret_cast<float4*>(static_cast<float*>(ydst) + base) =
                            make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
                    } else {
                        uint2 packed;
                        if (y_dtype == FH_F16) {
                            packed.x = f32_to_f16_bits(acc[t][0]) | (f32_to_f16_bits(acc[t][1]) << 16);
                            packed.y = f32_to_f16_bits(acc[t][2]) | (f32_to_f16_bits(acc[t][3]) << 16);
                        } else {
                            packed.x = f32_to_bf16_bits(acc[t][0]) | (f32_to_bf16_bits(acc[t][1]) << 16);
                            packed.y = f32_to_bf16_bits(acc[t][2]) | (f32_to_bf16_bits(acc[t][3]) << 16);
                        }
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(ydst) + base) = packed;
                    }
                }
                acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
            }
        }
        // (the last tile's wait left none of this wave's requests in flight; said where the next
        // item's loads can see it)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}

// Dense product of up to 16 activation rows where a workgroup owns only a few 16-row weight
// tiles (up to kFewTiles of them).  In expert_resident_kernel a wave walks whole tiles, so with
// five tiles per workgroup five waves each stream twenty super-blocks one after another and
// three idle: the length of that chain, not the memory system, sets the time.  Here the
// super-blocks of every tile are dealt over the waves (wave w takes blocks w, w + WAVES, .. of
// tile 0, shifted by four for the next tile so the odd ones even out), every wave keeps one
// accumulator per tile, and the partial sums of a tile meet in LDS, where the activation rows
// were, once nobody reads those any more; they are added in wave order, so the result is
// deterministic.  The first weight loads are issued before the activation rows are fetched.
constexpr int kFewTiles = 5;        // tiles per workgroup

// WAVES: 8 or 16 per workgroup; every wave takes up to 24 / WAVES super-blocks of each tile (rows
// of up to 24 super-blocks: more do not fit LDS anyway).  AHEAD: units in flight per wave.
template <uint32_t TYPE, int DT, int WAVES, int AHEAD>
__global__ __launch_bounds__(64 * WAVES) void dense_few_tiles_kernel(const uint8_t* __restrict__ w,
                                                                    const uint16_t* __restrict__ x,
                                                                    void* __restrict__ y, uint32_t m, uint32_t n,
                                                                    uint32_t nb, uint32_t y_dtype) {
    constexpr uint32_t kBB = Quarter<TYPE>::kBlockBytes;
    constexpr int kPerTile = 24 / WAVES + (24 % WAVES != 0 ? 1 : 0);
    constexpr int kUnits = kFewTiles * kPerTile;
    constexpr uint32_t kThreads = 64 * WAVES;
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint32_t k = nb * 256, ld = k, pieces = k / 8;
    const uint32_t tiles = (n + 15) / 16;
    const uint32_t per = (tiles + gridDim.x - 1) / gridDim.x;
    const uint32_t tile_begin = blockIdx.x * per;
    const uint32_t my_tiles = min(per, tiles - tile_begin);

    // unit i = (tile i / kPerTile, the (i % kPerTile)-th block of this wave in that tile)
    auto unit_block = [&](int i) {
        return ((wave + 4u * (uint32_t)(i / kPerTile)) & (uint32_t)(WAVES - 1)) + (uint32_t)WAVES * (uint32_t)(i % kPerTile);
    };
    auto unit_valid = [&](int i) { return (uint32_t)(i / kPerTile) < my_tiles && unit_block(i) < nb; };
    auto unit_ptr = [&](int i) {
        const uint32_t tile = tile_begin + min((uint32_t)(i / kPerTile), my_tiles - 1);
        const uint32_t row = min(tile * 16 + r, n - 1);
        return w + ((size_t)row * nb + min(unit_block(i), nb - 1)) * kBB;
    };
    // The activation rows, eight 16-byte pieces per thread in flight at a time; piece p of row
    // t sits at piece p ^ (t & 15), so the sixteen rows a B-operand read touches fall on different
    // banks.  The first pieces are requested first and the first weights right behind them: loads
    // return in order, the rows come from L2 (every workgroup reads the same ones) and are in LDS
    // while the weights are still on their way from memory.
    Quarter<TYPE> ring[AHEAD + 1];
    const uint32_t total = m * pieces;
    for (uint32_t base = 0; base < total; base += 8 * kThreads) {
        u32x4 v[8];
        uint32_t dst[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t idx = min(base + j * kThreads + tid, total - 1);
            const uint32_t tok = idx / pieces, pc = idx - tok * pieces;
            dst[j] = tok * ld + 8 * (pc ^ (tok & 15u));
            v[j] = *reinterpret_cast<const u32x4*>(x + (size_t)tok * k + 8 * pc);
        }
        if (base == 0) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < AHEAD; ++i) {
                if (unit_valid(i)) ring[i].load(unit_ptr(i), g);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(xs + dst[j]) = v[j];
    }
    __syncthreads();

    const uint32_t boff = min(r, m - 1) * ld;
    uint32_t kl[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) kl[s] = (((Quarter<TYPE>::klocal(g, s) >> 3) ^ r) << 3);
    float4v acc[kFewTiles];
#pragma unroll
    for (int t = 0; t < kFewTiles; ++t) acc[t] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < kUnits; ++i) {
        __builtin_amdgcn_sched_barrier(0);
        if (i + AHEAD < kUnits) {
            if (unit_valid(i + AHEAD)) ring[(i + AHEAD) % (AHEAD + 1)].load(unit_ptr(i + AHEAD), g);
        }
        if (unit_valid(i)) {
            uint4 a[8];
            ring[i % (AHEAD + 1)].template decode<DT>(g, a);
            const uint16_t* xb = xs + 256 * unit_block(i) + boff;
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const uint4 bfrag = *reinterpret_cast<const uint4*>(xb + kl[s]);
                acc[i / kPerTile] = mfma16<DT>(a[s], bfrag, acc[i / kPerTile]);
            }
        }
    }
    // the partial sums take the place of the activation rows
    __syncthreads();
    float4* partial = reinterpret_cast<float4*>(xs);
#pragma unroll
    for (int t = 0; t < kFewTiles; ++t)
        if ((uint32_t)t < my_tiles) partial[((uint32_t)t * WAVES + wave) * 64 + lane] = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
    __syncthreads();
    for (uint32_t idx = tid; idx < my_tiles * 64; idx += kThreads) {
        const uint32_t t = idx >> 6, l = idx & 63u;
        float4 sum = partial[(t * WAVES) * 64 + l];
#pragma unroll
        for (int wv = 1; wv < WAVES; ++wv) {
            const float4 v = partial[(t * WAVES + wv) * 64 + l];
            sum.x += v.x;
            sum.y += v.y;
            sum.z += v.z;
            sum.w += v.w;
        }
        // C layout of 16x16x32: lane (g, r) holds weight rows 4g .. 4g + 3 of token r
        const uint32_t token = l & 15u, out_row = (tile_begin + t) * 16 + 4 * (l >> 4);
        if (token < m) {
            const size_t base = (size_t)token * n + out_row;
            const float vals[4] = {sum.x, sum.y, sum.z, sum.w};
            if (y_dtype == FH_F32 && (n & 3u) == 0 && out_row + 3 < n) {
                *reinterpret_cast<float4*>(static_cast<float*>(y) + base) = sum;
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (out_row + v < n) store_from_f32(y, base + v, y_dtype, vals[v]);
            }
        }
    }
}

template <uint32_t TYPE, int DT>
void launch_tt(hipStream_t s, const GemmArgs& a) {
    const uint8_t* w = static_cast<const uint8_t*>(a.w);
    const uint16_t* x = static_cast<const uint16_t*>(a.x);
    const uint32_t nb = a.k / 256;
    if (a.use_resident && a.m <= 16 && a.few_tiles_split && nb <= 24u) {
        const uint32_t tiles = (a.n + 15) / 16;
        const uint32_t cus = a.cu_count > 0 ? (uint32_t)a.cu_count : 256u;
        const uint32_t per_wg = (tiles + cus - 1) / cus;
        if (per_wg <= (uint32_t)kFewTiles) {
            auto go = [&](auto kernel, uint32_t waves) {
                const size_t rows_bytes = (size_t)a.m * a.k * 2, partial_bytes = (size_t)per_wg * waves * 64 * 16;
                const size_t lds = rows_bytes > partial_bytes ? rows_bytes : partial_bytes;
                (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                hipLaunchKernelGGL(kernel, dim3((tiles + per_wg - 1) / per_wg), dim3(64 * waves), lds, s, w, x, a.y,
                                   a.m, a.n, nb, a.y_dtype);
            };
            // Sixteen waves with two units ahead where a tile has two super-blocks or more per
            // wave of eight and the format's raw quarter is small enough for 128 registers
            // (8 x 17408 x 5120 Q4_K: 17.4 us against 19.9 with eight waves and six ahead, 24.3
            // with whole tiles per wave; one or three units ahead, or 256 workgroups of four or
            // five tiles instead of 218 of five, each cost 0.5 - 1.5 us; Q5_K and Q6_K spill
            // there: 26.2 against 32.3 and 30.9 against 36.9 with eight waves); eight waves for
            // shorter rows (8 x 4096 x 2048: 4.9 against 5.3 and 7.9).
            if constexpr (TYPE == kQ5K || TYPE == kQ6K) {
                go(dense_few_tiles_kernel<TYPE, DT, 8, 4>, 8);
            } else if constexpr (DT != 1) {
                go(dense_few_tiles_kernel<TYPE, DT, 8, 6>, 8);  // the bf16 rounding needs more registers than 16 waves leave
            } else {
                if (nb >= 16) go(dense_few_tiles_kernel<TYPE, DT, 16, 2>, 16);
                else go(dense_few_tiles_kernel<TYPE, DT, 8, 6>, 8);
            }
            return;
        }
    }
    if (a.use_resident) {
        // dense product with the activation rows resident in LDS: (32-row group, row-tile slice)
        // pieces, about one per compute unit
        const bool wide = a.m > 16 && (size_t)32 * a.k * 2 <= kResLdsBytes;
        const uint32_t per_group = wide ? 32u : 16u;
        const size_t lds = (size_t)per_group * a.k * 2;
        const uint32_t tiles = (a.n + 15) / 16;
        const uint32_t cus = a.cu_count > 0 ? (uint32_t)a.cu_count : 256u;
        const uint32_t groups = (a.m + per_group - 1) / per_group;
        // never a few pieces more than workgroups: those would make a second round
        const uint32_t want = cus / groups > 0 ? cus / groups : 1;
        ResidentShared sh{};
        sh.w = w;
        sh.x = nullptr;
        sh.y = a.y;
        sh.tokens = a.m;
        sh.tiles_per_slice = (tiles + want - 1) / want;
        sh.slices = (tiles + sh.tiles_per_slice - 1) / sh.tiles_per_slice;
        const uint32_t pieces = groups * sh.slices;
        const dim3 rgrid(pieces < cus ? pieces : cus, 1);
        if (wide) {
            auto kernel = expert_resident_kernel<TYPE, DT, 2>;
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            hipLaunchKernelGGL(kernel, rgrid, dim3(kResThreads), lds, s, nullptr, x, nullptr, a.n, nb, a.y_dtype,
                               nullptr, nullptr, 0u, nullptr, 0u, 0u, sh);
        } else {
            auto kernel = expert_resident_kernel<TYPE, DT, 1>;
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            hipLaunchKernelGGL(kernel, rgrid, dim3(kResThreads), lds, s, nullptr, x, nullptr, a.n, nb, a.y_dtype,
                               nullptr, nullptr, 0u, nullptr, 0u, 0u, sh);
        }
        return;
    }
    if (a.expert_offsets != nullptr) {
        const bool wide = a.m > 8 * a.experts;   // mean tokens per expert > 8: 32 tokens a pass
        const size_t lds = (size_t)(wide ? 32 : 16) * a.k * 2;
        if (expert_rows_fit_lds(a.k, a.m, a.experts)) {
            // the expert's rows are cut into shares so that about one workgroup per compute unit
            // exists: every share gathers the expert's tokens again, and at 256 experts one share
            // each (236 us for the 512-token routed FFN) beats four (264 us)
            const uint32_t tiles = (a.n + 15) / 16;
            const uint32_t target = a.cu_count > 0 ? (uint32_t)a.cu_count : 256u;
            uint32_t shares = (target + a.experts - 1) / a.experts;
            shares = shares < 1 ? 1 : shares;
            uint32_t tiles_per_wg = (tiles + shares - 1) / shares;
            tiles_per_wg = (tiles_per_wg + kResWaves - 1) / kResWaves * kResWaves;
            const dim3 rgrid((tiles + tiles_per_wg - 1) / tiles_per_wg, a.experts);
            ResidentShared sh{};
            if (a.shared_w != nullptr) {
                sh.w = static_cast<const uint8_t*>(a.shared_w);
                sh.x = static_cast<const uint16_t*>(a.shared_x);
                sh.y = a.shared_y;
                sh.tokens = a.shared_rows;
                // about one piece per workgroup: a token group's rows are cut into as many slices
                const uint32_t per_group = wide ? 32u : 16u;
                const uint32_t groups = (a.shared_rows + per_group - 1) / per_group;
                const uint32_t want = rgrid.x * rgrid.y / groups > 0 ? rgrid.x * rgrid.y / groups : 1;
                sh.tiles_per_slice = (tiles + want - 1) / want;
                sh.slices = (tiles + sh.tiles_per_slice - 1) / sh.tiles_per_slice;
            }
            // weights through rings in LDS where those fit beside the rows (short rows: the down projections)
            // (Q4_K 49 against 55 us and Q6_K 74 against 77 for 256 experts x 2048 x 512 over 4096 rows; IQ4_XS,
            // whose rows' operands do not fit the registers beside its decode, 62 either way: it stays)
            if constexpr (TYPE == kQ4K || TYPE == kQ6K) {
                const size_t tile_bytes = (size_t)16 * nb * Quarter<TYPE>::kBlockBytes;
                const size_t room = kResLdsBytes > lds ? (kResLdsBytes - lds) / (kResWaves * tile_bytes) : 0;
                const uint32_t ring_tiles = room >= 3 ? 3u : (uint32_t)room;
                if (a.weight_ring && a.n % 16 == 0 && nb <= 4 && ring_tiles >= 2) {
                    const size_t ring_lds = lds + kResWaves * ring_tiles * tile_bytes;
                    typedef void (*Ring)(const uint8_t*, const uint16_t*, void*, uint32_t, uint32_t, uint32_t, const uint32_t*,
                                         const uint32_t*, uint32_t, const float*, uint32_t, uint32_t, const ResidentShared,
                                         uint32_t);
                    static const Ring rings[2][4] = {
                        {expert_ring_kernel<TYPE, DT, 1, 1>, expert_ring_kernel<TYPE, DT, 1, 2>, expert_ring_kernel<TYPE, DT, 1, 3>,
                         expert_ring_kernel<TYPE, DT, 1, 4>},
                        {expert_ring_kernel<TYPE, DT, 2, 1>, expert_ring_kernel<TYPE, DT, 2, 2>, expert_ring_kernel<TYPE, DT, 2, 3>,
                         expert_ring_kernel<TYPE, DT, 2, 4>}};
                    const Ring kernel = rings[wide ? 1 : 0][nb - 1];
                    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)ring_lds);
                    hipLaunchKernelGGL(kernel, rgrid, dim3(kResThreads), ring_lds, s, w, x, a.y, a.n, nb, a.y_dtype,
                                       a.expert_offsets, a.expert_order, tiles_per_wg, a.gather_metadata, a.x_rows, a.m, sh,
                                       ring_tiles);
                    return;
                }
            }
            if (wide) {
                auto kernel = expert_resident_kernel<TYPE, DT, 2>;
                (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                hipLaunchKernelGGL(kernel, rgrid, dim3(kResThreads), lds, s, w, x, a.y, a.n, nb, a.y_dtype,
                                   a.expert_offsets, a.expert_order, tiles_per_wg, a.gather_metadata, a.x_rows, a.m, sh);
            } else {
                auto kernel = expert_resident_kernel<TYPE, DT, 1>;
                (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                hipLaunchKernelGGL(kernel, rgrid, dim3(kResThreads), lds, s, w, x, a.y, a.n, nb, a.y_dtype,
                                   a.expert_offsets, a.expert_order, tiles_per_wg, a.gather_metadata, a.x_rows, a.m, sh);
            }
            return;
        }
        const dim3 grid((a.n + kSkRows - 1) / kSkRows, a.experts);
        if (!wide) {
            hipLaunchKernelGGL((gemm_skinny_kernel<TYPE, DT, 1, true>), grid, dim3(kSkThreads), 0, s, w, x,
                               a.y, a.m, a.n, nb, a.y_dtype, a.expert_offsets, a.expert_order);
        } else {
            hipLaunchKernelGGL((gemm_skinny_kernel<TYPE, DT, 2, true>), grid, dim3(kSkThreads), 0, s, w, x,
                               a.y, a.m, a.n, nb, a.y_dtype, a.expert_offsets, a.expert_order);
        }
        return;
    }
    const dim3 grid((a.n + kSkRows - 1) / kSkRows);
    if (a.m <= 16) {
        hipLaunchKernelGGL((gemm_skinny_kernel<TYPE, DT, 1, false>), grid, dim3(kSkThreads), 0, s, w, x, a.y,
                           a.m, a.n, nb, a.y_dtype, nullptr, nullptr);
    } else if (a.m > 32) {
        auto kernel = gemm_skinny_kernel<TYPE, DT, 4, false>;
        hipLaunchKernelGGL(kernel, grid, dim3(kSkThreads), 0, s, w, x, a.y, a.m, a.n, nb, a.y_dtype, nullptr,
                           nullptr);
    } else {
        hipLaunchKernelGGL((gemm_skinny_kernel<TYPE, DT, 2, false>), grid, dim3(kSkThreads), 0, s, w, x, a.y,
                           a.m, a.n, nb, a.y_dtype, nullptr, nullptr);
    }
}

}  // namespace

bool expert_rows_fit_lds(uint32_t k, uint32_t m, uint32_t experts) {
    // more than 8 tokens per expert on average: 32 tokens a pass, else 16
    return (size_t)(m > 8 * experts ? 32 : 16) * k * 2 <= kResLdsBytes;
}

const char* launch_gemm_resident(hipStream_t s, const GemmArgs& dense) {
    GemmArgs a = dense;
    a.use_resident = true;
    a.expert_offsets = nullptr;
    {
        static const char* const names[5] = {"q4_k_gemm_mfma_resident", "q5_k_gemm_mfma_resident",
                                             "q6_k_gemm_mfma_resident", "iq4_xs_gemm_mfma_resident",
                                             "q8_0_gemm_mfma_resident"};
        const int f = a.ggml_type == kQ4K ? 0 : a.ggml_type == kQ5K ? 1 : a.ggml_type == kQ6K ? 2 : a.ggml_type == kIQ4XS ? 3 : 4;
#define FH_RES(TYPE) \
    if (a.x_dtype == FH_F16) launch_tt<TYPE, 1>(s, a); else launch_tt<TYPE, 2>(s, a)
        if (f == 0) { FH_RES(kQ4K); } else if (f == 1) { FH_RES(kQ5K); } else if (f == 2) { FH_RES(kQ6K); }
        else if (f == 3) { FH_RES(kIQ4XS); } else { FH_RES(kQ8_0); }
#undef FH_RES
        return names[f];
    }
}

const char* launch_gemm_skinny(hipStream_t s, const GemmArgs& a) {
    const bool grouped = a.expert_offsets != nullptr;
    if (a.ggml_type == kQ4K) {
        if (a.x_dtype == FH_F16) launch_tt<kQ4K, 1>(s, a); else launch_tt<kQ4K, 2>(s, a);
        return grouped ? "expert_project_q4_k_grouped_mfma" : "q4_k_gemm_mfma_skinny";
    }
    if (a.ggml_type == kQ5K) {
        if (a.x_dtype == FH_F16) launch_tt<kQ5K, 1>(s, a); else launch_tt<kQ5K, 2>(s, a);
        return grouped ? "expert_project_q5_k_grouped_mfma" : "q5_k_gemm_mfma_skinny";
    }
    if (a.ggml_type == kIQ4XS) {
        if (a.x_dtype == FH_F16) launch_tt<kIQ4XS, 1>(s, a); else launch_tt<kIQ4XS, 2>(s, a);
        return grouped ? "expert_project_iq4_xs_grouped_mfma" : "iq4_xs_gemm_mfma_skinny";
    }
    if (a.ggml_type == kQ8_0) {
        if (a.x_dtype == FH_F16) launch_tt<kQ8_0, 1>(s, a); else launch_tt<kQ8_0, 2>(s, a);
        return grouped ? "expert_project_q8_0_grouped_mfma" : "q8_0_gemm_mfma_skinny";
    }
    if (a.x_dtype == FH_F16) launch_tt<kQ6K, 1>(s, a); else launch_tt<kQ6K, 2>(s, a);
    return grouped ? "expert_project_q6_k_grouped_mfma" : "q6_k_gemm_mfma_skinny";
}

}  // namespace fh
