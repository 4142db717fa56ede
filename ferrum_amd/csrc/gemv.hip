// Dequant-fused GEMV for GGUF Q4_K / Q5_K / Q6_K / IQ4_XS / Q8_0 on gfx950: y[n] = sum_k W[n,k] x[k].
//
// Stands in for the reference's M = 1 kernels q4_k_gemv_ksplit / _factored
// (src/metal/shaders/ops.metal:983-1070) and q6_k_gemv_ksplit / _factored
// (:1331-1439), for the f32 small-batch kernels q4_k_gemm / q6_k_gemm
// (:1102-1121, 1466-1485; one grid slice per batch row) and, with a metadata
// pointer, for the per-assignment expert form expert_project_q4_k_factored /
// _q6_k_factored (:1088-1101, 1452-1465).  Like those it uses the factored
// arithmetic: integer quants are dotted with the activations per run of
// equal scale, and the scale (and the minimum times the activation sum) is
// applied once per run.
//
// Wave64 mapping.  Four lanes own one 256-weight super-block, 64 weights
// each; a wave covers RS rows x BS consecutive super-blocks per step
// (RS * BS = 16) and takes IT steps, so every 128-bit weight load of the wave
// is issued before anything is consumed.  The 4*BS lanes of a row are
// contiguous, so row sums are DPP reductions inside 16-lane rows.
//
// Integer quants reach the FMA without a conversion instruction: a nibble
// masked in place inside a 16-bit half is the f16 subnormal q * 2^-24 (or
// q * 2^-20 four bits up), which v_fma_mix_f32 widens exactly; the power of
// two is folded into the run scale.
//
// Activations are requested first (loads return in order, so they arrive
// before the weights queued behind them), widened to f32 and staged in LDS in
// lane order: float4 number u*4 + c of a block is the u-th float4 of lane c.
// Rows of a wave read the same LDS words (broadcast).  Sums of 16 consecutive
// activations are formed during the fill with DPP adds.
//
// Long rows are cut into K segments across workgroups (grid.y); each writes
// its partial sums to a scratch buffer and the last to arrive (a counter per
// row tile) adds them in segment order, so results are deterministic.
#include "device_utils.hpp"
#include "internal.hpp"
#include "route_device.hpp"

namespace fh {
namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * kWave;
constexpr int kXStride = 68;  // float4 per block in LDS: 64 + 4, so neighbouring blocks use the other bank half
// most steps per wave: bounded by the registers that hold the weight fragments
constexpr int max_steps(int bs) { return bs >= 8 ? 3 : 5; }

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// exact widening of an f16 (sub)normal held in one half of a dword
__device__ __forceinline__ float lo_half(uint32_t v) { return (float)__builtin_bit_cast(half2v, v).x; }
__device__ __forceinline__ float hi_half(uint32_t v) { return (float)__builtin_bit_cast(half2v, v).y; }

// float4 index q (0..63) inside a super-block -> LDS slot u*4 + c (lane c, position u)
template <uint32_t TYPE>
__device__ __forceinline__ uint32_t x_slot(uint32_t q) {
    if constexpr (TYPE != kQ6K) {
        // element 64c + 32hi + 4u' : lane c, float4 u = 8hi + u'
        return (q & 15u) * 4u + (q >> 4);
    } else {
        // element 128h + 64hi + 32o + 4u' : lane c = 2h + o, float4 u = 8hi + u'
        uint32_t c = 2u * (q >> 5) + ((q >> 3) & 1u);
        uint32_t u = 8u * ((q >> 4) & 1u) + (q & 7u);
        return u * 4u + c;
    }
}

template <uint32_t TYPE>
struct Frag;

// Q4_K: lane c owns chunk c: 32 quant bytes = groups 2c (low nibbles) and 2c+1 (high).
template <>
struct Frag<kQ4K> {
    uint4 hdr, qa, qb;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c) {
        hdr = *reinterpret_cast<const uint4*>(block);
        qa = *reinterpret_cast<const uint4*>(block + 16 + 32 * c);
        qb = *reinterpret_cast<const uint4*>(block + 32 + 32 * c);
    }
    // xc: this lane's 16 float4 (stride 4 float4); s: sums of its four 16-runs
    __device__ __forceinline__ float dot(const float4* xc, float4 s, uint32_t c) const {
        float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc_lo, sc_hi, mn_lo, mn_hi;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, c, sc_lo, sc_hi, mn_lo, mn_hi);
        float a_lo = 0.f, a_hi = 0.f, b_lo = 0.f, b_hi = 0.f;
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float4 xl = xc[t * 4], xh = xc[(8 + t) * 4];
            uint32_t w0 = q[t], w1 = q[t] >> 8;
            uint32_t l02 = w0 & 0x000f000fu, h02 = w0 & 0x00f000f0u;  // bytes 0, 2
            uint32_t l13 = w1 & 0x000f000fu, h13 = w1 & 0x00f000f0u;  // bytes 1, 3
            a_lo = fmaf(lo_half(l02), xl.x, a_lo);
            b_lo = fmaf(lo_half(l13), xl.y, b_lo);
            a_lo = fmaf(hi_half(l02), xl.z, a_lo);
            b_lo = fmaf(hi_half(l13), xl.w, b_lo);
            a_hi = fmaf(lo_half(h02), xh.x, a_hi);
            b_hi = fmaf(lo_half(h13), xh.y, b_hi);
            a_hi = fmaf(hi_half(h02), xh.z, a_hi);
            b_hi = fmaf(hi_half(h13), xh.w, b_hi);
        }
        a_lo += b_lo;
        a_hi += b_hi;
        // low nibbles were q * 2^-24, high nibbles 16q * 2^-24
        float scaled = fmaf(sc_lo * 16777216.f, a_lo, (sc_hi * 1048576.f) * a_hi);
        float offset = fmaf(mn_lo, s.x + s.y, mn_hi * (s.z + s.w));
        return fmaf(d, scaled, -(dmin * offset));
    }
};

// Q5_K: the Q4_K lane layout plus the block's 32 qh bytes; bits 2c and 2c + 1 of
// qh[l] are the fifth bits of chunk c's low- and high-nibble weights at position l.
// All four lanes of a block fetch the same 32 qh bytes.
template <>
struct Frag<kQ5K> {
    uint4 hdr, ha, hb, qa, qb;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c) {
        hdr = *reinterpret_cast<const uint4*>(block);
        ha = *reinterpret_cast<const uint4*>(block + 16);
        hb = *reinterpret_cast<const uint4*>(block + 32);
        qa = *reinterpret_cast<const uint4*>(block + 48 + 32 * c);
        qb = *reinterpret_cast<const uint4*>(block + 64 + 32 * c);
    }
    __device__ __forceinline__ float dot(const float4* xc, float4 s, uint32_t c) const {
        float d = f16_bits_to_f32(hdr.x & 0xffffu), dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc_lo, sc_hi, mn_lo, mn_hi;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, c, sc_lo, sc_hi, mn_lo, mn_hi);
        float a_lo = 0.f, a_hi = 0.f, b_lo = 0.f, b_hi = 0.f;
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const uint32_t h[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        const uint32_t shift = 2u * c;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float4 xl = xc[t * 4], xh = xc[(8 + t) * 4];
            uint32_t w0 = q[t], w1 = q[t] >> 8;
            uint32_t p0 = h[t] >> shift, p1 = p0 >> 8;   // fifth bits: bit 0 low group, bit 1 high group
            // low nibble | fifth bit << 4 reads as q * 2^-24; high nibble in place | fifth bit << 8 as 16q * 2^-24
            uint32_t l02 = (w0 & 0x000f000fu) | ((p0 & 0x00010001u) << 4);
            uint32_t l13 = (w1 & 0x000f000fu) | ((p1 & 0x00010001u) << 4);
            uint32_t h02 = (w0 & 0x00f000f0u) | ((p0 & 0x00020002u) << 7);
            uint32_t h13 = (w1 & 0x00f000f0u) | ((p1 & 0x00020002u) << 7);
            a_lo = fmaf(lo_half(l02), xl.x, a_lo);
            b_lo = fmaf(lo_half(l13), xl.y, b_lo);
            a_lo = fmaf(hi_half(l02), xl.z, a_lo);
            b_lo = fmaf(hi_half(l13), xl.w, b_lo);
            a_hi = fmaf(lo_half(h02), xh.x, a_hi);
            b_hi = fmaf(lo_half(h13), xh.y, b_hi);
            a_hi = fmaf(hi_half(h02), xh.z, a_hi);
            b_hi = fmaf(hi_half(h13), xh.w, b_hi);
        }
        a_lo += b_lo;
        a_hi += b_hi;
        float scaled = fmaf(sc_lo * 16777216.f, a_lo, (sc_hi * 1048576.f) * a_hi);
        float offset = fmaf(mn_lo, s.x + s.y, mn_hi * (s.z + s.w));
        return fmaf(d, scaled, -(dmin * offset));
    }
};

// IQ4_XS: lane c owns sub-blocks 2c and 2c + 1 (qs bytes [32c, +32)), 32 weights each:
// low nibbles are a sub-block's first 16 weights, high nibbles its last 16.  The
// codebook is looked up four nibbles at a time as bytes of value + 128, which
// reach the FMA as f16 subnormals like the K-quants' nibbles; the 128 comes
// off through the activation sums of the sub-block.
template <>
struct Frag<kIQ4XS> {
    uint2 hdr;
    uint4 qa, qb;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c) {
        hdr = *reinterpret_cast<const uint2*>(block);
        qa = load_u4_unaligned(block + 8 + 32 * c);
        qb = load_u4_unaligned(block + 24 + 32 * c);
    }
    __device__ __forceinline__ float dot(const float4* xc, float4 s, uint32_t c) const {
        const float dl0 = iq4xs_scale(hdr.x, hdr.y, 2 * c), dl1 = iq4xs_scale(hdr.x, hdr.y, 2 * c + 1);
        float acc[2][2] = {{0.f, 0.f}, {0.f, 0.f}};  // [sub-block][two chains]
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int sub = t >> 2, u = 8 * sub + (t & 3);      // float4 of the low nibbles; the high ones sit 4 on
            const float4 xl = xc[u * 4], xh = xc[(u + 4) * 4];
            const uint32_t lo = iq4_lookup4(q[t]), hi = iq4_lookup4(q[t] >> 4);
            const uint32_t l01 = bytes01_as_halves(lo), l23 = bytes23_as_halves(lo);
            const uint32_t h01 = bytes01_as_halves(hi), h23 = bytes23_as_halves(hi);
            float& a = acc[sub][0];
            float& b = acc[sub][1];
            a = fmaf(lo_half(l01), xl.x, a);
            b = fmaf(hi_half(l01), xl.y, b);
            a = fmaf(lo_half(l23), xl.z, a);
            b = fmaf(hi_half(l23), xl.w, b);
            a = fmaf(lo_half(h01), xh.x, a);
            b = fmaf(hi_half(h01), xh.y, b);
            a = fmaf(lo_half(h23), xh.z, a);
            b = fmaf(hi_half(h23), xh.w, b);
        }
        // bytes were (value + 128) * 2^-24
        const float r0 = fmaf(acc[0][0] + acc[0][1], 16777216.f, -128.f * (s.x + s.y));
        const float r1 = fmaf(acc[1][0] + acc[1][1], 16777216.f, -128.f * (s.z + s.w));
        return fmaf(dl0, r0, dl1 * r1);
    }
};

// Q8_0: lane c owns blocks 2c and 2c + 1 of the 256-weight run (68 bytes).  q + 128
// is widened like a nibble; the 128 comes off through the activation sums.
template <>
struct Frag<kQ8_0> {
    Q8Pair p;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c) { p.load(block + 68 * c); }
    __device__ __forceinline__ float dot(const float4* xc, float4 s, uint32_t) const {
        float acc[2][2] = {{0.f, 0.f}, {0.f, 0.f}};  // [block][two chains]
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float4 x = xc[(8 * blk + j) * 4];
                const uint32_t u = p.biased(blk, j);
                const uint32_t u01 = bytes01_as_halves(u), u23 = bytes23_as_halves(u);
                acc[blk][0] = fmaf(lo_half(u01), x.x, acc[blk][0]);
                acc[blk][1] = fmaf(hi_half(u01), x.y, acc[blk][1]);
                acc[blk][0] = fmaf(lo_half(u23), x.z, acc[blk][0]);
                acc[blk][1] = fmaf(hi_half(u23), x.w, acc[blk][1]);
            }
        }
        const float r0 = fmaf(acc[0][0] + acc[0][1], 16777216.f, -128.f * (s.x + s.y));
        const float r1 = fmaf(acc[1][0] + acc[1][1], 16777216.f, -128.f * (s.z + s.w));
        return fmaf(p.d(0), r0, p.d(1) * r1);
    }
};

// Q6_K: lane c = 2h + o owns ql bytes [64h + 32o, +32): slice o in the low
// nibbles and slice o + 2 in the high nibbles, with the 2-bit planes 2o and
// 2o + 4 of qh bytes [32h, +32).  Four runs of 16 weights, one int8 scale each.
template <>
struct Frag<kQ6K> {
    uint4 la, lb, ha, hb;
    uint32_t scales;  // bytes: low run 0..15, low run 16..31, high run 0..15, high run 16..31
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t* block, uint32_t c) {
        uint32_t h = c >> 1, o = c & 1u;
        la = load_u4_unaligned(block + 64 * h + 32 * o);
        lb = load_u4_unaligned(block + 64 * h + 32 * o + 16);
        ha = load_u4_unaligned(block + 128 + 32 * h);
        hb = load_u4_unaligned(block + 128 + 32 * h + 16);
        uint32_t si = 192 + 8 * h + 2 * o;
        scales = load_u16_unaligned(block + si) | (load_u16_unaligned(block + si + 4) << 16);
        d = load_u16_unaligned(block + 208);
    }
    __device__ __forceinline__ float dot(const float4* xc, float4 s, uint32_t c) const {
        const uint32_t shift = (c & 1u) * 2u;
        const uint32_t l[8] = {la.x, la.y, la.z, la.w, lb.x, lb.y, lb.z, lb.w};
        const uint32_t p[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        float acc[4] = {0.f, 0.f, 0.f, 0.f};  // low 0..15, low 16..31, high 0..15, high 16..31
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float4 xl = xc[t * 4], xh = xc[(8 + t) * 4];
            uint32_t w0 = l[t], w1 = l[t] >> 8;
            uint32_t p0 = p[t] >> shift, p1 = p0 >> 8;
            // low slice: nibble | plane bits 0..1 << 4, read as q * 2^-24
            uint32_t l02 = (w0 & 0x000f000fu) | ((p0 & 0x00030003u) << 4);
            uint32_t l13 = (w1 & 0x000f000fu) | ((p1 & 0x00030003u) << 4);
            // high slice: nibble in bits 4..7 | plane bits 4..5 << 4, read as 16q * 2^-24
            uint32_t h02 = (w0 & 0x00f000f0u) | ((p0 & 0x00300030u) << 4);
            uint32_t h13 = (w1 & 0x00f000f0u) | ((p1 & 0x00300030u) << 4);
            float& al = acc[t >> 2];
            float& ah = acc[2 + (t >> 2)];
            al = fmaf(lo_half(l02), xl.x, al);
            al = fmaf(lo_half(l13), xl.y, al);
            al = fmaf(hi_half(l02), xl.z, al);
            al = fmaf(hi_half(l13), xl.w, al);
            ah = fmaf(lo_half(h02), xh.x, ah);
            ah = fmaf(lo_half(h13), xh.y, ah);
            ah = fmaf(hi_half(h02), xh.z, ah);
            ah = fmaf(hi_half(h13), xh.w, ah);
        }
        float s0 = (float)(int)(int8_t)scales, s1 = (float)(int)(int8_t)(scales >> 8);
        float s2 = (float)(int)(int8_t)(scales >> 16), s3 = (float)(int)(int8_t)(scales >> 24);
        // stored quants are weight + 32
        float r0 = fmaf(acc[0], 16777216.f, -32.f * s.x), r1 = fmaf(acc[1], 16777216.f, -32.f * s.y);
        float r2 = fmaf(acc[2], 1048576.f, -32.f * s.z), r3 = fmaf(acc[3], 1048576.f, -32.f * s.w);
        float total = fmaf(s0, r0, s1 * r1) + fmaf(s2, r2, s3 * r3);
        return f16_bits_to_f32(d) * total;
    }
};

__device__ __forceinline__ float4 load_x4(const void* x, uint32_t dtype, size_t quad) {
    if (dtype == FH_F32) return static_cast<const float4*>(x)[quad];
    uint2 raw = static_cast<const uint2*>(x)[quad];
    if (dtype == FH_F16)
        return make_float4(f16_bits_to_f32(raw.x & 0xffffu), f16_bits_to_f32(raw.x >> 16),
                           f16_bits_to_f32(raw.y & 0xffffu), f16_bits_to_f32(raw.y >> 16));
    return make_float4(bf16_bits_to_f32(raw.x & 0xffffu), bf16_bits_to_f32(raw.x >> 16),
                       bf16_bits_to_f32(raw.y & 0xffffu), bf16_bits_to_f32(raw.y >> 16));
}

// load_x4 in two steps, so that the load can be issued long before its value is needed
__device__ __forceinline__ uint4 raw_x4(const void* x, uint32_t dtype, size_t quad) {
    if (dtype == FH_F32) return static_cast<const uint4*>(x)[quad];
    const uint2 raw = static_cast<const uint2*>(x)[quad];
    return make_uint4(raw.x, raw.y, 0u, 0u);
}
__device__ __forceinline__ float4 widen_x4(uint4 raw, uint32_t dtype) {
    if (dtype == FH_F32)
        return make_float4(__uint_as_float(raw.x), __uint_as_float(raw.y), __uint_as_float(raw.z), __uint_as_float(raw.w));
    if (dtype == FH_F16)
        return make_float4(f16_bits_to_f32(raw.x & 0xffffu), f16_bits_to_f32(raw.x >> 16),
                           f16_bits_to_f32(raw.y & 0xffffu), f16_bits_to_f32(raw.y >> 16));
    return make_float4(bf16_bits_to_f32(raw.x & 0xffffu), bf16_bits_to_f32(raw.x >> 16),
                       bf16_bits_to_f32(raw.y & 0xffffu), bf16_bits_to_f32(raw.y >> 16));
}

// What expert_silu_mul would have stored for four columns, rounded to the
// activation dtype at the same two points.
__device__ __forceinline__ float4 silu_mul4(float4 g, float4 u, uint32_t dtype) {
    return make_float4(round_storage(round_storage(silu_stable(g.x), dtype) * u.x, dtype),
                       round_storage(round_storage(silu_stable(g.y), dtype) * u.y, dtype),
                       round_storage(round_storage(silu_stable(g.z), dtype) * u.z, dtype),
                       round_storage(round_storage(silu_stable(g.w), dtype) * u.w, dtype));
}

struct Params {
    const uint8_t* w;
    const void* x;
    void* y;
    const float* metadata;
    float* partials;     // [segments][m][n] when segments > 1
    uint32_t* counters;  // one per (row tile, m), zero between launches
    uint32_t n, nb, m;
    uint32_t seg_len;    // super-blocks per K segment
    uint32_t segments;
    uint32_t x_dtype, y_dtype, experts;
    uint32_t x_rows;     // rows of x, for kXGather
    uint32_t x_mode;     // kXPlain, kXGather (row = token of the assignment), kXSiluMul (x = silu(gate) * up)
                         // or kXDivide (row = m / x_div: the routes of a token share its row)
    uint32_t meta_stride;  // floats per batch entry in `metadata`: 3 (id, token, weight) or 1 (ids only)
    uint32_t x_div;
    // Batch entries from `routed` on belong to a shared expert that every token also runs:
    // entry routed + t multiplies token t's row with the dense matrix w_shared [n, k] into
    // row t of y_shared.  Its input is row t of x_shared when that is set (the shared
    // expert's own rows: packed gate|up for kXSiluMul, activated rows otherwise), else row
    // t of x (x holds the token rows: kXGather, kXDivide).
    uint32_t routed;
    const uint8_t* w_shared;
    const void* x_shared;
    void* y_shared;
};

// grid: (row tiles, K segments, m).  ROUTE: the launch's one token has not been routed yet; wave 0
// of every workgroup routes it (route_token, up to 256 experts) while the token's row, which
// needs no routing, is already on its way, and the entry's expert comes from that.
template <uint32_t TYPE, int BS, int IT, bool ROUTE>
__device__ __forceinline__ void gemv_body(const Params& p, const RouteTokenArgs* route) {
    constexpr int RS = 16 / BS;
    constexpr uint32_t kBlockBytes = block_bytes_of(TYPE);
    extern __shared__ float4 xs[];  // seg_len * kXStride float4, then seg_len * 16 run sums
    __shared__ uint32_t last_flag;
    float* rsum = reinterpret_cast<float*>(xs + (size_t)p.seg_len * kXStride);

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t c = lane & 3u, bs = (lane >> 2) % BS, rs = lane / (4 * BS);
    const uint32_t seg = blockIdx.y, m = blockIdx.z;
    const uint32_t b0 = seg * p.seg_len;
    const uint32_t cb = p.nb - b0 < p.seg_len ? p.nb - b0 : p.seg_len;  // blocks in this segment

    size_t row_base = 0;
    bool live = true;
    const bool shared = m >= p.routed;             // uniform over the workgroup
    const uint8_t* wmat = shared ? p.w_shared : p.w;
    const void* xmat = shared && p.x_shared != nullptr ? p.x_shared : p.x;
    void* ymat = shared ? p.y_shared : p.y;
    const uint32_t ym = shared ? m - p.routed : m;  // row of y this entry writes
    if constexpr (!ROUTE) {
        if (p.metadata != nullptr && !shared) {
            uint32_t expert = __float_as_uint(p.metadata[p.meta_stride * (size_t)m]);
            live = expert < p.experts;
            row_base = live ? (size_t)expert * p.n : 0;
        }
    }
    const uint32_t row = (blockIdx.x * kWaves + wave) * RS + rs;

    // 1. activations of this segment (requested first, consumed first)
    // float4 index of the segment start in the row this batch entry reads
    size_t xrow = ym;
    if (shared) {
        // token ym's own row, in either form
    } else if (ROUTE) {
        xrow = 0;   // the one token
    } else if (p.x_mode == kXGather) {
        const uint32_t token = __float_as_uint(p.metadata[3 * (size_t)m + 1]);
        xrow = token < p.x_rows ? token : p.x_rows - 1;
    } else if (p.x_mode == kXDivide) {
        xrow = m / p.x_div;
    }
    const size_t xbase = (xrow * (p.x_mode == kXSiluMul ? 2 : 1) * p.nb + b0) * 64;
    // the SiLU form computes on what it loads, so it fetches after the weight
    // loads are queued instead of ahead of them
    const bool early = p.x_mode != kXSiluMul;
    auto fetch = [&](uint32_t q) {
        float4 v = load_x4(xmat, p.x_dtype, xbase + q);
        if (p.x_mode == kXSiluMul) v = silu_mul4(v, load_x4(xmat, p.x_dtype, xbase + (size_t)p.nb * 64 + q), p.x_dtype);
        return v;
    };
    const uint32_t xq = cb * 64;
    constexpr int kXPer = (BS * IT + 3) / 4;  // float4 per thread that cover the longest segment
    float4 xr[kXPer];
#pragma unroll
    for (int i = 0; i < kXPer; ++i) {
        uint32_t q = tid + i * kThreads;
        xr[i] = q < xq && early ? load_x4(xmat, p.x_dtype, xbase + q) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    asm volatile("" ::: "memory");

    if constexpr (ROUTE) {
        __shared__ __attribute__((aligned(16))) float route_scores[256];
        __shared__ float route_records[3 * kMaxTopK];
        if (wave == 0)
            route_token<4>(*route, 0u, lane, route_scores, route_records, blockIdx.x == 0 && blockIdx.y == 0 && m == 0);
        __syncthreads();
        if (!shared) {
            const uint32_t expert = __float_as_uint(route_records[3 * m]);
            live = expert < p.experts;
            row_base = live ? (size_t)expert * p.n : 0;
        }
    }
    const uint8_t* rp = wmat + ((row_base + (row < p.n ? row : p.n - 1)) * (size_t)p.nb + b0) * kBlockBytes;

    // 2. every weight fragment of this wave
    Frag<TYPE> frag[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        uint32_t b = it * BS + bs;
        frag[it].load(rp + (size_t)(b < cb ? b : cb - 1) * kBlockBytes, c);
    }
    asm volatile("" ::: "memory");

    // 3. stage activations and the sums of their 16-runs
    auto stage = [&](uint32_t q, float4 v) {
        const uint32_t slot = x_slot<TYPE>(q & 63u);
        xs[(q >> 6) * kXStride + slot] = v;
        // four consecutive float4 (one quad of lanes) are one 16-run of one lane
        float s = (v.x + v.y) + (v.z + v.w);
        s = dpp_add<0xB1>(s);
        s = dpp_add<0x4E>(s);
        if ((q & 3u) == 0) rsum[(q >> 6) * 16 + (slot & 3u) * 4 + (slot >> 4)] = s;
    };
#pragma unroll
    for (int i = 0; i < kXPer; ++i) {
        uint32_t q = tid + i * kThreads;
        if (q < xq && early) stage(q, xr[i]);
    }
    for (uint32_t q = tid + (early ? kXPer * kThreads : 0); q < xq; q += kThreads)
        stage(q, fetch(q));
    __syncthreads();

    // 4. consume, one step at a time
    float acc = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        uint32_t b = it * BS + bs;
        bool valid = b < cb;
        uint32_t bb = valid ? b : 0;
        float4 s = *reinterpret_cast<const float4*>(rsum + bb * 16 + c * 4);
        float v = frag[it].dot(xs + bb * kXStride + c, s, c);
        acc += valid ? v : 0.f;
        asm volatile("" : "+v"(acc)::"memory");
    }
    acc = dpp_add<0xB1>(acc);
    acc = dpp_add<0x4E>(acc);
    if (BS >= 2) acc = dpp_add<0x141>(acc);
    if (BS >= 4) acc = dpp_add<0x140>(acc);
    if (BS >= 8) acc += __shfl_xor(acc, 16, 64);
    const bool writer = (lane & (4 * BS - 1)) == 0 && row < p.n;
    if (!live) acc = 0.f;

    if (p.segments == 1) {
        if (writer) store_from_f32(ymat, (size_t)ym * p.n + row, p.y_dtype, acc);
        return;
    }
    // 5. K segments meet in the scratch buffer; the last workgroup of a tile adds
    // them.  Partials and the counter use device-scope atomic accesses, which
    // are coherent across the chip's L2 slices without cache-wide flushes.
    if (writer)
        __hip_atomic_store(&p.partials[((size_t)seg * p.m + m) * p.n + row], acc, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the stores above have completed
    __syncthreads();
    if (tid == 0) {
        uint32_t* counter = p.counters + (size_t)m * gridDim.x + blockIdx.x;
        uint32_t ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t last = ticket == p.segments - 1 ? 1u : 0u;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = last;
    }
    __syncthreads();
    if (last_flag == 0) return;
    if (tid < kWaves * RS) {
        uint32_t r = blockIdx.x * (kWaves * RS) + tid;
        if (r < p.n) {
            float total = 0.f;
            for (uint32_t s = 0; s < p.segments; ++s)
                total += __hip_atomic_load(&p.partials[((size_t)s * p.m + m) * p.n + r], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
            store_from_f32(ymat, (size_t)ym * p.n + r, p.y_dtype, total);
        }
    }
}

template <uint32_t TYPE, int BS, int IT>
__global__ __launch_bounds__(kThreads) void gemv_kernel(const Params p) {
    gemv_body<TYPE, BS, IT, false>(p, nullptr);
}

template <uint32_t TYPE, int BS, int IT>
__global__ __launch_bounds__(kThreads) void gemv_route_kernel(const Params p, const RouteTokenArgs route) {
    gemv_body<TYPE, BS, IT, true>(p, &route);
}

// The routed FFN's last two stages in one launch for a few tokens: the down projection of
// every entry of a token (its top_k routed experts in rank order, then the shared expert) and
// expert_combine's weighted sum over them (src/metal/shaders/ops.metal:1088-1101, 2234-2246;
// the two launches src/nn/moe.rs:349-397 makes).  A workgroup owns RS rows of one token's
// output; wave w computes entry w (and w + 16 when there are more than 16) exactly as
// gemv_kernel does with the SiLU input form: the same fragments, the same order of
// additions, rounded to the activation dtype where that launch would have stored it.  The
// rounded values meet in LDS and the first RS threads add them in rank order with
// expert_combine's rounding, so the result has the bits of the two separate launches.
struct DownCombineParams {
    const uint8_t* w;          // [experts][n][nb] blocks
    const uint8_t* w_shared;   // [n][nb] blocks, or null
    const void* x;             // [tokens * top_k][2 * k]: packed gate|up rows of the routed entries
    const void* x_shared;      // [tokens][2 * k]
    const float* metadata;     // [tokens * top_k][3]: expert id, token, weight
    const float* shared_gate;  // [tokens], or null = 1
    void* y;                   // [tokens][n]
    uint32_t n, nb, top_k, experts;
    uint32_t dtype;            // of x, of the rounding between the stages and of y
};

constexpr int kDownCombineMaxWaves = 16;

template <uint32_t TYPE, int BS, int IT>
__global__ __launch_bounds__(kDownCombineMaxWaves * kWave) void expert_down_combine_kernel(const DownCombineParams p) {
    constexpr int RS = 16 / BS;
    constexpr uint32_t kBlockBytes = block_bytes_of(TYPE);
    extern __shared__ float4 xs_all[];  // per wave: nb * kXStride float4, then nb * 16 run sums
    __shared__ float values[2 * kDownCombineMaxWaves][16];
    __shared__ float weights[2 * kDownCombineMaxWaves];  // fetched next to the expert ids, before anything waits

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, waves = blockDim.x >> 6;
    const uint32_t c = lane & 3u, bs = (lane >> 2) % BS, rs = lane / (4 * BS);
    const uint32_t token = blockIdx.y;
    const uint32_t entries = p.top_k + (p.w_shared != nullptr ? 1u : 0u);
    const size_t wave_floats = (size_t)p.nb * kXStride * 4 + (size_t)p.nb * 16;
    float4* xs = reinterpret_cast<float4*>(reinterpret_cast<float*>(xs_all) + wave * wave_floats);
    float* rsum = reinterpret_cast<float*>(xs + (size_t)p.nb * kXStride);
    const uint32_t row = blockIdx.x * RS + rs;

    for (uint32_t entry = wave; entry < entries; entry += waves) {
        const bool shared = entry >= p.top_k;
        const size_t slot = (size_t)token * p.top_k + entry;
        // the entry's packed gate|up row does not depend on the routing record: its first 512
        // columns are requested before the record, whose expert id the weight loads wait for
        const void* xmat = shared ? p.x_shared : p.x;
        const size_t xbase = (shared ? (size_t)token : slot) * 2 * p.nb * 64;
        const uint32_t xq = p.nb * 64;
        uint4 raw_gate[2], raw_up[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t q = lane + 64 * j < xq ? lane + 64 * j : xq - 1;
            raw_gate[j] = raw_x4(xmat, p.dtype, xbase + q);
            raw_up[j] = raw_x4(xmat, p.dtype, xbase + (size_t)p.nb * 64 + q);
        }
        asm volatile("" ::: "memory");
        bool live = true;
        size_t row_base = 0;
        float weight;
        if (!shared) {
            const uint32_t expert = __float_as_uint(p.metadata[3 * slot]);
            weight = p.metadata[3 * slot + 2];
            live = expert < p.experts;
            row_base = live ? (size_t)expert * p.n : 0;
        } else {
            weight = p.shared_gate != nullptr ? p.shared_gate[token] : 1.f;
        }
        if (lane == 0) weights[entry] = weight;
        const uint8_t* wmat = shared ? p.w_shared : p.w;
        const uint8_t* rp = wmat + (row_base + (row < p.n ? row : p.n - 1)) * (size_t)p.nb * kBlockBytes;
        Frag<TYPE> frag[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const uint32_t b = it * BS + bs;
            frag[it].load(rp + (size_t)(b < p.nb ? b : p.nb - 1) * kBlockBytes, c);
        }
        asm volatile("" ::: "memory");
        // the entry's activations: silu(gate) * up of its packed row, staged as gemv_kernel stages them
        if (entry != wave) __builtin_amdgcn_wave_barrier();
        for (uint32_t q = lane, j = 0; q < xq; q += 64, ++j) {
            float4 gate, up;
            if (j < 2) {
                gate = widen_x4(j == 0 ? raw_gate[0] : raw_gate[1], p.dtype);
                up = widen_x4(j == 0 ? raw_up[0] : raw_up[1], p.dtype);
            } else {
                gate = load_x4(xmat, p.dtype, xbase + q);
                up = load_x4(xmat, p.dtype, xbase + (size_t)p.nb * 64 + q);
            }
            const float4 v = silu_mul4(gate, up, p.dtype);
            const uint32_t at = x_slot<TYPE>(q & 63u);
            xs[(q >> 6) * kXStride + at] = v;
            float s = (v.x + v.y) + (v.z + v.w);
            s = dpp_add<0xB1>(s);
            s = dpp_add<0x4E>(s);
            if ((q & 3u) == 0) rsum[(q >> 6) * 16 + (at & 3u) * 4 + (at >> 4)] = s;
        }
        // the wave reads what its own lanes wrote: LDS operations of a wave complete in order
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
        float acc = 0.f;
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const uint32_t b = it * BS + bs;
            const bool valid = b < p.nb;
            const uint32_t bb = valid ? b : 0;
            const float4 s = *reinterpret_cast<const float4*>(rsum + bb * 16 + c * 4);
            const float v = frag[it].dot(xs + bb * kXStride + c, s, c);
            acc += valid ? v : 0.f;
            asm volatile("" : "+v"(acc)::"memory");
        }
        acc = dpp_add<0xB1>(acc);
        acc = dpp_add<0x4E>(acc);
        if (BS >= 2) acc = dpp_add<0x141>(acc);
        if (BS >= 4) acc = dpp_add<0x140>(acc);
        if (BS >= 8) acc += __shfl_xor(acc, 16, 64);
        if (!live) acc = 0.f;
        if ((lane & (4 * BS - 1)) == 0) values[entry][rs] = round_storage(acc, p.dtype);
    }
    __syncthreads();
    if (tid < (uint32_t)RS) {
        const uint32_t r = blockIdx.x * RS + tid;
        if (r < p.n) {
            // each product is rounded before it is added, as expert_combine does
#pragma clang fp contract(off)
            float sum = 0.f;
            for (uint32_t entry = 0; entry < entries; ++entry)
                sum += round_storage(round_storage(weights[entry], p.dtype) * values[entry][tid], p.dtype);
            store_from_f32(p.y, (size_t)token * p.n + r, p.dtype, sum);
        }
    }
}

typedef void (*DownCombineFn)(dim3, dim3, size_t, hipStream_t, const DownCombineParams&);

template <uint32_t TYPE, int BS, int IT>
void launch_down_combine_impl(dim3 grid, dim3 block, size_t lds, hipStream_t s, const DownCombineParams& p) {
    hipLaunchKernelGGL((expert_down_combine_kernel<TYPE, BS, IT>), grid, block, lds, s, p);
}

template <uint32_t TYPE>
DownCombineFn pick_down_combine(int bs, int it) {
#define FH_CASE(B, I) \
    if (bs == B && it == I) return launch_down_combine_impl<TYPE, B, I>;
    FH_CASE(8, 1) FH_CASE(8, 2) FH_CASE(4, 1) FH_CASE(4, 2) FH_CASE(2, 1) FH_CASE(2, 2) FH_CASE(1, 1)
#undef FH_CASE
    return nullptr;
}

typedef void (*LaunchFn)(dim3, size_t, hipStream_t, const Params&);

template <uint32_t TYPE, int BS, int IT>
void launch_impl(dim3 grid, size_t lds, hipStream_t s, const Params& p) {
    hipLaunchKernelGGL((gemv_kernel<TYPE, BS, IT>), grid, dim3(kThreads), lds, s, p);
}

template <uint32_t TYPE>
LaunchFn pick(int bs, int it) {
#define FH_CASE(B, I) \
    if (bs == B && it == I) return launch_impl<TYPE, B, I>;
    FH_CASE(8, 1) FH_CASE(8, 2) FH_CASE(8, 3)
    FH_CASE(4, 1) FH_CASE(4, 2) FH_CASE(4, 3) FH_CASE(4, 4) FH_CASE(4, 5)
    FH_CASE(2, 1) FH_CASE(2, 2) FH_CASE(2, 3)
    FH_CASE(1, 1) FH_CASE(1, 2) FH_CASE(1, 3)
#undef FH_CASE
    return nullptr;
}

typedef void (*RouteLaunchFn)(dim3, size_t, hipStream_t, const Params&, const RouteTokenArgs&);

template <uint32_t TYPE, int BS, int IT>
void launch_route_impl(dim3 grid, size_t lds, hipStream_t s, const Params& p, const RouteTokenArgs& r) {
    hipLaunchKernelGGL((gemv_route_kernel<TYPE, BS, IT>), grid, dim3(kThreads), lds, s, p, r);
}

template <uint32_t TYPE>
RouteLaunchFn pick_route(int bs, int it) {
#define FH_CASE(B, I) \
    if (bs == B && it == I) return launch_route_impl<TYPE, B, I>;
    FH_CASE(8, 1) FH_CASE(8, 2) FH_CASE(8, 3) FH_CASE(4, 1) FH_CASE(2, 1) FH_CASE(1, 1)
#undef FH_CASE
    return nullptr;
}

}  // namespace

namespace {

// Segments, segment length and steps for a block-slot count.
GemvPlan plan_for(uint32_t nb, int bs, int forced_segments) {
    GemvPlan plan{};
    const uint32_t span = (uint32_t)(bs * max_steps(bs));
    uint32_t segments = (nb + span - 1) / span;
    if (forced_segments > 0) {
        // the reference's K-split switch: at least that many segments, as far
        // as the row length allows
        uint32_t want = (uint32_t)forced_segments;
        const uint32_t most = (nb + bs - 1) / bs;
        if (want > most) want = most;
        if (want > segments) segments = want;
    }
    const uint32_t seg_len = (nb + segments - 1) / segments;
    plan.bs = bs;
    plan.it = (int)((seg_len + bs - 1) / bs);
    plan.segments = (nb + seg_len - 1) / seg_len;
    plan.seg_len = seg_len;
    return plan;
}

}  // namespace

GemvPlan gemv_plan(uint32_t n, uint32_t k, uint32_t m, int forced_segments) {
    const uint32_t nb = k / 256;
    // widest block-slot count the row length fills ...
    const int bs = nb >= 8 ? 8 : nb >= 4 ? 4 : nb >= 2 ? 2 : 1;
    GemvPlan plan = plan_for(nb, bs, forced_segments);
    if (bs == 8 && n >= 16384) {
        // ... unless four slots and more steps leave fewer idle slot-steps (20
        // blocks: 4 x 5 covers them exactly, 8 x 3 idles a sixth of the wave)
        // and the matrix still makes a thousand 16-row workgroups
        const GemvPlan narrow = plan_for(nb, 4, forced_segments);
        const uint32_t idle_wide = plan.segments * (uint32_t)(plan.bs * plan.it) - nb;
        const uint32_t idle_narrow = narrow.segments * (uint32_t)(narrow.bs * narrow.it) - nb;
        if (idle_narrow < idle_wide && narrow.segments <= plan.segments) plan = narrow;
    }
    plan.rows_per_wg = (uint32_t)(kWaves * (16 / plan.bs));
    plan.tiles = (n + plan.rows_per_wg - 1) / plan.rows_per_wg;
    (void)m;
    return plan;
}

bool gemv_takes_stream(const GemvArgs& a, StreamPlan* plan) {
    if (a.stream == 0 || (a.ggml_type != kQ4K && a.ggml_type != kQ6K) || a.metadata != nullptr || a.x_mode != kXPlain ||
        a.shared_w != nullptr)
        return false;
    *plan = gemv_stream_plan(a.ggml_type, a.n, a.k, a.m, a.cu_count, a.stream == 2, a.ksplit);
    return plan->ok;
}

GemvScratch gemv_scratch(const GemvArgs& a) {
    StreamPlan stream;
    if (gemv_takes_stream(a, &stream)) return {stream.segments, stream.tiles};
    const GemvPlan plan = gemv_plan(a.n, a.k, a.m, a.ksplit);
    return {plan.segments, plan.tiles};
}

const char* launch_gemv(hipStream_t s, const GemvArgs& a) {
    StreamPlan stream;
    if (gemv_takes_stream(a, &stream)) return launch_gemv_stream(s, a, stream);
    const GemvPlan plan = gemv_plan(a.n, a.k, a.m, a.ksplit);
    Params p{};
    p.w = static_cast<const uint8_t*>(a.w);
    p.x = a.x;
    p.y = a.y;
    p.metadata = a.metadata;
    p.partials = a.partials;
    p.counters = a.counters;
    p.n = a.n;
    p.nb = a.k / 256;
    p.m = a.m;
    p.seg_len = plan.seg_len;
    p.segments = plan.segments;
    p.x_dtype = a.x_dtype;
    p.y_dtype = a.y_dtype;
    p.experts = a.experts;
    p.x_mode = a.x_mode;
    p.x_rows = a.x_rows;
    p.meta_stride = a.meta_stride == 0 ? 3u : a.meta_stride;
    p.x_div = a.x_div == 0 ? 1u : a.x_div;
    p.routed = a.shared_w != nullptr ? a.m - a.shared_rows : 0xffffffffu;
    p.w_shared = static_cast<const uint8_t*>(a.shared_w);
    p.x_shared = a.shared_x;
    p.y_shared = a.shared_y;
    const size_t lds = (size_t)plan.seg_len * kXStride * 16 + (size_t)plan.seg_len * 64;
    dim3 grid(plan.tiles, plan.segments, a.m);
    LaunchFn fn = a.ggml_type == kQ4K     ? pick<kQ4K>(plan.bs, plan.it)
                  : a.ggml_type == kQ5K   ? pick<kQ5K>(plan.bs, plan.it)
                  : a.ggml_type == kIQ4XS ? pick<kIQ4XS>(plan.bs, plan.it)
                  : a.ggml_type == kQ8_0  ? pick<kQ8_0>(plan.bs, plan.it)
                                          : pick<kQ6K>(plan.bs, plan.it);
    if (a.route != nullptr) {
        RouteLaunchFn rf = a.ggml_type == kQ4K     ? pick_route<kQ4K>(plan.bs, plan.it)
                           : a.ggml_type == kQ5K   ? pick_route<kQ5K>(plan.bs, plan.it)
                           : a.ggml_type == kIQ4XS ? pick_route<kIQ4XS>(plan.bs, plan.it)
                           : a.ggml_type == kQ8_0  ? pick_route<kQ8_0>(plan.bs, plan.it)
                                                   : pick_route<kQ6K>(plan.bs, plan.it);
        rf(grid, lds, s, p, *a.route);   // gemv_routes said the pair exists
    } else {
        fn(grid, lds, s, p);
    }
    const int f = a.ggml_type == kQ4K ? 0 : a.ggml_type == kQ5K ? 1 : a.ggml_type == kQ6K ? 2 : a.ggml_type == kIQ4XS ? 3 : 4;
    static const char* const expert_names[5] = {"expert_project_q4_k_factored", "expert_project_q5_k_factored",
                                                "expert_project_q6_k_factored", "expert_project_iq4_xs_factored",
                                                "expert_project_q8_0_factored"};
    static const char* const ksplit_names[5] = {"q4_k_gemv_ksplit", "q5_k_gemv_ksplit", "q6_k_gemv_ksplit",
                                                "iq4_xs_gemv_ksplit", "q8_0_gemv_ksplit"};
    static const char* const factored_names[5] = {"q4_k_gemv_factored", "q5_k_gemv_factored", "q6_k_gemv_factored",
                                                  "iq4_xs_gemv_factored", "q8_0_gemv_factored"};
    if (a.route != nullptr) return a.route->rank_order ? "h_moe_route + expert_project" : "moe_route + expert_project";
    if (a.metadata != nullptr) return expert_names[f];
    if (plan.segments > 1) return ksplit_names[f];
    return factored_names[f];
}

// Whether the projection of one token's entries can route the token itself: rows of one K
// segment (up to 24 super-blocks) and a router of up to 256 experts.
bool gemv_routes(uint32_t n, uint32_t k, uint32_t experts, uint32_t top_k) {
    const GemvPlan plan = gemv_plan(n, k, 1, 0);
    return plan.segments == 1 && pick_route<kQ4K>(plan.bs, plan.it) != nullptr && experts <= 256 && top_k <= (uint32_t)kMaxTopK;
}

bool expert_down_combine_fits(uint32_t ggml_type, uint32_t n, uint32_t k, uint32_t top_k, bool shared) {
    const GemvPlan plan = gemv_plan(n, k, 1, 0);
    if (plan.segments != 1 || plan.it > 2 || (plan.bs == 1 && plan.it != 1)) return false;
    const uint32_t entries = top_k + (shared ? 1u : 0u);
    if (entries > 2u * kDownCombineMaxWaves) return false;
    const uint32_t waves = entries < (uint32_t)kDownCombineMaxWaves ? entries : (uint32_t)kDownCombineMaxWaves;
    // every wave stages its entry's activations in LDS
    if ((size_t)waves * (k / 256) * ((size_t)kXStride * 16 + 64) > 64u * 1024) return false;
    (void)ggml_type;
    return true;
}

const char* launch_expert_down_combine(hipStream_t s, const ExpertDownCombineArgs& a) {
    const GemvPlan plan = gemv_plan(a.n, a.k, 1, 0);
    DownCombineParams p{};
    p.w = static_cast<const uint8_t*>(a.w);
    p.w_shared = static_cast<const uint8_t*>(a.w_shared);
    p.x = a.x;
    p.x_shared = a.x_shared;
    p.metadata = a.metadata;
    p.shared_gate = a.shared_gate;
    p.y = a.y;
    p.n = a.n;
    p.nb = a.k / 256;
    p.top_k = a.top_k;
    p.experts = a.experts;
    p.dtype = a.dtype;
    const uint32_t entries = a.top_k + (a.w_shared != nullptr ? 1u : 0u);
    const uint32_t waves = entries < (uint32_t)kDownCombineMaxWaves ? entries : (uint32_t)kDownCombineMaxWaves;
    const uint32_t rs = 16u / (uint32_t)plan.bs;
    const size_t lds = (size_t)waves * ((size_t)p.nb * kXStride * 16 + (size_t)p.nb * 64);
    DownCombineFn fn = a.ggml_type == kQ4K     ? pick_down_combine<kQ4K>(plan.bs, plan.it)
                       : a.ggml_type == kQ5K   ? pick_down_combine<kQ5K>(plan.bs, plan.it)
                       : a.ggml_type == kIQ4XS ? pick_down_combine<kIQ4XS>(plan.bs, plan.it)
                       : a.ggml_type == kQ8_0  ? pick_down_combine<kQ8_0>(plan.bs, plan.it)
                                               : pick_down_combine<kQ6K>(plan.bs, plan.it);
    fn(dim3((a.n + rs - 1) / rs, a.tokens), dim3(waves * 64), lds, s, p);
    return a.w_shared != nullptr ? "expert_project + h_moe_combine" : "expert_project + expert_combine";
}


}  // namespace fh
