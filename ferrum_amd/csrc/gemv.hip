// Dequant-fused GEMV for GGUF Q4_K / Q6_K on gfx950: y[n] = sum_k W[n,k] x[k].
//
// Stands in for the reference's M = 1 kernels q4_k_gemv_ksplit / _factored
// (src/metal/shaders/ops.metal:983-1070) and q6_k_gemv_ksplit / _factored
// (:1331-1439), and, with a metadata pointer, for the per-assignment expert
// form expert_project_q4_k_factored / _q6_k_factored (:1088-1101, 1452-1465).
// Like those it uses the factored arithmetic: per 16-weight run the integer
// quants are dotted with the activations and the block scale (and, for Q4_K,
// the minimum times the activation sum) is applied once.
//
// Wave64 mapping.  Eight lanes own one 256-weight super-block: lane `sub`
// loads 16 bytes of 4-bit quants (32 weights: a run of 16 in their low
// nibbles and a run of 16 in their high nibbles).  A wave therefore streams
// eight consecutive super-blocks of a row per step with 128-bit loads, and
// keeps the 32 activations it needs in registers across R rows.
//
// Activations are staged once per workgroup in LDS as f32, permuted so that
// the eight float4 reads of a lane are conflict free: float4 number
// (4*seg + jj)*8 + sub of a block holds the jj-th float4 of lane `sub`'s
// low-nibble (seg 0) or high-nibble (seg 1) run.
//
// KS waves of a workgroup may share the same rows and interleave super-blocks
// (the reference's K-split); partial sums meet in LDS in a fixed order, so
// results do not depend on scheduling.
#include "device_utils.hpp"
#include "internal.hpp"

namespace fh {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;


// ---- activation permutation ------------------------------------------------------

// float4 index q (0..63) inside a super-block -> LDS float4 slot.
template <uint32_t TYPE>
__device__ __forceinline__ uint32_t x_slot(uint32_t q) {
    uint32_t jj = q & 3u;
    if constexpr (TYPE == kQ4K) {
        // element e = 64c + 32seg + 16h + 4jj + t
        uint32_t c = q >> 4, seg = (q >> 3) & 1u, h = (q >> 2) & 1u;
        return (4u * seg + jj) * 8u + (2u * c + h);
    } else {
        // element e = 128half + 32slice + 16hh + 4jj + t; low nibbles hold
        // slices 0/1, high nibbles slices 2/3
        uint32_t half = q >> 5, slice = (q >> 3) & 3u, hh = (q >> 2) & 1u;
        return (4u * (slice >> 1) + jj) * 8u + (4u * half + 2u * (slice & 1u) + hh);
    }
}

// ---- per-format fragments ---------------------------------------------------------

template <uint32_t TYPE>
struct Frag;

template <>
struct Frag<kQ4K> {
    uint4 hdr;  // d, dmin, 12 scale bytes
    uint4 qs;   // this lane's 32 nibbles

    __device__ __forceinline__ void load(const uint8_t* block, uint32_t sub) {
        hdr = *reinterpret_cast<const uint4*>(block);
        qs = *reinterpret_cast<const uint4*>(block + 16 + 16 * sub);
    }

    // dot of this lane's 32 weights with xv; sums are the activation sums of
    // the low- and high-nibble runs.
    __device__ __forceinline__ float dot(const float4 (&xv)[8], float sum_lo, float sum_hi,
                                         uint32_t sub) const {
        float d = f16_bits_to_f32(hdr.x & 0xffffu);
        float dmin = f16_bits_to_f32(hdr.x >> 16);
        float sc_lo, sc_hi, mn_lo, mn_hi;
        q4k_chunk_scales(hdr.y, hdr.z, hdr.w, sub >> 1, sc_lo, sc_hi, mn_lo, mn_hi);
        float a_lo = 0.f, a_hi = 0.f;
        const uint32_t q[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t lo = q[t] & 0x0f0f0f0fu;
            uint32_t hi = (q[t] >> 4) & 0x0f0f0f0fu;
            a_lo = fmaf(xv[t].x, (float)(lo & 0xffu), a_lo);
            a_lo = fmaf(xv[t].y, (float)((lo >> 8) & 0xffu), a_lo);
            a_lo = fmaf(xv[t].z, (float)((lo >> 16) & 0xffu), a_lo);
            a_lo = fmaf(xv[t].w, (float)(lo >> 24), a_lo);
            a_hi = fmaf(xv[4 + t].x, (float)(hi & 0xffu), a_hi);
            a_hi = fmaf(xv[4 + t].y, (float)((hi >> 8) & 0xffu), a_hi);
            a_hi = fmaf(xv[4 + t].z, (float)((hi >> 16) & 0xffu), a_hi);
            a_hi = fmaf(xv[4 + t].w, (float)(hi >> 24), a_hi);
        }
        float scaled = fmaf(sc_lo, a_lo, sc_hi * a_hi);
        float offset = fmaf(mn_lo, sum_lo, mn_hi * sum_hi);
        return fmaf(d, scaled, -(dmin * offset));
    }
};

template <>
struct Frag<kQ6K> {
    uint4 ql;      // 16 bytes: low nibbles slice s, high nibbles slice s+2
    uint4 qh;      // 16 bytes of 2-bit planes for the same 16 positions
    uint32_t tail; // {scale of the low run, scale of the high run} << 16 | f16 d

    __device__ __forceinline__ void load(const uint8_t* block, uint32_t sub) {
        uint32_t half = sub >> 2, hh = sub & 1u, sl = (sub >> 1) & 1u;
        ql = load_u4_unaligned(block + 16 * sub);
        qh = load_u4_unaligned(block + 128 + 32 * half + 16 * hh);
        uint32_t si = 192 + 8 * half + 2 * sl + hh;
        uint32_t lo = block[si], hi = block[si + 4];
        uint32_t d = load_u16_unaligned(block + 208);
        tail = d | (lo << 16) | (hi << 24);
    }

    __device__ __forceinline__ float dot(const float4 (&xv)[8], float sum_lo, float sum_hi,
                                         uint32_t sub) const {
        float d = f16_bits_to_f32(tail & 0xffffu);
        float sc_lo = (float)(int)(int8_t)(tail >> 16);
        float sc_hi = (float)(int)(int8_t)(tail >> 24);
        uint32_t shift = (sub & 2u);  // slice&1 -> 2-bit plane 0/1 for low, +4 for high
        float a_lo = 0.f, a_hi = 0.f;
        const uint32_t l[4] = {ql.x, ql.y, ql.z, ql.w};
        const uint32_t h[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            uint32_t hb = h[t] >> shift;
            uint32_t lo = (l[t] & 0x0f0f0f0fu) | ((hb & 0x03030303u) << 4);
            uint32_t hi = ((l[t] >> 4) & 0x0f0f0f0fu) | (((hb >> 4) & 0x03030303u) << 4);
            a_lo = fmaf(xv[t].x, (float)(lo & 0xffu), a_lo);
            a_lo = fmaf(xv[t].y, (float)((lo >> 8) & 0xffu), a_lo);
            a_lo = fmaf(xv[t].z, (float)((lo >> 16) & 0xffu), a_lo);
            a_lo = fmaf(xv[t].w, (float)(lo >> 24), a_lo);
            a_hi = fmaf(xv[4 + t].x, (float)(hi & 0xffu), a_hi);
            a_hi = fmaf(xv[4 + t].y, (float)((hi >> 8) & 0xffu), a_hi);
            a_hi = fmaf(xv[4 + t].z, (float)((hi >> 16) & 0xffu), a_hi);
            a_hi = fmaf(xv[4 + t].w, (float)(hi >> 24), a_hi);
        }
        // stored quants are weight + 32
        a_lo = fmaf(-32.f, sum_lo, a_lo);
        a_hi = fmaf(-32.f, sum_hi, a_hi);
        return d * fmaf(sc_lo, a_lo, sc_hi * a_hi);
    }
};

// ---- kernel -----------------------------------------------------------------------

template <int XDT>
__device__ __forceinline__ float4 load_x4(const void* x, size_t quad) {
    if constexpr (XDT == 0) {
        return static_cast<const float4*>(x)[quad];
    } else {
        uint2 raw = static_cast<const uint2*>(x)[quad];
        if constexpr (XDT == 1) {
            return make_float4(f16_bits_to_f32(raw.x & 0xffffu), f16_bits_to_f32(raw.x >> 16),
                               f16_bits_to_f32(raw.y & 0xffffu), f16_bits_to_f32(raw.y >> 16));
        } else {
            return make_float4(bf16_bits_to_f32(raw.x & 0xffffu), bf16_bits_to_f32(raw.x >> 16),
                               bf16_bits_to_f32(raw.y & 0xffffu), bf16_bits_to_f32(raw.y >> 16));
        }
    }
}

// grid: (ceil(n / rows_per_group / groups), m).  chunk_blocks super-blocks of x
// fit the dynamic LDS allocation; longer rows take several passes.
template <uint32_t TYPE, int R, int KS, int XDT>
__global__ __launch_bounds__(kThreads) void gemv_kernel(
    const uint8_t* __restrict__ w, const void* __restrict__ x, void* __restrict__ y, uint32_t n,
    uint32_t nb, uint32_t y_dtype, uint32_t chunk_blocks, const float* __restrict__ metadata,
    uint32_t experts) {
    extern __shared__ float4 xs[];
    __shared__ float partial[kWaves][R];
    constexpr int kGroups = kWaves / KS;  // row groups per workgroup
    constexpr uint32_t kBlockBytes = TYPE == kQ4K ? 144 : 210;

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t group = wave / KS, ks = wave % KS;
    const uint32_t slot = lane >> 3, sub = lane & 7u;
    const uint32_t m = blockIdx.y;
    const uint32_t k = nb << 8;

    size_t row_base = 0;
    bool live = true;
    if (metadata != nullptr) {
        uint32_t expert = __float_as_uint(metadata[3 * (size_t)m]);
        live = expert < experts;
        row_base = live ? (size_t)expert * n : 0;
    }
    const uint32_t r0 = (blockIdx.x * kGroups + group) * R;
    const uint8_t* rows[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        uint32_t row = r0 + r < n ? r0 + r : n - 1;
        rows[r] = w + (row_base + row) * (size_t)nb * kBlockBytes;
    }
    const void* xrow = static_cast<const uint8_t*>(x) + (size_t)m * k * (XDT == 0 ? 4 : 2);

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;

    for (uint32_t c0 = 0; c0 < nb; c0 += chunk_blocks) {
        const uint32_t cb = nb - c0 < chunk_blocks ? nb - c0 : chunk_blocks;
        // first fragments of this pass are requested before the LDS fill
        Frag<TYPE> cur[R];
        uint32_t bl = ks * 8 + slot;
        {
            uint32_t b = c0 + (bl < cb ? bl : cb - 1);
#pragma unroll
            for (int r = 0; r < R; ++r) cur[r].load(rows[r] + (size_t)b * kBlockBytes, sub);
        }
        if (c0) __syncthreads();
        for (uint32_t q = tid; q < cb * 64; q += kThreads) {
            float4 v = load_x4<XDT>(xrow, (size_t)c0 * 64 + q);
            xs[(q & ~63u) + x_slot<TYPE>(q & 63u)] = v;
        }
        __syncthreads();

        for (; bl - slot < cb; bl += 8 * KS) {   // uniform trip count per wave
            const bool valid = bl < cb;
            Frag<TYPE> nxt[R];
            {
                uint32_t nb_l = bl + 8 * KS;
                uint32_t b = c0 + (nb_l < cb ? nb_l : cb - 1);
#pragma unroll
                for (int r = 0; r < R; ++r) nxt[r].load(rows[r] + (size_t)b * kBlockBytes, sub);
            }
            float4 xv[8];
            const float4* xb = xs + (size_t)(valid ? bl : 0) * 64 + sub;
#pragma unroll
            for (int j = 0; j < 8; ++j) xv[j] = xb[j * 8];
            float sum_lo = 0.f, sum_hi = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sum_lo += (xv[j].x + xv[j].y) + (xv[j].z + xv[j].w);
                sum_hi += (xv[4 + j].x + xv[4 + j].y) + (xv[4 + j].z + xv[4 + j].w);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float v = cur[r].dot(xv, sum_lo, sum_hi, sub);
                acc[r] += valid ? v : 0.f;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) cur[r] = nxt[r];
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);

    if constexpr (KS == 1) {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (r0 + r < n)
                    store_from_f32(y, (size_t)m * n + r0 + r, y_dtype, live ? acc[r] : 0.f);
        }
    } else {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) partial[wave][r] = acc[r];
        }
        __syncthreads();
        if (tid < kGroups * R) {
            uint32_t g = tid / R, r = tid % R;
            float total = 0.f;
#pragma unroll
            for (int s = 0; s < KS; ++s) total += partial[g * KS + s][r];
            uint32_t row = (blockIdx.x * kGroups + g) * R + r;
            if (row < n) store_from_f32(y, (size_t)m * n + row, y_dtype, live ? total : 0.f);
        }
    }
}

struct Launch {
    void (*set_lds)(size_t);
    void (*run)(dim3, size_t, hipStream_t, const GemvArgs&, uint32_t nb, uint32_t chunk);
};

template <uint32_t TYPE, int R, int KS, int XDT>
void set_lds_impl(size_t bytes) {
    static size_t configured = 0;
    if (bytes > configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_kernel<TYPE, R, KS, XDT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        configured = bytes;
    }
}

template <uint32_t TYPE, int R, int KS, int XDT>
void run_impl(dim3 grid, size_t lds, hipStream_t s, const GemvArgs& a, uint32_t nb,
              uint32_t chunk) {
    hipLaunchKernelGGL((gemv_kernel<TYPE, R, KS, XDT>), grid, dim3(kThreads), lds, s,
                       static_cast<const uint8_t*>(a.w), a.x, a.y, a.n, nb, a.y_dtype, chunk,
                       a.metadata, a.experts);
}

template <uint32_t TYPE, int R, int KS>
Launch pick_dtype(uint32_t x_dtype) {
    switch (x_dtype) {
        case FH_F32: return {set_lds_impl<TYPE, R, KS, 0>, run_impl<TYPE, R, KS, 0>};
        case FH_F16: return {set_lds_impl<TYPE, R, KS, 1>, run_impl<TYPE, R, KS, 1>};
        default: return {set_lds_impl<TYPE, R, KS, 2>, run_impl<TYPE, R, KS, 2>};
    }
}

template <uint32_t TYPE>
Launch pick(int r, int ks, uint32_t x_dtype) {
#define FH_CASE(RR, KK) \
    if (r == RR && ks == KK) return pick_dtype<TYPE, RR, KK>(x_dtype);
    FH_CASE(1, 1) FH_CASE(1, 2) FH_CASE(1, 4)
    FH_CASE(2, 1) FH_CASE(2, 2) FH_CASE(2, 4)
    FH_CASE(4, 1) FH_CASE(4, 2) FH_CASE(4, 4)
#undef FH_CASE
    return pick_dtype<TYPE, 2, 1>(x_dtype);
}

}  // namespace

const char* launch_gemv(hipStream_t s, const GemvArgs& a) {
    const uint32_t nb = a.k / 256;
    // Automatic geometry: enough workgroups to cover the chip several times,
    // K-split when rows alone cannot (the reference's rule of thumb,
    // src/ops/transformer.rs:262-270, re-derived for 256 CUs).
    int r = a.rows_per_wave, ks = a.ksplit;
    const uint64_t total_rows = (uint64_t)a.n * a.m;
    if (r == 0) r = total_rows >= 16384 ? 4 : total_rows >= 4096 ? 2 : 1;
    if (ks == 0) {
        ks = 1;
        uint64_t waves = total_rows / r;
        while (ks < 4 && waves * ks < (uint64_t)a.cu_count * 8 && nb >= (uint32_t)(16 * ks)) ks *= 2;
    }
    if (r != 1 && r != 2 && r != 4) r = 2;
    if (ks != 1 && ks != 2 && ks != 4) ks = 1;

    const uint32_t max_chunk = 144;  // 144 KiB of the 160 KiB LDS
    const uint32_t chunk = nb < max_chunk ? nb : max_chunk;
    const size_t lds = (size_t)chunk * 1024;
    const uint32_t rows_per_wg = (uint32_t)(r * (kWaves / ks));
    dim3 grid((a.n + rows_per_wg - 1) / rows_per_wg, a.m);

    Launch l = a.ggml_type == kQ4K ? pick<kQ4K>(r, ks, a.x_dtype) : pick<kQ6K>(r, ks, a.x_dtype);
    if (lds > 48 * 1024) l.set_lds(lds);
    l.run(grid, lds, s, a, nb, chunk);
    if (a.metadata != nullptr)
        return a.ggml_type == kQ4K ? "expert_project_q4_k_factored" : "expert_project_q6_k_factored";
    if (ks > 1) return a.ggml_type == kQ4K ? "q4_k_gemv_ksplit" : "q6_k_gemv_ksplit";
    return a.ggml_type == kQ4K ? "q4_k_gemv_factored" : "q6_k_gemv_factored";
}

}  // namespace fh
