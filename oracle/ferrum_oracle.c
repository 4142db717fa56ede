/*
 * ferrum_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C CPU restatement of Ferrum's reference arithmetic for the
 * quantized-matmul path (GGUF Q4_K / Q6_K dequant, dense projection, MoE
 * routing and expert stages).  It is the checker the GPU library is compared
 * against and the CPU baseline that the benchmark times; nothing that ships
 * links it.  Build with: gcc -O2 -ffp-contract=off -fno-fast-math (see the
 * Makefile beside this file): an FMA would change the dequantized bits.
 *
 * Every function cites the reference source it follows (paths relative to
 * the Ferrum tree).  Pinning status (what independent evidence fixes each
 * function) is stated per function; the checks live in tests/test_oracle*.py.
 *
 *   fo_f16_to_f32 / fo_f32_to_f16 / fo_f32_to_bf16   pinned: exhaustive f16
 *       widening vs numpy.float16, RNE narrowing vs numpy on random + tie
 *       cases, bf16 ties/NaN cases of tests/correctness.rs:300-318.
 *   fo_q4_k_scale_min      pinned: three restatements agree (direct form,
 *       llama.cpp kmask word form, brute force over all byte pairs).
 *   fo_dequantize (block form) and fo_weight (per-element form), Q4_K, Q5_K, Q6_K
 *                          pinned: both forms agree bitwise on the
 *       reference's closed-form fixtures; exact-rational step-by-step
 *       rounding on a (d, sc, m, q) grid; Q3_K -> Q6_K value identity.
 *   fo_dequantize / fo_weight, IQ4_XS
 *                          pinned without a fixture (the reference holds no
 *       CPU twin or test vector for this format): the block form follows
 *       dequantize_iq4_xs and the per-element form the indexing of the GEMV
 *       kernel mv_iq4_xs, two separate statements in the reference, and they
 *       agree bitwise; with every sub-block scale at ls = 33 a sub-block
 *       equals the reference's CPU IQ4_NL decoder (src/hybrid/iq_tests.rs:
 *       1606-1620, src/hybrid/ple.rs:150-158) on the same bytes; the 6-bit
 *       scale assembly is checked for all 64 values at all 8 positions
 *       against blocks packed by a separately written packer; the value is
 *       exact in f32 (17-bit scale x 7-bit codebook), checked in rationals.
 *   fo_dequantize / fo_weight, Q8_0
 *                          pinned: numpy (int8 view times float16 view) on the
 *       reference's random-block generator; block form = per-element form.
 *       Rows of 32 n weights with n not a multiple of 8 (cols / 32 * 34 bytes,
 *       src/hybrid/weights.rs:1167): the same byte stream read as rows of 256
 *       weights gives the same values in the same order, and projections
 *       equal the numpy product and the hand-written sequential loop.
 *   fo_project_f32seq / fo_project_f64
 *                          pinned: integer special case (d=1, sc=1, dmin=0)
 *       equals an exact integer dot; all-zero quants equal -dmin*m*sum(x);
 *       numpy float64 matmul of the dequantized matrix.
 *   fo_select_routes       pinned: literal expectations of
 *       src/nn/moe.rs:666-739; ids bitwise.  Weights depend on libm expf in
 *       the last ulp (reference tolerance 2e-6).
 *   fo_expert_*            pinned: hand-computed 3-wide MoE of
 *       src/nn/moe.rs:530-664 restated in numpy float64.
 *   fo_select_routes_ranked, fo_shared_gate
 *                          ids pinned: the CPU procedure of the reference's
 *       own routing test (src/hybrid/engine.rs:5004-5024) in numpy float64,
 *       and equal-logit ties.  Weights and gate: PARITY UNPINNED in the last
 *       ulps (the reference's threadgroup summation order is its own); held
 *       to that test's tolerances, 1e-5 and 1e-4.
 *   fo_expert_combine_shared   pinned: numpy float64 evaluation; equals
 *       fo_expert_combine when the shared rows are zero.
 *   fo_argmax_rows         pinned for finite rows: numpy argmax (first
 *       maximal index) and ties; rows holding NaN follow the reference
 *       kernel's scan and merge order as read (flagged rows: parity unpinned).
 *   fo_moe_map             pinned: numpy's stable argsort and bincount (integer
 *       work, exact).
 *   fo_hybrid_combine      pinned: numpy float64 evaluation (f32 sums in rank
 *       order; the reference kernel's own fma contraction is its compiler's
 *       choice, so the last ulp is held to the reference test's 1e-4).
 *   fo_add_rmsnorm         pinned: the residual is the storage-rounded f32 sum
 *       (exact); the normalised rows follow the reference's own CPU rmsnorm
 *       (src/reference.rs:23-35, float64) and are checked against closed
 *       forms (constant rows, one-hot rows, scale invariance).
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FO_Q4_K 12u
#define FO_Q5_K 13u
#define FO_Q6_K 14u
#define FO_IQ4_XS 23u
#define FO_Q8_0 8u

/* ---------------------------------------------------------------- scalars */

/* IEEE binary16 -> binary32, exact (half crate 2.7.1 f16::to_f32, used at
 * src/quantization.rs:225). */
float fo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                shift++;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(113 - shift) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (half crate f16::from_f32,
 * src/tensor/mod.rs:19-25 DType::round). */
uint16_t fo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 255) {
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x0200u | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = sign | ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (uint16_t)half;
}

/* binary32 -> bfloat16 bits, RNE with NaN quieting
 * (src/metal/shaders/ops.metal:11-20 store(), :25-33 round_storage()). */
uint16_t fo_f32_to_bf16(float f) {
    uint32_t bits;
    memcpy(&bits, &f, 4);
    if (f != f) return (uint16_t)((bits >> 16) | 0x40u);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

float fo_bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Storage rounding: dtype 0 f32, 1 f16, 2 bf16 (ops.metal:25-33). */
float fo_round_storage(float x, uint32_t dtype) {
    if (dtype == 1) return fo_f16_to_f32(fo_f32_to_f16(x));
    if (dtype == 2) return fo_bf16_to_f32(fo_f32_to_bf16(x));
    return x;
}

void fo_round_storage_array(const float* in, size_t n, uint32_t dtype, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = fo_round_storage(in[i], dtype);
}

/* ------------------------------------------------------------- geometry */

/* src/quantization.rs:50-74: 256 weights per super-block, 144 / 210 bytes. */
size_t fo_block_bytes(uint32_t ggml_type) {
    if (ggml_type == FO_Q4_K) return 144;
    if (ggml_type == FO_Q5_K) return 176;
    if (ggml_type == FO_Q6_K) return 210;
    if (ggml_type == FO_IQ4_XS) return 136; /* src/loader/gguf.rs:111 */
    if (ggml_type == FO_Q8_0) return 8 * 34;  /* 256 weights = eight 34-byte blocks, src/loader/gguf.rs:99 */
    return 0;
}

/* A row is whole blocks of the format's own geometry: 256 weights, or 32 weights in 34 bytes for
 * Q8_0 (src/loader/gguf.rs:99), whose rows need not end on a run of eight blocks. */
static size_t row_unit(uint32_t ggml_type) { return ggml_type == FO_Q8_0 ? 32 : 256; }
static size_t row_unit_bytes(uint32_t ggml_type) { return ggml_type == FO_Q8_0 ? 34 : fo_block_bytes(ggml_type); }
int fo_columns_ok(uint32_t ggml_type, size_t cols) {
    return fo_block_bytes(ggml_type) != 0 && cols != 0 && cols % row_unit(ggml_type) == 0;
}
size_t fo_row_bytes(uint32_t ggml_type, size_t cols) {
    return cols / row_unit(ggml_type) * row_unit_bytes(ggml_type);
}

/* ------------------------------------------------------------ Q4_K / Q6_K */

/* 6-bit scale and minimum of 32-weight group `group` (0..7) from the 12
 * packed bytes (src/ops/transformer.rs:2905-2917; ops.metal:826-833). */
void fo_q4_k_scale_min(const uint8_t* scales, uint32_t group, uint32_t* sc, uint32_t* mn) {
    if (group < 4) {
        *sc = scales[group] & 63u;
        *mn = scales[group + 4] & 63u;
    } else {
        *sc = (uint32_t)(scales[group + 4] & 15u) | ((uint32_t)(scales[group - 4] >> 6) << 4);
        *mn = (uint32_t)(scales[group + 4] >> 4) | ((uint32_t)(scales[group] >> 6) << 4);
    }
}

static inline uint16_t le16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* Block form, Q4_K: the ggml dequantize_row_q4_K walk restated at
 * src/diffusion/tests.rs:811-836.  Expression order ((d*sc)*q) - (dmin*m),
 * every step rounded to f32. */
static void dequant_q4_k_block(const uint8_t* b, float* out) {
    float d = fo_f16_to_f32(le16(b));
    float dmin = fo_f16_to_f32(le16(b + 2));
    const uint8_t* scales = b + 4;
    const uint8_t* qs = b + 16;
    for (int chunk = 0; chunk < 4; chunk++) {
        const uint8_t* q = qs + 32 * chunk;
        for (int half = 0; half < 2; half++) {
            uint32_t sc, mn;
            fo_q4_k_scale_min(scales, (uint32_t)(2 * chunk + half), &sc, &mn);
            float fsc = (float)sc, fmn = (float)mn;
            for (int l = 0; l < 32; l++) {
                uint32_t low = half == 0 ? (q[l] & 15u) : (uint32_t)(q[l] >> 4);
                float scaled = d * fsc;
                float value = scaled * (float)low;
                float offset = dmin * fmn;
                *out++ = value - offset;
            }
        }
    }
}

/* Block form, Q5_K (176 B: d, dmin, scales[12], qh[32], qs[128]): the Q4_K
 * walk with bit (2*chunk + half) of qh[l] as the quant's fifth bit
 * (src/diffusion/tests.rs:811-836, `high` branch). */
static void dequant_q5_k_block(const uint8_t* b, float* out) {
    float d = fo_f16_to_f32(le16(b));
    float dmin = fo_f16_to_f32(le16(b + 2));
    const uint8_t* scales = b + 4;
    const uint8_t* qh = b + 16;
    const uint8_t* qs = b + 48;
    for (int chunk = 0; chunk < 4; chunk++) {
        const uint8_t* q = qs + 32 * chunk;
        for (int half = 0; half < 2; half++) {
            uint32_t sc, mn;
            fo_q4_k_scale_min(scales, (uint32_t)(2 * chunk + half), &sc, &mn);
            float fsc = (float)sc, fmn = (float)mn;
            uint8_t bit = (uint8_t)(1u << (2 * chunk + half));
            for (int l = 0; l < 32; l++) {
                uint32_t low = half == 0 ? (q[l] & 15u) : (uint32_t)(q[l] >> 4);
                uint32_t top = (qh[l] & bit) ? 16u : 0u;
                float scaled = d * fsc;
                float value = scaled * (float)(low + top);
                float offset = dmin * fmn;
                *out++ = value - offset;
            }
        }
    }
}

/* Block form, Q6_K: ggml dequantize_row_q6_K restated at
 * src/diffusion/tests.rs:843-864 and src/hybrid/iq_tests.rs:1481-1500.
 * Expression order (d*scale)*q. */
static void dequant_q6_k_block(const uint8_t* b, float* out) {
    float d = fo_f16_to_f32(le16(b + 208));
    for (int n = 0; n < 2; n++) {
        const uint8_t* ql = b + 64 * n;
        const uint8_t* qh = b + 128 + 32 * n;
        const int8_t* sc = (const int8_t*)(b + 192 + 8 * n);
        float* y = out + 128 * n;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int q1 = (int)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32;
            int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            float s1 = d * (float)sc[is];
            float s2 = d * (float)sc[is + 2];
            float s3 = d * (float)sc[is + 4];
            float s4 = d * (float)sc[is + 6];
            y[l] = s1 * (float)q1;
            y[l + 32] = s2 * (float)q2;
            y[l + 64] = s3 * (float)q3;
            y[l + 96] = s4 * (float)q4;
        }
    }
}

/* The 16-entry codebook shared by IQ4_NL and IQ4_XS (kvalues_iq4nl_f,
 * src/metal/shaders/hybrid.metal:34-37; CPU copies src/hybrid/ple.rs:25-27,
 * src/hybrid/iq_tests.rs:1608-1610). */
static const float iq4_values[16] = {-127.f, -104.f, -83.f, -65.f, -49.f, -35.f, -22.f, -10.f,
                                     1.f,    13.f,   25.f,  38.f,  53.f,  69.f,  89.f,  113.f};

/* Block form, IQ4_XS (136 B: f16 d, u16 scales_h, scales_l[4], qs[128]):
 * dequantize_iq4_xs (src/metal/shaders/hybrid.metal:580-596), which takes the
 * block 16 values at a time: chunk il is half il % 2 (low or high nibbles) of
 * the four qs words of sub-block il / 2, scaled by d * (ls - 32). */
static void dequant_iq4_xs_block(const uint8_t* b, float* out) {
    float d = fo_f16_to_f32(le16(b));
    uint32_t scales_h = le16(b + 2);
    const uint8_t* scales_l = b + 4;
    const uint8_t* qs = b + 8;
    for (int il = 0; il < 16; il++) {
        int ib32 = il / 2, half = il % 2;
        int ls = (int)(((uint32_t)(scales_l[ib32 / 2] >> (4 * (ib32 % 2))) & 0xfu) | (((scales_h >> (2 * ib32)) & 3u) << 4));
        float dl = d * (float)(ls - 32);
        for (int i = 0; i < 4; i++) {
            const uint8_t* word = qs + 16 * ib32 + 4 * i;
            for (int j = 0; j < 4; j++) {
                uint32_t index = ((uint32_t)word[j] >> (4 * half)) & 0xfu;
                out[16 * il + 4 * i + j] = dl * iq4_values[index];
            }
        }
    }
}

/* Q8_0, one block of 32 weights {f16 d, int8 qs[32]}: value = q * d
 * (src/hybrid/draft/gguf.rs:331-338; dequantize_q8_0,
 * src/metal/shaders/hybrid.metal:499-508). */
static void dequant_q8_0_block(const uint8_t* p, float* out) {
    float d = fo_f16_to_f32(le16(p));
    for (int j = 0; j < 32; j++) out[j] = (float)(int8_t)p[2 + j] * d;
}

static void dequant_block(uint32_t ggml_type, const uint8_t* block, float* out) {
    if (ggml_type == FO_Q4_K)
        dequant_q4_k_block(block, out);
    else if (ggml_type == FO_Q5_K)
        dequant_q5_k_block(block, out);
    else if (ggml_type == FO_IQ4_XS)
        dequant_iq4_xs_block(block, out);
    else if (ggml_type == FO_Q8_0)
        dequant_q8_0_block(block, out);
    else
        dequant_q6_k_block(block, out);
}

/* One packed row of `cols` weights, block by block. */
static void dequant_row(uint32_t ggml_type, const uint8_t* src, size_t cols, float* out) {
    size_t unit = row_unit(ggml_type), bytes = row_unit_bytes(ggml_type);
    for (size_t b = 0; b < cols / unit; b++) dequant_block(ggml_type, src + b * bytes, out + b * unit);
}

/* Dequantize a packed row-major [rows, cols] matrix to f32 (block form). */
int fo_dequantize(uint32_t ggml_type, const uint8_t* packed, size_t rows, size_t cols, float* out) {
    if (!fo_columns_ok(ggml_type, cols)) return 1;
    size_t row_bytes = fo_row_bytes(ggml_type, cols);
    for (size_t row = 0; row < rows; row++) dequant_row(ggml_type, packed + row * row_bytes, cols, out + row * cols);
    return 0;
}

/* Per-element form (GPU q4_k_weight ops.metal:834-845, q6_k_weight
 * ops.metal:1316-1329; CPU twins src/ops/transformer.rs:2919-2956 and
 * :4153-4169).  Written independently of the block form above so that the
 * two can be compared bitwise. */
float fo_weight(uint32_t ggml_type, const uint8_t* packed, size_t row, size_t column, size_t cols) {
    size_t blocks = cols >> 8, block_index = column >> 8;
    uint32_t within = (uint32_t)(column & 255);
    uint32_t group = within >> 5, lane = within & 31;
    if (ggml_type == FO_Q4_K) {
        const uint8_t* block = packed + (row * blocks + block_index) * 144;
        uint32_t chunk = within >> 6;
        uint8_t byte = block[16 + chunk * 32 + lane];
        uint32_t q = (group & 1) == 0 ? (uint32_t)(byte & 15) : (uint32_t)(byte >> 4);
        float d = fo_f16_to_f32(le16(block));
        float dmin = fo_f16_to_f32(le16(block + 2));
        uint32_t sc, mn;
        fo_q4_k_scale_min(block + 4, group, &sc, &mn);
        float a = d * (float)sc;
        float b = a * (float)q;
        float c = dmin * (float)mn;
        return b - c;
    }
    if (ggml_type == FO_Q5_K) {
        /* q5_k_weight (ops.metal:846-857; CPU twin src/ops/transformer.rs:2946-2952) */
        const uint8_t* block = packed + (row * blocks + block_index) * 176;
        uint32_t chunk = within >> 6;
        uint8_t byte = block[48 + chunk * 32 + lane];
        uint32_t nibble = (group & 1) == 0 ? (uint32_t)(byte & 15) : (uint32_t)(byte >> 4);
        uint32_t high = ((uint32_t)block[16 + lane] >> group) & 1u;
        uint32_t q = nibble | (high << 4);
        float d = fo_f16_to_f32(le16(block));
        float dmin = fo_f16_to_f32(le16(block + 2));
        uint32_t sc, mn;
        fo_q4_k_scale_min(block + 4, group, &sc, &mn);
        float a = d * (float)sc;
        float b = a * (float)q;
        float c = dmin * (float)mn;
        return b - c;
    }
    if (ggml_type == FO_Q8_0) {
        /* one value of the row's flat run of 34-byte blocks: block column / 32, quant column % 32 */
        const uint8_t* block = packed + row * ((cols >> 5) * 34) + (column >> 5) * 34;
        return fo_f16_to_f32(le16(block)) * (float)(int8_t)block[2 + (column & 31)];
    }
    if (ggml_type == FO_IQ4_XS) {
        /* the indexing of the GEMV kernel mv_iq4_xs (src/metal/shaders/hybrid.metal:899-951):
         * sub-block ib = group, byte 16 ib + (lane & 15), low nibble for lanes 0..15 and high
         * nibble for 16..31, and (d * ls) applied to the codebook value */
        const uint8_t* block = packed + (row * blocks + block_index) * 136;
        uint32_t ib = group;
        uint8_t byte = block[8 + 16 * ib + (lane & 15)];
        uint32_t index = lane < 16 ? (uint32_t)(byte & 0x0f) : (uint32_t)(byte >> 4);
        uint32_t scales_h = le16(block + 2);
        int ls = (int)(((uint32_t)(block[4 + ib / 2] >> (4 * (ib % 2))) & 0xfu) | (((scales_h >> (2 * ib)) & 3u) << 4)) - 32;
        float dl = fo_f16_to_f32(le16(block)) * (float)ls;
        return dl * iq4_values[index];
    }
    const uint8_t* block = packed + (row * blocks + block_index) * 210;
    uint32_t half_block = group >> 2, slice = group & 3;
    uint8_t byte = block[half_block * 64 + (slice & 1) * 32 + lane];
    uint32_t low = slice < 2 ? (uint32_t)(byte & 15) : (uint32_t)(byte >> 4);
    uint32_t high = ((uint32_t)block[128 + half_block * 32 + lane] >> (slice * 2)) & 3u;
    int q = (int)(low | (high << 4)) - 32;
    int8_t scale = (int8_t)block[192 + half_block * 8 + slice * 2 + (lane >> 4)];
    float d = fo_f16_to_f32(le16(block + 208));
    float a = d * (float)scale;
    return a * (float)q;
}

/* src/quantization.rs:212-261 validate_gguf_quantized_payload for the two
 * K formats: 0 ok, 1 partial block, 2 non-finite scale. */
int fo_validate_payload(uint32_t ggml_type, const uint8_t* payload, size_t len) {
    size_t bb = fo_block_bytes(ggml_type) == 0 ? 0 : row_unit_bytes(ggml_type);
    if (bb == 0 || len % bb != 0) return 1;
    for (size_t off = 0; off < len; off += bb) {
        const uint8_t* b = payload + off;
        if (ggml_type == FO_Q4_K || ggml_type == FO_Q5_K) {
            if (!isfinite(fo_f16_to_f32(le16(b))) || !isfinite(fo_f16_to_f32(le16(b + 2)))) return 2;
        } else if (ggml_type == FO_IQ4_XS) {
            if (!isfinite(fo_f16_to_f32(le16(b)))) return 2;
        } else if (ggml_type == FO_Q8_0) {
            if (!isfinite(fo_f16_to_f32(le16(b)))) return 2;
        } else {
            if (!isfinite(fo_f16_to_f32(le16(b + 208)))) return 2;
        }
    }
    return 0;
}

/* -------------------------------------------------------------- projection */

typedef struct {
    uint32_t ggml_type;
    const uint8_t* packed;
    size_t n, k, m;
    const float* x;
    float* y;
    int weight_round; /* 0 none, 1 f16, 2 bf16: the tile dtype of the GEMM tier */
    int out_round;    /* storage rounding of the result */
    int f64;          /* accumulate in double */
    size_t row_begin, row_end;
} project_job;

static void* project_worker(void* arg) {
    project_job* j = (project_job*)arg;
    size_t row_bytes = fo_row_bytes(j->ggml_type, j->k);
    float* w = (float*)malloc(j->k * sizeof(float));
    for (size_t row = j->row_begin; row < j->row_end; row++) {
        dequant_row(j->ggml_type, j->packed + row * row_bytes, j->k, w);
        if (j->weight_round)
            for (size_t c = 0; c < j->k; c++) w[c] = fo_round_storage(w[c], (uint32_t)j->weight_round);
        for (size_t mi = 0; mi < j->m; mi++) {
            const float* x = j->x + mi * j->k;
            float r;
            if (j->f64) {
                double acc = 0.0;
                for (size_t c = 0; c < j->k; c++) acc += (double)x[c] * (double)w[c];
                r = (float)acc;
            } else {
                /* `.sum::<f32>()` of input*weight, K ascending
                 * (src/ops/transformer.rs:2964-2980). */
                float acc = 0.0f;
                for (size_t c = 0; c < j->k; c++) {
                    float p = x[c] * w[c];
                    acc = acc + p;
                }
                r = acc;
            }
            j->y[mi * j->n + row] = fo_round_storage(r, (uint32_t)j->out_round);
        }
    }
    free(w);
    return NULL;
}

static int run_project(project_job base, int threads) {
    if (!fo_columns_ok(base.ggml_type, base.k)) return 1;
    if (threads < 1) threads = 1;
    if ((size_t)threads > base.n) threads = (int)base.n;
    if (threads == 1) {
        base.row_begin = 0;
        base.row_end = base.n;
        project_worker(&base);
        return 0;
    }
    pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
    project_job* jobs = (project_job*)malloc(sizeof(project_job) * (size_t)threads);
    size_t per = (base.n + (size_t)threads - 1) / (size_t)threads;
    for (int t = 0; t < threads; t++) {
        jobs[t] = base;
        jobs[t].row_begin = (size_t)t * per < base.n ? (size_t)t * per : base.n;
        jobs[t].row_end = jobs[t].row_begin + per < base.n ? jobs[t].row_begin + per : base.n;
        pthread_create(&tid[t], NULL, project_worker, &jobs[t]);
    }
    for (int t = 0; t < threads; t++) pthread_join(tid[t], NULL);
    free(tid);
    free(jobs);
    return 0;
}

/* Y[M,N] = X[M,K] * W[N,K]^T with sequential f32 accumulation: the
 * reference's `expected()` (src/ops/transformer.rs:2964-2980, :4177-4187).
 * weight_round mirrors the tile tests (:3130-3141): dequantized weights are
 * rounded to the tile dtype before the product. */
int fo_project_f32seq(uint32_t ggml_type, const uint8_t* packed, size_t n, size_t k, const float* x,
                      size_t m, float* y, int weight_round, int out_round, int threads) {
    project_job j = {ggml_type, packed, n, k, m, x, y, weight_round, out_round, 0, 0, 0};
    return run_project(j, threads);
}

/* Same product with f64 accumulation (src/diffusion/tests.rs:736-745,
 * src/hybrid/iq_tests.rs:1316-1326). */
int fo_project_f64(uint32_t ggml_type, const uint8_t* packed, size_t n, size_t k, const float* x,
                   size_t m, float* y, int weight_round, int threads) {
    project_job j = {ggml_type, packed, n, k, m, x, y, weight_round, 0, 1, 0, 0};
    return run_project(j, threads);
}

/* ------------------------------------------------------------------- MoE */

static uint32_t total_order_key(float x) {
    /* ops.metal:21-24; equals f32::total_cmp ordering. */
    uint32_t bits;
    memcpy(&bits, &x, 4);
    return (bits & 0x80000000u) ? ~bits : (bits ^ 0x80000000u);
}

static float bits_to_float(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}

static uint32_t float_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* SparseMoe::select_routes (src/nn/moe.rs:392-458): scores over all experts
 * (softmax with max subtraction, or sigmoid); top-k by score+bias under a
 * total order, ties to the lower index; weights are the raw scores,
 * optionally divided by (sum of selected in selection order + eps), times
 * the scaling factor; rows sorted by expert id.  metadata is [tokens*k, 3]
 * f32 {expert id bits, token id bits, weight}.  Returns 0, or 1 on invalid
 * logits / geometry, 2 on an invalid normaliser. */
static int select_routes(const float* logits, size_t tokens, size_t experts, size_t top_k, int sigmoid,
                         int normalize, float eps, float scaling, const float* bias, float* metadata,
                         int ranked) {
    if (experts == 0 || top_k == 0 || top_k > experts) return 1;
    for (size_t i = 0; i < tokens * experts; i++)
        if (!isfinite(logits[i])) return 1;
    float* scores = (float*)malloc(experts * sizeof(float));
    uint8_t* used = (uint8_t*)malloc(experts);
    size_t* sel = (size_t*)malloc(top_k * sizeof(size_t));
    float* selw = (float*)malloc(top_k * sizeof(float));
    int status = 0;
    for (size_t token = 0; token < tokens && status == 0; token++) {
        const float* row = logits + token * experts;
        if (sigmoid) {
            for (size_t e = 0; e < experts; e++) scores[e] = 1.0f / (1.0f + expf(-row[e]));
        } else {
            float maximum = -INFINITY;
            for (size_t e = 0; e < experts; e++) maximum = fmaxf(maximum, row[e]);
            float normalizer = 0.0f;
            for (size_t e = 0; e < experts; e++) {
                scores[e] = expf(row[e] - maximum);
                normalizer = normalizer + scores[e];
            }
            for (size_t e = 0; e < experts; e++) scores[e] = scores[e] / normalizer;
        }
        memset(used, 0, experts);
        for (size_t rank = 0; rank < top_k; rank++) {
            size_t best = experts;
            uint32_t best_key = 0;
            for (size_t e = 0; e < experts; e++) {
                if (used[e]) continue;
                float s = scores[e] + (bias ? bias[e] : 0.0f);
                uint32_t key = total_order_key(s);
                if (best == experts || key > best_key) {
                    best = e;
                    best_key = key;
                }
            }
            used[best] = 1;
            sel[rank] = best;
            selw[rank] = scores[best];
        }
        if (normalize) {
            float normalizer = 0.0f;
            for (size_t r = 0; r < top_k; r++) normalizer = normalizer + selw[r];
            float denominator = normalizer + eps;
            if (!isfinite(denominator) || denominator <= 0.0f) {
                status = 2;
                break;
            }
            for (size_t r = 0; r < top_k; r++) selw[r] = selw[r] / denominator;
        }
        for (size_t r = 0; r < top_k; r++) selw[r] = selw[r] * scaling;
        /* stable insertion sort by expert id (the hybrid engine keeps selection order) */
        for (size_t i = 1; i < top_k && !ranked; i++) {
            size_t id = sel[i];
            float w = selw[i];
            size_t j = i;
            while (j > 0 && sel[j - 1] > id) {
                sel[j] = sel[j - 1];
                selw[j] = selw[j - 1];
                j--;
            }
            sel[j] = id;
            selw[j] = w;
        }
        for (size_t r = 0; r < top_k; r++) {
            float* o = metadata + (token * top_k + r) * 3;
            o[0] = bits_to_float((uint32_t)sel[r]);
            o[1] = bits_to_float((uint32_t)token);
            o[2] = selw[r];
        }
    }
    free(scores);
    free(used);
    free(sel);
    free(selw);
    return status;
}

int fo_select_routes(const float* logits, size_t tokens, size_t experts, size_t top_k, int sigmoid,
                     int normalize, float eps, float scaling, const float* bias, float* metadata) {
    return select_routes(logits, tokens, experts, top_k, sigmoid, normalize, eps, scaling, bias, metadata, 0);
}

/* h_moe_route (src/metal/shaders/hybrid.metal:2259-2319): the same scores and
 * top-k (greater probability wins, ties to the lower index), weights divided
 * by the sum of the picked ones taken in rank order, rows left in rank order.
 * The reference sums the softmax denominator with a threadgroup tree whose
 * order is its own; this restatement sums in expert order, so weights agree
 * to the last few ulp, not bitwise (ids are exact away from exact ties). */
int fo_select_routes_ranked(const float* logits, size_t tokens, size_t experts, size_t top_k, int sigmoid,
                            int normalize, float* metadata) {
    return select_routes(logits, tokens, experts, top_k, sigmoid, normalize, 0.0f, 1.0f, NULL, metadata, 1);
}

/* Shared-expert gate of h_moe_route: sigmoid(dot(x[t], w)); the dot product is
 * accumulated in f64 here (the reference's threadgroup tree is unpinned). */
void fo_shared_gate(const float* x, const float* w, size_t tokens, size_t hidden, float* out) {
    for (size_t t = 0; t < tokens; t++) {
        double dot = 0.0;
        for (size_t i = 0; i < hidden; i++) dot += (double)x[t * hidden + i] * (double)w[i];
        out[t] = (float)(1.0 / (1.0 + exp(-dot)));
    }
}

/* h_moe_combine (hybrid.metal:2374-2388) in f32: out[t,c] = sum over ranks of
 * w * down, then + gate[t] * shared[t,c] (gate may be NULL: 1).  With a 16-bit
 * dtype the products and the gate are rounded like fo_expert_combine's. */
void fo_expert_combine_shared(const float* in, const float* metadata, size_t tokens, size_t hidden,
                              size_t top_k, uint32_t dtype, const float* shared, const float* gate, float* out) {
    for (size_t t = 0; t < tokens; t++) {
        for (size_t c = 0; c < hidden; c++) {
            float total = 0.0f;
            for (size_t rank = 0; rank < top_k; rank++) {
                size_t a = t * top_k + rank;
                float w = fo_round_storage(metadata[a * 3 + 2], dtype);
                float product = w * in[a * hidden + c];
                total = total + fo_round_storage(product, dtype);
            }
            float g = fo_round_storage(gate ? gate[t] : 1.0f, dtype);
            float product = g * shared[t * hidden + c];
            total = total + fo_round_storage(product, dtype);
            out[t * hidden + c] = fo_round_storage(total, dtype);
        }
    }
}

/* expert_assign (ops.metal:1959-1967): out[a,:] = hidden[token(a),:]. */
void fo_expert_assign(const float* hidden, const float* metadata, size_t assignments, size_t width,
                      float* out) {
    for (size_t a = 0; a < assignments; a++) {
        uint32_t token = float_to_bits(metadata[a * 3 + 1]);
        memcpy(out + a * width, hidden + (size_t)token * width, width * sizeof(float));
    }
}

/* expert_project_q4_k / q6_k (ops.metal:2042-2066): out[a,r] = sum_k
 * in[a,k] * W[expert(a)*rows + r, k]; f32 sequential accumulation here, the
 * result rounded to the storage dtype (src/ops/transformer.rs:3360-3380).
 * Assignments whose expert id is out of range produce 0. */
int fo_expert_project(uint32_t ggml_type, const uint8_t* packed, size_t experts, size_t rows,
                      size_t k, const float* x, const float* metadata, size_t assignments, float* y,
                      int weight_round, int out_round, int f64) {
    if (!fo_columns_ok(ggml_type, k)) return 1;
    size_t row_bytes = fo_row_bytes(ggml_type, k);
    float* w = (float*)malloc(k * sizeof(float));
    for (size_t a = 0; a < assignments; a++) {
        uint32_t expert = float_to_bits(metadata[a * 3]);
        for (size_t r = 0; r < rows; r++) {
            float result = 0.0f;
            if (expert < experts) {
                dequant_row(ggml_type, packed + ((size_t)expert * rows + r) * row_bytes, k, w);
                if (weight_round)
                    for (size_t c = 0; c < k; c++) w[c] = fo_round_storage(w[c], (uint32_t)weight_round);
                const float* xi = x + a * k;
                if (f64) {
                    double acc = 0.0;
                    for (size_t c = 0; c < k; c++) acc += (double)xi[c] * (double)w[c];
                    result = (float)acc;
                } else {
                    float acc = 0.0f;
                    for (size_t c = 0; c < k; c++) {
                        float p = xi[c] * w[c];
                        acc = acc + p;
                    }
                    result = acc;
                }
            }
            y[a * rows + r] = fo_round_storage(result, (uint32_t)out_round);
        }
    }
    free(w);
    return 0;
}

static float silu(float gate) {
    /* ops.metal:2229: the branch-stable form. */
    float s = gate >= 0.0f ? 1.0f / (1.0f + expf(-gate)) : expf(gate) / (1.0f + expf(gate));
    return gate * s;
}

/* expert_silu_mul (ops.metal:2223-2232): out[a,j] = store(round(silu(g))*u)
 * on packed [A, 2I] rows (gate first). */
void fo_expert_silu_mul(const float* in, size_t assignments, size_t intermediate, uint32_t dtype,
                        float* out) {
    for (size_t a = 0; a < assignments; a++) {
        const float* row = in + a * 2 * intermediate;
        for (size_t j = 0; j < intermediate; j++) {
            float activated = fo_round_storage(silu(row[j]), dtype);
            float product = activated * row[intermediate + j];
            out[a * intermediate + j] = fo_round_storage(product, dtype);
        }
    }
}

/* expert_combine (ops.metal:2234-2246): out[t,c] = sum over ranks, in
 * metadata order, of round(round(w)*v), f32 running total, stored rounded. */
void fo_expert_combine(const float* in, const float* metadata, size_t tokens, size_t hidden,
                       size_t top_k, uint32_t dtype, float* out) {
    for (size_t t = 0; t < tokens; t++) {
        for (size_t c = 0; c < hidden; c++) {
            float total = 0.0f;
            for (size_t rank = 0; rank < top_k; rank++) {
                size_t a = t * top_k + rank;
                float gate = fo_round_storage(metadata[a * 3 + 2], dtype);
                float value = in[a * hidden + c];
                float product = gate * value;
                total = total + fo_round_storage(product, dtype);
            }
            out[t * hidden + c] = fo_round_storage(total, dtype);
        }
    }
}

/* argmax_rows (src/metal/shaders/ops.metal:2438-2464), restated with its own
 * schedule so that rows holding NaN give the same (flagged) index: 1024
 * threads scan columns tid, tid + 1024, ...; groups of 32 threads merge by a
 * shuffle-down tree; thread 0 folds the 32 group results in order.  A later
 * candidate wins when it is greater, or equal with a lower index.  out[2*row]
 * = index, out[2*row + 1] = 1 when the row holds a non-finite value.  For
 * finite rows this is the first maximal index. */
void fo_argmax_rows(const float* logits, size_t rows, size_t width, uint32_t* out) {
    enum { THREADS = 1024, GROUP = 32 };
    static float best[THREADS];
    static uint32_t index[THREADS];
    for (size_t row = 0; row < rows; row++) {
        const float* x = logits + row * width;
        uint32_t bad = 0;
        for (uint32_t tid = 0; tid < THREADS; tid++) {
            best[tid] = -INFINITY;
            index[tid] = 0xffffffffu;
            for (size_t j = tid; j < width; j += THREADS) {
                float v = x[j];
                if (!isfinite(v)) bad = 1;
                if (v > best[tid] || index[tid] == 0xffffffffu) {
                    best[tid] = v;
                    index[tid] = (uint32_t)j;
                }
            }
        }
        for (uint32_t offset = GROUP / 2; offset > 0; offset /= 2) {
            /* shuffle_down reads the pre-step value of lane + offset; ascending tid
             * only ever reads lanes not yet rewritten in this step */
            for (uint32_t tid = 0; tid < THREADS; tid++) {
                uint32_t lane = tid % GROUP;
                uint32_t from = lane + offset < GROUP ? tid + offset : tid;
                float other = best[from];
                uint32_t other_index = index[from];
                if (other > best[tid] || (other == best[tid] && other_index < index[tid])) {
                    best[tid] = other;
                    index[tid] = other_index;
                }
            }
        }
        float b = best[0];
        uint32_t bi = index[0];
        for (uint32_t g = 1; g < THREADS / GROUP; g++) {
            float v = best[g * GROUP];
            uint32_t vi = index[g * GROUP];
            if (v > b || (v == b && vi < bi)) {
                b = v;
                bi = vi;
            }
        }
        out[2 * row] = bi;
        out[2 * row + 1] = bad;
    }
}

/* add_rmsnorm (src/metal/shaders/ops.metal:99-124): residual = the sum rounded
 * to the storage type, as a separate `add` stores it; normed = the reference's
 * CPU rmsnorm (src/reference.rs:23-35) of the residual: float64 mean of
 * squares, inv = 1 / sqrt(mean + eps), x * inv * w rounded once to f32.  The
 * caller compares the device's storage-rounded rows against it. */
void fo_add_rmsnorm(const float* a, const float* b, const float* weight, size_t rows, size_t width,
                    float eps, uint32_t dtype, float* residual, float* normed) {
    for (size_t r = 0; r < rows; r++) {
        double squares = 0.0;
        for (size_t j = 0; j < width; j++) {
            float x = fo_round_storage(a[r * width + j] + b[r * width + j], dtype);
            residual[r * width + j] = x;
            squares += (double)x * (double)x;
        }
        double inv = 1.0 / sqrt(squares / (double)width + (double)eps);
        for (size_t j = 0; j < width; j++)
            normed[r * width + j] = (float)((double)residual[r * width + j] * inv * (double)weight[j]);
    }
}

/* h_moe_map (src/metal/shaders/hybrid.metal:2321-2358): expert-major order of
 * routes, stable inside an expert.  offsets[experts + 1], sorted[routes],
 * position[routes]; routes whose id is not an expert are left untouched. */
void fo_moe_map(const uint32_t* ids, size_t experts, size_t routes, uint32_t* offsets, uint32_t* sorted,
                uint32_t* position) {
    uint32_t acc = 0;
    for (size_t e = 0; e < experts; e++) {
        offsets[e] = acc;
        for (size_t r = 0; r < routes; r++) acc += ids[r] == e ? 1u : 0u;
    }
    offsets[experts] = acc;
    for (size_t e = 0; e < experts; e++) {
        uint32_t at = offsets[e];
        for (size_t r = 0; r < routes; r++) {
            if (ids[r] == e) {
                sorted[at] = (uint32_t)r;
                position[r] = at;
                at++;
            }
        }
    }
}

/* h_moe_combine (src/metal/shaders/hybrid.metal:2372-2388), f32, each product
 * and sum rounded to f32 in rank order: out[t] = sum_s weights[t*used + s] *
 * down[row] + shared_gate[t] * shared[t], row = position[r] or r itself when
 * position is NULL. */
void fo_hybrid_combine(const float* down, const float* weights, const uint32_t* position, const float* shared,
                       const float* shared_gate, size_t hidden, size_t used, size_t tokens, float* out) {
    for (size_t t = 0; t < tokens; t++) {
        for (size_t i = 0; i < hidden; i++) {
            float acc = 0.0f;
            for (size_t s = 0; s < used; s++) {
                size_t r = t * used + s;
                size_t row = position ? position[r] : r;
                float product = weights[r] * down[row * hidden + i];
                acc = acc + product;
            }
            float tail = shared_gate[t] * shared[t * hidden + i];
            out[t * hidden + i] = acc + tail;
        }
    }
}
