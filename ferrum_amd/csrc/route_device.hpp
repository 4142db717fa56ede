// moe_route for one token by one wave (src/metal/shaders/ops.metal:1894-1967; the hybrid
// engine's h_moe_route, src/metal/shaders/hybrid.metal:2259-2319): shared by the routing
// kernel and by the projection that routes its one token itself.
#pragma once

#include "device_utils.hpp"
#include "internal.hpp"

namespace fh {

constexpr int kMaxPerLane = 16;  // experts <= 1024
constexpr int kMaxTopK = 16;

__device__ __forceinline__ uint32_t total_order_key(float x) {
    uint32_t bits = __float_as_uint(x);
    return (bits & 0x80000000u) ? ~bits : (bits ^ 0x80000000u);
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
    const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
    return other > v ? other : v;
}

// Maximum over the 64 lanes as a wave-uniform value; every lane must be active.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = dpp_max_u32<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_max_u32<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_max_u32<0x141>(v);  // row_half_mirror
    v = dpp_max_u32<0x140>(v);  // row_mirror: every lane now holds its row's maximum
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

// One wave per token.  Scores are computed by all lanes in parallel; the
// softmax normaliser is then summed by one lane in expert order so it carries
// the same f32 rounding as a sequential host loop.  Selection runs top_k
// rounds of a wave-wide arg-max over (total-order key, lower id wins).  With one
// token the kernel is one wave's dependent instruction stream, so its length is
// its duration: reductions are DPP, owners are found by ballot.
// `local`: when set, the token's top_k records {id, token, weight} are also written there (LDS of
// the calling workgroup); `publish`: whether this wave writes the outputs in device memory.
template <int kPerLane>   // experts <= 64 * kPerLane
__device__ __forceinline__ void route_token(const RouteTokenArgs& a, uint32_t token, uint32_t lane, float* scores_lds,
                                            float* local = nullptr, bool publish = true) {
    const void* logits = a.logits;
    const uint32_t logits_dtype = a.logits_dtype;
    const float* bias = a.bias;
    float* metadata = a.metadata;
    const uint32_t experts = a.experts, top_k = a.top_k, sigmoid = a.sigmoid, normalize = a.normalize;
    const float eps = a.eps, scaling = a.scaling;
    const uint32_t rank_order = a.rank_order;
    const void* gate_x = a.gate_x;
    const uint32_t gate_x_dtype = a.gate_x_dtype;
    const float* gate_w = a.gate_w;
    const uint32_t hidden = a.hidden;
    float* shared_gate = a.shared_gate;
    float* ids_out = a.ids_out;
    float* weights_out = a.weights_out;
    const size_t base = (size_t)token * experts;

    float score[kPerLane];
    float logit[kPerLane];
    float maximum = -INFINITY;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        uint32_t e = lane + 64u * i;
        logit[i] = e < experts ? load_as_f32(logits, base + e, logits_dtype) : -INFINITY;
        maximum = fmaxf(maximum, logit[i]);
    }
    if (sigmoid) {
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) score[i] = 1.f / (1.f + expf(-logit[i]));
    } else {
        maximum = wave_max(maximum);
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
            uint32_t e = lane + 64u * i;
            score[i] = expf(logit[i] - maximum);
            if (e < ((experts + 3u) & ~3u)) scores_lds[e] = e < experts ? score[i] : 0.f;
        }
        // the wave reads what its own lanes wrote: LDS operations of a wave complete in order
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
        float normalizer = 0.f;
        if (lane == 0) {
            // expert order, four per LDS read; the zero padding does not change the sum
            // the reads of a batch are issued together; the additions stay in expert order
            const float4* in = reinterpret_cast<const float4*>(scores_lds);
            const uint32_t quads = (experts + 3u) / 4u;
            uint32_t q = 0;
            for (; q + 8 <= quads; q += 8) {
                float4 v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = in[q + i];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    normalizer += v[i].x;
                    normalizer += v[i].y;
                    normalizer += v[i].z;
                    normalizer += v[i].w;
                }
            }
            for (; q < quads; ++q) {
                const float4 v = in[q];
                normalizer += v.x;
                normalizer += v.y;
                normalizer += v.z;
                normalizer += v.w;
            }
        }
        normalizer = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(normalizer)));
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) score[i] = score[i] / normalizer;
    }

    // Selection: top_k rounds of a wave-wide arg-max over the total-order key of the
    // biased score, the lower expert id winning ties.  The maximum is a 32-bit DPP
    // reduction; its owner is then found by ballot: expert ids grow with the slot i first
    // and the lane second, so the lowest id is the first lane of the first slot that holds it.
    uint32_t key[kPerLane];
    uint32_t alive = 0;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const uint32_t e = lane + 64u * i;
        const float selection = score[i] + (bias != nullptr && e < experts ? bias[e] : 0.f);
        key[i] = e < experts ? total_order_key(selection) : 0u;
        alive |= e < experts ? 1u << i : 0u;
    }

    uint32_t my_id = 0xffffffffu;   // lane r < top_k: the expert of rank r and its raw score
    float my_score = 0.f;
    float selected_sum = 0.f;
#pragma unroll
    for (int rank = 0; rank < kMaxTopK; ++rank) {
        if ((uint32_t)rank < top_k) {
            uint32_t best = 0;
#pragma unroll
            for (int i = 0; i < kPerLane; ++i) best = key[i] > best ? key[i] : best;
            best = wave_max_u32(best);
            uint32_t slot = kPerLane;
            unsigned long long owners = 0ull;
#pragma unroll
            for (int i = kPerLane - 1; i >= 0; --i) {
                const unsigned long long mask = __ballot(((alive >> i) & 1u) != 0 && key[i] == best);
                if (mask != 0ull) {
                    slot = (uint32_t)i;
                    owners = mask;
                }
            }
            const uint32_t owner = (uint32_t)__ffsll((long long)owners) - 1u;
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < kPerLane; ++i) {
                if ((uint32_t)i == slot && lane == owner) {
                    mine = score[i];   // the raw score (bias excluded)
                    key[i] = 0u;
                    alive &= ~(1u << i);
                }
            }
            const float chosen = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mine), owner));
            selected_sum += chosen;
            if (lane == (uint32_t)rank) {
                my_id = owner + 64u * slot;
                my_score = chosen;
            }
        }
    }
    const float denominator = selected_sum + eps;

    // Rows are written in expert-id order (lane r places entry r at the number of selected
    // ids below its own), or in selection order for the hybrid engine's router.
    uint32_t position = 0;
#pragma unroll
    for (int other = 0; other < kMaxTopK; ++other) {
        if ((uint32_t)other < top_k) {
            const uint32_t id = (uint32_t)__builtin_amdgcn_readlane((int)my_id, other);
            position += id < my_id ? 1u : 0u;
        }
    }
    if (rank_order) position = lane;
    if (lane < top_k) {
        float weight = my_score;
        if (normalize) weight = weight / denominator;
        weight = weight * scaling;
        const size_t slot = (size_t)token * top_k + position;
        if (local != nullptr) {
            local[3 * position + 0] = __uint_as_float(my_id);
            local[3 * position + 1] = __uint_as_float(token);
            local[3 * position + 2] = weight;
        }
        if (metadata != nullptr && publish) {
            float* out = metadata + slot * 3;
            out[0] = __uint_as_float(my_id);
            out[1] = __uint_as_float(token);
            out[2] = weight;
        }
        // the hybrid engine's layout: ids and weights as two [tokens, top_k] arrays
        if (ids_out != nullptr && publish) ids_out[slot] = __uint_as_float(my_id);
        if (weights_out != nullptr && publish) weights_out[slot] = weight;
    }

    // Shared-expert gate of h_moe_route (src/metal/shaders/hybrid.metal:2259-2319):
    // sigmoid(dot(x[token], gate_w)), or 1 without a gate vector.
    if (shared_gate != nullptr && publish) {
        float dot = 0.f;
        if (gate_w != nullptr) {
            for (uint32_t i = lane; i < hidden; i += 64)
                dot += load_as_f32(gate_x, (size_t)token * hidden + i, gate_x_dtype) * gate_w[i];
            dot = wave_sum(dot);
        }
        if (lane == 0) shared_gate[token] = gate_w != nullptr ? 1.f / (1.f + expf(-dot)) : 1.f;
    }
}

}  // namespace fh
