// Top-k select + softmax weights of one row of router logits by one wave.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace ffmoe {
namespace {

__device__ __forceinline__ uint32_t orderable(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Largest value of an unsigned quantity over the 64 lanes (zero if all are zero), the same in every lane:
// four shifts inside each row of 16 lanes, two row broadcasts, one lane read. These are register-to-register
// moves of a few cycles each; a butterfly of __shfl_xor would go through the LDS crossbar at more than a
// hundred cycles a step, and the eight rounds of a select are one dependent chain.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    auto shifted = [](uint32_t x, auto ctrl, auto rows) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, decltype(ctrl)::value, decltype(rows)::value, 0xF, false);
    };
    using std::integral_constant;
    v = max(v, shifted(v, integral_constant<int, 0x111>{}, integral_constant<int, 0xF>{}));   // row_shr:1
    v = max(v, shifted(v, integral_constant<int, 0x112>{}, integral_constant<int, 0xF>{}));   // row_shr:2
    v = max(v, shifted(v, integral_constant<int, 0x114>{}, integral_constant<int, 0xF>{}));   // row_shr:4
    v = max(v, shifted(v, integral_constant<int, 0x118>{}, integral_constant<int, 0xF>{}));   // row_shr:8: lane 15 of a row holds the row
    v = max(v, shifted(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{}));   // row_bcast:15 into rows 1 and 3
    v = max(v, shifted(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{}));   // row_bcast:31 into rows 2 and 3
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// One wave: candidate e lives in lane e % 64, slot e / 64 (E <= 256). top_k rounds of a wave-wide
// argmax over the total order (score desc, index asc): the largest score by wave_max_u32, then the lowest
// index that holds it by ballots, slot by slot. Scores <= -inf and NaN are never taken; empty rounds give
// (index 0, -inf) and weight 0 (moe.metal:194-236). The weights: lane i takes exp(score_i - max) and the
// division for rank i, the sum runs over the ranks in order as a serial loop would.
// The three parts of a row's select: load, select, store.
struct TopkRow {
    uint32_t key[4];        // in: orderable score of candidate 64 c + lane, 0 = not a candidate
    float ex, sum;          // out: lane i: exp(score_i - max); the sum over the ranks in order
    uint32_t idx;           // out: lane i: index of rank i
};

__device__ __forceinline__ void topk_load(TopkRow &t, const float *row, uint32_t n_experts, uint32_t lane) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t e = c * 64 + lane;
        const float v = e < n_experts ? row[e] : -INFINITY;
        t.key[c] = v > -INFINITY ? orderable(v) : 0u;     // the comparison is false for NaN and -inf (every candidate's key is above 0x007FFFFF)
    }
}

// SLOTS: how many of the four key slots can hold a candidate (E <= 64 SLOTS).
template <int SLOTS = 4>
__device__ __forceinline__ void topk_select(TopkRow &t, uint32_t top_k, uint32_t lane) {
    float mine = -INFINITY, max_s = -INFINITY;      // lane i: score of rank i
    t.idx = 0;
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        if (r < top_k) {
            uint32_t mine_best = t.key[0];
#pragma unroll
            for (int c = 1; c < SLOTS; ++c) mine_best = max(mine_best, t.key[c]);
            const uint32_t best = wave_max_u32(mine_best);
            uint32_t e = 0;
            float score = -INFINITY;
            if (best != 0u) {
                // recover the score from the key: orderable() is a bijection
                score = __uint_as_float((best & 0x80000000u) ? (best & 0x7FFFFFFFu) : ~best);
                bool found = false;
#pragma unroll
                for (int c = 0; c < SLOTS; ++c) {
                    const unsigned long long holders = __ballot(t.key[c] == best);
                    if (!found && holders != 0ull) {
                        const uint32_t l = (uint32_t)__builtin_ctzll(holders);
                        e = c * 64 + l;
                        if (lane == l) t.key[c] = 0u;
                        found = true;
                    }
                }
            }
            if (r == 0) max_s = score;
            if (lane == r) {
                mine = score;
                t.idx = e;
            }
        }
    }
    t.ex = expf(mine - max_s);
    t.sum = 0.0f;
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i)
        if (i < top_k) t.sum += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(t.ex), (int)i));
}

__device__ __forceinline__ void topk_store(const TopkRow &t, const uint16_t *__restrict__ per_expert_scale, uint32_t top_k,
                                           uint32_t *__restrict__ out_idx, uint16_t *__restrict__ out_w, uint32_t lane,
                                           bool w_f16) {
    if (lane < top_k) {
        const float gain = per_expert_scale ? bf16_to_f32(per_expert_scale[t.idx]) : 1.0f;
        const float weight = t.ex / t.sum * gain;
        out_idx[lane] = t.idx;
        out_w[lane] = w_f16 ? Act<true>::round(weight) : Act<false>::round(weight);
    }
}

__device__ __forceinline__ void wave_topk(const float *row, const uint16_t *__restrict__ per_expert_scale,
                                          uint32_t n_experts, uint32_t top_k, uint32_t *__restrict__ out_idx,
                                          uint16_t *__restrict__ out_w, uint32_t lane, bool w_f16) {
    TopkRow t;
    topk_load(t, row, n_experts, lane);
    if (n_experts <= 128) topk_select<2>(t, top_k, lane);
    else topk_select<4>(t, top_k, lane);
    topk_store(t, per_expert_scale, top_k, out_idx, out_w, lane, w_f16);
}

}  // namespace
}  // namespace ffmoe
