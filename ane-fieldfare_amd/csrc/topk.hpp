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

// The weights' part of a select, shared by its two forms: lane i < top_k holds the score of rank i (`mine`; -inf
// for an empty rank), `max_s` is rank 0's score in every lane.
__device__ __forceinline__ void topk_weights(TopkRow &t, float mine, float max_s, uint32_t top_k) {
    t.ex = expf(mine - max_s);
    t.sum = 0.0f;
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i)
        if (i < top_k) t.sum += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(t.ex), (int)i));
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
    topk_weights(t, mine, max_s, top_k);
}

// The same select by the four waves of a block together (moe.metal:186-237 ranks with a SIMD-wide pass as well):
// instead of top_k dependent rounds of a wave-wide maximum, every candidate's rank is COUNTED - how many candidates
// have a larger key - and the candidates of rank < top_k go to their places. Every wave holds the row's keys (t.key,
// identical in the four waves); wave v counts over a quarter of the candidates (two vector instructions per pair of
// keys: compare, add with carry), the partial counts meet in `cnt` ([wave][slot][lane], LDS) behind one barrier, and
// wave `finisher` adds them, moves the winners to lanes 0 .. top_k - 1 by cross-lane writes and computes the weights.
// Equal keys (two experts with the same logit bits) get equal counts; the total order breaks such a tie by index,
// so when two candidates land on one rank - seen as fewer filled ranks than placed candidates - the finisher runs
// topk_select instead. Same routes and weights as topk_select bit for bit either way: without a tie the ranks are
// those of the total order, and the weights come from the same code. Returns in `t` for the finisher wave only.
// Every wave of the block has to call it.
template <int SLOTS>
__device__ __forceinline__ void block_topk_select(TopkRow &t, uint32_t top_k, uint32_t lane, uint32_t wave, uint32_t finisher,
                                                  uint32_t (*cnt)[4][64]) {
    constexpr uint32_t kPerWave = 16 * SLOTS;                 // candidates a wave counts over
    const uint32_t first = wave * kPerWave, c_other = __builtin_amdgcn_readfirstlane(first >> 6);
    const uint32_t l0 = __builtin_amdgcn_readfirstlane(first & 63);
    uint32_t theirs = t.key[0];
#pragma unroll
    for (int c = 1; c < SLOTS; ++c) theirs = c_other == (uint32_t)c ? t.key[c] : theirs;
    // a non-candidate's key is 0 and is larger than nothing; what is counted for a lane's own empty slot is never used
    uint32_t count[SLOTS];
#pragma unroll
    for (int c = 0; c < SLOTS; ++c) count[c] = 0;
#pragma unroll 8
    for (uint32_t i = 0; i < kPerWave; ++i) {
        const uint32_t ko = (uint32_t)__builtin_amdgcn_readlane((int)theirs, (int)(l0 + i));
#pragma unroll
        for (int c = 0; c < SLOTS; ++c) count[c] += ko > t.key[c] ? 1u : 0u;
    }
#pragma unroll
    for (int c = 0; c < SLOTS; ++c) cnt[wave][c][lane] = count[c];
    lds_barrier();
    if (wave != finisher) return;
    uint32_t got_key = 0, got_idx = 0, placed_n = 0;
#pragma unroll
    for (int c = 0; c < SLOTS; ++c) {
        const uint32_t rank = cnt[0][c][lane] + cnt[1][c][lane] + cnt[2][c][lane] + cnt[3][c][lane];
        const bool placed = t.key[c] != 0u && rank < top_k;
        placed_n += (uint32_t)__popcll(__ballot(placed));
        // a cross-lane write: lane `rank` receives the value, lanes nobody writes to receive 0; the others aim at
        // lane 63, which holds no rank (top_k <= 8)
        const int to = (int)((placed ? rank : 63u) * 4u);
        got_key |= (uint32_t)__builtin_amdgcn_ds_permute(to, (int)(placed ? t.key[c] : 0u));
        got_idx |= (uint32_t)__builtin_amdgcn_ds_permute(to, (int)(placed ? (uint32_t)c * 64u + lane : 0u));
    }
    const bool have = lane < top_k && got_key != 0u;
    if ((uint32_t)__popcll(__ballot(have)) != placed_n) {      // two candidates on one rank: equal keys
        topk_select<SLOTS>(t, top_k, lane);
        return;
    }
    // recover the score from the key: orderable() is a bijection
    const float mine = have ? __uint_as_float((got_key & 0x80000000u) ? (got_key & 0x7FFFFFFFu) : ~got_key) : -INFINITY;
    t.idx = have ? got_idx : 0u;
    const float max_s = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(mine), 0));
    topk_weights(t, mine, max_s, top_k);
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
