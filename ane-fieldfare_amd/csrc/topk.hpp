// Top-k select + softmax weights of one row of router logits by one wave; shared by the router's own
// kernel and by the gate/up kernel when it routes small blocks of rows itself.
#pragma once

#include "common.hpp"

namespace ffmoe {
namespace {

__device__ __forceinline__ uint32_t orderable(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One wave: candidate e lives in lane e % 64, slot e / 64 (E <= 256). top_k rounds of a wave-wide
// argmax over the total order (score desc, index asc); scores <= -inf and NaN are never taken; empty
// rounds give (index 0, -inf) and weight 0 (moe.metal:194-236). 
__device__ __forceinline__ void wave_topk(const float *row, const uint16_t *__restrict__ per_expert_scale,
                                          uint32_t n_experts, uint32_t top_k, uint32_t *__restrict__ out_idx,
                                          uint16_t *__restrict__ out_w, uint32_t lane) {
    unsigned long long key[4];
    float val[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t e = c * 64 + lane;
        val[c] = e < n_experts ? row[e] : -INFINITY;
        const bool live = (val[c] > -INFINITY);   // false for NaN and -inf
        key[c] = live ? (((unsigned long long)orderable(val[c]) << 32) | (0xFFFFFFFFu - e)) : 0ull;
    }
    uint32_t top_idx[8];
    float top_score[8];
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        if (r < top_k) {
            unsigned long long best = key[0];
#pragma unroll
            for (int c = 1; c < 4; ++c) best = key[c] > best ? key[c] : best;
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) {
                const unsigned long long o = __shfl_xor(best, m, 64);
                best = o > best ? o : best;
            }
            if (best == 0ull) {
                top_idx[r] = 0;
                top_score[r] = -INFINITY;
            } else {
                const uint32_t e = 0xFFFFFFFFu - (uint32_t)best;
                top_idx[r] = e;
                // recover the score from the key: orderable() is a bijection
                const uint32_t o = (uint32_t)(best >> 32);
                top_score[r] = __uint_as_float((o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o);
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (key[c] == best) key[c] = 0ull;
            }
        }
    }
    if (lane != 0) return;
    const float max_s = top_score[0];
    float sum = 0.0f, ex[8];
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
        if (i < top_k) {
            ex[i] = expf(top_score[i] - max_s);
            sum += ex[i];
        }
    }
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
        if (i < top_k) {
            const float gain = per_expert_scale ? bf16_to_f32(per_expert_scale[top_idx[i]]) : 1.0f;
            out_idx[i] = top_idx[i];
            out_w[i] = f32_to_bf16(ex[i] / sum * gain);
        }
    }
}

}  // namespace
}  // namespace ffmoe
