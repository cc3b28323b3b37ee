// Router: logits in a pinned summation order, then top-k select + softmax weights.
//
// Replaces router_gemv_gemma4_* and router_topk_select_k8* (Metal/MoE/moe.metal:65-319) and
// prefill_router_gemma4_block (Metal/Prefill/prefill.metal:447-542).
//
// Summation order (fixed so that a CPU restatement reproduces every logit bit for bit, which makes the
// selected indices exact): lane l of a 64-lane wave accumulates k = l + 64 i for increasing i with
// fmaf, then a xor-butterfly (masks 32..1) of plain adds combines the 64 partials.
#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {
namespace {

constexpr int kRouterTokens = 16;   // tokens per block row

template <bool W_F32>
__global__ __launch_bounds__(256) void router_logits_kernel(const void *__restrict__ w_, const uint16_t *__restrict__ es,
                                                            const uint16_t *__restrict__ x, uint32_t x_stride,
                                                            uint32_t t, uint32_t n_experts, uint32_t d,
                                                            float *__restrict__ logits) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t e = blockIdx.x * 4 + wave;
    const uint32_t t0 = blockIdx.y * kRouterTokens;
    if (e >= n_experts) return;
    const uint32_t nt = min((uint32_t)kRouterTokens, t - t0);
    float acc[kRouterTokens];
#pragma unroll
    for (int r = 0; r < kRouterTokens; ++r) acc[r] = 0.0f;
    const uint32_t steps = d / 64;
    for (uint32_t i = 0; i < steps; ++i) {
        const uint32_t k = lane + 64 * i;
        float wv;
        if (W_F32) wv = reinterpret_cast<const float *>(w_)[(size_t)e * d + k];
        else wv = bf16_to_f32(reinterpret_cast<const uint16_t *>(w_)[(size_t)e * d + k]);
        const float sc = es ? bf16_to_f32(es[k]) : 1.0f;
#pragma unroll
        for (int r = 0; r < kRouterTokens; ++r) {
            // rows past the block's last token re-read that token: same arithmetic, result unused
            const uint32_t row = t0 + min((uint32_t)r, nt - 1);
            float xv = bf16_to_f32(x[(size_t)row * x_stride + k]);
            if (es) xv = xv * sc;     // product of two bf16 values: exact in fp32 (moe.metal:96-97)
            acc[r] = __builtin_fmaf(wv, xv, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < kRouterTokens; ++r) {
        const float v = wave_butterfly_sum(acc[r]);
        if (lane == 0 && (uint32_t)r < nt) logits[(size_t)(t0 + r) * n_experts + e] = v;
    }
}

__device__ __forceinline__ uint32_t orderable(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One wave per token. Candidate e lives in lane e % 64, slot e / 64 (E <= 256). top_k rounds of a
// wave-wide argmax over the total order (score desc, index asc); scores <= -inf and NaN are never
// taken; empty rounds give (index 0, -inf) and weight 0 (moe.metal:194-236).
__global__ __launch_bounds__(64) void router_topk_kernel(const float *__restrict__ logits,
                                                         const uint16_t *__restrict__ per_expert_scale,
                                                         uint32_t n_experts, uint32_t top_k,
                                                         uint32_t *__restrict__ out_idx, uint16_t *__restrict__ out_w) {
    const uint32_t lane = threadIdx.x, tok = blockIdx.x;
    const float *row = logits + (size_t)tok * n_experts;
    unsigned long long key[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t e = c * 64 + lane;
        float v = e < n_experts ? row[e] : -INFINITY;
        const bool live = (v > -INFINITY);   // false for NaN and -inf
        key[c] = live ? (((unsigned long long)orderable(v) << 32) | (0xFFFFFFFFu - e)) : 0ull;
    }
    uint32_t top_idx[8];
    float top_score[8];
    for (uint32_t r = 0; r < top_k; ++r) {
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
            top_score[r] = row[e];
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (key[c] == best) key[c] = 0ull;
        }
    }
    if (lane != 0) return;
    const float max_s = top_score[0];
    float sum = 0.0f, ex[8];
    for (uint32_t i = 0; i < top_k; ++i) {
        ex[i] = expf(top_score[i] - max_s);
        sum += ex[i];
    }
    for (uint32_t i = 0; i < top_k; ++i) {
        const float gain = per_expert_scale ? bf16_to_f32(per_expert_scale[top_idx[i]]) : 1.0f;
        out_idx[(size_t)tok * top_k + i] = top_idx[i];
        out_w[(size_t)tok * top_k + i] = f32_to_bf16(ex[i] / sum * gain);
    }
}

}  // namespace

hipError_t launch_router(hipStream_t s, RouterWeights rw, const uint16_t *x, uint32_t x_stride, uint32_t t,
                         uint32_t n_experts, uint32_t d, uint32_t top_k, float *logits, uint32_t *out_idx,
                         uint16_t *out_w, KernelTimer *timer) {
    timer->begin(s);
    const dim3 grid((n_experts + 3) / 4, (t + kRouterTokens - 1) / kRouterTokens);
    if (rw.w_is_f32)
        hipLaunchKernelGGL(router_logits_kernel<true>, grid, dim3(256), 0, s, rw.w, rw.effective_scale, x,
                           x_stride, t, n_experts, d, logits);
    else
        hipLaunchKernelGGL(router_logits_kernel<false>, grid, dim3(256), 0, s, rw.w, rw.effective_scale, x,
                           x_stride, t, n_experts, d, logits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_ROUTER_LOGITS);
    hipLaunchKernelGGL(router_topk_kernel, dim3(t), dim3(64), 0, s, logits, rw.per_expert_scale, n_experts,
                       top_k, out_idx, out_w);
    timer->mark(s, FFMOE_K_ROUTER_TOPK);
    timer->finish();
    return hipGetLastError();
}

}  // namespace ffmoe
