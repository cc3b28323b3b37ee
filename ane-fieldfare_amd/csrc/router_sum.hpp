// The pinned per-lane accumulation of the router logits, shared by the router kernels and by the launch that
// routes and runs gate/up in one go: lane l of a 64-lane wave owns the elements k = 256 i + 4 l + j (j = 0..3)
// of an expert row, accumulated with fmaf in increasing i, then j (the CPU restatement reproduces every logit bit
// for bit, which makes the selected indices exact).
#pragma once

#include "common.hpp"

namespace ffmoe {
namespace {

constexpr int kChunkTokens = 4;      // token rows a wave keeps in flight at once

template <bool W_F32>
__device__ __forceinline__ void load_w4(const void *w_, size_t off, bool ok, float (&out)[4]) {
    if (!ok) {
        out[0] = out[1] = out[2] = out[3] = 0.0f;
        return;
    }
    if (W_F32) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(w_) + off);
        out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3];
    } else {
        const uint2 v = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(w_) + off);
        out[0] = bf16lo_to_f32(v.x); out[1] = bf16hi_to_f32(v.x);
        out[2] = bf16lo_to_f32(v.y); out[3] = bf16hi_to_f32(v.y);
    }
}

// Four bf16 inputs starting at element `off` of a row that needs 2-byte alignment only.
template <bool X_ALIGNED>
__device__ __forceinline__ uint2 load_x4(const uint16_t *p) {
    if (X_ALIGNED) return *reinterpret_cast<const uint2 *>(p);
    uint2 r;
    r.x = (uint32_t)p[0] | ((uint32_t)p[1] << 16);
    r.y = (uint32_t)p[2] | ((uint32_t)p[3] << 16);
    return r;
}

// Per-lane accumulation shared by both logits kernels: sub-accumulator `s` of lane `lane` over the
// elements k = 1024 i + 256 s + 4 lane + j, i ascending then j, for kChunkTokens token rows at once.
// XK: how the input rows arrive - 0: bf16, rows 2-byte aligned only; 1: bf16, 8-byte aligned; 2: FP16, 8-byte aligned.
template <bool W_F32, int XK>
__device__ __forceinline__ void accumulate_sub(const void *__restrict__ w_, const uint16_t *__restrict__ es,
                                               const uint16_t *__restrict__ x, uint32_t x_stride, uint32_t e,
                                               uint32_t d, uint32_t s, uint32_t lane, uint32_t t0, uint32_t t_last,
                                               float (&acc)[kChunkTokens]) {
    const uint32_t steps = (d + 1023) / 1024;
    // Four steps at a time: all their loads (weights, scale, token rows) are requested before the first
    // product, from clamped addresses so that no load sits behind a branch; the sums then run in the pinned
    // order. (A load per loop turn behind `if (k < d)` is a serial chain of memory round trips in a kernel
    // that is nothing but latency.)
    constexpr int kBatch = 4;
    for (uint32_t i0 = 0; i0 < steps; i0 += kBatch) {
        float wv[kBatch][4];
        uint2 ev[kBatch], xv[kBatch][kChunkTokens];
        bool live[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const uint32_t k = 1024 * (i0 + b) + 256 * s + 4 * lane;
            live[b] = k < d;
            const uint32_t kc = live[b] ? k : 0;
            load_w4<W_F32>(w_, (size_t)e * d + kc, true, wv[b]);
            ev[b] = es ? *reinterpret_cast<const uint2 *>(es + kc) : make_uint2(0x3F803F80u, 0x3F803F80u);
#pragma unroll
            for (int r = 0; r < kChunkTokens; ++r) {
                // rows past the last token re-read it: same arithmetic, result unused
                const uint32_t row = min(t0 + r, t_last);
                xv[b][r] = load_x4<XK != 0>(x + (size_t)row * x_stride + kc);
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            if (live[b]) {
                const float sc[4] = {bf16lo_to_f32(ev[b].x), bf16hi_to_f32(ev[b].x), bf16lo_to_f32(ev[b].y), bf16hi_to_f32(ev[b].y)};
#pragma unroll
                for (int r = 0; r < kChunkTokens; ++r) {
                    const float xf[4] = {Act<XK == 2>::lo(xv[b][r].x), Act<XK == 2>::hi(xv[b][r].x), Act<XK == 2>::lo(xv[b][r].y),
                                         Act<XK == 2>::hi(xv[b][r].y)};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // x * effective_scale: 8 or 11 significant bits times 8, exact in fp32 (moe.metal:96-97)
                        const float xe = es ? xf[j] * sc[j] : xf[j];
                        acc[r] = __builtin_fmaf(wv[b][j], xe, acc[r]);
                    }
                }
            }
        }
    }
}

// The four sub-accumulators of a lane and the 64 lanes of one (token, expert) pair: (s0 + s1) + (s2 + s3), then the
// xor-butterfly. `part` = [sub-accumulator][token][lane].
__device__ __forceinline__ float router_finish(const float (*part)[kChunkTokens][64], int r, uint32_t lane) {
    return wave_butterfly_sum((part[0][r][lane] + part[1][r][lane]) + (part[2][r][lane] + part[3][r][lane]));
}

}  // namespace
}  // namespace ffmoe
