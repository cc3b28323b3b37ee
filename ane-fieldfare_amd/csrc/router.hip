// Router: logits in a pinned summation order, then top-k select + softmax weights.
//
// Replaces router_gemv_gemma4_* and router_topk_select_k8* (Metal/MoE/moe.metal:65-319) and
// prefill_router_gemma4_block (Metal/Prefill/prefill.metal:447-542).
//
// Summation order (fixed so that a CPU restatement reproduces every logit bit for bit, which makes the
// selected indices exact): lane l of a 64-lane wave owns the elements k = 256 i + 4 l + j (j = 0..3) and
// accumulates them with fmaf in increasing i, then j; a xor-butterfly (masks 32..1) of plain adds
// combines the 64 partials. Four consecutive elements per lane make every load 8 bytes wide.
#include "common.hpp"
#include "kernels.hpp"
#include "router_sum.hpp"
#include "topk.hpp"

namespace ffmoe {
namespace {

// Decode / verify router logits (T <= 16). grid = (E, ceil(T / 4)); the four waves of a block are the
// four sub-accumulators of one expert row for four tokens; wave 0 combines them. (A variant whose last
// block also selected the top-k behind a device-scope counter measured 2.5x slower: every block paid
// for the same-address atomic and the L2 write-back of its release fence.)
template <bool W_F32, int XK>
__global__ __launch_bounds__(256) void router_small_kernel(const void *__restrict__ w_, const uint16_t *__restrict__ es,
                                                           const uint16_t *__restrict__ x, uint32_t x_stride,
                                                           uint32_t t, uint32_t n_experts, uint32_t d,
                                                           float *__restrict__ logits) {
    __shared__ float s_part[4][kChunkTokens][64];
    const uint32_t lane = threadIdx.x & 63, s = threadIdx.x >> 6;
    const uint32_t e = blockIdx.x;
    const uint32_t t0 = blockIdx.y * kChunkTokens;
    const uint32_t t_end = min(t, t0 + kChunkTokens);
    float acc[kChunkTokens] = {0.f, 0.f, 0.f, 0.f};
    accumulate_sub<W_F32, XK>(w_, es, x, x_stride, e, d, s, lane, t0, t_end - 1, acc);
#pragma unroll
    for (int r = 0; r < kChunkTokens; ++r) s_part[s][r][lane] = acc[r];
    __syncthreads();
    if (s != 0) return;
#pragma unroll
    for (int r = 0; r < kChunkTokens; ++r) {
        const float v = router_finish(s_part, r, lane);
        if (lane == 0 && t0 + r < t_end) logits[(size_t)(t0 + r) * n_experts + e] = v;
    }
}

// Prefill router logits: a register-tiled fp32 GEMM that keeps the pinned order. A block owns a tile of
// 8 tokens x 8 experts; its four waves are the four sub-accumulators, each walking its own k-blocks with
// the next block's operands already in flight, so every x and W load feeds 8 rows of fmaf. The partials
// meet in LDS (pairwise first, which halves the space and lets three blocks share a CU), each wave
// then finishes 16 of the 64 outputs: (s0 + s1) + (s2 + s3) per lane and the
// xor-butterfly done as a halving exchange (a lane keeps half of its values and receives the partner's
// matching half; fp addition is commutative, so every sum has the same operands as the full butterfly).
// Blocks are numbered so that all expert groups of one token group run on the same XCD and share its L2.
constexpr int kTileTok = 8, kTileExp = 8;

template <bool W_F32> struct WRaw { uint2 v; };
template <> struct WRaw<true> { f32x4 v; };

template <bool W_F32, int XK, bool HAS_ES>
__global__ __launch_bounds__(256) void router_tile_kernel(const void *__restrict__ w_, const uint16_t *__restrict__ es,
                                                          const uint16_t *__restrict__ x, uint32_t x_stride,
                                                          uint32_t t, uint32_t n_experts, uint32_t d,
                                                          uint32_t n_egroups, uint32_t n_tgroups,
                                                          float *__restrict__ logits) {
    __shared__ float s_part[2][kTileTok * kTileExp][64];
    const uint32_t lane = threadIdx.x & 63, s = threadIdx.x >> 6;
    const uint32_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const uint32_t tg = (slot / n_egroups) * 8 + xcd, eg = slot % n_egroups;
    if (tg >= n_tgroups) return;
    const uint32_t t0 = tg * kTileTok, e0 = eg * kTileExp;

    const uint16_t *xrow[kTileTok];
    size_t wrow[kTileExp];
#pragma unroll
    for (int r = 0; r < kTileTok; ++r) xrow[r] = x + (size_t)min(t0 + r, t - 1) * x_stride;
#pragma unroll
    for (int c = 0; c < kTileExp; ++c) wrow[c] = (size_t)min(e0 + c, n_experts - 1) * d;

    float acc[kTileTok][kTileExp];
#pragma unroll
    for (int r = 0; r < kTileTok; ++r)
#pragma unroll
        for (int c = 0; c < kTileExp; ++c) acc[r][c] = 0.0f;

    WRaw<W_F32> wn[kTileExp];
    uint2 xn[kTileTok], en = make_uint2(0x3F803F80u, 0x3F803F80u);
    auto fetch = [&](uint32_t k) {
        if (k >= d) return;
#pragma unroll
        for (int c = 0; c < kTileExp; ++c) {
            if (W_F32) wn[c].v = *reinterpret_cast<const decltype(wn[c].v) *>(reinterpret_cast<const float *>(w_) + wrow[c] + k);
            else wn[c].v = *reinterpret_cast<const decltype(wn[c].v) *>(reinterpret_cast<const uint16_t *>(w_) + wrow[c] + k);
        }
#pragma unroll
        for (int r = 0; r < kTileTok; ++r) xn[r] = load_x4<XK != 0>(xrow[r] + k);
        if (HAS_ES) en = *reinterpret_cast<const uint2 *>(es + k);
    };

    const uint32_t steps = (d + 1023) / 1024;
    uint32_t k = 256 * s + 4 * lane;
    fetch(k);
    for (uint32_t i = 0; i < steps; ++i, k += 1024) {
        const bool live = k < d;
        float wv[kTileExp][4];
        uint2 xc[kTileTok];
#pragma unroll
        for (int c = 0; c < kTileExp; ++c) {
            if constexpr (W_F32) {
                wv[c][0] = wn[c].v[0]; wv[c][1] = wn[c].v[1]; wv[c][2] = wn[c].v[2]; wv[c][3] = wn[c].v[3];
            } else {
                wv[c][0] = bf16lo_to_f32(wn[c].v.x); wv[c][1] = bf16hi_to_f32(wn[c].v.x);
                wv[c][2] = bf16lo_to_f32(wn[c].v.y); wv[c][3] = bf16hi_to_f32(wn[c].v.y);
            }
        }
#pragma unroll
        for (int r = 0; r < kTileTok; ++r) xc[r] = xn[r];
        const float sc[4] = {bf16lo_to_f32(en.x), bf16hi_to_f32(en.x), bf16lo_to_f32(en.y), bf16hi_to_f32(en.y)};
        if (i + 1 < steps) fetch(k + 1024);
        if (live) {
#pragma unroll
            for (int r = 0; r < kTileTok; ++r) {
                const float xf[4] = {Act<XK == 2>::lo(xc[r].x), Act<XK == 2>::hi(xc[r].x), Act<XK == 2>::lo(xc[r].y),
                                     Act<XK == 2>::hi(xc[r].y)};
                float xe[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) xe[j] = HAS_ES ? xf[j] * sc[j] : xf[j];   // exact: at most 11 + 8 significant bits
#pragma unroll
                for (int c = 0; c < kTileExp; ++c)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[r][c] = __builtin_fmaf(wv[c][j], xe[j], acc[r][c]);
            }
        }
    }
    // (s0 + s1) and (s2 + s3) first, each in the even wave of the pair, through two 16 KiB regions
    if (s & 1) {
#pragma unroll
        for (int r = 0; r < kTileTok; ++r)
#pragma unroll
            for (int c = 0; c < kTileExp; ++c) s_part[s >> 1][r * kTileExp + c][lane] = acc[r][c];
    }
    __syncthreads();
    if (!(s & 1)) {
#pragma unroll
        for (int r = 0; r < kTileTok; ++r)
#pragma unroll
            for (int c = 0; c < kTileExp; ++c) {
                float *cell = &s_part[s >> 1][r * kTileExp + c][lane];
                *cell = acc[r][c] + *cell;
            }
    }
    __syncthreads();

    // wave s finishes outputs 16 s .. 16 s + 15
    float v[16];
#pragma unroll
    for (int o = 0; o < 16; ++o) {
        const uint32_t q = 16 * s + o;
        v[o] = s_part[0][q][lane] + s_part[1][q][lane];
    }
    // halving exchange: after the step with mask m the lane keeps the outputs whose index bit matches
    // its own lane bit; four steps leave output (lane >> 2) & 15, two plain butterfly steps finish it.
#pragma unroll
    for (int step = 0; step < 4; ++step) {
        const int m = 32 >> step, half = 8 >> step;
        const bool upper = (lane & m) != 0;
#pragma unroll
        for (int o = 0; o < half; ++o) {
            // both candidates are pinned in registers first: left alone, the compiler folds the two selects
            // into one load of v[] at a lane-dependent index, i.e. a 16-way compare-and-select chain
            float lo = v[o], hi = v[o + half];
            asm("" : "+v"(lo), "+v"(hi));
            const float keep = upper ? hi : lo;
            const float send = upper ? lo : hi;
            v[o] = keep + __shfl_xor(send, m, 64);
        }
    }
    float r0 = v[0];
    r0 = r0 + __shfl_xor(r0, 2, 64);
    r0 = r0 + __shfl_xor(r0, 1, 64);
    if ((lane & 3) == 0) {
        const uint32_t q = 16 * s + (lane >> 2);
        const uint32_t tok = t0 + q / kTileExp, e = e0 + q % kTileExp;
        if (tok < t && e < n_experts) logits[(size_t)tok * n_experts + e] = r0;
    }
}

__global__ __launch_bounds__(64) void router_topk_kernel(const float *logits, const uint16_t *__restrict__ per_expert_scale,
                                                         uint32_t n_experts, uint32_t top_k,
                                                         uint32_t *__restrict__ out_idx, uint16_t *__restrict__ out_w, bool w_f16) {
    const uint32_t tok = blockIdx.x;
    wave_topk(logits + (size_t)tok * n_experts, per_expert_scale, n_experts, top_k, out_idx + (size_t)tok * top_k,
              out_w + (size_t)tok * top_k, threadIdx.x, w_f16);
}

}  // namespace

hipError_t launch_router(hipStream_t s, RouterWeights rw, const uint16_t *x, uint32_t x_stride, uint32_t t,
                         uint32_t n_experts, uint32_t d, uint32_t top_k, float *logits, uint32_t *out_idx,
                         uint16_t *out_w, KernelTimer *timer, bool f16) {
    timer->begin(s);
    const bool x_aligned = (reinterpret_cast<uintptr_t>(x) % 8 == 0) && (x_stride % 4 == 0);
    if (f16 && !x_aligned) return hipErrorInvalidValue;     // FP16 rows come 8-byte aligned (checked at the boundary)
    if (t <= FFMOE_MAX_VERIFY_ROWS) {
        const dim3 grid(n_experts, (t + kChunkTokens - 1) / kChunkTokens);
#define FFMOE_ROUTER(WF, XA)                                                                                 \
    hipLaunchKernelGGL((router_small_kernel<WF, XA>), grid, dim3(256), 0, s, rw.w, rw.effective_scale, x,   \
                       x_stride, t, n_experts, d, logits)
        if (rw.w_is_f32) { if (f16) FFMOE_ROUTER(true, 2); else if (x_aligned) FFMOE_ROUTER(true, 1); else FFMOE_ROUTER(true, 0); }
        else { if (f16) FFMOE_ROUTER(false, 2); else if (x_aligned) FFMOE_ROUTER(false, 1); else FFMOE_ROUTER(false, 0); }
#undef FFMOE_ROUTER
        timer->mark(s, FFMOE_K_ROUTER_LOGITS);
        hipLaunchKernelGGL(router_topk_kernel, dim3(t), dim3(64), 0, s, logits, rw.per_expert_scale, n_experts, top_k, out_idx,
                           out_w, f16);
        timer->mark(s, FFMOE_K_ROUTER_TOPK);
        timer->finish();
        return hipGetLastError();
    }
    const uint32_t n_egroups = (n_experts + kTileExp - 1) / kTileExp, n_tgroups = (t + kTileTok - 1) / kTileTok;
    const dim3 grid(n_egroups * ((n_tgroups + 7) / 8) * 8);
#define FFMOE_ROUTER(WF, XA)                                                                                 \
    do {                                                                                                     \
        if (rw.effective_scale)                                                                              \
            hipLaunchKernelGGL((router_tile_kernel<WF, XA, true>), grid, dim3(256), 0, s, rw.w,              \
                               rw.effective_scale, x, x_stride, t, n_experts, d, n_egroups, n_tgroups, logits); \
        else                                                                                                 \
            hipLaunchKernelGGL((router_tile_kernel<WF, XA, false>), grid, dim3(256), 0, s, rw.w,             \
                               rw.effective_scale, x, x_stride, t, n_experts, d, n_egroups, n_tgroups, logits); \
    } while (0)
    if (rw.w_is_f32) { if (f16) FFMOE_ROUTER(true, 2); else if (x_aligned) FFMOE_ROUTER(true, 1); else FFMOE_ROUTER(true, 0); }
    else { if (f16) FFMOE_ROUTER(false, 2); else if (x_aligned) FFMOE_ROUTER(false, 1); else FFMOE_ROUTER(false, 0); }
#undef FFMOE_ROUTER
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_ROUTER_LOGITS);
    hipLaunchKernelGGL(router_topk_kernel, dim3(t), dim3(64), 0, s, logits, rw.per_expert_scale, n_experts, top_k,
                       out_idx, out_w, f16);
    timer->mark(s, FFMOE_K_ROUTER_TOPK);
    timer->finish();
    return hipGetLastError();
}

}  // namespace ffmoe
