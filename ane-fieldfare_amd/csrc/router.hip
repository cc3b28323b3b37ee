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


// ---------------------------------------------------------------------------------------------------
// Prefill router, fast form: the same routes and weights, bit for bit, without the pinned fp32 sums of all
// E logits per token. The pinned order makes the logits a vector-ALU GEMM (2.2 GFLOP at 3,072 tokens: 31 us of
// fma alone); only the selected experts' logits have to be the pinned ones.
//   1. router_approx_kernel: every logit on the matrix unit (bf16 products are exact, the fp32 sum runs in
//      whatever order the unit uses), plus the squared norm of every row.
//   2. router_exact_topk_kernel, one wave per token. Let a_e be the approximate and p_e the pinned logit of expert e, and
//      B >= |a_e - p_e|. An expert among the pinned top k has a_e >= v_k - 2 B, v_k the k-th largest approximate logit:
//      were a_e below that, the k experts with a >= v_k would all have p >= a - B > a_e + B >= p_e. The wave computes
//      the pinned logit of every expert above that threshold (eight or nine at 128 experts) and selects among them
//      with the same code as the other router kernels. A row with a non-finite value anywhere takes every expert as
//      a candidate.
//      B: both sums add the same exact products (bf16 x bf16 fits fp32), so each differs from the real-number sum
//      by at most (roundings on the longest path of its summation tree) x (relative size of one rounding) x
//      sum_k |x_k w_ek| <= ... x ||x|| max_e ||w_e||. Approximate pass: a block sums one part of K (a quarter) with
//      d / 128 matrix instructions, each adding 32 products to the running sum in an order the unit does not document;
//      the count assumes the worst one, the running sum carried through all 33 additions of every instruction:
//      33 d / 128 roundings of 2^-23, and 2 to add the four parts in a tree. Pinned order: 4 fmaf per 1024-wide step, 2 adds for the sub-accumulators, 6 for the butterfly,
//      2^-24 each (the order is this build's own, so the count is exact).
// FP16 rows enter the approximate pass as two bf16 halves per value (split_f16x8: exact), which doubles its
// instructions and its rounding count; the pinned sums widen them to fp32 as every other kernel does.
// Needs: bf16 weights, no per-input scale, d a multiple of 256 up to 4096, E a multiple of 16 up to 128
// (the four waves of a block of the approximate pass hold two 16-expert fragments each).
// ---------------------------------------------------------------------------------------------------
constexpr int kApproxFrags = 2;                      // 16-row operand fragments of token rows per block of the approximate pass
constexpr int kApproxTok = 16 * kApproxFrags;
constexpr int kApproxKParts = 4;        // K is cut into parts, one block each; the pass that follows adds the parts' sums

// Router weights in matrix-operand order: frag[(h * E/16 + n) * 64 + lane] = the eight values
// w[16 n + lane % 16][32 h + 8 (lane / 16) .. + 7], so that a wave's operand load is 1 KiB contiguous.
__global__ __launch_bounds__(256) void router_frag_kernel(const uint16_t *__restrict__ w, uint32_t n_experts, uint32_t d,
                                                          uint4 *__restrict__ frag) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x, lane = i & 63, piece = i >> 6;
    const uint32_t nfrag = n_experts / 16, n = piece % nfrag, h = piece / nfrag;
    if (h >= d / 32) return;
    frag[i] = *reinterpret_cast<const uint4 *>(w + (size_t)(16 * n + (lane & 15)) * d + 32 * h + 8 * (lane >> 4));
}

// One block = 32 token rows x one quarter of K x all experts, four waves: wave nq takes a quarter of the experts'
// 16-column fragments (NF of them) against both 16-row fragments of the block's rows, with four k-steps of operands in
// flight. Every block reads its quarter of the weights once, so what the pass moves through the second-level cache is
// (rows / 32) x the weights - the time of this pass is that traffic and the round trips it is made of, not its
// arithmetic; 16 rows per block with K inside the block moved twice as much on three quarters of the compute units.
// Block 4 b + q leaves the sums of K quarter q for rows 32 b .. 32 b + 31 in approx[q] and the rows' squares in
// xnorm2[q]; the reader adds them as (q0 + q1) + (q2 + q3). The loop body has no branch: the compiler then counts the
// loads in flight exactly and waits for the oldest step only (behind a branch it waits for all of them, and the pass is
// one round trip per step).
constexpr int kApproxDepth = 4;

// Eight FP16 values as two sets of eight bf16 values whose sums are the FP16 values exactly (eleven significant bits =
// the leading eight + the remaining three), so that FP16 rows meet the bf16 weights on the bf16 matrix instruction with
// exact products. A value that is not finite leaves a NaN in one of the halves, and the row takes every expert.
__device__ __forceinline__ void split_f16x8(const uint4 &v, uint4 &lead, uint4 &rest, float &x2) {
    const uint32_t in[4] = {v.x, v.y, v.z, v.w};
    uint32_t a[4], b[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float f0 = Act<true>::lo(in[q]), f1 = Act<true>::hi(in[q]);
        x2 = __builtin_fmaf(f0, f0, x2);
        x2 = __builtin_fmaf(f1, f1, x2);
        const uint32_t l0 = __float_as_uint(f0) & 0xFFFF0000u, l1 = __float_as_uint(f1) & 0xFFFF0000u;
        const uint32_t r0 = __float_as_uint(f0 - __uint_as_float(l0)), r1 = __float_as_uint(f1 - __uint_as_float(l1));
        a[q] = (l0 >> 16) | l1;
        b[q] = (r0 >> 16) | (r1 & 0xFFFF0000u);
    }
    lead = uint4{a[0], a[1], a[2], a[3]};
    rest = uint4{b[0], b[1], b[2], b[3]};
}

template <int NF, bool F16>
__global__ __launch_bounds__(256) void router_approx_kernel(const uint4 *__restrict__ wfrag, const uint16_t *__restrict__ x,
                                                            uint32_t x_stride, uint32_t t, uint32_t t_pad, uint32_t n_experts,
                                                            uint32_t d, float *__restrict__ approx, float *__restrict__ xnorm2) {
    const uint32_t lane = threadIdx.x & 63, nq = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t kq = blockIdx.x % kApproxKParts, t0 = (blockIdx.x / kApproxKParts) * kApproxTok;
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint32_t nfrag = n_experts / 16, nh = d / 32;
    const uint32_t h0 = kq * nh / kApproxKParts, h1 = (kq + 1) * nh / kApproxKParts, span = h1 - h0;
    const uint32_t n0 = nq * NF;                       // this wave's fragments: n0 .. n0 + NF - 1 (those below nfrag)
    // the rows are loaded four neighbouring lanes per 64 contiguous bytes (row lane / 4, chunk lane % 4: 16 requests per
    // instruction instead of 64) and turned into the operand layout (lane (j, jq): row j, chunk jq) by cross-lane moves
    const uint16_t *xr[kApproxFrags];
#pragma unroll
    for (int f = 0; f < kApproxFrags; ++f) xr[f] = x + (size_t)min(t0 + 16 * f + (lane >> 2), t - 1) * x_stride + 8 * (lane & 3);
    const int pull = (int)((4 * j + jq) * 4);
    const uint4 *wf = wfrag + lane;
    f32x4 acc[kApproxFrags][NF];
    float x2[kApproxFrags];
#pragma unroll
    for (int f = 0; f < kApproxFrags; ++f) {
        x2[f] = 0.0f;
#pragma unroll
        for (int n = 0; n < NF; ++n) acc[f][n] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    uint4 a_q[kApproxDepth][kApproxFrags], b_q[kApproxDepth][NF];
    // step i of this block = k-step h0 + i; past the end it repeats the last step and enters with zero rows
    auto fetch = [&](int slot, uint32_t i) {
        const uint32_t h = h0 + min(i, span - 1);
#pragma unroll
        for (int f = 0; f < kApproxFrags; ++f) a_q[slot][f] = *reinterpret_cast<const uint4 *>(xr[f] + 32 * h);
#pragma unroll
        for (int n = 0; n < NF; ++n) b_q[slot][n] = wf[((size_t)h * nfrag + min(n0 + n, nfrag - 1)) * 64];
    };
    if (span) {
#pragma unroll
        for (int u = 0; u < kApproxDepth; ++u) fetch(u, u);
        for (uint32_t ib = 0; ib < span; ib += kApproxDepth) {
#pragma unroll
            for (int u = 0; u < kApproxDepth; ++u) {
                uint4 a[kApproxFrags], b[NF];
#pragma unroll
                for (int f = 0; f < kApproxFrags; ++f) a[f] = a_q[u][f];
#pragma unroll
                for (int n = 0; n < NF; ++n) b[n] = b_q[u][n];
                fetch(u, ib + u + kApproxDepth);
#pragma unroll
                for (int f = 0; f < kApproxFrags; ++f) {
                    a[f].x = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)a[f].x);
                    a[f].y = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)a[f].y);
                    a[f].z = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)a[f].z);
                    a[f].w = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)a[f].w);
                    if (ib + u >= span) a[f] = uint4{0, 0, 0, 0};
                    if constexpr (F16) {
                        uint4 lead, rest;
                        split_f16x8(a[f], lead, rest, x2[f]);
#pragma unroll
                        for (int n = 0; n < NF; ++n) {
                            acc[f][n] = Act<false>::mfma(lead, b[n], acc[f][n]);
                            acc[f][n] = Act<false>::mfma(rest, b[n], acc[f][n]);
                        }
                    } else {
                        const uint32_t aw[4] = {a[f].x, a[f].y, a[f].z, a[f].w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float lo = bf16lo_to_f32(aw[q]), hi = bf16hi_to_f32(aw[q]);
                            x2[f] = __builtin_fmaf(lo, lo, x2[f]);
                            x2[f] = __builtin_fmaf(hi, hi, x2[f]);
                        }
#pragma unroll
                        for (int n = 0; n < NF; ++n) acc[f][n] = Act<false>::mfma(a[f], b[n], acc[f][n]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int f = 0; f < kApproxFrags; ++f) {
        // the row's squares over this part of K: the four k-chunk lanes of a row
        x2[f] += __shfl_xor(x2[f], 16, 64);
        x2[f] += __shfl_xor(x2[f], 32, 64);
        const uint32_t row = t0 + 16 * f + j;
        if (nq == 0 && jq == 0 && row < t) xnorm2[(size_t)kq * t_pad + row] = x2[f];
        // the lane holds tokens 4 jq .. + 3 of expert column j of each of its fragments
#pragma unroll
        for (int n = 0; n < NF; ++n) {
            if (n0 + n < nfrag) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t tok = t0 + 16 * f + 4 * jq + r;
                    if (tok < t) approx[((size_t)kq * t_pad + tok) * n_experts + 16 * (n0 + n) + j] = acc[f][n][r];
                }
            }
        }
    }
}

// What the approximate pass left per part of K, added pairwise (a tree of log2(parts) levels; all loads first).
__device__ __forceinline__ float sum_k_parts(const float *__restrict__ p, size_t part_stride) {
    float v[kApproxKParts];
#pragma unroll
    for (int q = 0; q < kApproxKParts; ++q) v[q] = p[q * part_stride];
#pragma unroll
    for (int w = 1; w < kApproxKParts; w *= 2)
#pragma unroll
        for (int q = 0; q + w < kApproxKParts; q += 2 * w) v[q] += v[q + w];
    return v[0];
}

constexpr int kExactSteps = 4;          // d <= 4096: k = 1024 i + 256 s + 4 lane + j, i < 4

// STEPS: 1024-wide steps of the pinned order that d needs; CHUNK: candidates whose rows are requested together.
template <int STEPS, int CHUNK, bool F16>
__global__ __launch_bounds__(256, 3) void router_exact_topk_kernel(const uint16_t *__restrict__ w, const uint16_t *__restrict__ x,
                                                                   uint32_t x_stride, uint32_t t, uint32_t n_experts, uint32_t d,
                                                                   uint32_t top_k, const float *__restrict__ approx,
                                                                   const float *__restrict__ xnorm2, uint32_t t_pad,
                                                                   float bound_per_norm,
                                                                   const uint16_t *__restrict__ per_expert_scale,
                                                                   uint32_t *__restrict__ out_idx, uint16_t *__restrict__ out_w) {
    const uint32_t lane = threadIdx.x & 63, tok = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= t) return;
    // the token's row, as the pinned order walks it: element j of (step i, sub-accumulator s) = x[1024 i + 256 s + 4 lane + j]
    const uint16_t *xr = x + (size_t)tok * x_stride;
    float xf[STEPS][4][4];
    {
        uint2 xraw[STEPS][4];
#pragma unroll
        for (int i = 0; i < STEPS; ++i)
#pragma unroll
            for (int s_ = 0; s_ < 4; ++s_) {
                // d is a multiple of 256: a (step, sub-accumulator) pair is inside the row for every lane or for none
                const uint32_t k = 1024 * i + 256 * s_;
                xraw[i][s_] = k < d ? *reinterpret_cast<const uint2 *>(xr + k + 4 * lane) : make_uint2(0u, 0u);
            }
#pragma unroll
        for (int i = 0; i < STEPS; ++i)
#pragma unroll
            for (int s_ = 0; s_ < 4; ++s_) {
                xf[i][s_][0] = Act<F16>::lo(xraw[i][s_].x), xf[i][s_][1] = Act<F16>::hi(xraw[i][s_].x);
                xf[i][s_][2] = Act<F16>::lo(xraw[i][s_].y), xf[i][s_][3] = Act<F16>::hi(xraw[i][s_].y);
            }
    }
    // at most 128 experts: the lane's candidates are experts lane and 64 + lane
    float a[2];
    bool odd = false;       // a value that is not finite
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const uint32_t e = c * 64 + lane;
        a[c] = e < n_experts ? sum_k_parts(approx + (size_t)tok * n_experts + e, (size_t)t_pad * n_experts) : -INFINITY;
        odd = odd || (e < n_experts && !(fabsf(a[c]) < INFINITY));
    }
    // 2 B: see the comment above; the absolute term covers products the matrix unit may flush to zero
    const float norm2 = sum_k_parts(xnorm2 + tok, t_pad);
    const float bound = bound_per_norm * sqrtf(norm2) + 1e-30f;
    const bool everyone = __any(odd) || !(bound < INFINITY);
    // v_k, the k-th largest approximate logit (equal values leave together, which can only lower it)
    uint32_t key0 = a[0] > -INFINITY ? orderable(a[0]) : 0u, key1 = a[1] > -INFINITY ? orderable(a[1]) : 0u;
    uint32_t kth = 0;
    for (uint32_t r = 0; r < top_k; ++r) {
        kth = wave_max_u32(max(key0, key1));
        if (key0 == kth) key0 = 0u;
        if (key1 == kth) key1 = 0u;
    }
    const float v_k = kth ? __uint_as_float((kth & 0x80000000u) ? (kth & 0x7FFFFFFFu) : ~kth) : -INFINITY;
    const float threshold = v_k - bound;        // -inf when fewer than k candidates exist: everyone is in
    unsigned long long m0 = __ballot(lane < n_experts && (everyone || a[0] >= threshold));
    unsigned long long m1 = __ballot(64 + lane < n_experts && (everyone || a[1] >= threshold));
    uint32_t exact0 = 0u, exact1 = 0u;      // the pinned logits of this lane's two experts, as keys of the select
    // The candidates CHUNK at a time: all rows of a chunk are requested before the first sum runs, so a token pays a
    // few round trips to the weights instead of one per candidate.
    while (m0 | m1) {
        uint32_t e[CHUNK];
        uint2 wq[CHUNK][STEPS][4];
#pragma unroll
        for (int q = 0; q < CHUNK; ++q) {
            if (m0) {
                e[q] = (uint32_t)__builtin_ctzll(m0);
                m0 &= m0 - 1;
            } else if (m1) {
                e[q] = 64u + (uint32_t)__builtin_ctzll(m1);
                m1 &= m1 - 1;
            } else {
                e[q] = 0xFFFFFFFFu;
            }
            const uint16_t *wr = w + (size_t)(e[q] == 0xFFFFFFFFu ? 0u : e[q]) * d;
#pragma unroll
            for (int i = 0; i < STEPS; ++i)
#pragma unroll
                for (int s_ = 0; s_ < 4; ++s_) {
                    const uint32_t k = 1024 * i + 256 * s_;
                    wq[q][i][s_] = k < d && e[q] != 0xFFFFFFFFu ? *reinterpret_cast<const uint2 *>(wr + k + 4 * lane) : make_uint2(0u, 0u);
                }
        }
#pragma unroll
        for (int q = 0; q < CHUNK; ++q) {
            if (e[q] == 0xFFFFFFFFu) continue;
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < STEPS; ++i)
#pragma unroll
                for (int s_ = 0; s_ < 4; ++s_) {
                    if (1024u * i + 256u * s_ < d) {
                        const uint2 wv = wq[q][i][s_];
                        acc[s_] = __builtin_fmaf(bf16lo_to_f32(wv.x), xf[i][s_][0], acc[s_]);
                        acc[s_] = __builtin_fmaf(bf16hi_to_f32(wv.x), xf[i][s_][1], acc[s_]);
                        acc[s_] = __builtin_fmaf(bf16lo_to_f32(wv.y), xf[i][s_][2], acc[s_]);
                        acc[s_] = __builtin_fmaf(bf16hi_to_f32(wv.y), xf[i][s_][3], acc[s_]);
                    }
                }
            const float v = wave_butterfly_sum((acc[0] + acc[1]) + (acc[2] + acc[3]));
            const uint32_t k_ = v > -INFINITY ? orderable(v) : 0u;
            if (e[q] == lane) exact0 = k_;
            if (e[q] == 64u + lane) exact1 = k_;
        }
    }
    TopkRow tr;
    tr.key[0] = exact0, tr.key[1] = exact1, tr.key[2] = 0u, tr.key[3] = 0u;
    topk_select<2>(tr, top_k, lane);
    topk_store(tr, per_expert_scale, top_k, out_idx + (size_t)tok * top_k, out_w + (size_t)tok * top_k, lane, F16);
}

}  // namespace

hipError_t launch_router(hipStream_t s, RouterWeights rw, const uint16_t *x, uint32_t x_stride, uint32_t t,
                         uint32_t n_experts, uint32_t d, uint32_t top_k, float *logits, uint32_t *out_idx,
                         uint16_t *out_w, KernelTimer *timer, bool f16, bool want_logits, float *scratch) {
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
    if (rw.w_frag && !rw.w_is_f32 && !rw.effective_scale && !want_logits && d % 256 == 0 && d <= 1024 * kExactSteps &&
        n_experts % 16 == 0 && n_experts <= 128 && top_k <= 8 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && x_stride % 8 == 0 && scratch) {
        // approximate logits of every expert on the matrix unit, the pinned ones only where the select can tell
        const uint32_t t_pad = (t + 63) & ~63u;
        float *xnorm2 = scratch, *approx = scratch + (size_t)kApproxKParts * t_pad;
        const dim3 agrid((t + kApproxTok - 1) / kApproxTok * kApproxKParts);
        const uint32_t per_wave = (n_experts / 16 + 3) / 4;       // fragments per wave: the four N quarters cover all of them
#define FFMOE_APPROX(NF, H)                                                                                            \
    hipLaunchKernelGGL((router_approx_kernel<NF, H>), agrid, dim3(256), 0, s, rw.w_frag, x, x_stride, t, t_pad, n_experts, d,  \
                       approx, xnorm2)
        if (f16) { if (per_wave <= 1) FFMOE_APPROX(1, true); else FFMOE_APPROX(2, true); }
        else { if (per_wave <= 1) FFMOE_APPROX(1, false); else FFMOE_APPROX(2, false); }
#undef FFMOE_APPROX
        timer->mark(s, FFMOE_K_ROUTER_LOGITS);
        // 2 B per unit of ||x||: the rounding counts of the two sums (see above), 1 % on top for the norms' own rounding
        static_assert(kApproxKParts == 4, "the rounding count below is that of four parts of K added in a tree of two levels");
        // (FP16 rows enter as two bf16 halves: two instructions, 66 additions, per 32 elements)
        const float approx_roundings = (f16 ? 66.0f : 33.0f) * (float)(d / 128) + 2.0f, pinned_roundings = 4.0f * ((d + 1023) / 1024) + 8.0f;
        const float bound_per_norm = 2.02f * (approx_roundings * 0x1p-23f + pinned_roundings * 0x1p-24f) * rw.w_norm_max;
#define FFMOE_EXACT_AS(STEPS, CHUNK, H)                                                                                    \
    hipLaunchKernelGGL((router_exact_topk_kernel<STEPS, CHUNK, H>), dim3((t + 3) / 4), dim3(256), 0, s,                      \
                       static_cast<const uint16_t *>(rw.w), x, x_stride, t, n_experts, d, top_k, approx, xnorm2, t_pad,        \
                       bound_per_norm,                                                                                      \
                       rw.per_expert_scale, out_idx, out_w)
#define FFMOE_EXACT(STEPS, CHUNK)                                     \
    do {                                                              \
        if (f16) FFMOE_EXACT_AS(STEPS, CHUNK, true);                  \
        else FFMOE_EXACT_AS(STEPS, CHUNK, false);                     \
    } while (0)
        if (d <= 1024) FFMOE_EXACT(1, 4); else if (d <= 2048) FFMOE_EXACT(2, 4); else if (d <= 3072) FFMOE_EXACT(3, 4); else FFMOE_EXACT(4, 2);
#undef FFMOE_EXACT
#undef FFMOE_EXACT_AS
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

namespace ffmoe {
hipError_t launch_router_fragments(hipStream_t s, const uint16_t *w, uint32_t n_experts, uint32_t d, void *frag) {
    const uint32_t pieces = (d / 32) * (n_experts / 16);
    hipLaunchKernelGGL(router_frag_kernel, dim3((pieces * 64 + 255) / 256), dim3(256), 0, s, w, n_experts, d, static_cast<uint4 *>(frag));
    return hipGetLastError();
}
}  // namespace ffmoe
