// Routed experts for a decode step or a verify block (1..16 tokens): every expert the block touches
// streams its INT4 weights from HBM exactly once, and all of its tokens ride the same pass.
//
// Replaces moe_phase1_gate_up_act_u16load / moe_phase2_down_reduce_k8 / moe_gather_routed_slots
// (Metal/MoE/moe.metal:500-638) and verify_bound_plan / verify_*_gate_up_act / verify_*_down
// (Metal/Prefill/prefill.metal:1246-1529), plus prefill_moe_reduce_token_major (:544-565).
//
// Arithmetic per weight row and token (the factored form of moe.metal:323-378):
//     y = sum_g [ s_g * sum_k q_k x_k + b_g * sum_k x_k ]
// The inner sums over a 64-wide group run on the matrix unit: a wave owns one arena tile (16 gate rows
// and 16 up rows, or 32 down rows) per group, turns each dword of nibbles into eight bf16 values
// 128 + q with four and-or operations, and issues v_mfma_f32_16x16x32_bf16 with the (up to 16) token
// rows as the other operand. The offset is removed with the group's sum of x:
//     s * (acc - 128 * sx) + b * sx = s * acc + (b - 128 s) * sx.
#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {
namespace {

constexpr int kMaxRows = FFMOE_MAX_VERIFY_ROWS;

// ---------------------------------------------------------------------------------------------------
// Plan: invert routes [t][top_k] into per-expert route lists, compact the live experts in expert
// order (deterministic: ballot prefix, no atomics), and sum x per (token, 64-group).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void verify_plan_kernel(const uint32_t *__restrict__ idx,
                                                          const uint16_t *__restrict__ w, uint32_t t,
                                                          uint32_t top_k, uint32_t n_experts,
                                                          const uint16_t *__restrict__ x, uint32_t x_stride,
                                                          uint32_t gd, VerifyPlan *__restrict__ plan,
                                                          float *__restrict__ xsum) {
    __shared__ uint32_t s_idx[kMaxRows * 8];
    __shared__ uint32_t s_live[kMaxRows * 8];
    __shared__ uint32_t s_wave_count[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t n_routes = t * top_k;
    if (tid < n_routes) {
        const uint32_t e = idx[tid];
        const bool nonzero = (w[tid] & 0x7FFFu) != 0;
        s_idx[tid] = e;
        s_live[tid] = (nonzero && e < n_experts) ? 1u : 0u;
    }
    if (tid < kMaxRows * 8) plan->route_valid[tid] = 0;
    __syncthreads();

    uint32_t routes[kMaxRows];
    uint32_t n = 0;
    if (tid < n_experts) {
        for (uint32_t i = 0; i < n_routes; ++i) {
            if (s_live[i] && s_idx[i] == tid && n < (uint32_t)kMaxRows) {
#pragma unroll
                for (int r = 0; r < kMaxRows; ++r)
                    if ((uint32_t)r == n) routes[r] = i;
                ++n;
            }
        }
    }
    const unsigned long long mask = __ballot(n > 0);
    const uint32_t before = __popcll(mask & ((1ull << lane) - 1ull));
    if (lane == 0) s_wave_count[wave] = __popcll(mask);
    __syncthreads();
    uint32_t base = 0;
    for (uint32_t v = 0; v < wave; ++v) base += s_wave_count[v];
    if (n > 0) {
        PlanSlot &slot = plan->slots[base + before];
        slot.expert = tid;
        slot.n = n;
#pragma unroll
        for (int r = 0; r < kMaxRows; ++r) {
            if ((uint32_t)r < n) {
                slot.routes[r] = routes[r];
                plan->route_valid[routes[r]] = 1;
            } else {
                slot.routes[r] = 0;
            }
        }
    }
    if (tid == 0) plan->n_live = s_wave_count[0] + s_wave_count[1] + s_wave_count[2] + s_wave_count[3];

    // sum of x over each 64-group, fp32, fixed order (8 x 16-byte loads, elements left to right)
    for (uint32_t p = tid; p < t * gd; p += blockDim.x) {
        const uint32_t tok = p / gd, g = p % gd;
        const uint4 *src = reinterpret_cast<const uint4 *>(x + (size_t)tok * x_stride + (size_t)g * kGroup);
        float sum = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint4 v = src[c];
            sum += bf16lo_to_f32(v.x); sum += bf16hi_to_f32(v.x);
            sum += bf16lo_to_f32(v.y); sum += bf16hi_to_f32(v.y);
            sum += bf16lo_to_f32(v.z); sum += bf16hi_to_f32(v.z);
            sum += bf16lo_to_f32(v.w); sum += bf16hi_to_f32(v.w);
        }
        xsum[p] = sum;
    }
}

// ---------------------------------------------------------------------------------------------------
// One (expert, row block) pass over K. Streams A / B of a tile are gate / up rows (same row index) or
// two down row blocks. Lane l: weight row l % 16 of each stream and k-quarter l / 16; as the token
// operand it supplies token slot l % 16; it ends up holding token slots 4 * (l / 16) + 0..3.
// ---------------------------------------------------------------------------------------------------
struct TwoStreamAcc {
    f32x4 a, b;
};

template <int UNROLL>
__device__ __forceinline__ TwoStreamAcc stream_tiles(const uint8_t *__restrict__ tiles,
                                                     const uint8_t *__restrict__ scales,
                                                     const uint16_t *__restrict__ act_row,
                                                     const float *__restrict__ s_sum, uint32_t g0, uint32_t g1,
                                                     uint32_t lane) {
    const uint32_t j = lane & 15, jq = lane >> 4;
    TwoStreamAcc tot;
    tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
    tot.b = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    auto step = [&](uint32_t g) {
        const uint4 tile = reinterpret_cast<const uint4 *>(tiles + (size_t)g * kTileBytes)[lane];
        const uint2 sc = reinterpret_cast<const uint2 *>(scales + (size_t)g * kTileScaleBytes)[j];
        const uint4 x0 = *reinterpret_cast<const uint4 *>(act_row + g * kGroup + 8 * jq);
        const uint4 x1 = *reinterpret_cast<const uint4 *>(act_row + g * kGroup + 32 + 8 * jq);
        const f32x4 sx = *reinterpret_cast<const f32x4 *>(s_sum + g * kMaxRows + 4 * jq);
        const bf16x8 a0 = __builtin_bit_cast(bf16x8, x0), a1 = __builtin_bit_cast(bf16x8, x1);
        f32x4 acc_a = mfma16(a0, unpack8_offset128(tile.x), zero);
        acc_a = mfma16(a1, unpack8_offset128(tile.y), acc_a);
        f32x4 acc_b = mfma16(a0, unpack8_offset128(tile.z), zero);
        acc_b = mfma16(a1, unpack8_offset128(tile.w), acc_b);
        const float sa = bf16lo_to_f32(sc.x), ba = bf16hi_to_f32(sc.x);
        const float sb = bf16lo_to_f32(sc.y), bb = bf16hi_to_f32(sc.y);
        const float ta = __builtin_fmaf(-128.0f, sa, ba), tb = __builtin_fmaf(-128.0f, sb, bb);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            tot.a[r] = __builtin_fmaf(sa, acc_a[r], tot.a[r]);
            tot.a[r] = __builtin_fmaf(ta, sx[r], tot.a[r]);
            tot.b[r] = __builtin_fmaf(sb, acc_b[r], tot.b[r]);
            tot.b[r] = __builtin_fmaf(tb, sx[r], tot.b[r]);
        }
    };
    uint32_t g = g0;
    for (; g + UNROLL <= g1; g += UNROLL) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) step(g + u);
    }
    for (; g < g1; ++g) step(g);
    return tot;
}

// gate/up + GELU-tanh gating. grid = (ceil(F/16 / (4/KSPLIT)), live-slot capacity); block = 4 waves.
// KSPLIT waves of a block share one row block and split K; partial sums meet in LDS in wave order.
template <int KSPLIT>
__global__ __launch_bounds__(256) void skinny_gate_up_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                             uint32_t top_k, const VerifyPlan *__restrict__ plan,
                                                             const float *__restrict__ xsum,
                                                             const uint16_t *__restrict__ x, uint32_t x_stride,
                                                             uint16_t *__restrict__ acts) {
    extern __shared__ float s_dyn[];
    float *s_sum = s_dyn;                                  // [gd][16]
    float *s_red = s_dyn + (size_t)g.gd * kMaxRows;        // [4 waves][8][64] when KSPLIT > 1
    const uint32_t slot_id = blockIdx.y;
    if (slot_id >= plan->n_live) return;
    const PlanSlot &slot = plan->slots[slot_id];
    const uint32_t n = slot.n;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (uint32_t p = tid; p < g.gd * kMaxRows; p += 256) {
        const uint32_t grp = p / kMaxRows, r = min(p % kMaxRows, n - 1);
        s_sum[p] = xsum[(slot.routes[r] / top_k) * g.gd + grp];
    }
    __syncthreads();

    constexpr uint32_t kRbPerBlock = 4 / KSPLIT;
    const uint32_t rb = blockIdx.x * kRbPerBlock + wave / KSPLIT;
    const uint32_t ks = wave % KSPLIT;
    const bool active = rb < g.gu_rb;
    TwoStreamAcc tot;
    tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
    tot.b = tot.a;
    if (active) {
        const uint8_t *expert = arena_layer + (size_t)slot.expert * g.expert_bytes;
        const uint8_t *tiles = expert + g.gu_tiles_off + (size_t)rb * g.gd * kTileBytes;
        const uint8_t *scales = expert + g.gu_scales_off + (size_t)rb * g.gd * kTileScaleBytes;
        const uint32_t tok = slot.routes[min(lane & 15u, n - 1)] / top_k;
        const uint16_t *xrow = x + (size_t)tok * x_stride;
        const uint32_t per = (g.gd + KSPLIT - 1) / KSPLIT;
        const uint32_t g0 = ks * per, g1 = min(g.gd, g0 + per);
        tot = stream_tiles<4>(tiles, scales, xrow, s_sum, g0, g1, lane);
    }
    if (KSPLIT > 1) {
        if (ks != 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                s_red[(wave * 8 + r) * 64 + lane] = tot.a[r];
                s_red[(wave * 8 + 4 + r) * 64 + lane] = tot.b[r];
            }
        }
        __syncthreads();
        if (ks != 0) return;
        for (uint32_t o = 1; o < (uint32_t)KSPLIT; ++o) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                tot.a[r] += s_red[((wave + o) * 8 + r) * 64 + lane];
                tot.b[r] += s_red[((wave + o) * 8 + 4 + r) * 64 + lane];
            }
        }
    }
    if (!active) return;
    const uint32_t jq = lane >> 4, row = rb * kTileRows + (lane & 15);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t ts = 4 * jq + r;
        if (ts < n) {
            // one rounding to 16 bits, gate and up themselves stay fp32 (moe.metal:496)
            acts[(size_t)slot.routes[ts] * g.f + row] = f32_to_bf16(gelu_tanh(tot.a[r]) * tot.b[r]);
        }
    }
}

// down projection. grid = (ceil(D/32 / 4), live-slot capacity); each wave owns one pair of 16-row blocks.
// Output: un-weighted rows, fp32 into `partials_f32` (fused combine) or bf16 into `partials_bf16`.
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void skinny_down_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                          const VerifyPlan *__restrict__ plan,
                                                          const uint16_t *__restrict__ acts,
                                                          float *__restrict__ partials_f32,
                                                          uint16_t *__restrict__ partials_bf16) {
    extern __shared__ float s_dyn[];
    float *s_sum = s_dyn;   // [gf][16]
    const uint32_t slot_id = blockIdx.y;
    if (slot_id >= plan->n_live) return;
    const PlanSlot &slot = plan->slots[slot_id];
    const uint32_t n = slot.n;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // group sums of the rounded activations, fixed order
    for (uint32_t p = tid; p < g.gf * kMaxRows; p += 256) {
        const uint32_t grp = p / kMaxRows, r = min(p % kMaxRows, n - 1);
        const uint4 *src = reinterpret_cast<const uint4 *>(acts + (size_t)slot.routes[r] * g.f + (size_t)grp * kGroup);
        float sum = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint4 v = src[c];
            sum += bf16lo_to_f32(v.x); sum += bf16hi_to_f32(v.x);
            sum += bf16lo_to_f32(v.y); sum += bf16hi_to_f32(v.y);
            sum += bf16lo_to_f32(v.z); sum += bf16hi_to_f32(v.z);
            sum += bf16lo_to_f32(v.w); sum += bf16hi_to_f32(v.w);
        }
        s_sum[p] = sum;
    }
    __syncthreads();
    const uint32_t rbp = blockIdx.x * 4 + wave;
    if (rbp >= g.dn_rbp) return;
    const uint8_t *expert = arena_layer + (size_t)slot.expert * g.expert_bytes;
    const uint8_t *tiles = expert + g.dn_tiles_off + (size_t)rbp * g.gf * kTileBytes;
    const uint8_t *scales = expert + g.dn_scales_off + (size_t)rbp * g.gf * kTileScaleBytes;
    const uint16_t *arow = acts + (size_t)slot.routes[min(lane & 15u, n - 1)] * g.f;
    const TwoStreamAcc tot = stream_tiles<4>(tiles, scales, arow, s_sum, 0, g.gf, lane);
    const uint32_t jq = lane >> 4, row_a = rbp * 2 * kTileRows + (lane & 15), row_b = row_a + kTileRows;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t ts = 4 * jq + r;
        if (ts < n) {
            const size_t base = (size_t)slot.routes[ts] * g.d;
            if (OUT_BF16) {
                partials_bf16[base + row_a] = f32_to_bf16(tot.a[r]);
                partials_bf16[base + row_b] = f32_to_bf16(tot.b[r]);
            } else {
                partials_f32[base + row_a] = tot.a[r];
                partials_f32[base + row_b] = tot.b[r];
            }
        }
    }
}

// y[t][c] = bf16(residual + sum_r w[t][r] * partial[t*k + r][c]) in rank order with fmaf, fp32 partials,
// one rounding at the end (the decode form, moe.metal:627-636). Unplanned routes add nothing.
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ partials,
                                                      const uint16_t *__restrict__ w,
                                                      const uint32_t *__restrict__ route_valid,
                                                      const uint16_t *__restrict__ residual, uint32_t top_k,
                                                      uint32_t d, uint16_t *__restrict__ y) {
    const uint32_t tok = blockIdx.y;
    const uint32_t c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= d) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (residual) {
        const uint2 rv = *reinterpret_cast<const uint2 *>(residual + (size_t)tok * d + c);
        acc[0] = bf16lo_to_f32(rv.x); acc[1] = bf16hi_to_f32(rv.x);
        acc[2] = bf16lo_to_f32(rv.y); acc[3] = bf16hi_to_f32(rv.y);
    }
    for (uint32_t r = 0; r < top_k; ++r) {
        const uint32_t route = tok * top_k + r;
        if (!route_valid[route]) continue;
        const float wv = bf16_to_f32(w[route]);
        const f32x4 p = *reinterpret_cast<const f32x4 *>(partials + (size_t)route * d + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(wv, p[i], acc[i]);
    }
    uint2 o;
    o.x = pack_bf16x2(acc[0], acc[1]);
    o.y = pack_bf16x2(acc[2], acc[3]);
    *reinterpret_cast<uint2 *>(y + (size_t)tok * d + c) = o;
}

// prefill_moe_reduce_token_major (prefill.metal:544-565) on 16-bit partials.
__global__ __launch_bounds__(256) void reduce_token_major_kernel(const uint16_t *__restrict__ partials,
                                                                 const uint16_t *__restrict__ w, uint32_t top_k,
                                                                 uint32_t d, uint16_t *__restrict__ h2) {
    const uint32_t tok = blockIdx.y;
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    float acc = 0.0f;
    for (uint32_t r = 0; r < top_k; ++r) {
        const size_t route = (size_t)tok * top_k + r;
        acc = __builtin_fmaf(bf16_to_f32(w[route]), bf16_to_f32(partials[route * d + c]), acc);
    }
    h2[(size_t)tok * d + c] = f32_to_bf16(acc);
}

}  // namespace

hipError_t launch_verify(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts,
                         uint32_t top_k, const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx,
                         const uint16_t *w, const uint16_t *residual, uint16_t *y, uint16_t *partials_bf16,
                         VerifyPlan *plan, float *xsum, uint16_t *acts, float *partials_f32, KernelTimer *timer) {
    timer->begin(s);
    hipLaunchKernelGGL(verify_plan_kernel, dim3(1), dim3(256), 0, s, idx, w, t, top_k, n_experts, x, x_stride,
                       g.gd, plan, xsum);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_PLAN);
    const uint32_t slots = min(n_experts, t * top_k);
    const size_t sum_bytes_gu = (size_t)g.gd * kMaxRows * sizeof(float);
    if (slots <= 16) {
        // decode-sized blocks: split K over the four waves of a block to put more loads in flight
        hipLaunchKernelGGL(skinny_gate_up_kernel<4>, dim3(g.gu_rb, slots), dim3(256),
                           sum_bytes_gu + 4 * 8 * 64 * sizeof(float), s, arena_layer, g, top_k, plan, xsum, x,
                           x_stride, acts);
    } else {
        hipLaunchKernelGGL(skinny_gate_up_kernel<1>, dim3((g.gu_rb + 3) / 4, slots), dim3(256), sum_bytes_gu, s,
                           arena_layer, g, top_k, plan, xsum, x, x_stride, acts);
    }
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_GATE_UP);
    const size_t sum_bytes_dn = (size_t)g.gf * kMaxRows * sizeof(float);
    const dim3 dn_grid((g.dn_rbp + 3) / 4, slots);
    if (partials_bf16) {
        hipLaunchKernelGGL(skinny_down_kernel<true>, dn_grid, dim3(256), sum_bytes_dn, s, arena_layer, g, plan,
                           acts, partials_f32, partials_bf16);
        timer->mark(s, FFMOE_K_DOWN);
        timer->finish();
        return hipGetLastError();
    }
    hipLaunchKernelGGL(skinny_down_kernel<false>, dn_grid, dim3(256), sum_bytes_dn, s, arena_layer, g, plan, acts,
                       partials_f32, partials_bf16);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_DOWN);
    hipLaunchKernelGGL(combine_kernel, dim3((g.d / 4 + 255) / 256, t), dim3(256), 0, s, partials_f32, w,
                       plan->route_valid, residual, top_k, g.d, y);
    timer->mark(s, FFMOE_K_COMBINE);
    timer->finish();
    return hipGetLastError();
}

hipError_t launch_reduce_token_major(hipStream_t s, const uint16_t *partials, const uint16_t *weights,
                                     uint16_t *h2, uint32_t t, uint32_t top_k, uint32_t d) {
    hipLaunchKernelGGL(reduce_token_major_kernel, dim3((d + 255) / 256, t), dim3(256), 0, s, partials, weights,
                       top_k, d, h2);
    return hipGetLastError();
}

}  // namespace ffmoe
