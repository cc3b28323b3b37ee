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
// rows as the other operand. A third product against an all-ones operand yields the group's sum of x
// in the same register layout, which removes the offset and applies the bias:
//     s * (acc - 128 * sx) + b * sx = s * acc + (b - 128 s) * sx.
// Nothing is staged in LDS: weights, scales and token rows ride one register ring of PD groups, so a
// wave has PD KiB of weights in flight from its first instruction.
#include "common.hpp"
#include "kernels.hpp"
#include "router_sum.hpp"
#include "stream.hpp"
#include "topk.hpp"

namespace ffmoe {
namespace {

constexpr int kMaxRows = FFMOE_MAX_VERIFY_ROWS;
constexpr int kMaxRoutes = kMaxRows * 8;

// ---------------------------------------------------------------------------------------------------
// Plan: invert routes [t][top_k] into per-expert route lists and compact the live experts in expert
// order. Deterministic: the LDS atomics only build sets; every ordering comes from ballot prefixes and
// bit positions. A route takes part when its weight is not +-0 and its expert is in range; an expert
// keeps its first 16 routes. Slots past the last live expert get n = 0.
// ---------------------------------------------------------------------------------------------------
static_assert(kMaxRoutes <= 128, "an expert's routes are kept as one 128-bit set");

struct PlanScratch {
    uint4 routes_of[FFMOE_MAX_EXPERTS];     // bit r set: route r goes to this expert
    uint32_t cnt[FFMOE_MAX_EXPERTS];
    uint32_t slot_of[FFMOE_MAX_EXPERTS];
    uint32_t expert_of[FFMOE_MAX_EXPERTS];
    uint32_t wave_total[4];
};

// Run by all 256 threads of a block. Builds the plan in LDS and writes it to `plan_out` when that is not
// null. Returns n_live. `slot_from_total` maps the number of live experts to the caller's slot (or to ~0u
// for none). Thread r < n_routes brings route r's expert and weight (`route_idx`, `route_w`), so that the
// caller decides when that load is issued.
// Phase A: every expert's set of routes (one LDS or per route; a set has no order to get wrong), live
// experts compacted in expert order (ps.expert_of, ps.slot_of, ps.cnt); returns n_live and leaves the
// calling thread's own route expert in `e`. Phase B: the route lists, a route's place being the number of
// lower routes in its expert's set; only a block that writes the plan out needs it.
template <typename SlotFn>
__device__ __forceinline__ uint32_t build_plan_experts(PlanScratch &ps, uint32_t route_idx, uint16_t route_w, uint32_t n_routes,
                                                       uint32_t n_experts, VerifyPlan *plan_out, SlotFn slot_from_total,
                                                       uint32_t &my_slot, uint32_t &e) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    e = tid < n_routes && (route_w & 0x7FFFu) != 0 && route_idx < n_experts ? route_idx : 0xFFFFFFFFu;
    ps.routes_of[tid] = uint4{0, 0, 0, 0};
    lds_barrier();      // LDS only: the token rows requested before the plan stay in flight across it
    if (e != 0xFFFFFFFFu) atomicOr(reinterpret_cast<uint32_t *>(&ps.routes_of[e]) + (tid >> 5), 1u << (tid & 31));
    lds_barrier();      // LDS only: the token rows requested before the plan stay in flight across it
    const uint4 mine = ps.routes_of[tid];
    const uint32_t count = tid < n_experts ? __popc(mine.x) + __popc(mine.y) + __popc(mine.z) + __popc(mine.w) : 0;
    ps.cnt[tid] = count;
    const bool live = count > 0;
    const unsigned long long mask = __ballot(live);
    const uint32_t before = __popcll(mask & ((1ull << lane) - 1ull));
    if (lane == 0) ps.wave_total[wave] = __popcll(mask);
    lds_barrier();      // LDS only: the token rows requested before the plan stay in flight across it
    uint32_t base = 0, total = 0;
#pragma unroll
    for (uint32_t v = 0; v < 4; ++v) {
        const uint32_t c = ps.wave_total[v];
        base += v < wave ? c : 0;
        total += c;
    }
    if (live) {
        ps.slot_of[tid] = base + before;
        ps.expert_of[base + before] = tid;
        if (plan_out) {
            plan_out->slots[base + before].expert = tid;
            plan_out->slots[base + before].n = min(count, (uint32_t)kMaxRows);
        }
    }
    if (plan_out) {
        if (tid >= total) plan_out->slots[tid].n = 0;
        if (tid == 0) plan_out->n_live = total;
    }
    // every thread read the same four counts from LDS; say so, or all that derives from the total (slot,
    // row ranges, loop bounds, load offsets) is treated as per-lane data and computed in vector registers
    total = __builtin_amdgcn_readfirstlane(total);
    my_slot = slot_from_total(total);
    lds_barrier();      // LDS only: the token rows requested before the plan stay in flight across it
    return total;
}

__device__ __forceinline__ void build_plan_routes(PlanScratch &ps, uint32_t n_routes, VerifyPlan *plan_out, uint32_t e) {
    const uint32_t tid = threadIdx.x;
    if (tid < n_routes && e != 0xFFFFFFFFu) {
        const uint4 set = ps.routes_of[e];
        const uint32_t word = tid >> 5, below = (1u << (tid & 31)) - 1u;
        const uint32_t pos = __popc(set.x & (word > 0 ? 0xFFFFFFFFu : below)) +
                             (word >= 1 ? __popc(set.y & (word > 1 ? 0xFFFFFFFFu : below)) : 0) +
                             (word >= 2 ? __popc(set.z & (word > 2 ? 0xFFFFFFFFu : below)) : 0) +
                             (word >= 3 ? __popc(set.w & below) : 0);
        if (pos < (uint32_t)kMaxRows) plan_out->slots[ps.slot_of[e]].routes[pos] = tid;
        plan_out->route_valid[tid] = pos < (uint32_t)kMaxRows ? 1u : 0u;
    } else if (tid < (uint32_t)kMaxRoutes) {
        plan_out->route_valid[tid] = 0u;
    }
}

__global__ __launch_bounds__(256) void verify_plan_kernel(const uint32_t *__restrict__ idx,
                                                          const uint16_t *__restrict__ w, uint32_t n_routes,
                                                          uint32_t n_experts, VerifyPlan *__restrict__ plan) {
    __shared__ PlanScratch ps;
    uint32_t my_slot, e;
    const bool has_route = threadIdx.x < n_routes;
    build_plan_experts(ps, has_route ? idx[threadIdx.x] : 0u, has_route ? w[threadIdx.x] : (uint16_t)0, n_routes, n_experts, plan,
                       [](uint32_t) { return 0xFFFFFFFFu; }, my_slot, e);
    build_plan_routes(ps, n_routes, plan, e);
}

// ---------------------------------------------------------------------------------------------------
// One (expert, row block) pass over groups [g0, g1). Streams A / B of a tile are gate / up rows (same
// row index) or two down row blocks. Lane l: weight row l % 16 of each stream and k-quarter l / 16; as
// the token operand it supplies token slot l % 16 (`xrow` = that token's row, already offset by
// 8 * (l / 16) elements); it ends up holding token slots 4 * (l / 16) + 0..3.
// ---------------------------------------------------------------------------------------------------
template <int PD, bool F16>
__device__ __forceinline__ TwoStreamAcc stream_tiles(const uint8_t *__restrict__ tiles,
                                                     const uint8_t *__restrict__ scales,
                                                     const uint16_t *__restrict__ xrow, uint32_t g0, uint32_t g1,
                                                     uint32_t lane) {
    const uint32_t j = lane & 15;
    TwoStreamAcc tot;
    tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
    tot.b = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const uint4 ones = {Act<F16>::kOnesBits, Act<F16>::kOnesBits, Act<F16>::kOnesBits, Act<F16>::kOnesBits};
    uint4 tbuf[PD], xb0[PD], xb1[PD];
    uint2 sbuf[PD];
#pragma unroll
    for (int u = 0; u < PD; ++u) {
        const uint32_t g = min(g0 + u, g1 - 1);
        tbuf[u] = reinterpret_cast<const uint4 *>(tiles + (size_t)g * kTileBytes)[lane];
        sbuf[u] = reinterpret_cast<const uint2 *>(scales + (size_t)g * kTileScaleBytes)[j];
    }
#pragma unroll
    for (int u = 0; u < PD; ++u) {
        const uint32_t g = min(g0 + u, g1 - 1);
        xb0[u] = *reinterpret_cast<const uint4 *>(xrow + g * kGroup);
        xb1[u] = *reinterpret_cast<const uint4 *>(xrow + g * kGroup + 32);
    }
    for (uint32_t gb = g0; gb < g1; gb += PD) {
#pragma unroll
        for (int u = 0; u < PD; ++u) {
            const uint32_t g = gb + u;
            if (g < g1) {
                const uint4 tile = tbuf[u];
                const uint2 sc = sbuf[u];
                const uint4 x0 = xb0[u], x1 = xb1[u];
                if (g + PD < g1) {
                    tbuf[u] = reinterpret_cast<const uint4 *>(tiles + (size_t)(g + PD) * kTileBytes)[lane];
                    sbuf[u] = reinterpret_cast<const uint2 *>(scales + (size_t)(g + PD) * kTileScaleBytes)[j];
                    xb0[u] = *reinterpret_cast<const uint4 *>(xrow + (g + PD) * kGroup);
                    xb1[u] = *reinterpret_cast<const uint4 *>(xrow + (g + PD) * kGroup + 32);
                }
                f32x4 acc_a = Act<F16>::mfma(x0, unpack8_offset<F16>(tile.x), zero);
                acc_a = Act<F16>::mfma(x1, unpack8_offset<F16>(tile.y), acc_a);
                f32x4 acc_b = Act<F16>::mfma(x0, unpack8_offset<F16>(tile.z), zero);
                acc_b = Act<F16>::mfma(x1, unpack8_offset<F16>(tile.w), acc_b);
                f32x4 sx = Act<F16>::mfma(x0, ones, zero);
                sx = Act<F16>::mfma(x1, ones, sx);
                const float sa = bf16lo_to_f32(sc.x), ba = bf16hi_to_f32(sc.x);
                const float sb = bf16lo_to_f32(sc.y), bb = bf16hi_to_f32(sc.y);
                const float ta = __builtin_fmaf(-Act<F16>::kOffset, sa, ba), tb = __builtin_fmaf(-Act<F16>::kOffset, sb, bb);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    tot.a[r] = __builtin_fmaf(sa, acc_a[r], tot.a[r]);
                    tot.a[r] = __builtin_fmaf(ta, sx[r], tot.a[r]);
                    tot.b[r] = __builtin_fmaf(sb, acc_b[r], tot.b[r]);
                    tot.b[r] = __builtin_fmaf(tb, sx[r], tot.b[r]);
                }
            }
        }
    }
    return tot;
}

// gate/up + GELU-tanh gating. grid = (F / 16, live-slot capacity); the four waves of a block share one
// row block and split K four ways; their partial sums meet in LDS and are added in wave order.
template <bool F16>
__global__ __launch_bounds__(256) void skinny_gate_up_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                             uint32_t top_k, const VerifyPlan *__restrict__ plan,
                                                             const uint16_t *__restrict__ x, uint32_t x_stride,
                                                             uint16_t *__restrict__ acts) {
    __shared__ float s_red[kKSplit * 8 * 64];
    const PlanSlot &slot = plan->slots[blockIdx.y];
    const uint32_t n = slot.n, expert = slot.expert;
    if (n == 0) return;
    const uint32_t tid = threadIdx.x, lane = tid & 63, ks = tid >> 6;
    const uint32_t rb = blockIdx.x;
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint8_t *expert_base = arena_layer + (size_t)expert * g.expert_bytes;
    const uint8_t *tiles = expert_base + g.gu_tiles_off + (size_t)rb * g.gd * kTileBytes;
    const uint8_t *scales = expert_base + g.gu_scales_off + (size_t)rb * g.gd * kTileScaleBytes;
    const uint32_t per = (g.gd + kKSplit - 1) / kKSplit;
    const uint32_t g0 = ks * per, g1 = min(g.gd, g0 + per);
    TwoStreamAcc tot;
    tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
    tot.b = tot.a;
    if (g0 < g1) {
        const uint32_t tok = slot.routes[min(j, n - 1)] / top_k;
        tot = stream_tiles<kRing, F16>(tiles, scales, x + (size_t)tok * x_stride + 8 * jq, g0, g1, lane);
    }
    if (ks != 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s_red[(ks * 8 + r) * 64 + lane] = tot.a[r];
            s_red[(ks * 8 + 4 + r) * 64 + lane] = tot.b[r];
        }
    }
    __syncthreads();
    if (ks != 0) return;
#pragma unroll
    for (int o = 1; o < kKSplit; ++o) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            tot.a[r] += s_red[(o * 8 + r) * 64 + lane];
            tot.b[r] += s_red[(o * 8 + 4 + r) * 64 + lane];
        }
    }
    const uint32_t row = rb * kTileRows + j;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t ts = 4 * jq + r;
        // one rounding to 16 bits, gate and up themselves stay fp32 (moe.metal:496)
        if (ts < n) acts[(size_t)slot.routes[ts] * g.f + row] = Act<F16>::round(gelu_tanh_fast(tot.a[r]) * tot.b[r]);
    }
}

// down projection. grid = (ceil(D/32 / 4), live-slot capacity); each wave owns one pair of 16-row blocks,
// the whole K = F, and all (<= 16) routes of the expert.
// Output: un-weighted rows, fp32 into `partials_f32` (fused combine) or bf16 into `partials_bf16`.
template <bool OUT_BF16, bool F16>
__global__ __launch_bounds__(256) void skinny_down_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                          const VerifyPlan *__restrict__ plan,
                                                          const uint16_t *__restrict__ acts,
                                                          float *__restrict__ partials_f32,
                                                          uint16_t *__restrict__ partials_bf16) {
    const PlanSlot &slot = plan->slots[blockIdx.y];
    const uint32_t n = slot.n, expert = slot.expert;
    if (n == 0) return;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t rbp = blockIdx.x * 4 + wave;
    if (rbp >= g.dn_rbp) return;
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint8_t *expert_base = arena_layer + (size_t)expert * g.expert_bytes;
    const uint8_t *tiles = expert_base + g.dn_tiles_off + (size_t)rbp * g.gf * kTileBytes;
    const uint8_t *scales = expert_base + g.dn_scales_off + (size_t)rbp * g.gf * kTileScaleBytes;
    const uint16_t *arow = acts + (size_t)slot.routes[min(j, n - 1)] * g.f + 8 * jq;
    const TwoStreamAcc tot = stream_tiles<kRing, F16>(tiles, scales, arow, 0, g.gf, lane);
    const uint32_t row_a = rbp * 2 * kTileRows + j, row_b = row_a + kTileRows;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t ts = 4 * jq + r;
        if (ts < n) {
            const size_t base = (size_t)slot.routes[ts] * g.d;
            if (OUT_BF16) {
                partials_bf16[base + row_a] = Act<F16>::round(tot.a[r]);
                partials_bf16[base + row_b] = Act<F16>::round(tot.b[r]);
            } else {
                partials_f32[base + row_a] = tot.a[r];
                partials_f32[base + row_b] = tot.b[r];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Persistent forms of the two kernels above for experts whose K-slice fits the register ring
// (D <= 4 * 11 * 64 and F <= 11 * 64, which covers the reference model). The grid is sized to what the
// chip holds at once; every wave keeps its token operand in registers and walks several row blocks with
// the weight ring refilled across row-block boundaries, so from its first instruction to its last a wave
// has one full K-slice (about 12 KiB) of weights in flight and never pays the load latency again.
// Groups past the end of a short K-slice are read from the last valid tile and enter with zero scales.
// ---------------------------------------------------------------------------------------------------
// gate/up + GELU-tanh gating, persistent. grid = (blocks); the blocks are dealt to the live experts, each
// block walks a range of 16-row blocks of its expert; its four waves split K and meet in LDS per row block
// (partials added in wave order), each wave finishing a quarter of the token slots.
typedef float GateUpMerge[2][kKSplit][8][64];
constexpr unsigned long long kFirstPollTicks = 100;      // 1 us (100 MHz ticks) between a block's own logits and its first look at the routes

// The token rows into the operand layout and, per group, the sum of its inputs per token column (once for all the
// tile rows a wave walks). Depends on the rows only: the launch that waits for its routes does this while it waits
// (`prepared` in gate_up_rows; measured at 1 / 8 / 16 rows: 1.0 / 1.3 / 1.5 us per call less than behind the first
// weight request), the launch that is handed its routes does it behind that request.
template <bool F16>
__device__ __forceinline__ void prepare_token_rows(uint32_t lane, uint4 (&x0)[kRing], uint4 (&x1)[kRing], f32x4 (&sx)[kRing]) {
    turn_token_rows(lane, x0, x1);
#pragma unroll
    for (int u = 0; u < kRing; ++u) sx[u] = group_input_sum<F16>(x0[u], x1[u]);
}

// From the routes (thread r < n_routes brings route r) to the stored activations: the plan, the block's share of
// its expert's row blocks, the weight stream. x0 / x1: the wave's token rows as load_token_rows() left them.
// DENSE: the one expert of a dense FFN takes every row at weight 1 (route r = row r): nothing to plan, the first
// weight request goes out with the kernel's first instructions, and block 0 writes the plan the down kernel's
// general forms and ffmoe_last_live_experts read without any block waiting for it (no plan given: none written).
template <bool F16, bool DENSE = false>
__device__ __forceinline__ void gate_up_rows(GateUpMerge &s_red, PlanScratch &ps, const uint8_t *__restrict__ arena_layer,
                                             const ArenaGeom &g, uint32_t top_k, uint32_t n_experts, uint32_t route_idx,
                                             uint16_t route_w, uint32_t n_routes, VerifyPlan *__restrict__ plan,
                                             const KSlice &k, uint4 (&x0)[kRing], uint4 (&x1)[kRing], f32x4 (&sx)[kRing],
                                             bool prepared, uint16_t *__restrict__ acts, uint32_t bid, uint32_t n_blocks) {
    const uint32_t rows = n_routes / top_k;
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint32_t g0 = k.g0, ng = k.ng, g_last = k.g_last;
    // Every block derives the routing plan itself from the (at most 128) routes: a few dozen LDS
    // operations, against a separate launch plus two dependent global reads per block. Block 0 also
    // writes the plan out for the down kernel.
    const uint32_t gu_rb = g.gu_rb;       // bid of n_blocks: this block among those that share the work
    uint32_t slot_id = 0, route_expert = 0, n_live = 1;
    VerifyPlan *plan_out = bid == 0 ? plan : nullptr;
    if constexpr (DENSE) {
        slot_id = bid / max(1u, min(gu_rb, n_blocks));
        if (plan_out) {
            const uint32_t tid = threadIdx.x;
            if (tid == 0) {
                plan_out->n_live = 1;
                plan_out->slots[0].expert = 0;
                plan_out->slots[0].n = rows;
            } else if (tid < (uint32_t)FFMOE_MAX_EXPERTS) {
                plan_out->slots[tid].n = 0;
            }
            if (tid < (uint32_t)kMaxRows) plan_out->slots[0].routes[tid] = tid;
            if (tid < (uint32_t)kMaxRoutes) plan_out->route_valid[tid] = tid < rows ? 1u : 0u;
        }
    } else {
        n_live = build_plan_experts(
            ps, route_idx, route_w, n_routes, n_experts, plan_out,
            [=](uint32_t total) { return total ? bid / max(1u, min(gu_rb, n_blocks / total)) : 0xFFFFFFFFu; }, slot_id,
            route_expert);
    }
    const bool has_slot = n_live != 0 && slot_id < n_live;
    const uint32_t blocks_per_slot = max(1u, min(gu_rb, n_blocks / max(1u, n_live)));
    uint32_t rb0 = 0, rb1 = 0;
    if (has_slot) split_range(gu_rb, blocks_per_slot, bid % blocks_per_slot, rb0, rb1);
    const bool has_rows = has_slot && rb0 < rb1;
    const uint32_t slot_expert = DENSE ? 0u : has_slot ? __builtin_amdgcn_readfirstlane(ps.expert_of[slot_id]) : 0;
    const uint8_t *expert_base = arena_layer + (size_t)slot_expert * g.expert_bytes;
    const TileSource gu_src = make_tile_source(expert_base + g.gu_tiles_off, (size_t)g.gu_rb * g.gd * kTileBytes,
                                               expert_base + g.gu_scales_off, (size_t)g.gu_rb * g.gd * kTileScaleBytes);
    WeightRing ring;
    if (has_rows) {
#pragma unroll
        for (int u = 0; u < kRing; ++u) ring_fill(ring, u, gu_src, rb0 * g.gd + min(g0 + u, g_last), lane);
    }
    if (!DENSE && plan_out) build_plan_routes(ps, n_routes, plan_out, route_expert);
    if (!has_rows) return;
    if (!prepared) prepare_token_rows<F16>(lane, x0, x1, sx);
    // this lane finishes token column 4 jq + ks; `stores` = which of that row's top_k routes go to the expert
    // (one bit at most unless a row names an expert twice)
    const uint32_t col = 4 * jq + ks;
    uint32_t stores = 0;
    if (DENSE) {
        stores = col < rows ? 1u : 0u;
    } else if (col < rows) {
        const uint32_t *set = reinterpret_cast<const uint32_t *>(&ps.routes_of[slot_expert]);
        const uint32_t first = col * top_k, word = first >> 5;
        const uint64_t pair = (uint64_t)set[word] | ((uint64_t)(word < 3 ? set[word + 1] : 0u) << 32);
        stores = (uint32_t)(pair >> (first & 31)) & ((1u << top_k) - 1u);
    }
    uint16_t *out_col = acts + (size_t)col * top_k * g.f + j;

    for (uint32_t rb = rb0; rb < rb1; ++rb) {
        // the refill targets the next row block; past the last one it re-reads the current tiles (cache hits)
        const uint32_t next_row = min(rb + 1, rb1 - 1) * g.gd;
        TwoStreamAcc tot;
        tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
        tot.b = tot.a;
#pragma unroll
        for (int u = 0; u < kRing; ++u)
            ring_step<F16>(ring, u, (uint32_t)u < ng, x0[u], x1[u], sx[u], tot, gu_src, next_row + min(g0 + u, g_last), lane);
        const int buf = (rb - rb0) & 1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s_red[buf][ks][r][lane] = tot.a[r];
            s_red[buf][ks][4 + r][lane] = tot.b[r];
        }
        lds_barrier();
        float ga = s_red[buf][0][ks][lane], ub = s_red[buf][0][4 + ks][lane];
#pragma unroll
        for (int o = 1; o < kKSplit; ++o) {
            ga += s_red[buf][o][ks][lane];
            ub += s_red[buf][o][4 + ks][lane];
        }
        // one rounding to 16 bits, gate and up themselves stay fp32 (moe.metal:496)
        const uint16_t v = Act<F16>::round(gelu_tanh_fast(ga) * ub);
        for (uint32_t todo = stores; todo; todo &= todo - 1)
            out_col[(size_t)__builtin_ctz(todo) * g.f + rb * kTileRows] = v;
    }
}

// The shared expert's gate/up as the last `blocks` blocks of a routed gate/up launch (blocks == 0: none).
struct SharedGateUp {
    const uint8_t *arena_layer;
    ArenaGeom g;
    const uint16_t *x;
    uint32_t x_stride;
    uint16_t *acts;
    uint32_t blocks;
    // an 8-bit shared expert (not null): its gate and up projections as one gated matrix of nibble planes, tiles
    // 2 p and 2 p + 1 = rows 16 p ... 16 p + 15 of the gate and of the up projection (matrix.hip); arena_layer is unused
    const uint8_t *tiles8, *scales8;
};

// What a kernel instantiated without the shared expert's role takes in its place: nothing to pass, nothing to load.
struct NoSharedExpert {};
// SHARED: 0 = no shared expert in the launch, 1 = a 4-bit one (arena tiles), 2 = an 8-bit one (nibble planes; the
// gate/up kernels only - an instantiation of its own, so the 4-bit role's registers stay as they are)
template <int SHARED, typename T>
using SharedArg = std::conditional_t<SHARED != 0, T, NoSharedExpert>;
template <int SHARED, typename T>
SharedArg<SHARED, T> shared_arg(const T &v) {
    if constexpr (SHARED != 0) return v;
    else return NoSharedExpert{};
}

// The 8-bit shared expert's gate/up rows: block `bid` of sh.blocks walks its share of the tile pairs. A pair's first tile
// gives 16 gate rows (the sum of its two nibble-plane streams), its second the up rows; both are rounded to 16 bits in
// front of the activation, as the resident-matrix GEMV does on the same tiles (matrix_gemv_kernel, gated form) and as the
// reference's shared_int8_gate_up_act_simd does (Metal/Quant/dequant_int8.metal:131-136).
template <bool F16>
__device__ __forceinline__ void shared_gate_up8_rows(GateUpMerge &s_red, const SharedGateUp &sh, uint32_t rows, uint32_t bid,
                                                     const KSlice &k, uint4 (&x0)[kRing], uint4 (&x1)[kRing], f32x4 (&sx)[kRing]) {
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint32_t pairs = sh.g.gu_rb, gd = sh.g.gd;
    uint32_t rb0, rb1;
    split_range(pairs, sh.blocks, bid, rb0, rb1);
    rb0 *= 2;
    rb1 *= 2;
    if (rb0 >= rb1) return;
    const TileSource src = make_tile_source(sh.tiles8, (size_t)2 * pairs * gd * kTileBytes, sh.scales8,
                                            (size_t)2 * pairs * gd * kTileScaleBytes);
    WeightRing ring;
#pragma unroll
    for (int u = 0; u < kRing; ++u) ring_fill(ring, u, src, rb0 * gd + min(k.g0 + u, k.g_last), lane);
    prepare_token_rows<F16>(lane, x0, x1, sx);
    const uint32_t col = 4 * jq + ks;       // the input row this lane finishes
    uint16_t *out_col = sh.acts + (size_t)col * sh.g.f + j;
    float gate_kept = 0.0f;
    for (uint32_t rb = rb0; rb < rb1; ++rb) {
        const uint32_t next_row = min(rb + 1, rb1 - 1) * gd;
        TwoStreamAcc tot;
        tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
        tot.b = tot.a;
#pragma unroll
        for (int u = 0; u < kRing; ++u)
            ring_step<F16>(ring, u, (uint32_t)u < k.ng, x0[u], x1[u], sx[u], tot, src, next_row + min(k.g0 + u, k.g_last), lane);
        const int buf = (rb - rb0) & 1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s_red[buf][ks][r][lane] = tot.a[r];
            s_red[buf][ks][4 + r][lane] = tot.b[r];
        }
        lds_barrier();
        float va = s_red[buf][0][ks][lane], vb = s_red[buf][0][4 + ks][lane];
#pragma unroll
        for (int o = 1; o < kKSplit; ++o) {
            va += s_red[buf][o][ks][lane];
            vb += s_red[buf][o][4 + ks][lane];
        }
        const float v = Act<F16>::widen(Act<F16>::round(va + vb));
        if (!(rb & 1u)) gate_kept = v;
        else if (col < rows) out_col[(rb >> 1) * kTileRows] = Act<F16>::round(gelu_tanh_fast(gate_kept) * v);
    }
}

// A block in that role: block `bid` of sh.blocks walks its share of the dense expert's row blocks for all `rows` rows.
template <bool F16, bool PLANES8>
__device__ __forceinline__ void shared_gate_up_role(GateUpMerge &s_red, PlanScratch &ps, const SharedGateUp &sh, uint32_t rows,
                                                    uint32_t bid) {
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const KSlice k = k_slice(sh.g.gd, ks);
    uint4 x0[kRing], x1[kRing];
    f32x4 sx[kRing];
    load_token_rows(sh.x, sh.x_stride, rows, lane, k, x0, x1);
    if constexpr (PLANES8) {
        shared_gate_up8_rows<F16>(s_red, sh, rows, bid, k, x0, x1, sx);
        return;
    }
    gate_up_rows<F16, true>(s_red, ps, sh.arena_layer, sh.g, 1u, 1u, 0u, (uint16_t)0, rows, nullptr, k, x0, x1, sx, false, sh.acts,
                            bid, sh.blocks);
}

template <bool F16, bool DENSE = false, int SHARED = 0>
__global__ __launch_bounds__(256, 2) void skinny_gate_up_persistent(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                                    uint32_t top_k, uint32_t n_experts,
                                                                    const uint32_t *__restrict__ idx,
                                                                    const uint16_t *__restrict__ w, uint32_t n_routes,
                                                                    VerifyPlan *__restrict__ plan,
                                                                    const uint16_t *__restrict__ x, uint32_t x_stride,
                                                                    uint16_t *__restrict__ acts,
                                                                    SharedArg<SHARED, SharedGateUp> sh) {
    __shared__ GateUpMerge s_red;
    __shared__ PlanScratch ps;
    uint32_t routed_blocks = gridDim.x;
    if constexpr (SHARED != 0) {
        routed_blocks -= sh.blocks;
        if (blockIdx.x >= routed_blocks) {
            shared_gate_up_role<F16, SHARED == 2>(s_red, ps, sh, n_routes / top_k, blockIdx.x - routed_blocks);
            return;
        }
    }
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint32_t route_idx = 0;
    uint16_t route_w = 0;
    if (!DENSE && threadIdx.x < n_routes) {
        route_idx = idx[threadIdx.x];
        route_w = w[threadIdx.x];
    }
    // the rows are requested first and are there when the plan is; no gather waits for the routing
    const KSlice k = k_slice(g.gd, ks);
    uint4 x0[kRing], x1[kRing];
    load_token_rows(x, x_stride, n_routes / top_k, lane, k, x0, x1);
    f32x4 sx[kRing];
    gate_up_rows<F16, DENSE>(s_red, ps, arena_layer, g, top_k, n_experts, route_idx, route_w, n_routes, plan, k, x0, x1, sx, false, acts,
                             blockIdx.x, routed_blocks);
}

// Router and gate/up of a decode step or verify block in ONE launch: the logits, the top-k select and the routes'
// way to every block, which otherwise are two launches in front of the kernel above, become hand-overs inside it.
// A hand-over is a 64-bit word {epoch, payload} written and polled with device-coherent accesses (relaxed atomics
// at agent scope: the store goes through to memory, the load does not stop at this chip's non-coherent L2): a word
// is either the old one or the new one, so a consumer needs no flag, fence or counter beside the data, and the
// producers wait for nobody. Measured on this part, such an edge costs 0.9 us against 2.4 us for a kernel boundary.
//   1. logits: block b takes work items b, b + grid, ... = (expert, chunk of four rows) as router_small_kernel does,
//      same pinned order, and writes the four logits as words mail->logits[row][expert].
//   2. select: the four waves of block r < rows poll row r's words and rank its candidates together
//      (block_topk_select); wave 1 writes the row's routes as words
//      mail->routes[row * top_k + rank] = {epoch, weight bits << 16 | expert} (and as plain idx / w for the caller and
//      the combine).
//   3. every block polls the routes, then continues as the kernel above. The token rows of the expert pass are
//      requested between 1 and 3, so they arrive while the block waits.
// The epoch is read from mail->epoch by every block at its start and is advanced by a later launch of the same call
// (the combine), which keeps a replayed HIP graph correct. The hand-overs are fast when every block of the grid is
// resident at once (the grid is at most the kernel's occupancy on a GPU the stream has to itself), and the results
// do not depend on it: a wave whose poll has waited `poll_ticks` (100 MHz ticks) stops waiting and makes what it
// waited for itself - the row's logits in step 2, the rows' logits, select and weights in step 3 - with the same
// arithmetic in the same order, so the call returns the same bits, later. mail->faults counts such waves.

// The next epoch, never 0: words that were never written are zero and must not look current after a wrap.
__device__ __forceinline__ void advance_epoch(RouteMail *mail) {
    const uint32_t next = mail->epoch + 1u;
    mail->epoch = next ? next : 1u;
}
// A call that cannot launch what follows its routing launch still has to retire the words that launch wrote.
__global__ void advance_epoch_kernel(RouteMail *mail) { advance_epoch(mail); }

__device__ __forceinline__ unsigned long long mail_load(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void mail_store(unsigned long long *p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The weight bits topk_store writes for the rank a lane holds (lane < top_k).
template <bool F16>
__device__ __forceinline__ uint16_t route_weight_bits(const TopkRow &tr, const uint16_t *__restrict__ per_expert_scale) {
    const float gain = per_expert_scale ? bf16_to_f32(per_expert_scale[tr.idx]) : 1.0f;
    return Act<F16>::round(tr.ex / tr.sum * gain);
}

// What a wave does when a hand-over never arrives: the logits of rows t0 .. t_last (at most kChunkTokens of them)
// against every expert by this wave alone, in the pinned order - the four sub-accumulators one after the other
// instead of one per wave, merged as router_finish merges them - as select keys (slot c, lane l: expert 64 c + l).
// Slow (hundreds of dependent memory round trips) and exact: the bits of the block-wide form.
template <bool W_F32, bool F16>
__device__ __forceinline__ void lone_wave_keys(const void *__restrict__ router_w, const uint16_t *__restrict__ effective_scale,
                                               const uint16_t *__restrict__ router_x, uint32_t router_x_stride,
                                               uint32_t n_experts, uint32_t d, uint32_t t0, uint32_t t_last, uint32_t lane,
                                               uint32_t (&keys)[kChunkTokens][4]) {
#pragma unroll
    for (int r = 0; r < kChunkTokens; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) keys[r][c] = 0u;
    for (uint32_t e = 0; e < n_experts; ++e) {
        float p0[kChunkTokens] = {0.f, 0.f, 0.f, 0.f}, p1[kChunkTokens] = {0.f, 0.f, 0.f, 0.f};
        float p2[kChunkTokens] = {0.f, 0.f, 0.f, 0.f}, p3[kChunkTokens] = {0.f, 0.f, 0.f, 0.f};
        accumulate_sub<W_F32, F16 ? 2 : 1>(router_w, effective_scale, router_x, router_x_stride, e, d, 0, lane, t0, t_last, p0);
        accumulate_sub<W_F32, F16 ? 2 : 1>(router_w, effective_scale, router_x, router_x_stride, e, d, 1, lane, t0, t_last, p1);
        accumulate_sub<W_F32, F16 ? 2 : 1>(router_w, effective_scale, router_x, router_x_stride, e, d, 2, lane, t0, t_last, p2);
        accumulate_sub<W_F32, F16 ? 2 : 1>(router_w, effective_scale, router_x, router_x_stride, e, d, 3, lane, t0, t_last, p3);
        const bool holder = lane == (e & 63u);
#pragma unroll
        for (int r = 0; r < kChunkTokens; ++r) {
            const float v = wave_butterfly_sum((p0[r] + p1[r]) + (p2[r] + p3[r]));
            const uint32_t key = v > -INFINITY ? orderable(v) : 0u;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (holder && (e >> 6) == (uint32_t)c) keys[r][c] = key;
        }
    }
}

template <bool W_F32, bool F16, int SHARED>
__global__ __launch_bounds__(256, 2) void route_gate_up_persistent(
    const uint8_t *__restrict__ arena_layer, ArenaGeom g, uint32_t top_k, uint32_t n_experts, const void *__restrict__ router_w,
    const uint16_t *__restrict__ effective_scale, const uint16_t *__restrict__ per_expert_scale,
    const uint16_t *__restrict__ router_x, uint32_t router_x_stride, uint32_t rows, RouteMail *__restrict__ mail,
    unsigned long long poll_ticks,
    uint32_t *__restrict__ out_idx, uint16_t *__restrict__ out_w, VerifyPlan *__restrict__ plan,
    const uint16_t *__restrict__ x, uint32_t x_stride, uint16_t *__restrict__ acts, SharedArg<SHARED, SharedGateUp> sh,
    uint32_t prefetch_blocks) {
    __shared__ GateUpMerge s_red;
    __shared__ PlanScratch ps;
    float(*s_part)[kChunkTokens][64] = reinterpret_cast<float(*)[kChunkTokens][64]>(&s_red[0][0][0][0]);   // 4 KiB of the 16
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t epoch = __builtin_amdgcn_readfirstlane(mail->epoch);
    const unsigned long long stamp = (unsigned long long)epoch << 32;
    const uint32_t n_routes = rows * top_k;

    // 1. logits
    const uint32_t chunks = (rows + kChunkTokens - 1) / kChunkTokens;
    for (uint32_t item = blockIdx.x; item < n_experts * chunks; item += gridDim.x) {
        const uint32_t e = item % n_experts, t0 = (item / n_experts) * kChunkTokens;
        const uint32_t t_end = min(rows, t0 + kChunkTokens);
        float acc[kChunkTokens] = {0.f, 0.f, 0.f, 0.f};
        accumulate_sub<W_F32, F16 ? 2 : 1>(router_w, effective_scale, router_x, router_x_stride, e, g.d, ks, lane, t0, t_end - 1, acc);
        if (item != blockIdx.x) __syncthreads();      // the previous item's partials have been read
#pragma unroll
        for (int r = 0; r < kChunkTokens; ++r) s_part[ks][r][lane] = acc[r];
        __syncthreads();
        if (ks == 0) {
            float mine = 0.0f;
#pragma unroll
            for (int r = 0; r < kChunkTokens; ++r) {
                const float v = router_finish(s_part, r, lane);
                if (lane == (uint32_t)r) mine = v;
            }
            if (lane < t_end - t0)
                mail_store(&mail->logits[t0 + lane][e], stamp | __float_as_uint(mine));
        }
    }
    // the blocks that serve the shared expert need no routes: they start on its rows now
    uint32_t routed_blocks = gridDim.x;
    if constexpr (SHARED == 0) routed_blocks -= prefetch_blocks;        // (the launch with the shared expert has no blocks to spare)
    if (SHARED == 0 && blockIdx.x >= routed_blocks) {
        // A decode step's spare blocks: once the row's routes are out they read the down tiles of its experts - the rows
        // the next launch's block on THIS XCD will want (blocks go to XCDs round robin) - so that launch finds them in
        // the XCD's L2. Nothing is kept; a block that never sees the routes just leaves.
        const uint32_t p = blockIdx.x - routed_blocks, xcd = blockIdx.x & 7, rb = xcd + 8 * (p >> 3);
        if (rb >= g.dn_rbp) return;
        const unsigned long long t0 = wall_clock64();
        unsigned long long word = 0;
        for (;;) {
            word = lane < n_routes ? mail_load(&mail->routes[lane]) : stamp;
            if (__all((uint32_t)(word >> 32) == epoch)) break;
            if (wall_clock64() - t0 > min(poll_ticks, 3000ull)) return;      // 30 us: the step is over (or nobody hands anything over)
            __builtin_amdgcn_s_sleep(4);
        }
        uint4 tv[2][kRing];
        uint2 sv[2][kRing];
#pragma unroll
        for (uint32_t h = 0; h < 2; ++h) {
            const uint32_t r = min(2 * ks + h, n_routes - 1);
            const uint32_t e = min((uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)word, (int)r) & 0xFFFFu, n_experts - 1);
            const uint8_t *eb = arena_layer + (size_t)e * g.expert_bytes;
            const uint4 *tiles = reinterpret_cast<const uint4 *>(eb + g.dn_tiles_off + (size_t)rb * g.gf * kTileBytes);
            const uint2 *scl = reinterpret_cast<const uint2 *>(eb + g.dn_scales_off + (size_t)rb * g.gf * kTileScaleBytes);
#pragma unroll
            for (int u = 0; u < kRing; ++u) {
                const uint32_t uu = min((uint32_t)u, g.gf - 1);
                tv[h][u] = tiles[uu * 64 + lane];
                sv[h][u] = scl[uu * 16 + (lane & 15)];
            }
        }
        // the values are wanted by nobody: an empty statement that names them keeps the loads, and nothing is stored
#pragma unroll
        for (uint32_t h = 0; h < 2; ++h)
#pragma unroll
            for (int u = 0; u < kRing; ++u)
                asm volatile("" ::"v"(tv[h][u].x), "v"(tv[h][u].y), "v"(tv[h][u].z), "v"(tv[h][u].w), "v"(sv[h][u].x), "v"(sv[h][u].y));
        return;
    }
    if constexpr (SHARED != 0) {
        routed_blocks -= sh.blocks;
        if (blockIdx.x >= routed_blocks) {
            __syncthreads();      // the logits' partial sums (in s_red) have been read
            shared_gate_up_role<F16, SHARED == 2>(s_red, ps, sh, rows, blockIdx.x - routed_blocks);
            return;
        }
    }
    // the expert pass's token rows: in flight while the routes are made
    const KSlice k = k_slice(g.gd, ks);
    uint4 x0[kRing], x1[kRing];
    load_token_rows(x, x_stride, rows, lane, k, x0, x1);

    const unsigned long long t_start = wall_clock64();
    // 2. select: the four waves of block r < rows rank row r's candidates together, wave 1 publishes the routes
    if (blockIdx.x < rows) {
        const uint32_t row = blockIdx.x;
        TopkRow tr;
        for (;;) {
            bool ok = true;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t e = c * 64 + lane;
                unsigned long long word = stamp;     // not a candidate: valid, and below every score
                float v = -INFINITY;
                if (e < n_experts) {
                    word = mail_load(&mail->logits[row][e]);
                    v = __uint_as_float((uint32_t)word);
                }
                ok = ok && (uint32_t)(word >> 32) == epoch;
                tr.key[c] = v > -INFINITY ? orderable(v) : 0u;
            }
            if (__all(ok)) break;
            if (wall_clock64() - t_start > poll_ticks) {
                // the row's logits are not coming (a block that makes them is not running): this wave makes them itself
                if (lane == 0 && ks == 1) atomicAdd(&mail->faults, 1u);
                uint32_t keys[kChunkTokens][4];
                lone_wave_keys<W_F32, F16>(router_w, effective_scale, router_x, router_x_stride, n_experts, g.d, row, row, lane, keys);
#pragma unroll
                for (int c = 0; c < 4; ++c) tr.key[c] = keys[0][c];
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        uint32_t(*s_cnt)[4][64] = reinterpret_cast<uint32_t(*)[4][64]>(&s_red[0][2][0][0]);    // the 4 KiB behind the logits' partial sums
        if (n_experts <= 128) block_topk_select<2>(tr, top_k, lane, ks, 1, s_cnt);
        else block_topk_select<4>(tr, top_k, lane, ks, 1, s_cnt);
        if (ks == 1) {
            topk_store(tr, per_expert_scale, top_k, out_idx + (size_t)row * top_k, out_w + (size_t)row * top_k, lane, F16);
            if (lane < top_k)
                mail_store(&mail->routes[row * top_k + lane], stamp | ((unsigned long long)route_weight_bits<F16>(tr, per_expert_scale) << 16) | (tr.idx & 0xFFFFu));
        }
    }
    // the rows into operand order while the routes are on their way
    f32x4 sx[kRing];
    prepare_token_rows<F16>(lane, x0, x1, sx);
    // 3. the routes
    uint32_t route_idx = 0;
    uint16_t route_w = 0;
    if (ks * 64 < n_routes) {
        const bool mine = threadIdx.x < n_routes;
        // the routes cannot be there yet: the logits' hand-over and the select come first (3 us at least). Every read
        // of the words that is spared until then is one request less for the few lines that all blocks ask for
        // (measured: 0.35 us per call; three reads in flight per wave instead of one cost 0.7 to 1.5 us)
        while (wall_clock64() - t_start < kFirstPollTicks) __builtin_amdgcn_s_sleep(8);
        for (;;) {
            const unsigned long long word = mine ? mail_load(&mail->routes[threadIdx.x]) : stamp;
            if (__all((uint32_t)(word >> 32) == epoch)) {
                route_idx = (uint32_t)word & 0xFFFFu;
                route_w = (uint16_t)((uint32_t)word >> 16);
                break;
            }
            if (wall_clock64() - t_start > poll_ticks) {
                // the routes are not coming (a block that selects is not running): this wave routes the rows of its
                // 64 routes itself - the same logits, select and weights, so the same bits
                if (lane == 0) atomicAdd(&mail->faults, 1u);
                const uint32_t r_first = (ks * 64) / top_k, r_last = min(rows - 1, (ks * 64 + 63) / top_k);
                const uint32_t my_row = threadIdx.x / top_k, my_rank = threadIdx.x % top_k;
                for (uint32_t t0 = r_first; t0 <= r_last; t0 += kChunkTokens) {
                    uint32_t keys[kChunkTokens][4];
                    lone_wave_keys<W_F32, F16>(router_w, effective_scale, router_x, router_x_stride, n_experts, g.d, t0,
                                               min(t0 + kChunkTokens - 1, rows - 1), lane, keys);
#pragma unroll
                    for (int i = 0; i < kChunkTokens; ++i) {
                        TopkRow tr;
#pragma unroll
                        for (int c = 0; c < 4; ++c) tr.key[c] = keys[i][c];
                        if (n_experts <= 128) topk_select<2>(tr, top_k, lane);
                        else topk_select<4>(tr, top_k, lane);
                        const uint32_t packed = ((uint32_t)route_weight_bits<F16>(tr, per_expert_scale) << 16) | (tr.idx & 0xFFFFu);
                        const uint32_t got = (uint32_t)__shfl((int)packed, (int)my_rank, 64);
                        if (mine && my_row == t0 + i) {
                            route_idx = got & 0xFFFFu;
                            route_w = (uint16_t)(got >> 16);
                        }
                    }
                }
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    gate_up_rows<F16>(s_red, ps, arena_layer, g, top_k, n_experts, route_idx, route_w, n_routes, plan, k, x0, x1, sx, true, acts,
                      blockIdx.x, routed_blocks);
}

// down projection with the expert's activation rows in LDS: one block = four consecutive 32-row tile rows of one
// expert, one per wave, the whole K = F (at most kRing groups) requested in one go. Without the rows in registers a
// wave fits 96 registers, so a compute unit holds twenty waves, and it is the number of waves with requests in
// flight, not the depth of each wave's queue, that this 55 MB stream responds to: measured on the same tiles, one
// wave per tile row reads them in 10 us, a persistent form's 1,024 waves of four to five tile rows each in 15 us.
// With five blocks per compute unit the blocks of up to 58 live experts are all resident from the start.
// Order of the requests: the slot's count and expert (scalar loads; a slot past the last live expert holds n = 0
// and its block leaves before it has issued anything else), the routes, then the first pieces of the activation rows
// and only then the weights. (The rows sit two dependent round trips behind the slot; a form that found them from
// the slot alone - the gate/up kernel storing them per expert - ran at the same speed: they are not what the first
// product waits for.)
constexpr int kDownLdsRow = kRing * kGroup * 2 + 16;      // bytes per activation row in LDS, padded against bank conflicts
// Weight tiles a wave has in flight. With all eleven requested at once the compute unit's twenty waves are served one
// after the other - a wave's tiles arrive in a burst, the last wave's burst at the very end of the stream, and its
// eleven products (3 us) run after everything else has finished. With four in flight and a refill per product the
// waves advance together and the stream ends with about one product per wave: 15.8 -> 13.5 us per launch
// (3 / 4 / 6 / 11 in flight: 13.8 / 13.5 / 14.2 / 15.8 us; four tiles x twenty waves = 80 KiB per compute unit in
// flight still covers the memory latency).
constexpr int kDownDepth = 4;
constexpr int kDownEarly = 2;      // 16-byte pieces of the activation rows a thread requests ahead of the weights (covers 5 rows)

// The shared expert's down projection as extra slots of the launch (first_slot = the routed slots' count; ~0u: none):
// slot first_slot + c takes groups [kRing c, kRing c + kRing) of the dense expert's K for all `rows` rows (route r = row r)
// and leaves its un-weighted fp32 rows in partials[c].
struct SharedDown {
    const uint8_t *arena_layer;
    ArenaGeom g;
    const uint16_t *acts;       // [rows][g.f]
    float *partials;            // [chunks][rows][g.d]
    uint32_t first_slot, rows;
    // an 8-bit shared expert (not null): its down projection as nibble planes, 16 weight rows per tile row (matrix.hip) -
    // twice the tile rows, so a chunk of its K takes two slots: first_slot + 2 c + h walks half h of chunk c's tile rows
    const uint8_t *tiles8, *scales8;
};

template <bool OUT_BF16, bool F16, bool SHARED>
__global__ __launch_bounds__(256, 5) void skinny_down_lds(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                          const VerifyPlan *__restrict__ plan,
                                                          const uint16_t *__restrict__ acts,
                                                          float *__restrict__ partials_f32,
                                                          uint16_t *__restrict__ partials_bf16, uint32_t parts, RouteMail *mail,
                                                          SharedArg<SHARED, SharedDown> sh_arg) {
    SharedDown sh{nullptr, g, nullptr, nullptr, 0xFFFFFFFFu, 0u, nullptr, nullptr};
    if constexpr (SHARED) sh = sh_arg;
    __shared__ __align__(16) uint8_t s_act[kMaxRows * kDownLdsRow];
    __shared__ uint32_t s_route[kMaxRows];
    // the last launch of a call that leaves its rows un-combined: the routing launch of this call has read the epoch
    if (mail && blockIdx.x == 0 && threadIdx.x == 0) advance_epoch(mail);
    const uint32_t slot_id = blockIdx.x / parts, part = blockIdx.x % parts;
    const bool shared = SHARED && slot_id >= sh.first_slot;
    const bool planes8 = SHARED && shared && sh.tiles8 != nullptr;
    const uint32_t shared_slot = shared ? slot_id - sh.first_slot : 0u;
    const uint32_t chunk = planes8 ? shared_slot >> 1 : shared_slot;
    const PlanSlot &slot = plan->slots[shared ? 0u : slot_id];
    const uint32_t n = shared ? sh.rows : __builtin_amdgcn_readfirstlane(slot.n);
    const uint32_t expert = shared ? 0u : __builtin_amdgcn_readfirstlane(slot.expert);
    if (n == 0) return;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, jq = lane >> 4;
    // the slot's share of K: all of a routed expert's f, one chunk of the shared expert's
    const uint32_t row_groups = shared ? sh.g.gf : g.gf;                                           // groups per tile row
    const uint32_t g_first = shared ? chunk * (uint32_t)kRing : 0u;
    const uint32_t ng = shared ? min((uint32_t)kRing, sh.g.gf - g_first) : g.gf, g_last = ng - 1;
    const uint32_t act_stride = shared ? sh.g.f : g.f;
    const uint16_t *act_rows = shared ? sh.acts + g_first * kGroup : acts;
    const uint32_t chunks = ng * (kGroup / 8);            // 16-byte pieces per row
    auto route_of = [&](uint32_t i) { return shared ? i : slot.routes[i]; };
    const uint32_t route_t = threadIdx.x < (uint32_t)kMaxRows ? route_of(threadIdx.x) : 0u;
    uint4 early[kDownEarly];
#pragma unroll
    for (int k = 0; k < kDownEarly; ++k) {
        const uint32_t i = threadIdx.x + 256u * k, r = i / chunks, c = i % chunks;
        // rows past the count re-read the last one (never stored): no load sits behind a branch
        early[k] = *reinterpret_cast<const uint4 *>(act_rows + (size_t)route_of(min(r, n - 1)) * act_stride + c * 8);
    }
    const uint32_t rb = planes8 ? ((shared_slot & 1u) * parts + part) * 4 + wave : part * 4 + wave;
    const bool has_row = rb < (planes8 ? 2 * g.dn_rbp : g.dn_rbp);        // d is a multiple of 32: twice as many 16-row tile rows
    const ArenaGeom &eg = shared ? sh.g : g;
    const uint8_t *expert_base = shared ? sh.arena_layer : arena_layer + (size_t)expert * g.expert_bytes;
    const TileSource src =
        planes8 ? make_tile_source(sh.tiles8, (size_t)2 * g.dn_rbp * eg.gf * kTileBytes, sh.scales8,
                                   (size_t)2 * g.dn_rbp * eg.gf * kTileScaleBytes)
                : make_tile_source(expert_base + eg.dn_tiles_off, (size_t)eg.dn_rbp * eg.gf * kTileBytes,
                                   expert_base + eg.dn_scales_off, (size_t)eg.dn_rbp * eg.gf * kTileScaleBytes);
    const uint32_t tile0 = rb * row_groups + g_first;      // the wave's first tile
    WeightRing ring;
    if (has_row) {
#pragma unroll
        for (int u = 0; u < kDownDepth; ++u) ring_fill(ring, u, src, tile0 + min((uint32_t)u, g_last), lane);
    }
    if (threadIdx.x < (uint32_t)kMaxRows) s_route[threadIdx.x] = threadIdx.x < n ? route_t : 0u;
#pragma unroll
    for (int k = 0; k < kDownEarly; ++k) {
        const uint32_t i = threadIdx.x + 256u * k, r = i / chunks, c = i % chunks;
        if (r < n) *reinterpret_cast<uint4 *>(s_act + r * kDownLdsRow + c * 16) = early[k];
    }
    if (n * chunks > 256u * kDownEarly) {
        // an expert with many rows: the remaining pieces, 16 bytes per thread and turn (these do queue behind the weights)
        lds_barrier();
        for (uint32_t i = threadIdx.x + 256u * kDownEarly; i < n * chunks; i += 256) {
            const uint32_t r = i / chunks, c = i % chunks;
            *reinterpret_cast<uint4 *>(s_act + r * kDownLdsRow + c * 16) =
                *reinterpret_cast<const uint4 *>(act_rows + (size_t)s_route[r] * act_stride + c * 8);
        }
    }
    lds_barrier();      // LDS only: the weight tiles stay in flight across it
    if (!has_row) return;
    // token slot j of the operand: row j of the expert's list, row 0 again past the count (columns never stored)
    const uint8_t *xrow = s_act + (j < n ? j : 0u) * kDownLdsRow + jq * 16;
    TwoStreamAcc tot;
    tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
    tot.b = tot.a;
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
        const bool live = (uint32_t)u < ng;
        const uint32_t gg = min((uint32_t)u, g_last);
        const uint4 x0 = *reinterpret_cast<const uint4 *>(xrow + gg * (kGroup * 2));
        const uint4 x1 = *reinterpret_cast<const uint4 *>(xrow + gg * (kGroup * 2) + 64);
        const f32x4 sx = group_input_sum<F16>(x0, x1);
        // consume slot u % kDownDepth; the load that refills it (group u + kDownDepth) starts inside the step
        if (u + kDownDepth < kRing)
            ring_step<F16, true>(ring, u % kDownDepth, live, x0, x1, sx, tot, src, tile0 + min((uint32_t)(u + kDownDepth), g_last), lane);
        else
            ring_step<F16, false>(ring, u % kDownDepth, live, x0, x1, sx, tot, src, 0u, lane);
        // The running sums are pinned here: left alone, the compiler sinks the scale-and-bias arithmetic of every
        // group into the branches of the stores at the end and carries all eleven groups' matrix results there,
        // which does not fit the register budget.
#pragma unroll
        for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(tot.a[r]), "+v"(tot.b[r]));
    }
    const uint32_t row_a = rb * 2 * kTileRows + j, row_b = row_a + kTileRows;
    float *rows_f32 = shared ? sh.partials + (size_t)chunk * sh.rows * g.d : partials_f32;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t ts = 4 * jq + r;
        if (ts < n) {
            const size_t base = (size_t)s_route[ts] * g.d;
            if (planes8) {
                rows_f32[base + rb * kTileRows + j] = tot.a[r] + tot.b[r];       // the two planes of one weight row
            } else if (OUT_BF16 && !shared) {
                partials_bf16[base + row_a] = Act<F16>::round(tot.a[r]);
                partials_bf16[base + row_b] = Act<F16>::round(tot.b[r]);
            } else {
                rows_f32[base + row_a] = tot.a[r];
                rows_f32[base + row_b] = tot.b[r];
            }
        }
    }
}

// down projection, persistent, for K = F of more than kRing groups (a wide dense expert): the blocks of the
// grid are dealt to the live experts and the four waves of a block split K as in the gate/up kernel, each
// with its slice of the activation rows in registers; the partial sums meet in LDS and wave ks finishes
// token slots 4 * (lane / 16) + ks.
// DENSE (dense_rows > 0 rows of a dense FFN: expert 0, route r = row r): nothing is read from the plan, so the weights
// and the activation rows are requested with the kernel's first instructions instead of two and three dependent
// round trips in.
template <bool OUT_BF16, bool F16, bool DENSE = false>
__global__ __launch_bounds__(256, 2) void skinny_down_ksplit_persistent(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                                        const VerifyPlan *__restrict__ plan,
                                                                        const uint16_t *__restrict__ acts,
                                                                        float *__restrict__ partials_f32,
                                                                        uint16_t *__restrict__ partials_bf16, uint32_t dense_rows) {
    __shared__ float s_red[2][kKSplit][8][64];
    const uint32_t n_live = DENSE ? 1u : __builtin_amdgcn_readfirstlane(plan->n_live);
    if (n_live == 0) return;
    const uint32_t bid = blockIdx.x;
    const uint32_t blocks_per_slot = max(1u, min(g.dn_rbp, gridDim.x / n_live));
    const uint32_t slot_id = bid / blocks_per_slot;
    if (slot_id >= n_live) return;
    uint32_t rb0, rb1;
    split_range(g.dn_rbp, blocks_per_slot, bid % blocks_per_slot, rb0, rb1);
    if (rb0 >= rb1) return;
    const PlanSlot &slot = plan->slots[slot_id];
    const uint32_t n = DENSE ? dense_rows : __builtin_amdgcn_readfirstlane(slot.n);
    const uint32_t expert = DENSE ? 0u : __builtin_amdgcn_readfirstlane(slot.expert);
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, jq = lane >> 4;
    auto route_of = [&](uint32_t i) { return DENSE ? i : slot.routes[i]; };
    const uint8_t *expert_base = arena_layer + (size_t)expert * g.expert_bytes;
    const uint32_t per = (g.gf + kKSplit - 1) / kKSplit;
    const uint32_t g0 = min(ks * per, g.gf), g1 = min(g.gf, g0 + per), ng = g1 - g0;
    const uint32_t g_last = g1 > g0 ? g1 - 1 : g.gf - 1;
    const TileSource src = make_tile_source(expert_base + g.dn_tiles_off, (size_t)g.dn_rbp * g.gf * kTileBytes,
                                            expert_base + g.dn_scales_off, (size_t)g.dn_rbp * g.gf * kTileScaleBytes);
    WeightRing ring;
#pragma unroll
    for (int u = 0; u < kRing; ++u) ring_fill(ring, u, src, rb0 * g.gf + min(g0 + u, g_last), lane);
    // a wide expert is a dense one: up to 16 distinct activation rows, fetched four lanes per 64 contiguous
    // bytes (slot lane / 4, chunk lane % 4) and turned into the operand layout by cross-lane moves
    // (with one or two rows the operand layout itself is as cheap to load, and needs no moves)
    const bool gather4 = n > 2;
    const uint16_t *arow = gather4 ? acts + (size_t)route_of(min(lane >> 2, n - 1)) * g.f + 8 * (lane & 3)
                                   : acts + (size_t)route_of(min(j, n - 1)) * g.f + 8 * jq;
    uint4 x0[kRing], x1[kRing];
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
        const bool live = (uint32_t)u < ng;
        const uint32_t gg = min(g0 + u, g_last);
        x0[u] = live ? *reinterpret_cast<const uint4 *>(arow + gg * kGroup) : uint4{0, 0, 0, 0};
        x1[u] = live ? *reinterpret_cast<const uint4 *>(arow + gg * kGroup + 32) : uint4{0, 0, 0, 0};
    }
    if (gather4) {
        const int pull = (int)((4 * j + jq) * 4);
        auto turn = [&](uint4 &v) {
            v.x = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.x);
            v.y = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.y);
            v.z = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.z);
            v.w = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.w);
        };
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
            turn(x0[u]);
            turn(x1[u]);
        }
    }
    // per group: the sum of its inputs per token column, once for all the tile rows this wave walks
    f32x4 sx[kRing];
#pragma unroll
    for (int u = 0; u < kRing; ++u) sx[u] = group_input_sum<F16>(x0[u], x1[u]);
    const uint32_t my_ts = 4 * jq + ks;     // the token slot this lane finishes
    const size_t out_base = (size_t)route_of(min(my_ts, n - 1)) * g.d;

    for (uint32_t rb = rb0; rb < rb1; ++rb) {
        const uint32_t next_row = min(rb + 1, rb1 - 1) * g.gf;
        TwoStreamAcc tot;
        tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
        tot.b = tot.a;
#pragma unroll
        for (int u = 0; u < kRing; ++u)
            ring_step<F16>(ring, u, (uint32_t)u < ng, x0[u], x1[u], sx[u], tot, src, next_row + min(g0 + u, g_last), lane);
        const int buf = (rb - rb0) & 1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s_red[buf][ks][r][lane] = tot.a[r];
            s_red[buf][ks][4 + r][lane] = tot.b[r];
        }
        lds_barrier();
        float va = s_red[buf][0][ks][lane], vb = s_red[buf][0][4 + ks][lane];
#pragma unroll
        for (int o = 1; o < kKSplit; ++o) {
            va += s_red[buf][o][ks][lane];
            vb += s_red[buf][o][4 + ks][lane];
        }
        const uint32_t row_a = rb * 2 * kTileRows + j, row_b = row_a + kTileRows;
        if (my_ts < n) {
            if (OUT_BF16) {
                partials_bf16[out_base + row_a] = Act<F16>::round(va);
                partials_bf16[out_base + row_b] = Act<F16>::round(vb);
            } else {
                partials_f32[out_base + row_a] = va;
                partials_f32[out_base + row_b] = vb;
            }
        }
    }
}

// Decode step (one row): down projection and combine in one launch. A block owns one 32-row tile row of the
// output for ALL of the row's routes, wave r the expert of route r: every wave requests its 11 KiB of
// weights and its activation row at once, the eight results meet in LDS and are added in rank order with
// the arithmetic of combine_kernel (residual first, fmaf per route), so the output is bit for bit what the
// two launches give. No plan is read: a wave takes its expert and weight straight from the routes.
template <bool F16>
__global__ __launch_bounds__(512, 1) void decode_down_combine_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                                     uint32_t n_experts, uint32_t top_k,
                                                                     const uint32_t *__restrict__ idx,
                                                                     const uint16_t *__restrict__ w,
                                                                     const uint16_t *__restrict__ acts,
                                                                     const uint16_t *__restrict__ residual,
                                                                     uint16_t *__restrict__ y, RouteMail *mail) {
    __shared__ float s_row[8][2 * kTileRows];
    if (mail && blockIdx.x == 0 && threadIdx.x == 0) advance_epoch(mail);      // the routing launch of this call has read it
    __shared__ float s_w[8];
    const uint32_t lane = threadIdx.x & 63, r = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t rb = blockIdx.x, j = lane & 15, jq = lane >> 4;
    uint32_t expert = 0;
    uint16_t wbits = 0;
    if (r < top_k) {
        expert = __builtin_amdgcn_readfirstlane(idx[r]);
        wbits = (uint16_t)__builtin_amdgcn_readfirstlane((uint32_t)w[r]);
    }
    const bool live = r < top_k && (wbits & 0x7FFFu) != 0 && expert < n_experts;
    if (lane == 0) s_w[r] = live ? Act<F16>::widen(wbits) : 0.0f;
    if (live) {
        const uint8_t *expert_base = arena_layer + (size_t)expert * g.expert_bytes;
        const TileSource src = make_tile_source(expert_base + g.dn_tiles_off, (size_t)g.dn_rbp * g.gf * kTileBytes,
                                                expert_base + g.dn_scales_off, (size_t)g.dn_rbp * g.gf * kTileScaleBytes);
        const uint32_t ng = g.gf, g_last = g.gf - 1;
        WeightRing ring;
#pragma unroll
        for (int u = 0; u < kRing; ++u) ring_fill(ring, u, src, rb * ng + min((uint32_t)u, g_last), lane);
        const uint16_t *arow = acts + (size_t)r * g.f + 8 * jq;      // one row: every token column reads it
        uint4 x0[kRing], x1[kRing];
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
            const bool in = (uint32_t)u < ng;
            const uint32_t gg = min((uint32_t)u, g_last);
            x0[u] = in ? *reinterpret_cast<const uint4 *>(arow + gg * kGroup) : uint4{0, 0, 0, 0};
            x1[u] = in ? *reinterpret_cast<const uint4 *>(arow + gg * kGroup + 32) : uint4{0, 0, 0, 0};
        }
        // per group: the sum of its inputs per token column, once for all the tile rows this wave walks
        f32x4 sx[kRing];
#pragma unroll
        for (int u = 0; u < kRing; ++u) sx[u] = group_input_sum<F16>(x0[u], x1[u]);
        TwoStreamAcc tot;
        tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
        tot.b = tot.a;
#pragma unroll
        for (int u = 0; u < kRing; ++u)
            ring_step<F16>(ring, u, (uint32_t)u < ng, x0[u], x1[u], sx[u], tot, src, rb * ng + min((uint32_t)u, g_last), lane);
        if (jq == 0) {          // token column 0 sits in the first element of lanes 0..15
            s_row[r][j] = tot.a[0];
            s_row[r][kTileRows + j] = tot.b[0];
        }
    }
    __syncthreads();
    if (threadIdx.x < 2 * kTileRows) {
        const uint32_t row = rb * 2 * kTileRows + threadIdx.x;
        float acc = residual ? Act<F16>::widen(residual[row]) : 0.0f;
        for (uint32_t q = 0; q < top_k; ++q) {
            const float wv = s_w[q];
            if (wv != 0.0f) acc = __builtin_fmaf(wv, s_row[q][threadIdx.x], acc);      // a dead route left no row
        }
        y[row] = Act<F16>::round(acc);
    }
}

// y[t][c] = bf16(residual + sum_r w[t][r] * partial[t*k + r][c]) in rank order with fmaf, fp32 partials,
// one rounding at the end (the decode form, moe.metal:627-636). Routes the plan skips (zero weight, expert
// out of range, or beyond an expert's first 16 routes) add nothing: their rows were never written.
template <bool F16>
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ partials,
                                                      const uint16_t *__restrict__ w,
                                                      const VerifyPlan *__restrict__ plan,
                                                      const uint16_t *__restrict__ residual, uint32_t top_k,
                                                      uint32_t d, uint16_t *__restrict__ y, RouteMail *mail) {
    const uint32_t tok = blockIdx.y;
    if (mail && blockIdx.x == 0 && tok == 0 && threadIdx.x == 0) advance_epoch(mail);      // the routing launch of this call has read it
    const uint32_t c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= d) return;
    // One round trip: the routes' weights and validity and all eight rows are requested together. A row the plan
    // skipped was never written and may hold anything: it is loaded like the others and dropped by the select below
    // (its address is inside the buffer either way), instead of being asked for only once its validity has arrived.
    float wv[8];
    uint32_t valid[8];
    f32x4 p[8];
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        const uint32_t route = tok * top_k + min(r, top_k - 1);
        wv[r] = Act<F16>::widen(w[route]);
        valid[r] = plan->route_valid[route];
        p[r] = *reinterpret_cast<const f32x4 *>(partials + (size_t)route * d + c);
    }
    bool live[8];
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) live[r] = r < top_k && valid[r] != 0;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (residual) {
        const uint2 rv = *reinterpret_cast<const uint2 *>(residual + (size_t)tok * d + c);
        acc[0] = Act<F16>::lo(rv.x); acc[1] = Act<F16>::hi(rv.x);
        acc[2] = Act<F16>::lo(rv.y); acc[3] = Act<F16>::hi(rv.y);
    }
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        if (live[r]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(wv[r], p[r][i], acc[i]);
        }
    }
    uint2 o;
    o.x = Act<F16>::pack(acc[0], acc[1]);
    o.y = Act<F16>::pack(acc[2], acc[3]);
    *reinterpret_cast<uint2 *>(y + (size_t)tok * d + c) = o;
}

// prefill_moe_reduce_token_major (prefill.metal:544-565) on 16-bit partials.
template <bool F16>
__global__ __launch_bounds__(256) void reduce_token_major_kernel(const uint16_t *__restrict__ partials,
                                                                 const uint16_t *__restrict__ w, uint32_t top_k,
                                                                 uint32_t d, uint16_t *__restrict__ h2) {
    const uint32_t tok = blockIdx.y;
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    float acc = 0.0f;
    for (uint32_t r = 0; r < top_k; ++r) {
        const size_t route = (size_t)tok * top_k + r;
        acc = __builtin_fmaf(Act<F16>::widen(w[route]), Act<F16>::widen(partials[route * d + c]), acc);
    }
    h2[(size_t)tok * d + c] = Act<F16>::round(acc);
}

}  // namespace

namespace {

template <bool F16>
hipError_t launch_verify_as(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts, uint32_t top_k,
                            const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx, const uint16_t *w,
                            const uint16_t *residual, uint16_t *y, uint16_t *partials_bf16, VerifyPlan *plan, uint16_t *acts,
                            float *partials_f32, uint32_t n_cus, KernelTimer *timer, const RouteFusion *route, bool dense,
                            const SharedExpert *shared) {
    // `route`: the routes are not there yet - idx / w are where this call has to write them. One launch does the
    // router and gate/up when the expert fits the persistent kernel, the combine follows in this call (it advances
    // the epoch) and the router rows are 8-byte aligned; otherwise the router's own two launches go first.
    const bool fits_ring = (g.gd + kKSplit - 1) / kKSplit <= (uint32_t)kRing;
    // y == nullptr (and no 16-bit rows wanted): the call ends with the down projection and leaves the un-weighted fp32
    // rows, the plan's route_valid and the routes' weights to a later launch that combines them (the layer tail)
    const bool rows_only = !y && !partials_bf16;
    const bool fuse = route && route->one_launch && route->resident_blocks >= t && fits_ring && !partials_bf16 && top_k <= 8 &&
                      n_experts <= FFMOE_MAX_EXPERTS && reinterpret_cast<uintptr_t>(route->router_x) % 8 == 0 &&
                      route->router_x_stride % 4 == 0;
    if (route && !fuse) {
        const hipError_t e = launch_router(s, route->rw, route->router_x, route->router_x_stride, t, n_experts, g.d, top_k,
                                           route->logits, const_cast<uint32_t *>(idx), const_cast<uint16_t *>(w), timer, F16);
        if (e != hipSuccess) return e;
    }
    timer->begin(s);
    const uint32_t slots = min(n_experts, t * top_k);
    // the persistent kernels hold a K-slice of kRing groups per wave; larger experts take the one-shot grids
    const bool gu_persistent = (g.gd + kKSplit - 1) / kKSplit <= (uint32_t)kRing;
    const bool dn_whole = g.gf <= (uint32_t)kRing;                                     // a wave holds all of K
    const bool dn_ksplit = !dn_whole && (g.gf + kKSplit - 1) / kKSplit <= (uint32_t)kRing;
    const uint32_t resident = 2 * n_cus;       // blocks the chip holds at once (__launch_bounds__(256, 2))
    const bool decode_form = t == 1 && dn_whole && !partials_bf16 && !rows_only && top_k <= 8;
    // The shared expert rides along in the persistent gate/up launch and the LDS form of the down launch.
    if (shared && !(gu_persistent && dn_whole && rows_only && shared->g.d == g.d && shared->g.gd == g.gd))
        return hipErrorInvalidValue;
    const bool shared8 = shared && shared->gu_tiles8;
    if (shared8 && (!shared->gu_scales8 || !shared->dn_tiles8 || !shared->dn_scales8 || shared->g.f % 16 || g.d % 32))
        return hipErrorInvalidValue;
    SharedGateUp sh_gu{nullptr, g, nullptr, 0u, nullptr, 0u, nullptr, nullptr};
    SharedDown sh_dn{nullptr, g, nullptr, nullptr, 0xFFFFFFFFu, 0u, nullptr, nullptr};
    auto shared_blocks = [&](uint32_t cap, uint32_t routed_wanted) -> uint32_t {
        // Blocks for the shared expert's row blocks: one each when the grid has room (a decode step); else its share of
        // the resident blocks by row blocks, the routed experts counted at the number of live ones a block of t rows
        // typically has (three per row). They start while the routed blocks wait for their routes, so a block of
        // theirs may walk a row block or two more than a routed one: a fifth fewer than the fair share. Measured per
        // layer block of 16 / 8 / 4 rows with 12 ... 132 such blocks: flat within 0.5 us from 19 / 27 / 33 blocks up
        // (70.0 / 55.8 / 44.4 us; this rule picks 23 / 42 / 72), 6 to 12 us worse at 12 blocks.
        const uint32_t rb = shared->g.gu_rb, work = shared8 ? 2 * rb : rb;      // 8-bit: a row block is a pair of tiles
        if (routed_wanted + rb <= cap) return rb;
        const uint32_t live = min(slots, 3 * t + 2);
        const uint32_t fair = (uint32_t)(((uint64_t)cap * work) / ((uint64_t)live * g.gu_rb + work));
        return max(1u, min(rb, min(cap / 2, fair - fair / 5)));
    };
    if (fuse) {
        // at least one block per row (it selects the row's routes), at most what is resident at once
        uint32_t blocks = min(route->resident_blocks, max(max(slots, t), min(route->resident_blocks, slots * g.gu_rb)));
        if (shared) {
            const uint32_t sb = shared_blocks(route->resident_blocks, blocks);
            sh_gu = SharedGateUp{shared->arena_layer, shared->g, shared->x, shared->x_stride, shared->acts, sb, shared->gu_tiles8, shared->gu_scales8};
            blocks = max(t, min(blocks, route->resident_blocks - sb)) + sb;
        }
        // A decode step leaves blocks to spare: one per tile row of the down projection reads that row's tiles of the
        // step's experts as soon as the routes are out, into the L2 of the XCD whose block of the next launch will want
        // them (measured: 21.6 -> 20.3 us per step; the next launch is a round trip of eight 11 KiB reads per wave and
        // little else)
        uint32_t prefetch_blocks = 0;
        if (decode_form && !shared && (blocks + 7) / 8 * 8 + 8 * ((g.dn_rbp + 7) / 8) <= route->resident_blocks) {
            prefetch_blocks = 8 * ((g.dn_rbp + 7) / 8);
            blocks = (blocks + 7) / 8 * 8 + prefetch_blocks;       // the spare blocks start on XCD 0 (blocks go to XCDs round robin)
        }
#define FFMOE_ROUTE_GU(WF, SH)                                                                                              \
    hipLaunchKernelGGL((route_gate_up_persistent<WF, F16, SH>), dim3(blocks), dim3(256), 0, s, arena_layer, g, top_k, n_experts, \
                       route->rw.w, route->rw.effective_scale, route->rw.per_expert_scale, route->router_x,                  \
                       route->router_x_stride, t, route->mail, route->poll_ticks, const_cast<uint32_t *>(idx),                \
                       const_cast<uint16_t *>(w), plan,                                                                     \
                       x, x_stride, acts, shared_arg<SH>(sh_gu), prefetch_blocks)
        if (shared8) { if (route->rw.w_is_f32) FFMOE_ROUTE_GU(true, 2); else FFMOE_ROUTE_GU(false, 2); }
        else if (shared) { if (route->rw.w_is_f32) FFMOE_ROUTE_GU(true, 1); else FFMOE_ROUTE_GU(false, 1); }
        else { if (route->rw.w_is_f32) FFMOE_ROUTE_GU(true, 0); else FFMOE_ROUTE_GU(false, 0); }
#undef FFMOE_ROUTE_GU
    } else if (gu_persistent) {
        // plan slot of the profile stays empty: the gate/up kernel builds the plan itself
        uint32_t blocks = max(slots, min(resident, slots * g.gu_rb));
        if (shared) {
            const uint32_t sb = shared_blocks(max(resident, blocks), blocks);
            sh_gu = SharedGateUp{shared->arena_layer, shared->g, shared->x, shared->x_stride, shared->acts, sb, shared->gu_tiles8, shared->gu_scales8};
            blocks = max(1u, min(blocks, max(resident, blocks) - sb)) + sb;
        }
        if (dense)
            hipLaunchKernelGGL((skinny_gate_up_persistent<F16, true>), dim3(blocks), dim3(256), 0, s, arena_layer, g, top_k,
                               n_experts, idx, w, t * top_k, plan, x, x_stride, acts, NoSharedExpert{});
        else if (shared8)
            hipLaunchKernelGGL((skinny_gate_up_persistent<F16, false, 2>), dim3(blocks), dim3(256), 0, s, arena_layer, g, top_k,
                               n_experts, idx, w, t * top_k, plan, x, x_stride, acts, sh_gu);
        else if (shared)
            hipLaunchKernelGGL((skinny_gate_up_persistent<F16, false, 1>), dim3(blocks), dim3(256), 0, s, arena_layer, g, top_k,
                               n_experts, idx, w, t * top_k, plan, x, x_stride, acts, sh_gu);
        else
            hipLaunchKernelGGL(skinny_gate_up_persistent<F16>, dim3(blocks), dim3(256), 0, s, arena_layer, g, top_k, n_experts, idx,
                               w, t * top_k, plan, x, x_stride, acts, NoSharedExpert{});
    } else {
        hipLaunchKernelGGL(verify_plan_kernel, dim3(1), dim3(256), 0, s, idx, w, t * top_k, n_experts, plan);
        timer->mark(s, FFMOE_K_PLAN);
        hipLaunchKernelGGL(skinny_gate_up_kernel<F16>, dim3(g.gu_rb, slots), dim3(256), 0, s, arena_layer, g, top_k, plan, x,
                           x_stride, acts);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, fuse ? FFMOE_K_ROUTE_GATE_UP : FFMOE_K_GATE_UP);
    RouteMail *const mail = fuse ? route->mail : nullptr;
    // from here on the routing launch's words are out: whatever else fails, the epoch moves on, or the next call
    // would take this call's words for its own
    auto give_up = [&](hipError_t why) {
        if (mail) hipLaunchKernelGGL(advance_epoch_kernel, dim3(1), dim3(1), 0, s, mail);
        (void)hipGetLastError();
        timer->finish();
        return why;
    };
    if (decode_form) {
        // a decode step: down projection and combine in one launch (its time sits in the down slot)
        hipLaunchKernelGGL(decode_down_combine_kernel<F16>, dim3(g.dn_rbp), dim3(512), 0, s, arena_layer, g, n_experts, top_k, idx,
                           w, acts, residual, y, mail);
        e = hipGetLastError();
        if (e != hipSuccess) return give_up(e);
        timer->mark(s, FFMOE_K_DOWN);
        timer->finish();
        return hipSuccess;
    }
    const uint32_t dn_parts = (g.dn_rbp + 3) / 4;          // blocks per expert of the LDS form: four tile rows each
    const bool dense_ksplit = dense && gu_persistent;      // the plan-free forms go together
    if (shared) sh_dn = SharedDown{shared->arena_layer, shared->g, shared->acts, shared->partials, slots, t, shared->dn_tiles8, shared->dn_scales8};
    const dim3 dn_grid = dn_whole    ? dim3((slots + (shared ? shared_chunks(shared->g) * (shared8 ? 2u : 1u) : 0u)) * dn_parts)
                         : dn_ksplit ? dim3(max(slots, min(resident, slots * g.dn_rbp)))
                                     : dim3((g.dn_rbp + 3) / 4, slots);
#define FFMOE_DOWN(BF)                                                                                                \
    if (dn_whole && shared)                                                                                           \
        hipLaunchKernelGGL((skinny_down_lds<BF, F16, true>), dn_grid, dim3(256), 0, s, arena_layer, g, plan, acts,    \
                           partials_f32, partials_bf16, dn_parts, rows_only ? mail : nullptr, sh_dn);                  \
    else if (dn_whole)                                                                                                \
        hipLaunchKernelGGL((skinny_down_lds<BF, F16, false>), dn_grid, dim3(256), 0, s, arena_layer, g, plan, acts,   \
                           partials_f32, partials_bf16, dn_parts, rows_only ? mail : nullptr, NoSharedExpert{});       \
    else if (dn_ksplit && dense_ksplit)                                                                               \
        hipLaunchKernelGGL((skinny_down_ksplit_persistent<BF, F16, true>), dn_grid, dim3(256), 0, s, arena_layer, g,  \
                           plan, acts, partials_f32, partials_bf16, t);                                               \
    else if (dn_ksplit)                                                                                               \
        hipLaunchKernelGGL((skinny_down_ksplit_persistent<BF, F16>), dn_grid, dim3(256), 0, s, arena_layer, g, plan,  \
                           acts, partials_f32, partials_bf16, 0u);                                                    \
    else                                                                                                              \
        hipLaunchKernelGGL((skinny_down_kernel<BF, F16>), dn_grid, dim3(256), 0, s, arena_layer, g, plan, acts,       \
                           partials_f32, partials_bf16)
    if (partials_bf16) {
        FFMOE_DOWN(true);
        timer->mark(s, FFMOE_K_DOWN);
        timer->finish();
        return hipGetLastError();
    }
    FFMOE_DOWN(false);
#undef FFMOE_DOWN
    e = hipGetLastError();
    if (e != hipSuccess) return give_up(e);
    timer->mark(s, FFMOE_K_DOWN);
    if (rows_only) {
        // the epoch went on with the down launch; a down kernel that takes no mail gets a launch of its own for it
        if (mail && !dn_whole) hipLaunchKernelGGL(advance_epoch_kernel, dim3(1), dim3(1), 0, s, mail);
        timer->finish();
        return hipGetLastError();
    }
    hipLaunchKernelGGL(combine_kernel<F16>, dim3((g.d / 4 + 255) / 256, t), dim3(256), 0, s, partials_f32, w, plan, residual,
                       top_k, g.d, y, mail);
    e = hipGetLastError();
    if (e != hipSuccess) return give_up(e);
    timer->mark(s, FFMOE_K_COMBINE);
    timer->finish();
    return hipSuccess;
}

}  // namespace

namespace {

// ---------------------------------------------------------------------------------------------------
// Stream probe: the tile and scale loads of the two expert kernels for `n_live` experts, in their grids, with their
// ring and their refill order - and nothing else: no routes, no token rows, no matrix products, no stores (the or of
// everything a lane read ends in an empty statement that names it, which is all the loads need to stay). What these
// two launches take is what this memory system gives the access pattern: the ceiling the expert pass is held against.
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t ring_or(const WeightRing &ring, int u) {
    return ring.t[u].x | ring.t[u].y | ring.t[u].z | ring.t[u].w | ring.s[u].x | ring.s[u].y;
}

__global__ __launch_bounds__(256, 2) void probe_gate_up_stream_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                                      uint32_t n_experts, uint32_t n_live) {
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const KSlice k = k_slice(g.gd, ks);
    const uint32_t blocks_per_slot = max(1u, min(g.gu_rb, gridDim.x / n_live));
    const uint32_t slot_id = blockIdx.x / blocks_per_slot;
    if (slot_id >= n_live) return;
    uint32_t rb0, rb1;
    split_range(g.gu_rb, blocks_per_slot, blockIdx.x % blocks_per_slot, rb0, rb1);
    if (rb0 >= rb1) return;
    const uint32_t expert = (uint32_t)((uint64_t)slot_id * n_experts / n_live);      // spread over the layer
    const uint8_t *expert_base = arena_layer + (size_t)expert * g.expert_bytes;
    const TileSource src = make_tile_source(expert_base + g.gu_tiles_off, (size_t)g.gu_rb * g.gd * kTileBytes,
                                            expert_base + g.gu_scales_off, (size_t)g.gu_rb * g.gd * kTileScaleBytes);
    WeightRing ring;
#pragma unroll
    for (int u = 0; u < kRing; ++u) ring_fill(ring, u, src, rb0 * g.gd + min(k.g0 + u, k.g_last), lane);
    uint32_t seen = 0;
    for (uint32_t rb = rb0; rb < rb1; ++rb) {
        const uint32_t next_row = min(rb + 1, rb1 - 1) * g.gd;
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
            seen |= ring_or(ring, u);
            ring_fill(ring, u, src, next_row + min(k.g0 + u, k.g_last), lane);
        }
    }
#pragma unroll
    for (int u = 0; u < kRing; ++u) seen |= ring_or(ring, u);
    asm volatile("" ::"v"(seen));      // names the value: the loads stay, nothing is stored
}

__global__ __launch_bounds__(256, 5) void probe_down_stream_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                                   uint32_t n_experts, uint32_t n_live, uint32_t parts) {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t slot_id = blockIdx.x / parts, part = blockIdx.x % parts;
    if (slot_id >= n_live) return;
    const uint32_t rb = part * 4 + wave;
    if (rb >= g.dn_rbp) return;
    const uint32_t expert = (uint32_t)((uint64_t)slot_id * n_experts / n_live);
    const uint8_t *expert_base = arena_layer + (size_t)expert * g.expert_bytes;
    const TileSource src = make_tile_source(expert_base + g.dn_tiles_off, (size_t)g.dn_rbp * g.gf * kTileBytes,
                                            expert_base + g.dn_scales_off, (size_t)g.dn_rbp * g.gf * kTileScaleBytes);
    WeightRing ring;
#pragma unroll
    for (int u = 0; u < kRing; ++u) ring_fill(ring, u, src, rb * g.gf + min((uint32_t)u, g.gf - 1), lane);
    uint32_t seen = 0;
#pragma unroll
    for (int u = 0; u < kRing; ++u) seen |= ring_or(ring, u);
    asm volatile("" ::"v"(seen));      // names the value: the loads stay, nothing is stored
}

}  // namespace

hipError_t launch_probe_stream(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts, uint32_t n_live,
                               uint32_t n_cus, KernelTimer *timer) {
    timer->begin(s);
    const uint32_t resident = 2 * n_cus;
    const uint32_t gu_blocks = max(n_live, min(resident, n_live * g.gu_rb));
    hipLaunchKernelGGL(probe_gate_up_stream_kernel, dim3(gu_blocks), dim3(256), 0, s, arena_layer, g, n_experts, n_live);
    timer->mark(s, FFMOE_K_PROBE_GATE_UP);
    const uint32_t dn_parts = (g.dn_rbp + 3) / 4;
    hipLaunchKernelGGL(probe_down_stream_kernel, dim3(n_live * dn_parts), dim3(256), 0, s, arena_layer, g, n_experts, n_live,
                       dn_parts);
    timer->mark(s, FFMOE_K_PROBE_DOWN);
    timer->finish();
    return hipGetLastError();
}

// Blocks of the routing launch that one GPU holds at once: the kernel's own occupancy (registers, LDS) as the runtime
// reports it for every instantiation, times the compute units. 0 when the query fails: the call then routes with
// launches of its own.
uint32_t route_launch_resident_blocks(uint32_t n_cus) {
    int least = 1 << 30;
    auto ask = [&](auto kernel) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0) != hipSuccess) n = 0;
        least = n < least ? n : least;
    };
    ask(route_gate_up_persistent<false, false, 0>);
    ask(route_gate_up_persistent<true, false, 0>);
    ask(route_gate_up_persistent<false, true, 0>);
    ask(route_gate_up_persistent<true, true, 0>);
    ask(route_gate_up_persistent<false, false, 1>);
    ask(route_gate_up_persistent<true, false, 1>);
    ask(route_gate_up_persistent<false, true, 1>);
    ask(route_gate_up_persistent<true, true, 1>);
    ask(route_gate_up_persistent<false, false, 2>);
    ask(route_gate_up_persistent<true, false, 2>);
    ask(route_gate_up_persistent<false, true, 2>);
    ask(route_gate_up_persistent<true, true, 2>);
    (void)hipGetLastError();
    return least > 0 ? (uint32_t)least * n_cus : 0u;
}

// x, w, residual, y and the 16-bit partial rows are FP16 when `f16`, bf16 otherwise
hipError_t launch_verify(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts,
                         uint32_t top_k, const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx,
                         const uint16_t *w, const uint16_t *residual, uint16_t *y, uint16_t *partials_bf16,
                         VerifyPlan *plan, uint16_t *acts, float *partials_f32, uint32_t n_cus, KernelTimer *timer, bool f16,
                         const RouteFusion *route, bool dense, const SharedExpert *shared) {
    // dense: the caller vouches that this is a dense FFN - one expert, top_k = 1, every row at weight 1
    dense = dense && n_experts == 1 && top_k == 1 && !route;
    return f16 ? launch_verify_as<true>(s, arena_layer, g, n_experts, top_k, x, x_stride, t, idx, w, residual, y, partials_bf16,
                                        plan, acts, partials_f32, n_cus, timer, route, dense, shared)
               : launch_verify_as<false>(s, arena_layer, g, n_experts, top_k, x, x_stride, t, idx, w, residual, y, partials_bf16,
                                         plan, acts, partials_f32, n_cus, timer, route, dense, shared);
}

hipError_t launch_reduce_token_major(hipStream_t s, const uint16_t *partials, const uint16_t *weights,
                                     uint16_t *h2, uint32_t t, uint32_t top_k, uint32_t d, bool f16) {
    if (f16)
        hipLaunchKernelGGL(reduce_token_major_kernel<true>, dim3((d + 255) / 256, t), dim3(256), 0, s, partials, weights, top_k,
                           d, h2);
    else
        hipLaunchKernelGGL(reduce_token_major_kernel<false>, dim3((d + 255) / 256, t), dim3(256), 0, s, partials, weights, top_k,
                           d, h2);
    return hipGetLastError();
}

}  // namespace ffmoe
