// Prefill routed experts: expert-sorted (token, expert) pairs, then two grouped GEMMs on the matrix
// units whose weight tiles are dequantised INT4 -> bf16 into LDS.
//
// Replaces the host-side pair sort of PrefillMoEGrouping.groupTokenExpertPairs
// (Kernels/Prefill/MoE/PrefillMoEGrouping.swift:49-110), prefill_routed_gate_up_tensorops /
// prefill_routed_down_tensorops (Metal/Prefill/prefill.metal:609-779) and the ANE guest
// (Runtime/Inference/ANERoutedPrefillBackend.swift:348-427, Metal/ANE/ane_prefill.metal).
//
// Sort: a stable counting sort keyed by expert. Items keep their input order inside an expert, so
// routes taken from the router's [token][rank] table come out in (expert, token, rank) order - the
// order the reference's comparator produces (PrefillMoEGrouping.swift:66-75). Only integer counting uses
// LDS atomics; every position comes from prefix sums, so the result does not depend on timing.
//
// GEMM: one block = one M-tile of up to 128 same-expert pairs x 128 weight rows (4 arena tiles per
// 64-wide group). Per group the block stages the pairs' inputs (bf16) and the four tiles' weights,
// each expanded once to bf16(fma(q, scale, bias)) - the reference's 16-bit tile weight
// (prefill.metal:581-590) - in the register layout v_mfma_f32_16x16x32_bf16 wants, so every wave reads
// its operands with 16-byte LDS loads. fp32 accumulation; GELU-tanh(gate) * up in the epilogue.
// bf16 activations make the reference's power-of-two block scaling (prefill.metal:593-598, an FP16 range
// fix) unnecessary.
#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {
namespace {

constexpr int kSortBlock = 256;
constexpr int kBM = FFMOE_PREFILL_TILE_M;   // pairs per M-tile
constexpr int kTilesPerBlock = 4;           // arena tiles (of 16 + 16 rows) per N-block

// ---------------------------------------------------------------------------------------------------
// Item sources: a router table [t][top_k] (item = route) or an explicit pair list.
// ---------------------------------------------------------------------------------------------------
struct ItemSource {
    const uint32_t *idx;       // router table: expert per route, or nullptr
    const uint16_t *w;         // router table: weight bits per route
    const ffmoe_pair *pairs;   // explicit pairs, or nullptr
    uint32_t n_items;
    uint32_t top_k;
    uint32_t n_experts;
    uint32_t t;
};

__device__ __forceinline__ uint32_t item_expert(const ItemSource &src, uint32_t i) {
    if (i >= src.n_items) return 0xFFFFFFFFu;
    if (src.pairs) {
        const ffmoe_pair p = src.pairs[i];
        return (p.expert < src.n_experts && p.token < src.t && p.rank < src.top_k) ? p.expert : 0xFFFFFFFFu;
    }
    const uint32_t e = src.idx[i];
    // zero-weight routes are dropped, as the reference's prefill does (RealForwardRunner.swift:1528-1530)
    return ((src.w[i] & 0x7FFFu) != 0 && e < src.n_experts) ? e : 0xFFFFFFFFu;
}

__global__ __launch_bounds__(kSortBlock) void prefill_hist_kernel(ItemSource src, uint32_t *__restrict__ block_cnt) {
    __shared__ uint32_t cnt[FFMOE_MAX_EXPERTS];
    cnt[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t e = item_expert(src, blockIdx.x * kSortBlock + threadIdx.x);
    if (e != 0xFFFFFFFFu) atomicAdd(&cnt[e], 1u);
    __syncthreads();
    if (threadIdx.x < src.n_experts) block_cnt[(size_t)blockIdx.x * src.n_experts + threadIdx.x] = cnt[threadIdx.x];
}

// One block: per expert, turn the per-block counts into per-block bases, then lay out the experts one
// after the other and cut each into M-tiles.
__global__ __launch_bounds__(256) void prefill_scan_kernel(uint32_t n_blocks, uint32_t n_experts,
                                                           uint32_t *__restrict__ block_cnt, PrefillPlan *__restrict__ plan,
                                                           PrefillTile *__restrict__ tiles, uint32_t max_tiles) {
    __shared__ uint32_t total[FFMOE_MAX_EXPERTS];
    __shared__ uint32_t offset[FFMOE_MAX_EXPERTS + 1];
    __shared__ uint32_t tile_off[FFMOE_MAX_EXPERTS + 1];
    const uint32_t e = threadIdx.x;
    uint32_t sum = 0;
    if (e < n_experts) {
#pragma unroll 16
        for (uint32_t b = 0; b < n_blocks; ++b) sum += block_cnt[(size_t)b * n_experts + e];
    }
    total[e] = e < n_experts ? sum : 0;
    __syncthreads();
    if (e == 0) {
        uint32_t run = 0, trun = 0;
        for (uint32_t i = 0; i < n_experts; ++i) {
            offset[i] = run;
            tile_off[i] = trun;
            run += total[i];
            trun += (total[i] + kBM - 1) / kBM;
        }
        offset[n_experts] = run;
        tile_off[n_experts] = trun;
        plan->n_pairs = run;
        plan->n_tiles = min(trun, max_tiles);
    }
    __syncthreads();
    if (e < n_experts) {
        uint32_t run = offset[e];
        plan->expert_offset[e] = run;
        plan->expert_count[e] = total[e];
        for (uint32_t b0 = 0; b0 < n_blocks; b0 += 16) {
            uint32_t c[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) c[u] = b0 + u < n_blocks ? block_cnt[(size_t)(b0 + u) * n_experts + e] : 0;
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                if (b0 + u < n_blocks) block_cnt[(size_t)(b0 + u) * n_experts + e] = run;      // count -> base, in place
                run += c[u];
            }
        }
        const uint32_t nt = (total[e] + kBM - 1) / kBM;
        for (uint32_t i = 0; i < nt; ++i) {
            const uint32_t ti = tile_off[e] + i;
            if (ti < max_tiles) {
                PrefillTile tl;
                tl.expert = e;
                tl.row_start = offset[e] + i * kBM;
                tl.rows = min((uint32_t)kBM, total[e] - i * kBM);
                tl.pad = 0;
                tiles[ti] = tl;
            }
        }
    }
    if (e == 0) plan->expert_offset[n_experts] = offset[n_experts];
}

__global__ __launch_bounds__(kSortBlock) void prefill_scatter_kernel(ItemSource src, const uint32_t *__restrict__ block_base,
                                                                     uint32_t *__restrict__ sorted_token,
                                                                     uint32_t *__restrict__ sorted_out_row) {
    __shared__ uint32_t ex[kSortBlock];
    const uint32_t i = blockIdx.x * kSortBlock + threadIdx.x;
    const uint32_t e = item_expert(src, i);
    ex[threadIdx.x] = e;
    __syncthreads();
    if (e == 0xFFFFFFFFu) return;
    uint32_t rank = 0;
    for (uint32_t j = 0; j < threadIdx.x; ++j) rank += ex[j] == e ? 1u : 0u;
    const uint32_t pos = block_base[(size_t)blockIdx.x * src.n_experts + e] + rank;
    uint32_t token, out_row;
    if (src.pairs) {
        const ffmoe_pair p = src.pairs[i];
        token = p.token;
        out_row = p.token * src.top_k + p.rank;
    } else {
        token = i / src.top_k;
        out_row = i;
    }
    sorted_token[pos] = token;
    sorted_out_row[pos] = out_row;
}

// ---------------------------------------------------------------------------------------------------
// Grouped GEMM. grid = (N-blocks, tile capacity); block = 4 waves. Wave w expands arena tile w of the
// N-block per group and owns pairs [32 w, 32 w + 32) of the M-tile against all 128 weight rows.
// GATE_UP: A rows are gathered token rows of x; streams are gate / up; out = acts[pair][F].
// else:    A rows are acts[pair][F]; streams are two 16-row blocks; out = partials[out_row][D] (bf16).
// ---------------------------------------------------------------------------------------------------
template <bool GATE_UP>
__global__ __launch_bounds__(256) void prefill_gemm_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                           const PrefillPlan *__restrict__ plan,
                                                           const PrefillTile *__restrict__ tiles,
                                                           const uint32_t *__restrict__ sorted_token,
                                                           const uint32_t *__restrict__ sorted_out_row,
                                                           const uint16_t *__restrict__ a, uint32_t a_stride,
                                                           uint16_t *__restrict__ out) {
    constexpr uint32_t kRowElems = kGroup + 8;      // +16 B per row: 16-row fragments spread over the banks
    __shared__ __align__(16) uint16_t xs[kBM][kRowElems];
    __shared__ __align__(16) uint4 wb[kTilesPerBlock][2][2][kWave];   // [tile][stream][k-half][lane]
    __shared__ uint32_t s_src[kBM];

    if (blockIdx.y >= plan->n_tiles) return;
    const PrefillTile tile = tiles[blockIdx.y];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint32_t n_groups = GATE_UP ? g.gd : g.gf;
    const uint32_t n_arena_tiles = GATE_UP ? g.gu_rb : g.dn_rbp;
    const uint32_t at = blockIdx.x * kTilesPerBlock + wave;            // this wave's arena tile row
    const bool at_ok = at < n_arena_tiles;
    const uint8_t *expert_base = arena_layer + (size_t)tile.expert * g.expert_bytes;
    const uint8_t *w_tiles = expert_base + (GATE_UP ? g.gu_tiles_off : g.dn_tiles_off) + (size_t)at * n_groups * kTileBytes;
    const uint8_t *w_scales = expert_base + (GATE_UP ? g.gu_scales_off : g.dn_scales_off) + (size_t)at * n_groups * kTileScaleBytes;

    // source row of every pair of the tile: a token row of x, or the pair's own activation row
    if (tid < (uint32_t)kBM) {
        const uint32_t row = tile.row_start + min(tid, tile.rows - 1);
        s_src[tid] = GATE_UP ? sorted_token[row] : row;
    }
    __syncthreads();

    f32x4 acc[2][2 * kTilesPerBlock];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nf = 0; nf < 2 * kTilesPerBlock; ++nf) acc[mb][nf] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (uint32_t grp = 0; grp < n_groups; ++grp) {
        // A: 128 rows x 64 k = 1024 16-byte chunks, four per thread
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t i = tid + 256 * c, row = i >> 3, ch = i & 7;
            const uint4 v = *reinterpret_cast<const uint4 *>(a + (size_t)s_src[row] * a_stride + grp * kGroup + ch * 8);
            *reinterpret_cast<uint4 *>(&xs[row][ch * 8]) = v;
        }
        // B: one arena tile per wave, expanded to bf16 in MFMA operand order
        uint4 wt = {0, 0, 0, 0};
        uint2 sc = {0, 0};
        if (at_ok) {
            wt = reinterpret_cast<const uint4 *>(w_tiles + (size_t)grp * kTileBytes)[lane];
            sc = reinterpret_cast<const uint2 *>(w_scales + (size_t)grp * kTileScaleBytes)[j];
        }
        wb[wave][0][0][lane] = dequant8_bf16(wt.x, bf16lo_to_f32(sc.x), bf16hi_to_f32(sc.x));
        wb[wave][0][1][lane] = dequant8_bf16(wt.y, bf16lo_to_f32(sc.x), bf16hi_to_f32(sc.x));
        wb[wave][1][0][lane] = dequant8_bf16(wt.z, bf16lo_to_f32(sc.y), bf16hi_to_f32(sc.y));
        wb[wave][1][1][lane] = dequant8_bf16(wt.w, bf16lo_to_f32(sc.y), bf16hi_to_f32(sc.y));
        __syncthreads();
        bf16x8 af[2][2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                af[mb][h] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(&xs[32 * wave + 16 * mb + j][32 * h + 8 * jq]));
#pragma unroll
        for (int nf = 0; nf < 2 * kTilesPerBlock; ++nf) {
            const bf16x8 b0 = __builtin_bit_cast(bf16x8, wb[nf >> 1][nf & 1][0][lane]);
            const bf16x8 b1 = __builtin_bit_cast(bf16x8, wb[nf >> 1][nf & 1][1][lane]);
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                acc[mb][nf] = mfma16(af[mb][0], b0, acc[mb][nf]);
                acc[mb][nf] = mfma16(af[mb][1], b1, acc[mb][nf]);
            }
        }
        __syncthreads();
    }

    // epilogue: lane holds pairs 32 w + 16 mb + 4 jq + r, weight row j of every fragment
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t prow = 32 * wave + 16 * mb + 4 * jq + r;
            if (prow >= tile.rows) continue;
            const uint32_t pair = tile.row_start + prow;
#pragma unroll
            for (int tl = 0; tl < kTilesPerBlock; ++tl) {
                const uint32_t atl = blockIdx.x * kTilesPerBlock + tl;
                if (atl >= n_arena_tiles) continue;
                if (GATE_UP) {
                    const uint32_t f = atl * kTileRows + j;
                    out[(size_t)pair * g.f + f] = f32_to_bf16(gelu_tanh(acc[mb][2 * tl][r]) * acc[mb][2 * tl + 1][r]);
                } else {
                    const size_t base = (size_t)sorted_out_row[pair] * g.d + (size_t)atl * 2 * kTileRows + j;
                    out[base] = f32_to_bf16(acc[mb][2 * tl][r]);
                    out[base + kTileRows] = f32_to_bf16(acc[mb][2 * tl + 1][r]);
                }
            }
        }
    }
}

// h2[t][c] = bf16(sum_r w[t][r] * partial[t][r][c]) over the routes the sort kept, fma in rank order
// (prefill.metal:544-565); dropped routes (zero weight, expert out of range) add nothing, which equals
// the reference's zero-filled partial rows without having to clear 138 MB first.
__global__ __launch_bounds__(256) void prefill_combine_kernel(const uint16_t *__restrict__ partials,
                                                              const uint16_t *__restrict__ w,
                                                              const uint32_t *__restrict__ idx, uint32_t n_experts,
                                                              uint32_t top_k, uint32_t d, uint16_t *__restrict__ y) {
    const uint32_t tok = blockIdx.y;
    const uint32_t c = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (c >= d) return;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (uint32_t r = 0; r < top_k; ++r) {
        const uint32_t route = tok * top_k + r;
        const uint16_t wbits = w[route];
        if ((wbits & 0x7FFFu) == 0 || idx[route] >= n_experts) continue;
        const float wv = bf16_to_f32(wbits);
        const uint4 p = *reinterpret_cast<const uint4 *>(partials + (size_t)route * d + c);
        const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = __builtin_fmaf(wv, bf16lo_to_f32(pw[i]), acc[2 * i]);
            acc[2 * i + 1] = __builtin_fmaf(wv, bf16hi_to_f32(pw[i]), acc[2 * i + 1]);
        }
    }
    uint4 o;
    o.x = pack_bf16x2(acc[0], acc[1]);
    o.y = pack_bf16x2(acc[2], acc[3]);
    o.z = pack_bf16x2(acc[4], acc[5]);
    o.w = pack_bf16x2(acc[6], acc[7]);
    *reinterpret_cast<uint4 *>(y + (size_t)tok * d + c) = o;
}

}  // namespace

hipError_t launch_prefill(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts, uint32_t top_k,
                          const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx, const uint16_t *w,
                          const ffmoe_pair *pairs, uint32_t n_pairs_in, uint16_t *y, uint16_t *partials_out,
                          PrefillScratch sc, KernelTimer *timer) {
    timer->begin(s);
    ItemSource src{};
    src.idx = pairs ? nullptr : idx;
    src.w = pairs ? nullptr : w;
    src.pairs = pairs;
    src.n_items = pairs ? n_pairs_in : t * top_k;
    src.top_k = top_k;
    src.n_experts = n_experts;
    src.t = t;
    if (src.n_items == 0) return hipSuccess;
    const uint32_t n_blocks = (src.n_items + kSortBlock - 1) / kSortBlock;
    hipLaunchKernelGGL(prefill_hist_kernel, dim3(n_blocks), dim3(kSortBlock), 0, s, src, sc.block_cnt);
    hipLaunchKernelGGL(prefill_scan_kernel, dim3(1), dim3(256), 0, s, n_blocks, n_experts, sc.block_cnt, sc.plan, sc.tiles,
                       sc.max_tiles);
    hipLaunchKernelGGL(prefill_scatter_kernel, dim3(n_blocks), dim3(kSortBlock), 0, s, src, sc.block_cnt, sc.sorted_token,
                       sc.sorted_out_row);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_PREFILL_SORT);
    const uint32_t tile_cap = min(sc.max_tiles, (src.n_items + kBM - 1) / kBM + n_experts);
    hipLaunchKernelGGL(prefill_gemm_kernel<true>, dim3((g.gu_rb + kTilesPerBlock - 1) / kTilesPerBlock, tile_cap), dim3(256),
                       0, s, arena_layer, g, sc.plan, sc.tiles, sc.sorted_token, sc.sorted_out_row, x, x_stride, sc.acts);
    timer->mark(s, FFMOE_K_PREFILL_GATE_UP);
    uint16_t *partials = partials_out ? partials_out : sc.partials;
    hipLaunchKernelGGL(prefill_gemm_kernel<false>, dim3((g.dn_rbp + kTilesPerBlock - 1) / kTilesPerBlock, tile_cap),
                       dim3(256), 0, s, arena_layer, g, sc.plan, sc.tiles, sc.sorted_token, sc.sorted_out_row, sc.acts, g.f,
                       partials);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_PREFILL_DOWN);
    if (y) {
        hipLaunchKernelGGL(prefill_combine_kernel, dim3((g.d / 8 + 255) / 256, t), dim3(256), 0, s, partials, w, idx,
                           n_experts, top_k, g.d, y);
        timer->mark(s, FFMOE_K_PREFILL_COMBINE);
    }
    timer->finish();
    return hipGetLastError();
}

}  // namespace ffmoe
