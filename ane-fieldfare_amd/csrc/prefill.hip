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
// GEMM: one block = one M-tile of up to 256 same-expert pairs x 128 weight rows (4 arena tiles per
// 64-wide group). Per group the four tiles' weights are expanded once to bf16(fma(q, scale, bias)) - the
// reference's 16-bit tile weight (prefill.metal:581-590) - into LDS in the register layout
// v_mfma_f32_16x16x32_bf16 wants; the pairs' inputs go from global memory straight into that layout.
// fp32 accumulation; GELU-tanh(gate) * up in the epilogue.
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

// One block of 1024 threads: per expert, turn the per-block counts into per-block bases, then lay out the
// experts one after the other and cut each into M-tiles. Thread (expert e, chunk c) owns a contiguous run
// of sort blocks, so the counts of a whole column are in flight at once and - up to kScanKeep per thread -
// stay in registers between the summing pass and the pass that writes the bases.
constexpr int kScanThreads = 1024;
constexpr int kScanKeep = 16;

__global__ __launch_bounds__(kScanThreads) void prefill_scan_kernel(uint32_t n_blocks, uint32_t n_experts, uint32_t e_pad,
                                                                    uint32_t *__restrict__ block_cnt,
                                                                    PrefillPlan *__restrict__ plan,
                                                                    PrefillTile *__restrict__ tiles, uint32_t max_tiles) {
    __shared__ uint32_t total[FFMOE_MAX_EXPERTS];
    __shared__ uint32_t offset[FFMOE_MAX_EXPERTS + 1];
    __shared__ uint32_t tile_off[FFMOE_MAX_EXPERTS + 1];
    __shared__ uint32_t part[kScanThreads];                 // [chunk][e_pad]: chunk sums, then chunk bases
    __shared__ unsigned long long scan_own[FFMOE_MAX_EXPERTS], wave_sum[FFMOE_MAX_EXPERTS / 64];
    __shared__ uint32_t shorter[3][FFMOE_MAX_EXPERTS];      // per expert: shorter tiles in all, in front of it, ranked above its own
    const uint32_t e = threadIdx.x % e_pad, ch = threadIdx.x / e_pad, chunks = kScanThreads / e_pad;
    const uint32_t per = (n_blocks + chunks - 1) / chunks;
    const uint32_t b_lo = min(n_blocks, ch * per), b_hi = min(n_blocks, b_lo + per);
    const bool live = e < n_experts;
    uint32_t keep[kScanKeep];
    uint32_t sum = 0;
#pragma unroll
    for (int u = 0; u < kScanKeep; ++u) {
        keep[u] = live && b_lo + u < b_hi ? block_cnt[(size_t)(b_lo + u) * n_experts + e] : 0;
        sum += keep[u];
    }
    if (live)
        for (uint32_t b = b_lo + kScanKeep; b < b_hi; ++b) sum += block_cnt[(size_t)b * n_experts + e];
    part[threadIdx.x] = sum;
    if (threadIdx.x < FFMOE_MAX_EXPERTS) {
        total[threadIdx.x] = 0;
        shorter[0][threadIdx.x] = shorter[1][threadIdx.x] = shorter[2][threadIdx.x] = 0;
    }
    __syncthreads();
    if (ch == 0 && live) {
        uint32_t run = 0;
        for (uint32_t c = 0; c < chunks; ++c) {
            const uint32_t v = part[c * e_pad + e];
            part[c * e_pad + e] = run;
            run += v;
        }
        total[e] = run;
    }
    __syncthreads();
    // exclusive prefix sums over the experts of (pairs, tiles), packed into one 64-bit value: four waves scan 64
    // experts each, then add the waves in front of them
    if (threadIdx.x < FFMOE_MAX_EXPERTS) {
        const uint32_t i = threadIdx.x, lane = i & 63, wv = i >> 6;
        const uint32_t n = i < n_experts ? total[i] : 0;
        const unsigned long long own = ((unsigned long long)((n + kBM - 1) / kBM) << 32) | n;
        unsigned long long inc = own;
#pragma unroll
        for (int sh = 1; sh < 64; sh <<= 1) {
            const unsigned long long up = __shfl_up(inc, sh, 64);
            if (lane >= (uint32_t)sh) inc += up;
        }
        if (lane == 63) wave_sum[wv] = inc;
        scan_own[i] = inc - own;
    }
    __syncthreads();
    if (threadIdx.x < FFMOE_MAX_EXPERTS) {
        const uint32_t i = threadIdx.x, wv = i >> 6;
        unsigned long long base = 0;
        for (uint32_t v = 0; v < wv; ++v) base += wave_sum[v];
        const unsigned long long ex = base + scan_own[i];
        if (i <= n_experts) {
            offset[i] = (uint32_t)ex;
            tile_off[i] = (uint32_t)(ex >> 32);
        }
        if (i == n_experts || (i == FFMOE_MAX_EXPERTS - 1 && n_experts == FFMOE_MAX_EXPERTS)) {
            // the totals: the prefix in front of the first expert past the end (or, with every slot in use, the last
            // expert's prefix plus its own share)
            unsigned long long all = ex;
            if (i != n_experts) {
                const uint32_t n = total[i];
                all += ((unsigned long long)((n + kBM - 1) / kBM) << 32) | n;
                offset[n_experts] = (uint32_t)all;
                tile_off[n_experts] = (uint32_t)(all >> 32);
            }
            plan->n_pairs = (uint32_t)all;
            plan->n_tiles = min((uint32_t)(all >> 32), max_tiles);
            plan->expert_offset[n_experts] = (uint32_t)all;
        }
    }
    __syncthreads();
    // The tile list runs from the largest tile down: the full tiles in expert order, then every expert's last, shorter
    // tile by its rows (ties in expert order). The GEMM grids walk the list eight tiles at a time, so the launches end
    // with their shortest blocks instead of with whatever the last experts hold (a Zipf chunk's heavy experts sit
    // anywhere in the expert order). Where an expert's shorter tile goes takes a look at every other expert's: the
    // threads of an expert share that out (one thread alone is a chain of two thousand instructions).
    if (live) {
        const uint32_t rest = total[e] % kBM, per_o = (e_pad + chunks - 1) / chunks;
        const uint32_t o_lo = min(e_pad, ch * per_o), o_hi = min(e_pad, o_lo + per_o);
        uint32_t all = 0, in_front = 0, above = 0;
        for (uint32_t o = o_lo; o < o_hi; ++o) {
            const uint32_t r = total[o] % kBM;          // experts past n_experts hold zero
            const uint32_t has = r != 0 ? 1u : 0u;
            all += has;
            in_front += has & (o < e ? 1u : 0u);
            above += has & ((r > rest || (r == rest && o < e)) ? 1u : 0u);
        }
        if (all) {
            atomicAdd(&shorter[0][e], all);
            atomicAdd(&shorter[1][e], in_front);
            atomicAdd(&shorter[2][e], above);
        }
    }
    __syncthreads();
    if (!live) return;
    uint32_t run = offset[e] + part[threadIdx.x];
#pragma unroll
    for (int u = 0; u < kScanKeep; ++u) {
        if (b_lo + u < b_hi) block_cnt[(size_t)(b_lo + u) * n_experts + e] = run;      // count -> base, in place
        run += keep[u];
    }
    for (uint32_t b = b_lo + kScanKeep; b < b_hi; ++b) {
        const uint32_t c = block_cnt[(size_t)b * n_experts + e];
        block_cnt[(size_t)b * n_experts + e] = run;
        run += c;
    }
    if (ch != 0) return;
    plan->expert_offset[e] = offset[e];
    plan->expert_count[e] = total[e];
    // a tile keeps its number in row order, which places its activation blocks
    const uint32_t nt = (total[e] + kBM - 1) / kBM, n_full = total[e] / kBM;
    const uint32_t shorter_tiles = shorter[0][e], shorter_in_front = shorter[1][e], ranked_above = shorter[2][e];
    const uint32_t full_in_front = tile_off[e] - shorter_in_front, full_tiles = tile_off[n_experts] - shorter_tiles;
    for (uint32_t i = 0; i < nt; ++i) {
        const uint32_t ti = i < n_full ? full_in_front + i : full_tiles + ranked_above;
        if (ti < max_tiles) {
            PrefillTile tl;
            tl.expert = e;
            tl.row_start = offset[e] + i * kBM;
            tl.rows = min((uint32_t)kBM, total[e] - i * kBM);
            tl.order = tile_off[e] + i;
            tiles[ti] = tl;
        }
    }
}

__global__ __launch_bounds__(kSortBlock) void prefill_scatter_kernel(ItemSource src, const uint32_t *__restrict__ block_base,
                                                                     uint32_t *__restrict__ sorted_token,
                                                                     uint32_t *__restrict__ sorted_out_row) {
    // an item's place inside its block's share of its expert = the items of the same expert in front of it: those in
    // the waves in front (per-wave counts in LDS) plus those in lower lanes of its own wave (a mask built from one
    // ballot per bit of the expert number)
    __shared__ uint32_t wave_cnt[kSortBlock / 64][FFMOE_MAX_EXPERTS];
    static_assert(FFMOE_MAX_EXPERTS <= 256, "eight ballots tell the experts apart");
    const uint32_t i = blockIdx.x * kSortBlock + threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (uint32_t c = threadIdx.x; c < (kSortBlock / 64) * FFMOE_MAX_EXPERTS; c += kSortBlock) (&wave_cnt[0][0])[c] = 0;
    const uint32_t e = item_expert(src, i);
    const bool valid = e != 0xFFFFFFFFu;
    unsigned long long same = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const bool bit = (e >> b) & 1u;
        const unsigned long long with = __ballot(bit);
        same &= bit ? with : ~with;
    }
    const uint32_t in_front = __popcll(same & ((1ull << lane) - 1ull));
    __syncthreads();
    if (valid && in_front == 0) wave_cnt[wave][e] = __popcll(same);
    __syncthreads();
    if (!valid) return;
    uint32_t rank = in_front;
    for (uint32_t v = 0; v < wave; ++v) rank += wave_cnt[v][e];
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

// A dense FFN's chunk needs no sort: one expert, route r = row r. One launch writes what the three above would: the
// identity tables and the chunk cut into M-tiles.
__global__ __launch_bounds__(kSortBlock) void prefill_dense_plan_kernel(uint32_t t, PrefillPlan *__restrict__ plan,
                                                                       PrefillTile *__restrict__ tiles,
                                                                       uint32_t *__restrict__ sorted_token,
                                                                       uint32_t *__restrict__ sorted_out_row) {
    const uint32_t i = blockIdx.x * kSortBlock + threadIdx.x;
    if (i < t) {
        sorted_token[i] = i;
        sorted_out_row[i] = i;
    }
    const uint32_t n_tiles = (t + kBM - 1) / kBM;
    if (i < n_tiles) {
        PrefillTile tl;
        tl.expert = 0;
        tl.row_start = i * kBM;
        tl.rows = min((uint32_t)kBM, t - i * kBM);
        tl.order = i;
        tiles[i] = tl;
    }
    if (i == 0) {
        plan->n_pairs = t;
        plan->n_tiles = n_tiles;
        plan->expert_count[0] = t;
        plan->expert_offset[0] = 0;
        plan->expert_offset[1] = t;
    }
}

// ---------------------------------------------------------------------------------------------------
// Grouped GEMM. One block = one M-tile (up to 256 pairs of one expert) x one N-block (4 arena tiles =
// 128 weight rows); block ids are laid out so that all N-blocks of an M-tile run on one XCD and find the
// tile's A rows in that XCD's L2. The M-tile's 16-row blocks are dealt round-robin to the four waves
// (wave w owns blocks w, w + 4, ...), so a short tile still loads all four matrix units evenly.
//   A: every lane loads its own MFMA fragments straight from global memory (16 B per fragment), one
//      64-wide group ahead, into registers - the rows are private to the wave, LDS would add nothing.
//   B: wave w expands arena tile w of the next group to bf16(fma(q, scale, bias)) into the other half of
//      a double-buffered LDS area while all waves multiply from the current half; one barrier per group.
// GATE_UP: A rows are gathered token rows of x; streams are gate / up; out = the activations, stored in the order the
//          down GEMM's matrix instructions want them (below).
// else:    A = those activations, loaded straight into operand registers (1 KiB contiguous per wave and fragment, no
//          cross-lane re-layout); streams are two 16-row blocks; out = partials[out_row][D] (16-bit).
// Activation layout: [16-pair block][group of F][k-half][lane (j, jq)] x 8 values = pair j of the block at
// k = 32 * (k-half) + 8 * jq .. + 7 of the group. The 16-pair blocks of an M-tile start at block row_start / 16 + its number
// in row order: consecutive tiles never share a block (a tile adds at most one block of slack), so the buffer holds
// max_pairs / 16 + max_tiles + 1 blocks.
// ---------------------------------------------------------------------------------------------------

struct GemmWave {
    const uint8_t *w_tiles, *w_scales;    // this wave's arena tile row
    const uint16_t *a;                    // A matrix
    uint32_t a_stride, n_groups, n_arena_tiles, nb, wave, lane;
    uint32_t act_blocks;                  // 16-pair blocks the activation buffer holds (the scale tables' extent)
    uint32_t act_block0;                  // first 16-pair block of this M-tile in the activation layout
    PrefillTile tile;
};

// The k-loop and epilogue of one wave that owns NMB 16-row blocks (a compile-time count: the MFMA
// sequence has no branches, so the scheduler can interleave it with the expansion of the next tile).
// DUMP: a test instantiation that also copies every weight fragment out of LDS, read exactly as the matrix
// instructions read it, so that a test can hold the expanded tile itself against the reference's 16-bit weight.
// F16: the reference's FP16 prefill (prefill.metal:581-598,685-702,723-777): FP16 rows against FP16 tile weights
// half(fma(q, scale, bias)), fp32 sums; the activations between the two GEMMs are FP16 with a power-of-two scale per
// pair and 64-wide block of F (`act_scale[pair][block]`; the block's largest magnitude lands below 2^14), so values
// past FP16's range keep FP16's relative precision; the down GEMM brings every block of a pair to the pair's largest
// scale as it takes it in (exact unless a value falls below FP16's normal range relative to that largest) and
// applies that scale to the pair's sums.
template <bool GATE_UP, int NMB, bool F16, bool DUMP = false>
__device__ __forceinline__ void gemm_wave(const GemmWave &gw, const ArenaGeom &g, uint4 (*wb)[kTilesPerBlock][2][2][kWave],
                                          const uint32_t *__restrict__ sorted_token,
                                          const uint32_t *__restrict__ sorted_out_row, uint16_t *__restrict__ out,
                                          float *__restrict__ act_scale, uint4 *__restrict__ dump = nullptr) {
    constexpr int NA = NMB > 0 ? NMB : 1;
    const uint32_t lane = gw.lane, wave = gw.wave, j = lane & 15, jq = lane >> 4;
    const uint32_t n_groups = gw.n_groups;
    const uint16_t *arow[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        if (!GATE_UP) {
            // the activations are stored fragment by fragment: block, group, k-half, then 16 bytes per lane
            arow[i] = gw.a + ((size_t)(gw.act_block0 + wave + 4 * i) * n_groups * 2) * (kWave * 8) + lane * 8;
            continue;
        }
        // load layout: four neighbouring lanes read 64 contiguous bytes of one row (row lane / 4, 8-element
        // chunk lane % 4), so a load touches 16 half-lines instead of 64 scattered 16-byte pieces
        const uint32_t prow = min((wave + 4 * i) * 16 + (lane >> 2), gw.tile.rows - 1);
        const uint32_t src = sorted_token[gw.tile.row_start + prow];
        // rows 8..15 take their four chunks rotated by two: the lanes a half-wave then pulls from in the re-layout
        // below fall on 32 different LDS banks (in natural order rows r and r + 8 collide on every bank)
        arow[i] = gw.a + (size_t)src * gw.a_stride + 8 * (((lane & 3) - 2 * (lane >> 5)) & 3);
    }
    // MFMA layout: lane (j, jq) needs row j, chunk jq = what load-layout lane 4 j + ((jq + 2 (j / 8)) % 4) holds
    const int pull = (int)((4 * j + ((jq + 2 * (j >> 3)) & 3)) * 4);
    // FP16 down GEMM: the pair a lane holds in row block i (operand lane (j, jq) = pair j of the block), its largest
    // block scale and the reciprocal (powers of two: exact)
    // FP16: the block scales are laid out like the activations - act_scale[(16-pair block * groups of F + group) * 16 + j],
    // pair j of the block - so a lane's address is a wave-uniform base plus 4 j. The down GEMM finds them already
    // divided by the pair's largest (prefill_pair_scale_kernel ran in between: powers of two <= 1), and the largest
    // itself in a second table behind the first, [block * 16 + j].
    auto scale_at = [&](int i, uint32_t grp) { return ((size_t)(gw.act_block0 + wave + 4 * i) * g.gf + grp) * 16 + j; };
    auto to_frag = [&](const uint4 &v, float rel) {
        if (!GATE_UP) {                                           // already in operand order
            if constexpr (!F16) return v;
            const _Float16 r = (_Float16)rel;
            const f16x2 r2 = {r, r};
            uint4 o;
            o.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, v.x) * r2);
            o.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, v.y) * r2);
            o.z = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, v.z) * r2);
            o.w = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, v.w) * r2);
            return o;
        }
        uint4 r;
        r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.x);
        r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.y);
        r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.z);
        r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(pull, (int)v.w);
        return r;
    };
    f32x4 acc[NA][2 * kTilesPerBlock];
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int nf = 0; nf < 2 * kTilesPerBlock; ++nf) acc[i][nf] = f32x4{0.f, 0.f, 0.f, 0.f};

    // this wave's packed tile of the next kSlots groups to expand, in flight: group g waits in slot g % kSlots
    // (one slot where the row blocks leave no registers for a second: the steps are long enough there)
    constexpr int kSlots = ((GATE_UP || F16) && NMB >= 4) ? 1 : 2;      // (the FP16 down GEMM carries the pairs' block scales besides)
    uint4 wraw[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    uint2 sraw[2] = {{0, 0}, {0, 0}};
    auto load_b = [&](uint32_t grp, int slot) {
        wraw[slot] = reinterpret_cast<const uint4 *>(gw.w_tiles + (size_t)grp * kTileBytes)[lane];
        sraw[slot] = reinterpret_cast<const uint2 *>(gw.w_scales + (size_t)grp * kTileScaleBytes)[j];
    };
    // Expansion of the packed tile in `wcur` into wb[buf], cut into 16 pieces of about five VALU
    // instructions (piece 4 c + q = output dword q of packed word c; the word's last piece stores it).
    uint32_t wcur[4];
    float sc[2], bi[2];
    uint32_t lo = 0, hi = 0;
    uint4 ex = {0, 0, 0, 0};
    auto expand_begin = [&](int slot) {
        wcur[0] = wraw[slot].x, wcur[1] = wraw[slot].y, wcur[2] = wraw[slot].z, wcur[3] = wraw[slot].w;
        sc[0] = bf16lo_to_f32(sraw[slot].x), bi[0] = bf16hi_to_f32(sraw[slot].x);
        sc[1] = bf16lo_to_f32(sraw[slot].y), bi[1] = bf16hi_to_f32(sraw[slot].y);
    };
    auto expand_piece = [&](int buf, int piece) {
        const int c = piece >> 2, q = piece & 3;
        const float s_ = sc[c >> 1], b_ = bi[c >> 1];
        if (q == 0) {
            // even / odd nibbles as bytes; the empty asm keeps the masks as written (one v_cvt_f32_ubyteN per byte)
            lo = wcur[c] & 0x0F0F0F0Fu, hi = (wcur[c] >> 4) & 0x0F0F0F0Fu;
            asm("" : "+v"(lo), "+v"(hi));
            ex.x = Act<F16>::pack(__builtin_fmaf((float)(lo & 0xFFu), s_, b_), __builtin_fmaf((float)((lo >> 16) & 0xFFu), s_, b_));
        } else if (q == 1) {
            ex.y = Act<F16>::pack(__builtin_fmaf((float)(hi & 0xFFu), s_, b_), __builtin_fmaf((float)((hi >> 16) & 0xFFu), s_, b_));
        } else if (q == 2) {
            ex.z = Act<F16>::pack(__builtin_fmaf((float)((lo >> 8) & 0xFFu), s_, b_), __builtin_fmaf((float)(lo >> 24), s_, b_));
        } else {
            ex.w = Act<F16>::pack(__builtin_fmaf((float)((hi >> 8) & 0xFFu), s_, b_), __builtin_fmaf((float)(hi >> 24), s_, b_));
            wb[buf][wave][c >> 1][c & 1][lane] = ex;
        }
    };
    uint4 araw[NA][2];      // A in load layout, in flight: [.][0] k-half 0, [.][1] k-half 1
    uint4 af[NA][2];        // A as MFMA fragments
    float ablock[NA][2];    // FP16 down GEMM: the block scale of the group araw[.][half] belongs to
    auto load_a = [&](uint32_t grp, int half) {
        if (NMB == 0) return;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            araw[i][half] = GATE_UP ? *reinterpret_cast<const uint4 *>(arow[i] + grp * kGroup + 32 * half)
                                    : *reinterpret_cast<const uint4 *>(arow[i] + (size_t)(grp * 2 + half) * (kWave * 8));
            if constexpr (F16 && !GATE_UP) ablock[i][half] = act_scale[scale_at(i, grp)];
        }
    };
    auto frag_a = [&](int half) {
        if (NMB == 0) return;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            float rel = 1.0f;
            if constexpr (F16 && !GATE_UP) rel = ablock[i][half];
            af[i][half] = to_frag(araw[i][half], rel);
        }
    };
    // One 64-wide group = 16 units; unit u multiplies weight fragment (nf = u % 8, k-half u / 8) with the NA
    // row blocks, and is followed by one piece of the next group's expansion, so the matrix pipe and the
    // VALU run side by side inside the wave (a scheduling fence after every unit keeps the order as
    // written). On entry: af[.][0] = k-half 0 of this group; araw[.][1] = its k-half 1 in load layout;
    // araw[.][0] = k-half 0 of the next group in flight; wraw/sraw[grp % kSlots] = packed tile of the group after next
    // (it is expanded during this step, and its slot is reloaded at once with the group kSlots further on: with
    // two slots a packed tile has two steps to arrive); wb[buf] = expanded tiles of this group, the next group's are
    // there as well. The k-half 1 fragments are made at the start of the
    // step and the next k-half 0 fragments in its middle, each as soon as the registers they replace have
    // had their last use, with 8 units of MFMAs to cover the cross-lane latency; every register that a
    // conversion frees is reloaded at once for the following group. Loads past the last group run on clamped
    // indices and are never used: with no branch around them the compiler counts the loads in flight exactly.
    // The last two steps are a second instantiation without the expansion (their groups are in LDS already).
    // The expanded tiles sit in four LDS buffers (group g in buffer g % 4) and the expansion runs two groups ahead of the products, so one barrier per PAIR of groups orders both
    // the first read of a buffer behind its last write and its next write behind its last read.
    auto step = [&](uint32_t grp, auto expand_ahead, auto parity) {
        constexpr bool kExpand = decltype(expand_ahead)::value;     // false in the last two steps: nothing is left to expand
        constexpr int kSlot = decltype(parity)::value;              // grp % 2, known at compile time: the slots are registers
        const int buf = grp & 3;
        frag_a(1);
        load_a(min(grp + 1, n_groups - 1), 1);
        if (kExpand) {
            expand_begin(kSlot % kSlots);                           // group grp + 2
            load_b(min(grp + 2 + kSlots, n_groups - 1), kSlot % kSlots);
        }
        uint4 bq[3];
        auto read_b = [&](int u) { bq[u % 3] = wb[buf][(u & 7) >> 1][u & 1][u >> 3][lane]; };
        if (DUMP && wave == 0) {
            // fragment u of group grp of this N-block, as unit u of the loop below receives it
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                read_b(u);
                dump[(((size_t)gw.nb * n_groups + grp) * 16 + u) * kWave + lane] = bq[u % 3];
            }
        }
        if (NMB > 0) {
            read_b(0);
            read_b(1);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (NMB > 0) {
                if (u + 2 < 16) read_b(u + 2);
#pragma unroll
                for (int i = 0; i < NA; ++i)
                    // weights as the first operand: the lane ends up with four consecutive weight rows of
                    // one pair, which the epilogue packs into one 8-byte piece of that pair's output row
                    acc[i][u & 7] = Act<F16>::mfma(bq[u % 3], af[i][u >> 3], acc[i][u & 7]);
            }
            if (kExpand) expand_piece((buf + 2) & 3, u);
            __builtin_amdgcn_sched_barrier(0);
            if (u == 7) {
                frag_a(0);
                load_a(min(grp + 2, n_groups - 1), 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // one barrier per pair of groups: the expansion runs two groups ahead (the tail steps, which use no slot,
        // are one instantiation and look at the group's parity itself)
        if (kExpand && kSlots == 2 ? kSlot != 0 : (grp & 1) != 0) lds_barrier();
    };
    using Ahead = std::integral_constant<bool, true>;
    using Tail = std::integral_constant<bool, false>;
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;

    load_b(0, 0);
    if (kSlots == 2) load_b(min(1u, n_groups - 1), 1);
    load_a(0, 0);
    load_a(0, 1);
    expand_begin(0);
    load_b(min((uint32_t)kSlots, n_groups - 1), 0);
#pragma unroll
    for (int piece = 0; piece < 16; ++piece) expand_piece(0, piece);
    expand_begin(1 % kSlots);
    load_b(min(1u + kSlots, n_groups - 1), 1 % kSlots);
#pragma unroll
    for (int piece = 0; piece < 16; ++piece) expand_piece(1, piece);
    frag_a(0);
    load_a(min(1u, n_groups - 1), 0);
    lds_barrier();
    // steps in pairs (the slot of a group's packed tile and the barrier follow the group's parity); the last two
    // steps multiply only: their groups were expanded two steps earlier
    const uint32_t n_ahead = n_groups > 2 ? n_groups - 2 : 0;
    uint32_t grp = 0;
    if constexpr (kSlots == 2) {
        for (; grp + 2 <= n_ahead; grp += 2) {
            step(grp, Ahead{}, Even{});
            step(grp + 1, Ahead{}, Odd{});
        }
        if (grp < n_ahead) {             // an odd number of groups: one more expanding step
            step(grp, Ahead{}, Even{});
            ++grp;
        }
    } else {
        for (; grp < n_ahead; ++grp) step(grp, Ahead{}, Even{});
    }
    for (; grp < n_groups; ++grp) step(grp, Tail{}, Even{});
    if (n_groups & 1) lds_barrier();     // the last pair was half a pair
    if (NMB == 0) return;

    // epilogue: lane (j, jq) holds pair 16 (w + 4 i) + j, weight rows 4 jq .. 4 jq + 3 of every fragment
    if (GATE_UP) {
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const uint32_t prow = (wave + 4 * i) * 16 + j;
            if (prow >= gw.tile.rows) continue;
            // this N-block is group nb of F (four arena tiles = 64 activations); arena tile tl holds k = 16 tl .. + 15
            // of it, this lane the four values from k = 16 tl + 4 jq: k-half tl / 2, operand lane (j, 2 (tl % 2) + jq / 2),
            // values 4 (jq % 2) .. + 3 of that lane's eight
            uint16_t *oblk = out + ((size_t)(gw.act_block0 + wave + 4 * i) * g.gf + gw.nb) * 2 * (kWave * 8);
            float h[kTilesPerBlock][4];
#pragma unroll
            for (int tl = 0; tl < kTilesPerBlock; ++tl)
#pragma unroll
                for (int r = 0; r < 4; ++r) h[tl][r] = gelu_tanh_fast(acc[i][2 * tl][r]) * acc[i][2 * tl + 1][r];
            if constexpr (F16) {
                // the pair's 64 activations of this block sit in the four lanes (j, 0..3), sixteen each: their
                // largest magnitude peak < 2^e goes to 2^14 (frexp / ldexp as prefill.metal:689-702)
                float peak = 0.0f;
#pragma unroll
                for (int tl = 0; tl < kTilesPerBlock; ++tl)
#pragma unroll
                    for (int r = 0; r < 4; ++r) peak = fmaxf(peak, fabsf(h[tl][r]));
                peak = fmaxf(peak, __shfl_xor(peak, 16, 64));
                peak = fmaxf(peak, __shfl_xor(peak, 32, 64));
                int e = 0;
                (void)frexpf(peak, &e);
                e = max(e, -100);                                   // 2^(14 - e) stays finite for a block of denormal size
                const float to_half = ldexpf(1.0f, 14 - e);
#pragma unroll
                for (int tl = 0; tl < kTilesPerBlock; ++tl)
#pragma unroll
                    for (int r = 0; r < 4; ++r) h[tl][r] *= to_half;
                if (jq == 0) act_scale[scale_at(i, gw.nb)] = ldexpf(1.0f, e - 14);
            }
#pragma unroll
            for (int tl = 0; tl < kTilesPerBlock; ++tl) {
                uint16_t *dst = oblk + (tl >> 1) * (kWave * 8) + (((tl & 1) * 2 + (jq >> 1)) * 16 + j) * 8 + (jq & 1) * 4;
                *reinterpret_cast<uint2 *>(dst) = make_uint2(Act<F16>::pack(h[tl][0], h[tl][1]), Act<F16>::pack(h[tl][2], h[tl][3]));
            }
        }
        return;
    }
    // Down projection: a 16-pair block of this N-block is 16 rows x 256 B. Each wave turns its blocks
    // through a private LDS area (the weight buffers are free: the last step ended with a barrier) so that
    // 16 lanes store one row's 256 contiguous bytes, instead of 8-byte pieces 32 B apart per instruction.
    constexpr uint32_t kStageRow = 2 * kTilesPerBlock * kTileRows * 2 + 16;     // bytes: 128 columns + padding
    static_assert(4 * 16 * kStageRow <= sizeof(uint4) * 4 * kTilesPerBlock * 2 * 2 * kWave, "staging fits the weight buffers");
    uint8_t *stage = reinterpret_cast<uint8_t *>(wb) + wave * 16 * kStageRow;
    const uint32_t rsub = lane >> 4, chunk = lane & 15;                         // read side: row 4 p + rsub, columns 8 chunk ..
    const bool col_ok = gw.nb * kTilesPerBlock + (chunk >> 2) < gw.n_arena_tiles;
    float pair_largest[NA];
    if constexpr (F16) {
#pragma unroll
        for (int i = 0; i < NA; ++i) pair_largest[i] = act_scale[(size_t)gw.act_blocks * g.gf * 16 + (gw.act_block0 + wave + 4 * i) * 16 + j];
    }
    uint32_t orow_idx[NA][4];
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t prow = (wave + 4 * i) * 16 + 4 * p + rsub;
            orow_idx[i][p] = sorted_out_row[gw.tile.row_start + min(prow, gw.tile.rows - 1)];
        }
#pragma unroll
    for (int i = 0; i < NA; ++i) {
#pragma unroll
        for (int nf = 0; nf < 2 * kTilesPerBlock; ++nf) {
            f32x4 v = acc[i][nf];
            if constexpr (F16) {
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] *= pair_largest[i];      // the pair's sums back to their scale
            }
            *reinterpret_cast<uint2 *>(stage + j * kStageRow + nf * 32 + 8 * jq) =
                make_uint2(Act<F16>::pack(v[0], v[1]), Act<F16>::pack(v[2], v[3]));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t row = 4 * p + rsub, prow = (wave + 4 * i) * 16 + row;
            const uint4 v = *reinterpret_cast<const uint4 *>(stage + row * kStageRow + 16 * chunk);
            if (prow < gw.tile.rows && col_ok)
                *reinterpret_cast<uint4 *>(out + (size_t)orow_idx[i][p] * g.d + gw.nb * (2 * kTilesPerBlock * kTileRows) + 8 * chunk) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// F16: a context in FP16 mode - FP16 rows in, FP16 tiles, block-scaled FP16 activations, FP16 per-route rows out
template <bool GATE_UP, bool F16 = false, bool DUMP = false>
__global__ __launch_bounds__(256, 2) void prefill_gemm_kernel(const uint8_t *__restrict__ arena_layer, ArenaGeom g,
                                                              const PrefillPlan *__restrict__ plan,
                                                              const PrefillTile *__restrict__ tiles,
                                                              const uint32_t *__restrict__ sorted_token,
                                                              const uint32_t *__restrict__ sorted_out_row,
                                                              const uint16_t *__restrict__ a, uint32_t a_stride,
                                                              uint16_t *__restrict__ out, uint32_t n_nblocks,
                                                              bool nb_major, float *__restrict__ act_scale, uint32_t act_blocks,
                                                              uint4 *__restrict__ dump = nullptr) {
    __shared__ __align__(16) uint4 wb[4][kTilesPerBlock][2][2][kWave];   // [buffer][tile][stream][k-half][lane]: group g lives in buffer g % 4

    // Consecutive block ids go to consecutive XCDs. Many experts: all N-blocks of an M-tile share an XCD (its L2 holds
    // the tile's A rows). One expert (the dense FFN: few M-tiles, every one against the same weights): all M-tiles of
    // an N-block share an XCD instead, so each XCD reads its eighth of the weights once and every XCD is equally full.
    const uint32_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    uint32_t ti, nb;
    if (nb_major) {
        const uint32_t per_xcd = (n_nblocks + 7) / 8;
        ti = slot / per_xcd;
        nb = (slot % per_xcd) * 8 + xcd;
        if (nb >= n_nblocks) return;
    } else {
        ti = (slot / n_nblocks) * 8 + xcd;
        nb = slot % n_nblocks;
    }
    if (ti >= plan->n_tiles) return;
    GemmWave gw;
    gw.tile = tiles[ti];
    gw.lane = threadIdx.x & 63;
    gw.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // wave-uniform: branches on it stay scalar
    gw.n_groups = GATE_UP ? g.gd : g.gf;
    gw.n_arena_tiles = GATE_UP ? g.gu_rb : g.dn_rbp;
    gw.nb = nb;
    gw.a = a;
    gw.a_stride = a_stride;
    gw.act_block0 = gw.tile.row_start / 16 + gw.tile.order;
    gw.act_blocks = act_blocks;
    // the arena tile row this wave expands; past the last one it expands the last again (never stored)
    const uint32_t at = min(nb * kTilesPerBlock + gw.wave, gw.n_arena_tiles - 1);
    const uint8_t *expert_base = arena_layer + (size_t)gw.tile.expert * g.expert_bytes;
    gw.w_tiles = expert_base + (GATE_UP ? g.gu_tiles_off : g.dn_tiles_off) + (size_t)at * gw.n_groups * kTileBytes;
    gw.w_scales = expert_base + (GATE_UP ? g.gu_scales_off : g.dn_scales_off) + (size_t)at * gw.n_groups * kTileScaleBytes;

    const uint32_t n_mb = (gw.tile.rows + 15) / 16;
    const uint32_t my_mb = n_mb > gw.wave ? (n_mb - gw.wave + 3) / 4 : 0;    // 16-row blocks of this wave
    if (DUMP) {
        // the test launch runs one pair: wave 0 owns its row block, the others only expand their tiles
        if (my_mb) gemm_wave<GATE_UP, 1, F16, true>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale, dump);
        else gemm_wave<GATE_UP, 0, F16, true>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale, dump);
        return;
    }
    switch (my_mb) {
        case 0: gemm_wave<GATE_UP, 0, F16>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale); break;
        case 1: gemm_wave<GATE_UP, 1, F16>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale); break;
        case 2: gemm_wave<GATE_UP, 2, F16>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale); break;
        case 3: gemm_wave<GATE_UP, 3, F16>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale); break;
        default: gemm_wave<GATE_UP, 4, F16>(gw, g, wb, sorted_token, sorted_out_row, out, act_scale); break;
    }
}

// Between the two GEMMs of the FP16 prefill: a pair's block scales divided by its largest (powers of two: exact), the
// largest itself stored behind the table at [n_pairs * blocks + pair] - what prefill_routed_down_tensorops computes per
// threadgroup into `relative` and `pair_scale` (prefill.metal:731-741), done once per pair here.
// One block per M-tile, one thread per pair of it.
__global__ __launch_bounds__(kBM) void prefill_pair_scale_kernel(const PrefillPlan *__restrict__ plan,
                                                                 const PrefillTile *__restrict__ tiles, uint32_t groups,
                                                                 uint32_t act_blocks, float *__restrict__ act_scale) {
    const uint32_t ti = blockIdx.x;
    if (ti >= plan->n_tiles) return;
    const PrefillTile tile = tiles[ti];
    if (threadIdx.x >= tile.rows) return;
    const uint32_t block = tile.row_start / 16 + tile.order + threadIdx.x / 16, j = threadIdx.x % 16;
    float *s = act_scale + (size_t)block * groups * 16 + j;
    float largest = 0.0f;
    for (uint32_t b = 0; b < groups; ++b) largest = fmaxf(largest, s[b * 16]);
    const float inv = 1.0f / largest;          // a scale is 2^(e - 14) with e >= -100: never zero
    for (uint32_t b = 0; b < groups; ++b) s[b * 16] *= inv;
    act_scale[(size_t)act_blocks * groups * 16 + block * 16 + j] = largest;
}

// h2[t][c] = bf16(sum_r w[t][r] * partial[t][r][c]) over the routes the sort kept, fma in rank order
// (prefill.metal:544-565); dropped routes (zero weight, expert out of range) add nothing, which equals
// the reference's zero-filled partial rows without having to clear 138 MB first.
template <bool F16>
__global__ __launch_bounds__(256) void prefill_combine_kernel(const uint16_t *__restrict__ partials,
                                                              const uint16_t *__restrict__ w,
                                                              const uint32_t *__restrict__ idx, uint32_t n_experts,
                                                              uint32_t top_k, uint32_t d, uint32_t t,
                                                              uint16_t *__restrict__ y) {
    // one thread per 16-byte piece of an output row, pieces numbered across rows so that every block is full
    const uint32_t pieces = d / 8, piece = blockIdx.x * 256 + threadIdx.x;
    const uint32_t tok = piece / pieces, c = (piece % pieces) * 8;
    if (tok >= t) return;
    // every load of the thread is requested before the first is used: the routes' weights and experts, then the
    // rows of the live ones (a dropped route's row was never written and is not touched)
    float wv[8];
    bool live[8];
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        const uint32_t route = tok * top_k + min(r, top_k - 1);
        const uint16_t wbits = w[route];
        live[r] = r < top_k && (wbits & 0x7FFFu) != 0 && idx[route] < n_experts;
        wv[r] = Act<F16>::widen(wbits);
    }
    uint4 p[8];
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        const uint32_t route = tok * top_k + min(r, top_k - 1);
        p[r] = live[r] ? *reinterpret_cast<const uint4 *>(partials + (size_t)route * d + c) : uint4{0, 0, 0, 0};
    }
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        if (live[r]) {
            const uint32_t pw[4] = {p[r].x, p[r].y, p[r].z, p[r].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] = __builtin_fmaf(wv[r], Act<F16>::lo(pw[i]), acc[2 * i]);
                acc[2 * i + 1] = __builtin_fmaf(wv[r], Act<F16>::hi(pw[i]), acc[2 * i + 1]);
            }
        }
    }
    uint4 o;
    o.x = Act<F16>::pack(acc[0], acc[1]);
    o.y = Act<F16>::pack(acc[2], acc[3]);
    o.z = Act<F16>::pack(acc[4], acc[5]);
    o.w = Act<F16>::pack(acc[6], acc[7]);
    *reinterpret_cast<uint4 *>(y + (size_t)tok * d + c) = o;
}

// One pair of expert `expert` sent through the gate/up (or down) GEMM with the weight fragments copied out.
__global__ void prefill_dump_plan_kernel(uint32_t expert, PrefillPlan *plan, PrefillTile *tiles, uint32_t *sorted_token,
                                         uint32_t *sorted_out_row) {
    plan->n_pairs = 1;
    plan->n_tiles = 1;
    PrefillTile tl;
    tl.expert = expert;
    tl.row_start = 0;
    tl.rows = 1;
    tl.order = 0;
    tiles[0] = tl;
    sorted_token[0] = 0;
    sorted_out_row[0] = 0;
}

}  // namespace

uint32_t prefill_dump_fragments(const ArenaGeom &g, bool gate_up) {
    const uint32_t tiles = gate_up ? g.gu_rb : g.dn_rbp, groups = gate_up ? g.gd : g.gf;
    return (tiles + kTilesPerBlock - 1) / kTilesPerBlock * groups * 16;
}

hipError_t launch_prefill_dump_tiles(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t expert, bool gate_up,
                                     PrefillScratch sc, void *dump, bool f16) {
    if (f16 && !sc.act_scale) return hipErrorInvalidValue;
    hipLaunchKernelGGL(prefill_dump_plan_kernel, dim3(1), dim3(1), 0, s, expert, sc.plan, sc.tiles, sc.sorted_token,
                       sc.sorted_out_row);
    // the pair's input row is whatever row 0 of the scratch holds: only the weight side is looked at
#define FFMOE_DUMP(GU, H, A, STRIDE, OUT, NB)                                                                              \
    hipLaunchKernelGGL((prefill_gemm_kernel<GU, H, true>), dim3((NB) * 8), dim3(256), 0, s, arena_layer, g, sc.plan, sc.tiles,  \
                       sc.sorted_token, sc.sorted_out_row, A, STRIDE, OUT, NB, false, sc.act_scale, sc.act_blocks, static_cast<uint4 *>(dump))
    if (gate_up) {
        const uint32_t nb = (g.gu_rb + kTilesPerBlock - 1) / kTilesPerBlock;
        if (f16) FFMOE_DUMP(true, true, sc.partials, g.d, sc.acts, nb); else FFMOE_DUMP(true, false, sc.partials, g.d, sc.acts, nb);
    } else {
        const uint32_t nb = (g.dn_rbp + kTilesPerBlock - 1) / kTilesPerBlock;
        if (f16) FFMOE_DUMP(false, true, sc.acts, g.f, sc.partials, nb); else FFMOE_DUMP(false, false, sc.acts, g.f, sc.partials, nb);
    }
#undef FFMOE_DUMP
    return hipGetLastError();
}

hipError_t launch_prefill(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts, uint32_t top_k,
                          const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx, const uint16_t *w,
                          const ffmoe_pair *pairs, uint32_t n_pairs_in, uint16_t *y, uint16_t *partials_out,
                          PrefillScratch sc, KernelTimer *timer, bool f16, bool dense) {
    // dense: the caller vouches for a dense FFN's chunk - one expert, top_k = 1, every row routed to it at weight 1
    dense = dense && n_experts == 1 && top_k == 1 && !pairs && !y;
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
    if (dense) {
        hipLaunchKernelGGL(prefill_dense_plan_kernel, dim3(n_blocks), dim3(kSortBlock), 0, s, t, sc.plan, sc.tiles, sc.sorted_token,
                           sc.sorted_out_row);
    } else {
        hipLaunchKernelGGL(prefill_hist_kernel, dim3(n_blocks), dim3(kSortBlock), 0, s, src, sc.block_cnt);
        uint32_t e_pad = 1;
        while (e_pad < n_experts) e_pad <<= 1;          // n_experts <= FFMOE_MAX_EXPERTS = 256 <= kScanThreads
        hipLaunchKernelGGL(prefill_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, n_blocks, n_experts, e_pad, sc.block_cnt,
                           sc.plan, sc.tiles, sc.max_tiles);
        hipLaunchKernelGGL(prefill_scatter_kernel, dim3(n_blocks), dim3(kSortBlock), 0, s, src, sc.block_cnt, sc.sorted_token,
                           sc.sorted_out_row);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_PREFILL_SORT);
    const uint32_t tile_cap = min(sc.max_tiles, (src.n_items + kBM - 1) / kBM + n_experts);
    const uint32_t tile_slots = (tile_cap + 7) / 8 * 8;
    const uint32_t nb_gu = (g.gu_rb + kTilesPerBlock - 1) / kTilesPerBlock, nb_dn = (g.dn_rbp + kTilesPerBlock - 1) / kTilesPerBlock;
    if (f16 && !sc.act_scale) return hipErrorInvalidValue;      // allocated when the context was switched to FP16
    // grid: (N-blocks x tile slots) in either order of the kernel's block map
    const bool nb_major = n_experts == 1;
    auto grid_of = [&](uint32_t n_nblocks) { return nb_major ? 8 * ((n_nblocks + 7) / 8) * tile_cap : n_nblocks * tile_slots; };
    if (f16)
        hipLaunchKernelGGL((prefill_gemm_kernel<true, true>), dim3(grid_of(nb_gu)), dim3(256), 0, s, arena_layer, g, sc.plan,
                           sc.tiles, sc.sorted_token, sc.sorted_out_row, x, x_stride, sc.acts, nb_gu, nb_major, sc.act_scale, sc.act_blocks);
    else
        hipLaunchKernelGGL((prefill_gemm_kernel<true, false>), dim3(grid_of(nb_gu)), dim3(256), 0, s, arena_layer, g, sc.plan,
                           sc.tiles, sc.sorted_token, sc.sorted_out_row, x, x_stride, sc.acts, nb_gu, nb_major, nullptr, 0u);
    timer->mark(s, FFMOE_K_PREFILL_GATE_UP);
    uint16_t *partials = partials_out ? partials_out : sc.partials;
    if (f16)
        hipLaunchKernelGGL(prefill_pair_scale_kernel, dim3(tile_cap), dim3(kBM), 0, s, sc.plan, sc.tiles, g.gf, sc.act_blocks, sc.act_scale);
    if (f16)
        hipLaunchKernelGGL((prefill_gemm_kernel<false, true>), dim3(grid_of(nb_dn)), dim3(256), 0, s, arena_layer, g, sc.plan,
                           sc.tiles, sc.sorted_token, sc.sorted_out_row, sc.acts, g.f, partials, nb_dn, nb_major, sc.act_scale, sc.act_blocks);
    else
        hipLaunchKernelGGL((prefill_gemm_kernel<false, false>), dim3(grid_of(nb_dn)), dim3(256), 0, s, arena_layer, g, sc.plan,
                           sc.tiles, sc.sorted_token, sc.sorted_out_row, sc.acts, g.f, partials, nb_dn, nb_major, nullptr, 0u);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_PREFILL_DOWN);
    if (y) {
        if (f16)
            hipLaunchKernelGGL(prefill_combine_kernel<true>, dim3((t * (g.d / 8) + 255) / 256), dim3(256), 0, s, partials, w, idx,
                               n_experts, top_k, g.d, t, y);
        else
            hipLaunchKernelGGL(prefill_combine_kernel<false>, dim3((t * (g.d / 8) + 255) / 256), dim3(256), 0, s, partials, w, idx,
                               n_experts, top_k, g.d, t, y);
        timer->mark(s, FFMOE_K_PREFILL_COMBINE);
    }
    timer->finish();
    return hipGetLastError();
}

}  // namespace ffmoe
