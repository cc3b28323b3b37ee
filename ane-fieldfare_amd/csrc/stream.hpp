// Register-ring streaming of two-stream arena tiles, shared by the expert kernels and the resident-matrix
// GEMV: one wave consumes a group's tile (16 + 16 weight rows x 64 k) against up to 16 token rows on the
// matrix unit and immediately starts the load that refills the ring slot.
#pragma once

#include "common.hpp"

namespace ffmoe {

constexpr int kKSplit = 4;      // waves of a block that split K
constexpr int kRing = 11;       // groups in flight per wave (= one K-slice of D = 2816)

struct TwoStreamAcc {
    f32x4 a, b;
};

struct WeightRing {
    uint4 t[kRing];
    uint2 s[kRing];
};

// Where a wave's tiles come from: two buffer descriptors (scalar registers). A ring load is then a single
// buffer_load with the lane's fixed 32-bit offset and a scalar byte offset - no per-load 64-bit address
// arithmetic in vector registers, which otherwise costs two registers per load in flight - and a load
// past the end of the region returns zero instead of faulting.
struct TileSource {
    __amdgpu_buffer_rsrc_t tiles, scales;
};

__device__ __forceinline__ TileSource make_tile_source(const uint8_t *tiles, size_t tile_bytes, const uint8_t *scales,
                                                       size_t scale_bytes) {
    TileSource src;
    src.tiles = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(tiles), 0, (int)(uint32_t)tile_bytes, 0x00020000);
    src.scales = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(scales), 0, (int)(uint32_t)scale_bytes, 0x00020000);
    return src;
}

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// `tile_index` = index of the 1 KiB tile inside the region (wave-uniform).
__device__ __forceinline__ void ring_fill(WeightRing &ring, int u, const TileSource &src, uint32_t tile_index,
                                          uint32_t lane) {
    // the index is wave-uniform by contract; pinning it to a scalar register spares the waterfall loop the
    // compiler emits whenever it happened to compute a uniform value in a vector register
    tile_index = __builtin_amdgcn_readfirstlane(tile_index);
    const u32x4_t t = __builtin_amdgcn_raw_buffer_load_b128(src.tiles, (int)(lane * 16u), (int)(tile_index * kTileBytes), 0);
    const u32x2_t s = __builtin_amdgcn_raw_buffer_load_b64(src.scales, (int)((lane & 15u) * 8u),
                                                           (int)(tile_index * kTileScaleBytes), 0);
    ring.t[u] = make_uint4(t.x, t.y, t.z, t.w);
    ring.s[u] = make_uint2(s.x, s.y);
}

// Sum of a group's 64 inputs per token column, in the register layout of the matrix results: the product
// with an all-ones operand. It depends on the token operand only, so a wave that walks several tile rows
// with the same operand computes it once per group, not once per tile.
template <bool F16 = false>
__device__ __forceinline__ f32x4 group_input_sum(const uint4 &x0, const uint4 &x1) {
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const uint4 ones = {Act<F16>::kOnesBits, Act<F16>::kOnesBits, Act<F16>::kOnesBits, Act<F16>::kOnesBits};
    return Act<F16>::mfma(x1, ones, Act<F16>::mfma(x0, ones, zero));
}

// Consume ring slot u against the resident token operand (`sx` = its group_input_sum), then start the load
// that refills the slot (REFILL = false: a wave that walks one tile row only has nothing to refill).
template <bool F16 = false, bool REFILL = true>
__device__ __forceinline__ void ring_step(WeightRing &ring, int u, bool live, const uint4 &x0, const uint4 &x1,
                                          const f32x4 &sx, TwoStreamAcc &tot, const TileSource &src,
                                          uint32_t next_tile_index, uint32_t lane) {
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const uint4 tile = ring.t[u];
    uint2 sc = ring.s[u];
    if (!live) sc = make_uint2(0u, 0u);
    if (REFILL) ring_fill(ring, u, src, next_tile_index, lane);
    f32x4 acc_a = Act<F16>::mfma(x0, unpack8_offset<F16>(tile.x), zero);
    acc_a = Act<F16>::mfma(x1, unpack8_offset<F16>(tile.y), acc_a);
    f32x4 acc_b = Act<F16>::mfma(x0, unpack8_offset<F16>(tile.z), zero);
    acc_b = Act<F16>::mfma(x1, unpack8_offset<F16>(tile.w), acc_b);
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

// A wave's share of K when the four waves of a block split it.
struct KSlice {
    uint32_t g0, ng, g_last;      // first group, number of groups, last valid group of this wave's share of K
};
__device__ __forceinline__ KSlice k_slice(uint32_t groups, uint32_t ks) {
    const uint32_t per = (groups + kKSplit - 1) / kKSplit;
    const uint32_t g0 = min(ks * per, groups), g1 = min(groups, g0 + per);
    return KSlice{g0, g1 - g0, g1 > g0 ? g1 - 1 : groups - 1};
}

// The token operand is the call's rows themselves, row min(j, rows - 1) in token column j (in the expert kernels:
// which expert a block serves does not matter for fetching them, so they can be requested before the routes are
// known; an expert's routes only decide which columns of the result are stored).
// Load layout: four neighbouring lanes read 64 contiguous bytes of one row (row lane / 4, 8-element chunk
// lane % 4), 16 requests of 64 bytes per instruction; with the matrix unit's own layout (row lane % 16)
// every lane would be a request of its own and the 22 loads of a wave would keep the address unit busy
// for microseconds. turn_token_rows() re-lays them into the operand layout (lane (j, jq): row j, chunk jq).
__device__ __forceinline__ void load_token_rows(const uint16_t *__restrict__ x, uint32_t x_stride, uint32_t rows,
                                                uint32_t lane, const KSlice &k, uint4 (&x0)[kRing], uint4 (&x1)[kRing]) {
    const uint16_t *xrow = x + (size_t)min(lane >> 2, rows - 1) * x_stride + 8 * (lane & 3);
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
        const bool live = (uint32_t)u < k.ng;
        const uint32_t gg = min(k.g0 + u, k.g_last);
        x0[u] = live ? *reinterpret_cast<const uint4 *>(xrow + gg * kGroup) : uint4{0, 0, 0, 0};
        x1[u] = live ? *reinterpret_cast<const uint4 *>(xrow + gg * kGroup + 32) : uint4{0, 0, 0, 0};
    }
}

__device__ __forceinline__ void turn_token_rows(uint32_t lane, uint4 (&x0)[kRing], uint4 (&x1)[kRing]) {
    const uint32_t j = lane & 15, jq = lane >> 4;
    const int pull = (int)((4 * j + jq) * 4);       // operand lane (j, jq) takes what load lane 4 j + jq holds
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

// Split `n_items` of one expert over `parts` workers: worker `sub` gets [first, last).
__device__ __forceinline__ void split_range(uint32_t n_items, uint32_t parts, uint32_t sub, uint32_t &first,
                                            uint32_t &last) {
    first = (uint32_t)((uint64_t)sub * n_items / parts);
    last = (uint32_t)((uint64_t)(sub + 1) * n_items / parts);
}

}  // namespace ffmoe
