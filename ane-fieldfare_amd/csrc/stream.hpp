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

// `tiles` / `scales` are wave-uniform (scalar registers); the lane part is a 32-bit offset, so every ring load is
// one instruction with a scalar base and no per-load 64-bit address arithmetic.
__device__ __forceinline__ void ring_fill(WeightRing &ring, int u, const uint8_t *tiles, const uint8_t *scales,
                                          uint32_t g_clamped, uint32_t lane) {
    const uint8_t *tg = tiles + (size_t)g_clamped * kTileBytes, *sg = scales + (size_t)g_clamped * kTileScaleBytes;
    ring.t[u] = *reinterpret_cast<const uint4 *>(tg + lane * 16u);
    ring.s[u] = *reinterpret_cast<const uint2 *>(sg + (lane & 15u) * 8u);
}

// Consume ring slot u against the resident token operand, then start the load that refills the slot.
__device__ __forceinline__ void ring_step(WeightRing &ring, int u, bool live, const uint4 &x0, const uint4 &x1,
                                          TwoStreamAcc &tot, const uint8_t *next_tiles, const uint8_t *next_scales,
                                          uint32_t next_g, uint32_t lane) {
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const uint4 ones_bits = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones_bits);
    const uint4 tile = ring.t[u];
    uint2 sc = ring.s[u];
    if (!live) sc = make_uint2(0u, 0u);
    ring_fill(ring, u, next_tiles, next_scales, next_g, lane);
    const bf16x8 a0 = __builtin_bit_cast(bf16x8, x0), a1 = __builtin_bit_cast(bf16x8, x1);
    f32x4 acc_a = mfma16(a0, unpack8_offset128(tile.x), zero);
    acc_a = mfma16(a1, unpack8_offset128(tile.y), acc_a);
    f32x4 acc_b = mfma16(a0, unpack8_offset128(tile.z), zero);
    acc_b = mfma16(a1, unpack8_offset128(tile.w), acc_b);
    f32x4 sx = mfma16(a0, ones, zero);
    sx = mfma16(a1, ones, sx);
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
}

// Split `n_items` of one expert over `parts` workers: worker `sub` gets [first, last).
__device__ __forceinline__ void split_range(uint32_t n_items, uint32_t parts, uint32_t sub, uint32_t &first,
                                            uint32_t &last) {
    first = (uint32_t)((uint64_t)sub * n_items / parts);
    last = (uint32_t)((uint64_t)(sub + 1) * n_items / parts);
}

}  // namespace ffmoe
