// Re-tiling of reference-layout expert blobs into the HBM arena, and the exact bf16 expansion of
// arena tiles (the check that the re-tiling and the 16-bit dequantisation are bit-exact).
#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {

ArenaGeom make_geom(uint32_t d, uint32_t f) {
    ArenaGeom g{};
    g.d = d;
    g.f = f;
    g.gd = d / kGroup;
    g.gf = f / kGroup;
    g.gu_rb = f / kTileRows;
    g.dn_rbp = d / (2 * kTileRows);
    const size_t gu_tiles = (size_t)g.gu_rb * g.gd;
    const size_t dn_tiles = (size_t)g.dn_rbp * g.gf;
    g.gu_tiles_off = 0;
    g.gu_scales_off = g.gu_tiles_off + gu_tiles * kTileBytes;
    g.dn_tiles_off = g.gu_scales_off + gu_tiles * kTileScaleBytes;
    g.dn_scales_off = g.dn_tiles_off + dn_tiles * kTileBytes;
    g.expert_bytes = g.dn_scales_off + dn_tiles * kTileScaleBytes;
    return g;
}

namespace {

// Eight consecutive nibbles of a reference row (byte k low nibble = element 2k, high = 2k + 1,
// Metal/Quant/dequant_int4.metal:7-12) starting at element k0 (multiple of 8), read bytewise because
// packed sub-tensors need only 2-byte alignment (Kernels/Quant/DequantInt4GEMV.swift:199-202).
__device__ __forceinline__ uint32_t ref_nibbles8(const uint8_t *row, uint32_t k0) {
    const uint8_t *p = row + (k0 >> 1);
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

// Reference order (nibble j = element j) -> arena order (position m = element 2m, position m + 4 =
// element 2m + 1).
__device__ __forceinline__ uint32_t to_arena_order(uint32_t v) {
    uint32_t out = 0;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        out |= ((v >> (8 * m)) & 0xFu) << (4 * m);
        out |= ((v >> (8 * m + 4)) & 0xFu) << (4 * m + 16);
    }
    return out;
}

__device__ __forceinline__ uint16_t load_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }

// One thread per (expert, tile, lane): writes the lane's 16 B of a two-stream tile and, for lanes
// 0..15, the row's 8 B of scales. Streams: gate/up rows (A = gate row r, B = up row r) or down rows
// (A = row a, B = row a + 16).
__global__ __launch_bounds__(256) void repack_kernel(const uint8_t *__restrict__ blobs, size_t stride,
                                                     ffmoe_offsets off, uint32_t n_experts, ArenaGeom g,
                                                     uint8_t *__restrict__ arena) {
    const size_t gu_tiles = (size_t)g.gu_rb * g.gd;
    const size_t dn_tiles = (size_t)g.dn_rbp * g.gf;
    const size_t tiles_per_expert = gu_tiles + dn_tiles;
    const size_t total = (size_t)n_experts * tiles_per_expert * kWave;
    for (size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total;
         gid += (size_t)gridDim.x * blockDim.x) {
        const uint32_t lane = gid & 63;
        const size_t tile_global = gid >> 6;
        const uint32_t expert = tile_global / tiles_per_expert;
        size_t tile = tile_global % tiles_per_expert;
        const uint8_t *blob = blobs + (size_t)expert * stride;
        uint8_t *dst = arena + (size_t)expert * g.expert_bytes;
        const uint32_t i = lane & 15, jq = lane >> 4;

        const uint8_t *wa, *wb, *sa, *sb, *ba, *bb;
        uint32_t row_a, row_b, n_cols, grp;
        uint8_t *tile_dst, *scale_dst;
        if (tile < gu_tiles) {
            const uint32_t rb = tile / g.gd;
            grp = tile % g.gd;
            row_a = row_b = rb * kTileRows + i;
            n_cols = g.d;
            wa = blob + off.gate_w; sa = blob + off.gate_s; ba = blob + off.gate_b;
            wb = blob + off.up_w;   sb = blob + off.up_s;   bb = blob + off.up_b;
            tile_dst = dst + g.gu_tiles_off + tile * kTileBytes;
            scale_dst = dst + g.gu_scales_off + tile * kTileScaleBytes;
        } else {
            tile -= gu_tiles;
            const uint32_t rbp = tile / g.gf;
            grp = tile % g.gf;
            row_a = rbp * 2 * kTileRows + i;
            row_b = row_a + kTileRows;
            n_cols = g.f;
            wa = wb = blob + off.down_w; sa = sb = blob + off.down_s; ba = bb = blob + off.down_b;
            tile_dst = dst + g.dn_tiles_off + tile * kTileBytes;
            scale_dst = dst + g.dn_scales_off + tile * kTileScaleBytes;
        }
        const uint32_t row_bytes = n_cols / 2, n_groups = n_cols / kGroup;
        const uint32_t k0 = grp * kGroup + 8 * jq;
        uint4 chunk;
        chunk.x = to_arena_order(ref_nibbles8(wa + (size_t)row_a * row_bytes, k0));
        chunk.y = to_arena_order(ref_nibbles8(wa + (size_t)row_a * row_bytes, k0 + 32));
        chunk.z = to_arena_order(ref_nibbles8(wb + (size_t)row_b * row_bytes, k0));
        chunk.w = to_arena_order(ref_nibbles8(wb + (size_t)row_b * row_bytes, k0 + 32));
        reinterpret_cast<uint4 *>(tile_dst)[lane] = chunk;
        if (jq == 0) {
            uint2 sc;
            const size_t ia = ((size_t)row_a * n_groups + grp) * 2, ib = ((size_t)row_b * n_groups + grp) * 2;
            sc.x = (uint32_t)load_u16(sa + ia) | ((uint32_t)load_u16(ba + ia) << 16);
            sc.y = (uint32_t)load_u16(sb + ib) | ((uint32_t)load_u16(bb + ib) << 16);
            reinterpret_cast<uint2 *>(scale_dst)[i] = sc;
        }
    }
}

// One thread per (row, eight consecutive k): bf16(fma(q, s, b)) of one sub-tensor, row-major out.
__global__ __launch_bounds__(256) void dequant_expert_kernel(const uint8_t *__restrict__ expert, ArenaGeom g,
                                                             int which, uint16_t *__restrict__ out) {
    const uint32_t rows = which == FFMOE_DOWN ? g.d : g.f;
    const uint32_t cols = which == FFMOE_DOWN ? g.f : g.d;
    const uint32_t chunks = cols / 8;
    const size_t total = (size_t)rows * chunks;
    for (size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total;
         gid += (size_t)gridDim.x * blockDim.x) {
        const uint32_t row = gid / chunks, c = gid % chunks;
        const uint32_t k0 = c * 8, grp = k0 / kGroup, kk = k0 % kGroup;
        const uint32_t h = kk / 32, jq = (kk % 32) / 8, i = row % kTileRows;
        size_t tile;
        uint32_t dword;
        const uint8_t *tiles, *scales;
        if (which == FFMOE_DOWN) {
            const uint32_t rbp = row / (2 * kTileRows), half = (row / kTileRows) & 1;
            tile = (size_t)rbp * g.gf + grp;
            dword = 2 * half + h;
            tiles = expert + g.dn_tiles_off;
            scales = expert + g.dn_scales_off;
        } else {
            tile = (size_t)(row / kTileRows) * g.gd + grp;
            dword = (which == FFMOE_UP ? 2 : 0) + h;
            tiles = expert + g.gu_tiles_off;
            scales = expert + g.gu_scales_off;
        }
        const uint32_t lane = jq * 16 + i;
        const uint32_t w = reinterpret_cast<const uint32_t *>(tiles + tile * kTileBytes)[lane * 4 + dword];
        const uint32_t sb = reinterpret_cast<const uint32_t *>(scales + tile * kTileScaleBytes)[i * 2 + (dword >> 1)];
        const uint4 v = dequant8_bf16(w, bf16lo_to_f32(sb), bf16hi_to_f32(sb));
        *reinterpret_cast<uint4 *>(out + (size_t)row * cols + k0) = v;
    }
}

}  // namespace

hipError_t launch_repack_layer(hipStream_t s, const uint8_t *blobs, size_t stride, ffmoe_offsets off,
                               uint32_t n_experts, ArenaGeom g, uint8_t *arena_layer) {
    const size_t total = (size_t)n_experts * ((size_t)g.gu_rb * g.gd + (size_t)g.dn_rbp * g.gf) * kWave;
    const uint32_t blocks = (uint32_t)((total + 255) / 256 < 65535 * 8 ? (total + 255) / 256 : 65535 * 8);
    hipLaunchKernelGGL(repack_kernel, dim3(blocks), dim3(256), 0, s, blobs, stride, off, n_experts, g, arena_layer);
    return hipGetLastError();
}

hipError_t launch_dequant_expert(hipStream_t s, const uint8_t *arena_expert, ArenaGeom g, int which,
                                 uint16_t *out) {
    const size_t total = (size_t)(which == FFMOE_DOWN ? g.d : g.f) * ((which == FFMOE_DOWN ? g.f : g.d) / 8);
    hipLaunchKernelGGL(dequant_expert_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s,
                       arena_expert, g, which, out);
    return hipGetLastError();
}

}  // namespace ffmoe
