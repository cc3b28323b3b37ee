// Generic MLX-affine INT4 GEMV over weights in the reference's row-major layout (W uint8 [m][n/2],
// bf16 scale/bias per 64): y[r] = W x[r] for 1..16 input rows against one read of W.
//
// Replaces dequant_int4_gemv_simd / dequant_int4_gemv_rows (Metal/Quant/dequant_int4.metal:78-357) and
// the LM-head row GEMV (Metal/Sampling/logit.metal:614-667).
//
// A wave owns kRowsPerWave consecutive weight rows. Lane l owns the 16-byte chunks l, l + 64, ... of
// every row (32 nibbles = half a group each), so one load instruction covers 1 KiB of a row and the
// input values a lane needs are the same for all of its rows: they are loaded once per chunk round,
// paired as (x[m], x[m+4]) to line up with ((w >> 4m) & 0x000F000F), and reused for every weight row.
// Per chunk: acc = sum (128 + q) x by v_dot2_f32_bf16, then s * acc + (b - 128 s) * sum x, the factored
// form of dequant_int4.metal:104-139. Rows are reduced across the wave by a xor-butterfly.
// Each input row accumulates independently of the others, so row r of a multi-row call equals the
// single-row call bit for bit (the property DequantInt4SmallBatchTests.swift:74-78 asserts).
#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {
namespace {

constexpr int kRowsPerWave = 8;
constexpr int kRowTile = 4;   // input rows held in registers per pass

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

template <bool F16>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    if constexpr (F16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

template <bool ALIGNED>
__device__ __forceinline__ uint4 load_chunk(const uint8_t *p) {
    if (ALIGNED) return *reinterpret_cast<const uint4 *>(p);
    const uint16_t *h = reinterpret_cast<const uint16_t *>(p);   // 2-byte alignment is guaranteed
    uint4 r;
    r.x = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
    r.y = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
    r.z = (uint32_t)h[4] | ((uint32_t)h[5] << 16);
    r.w = (uint32_t)h[6] | ((uint32_t)h[7] << 16);
    return r;
}

// eight consecutive bf16 inputs as four dwords
template <bool X_ALIGNED>
__device__ __forceinline__ uint4 load_x8(const uint16_t *src) {
    if (X_ALIGNED) return *reinterpret_cast<const uint4 *>(src);
    uint4 r;
    r.x = (uint32_t)src[0] | ((uint32_t)src[1] << 16);
    r.y = (uint32_t)src[2] | ((uint32_t)src[3] << 16);
    r.z = (uint32_t)src[4] | ((uint32_t)src[5] << 16);
    r.w = (uint32_t)src[6] | ((uint32_t)src[7] << 16);
    return r;
}

// F16: inputs and 16-bit outputs are FP16 (a context in FP16 mode); the offset form is then 1024 + q
template <bool ALIGNED, bool X_ALIGNED, bool Y_F32, bool F16>
__global__ __launch_bounds__(256) void gemv_int4_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ scales,
                                                        const uint16_t *__restrict__ biases,
                                                        const uint16_t *__restrict__ x, void *__restrict__ y_,
                                                        uint32_t m, uint32_t n, uint32_t rows, uint32_t x_stride,
                                                        uint32_t y_stride, const uint32_t *__restrict__ ids) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t m0 = (blockIdx.x * 4 + wave) * kRowsPerWave;
    if (m0 >= m) return;
    // output o is weight row o, or row ids[o] of the table when a list is given (encodeRowsListed)
    uint32_t wrow[kRowsPerWave];
#pragma unroll
    for (int mi = 0; mi < kRowsPerWave; ++mi) {
        const uint32_t o = min(m0 + mi, m - 1);
        wrow[mi] = ids ? ids[o] : o;
    }
    const uint32_t row_bytes = n / 2, n_groups = n / kGroup, chunks = n / 32;
    const uint32_t rounds = (chunks + 63) / 64;

    for (uint32_t r0 = 0; r0 < rows; r0 += kRowTile) {
        float acc[kRowsPerWave][kRowTile];
#pragma unroll
        for (int mi = 0; mi < kRowsPerWave; ++mi)
#pragma unroll
            for (int r = 0; r < kRowTile; ++r) acc[mi][r] = 0.0f;

        for (uint32_t j = 0; j < rounds; ++j) {
            const uint32_t c = lane + 64 * j;
            if (c >= chunks) continue;
            // input values of this chunk, paired (x[e], x[e+4]) per run of eight, and their sum
            uint32_t xp[kRowTile][16];
            float sx[kRowTile];
#pragma unroll
            for (int r = 0; r < kRowTile; ++r) {
                const uint32_t row = min(r0 + r, rows - 1);
                const uint16_t *src = x + (size_t)row * x_stride + (size_t)c * 32;
                float sum = 0.0f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint4 dv = load_x8<X_ALIGNED>(src + q * 8);
                    const uint32_t d[4] = {dv.x, dv.y, dv.z, dv.w};
                    xp[r][q * 4 + 0] = (d[0] & 0xFFFFu) | (d[2] << 16);
                    xp[r][q * 4 + 1] = (d[0] >> 16) | (d[2] & 0xFFFF0000u);
                    xp[r][q * 4 + 2] = (d[1] & 0xFFFFu) | (d[3] << 16);
                    xp[r][q * 4 + 3] = (d[1] >> 16) | (d[3] & 0xFFFF0000u);
#pragma unroll
                    for (int i = 0; i < 4; ++i) { sum += Act<F16>::lo(d[i]); sum += Act<F16>::hi(d[i]); }
                }
                sx[r] = sum;
            }
            uint4 wv[kRowsPerWave];
            uint32_t sb[kRowsPerWave];
#pragma unroll
            for (int mi = 0; mi < kRowsPerWave; ++mi) {
                const uint32_t row = wrow[mi];
                wv[mi] = load_chunk<ALIGNED>(w + (size_t)row * row_bytes + (size_t)c * 16);
                const size_t gi = (size_t)row * n_groups + (c >> 1);
                sb[mi] = (uint32_t)scales[gi] | ((uint32_t)biases[gi] << 16);
            }
#pragma unroll
            for (int mi = 0; mi < kRowsPerWave; ++mi) {
                uint32_t q[16];
                const uint32_t ww[4] = {wv[mi].x, wv[mi].y, wv[mi].z, wv[mi].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int p = 0; p < 4; ++p) q[i * 4 + p] = ((ww[i] >> (4 * p)) & 0x000F000Fu) | Act<F16>::kOffsetBits;
                }
                const float s = bf16lo_to_f32(sb[mi]), b = bf16hi_to_f32(sb[mi]);
                const float tb = __builtin_fmaf(-Act<F16>::kOffset, s, b);
#pragma unroll
                for (int r = 0; r < kRowTile; ++r) {
                    float dsum = 0.0f;
#pragma unroll
                    for (int p = 0; p < 16; ++p) dsum = dot2<F16>(q[p], xp[r][p], dsum);
                    acc[mi][r] = __builtin_fmaf(s, dsum, acc[mi][r]);
                    acc[mi][r] = __builtin_fmaf(tb, sx[r], acc[mi][r]);
                }
            }
        }
#pragma unroll
        for (int mi = 0; mi < kRowsPerWave; ++mi) {
#pragma unroll
            for (int r = 0; r < kRowTile; ++r) {
                const float v = wave_butterfly_sum_shuffle(acc[mi][r]);
                if (lane == 0 && m0 + mi < m && r0 + r < rows) {
                    const size_t o = (size_t)(r0 + r) * y_stride + m0 + mi;
                    if (Y_F32) reinterpret_cast<float *>(y_)[o] = v;
                    else reinterpret_cast<uint16_t *>(y_)[o] = Act<F16>::round(v);
                }
            }
        }
    }
}

}  // namespace

hipError_t launch_gemv_int4(hipStream_t s, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                            const uint16_t *x, void *y, uint32_t m, uint32_t n, uint32_t rows,
                            uint32_t x_stride, uint32_t y_stride, int y_f32, const uint32_t *ids, bool f16) {
    const uint32_t waves = (m + kRowsPerWave - 1) / kRowsPerWave;
    const dim3 grid((waves + 3) / 4), block(256);
    const bool aligned = (reinterpret_cast<uintptr_t>(w) % 16 == 0) && ((n / 2) % 16 == 0);
    const bool x_aligned = (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (x_stride % 8 == 0);
#define FFMOE_GEMV16(A, F) \
    hipLaunchKernelGGL((gemv_int4_kernel<A, true, F, true>), grid, block, 0, s, w, scales, biases, x, y, m, n, rows, x_stride, y_stride, ids)
    if (f16) {
        if (!x_aligned) return hipErrorInvalidValue;     // FP16 rows come 16-byte aligned (checked at the boundary)
        if (aligned) { if (y_f32) FFMOE_GEMV16(true, true); else FFMOE_GEMV16(true, false); }
        else { if (y_f32) FFMOE_GEMV16(false, true); else FFMOE_GEMV16(false, false); }
        return hipGetLastError();
    }
#undef FFMOE_GEMV16
#define FFMOE_GEMV(A, X, F) \
    hipLaunchKernelGGL((gemv_int4_kernel<A, X, F, false>), grid, block, 0, s, w, scales, biases, x, y, m, n, rows, x_stride, y_stride, ids)
    if (aligned && x_aligned) { if (y_f32) FFMOE_GEMV(true, true, true); else FFMOE_GEMV(true, true, false); }
    else if (aligned) { if (y_f32) FFMOE_GEMV(true, false, true); else FFMOE_GEMV(true, false, false); }
    else if (x_aligned) { if (y_f32) FFMOE_GEMV(false, true, true); else FFMOE_GEMV(false, true, false); }
    else { if (y_f32) FFMOE_GEMV(false, false, true); else FFMOE_GEMV(false, false, false); }
#undef FFMOE_GEMV
    return hipGetLastError();
}

}  // namespace ffmoe
