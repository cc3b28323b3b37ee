// The steps either side of the MoE stage, one block per token row:
//   post-attention setup  fused_post_attn_setup (Metal/Fusions/fused.metal:210-296) and its block form
//                         prefill_post_attn_setup_block (Metal/Prefill/prefill.metal:243-318)
//   layer tail            prefill_layer_tail_block (Metal/Prefill/prefill.metal:320-399) and the decode
//                         tail of Kernels/Fusions/FusedLayerTail.swift
// Both are RMS norms around residual adds with every intermediate rounded to 16 bits where the reference
// rounds to FP16. A thread keeps its elements in registers from the first read to the last write (the
// reference stages rows in threadgroup memory); a row is read once and written once: HBM-bound.
//
// Summation order of the squares (the reference's simd_sum leaves it open): thread t owns the 8-element
// chunks t, t + 256, ... and adds their squares in index order with fmaf; the wave meets in a
// xor-butterfly; the four wave sums combine as (w0 + w1) + (w2 + w3); inv = 1 / sqrt(sum / D + eps) with
// IEEE division and square root. Rows that are not 16-byte aligned take scalar loads of the same elements,
// so both paths give the same bits.
#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {
namespace {

constexpr int kRowThreads = 256;
constexpr int kMaxChunks = 2;        // D <= 4096: at most two 8-element chunks per thread

struct Row8 {
    float v[8];
};

// Rows are in the context's activation type (F16: FP16, else bf16); norm weights are always bf16 (loadw8).
template <bool VEC, bool F16>
__device__ __forceinline__ Row8 load8(const uint16_t *__restrict__ row, uint32_t chunk) {
    Row8 r;
    if (VEC) {
        const uint4 q = reinterpret_cast<const uint4 *>(row)[chunk];
        r.v[0] = Act<F16>::lo(q.x); r.v[1] = Act<F16>::hi(q.x);
        r.v[2] = Act<F16>::lo(q.y); r.v[3] = Act<F16>::hi(q.y);
        r.v[4] = Act<F16>::lo(q.z); r.v[5] = Act<F16>::hi(q.z);
        r.v[6] = Act<F16>::lo(q.w); r.v[7] = Act<F16>::hi(q.w);
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) r.v[e] = Act<F16>::widen(row[8 * chunk + e]);
    }
    return r;
}

template <bool VEC>
__device__ __forceinline__ Row8 loadw8(const uint16_t *__restrict__ row, uint32_t chunk) {
    return load8<VEC, false>(row, chunk);
}

template <bool VEC, bool F16>
__device__ __forceinline__ void store8(uint16_t *__restrict__ row, uint32_t chunk, const Row8 &r) {
    if (VEC) {
        uint4 q;
        q.x = Act<F16>::pack(r.v[0], r.v[1]);
        q.y = Act<F16>::pack(r.v[2], r.v[3]);
        q.z = Act<F16>::pack(r.v[4], r.v[5]);
        q.w = Act<F16>::pack(r.v[6], r.v[7]);
        reinterpret_cast<uint4 *>(row)[chunk] = q;
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) row[8 * chunk + e] = Act<F16>::round(r.v[e]);
    }
}

template <bool F16>
__device__ __forceinline__ float round16(float x) { return Act<F16>::widen(Act<F16>::round(x)); }

// 1 / sqrt(mean of squares + eps) over the block's row; `slot` is a 4-float LDS area of its own
__device__ __forceinline__ float block_rms_inv(const Row8 (&x)[kMaxChunks], uint32_t n_mine, uint32_t d, float eps,
                                               float *slot) {
    float acc = 0.0f;
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = __builtin_fmaf(x[c].v[e], x[c].v[e], acc);
    acc = wave_butterfly_sum(acc);
    if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float total = (slot[0] + slot[1]) + (slot[2] + slot[3]);
    return 1.0f / sqrtf(total / (float)d + eps);
}

template <bool VEC, bool F16>
__global__ __launch_bounds__(kRowThreads) void post_attn_setup_kernel(
    uint16_t *__restrict__ hidden, uint32_t hidden_stride, const uint16_t *__restrict__ attn, uint32_t attn_stride,
    uint16_t *__restrict__ dense_x, uint32_t dense_stride, uint16_t *__restrict__ routed_x, uint32_t routed_stride,
    uint16_t *__restrict__ router_x, uint32_t router_stride, const uint16_t *__restrict__ w_post_attn,
    const uint16_t *__restrict__ w_pre_ffn, const uint16_t *__restrict__ w_pre_ffn2, uint32_t d, float eps) {
    __shared__ float s_sum[2][4];
    const uint32_t row = blockIdx.x, t = threadIdx.x, chunks = d / 8;
    const uint32_t n_mine = t < chunks ? (chunks - t + kRowThreads - 1) / kRowThreads : 0;
    uint16_t *hrow = hidden + (size_t)row * hidden_stride;
    const uint16_t *arow = attn + (size_t)row * attn_stride;
    Row8 a[kMaxChunks], h[kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            a[c] = load8<VEC, F16>(arow, t + c * kRowThreads);
            h[c] = load8<VEC, F16>(hrow, t + c * kRowThreads);
        }
    const float attn_inv = block_rms_inv(a, n_mine, d, eps, s_sum[0]);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const Row8 w = loadw8<VEC>(w_post_attn, t + c * kRowThreads);
#pragma unroll
            for (int e = 0; e < 8; ++e) h[c].v[e] = round16<F16>(h[c].v[e] + round16<F16>(a[c].v[e] * attn_inv * w.v[e]));
            store8<VEC, F16>(hrow, t + c * kRowThreads, h[c]);
        }
    const float hidden_inv = block_rms_inv(h, n_mine, d, eps, s_sum[1]);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
            const Row8 w1 = loadw8<VEC>(w_pre_ffn, chunk), w2 = loadw8<VEC>(w_pre_ffn2, chunk);
            Row8 o_dense, o_routed, o_router;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float v = h[c].v[e] * hidden_inv;
                o_dense.v[e] = v * w1.v[e];
                o_routed.v[e] = v * w2.v[e];
                o_router.v[e] = v;
            }
            store8<VEC, F16>(dense_x + (size_t)row * dense_stride, chunk, o_dense);
            store8<VEC, F16>(routed_x + (size_t)row * routed_stride, chunk, o_routed);
            store8<VEC, F16>(router_x + (size_t)row * router_stride, chunk, o_router);
        }
}

// NORMS: h1 arrives before its own norm (w_postffn1) and, when w_next is given, the norm of the new hidden
// row under w_next goes to `normed` (the next layer's input norm): fused_layer_tail_norms
// (Kernels/Fusions/FusedLayerTail.swift:74-117). h1 itself is left as it was found.
template <bool VEC, bool NORMS, bool F16>
__global__ __launch_bounds__(kRowThreads) void layer_tail_kernel(const uint16_t *__restrict__ h2, uint32_t h2_stride,
                                                                 const uint16_t *__restrict__ h1, uint32_t h1_stride,
                                                                 uint16_t *__restrict__ hidden, uint32_t hidden_stride,
                                                                 const uint16_t *__restrict__ w_postffn2,
                                                                 const uint16_t *__restrict__ w_postffn, uint32_t d,
                                                                 float eps, float layer_scalar,
                                                                 const uint16_t *__restrict__ w_postffn1,
                                                                 const uint16_t *__restrict__ w_next,
                                                                 uint16_t *__restrict__ normed, uint32_t normed_stride) {
    __shared__ float s_sum[4][4];
    const uint32_t row = blockIdx.x, t = threadIdx.x, chunks = d / 8;
    const uint32_t n_mine = t < chunks ? (chunks - t + kRowThreads - 1) / kRowThreads : 0;
    uint16_t *hrow = hidden + (size_t)row * hidden_stride;
    Row8 a[kMaxChunks], h12[kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            a[c] = load8<VEC, F16>(h2 + (size_t)row * h2_stride, t + c * kRowThreads);
            h12[c] = load8<VEC, F16>(h1 + (size_t)row * h1_stride, t + c * kRowThreads);
        }
    if (NORMS) {
        const float inv_h1 = block_rms_inv(h12, n_mine, d, eps, s_sum[2]);
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c)
            if ((uint32_t)c < n_mine) {
                const Row8 w = loadw8<VEC>(w_postffn1, t + c * kRowThreads);
#pragma unroll
                for (int e = 0; e < 8; ++e) h12[c].v[e] = round16<F16>(h12[c].v[e] * inv_h1 * w.v[e]);
            }
    }
    const float inv_h2 = block_rms_inv(a, n_mine, d, eps, s_sum[0]);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const Row8 w = loadw8<VEC>(w_postffn2, t + c * kRowThreads);
#pragma unroll
            for (int e = 0; e < 8; ++e) h12[c].v[e] = round16<F16>(h12[c].v[e] + round16<F16>(a[c].v[e] * inv_h2 * w.v[e]));
        }
    const float inv_h12 = block_rms_inv(h12, n_mine, d, eps, s_sum[1]);
    const float scale = round16<F16>(layer_scalar);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
            const Row8 w = loadw8<VEC>(w_postffn, chunk);
            Row8 hv = load8<VEC, F16>(hrow, chunk);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                hv.v[e] = round16<F16>(round16<F16>(hv.v[e] + round16<F16>(h12[c].v[e] * inv_h12 * w.v[e])) * scale);
            store8<VEC, F16>(hrow, chunk, hv);
            a[c] = hv;          // the new hidden row, as stored
        }
    if (NORMS && w_next) {
        const float inv_next = block_rms_inv(a, n_mine, d, eps, s_sum[3]);
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c)
            if ((uint32_t)c < n_mine) {
                const uint32_t chunk = t + c * kRowThreads;
                const Row8 w = loadw8<VEC>(w_next, chunk);
                Row8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o.v[e] = a[c].v[e] * inv_next * w.v[e];
                store8<VEC, F16>(normed + (size_t)row * normed_stride, chunk, o);
            }
    }
}

// rmsnorm_bf16w (RMSNorm.encodeBF16W): out = round((x * inv) * w) per row; out may be x.
template <bool VEC, bool F16>
__global__ __launch_bounds__(kRowThreads) void rmsnorm_kernel(const uint16_t *x, uint32_t x_stride, const uint16_t *__restrict__ w,
                                                              uint16_t *out, uint32_t out_stride, uint32_t d, float eps) {
    __shared__ float s_sum[4];
    const uint32_t row = blockIdx.x, t = threadIdx.x, chunks = d / 8;
    const uint32_t n_mine = t < chunks ? (chunks - t + kRowThreads - 1) / kRowThreads : 0;
    Row8 a[kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) a[c] = load8<VEC, F16>(x + (size_t)row * x_stride, t + c * kRowThreads);
    const float inv = block_rms_inv(a, n_mine, d, eps, s_sum);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
            const Row8 wv = loadw8<VEC>(w, chunk);
            Row8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o.v[e] = a[c].v[e] * inv * wv.v[e];
            store8<VEC, F16>(out + (size_t)row * out_stride, chunk, o);
        }
}

bool aligned16(const void *p, uint32_t stride) { return reinterpret_cast<uintptr_t>(p) % 16 == 0 && stride % 8 == 0; }

}  // namespace

hipError_t launch_post_attn_setup(hipStream_t s, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *attn,
                                  uint32_t attn_stride, uint16_t *dense_x, uint32_t dense_stride, uint16_t *routed_x,
                                  uint32_t routed_stride, uint16_t *router_x, uint32_t router_stride,
                                  const uint16_t *w_post_attn, const uint16_t *w_pre_ffn, const uint16_t *w_pre_ffn2,
                                  uint32_t t, uint32_t d, float eps, bool f16) {
    const bool vec = aligned16(hidden, hidden_stride) && aligned16(attn, attn_stride) && aligned16(dense_x, dense_stride) &&
                     aligned16(routed_x, routed_stride) && aligned16(router_x, router_stride) && aligned16(w_post_attn, 8) &&
                     aligned16(w_pre_ffn, 8) && aligned16(w_pre_ffn2, 8);
#define FFMOE_SETUP(V, H)                                                                                                  \
    hipLaunchKernelGGL((post_attn_setup_kernel<V, H>), dim3(t), dim3(kRowThreads), 0, s, hidden, hidden_stride, attn, attn_stride, \
                       dense_x, dense_stride, routed_x, routed_stride, router_x, router_stride, w_post_attn, w_pre_ffn,       \
                       w_pre_ffn2, d, eps)
    if (f16) { if (vec) FFMOE_SETUP(true, true); else FFMOE_SETUP(false, true); }
    else { if (vec) FFMOE_SETUP(true, false); else FFMOE_SETUP(false, false); }
#undef FFMOE_SETUP
    return hipGetLastError();
}

hipError_t launch_layer_tail(hipStream_t s, const uint16_t *h2, uint32_t h2_stride, const uint16_t *h1, uint32_t h1_stride,
                             uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2, const uint16_t *w_postffn,
                             uint32_t t, uint32_t d, float eps, float layer_scalar, const uint16_t *w_postffn1,
                             const uint16_t *w_next, uint16_t *normed, uint32_t normed_stride, bool f16) {
    const bool norms = w_postffn1 != nullptr;
    const bool vec = aligned16(h2, h2_stride) && aligned16(h1, h1_stride) && aligned16(hidden, hidden_stride) &&
                     aligned16(w_postffn2, 8) && aligned16(w_postffn, 8) &&
                     (!norms || (aligned16(w_postffn1, 8) && (!w_next || (aligned16(w_next, 8) && aligned16(normed, normed_stride)))));
#define FFMOE_TAIL(V, N)                                                                                              \
    do {                                                                                                              \
        if (f16)                                                                                                      \
            hipLaunchKernelGGL((layer_tail_kernel<V, N, true>), dim3(t), dim3(kRowThreads), 0, s, h2, h2_stride, h1, h1_stride, \
                               hidden, hidden_stride, w_postffn2, w_postffn, d, eps, layer_scalar, w_postffn1, w_next, normed, \
                               normed_stride);                                                                        \
        else                                                                                                          \
            hipLaunchKernelGGL((layer_tail_kernel<V, N, false>), dim3(t), dim3(kRowThreads), 0, s, h2, h2_stride, h1, h1_stride, \
                               hidden, hidden_stride, w_postffn2, w_postffn, d, eps, layer_scalar, w_postffn1, w_next, normed, \
                               normed_stride);                                                                        \
    } while (0)
    if (vec) { if (norms) FFMOE_TAIL(true, true); else FFMOE_TAIL(true, false); }
    else { if (norms) FFMOE_TAIL(false, true); else FFMOE_TAIL(false, false); }
#undef FFMOE_TAIL
    return hipGetLastError();
}

hipError_t launch_rmsnorm(hipStream_t s, const uint16_t *x, uint32_t x_stride, const uint16_t *w, uint16_t *out,
                          uint32_t out_stride, uint32_t t, uint32_t d, float eps, bool f16) {
    const bool vec = aligned16(x, x_stride) && aligned16(out, out_stride) && aligned16(w, 8);
#define FFMOE_NORM(V, H) \
    hipLaunchKernelGGL((rmsnorm_kernel<V, H>), dim3(t), dim3(kRowThreads), 0, s, x, x_stride, w, out, out_stride, d, eps)
    if (f16) { if (vec) FFMOE_NORM(true, true); else FFMOE_NORM(false, true); }
    else { if (vec) FFMOE_NORM(true, false); else FFMOE_NORM(false, false); }
#undef FFMOE_NORM
    return hipGetLastError();
}

}  // namespace ffmoe
