// The steps either side of the MoE stage, one block per token row:
//   post-attention setup  fused_post_attn_setup (Metal/Fusions/fused.metal:210-296) and its block form
//                         prefill_post_attn_setup_block (Metal/Prefill/prefill.metal:243-318)
//   layer tail            prefill_layer_tail_block (Metal/Prefill/prefill.metal:320-399) and the decode
//                         tail of Kernels/Fusions/FusedLayerTail.swift
// Both are RMS norms around residual adds with every intermediate rounded to 16 bits where the reference
// rounds to FP16. A thread keeps its elements in registers from the first read to the last write (the
// reference stages rows in threadgroup memory); a row is read once and written once: HBM-bound.
// Every input row and every weight vector of a launch is requested before the first reduction, so a launch is one
// memory round trip and its block reductions (a load issued behind a reduction is another dependent round trip, and
// at 16 rows these kernels are nothing but their round trips).
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
    Row8 a[kMaxChunks], h[kMaxChunks], w0[kMaxChunks], w1[kMaxChunks], w2[kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            a[c] = load8<VEC, F16>(arow, t + c * kRowThreads);
            h[c] = load8<VEC, F16>(hrow, t + c * kRowThreads);
            w0[c] = loadw8<VEC>(w_post_attn, t + c * kRowThreads);
            w1[c] = loadw8<VEC>(w_pre_ffn, t + c * kRowThreads);
            w2[c] = loadw8<VEC>(w_pre_ffn2, t + c * kRowThreads);
        }
    const float attn_inv = block_rms_inv(a, n_mine, d, eps, s_sum[0]);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
#pragma unroll
            for (int e = 0; e < 8; ++e) h[c].v[e] = round16<F16>(h[c].v[e] + round16<F16>(a[c].v[e] * attn_inv * w0[c].v[e]));
            store8<VEC, F16>(hrow, t + c * kRowThreads, h[c]);
        }
    const float hidden_inv = block_rms_inv(h, n_mine, d, eps, s_sum[1]);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
            Row8 o_dense, o_routed, o_router;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float v = h[c].v[e] * hidden_inv;
                o_dense.v[e] = v * w1[c].v[e];
                o_routed.v[e] = v * w2[c].v[e];
                o_router.v[e] = v;
            }
            store8<VEC, F16>(dense_x + (size_t)row * dense_stride, chunk, o_dense);
            store8<VEC, F16>(routed_x + (size_t)row * routed_stride, chunk, o_routed);
            store8<VEC, F16>(router_x + (size_t)row * router_stride, chunk, o_router);
        }
}

// Where h2 comes from when the routed experts' rows arrive un-combined (COMBINE): the un-weighted fp32 rows of a
// decode / verify call, the routes' weights and the plan's validity words. h2 = the combine kernel's row: fmaf over
// the valid routes in rank order from zero, one rounding to 16 bits - made in this kernel's load stage instead of a
// launch of its own, with the same arithmetic, so the tail's results keep their bits.
struct RoutedRows {
    const float *partials;           // [t * top_k][d]
    const uint16_t *w;               // [t][top_k]
    const uint32_t *route_valid;     // [t * top_k]
    uint32_t top_k;
    // h1 likewise, when the shared expert's down projection rode along in the routed experts' launch and left its K in
    // chunks: h1 = the chunks' fp32 rows added in chunk order, one rounding to 16 bits (what the dense FFN's own down
    // launch rounds once too). Null: h1 is read as a 16-bit row.
    const float *shared_partials;    // [shared_chunks][t][d]
    uint32_t shared_chunks, t;
};

template <bool F16>
__device__ __forceinline__ Row8 shared_row8(const RoutedRows &rr, uint32_t row, uint32_t d, uint32_t chunk) {
    Row8 out;
#pragma unroll
    for (int i = 0; i < 8; ++i) out.v[i] = 0.0f;
    f32x4 lo[4], hi[4];
#pragma unroll
    for (uint32_t c = 0; c < 4; ++c) {
        const float *src = rr.shared_partials + ((size_t)min(c, rr.shared_chunks - 1) * rr.t + row) * d + 8 * chunk;
        lo[c] = *reinterpret_cast<const f32x4 *>(src);
        hi[c] = *reinterpret_cast<const f32x4 *>(src + 4);
    }
#pragma unroll
    for (uint32_t c = 0; c < 4; ++c) {
        if (c < rr.shared_chunks) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                out.v[i] += lo[c][i];
                out.v[4 + i] += hi[c][i];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out.v[i] = round16<F16>(out.v[i]);
    return out;
}

template <bool F16>
__device__ __forceinline__ Row8 combine8(const RoutedRows &rr, uint32_t row, uint32_t d, uint32_t chunk) {
    float wv[8];
    uint32_t valid[8];
    f32x4 lo[8], hi[8];
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        const uint32_t route = row * rr.top_k + min(r, rr.top_k - 1);
        wv[r] = Act<F16>::widen(rr.w[route]);
        valid[r] = rr.route_valid[route];
        const float *src = rr.partials + (size_t)route * d + 8 * chunk;
        lo[r] = *reinterpret_cast<const f32x4 *>(src);
        hi[r] = *reinterpret_cast<const f32x4 *>(src + 4);
    }
    Row8 out;
#pragma unroll
    for (int i = 0; i < 8; ++i) out.v[i] = 0.0f;
#pragma unroll
    for (uint32_t r = 0; r < 8; ++r) {
        if (r < rr.top_k && valid[r] != 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                out.v[i] = __builtin_fmaf(wv[r], lo[r][i], out.v[i]);
                out.v[4 + i] = __builtin_fmaf(wv[r], hi[r][i], out.v[4 + i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out.v[i] = round16<F16>(out.v[i]);
    return out;
}

// NORMS: h1 arrives before its own norm (w_postffn1) and, when w_next is given, the norm of the new hidden
// row under w_next goes to `normed` (the next layer's input norm): fused_layer_tail_norms
// (Kernels/Fusions/FusedLayerTail.swift:74-117). h1 itself is left as it was found.
template <bool VEC, bool NORMS, bool F16, bool COMBINE = false>
__global__ __launch_bounds__(kRowThreads) void layer_tail_kernel(const uint16_t *__restrict__ h2, uint32_t h2_stride,
                                                                 const uint16_t *__restrict__ h1, uint32_t h1_stride,
                                                                 uint16_t *__restrict__ hidden, uint32_t hidden_stride,
                                                                 const uint16_t *__restrict__ w_postffn2,
                                                                 const uint16_t *__restrict__ w_postffn, uint32_t d,
                                                                 float eps, float layer_scalar,
                                                                 const uint16_t *__restrict__ w_postffn1,
                                                                 const uint16_t *__restrict__ w_next,
                                                                 uint16_t *__restrict__ normed, uint32_t normed_stride,
                                                                 RoutedRows routed) {
    __shared__ float s_sum[4][4];
    const uint32_t row = blockIdx.x, t = threadIdx.x, chunks = d / 8;
    const uint32_t n_mine = t < chunks ? (chunks - t + kRowThreads - 1) / kRowThreads : 0;
    uint16_t *hrow = hidden + (size_t)row * hidden_stride;
    Row8 a[kMaxChunks], h12[kMaxChunks], hv[kMaxChunks], wf1[kMaxChunks], wf2[kMaxChunks], wf[kMaxChunks], wn[kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
            if (!COMBINE) a[c] = load8<VEC, F16>(h2 + (size_t)row * h2_stride, chunk);
            if (!COMBINE || !routed.shared_partials) h12[c] = load8<VEC, F16>(h1 + (size_t)row * h1_stride, chunk);
            hv[c] = load8<VEC, F16>(hrow, chunk);
            wf2[c] = loadw8<VEC>(w_postffn2, chunk);
            wf[c] = loadw8<VEC>(w_postffn, chunk);
            if (NORMS) wf1[c] = loadw8<VEC>(w_postffn1, chunk);
            if (NORMS && w_next) wn[c] = loadw8<VEC>(w_next, chunk);
        }
    if (COMBINE) {
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c)
            if ((uint32_t)c < n_mine) {
                a[c] = combine8<F16>(routed, row, d, t + c * kRowThreads);
                if (routed.shared_partials) h12[c] = shared_row8<F16>(routed, row, d, t + c * kRowThreads);
            }
    }
    if (NORMS) {
        const float inv_h1 = block_rms_inv(h12, n_mine, d, eps, s_sum[2]);
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c)
            if ((uint32_t)c < n_mine) {
#pragma unroll
                for (int e = 0; e < 8; ++e) h12[c].v[e] = round16<F16>(h12[c].v[e] * inv_h1 * wf1[c].v[e]);
            }
    }
    const float inv_h2 = block_rms_inv(a, n_mine, d, eps, s_sum[0]);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
#pragma unroll
            for (int e = 0; e < 8; ++e) h12[c].v[e] = round16<F16>(h12[c].v[e] + round16<F16>(a[c].v[e] * inv_h2 * wf2[c].v[e]));
        }
    const float inv_h12 = block_rms_inv(h12, n_mine, d, eps, s_sum[1]);
    const float scale = round16<F16>(layer_scalar);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                hv[c].v[e] = round16<F16>(round16<F16>(hv[c].v[e] + round16<F16>(h12[c].v[e] * inv_h12 * wf[c].v[e])) * scale);
            store8<VEC, F16>(hrow, chunk, hv[c]);
            a[c] = hv[c];          // the new hidden row, as stored
        }
    if (NORMS && w_next) {
        const float inv_next = block_rms_inv(a, n_mine, d, eps, s_sum[3]);
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c)
            if ((uint32_t)c < n_mine) {
                const uint32_t chunk = t + c * kRowThreads;
                const Row8 &w = wn[c];
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
    Row8 a[kMaxChunks], wq[kMaxChunks];
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            a[c] = load8<VEC, F16>(x + (size_t)row * x_stride, t + c * kRowThreads);
            wq[c] = loadw8<VEC>(w, t + c * kRowThreads);
        }
    const float inv = block_rms_inv(a, n_mine, d, eps, s_sum);
#pragma unroll
    for (int c = 0; c < kMaxChunks; ++c)
        if ((uint32_t)c < n_mine) {
            const uint32_t chunk = t + c * kRowThreads;
            const Row8 &wv = wq[c];
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
                             const uint16_t *w_next, uint16_t *normed, uint32_t normed_stride, bool f16,
                             const float *routed_partials, const uint16_t *routed_w, const uint32_t *route_valid, uint32_t top_k,
                             const float *shared_partials, uint32_t shared_chunks) {
    const bool norms = w_postffn1 != nullptr;
    if (shared_partials && (!routed_partials || shared_chunks == 0 || shared_chunks > 4)) return hipErrorInvalidValue;
    const RoutedRows routed{routed_partials, routed_w, route_valid, top_k, shared_partials, shared_chunks, t};
    if (routed_partials) {
        // h2 is made from the un-combined rows (16-byte aligned fp32 rows: d % 8 == 0); the plain tail only
        const bool vec = (shared_partials || aligned16(h1, h1_stride)) && aligned16(hidden, hidden_stride) && aligned16(w_postffn2, 8) && aligned16(w_postffn, 8);
#define FFMOE_TAILC(V, H)                                                                                             \
    hipLaunchKernelGGL((layer_tail_kernel<V, false, H, true>), dim3(t), dim3(kRowThreads), 0, s, nullptr, 0u, h1, h1_stride, \
                       hidden, hidden_stride, w_postffn2, w_postffn, d, eps, layer_scalar, nullptr, nullptr, nullptr, 0u, routed)
        if (f16) { if (vec) FFMOE_TAILC(true, true); else FFMOE_TAILC(false, true); }
        else { if (vec) FFMOE_TAILC(true, false); else FFMOE_TAILC(false, false); }
#undef FFMOE_TAILC
        return hipGetLastError();
    }
    const bool vec = aligned16(h2, h2_stride) && aligned16(h1, h1_stride) && aligned16(hidden, hidden_stride) &&
                     aligned16(w_postffn2, 8) && aligned16(w_postffn, 8) &&
                     (!norms || (aligned16(w_postffn1, 8) && (!w_next || (aligned16(w_next, 8) && aligned16(normed, normed_stride)))));
#define FFMOE_TAIL(V, N)                                                                                              \
    do {                                                                                                              \
        if (f16)                                                                                                      \
            hipLaunchKernelGGL((layer_tail_kernel<V, N, true>), dim3(t), dim3(kRowThreads), 0, s, h2, h2_stride, h1, h1_stride, \
                               hidden, hidden_stride, w_postffn2, w_postffn, d, eps, layer_scalar, w_postffn1, w_next, normed, \
                               normed_stride, routed);                                                                \
        else                                                                                                          \
            hipLaunchKernelGGL((layer_tail_kernel<V, N, false>), dim3(t), dim3(kRowThreads), 0, s, h2, h2_stride, h1, h1_stride, \
                               hidden, hidden_stride, w_postffn2, w_postffn, d, eps, layer_scalar, w_postffn1, w_next, normed, \
                               normed_stride, routed);                                                                \
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
