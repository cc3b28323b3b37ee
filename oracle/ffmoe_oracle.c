/* CPU oracle for the quantized-MoE hot path: test infrastructure, never shipped or linked into the
 * product library. See ffmoe_oracle.h for the list of reference files followed and how each
 * function is pinned. Compile with -ffp-contract=off so that only the explicit fmaf calls fuse. */
#include "ffmoe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

/* Quantization.bf16Bits, Infrastructure/ModelIO/Quantization.swift:9-15: round half to even on the
 * dropped 16 bits, no NaN/Inf special case. */
uint16_t ffo_bf16_bits(float x) {
    uint32_t bits = f2u(x);
    uint32_t lsb = (bits >> 16) & 1u;
    uint32_t rounded = (bits + (0x7FFFu + lsb)) >> 16;
    return (uint16_t)rounded;
}

/* Quantization.bf16ToFloat, Quantization.swift:17-20 */
float ffo_bf16_to_float(uint16_t b) { return u2f((uint32_t)b << 16); }

/* IEEE binary16 encode, round to nearest even (what Swift's Float16(Float) and Metal's half(float)
 * do; the reference's text path is FP16, e.g. Metal/MoE/moe.metal:496). */
uint16_t ffo_fp16_bits(float x) {
    uint32_t u = f2u(x);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t exp = (u >> 23) & 0xFFu;
    uint32_t man = u & 0x7FFFFFu;
    if (exp == 0xFFu) return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0u));
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half & 1u))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

float ffo_fp16_to_float(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        float v = (float)man * 0x1p-24f;
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7F800000u | (man << 13));
    return u2f(sign | ((exp - 15 + 127) << 23) | (man << 13));
}

float ffo_round16(float x, int dtype) {
    if (dtype == FFO_BF16) return ffo_bf16_to_float(ffo_bf16_bits(x));
    if (dtype == FFO_FP16) return ffo_fp16_to_float(ffo_fp16_bits(x));
    return x;
}
uint16_t ffo_bits16(float x, int dtype) { return dtype == FFO_FP16 ? ffo_fp16_bits(x) : ffo_bf16_bits(x); }
float ffo_from_bits16(uint16_t b, int dtype) { return dtype == FFO_FP16 ? ffo_fp16_to_float(b) : ffo_bf16_to_float(b); }

/* SplitMix64.next, Tests/Support/Validation/PRNG/SplitMix64.swift:9-15 */
uint64_t ffo_splitmix64_next(uint64_t *state) {
    *state += 0x9E3779B97F4A7C15ull;
    uint64_t z = *state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* SplitMix64.uniform, SplitMix64.swift:17-21: 24-bit mantissa, lo + (hi - lo) * u in Float. */
float ffo_splitmix64_uniform(uint64_t *state, float lo, float hi) {
    float u = (float)(ffo_splitmix64_next(state) >> 40) / (float)(1 << 24);
    return lo + (hi - lo) * u;
}

void ffo_splitmix64_fill_uniform(uint64_t *state, float lo, float hi, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = ffo_splitmix64_uniform(state, lo, hi);
}

/* SeedTree.key, Tests/Support/Validation/PRNG/SeedTree.swift:12-19: root ^ FNV-1a(label). */
uint64_t ffo_seedtree_key(uint64_t root, const char *label) {
    uint64_t h = 0xCBF29CE484222325ull;
    for (const unsigned char *p = (const unsigned char *)label; *p; ++p) {
        h ^= (uint64_t)*p;
        h *= 0x100000001B3ull;
    }
    return root ^ h;
}

/* Quantization.quantizeInt4Affine, AffineQuantization.swift:24-76. Swift's .rounded() is
 * round-half-away-from-zero, i.e. roundf. */
void ffo_quantize_int4_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    int n_groups = n / FFO_GROUP;
    memset(packed, 0, (size_t)n / 2);
    for (int g = 0; g < n_groups; ++g) {
        float wmin = INFINITY, wmax = -INFINITY;
        for (int k = 0; k < FFO_GROUP; ++k) {
            float w = row[g * FFO_GROUP + k];
            if (w < wmin) wmin = w;
            if (w > wmax) wmax = w;
        }
        float scale_f, bias_f;
        if (wmax == wmin) { scale_f = 1.0f; bias_f = wmin; }
        else { scale_f = (wmax - wmin) / 15.0f; bias_f = wmin; }
        uint16_t s_bits = ffo_bf16_bits(scale_f), b_bits = ffo_bf16_bits(bias_f);
        scales[g] = s_bits;
        biases[g] = b_bits;
        float scale = ffo_bf16_to_float(s_bits), bias = ffo_bf16_to_float(b_bits);
        float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
        for (int k = 0; k < FFO_GROUP; ++k) {
            float w = row[g * FFO_GROUP + k];
            int q = (int)roundf((w - bias) * inv);
            if (q < 0) q = 0;
            if (q > 15) q = 15;
            int byte_idx = g * (FFO_GROUP / 2) + k / 2;
            if ((k & 1) == 0) packed[byte_idx] = (uint8_t)((packed[byte_idx] & 0xF0) | q);
            else packed[byte_idx] = (uint8_t)((packed[byte_idx] & 0x0F) | (q << 4));
        }
    }
}

/* Quantization.dequantizeInt4Affine, AffineQuantization.swift:78-93: Float(q) * scale + bias. */
void ffo_dequantize_int4_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases,
                                int n, float *out) {
    int n_groups = n / FFO_GROUP;
    for (int g = 0; g < n_groups; ++g) {
        float scale = ffo_bf16_to_float(scales[g]), bias = ffo_bf16_to_float(biases[g]);
        for (int k = 0; k < FFO_GROUP; ++k) {
            uint8_t b = packed[g * (FFO_GROUP / 2) + k / 2];
            int nib = (k & 1) == 0 ? (b & 0x0F) : (b >> 4);
            float prod = (float)nib * scale;
            out[g * FFO_GROUP + k] = prod + bias;
        }
    }
}

void ffo_dequantize_int4_bf16(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases,
                              int n, uint16_t *out) {
    int n_groups = n / FFO_GROUP;
    for (int g = 0; g < n_groups; ++g) {
        float scale = ffo_bf16_to_float(scales[g]), bias = ffo_bf16_to_float(biases[g]);
        for (int k = 0; k < FFO_GROUP; ++k) {
            uint8_t b = packed[g * (FFO_GROUP / 2) + k / 2];
            int nib = (k & 1) == 0 ? (b & 0x0F) : (b >> 4);
            float prod = (float)nib * scale;
            out[g * FFO_GROUP + k] = ffo_bf16_bits(prod + bias);
        }
    }
}

/* Quantization.quantizeInt8Affine, AffineQuantization.swift:109-151 */
void ffo_quantize_int8_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    int n_groups = n / FFO_GROUP;
    for (int g = 0; g < n_groups; ++g) {
        float wmin = INFINITY, wmax = -INFINITY;
        for (int k = 0; k < FFO_GROUP; ++k) {
            float w = row[g * FFO_GROUP + k];
            if (w < wmin) wmin = w;
            if (w > wmax) wmax = w;
        }
        float scale_f, bias_f;
        if (wmax == wmin) { scale_f = 1.0f; bias_f = wmin; }
        else { scale_f = (wmax - wmin) / 255.0f; bias_f = wmin; }
        uint16_t s_bits = ffo_bf16_bits(scale_f), b_bits = ffo_bf16_bits(bias_f);
        scales[g] = s_bits;
        biases[g] = b_bits;
        float scale = ffo_bf16_to_float(s_bits), bias = ffo_bf16_to_float(b_bits);
        float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
        for (int k = 0; k < FFO_GROUP; ++k) {
            float w = row[g * FFO_GROUP + k];
            int q = (int)roundf((w - bias) * inv);
            if (q < 0) q = 0;
            if (q > 255) q = 255;
            packed[g * FFO_GROUP + k] = (uint8_t)q;
        }
    }
}

/* Quantization.dequantizeInt8Affine, AffineQuantization.swift:153-165 */
void ffo_dequantize_int8_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases,
                                int n, float *out) {
    int n_groups = n / FFO_GROUP;
    for (int g = 0; g < n_groups; ++g) {
        float scale = ffo_bf16_to_float(scales[g]), bias = ffo_bf16_to_float(biases[g]);
        for (int k = 0; k < FFO_GROUP; ++k) {
            float prod = (float)packed[g * FFO_GROUP + k] * scale;
            out[g * FFO_GROUP + k] = prod + bias;
        }
    }
}

/* DequantInt4GemvRef.apply, Reference/Quant/DequantInt4Gemv.swift:9-38. vDSP_dotpr is replaced by
 * a left-to-right fp32 loop (Accelerate's summation order is not published). */
void ffo_gemv_int4_ref(const uint8_t *W, const uint16_t *S, const uint16_t *B, int m, int n,
                       const float *x, float *y) {
    int n_groups = n / FFO_GROUP;
    float *w_row = (float *)malloc((size_t)n * sizeof(float));
    for (int row = 0; row < m; ++row) {
        ffo_dequantize_int4_affine(W + (size_t)row * (n / 2), S + (size_t)row * n_groups,
                                   B + (size_t)row * n_groups, n, w_row);
        float dot = 0.0f;
        for (int i = 0; i < n; ++i) { float p = w_row[i] * x[i]; dot += p; }
        y[row] = dot;
    }
    free(w_row);
}

static inline uint16_t read_u16(const uint8_t *bytes, size_t off) {
    return (uint16_t)(bytes[off] | ((uint16_t)bytes[off + 1] << 8));
}

/* cpuInt4Dot, PrefillGroupedRoutedMoETests.swift:153-178: acc += (q*scale + bias) * x[col]. */
float ffo_int4_dot(const uint8_t *bytes, size_t base, size_t w_off, size_t s_off, size_t b_off,
                   int row, int n, const float *x) {
    int groups = n / FFO_GROUP;
    size_t row_bytes = (size_t)n / 2;
    size_t w_row = base + w_off + (size_t)row * row_bytes;
    size_t s_row = base + s_off + (size_t)row * groups * 2;
    size_t b_row = base + b_off + (size_t)row * groups * 2;
    float acc = 0.0f;
    for (int g = 0; g < groups; ++g) {
        float scale = ffo_bf16_to_float(read_u16(bytes, s_row + (size_t)g * 2));
        float bias = ffo_bf16_to_float(read_u16(bytes, b_row + (size_t)g * 2));
        for (int k = 0; k < FFO_GROUP; ++k) {
            int col = g * FFO_GROUP + k;
            uint8_t packed = bytes[w_row + col / 2];
            float q = (k & 1) == 0 ? (float)(packed & 0x0F) : (float)(packed >> 4);
            float w = q * scale;
            w = w + bias;
            float p = w * x[col];
            acc += p;
        }
    }
    return acc;
}

/* MoeRef.geluTanh, Reference/MoE/Moe.swift:13-21 (no clamp; the Metal clamp at moe.metal:43-45 is a
 * no-op in fp32 because tanh saturates long before |inner| = 20). */
float ffo_gelu_tanh(float x) {
    const float c = 0.7978845608028654f, k = 0.044715f;
    float x3 = x * x;
    x3 = x3 * x;
    float t = k * x3;
    t = x + t;
    float inner = c * t;
    float th = tanhf(inner);
    float h = 0.5f * x;
    return h * (1.0f + th);
}

/* MoeRef.runFFN, Moe.swift:25-45 */
void ffo_run_ffn(const uint8_t *blob, const ffo_offsets *o, int d, int f, const float *x, float *out) {
    float *act = (float *)malloc((size_t)f * sizeof(float));
    for (int r = 0; r < f; ++r) {
        float g = ffo_int4_dot(blob, 0, o->gate_w, o->gate_s, o->gate_b, r, d, x);
        float u = ffo_int4_dot(blob, 0, o->up_w, o->up_s, o->up_b, r, d, x);
        act[r] = ffo_gelu_tanh(g) * u;
    }
    for (int r = 0; r < d; ++r) out[r] = ffo_int4_dot(blob, 0, o->down_w, o->down_s, o->down_b, r, f, act);
    free(act);
}

/* MoeRef.applyStreamedRouted, Moe.swift:49-78 */
void ffo_apply_streamed_routed(const uint8_t *const *blobs, const ffo_offsets *o, int d, int f,
                               const float *x, const float *residual, const float *routing_w, int top_k,
                               float *y) {
    float *out = (float *)malloc((size_t)d * sizeof(float));
    for (int i = 0; i < d; ++i) y[i] = residual ? residual[i] : 0.0f;
    for (int slot = 0; slot < top_k; ++slot) {
        ffo_run_ffn(blobs[slot], o, d, f, x, out);
        float w = routing_w[slot];
        for (int i = 0; i < d; ++i) { float s = out[i] * w; y[i] = y[i] + s; }
    }
    free(out);
}

/* cpuSyntheticRoutePartials, PrefillGroupedRoutedMoETests.swift:122-151 */
void ffo_route_partials(const ffo_pair *pairs, size_t n_pairs, const uint8_t *pool, size_t stride,
                        const ffo_offsets *o, const uint16_t *hidden, size_t hidden_stride, int top_k,
                        int d, int f, int dtype, void *out, int n_threads) {
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#else
    (void)n_threads;
#endif
    int in_dtype = dtype == FFO_F32 ? FFO_BF16 : dtype;
#pragma omp parallel
    {
        float *x = (float *)malloc((size_t)d * sizeof(float));
        float *act = (float *)malloc((size_t)f * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (long p = 0; p < (long)n_pairs; ++p) {
            const ffo_pair pr = pairs[p];
            size_t base = (size_t)pr.expert * stride;
            for (int i = 0; i < d; ++i)
                x[i] = ffo_from_bits16(hidden[(size_t)pr.token * hidden_stride + i], in_dtype);
            for (int r = 0; r < f; ++r) {
                float g = ffo_int4_dot(pool, base, o->gate_w, o->gate_s, o->gate_b, r, d, x);
                float u = ffo_int4_dot(pool, base, o->up_w, o->up_s, o->up_b, r, d, x);
                act[r] = ffo_round16(ffo_gelu_tanh(g) * u, dtype);
            }
            size_t out_base = ((size_t)pr.token * top_k + pr.rank) * d;
            for (int r = 0; r < d; ++r) {
                float v = ffo_int4_dot(pool, base, o->down_w, o->down_s, o->down_b, r, f, act);
                if (dtype == FFO_F32) ((float *)out)[out_base + r] = v;
                else ((uint16_t *)out)[out_base + r] = ffo_bits16(v, dtype);
            }
        }
        free(x);
        free(act);
    }
}

/* prefill_moe_reduce_token_major, Metal/Prefill/prefill.metal:544-565: fma over ranks in order, one
 * rounding at the end (the Swift cpuReduce at PrefillMoETests.swift:46-64 uses mul+add; both are
 * inside the 2e-3 bar of that test). */
void ffo_reduce_token_major(const void *partials, int partial_dtype, const uint16_t *weights, int dtype,
                            int t, int top_k, int d, uint16_t *h2) {
    for (int tok = 0; tok < t; ++tok) {
        for (int col = 0; col < d; ++col) {
            float acc = 0.0f;
            for (int r = 0; r < top_k; ++r) {
                size_t pi = ((size_t)tok * top_k + r) * d + col;
                float pv = partial_dtype == FFO_F32 ? ((const float *)partials)[pi]
                                                    : ffo_from_bits16(((const uint16_t *)partials)[pi], partial_dtype);
                acc = fmaf(ffo_from_bits16(weights[(size_t)tok * top_k + r], dtype), pv, acc);
            }
            h2[(size_t)tok * d + col] = ffo_bits16(acc, dtype);
        }
    }
}

/* Router logits in this build's pinned order: 64 lanes x 4 sub-accumulators; sub-accumulator s of
 * lane l owns k = 1024*i + 256*s + 4*l + j (j = 0..3) and accumulates with fmaf in increasing i, then
 * j; the lane's value is (sub0 + sub1) + (sub2 + sub3); a xor-butterfly (32,16,8,4,2,1) of plain adds
 * combines the 64 lane values. The input is x[k] * effective_scale[k] as at
 * Metal/MoE/moe.metal:96-97 (product of two bf16 values: exact in fp32). Mathematically the row dot
 * of moe.metal:65-103 with dequantized weights. */
void ffo_router_logits_pinned(const void *W, int w_is_f32, const uint16_t *x, int x_dtype,
                              const uint16_t *es, int e, int d, float *logits) {
    float *xe = (float *)malloc((size_t)d * sizeof(float));
    for (int k = 0; k < d; ++k) {
        float xv = ffo_from_bits16(x[k], x_dtype);
        xe[k] = es ? xv * ffo_bf16_to_float(es[k]) : xv;
    }
    int steps = (d + 1023) / 1024;
    for (int row = 0; row < e; ++row) {
        float p[64], q[64];
        for (int l = 0; l < 64; ++l) {
            float sub[4];
            for (int s = 0; s < 4; ++s) {
                float acc = 0.0f;
                for (int i = 0; i < steps; ++i) {
                    for (int j = 0; j < 4; ++j) {
                        int k = 1024 * i + 256 * s + 4 * l + j;
                        if (k >= d) continue;
                        float w = w_is_f32 ? ((const float *)W)[(size_t)row * d + k]
                                           : ffo_bf16_to_float(((const uint16_t *)W)[(size_t)row * d + k]);
                        acc = fmaf(w, xe[k], acc);
                    }
                }
                sub[s] = acc;
            }
            float lo = sub[0] + sub[1], hi = sub[2] + sub[3];
            p[l] = lo + hi;
        }
        for (int m = 32; m >= 1; m >>= 1) {
            for (int l = 0; l < 64; ++l) q[l] = p[l] + p[l ^ m];
            memcpy(p, q, sizeof(p));
        }
        logits[row] = p[0];
    }
    free(xe);
}

/* router_topk_select_k8, Metal/MoE/moe.metal:269-319 (generalised to top_k <= 64 as
 * Metal/Prefill/prefill.metal:499-541): serial insertion keeps (score desc, index asc); a score at
 * or below -inf, or NaN, is never taken; missing slots stay (index 0, -inf) and get weight 0.
 * Weights: exp(s_i - s_0) / sum, times per_expert_scale[e_i]; returned in fp32 (the caller rounds). */
void ffo_topk_softmax(const float *logits, int e, int top_k, const uint16_t *per_expert_scale,
                      uint32_t *idx, float *w) {
    float score[64];
    for (int i = 0; i < top_k; ++i) { idx[i] = 0; score[i] = -INFINITY; }
    for (int ex = 0; ex < e; ++ex) {
        float s = logits[ex];
        if (!(s > score[top_k - 1])) continue;
        int pos = top_k;
        for (int i = 0; i < top_k; ++i) {
            if (s > score[i] || (s == score[i] && (uint32_t)ex < idx[i])) { pos = i; break; }
        }
        if (pos >= top_k) continue;
        for (int i = top_k - 1; i > pos; --i) { idx[i] = idx[i - 1]; score[i] = score[i - 1]; }
        idx[pos] = (uint32_t)ex;
        score[pos] = s;
    }
    float max_s = score[0], sum = 0.0f, ex_[64];
    for (int i = 0; i < top_k; ++i) { ex_[i] = expf(score[i] - max_s); sum += ex_[i]; }
    for (int i = 0; i < top_k; ++i) {
        float weight = ex_[i] / sum;
        float gain = per_expert_scale ? ffo_bf16_to_float(per_expert_scale[idx[i]]) : 1.0f;
        w[i] = weight * gain;
    }
}

void ffo_moe_experts(const uint8_t *pool, size_t stride, const ffo_offsets *o, int d, int f,
                     const uint16_t *x, size_t x_stride, int t, int top_k, int dtype,
                     const uint32_t *idx, const float *w, float *y, int n_threads) {
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#else
    (void)n_threads;
#endif
    size_t n_pairs = (size_t)t * top_k;
    float *partials = (float *)malloc(n_pairs * d * sizeof(float));
#pragma omp parallel
    {
        float *xf = (float *)malloc((size_t)d * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (long p = 0; p < (long)n_pairs; ++p) {
            int tok = (int)(p / top_k);
            for (int i = 0; i < d; ++i) xf[i] = ffo_from_bits16(x[(size_t)tok * x_stride + i], dtype);
            ffo_run_ffn(pool + (size_t)idx[p] * stride, o, d, f, xf, partials + (size_t)p * d);
        }
        free(xf);
    }
    /* rank-ordered weighted sum, as Moe.swift:72-76 */
    for (int tok = 0; tok < t; ++tok) {
        for (int i = 0; i < d; ++i) {
            float acc = 0.0f;
            for (int r = 0; r < top_k; ++r) {
                float s = partials[((size_t)tok * top_k + r) * d + i] * w[(size_t)tok * top_k + r];
                acc = acc + s;
            }
            y[(size_t)tok * d + i] = acc;
        }
    }
    free(partials);
}

void ffo_moe_layer(const uint8_t *pool, size_t stride, const ffo_offsets *o, int n_experts, int d, int f,
                   const uint16_t *router_w_bf16, const uint16_t *x, size_t x_stride, int t, int top_k,
                   int dtype, uint32_t *idx_out, float *w_out, float *y, int n_threads) {
    float *logits = (float *)malloc((size_t)n_experts * sizeof(float));
    for (int tok = 0; tok < t; ++tok) {
        ffo_router_logits_pinned(router_w_bf16, 0, x + (size_t)tok * x_stride, dtype, NULL, n_experts, d, logits);
        ffo_topk_softmax(logits, n_experts, top_k, NULL, idx_out + (size_t)tok * top_k, w_out + (size_t)tok * top_k);
        for (int r = 0; r < top_k; ++r)
            w_out[(size_t)tok * top_k + r] = ffo_round16(w_out[(size_t)tok * top_k + r], dtype);
    }
    free(logits);
    ffo_moe_experts(pool, stride, o, d, f, x, x_stride, t, top_k, dtype, idx_out, w_out, y, n_threads);
}

/* --- the steps either side of the MoE stage: post-attention setup and layer tail ---
 * Row-wise RMS norms around residual adds. The reference reduces the squares with simd_sum, whose
 * order is unspecified; this build pins one: thread t of 256 owns the 8-element chunks t, t + 256, ...
 * and sums their squares in index order with fmaf; the 64 threads of a wave meet in a xor-butterfly
 * (32,16,8,4,2,1) of plain adds; the four wave sums combine as (w0 + w1) + (w2 + w3);
 * inv = 1 / sqrt(sum / D + eps) with IEEE division and square root. d is a multiple of 8. */
static float rms_inv_pinned(const float *x, int d, float eps) {
    float lane[256];
    const int chunks = d / 8;
    for (int t = 0; t < 256; ++t) {
        float acc = 0.0f;
        for (int c = t; c < chunks; c += 256)
            for (int e = 0; e < 8; ++e) acc = fmaf(x[8 * c + e], x[8 * c + e], acc);
        lane[t] = acc;
    }
    float wave[4];
    for (int w = 0; w < 4; ++w) {
        float v[64];
        memcpy(v, lane + 64 * w, sizeof v);
        for (int m = 32; m >= 1; m >>= 1) {
            float nv[64];
            for (int l = 0; l < 64; ++l) nv[l] = v[l] + v[l ^ m];
            memcpy(v, nv, sizeof v);
        }
        wave[w] = v[0];
    }
    const float total = (wave[0] + wave[1]) + (wave[2] + wave[3]);
    return 1.0f / sqrtf(total / (float)d + eps);
}

/* fused_post_attn_setup (Metal/Fusions/fused.metal:210-296) = one row of prefill_post_attn_setup_block
 * (Metal/Prefill/prefill.metal:243-318): attn = norm(attn, w_post_attn) rounded; hidden += attn, rounded,
 * in place; from the norm of that hidden: dense_x (w_pre_ffn), routed_x (w_pre_ffn2), router_x (no weight). */
void ffo_post_attn_setup(uint16_t *hidden, const uint16_t *attn, uint16_t *dense_x, uint16_t *routed_x,
                         uint16_t *router_x, const uint16_t *w_post_attn, const uint16_t *w_pre_ffn,
                         const uint16_t *w_pre_ffn2, int d, float eps, int dtype) {
    float *a = (float *)calloc((size_t)d, sizeof(float)), *h = (float *)calloc((size_t)d, sizeof(float));
    for (int i = 0; i < d; ++i) a[i] = ffo_from_bits16(attn[i], dtype);
    const float attn_inv = rms_inv_pinned(a, d, eps);
    for (int i = 0; i < d; ++i) {
        const float an = ffo_round16(a[i] * attn_inv * ffo_bf16_to_float(w_post_attn[i]), dtype);
        hidden[i] = ffo_bits16(ffo_from_bits16(hidden[i], dtype) + an, dtype);
        h[i] = ffo_from_bits16(hidden[i], dtype);
    }
    const float hidden_inv = rms_inv_pinned(h, d, eps);
    for (int i = 0; i < d; ++i) {
        const float v = h[i] * hidden_inv;
        dense_x[i] = ffo_bits16(v * ffo_bf16_to_float(w_pre_ffn[i]), dtype);
        routed_x[i] = ffo_bits16(v * ffo_bf16_to_float(w_pre_ffn2[i]), dtype);
        router_x[i] = ffo_bits16(v, dtype);
    }
    free(a);
    free(h);
}

/* rmsnorm_bf16w (Metal/Norms/rmsnorm.metal; RMSNorm.encodeBF16W): out = r((x * inv) * w), one row. */
void ffo_rmsnorm(const uint16_t *x, const uint16_t *w, uint16_t *out, int d, float eps, int dtype) {
    float *a = (float *)calloc((size_t)d, sizeof(float));
    for (int i = 0; i < d; ++i) a[i] = ffo_from_bits16(x[i], dtype);
    const float inv = rms_inv_pinned(a, d, eps);
    for (int i = 0; i < d; ++i) out[i] = ffo_bits16(a[i] * inv * ffo_bf16_to_float(w[i]), dtype);
    free(a);
}

/* fused layer tail = one row of prefill_layer_tail_block (Metal/Prefill/prefill.metal:320-399), the
 * arithmetic of cpuReference in FusedLayerTailTests.swift:96-110: h12 = r(h1 + r(norm(h2, w_postffn2)));
 * hidden = r(r(hidden + r(norm(h12, w_postffn))) * r(layer_scalar)), every r a rounding to 16 bits. */
void ffo_layer_tail(const uint16_t *h2, const uint16_t *h1, uint16_t *hidden, const uint16_t *w_postffn2,
                    const uint16_t *w_postffn, int d, float eps, float layer_scalar, int dtype) {
    float *a = (float *)calloc((size_t)d, sizeof(float)), *h12 = (float *)calloc((size_t)d, sizeof(float));
    for (int i = 0; i < d; ++i) a[i] = ffo_from_bits16(h2[i], dtype);
    const float inv_h2 = rms_inv_pinned(a, d, eps);
    for (int i = 0; i < d; ++i) {
        const float tmp = ffo_round16(a[i] * inv_h2 * ffo_bf16_to_float(w_postffn2[i]), dtype);
        h12[i] = ffo_round16(ffo_from_bits16(h1[i], dtype) + tmp, dtype);
    }
    const float inv_h12 = rms_inv_pinned(h12, d, eps);
    const float scale = ffo_round16(layer_scalar, dtype);
    for (int i = 0; i < d; ++i) {
        const float tmp = ffo_round16(h12[i] * inv_h12 * ffo_bf16_to_float(w_postffn[i]), dtype);
        const float sum = ffo_round16(ffo_from_bits16(hidden[i], dtype) + tmp, dtype);
        hidden[i] = ffo_bits16(sum * scale, dtype);
    }
    free(a);
    free(h12);
}

int ffo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
