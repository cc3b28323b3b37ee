/*
 * CPU oracle for the quantized-MoE hot path. TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement, from the reference's source text, of the
 * arithmetic the HIP kernels must reproduce. It is the checker for the tests,
 * for the smoke run and for the CPU-baseline leg of the benchmark; the
 * product library never links, loads or calls it.
 *
 * The reference (Swift 6.2 + Metal + Accelerate) cannot be compiled in this
 * image, so there is no oracle/_ref build; each function below cites the
 * reference file:line it follows, paths relative to the reference root.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   bf16/fp16 codecs      all 65,536 patterns round-trip; RNE ties; torch / numpy
 *                         casts as independent implementations
 *   nibble order          literal packed bytes from the layout comment
 *                         Metal/Quant/dequant_int4.metal:7-12 and pack4 in
 *                         PrefillGroupedRoutedMoETests+Execution.swift:129-131
 *   quantizer             QuantizationAffineTests.swift:7-26 known answer, exact
 *                         recovery of representable rows, constant groups
 *   dequant (fp32, bf16)  closed form on the adversarial scale/bias set of
 *                         MPPPrefillInt4QMMTests.swift:26-37, fp64 cross-check
 *   GEMV / int4 dot       one-hot and all-ones inputs, linearity, fp64 BLAS
 *   GELU-tanh             torch.nn.functional.gelu(approximate="tanh") in fp64
 *   top-8                 brute-force full sort (RouterTopKTests.swift:55-63),
 *                         ties, fewer than 8 finite scores, all-equal scores
 *   routing weights       softmax identities; sum and order
 *   pair build/group      exact arrays of PrefillMoEGroupingTests.swift and
 *                         PrefillRouterTests.swift:12-22
 *   FFN / layer           torch fp64 matmul over dequantized weights
 *   combine               one-hot weights reproduce the selected partial;
 *                         cpuReduce of PrefillMoETests.swift:46-64
 *   PRNG                  SplitMix64 published test vector (seed 1234567)
 *   setup / layer tail    fp64 restatement of RmsNormRef (Reference/Primitives/RmsNorm.swift)
 *                         composed as cpuReference of FusedLayerTailTests.swift:96-110;
 *                         unit weights make the three setup outputs equal; router_x has
 *                         unit RMS; zero attention leaves hidden untouched
 * The pinned-order router logits (ffo_router_logits_pinned) define a summation
 * order of this build, not of the reference (Apple's simd_sum order is
 * unspecified); they are checked against a fp64 dot within rounding noise.
 */
#ifndef FFMOE_ORACLE_H
#define FFMOE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FFO_GROUP 64

/* MoEExpertOffsets, Kernels/MoE/MoE.swift:4-29 (byte offsets inside one expert blob). */
typedef struct {
    uint32_t gate_w, gate_s, gate_b;
    uint32_t up_w, up_s, up_b;
    uint32_t down_w, down_s, down_b;
} ffo_offsets;

/* PrefillTokenExpertPair, Kernels/Prefill/MoE/PrefillRouter.swift:5-21. */
typedef struct {
    uint32_t token, expert, rank, weight_bits;
} ffo_pair;

enum { FFO_BF16 = 0, FFO_FP16 = 1, FFO_F32 = 2 };

/* --- codecs: Infrastructure/ModelIO/Quantization.swift:9-20 --- */
uint16_t ffo_bf16_bits(float x);
float    ffo_bf16_to_float(uint16_t b);
uint16_t ffo_fp16_bits(float x);
float    ffo_fp16_to_float(uint16_t h);
/* round a float through the 16-bit type `dtype` (FFO_F32 = identity) */
float    ffo_round16(float x, int dtype);
uint16_t ffo_bits16(float x, int dtype);
float    ffo_from_bits16(uint16_t b, int dtype);

/* --- PRNG: Tests/Support/Validation/PRNG/SplitMix64.swift:9-21, SeedTree.swift:12-19 --- */
uint64_t ffo_splitmix64_next(uint64_t *state);
float    ffo_splitmix64_uniform(uint64_t *state, float lo, float hi);
void     ffo_splitmix64_fill_uniform(uint64_t *state, float lo, float hi, float *out, size_t n);
uint64_t ffo_seedtree_key(uint64_t root, const char *label);

/* --- quantizers: Tests/Support/Validation/Reference/Quant/AffineQuantization.swift --- */
void ffo_quantize_int4_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases);
void ffo_dequantize_int4_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases,
                                int n, float *out);
/* bf16Bits(q*s + b): the 16-bit weight a matrix-unit tile holds
   (MPPPrefillInt4QMMTests.swift:190-192, Metal/TensorCore/tensorops.metal:267). */
void ffo_dequantize_int4_bf16(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases,
                              int n, uint16_t *out);
void ffo_quantize_int8_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases);
void ffo_dequantize_int8_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases,
                                int n, float *out);

/* --- GEMV: Reference/Quant/DequantInt4Gemv.swift:9-38 (dequantize the row, then dot) --- */
void ffo_gemv_int4_ref(const uint8_t *W, const uint16_t *S, const uint16_t *B, int m, int n,
                       const float *x, float *y);
/* cpuInt4Dot, PrefillGroupedRoutedMoETests.swift:153-178 */
float ffo_int4_dot(const uint8_t *bytes, size_t base, size_t w_off, size_t s_off, size_t b_off,
                   int row, int n, const float *x);

/* --- FFN: Reference/MoE/Moe.swift:13-78 --- */
float ffo_gelu_tanh(float x);
/* MoeRef.runFFN on one expert blob: down(gelu(gate x) * up x), all fp32. */
void ffo_run_ffn(const uint8_t *blob, const ffo_offsets *o, int d, int f, const float *x, float *out);
/* MoeRef.applyStreamedRouted: y = residual + sum_k w_k * ffn_{e_k}(x). blobs[k] = expert of slot k. */
void ffo_apply_streamed_routed(const uint8_t *const *blobs, const ffo_offsets *o, int d, int f,
                               const float *x, const float *residual, const float *routing_w, int top_k,
                               float *y);
/* cpuSyntheticRoutePartials, PrefillGroupedRoutedMoETests.swift:122-151: per sorted pair, int4-dot FFN,
   activation rounded to `dtype`, partial rounded to `dtype`, written at (token*topK+rank)*d.
   `out` holds 16-bit patterns (or f32 bit patterns reinterpretable when dtype == FFO_F32: then out is float*). */
void ffo_route_partials(const ffo_pair *pairs, size_t n_pairs, const uint8_t *pool, size_t stride,
                        const ffo_offsets *o, const uint16_t *hidden, size_t hidden_stride, int top_k,
                        int d, int f, int dtype, void *out, int n_threads);

/* --- combine: Metal/Prefill/prefill.metal:544-565, PrefillMoETests.swift:46-64 --- */
void ffo_reduce_token_major(const void *partials, int partial_dtype, const uint16_t *weights, int dtype,
                            int t, int top_k, int d, uint16_t *h2);

/* --- router --- */
/* logits with this build's pinned summation order (see file header). W is bf16 bits [E][D] when
   w_is_f32 == 0, else float [E][D]. es = bf16 effective scale [D] or NULL. */
void ffo_router_logits_pinned(const void *W, int w_is_f32, const uint16_t *x, int x_dtype,
                              const uint16_t *es, int e, int d, float *logits);
/* Metal/MoE/moe.metal:269-319 (serial insertion top-8 + softmax); per_expert_scale bf16 [E] or NULL. */
void ffo_topk_softmax(const float *logits, int e, int top_k, const uint16_t *per_expert_scale,
                      uint32_t *idx, float *w);

/* --- whole layer, fp32 reference mode (no intermediate rounding except the routing weights, which
   are rounded to `dtype` as at moe.metal:235). x is `dtype` bits [T][x_stride]. y float [T][D]. --- */
void ffo_moe_layer(const uint8_t *pool, size_t stride, const ffo_offsets *o, int n_experts, int d, int f,
                   const uint16_t *router_w_bf16, const uint16_t *x, size_t x_stride, int t, int top_k,
                   int dtype, uint32_t *idx_out, float *w_out, float *y, int n_threads);
/* expert stage only, routes given: y[t] = sum_r w[t][r] * ffn_{idx[t][r]}(x[t]) */
void ffo_moe_experts(const uint8_t *pool, size_t stride, const ffo_offsets *o, int d, int f,
                     const uint16_t *x, size_t x_stride, int t, int top_k, int dtype,
                     const uint32_t *idx, const float *w, float *y, int n_threads);

/* --- steps either side of the MoE stage (summation order pinned by this build, see the .c file) ---
   Metal/Fusions/fused.metal:210-296, Metal/Prefill/prefill.metal:243-399. One row per call; 16-bit
   patterns of `dtype`, weights bf16 [d]; hidden is updated in place. d is a multiple of 8. */
void ffo_post_attn_setup(uint16_t *hidden, const uint16_t *attn, uint16_t *dense_x, uint16_t *routed_x,
                         uint16_t *router_x, const uint16_t *w_post_attn, const uint16_t *w_pre_ffn,
                         const uint16_t *w_pre_ffn2, int d, float eps, int dtype);
void ffo_rmsnorm(const uint16_t *x, const uint16_t *w, uint16_t *out, int d, float eps, int dtype);
void ffo_layer_tail(const uint16_t *h2, const uint16_t *h1, uint16_t *hidden, const uint16_t *w_postffn2,
                    const uint16_t *w_postffn, int d, float eps, float layer_scalar, int dtype);

int ffo_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
