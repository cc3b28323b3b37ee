/*
 * fieldfare_moe.h - C ABI of libfieldfare_moe_hip.so: the quantized-MoE hot path of
 * zw5/ane-fieldfare (router top-8 -> INT4 gate/up + GELU-tanh -> INT4 down -> weighted combine,
 * plus the generic INT4 GEMV) as hand-written CDNA4 (gfx950) HIP kernels.
 *
 * Conventions (modelled on Sources/ANEFieldfareANECarrier/include/ANEExpertCarrier.h:14-38 and on
 * the "encode" methods of the Swift operators this replaces):
 *   - every compute call ENQUEUES work on the caller's HIP stream (`stream` is a hipStream_t passed
 *     as void*, NULL = the default stream), returns without waiting, and allocates nothing; the
 *     stream plays the part of the reference's MTLCommandBuffer;
 *   - device buffers are caller-owned raw device pointers; scratch lives in the context and serves one stream at
 *     a time: a call that arrives on another stream than the context's previous call first makes its stream wait
 *     (on the device, hipStreamWaitEvent) for what the previous stream was given, so two streams that share a
 *     context run its calls one after the other instead of racing for the scratch; streams under graph capture
 *     are left alone (a capture orders its own nodes). The caller's own buffers are the caller's to order;
 *   - return value: FFMOE_OK (0) or a negative status; when `err` is non-NULL and the call fails,
 *     `*err` receives a strdup'd message the caller releases with free();
 *   - a context belongs to one host thread at a time (the reference's operators are not Sendable).
 * Activations, routing weights and outputs are 16-bit, all of one type per context: bf16 (FFMOE_BF16, the
 * default and the type the benchmark configurations name) or FP16 (FFMOE_FP16, the reference's text-path
 * type, Metal/MoE/moe.metal:69,389,555); see ffmoe_set_activation_dtype. Accumulation is fp32 in both.
 * All paths below are relative to the reference repository root.
 */
#ifndef FIELDFARE_MOE_H
#define FIELDFARE_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    FFMOE_OK = 0,
    FFMOE_ERR_INVALID = -1,   /* shape or argument misuse (a Swift precondition in the reference) */
    FFMOE_ERR_RUNTIME = -2,   /* HIP runtime failure (MetalError / command-buffer error in the reference) */
    FFMOE_ERR_ALLOC = -3,     /* PrefillGroupedRoutedMoEError.allocationFailed */
    FFMOE_ERR_NO_LAYER = -4   /* layer not uploaded */
};

enum { FFMOE_BF16 = 0, FFMOE_FP16 = 1 };

enum { FFMOE_GATE = 0, FFMOE_UP = 1, FFMOE_DOWN = 2 };

#define FFMOE_GROUP 64          /* Quantization.groupSize, Infrastructure/ModelIO/Quantization.swift:2 */
#define FFMOE_MAX_VERIFY_ROWS 16 /* maxVerifyTokens, Runtime/Inference/RealForwardRunner.swift:414 */
#define FFMOE_MAX_EXPERTS 256    /* router limit, Kernels/MoE/MoE.swift:137 */
#define FFMOE_PREFILL_TILE_M 256 /* pairs per M-tile of the prefill GEMMs (the role of groupTokenExpertPairs' tileM,
                                    Kernels/Prefill/MoE/PrefillMoEGrouping.swift:49); ffmoe_prefill_plan_stats counts these */

typedef struct ffmoe_ctx ffmoe_ctx;

/* Model shape of the routed-expert stage. Replaces the Metal function constants of
 * Kernels/MoE/MoE.swift:34-46 (D = 2816, F = 704, top-k = 8, 128 experts for Gemma-4-26B-A4B). */
typedef struct {
    uint32_t d;            /* hidden size, multiple of 64 */
    uint32_t f;            /* routed intermediate size, multiple of 64 */
    uint32_t n_experts;    /* <= FFMOE_MAX_EXPERTS */
    uint32_t top_k;        /* 1..8; the decode/verify kernels of the reference require 8 */
    uint32_t n_layers;     /* layers the HBM expert arena holds */
    uint32_t max_tokens;   /* largest T of a prefill call (PrefillRuntimeConfig.maxChunkTokens = 4096) */
} ffmoe_shape;

/* Byte offsets of the nine sub-tensors inside one expert blob.
 * Replaces MoEExpertOffsets, Kernels/MoE/MoE.swift:4-29. */
typedef struct {
    uint32_t gate_w, gate_s, gate_b;
    uint32_t up_w, up_s, up_b;
    uint32_t down_w, down_s, down_b;
} ffmoe_offsets;

/* One routed (token, expert) pair, 16 bytes.
 * Replaces PrefillTokenExpertPair, Kernels/Prefill/MoE/PrefillRouter.swift:5-21. */
typedef struct {
    uint32_t token, expert, rank, weight_bits_and_reserved;
} ffmoe_pair;

/* ---- lifetime -------------------------------------------------------------------------------- */

/* Creates the context on HIP device `device`: the HBM expert arena for `n_layers` layers and all
 * scratch. Replaces the operator constructors MoE.init / PrefillGroupedRoutedMoE.init
 * (Kernels/MoE/MoE.swift:72-123, Kernels/Prefill/MoE/PrefillGroupedRoutedMoE.swift:208-241). */
int ffmoe_create(int device, const ffmoe_shape *shape, ffmoe_ctx **out, char **err);
void ffmoe_destroy(ffmoe_ctx *ctx);

/* Bytes of HBM one layer's experts occupy in the arena (= n_experts * payload). */
size_t ffmoe_layer_arena_bytes(const ffmoe_ctx *ctx);

/* ---- weights --------------------------------------------------------------------------------- */

/* Copies one layer's expert blobs (reference byte layout: `n_experts` blobs `stride` bytes apart
 * starting at `blobs`, sub-tensors at `offsets`) into the HBM arena, re-tiled for the MFMA kernels.
 * `blobs` is host memory (e.g. the mmap of a layer file) when `src_is_device` == 0, else a device
 * pointer. Blocks until the copy is done. Replaces MappedExpertLayer + the per-expert MTLBuffer
 * binding (Infrastructure/Streaming/MappedExpertLayer.swift:118-128) and makeReusedRoutedArgumentBuffer
 * (Kernels/MoE/MoE.swift:302-310): with every expert resident, slots are base + expert * stride. */
int ffmoe_upload_layer(ffmoe_ctx *ctx, uint32_t layer, const void *blobs, size_t stride,
                       const ffmoe_offsets *offsets, int src_is_device, char **err);

/* Router weights of one layer: bf16 [n_experts][d] (the benchmark configs' form). Optional bf16
 * `effective_scale` [d] and `per_expert_scale` [n_experts] (NULL = 1), host pointers.
 * Replaces the router tensors bound by MoE.encodeRouterGemma4 (Kernels/MoE/MoE.swift:168-180). */
int ffmoe_upload_router_bf16(ffmoe_ctx *ctx, uint32_t layer, const uint16_t *w,
                             const uint16_t *effective_scale, const uint16_t *per_expert_scale, char **err);
/* Same for the reference's INT8-affine router (uint8 [E][d] + bf16 scale/bias per 64,
 * Metal/MoE/moe.metal:65-103): dequantised once to fp32(q*s + b) at upload. */
int ffmoe_upload_router_int8(ffmoe_ctx *ctx, uint32_t layer, const uint8_t *w, const uint16_t *scales,
                             const uint16_t *biases, const uint16_t *effective_scale,
                             const uint16_t *per_expert_scale, char **err);

/* Expands one sub-tensor (FFMOE_GATE / UP / DOWN) of one expert from the arena to bf16
 * [rows][cols], each element bf16(q*scale + bias) - the value a matrix-unit tile holds. Replaces
 * ane_expert_weights (Metal/ANE/ane_prefill.metal:17-36) as the exact-expansion check
 * (Tests/ANEFieldfareHotpathTests/ANEQuantizedCarrierTests.swift:59-67). */
int ffmoe_dequant_expert(ffmoe_ctx *ctx, void *stream, uint32_t layer, uint32_t expert, int which,
                         uint16_t *out_bf16, char **err);

/* Test hook for the grouped GEMM of ffmoe_prefill: runs one pair of `expert` through the gate/up (gate_up != 0) or
 * the down GEMM and copies out every weight fragment exactly as the matrix instructions read it from LDS:
 * out[N-block][group][fragment 0..15][lane 0..63] x 8 bf16, where an N-block is four 32-row arena tiles, fragment u is
 * arena tile (u % 8) / 2 of the N-block, stream u % 2 (gate / up rows 16 * tile + r; down rows 32 * tile + 16 * stream + r),
 * k-half u / 8, and lane l holds row r = l % 16 at k = 64 * group + 32 * (u / 8) + 8 * (l / 16) .. + 7. Tiles past the last
 * arena tile repeat the last one. The 16-bit tile weight is what "bit-exact dequantized weights" is a property of
 * (Tests/ANEFieldfareUpstreamTests/Kernels/TensorCore/MPPPrefillInt4QMMTests.swift:26-37,190-192 hold the Metal tile to
 * bfloat(fma(q, s, b)) the same way). out_bytes >= ceil(tiles / 4) * groups * 16 KiB. */
int ffmoe_prefill_dump_tiles(ffmoe_ctx *ctx, void *stream, uint32_t layer, uint32_t expert, int gate_up, void *out,
                             size_t out_bytes, char **err);

/* ---- router ---------------------------------------------------------------------------------- */

/* logits = W_router . (router_x * effective_scale); top-k by (score desc, index asc); weights =
 * softmax over the selected scores * per_expert_scale, rounded to bf16. `router_x` is bf16
 * [t][x_stride]. Writes out_idx uint32 [t][top_k] and out_w bf16 [t][top_k]; out_logits (fp32
 * [t][n_experts]) may be NULL. Replaces MoE.encodeRouterGemma4 (Kernels/MoE/MoE.swift:168-237),
 * MoE.encodeRouterRowsGemma4 (:249-300) and PrefillRouter.encodeGemma4Block
 * (Kernels/Prefill/MoE/PrefillRouter.swift:30-73). */
int ffmoe_router(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *router_x,
                 uint32_t x_stride, uint32_t t, uint32_t *out_idx, uint16_t *out_w, float *out_logits,
                 char **err);

/* ---- routed experts, decode and verify block (t <= 16) ---------------------------------------- */

/* y[t] = bf16(residual[t] + sum_r w[t][r] * down_e(gelu_tanh(gate_e x[t]) * up_e x[t])), e = idx[t][r].
 * Tokens that share an expert are batched against one read of its weights. `x` bf16 [t][x_stride],
 * `idx` uint32 [t][top_k], `w` bf16 [t][top_k], `residual` bf16 [t][d] or NULL, `y` bf16 [t][d]; all
 * device pointers. t == 1 replaces MoE.encodeRoutedPersistentPhase1U16Load + ...Phase2Reduce and
 * encodeGatherRoutedSlots / encodeRoutedPersistentGPUSlots (Kernels/MoE/MoE.swift:312-496); t <= 16
 * replaces PrefillGroupedRoutedMoE.encodeVerifyBound / encodeVerifyRows
 * (Kernels/Prefill/MoE/PrefillGroupedRoutedMoE.swift:331-448) followed by
 * PrefillMoE.encodeReduceTokenMajor. Routes whose weight is exactly zero are skipped. A row names an expert at most
 * once in the reference (top-k selects distinct experts); should a table name one expert more than 16 times in all,
 * its first 16 routes in [row][rank] order take part and the others add nothing. */
int ffmoe_verify(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                 uint32_t t, const uint32_t *idx, const uint16_t *w, const uint16_t *residual,
                 uint16_t *y, char **err);

/* ffmoe_verify for callers that cannot allocate or free device memory around the call: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. Same
 * arguments, same kernels and bit-identical results; its scratch (route plan, activation rows, un-weighted fp32
 * rows) is a fixed array inside the library image instead of the context's allocations, and the call itself
 * allocates nothing. Limit: 32 KiB + 16 * top_k * (2 f + 4 d) bytes must fit FFMOE_STATIC_SCRATCH_BYTES (3 MiB; the
 * reference model takes 1.6 MiB); larger shapes are refused with FFMOE_ERR_INVALID. Every GPU holds one such array
 * for the life of the process, shared by all contexts and calls on that GPU. Calls from one host thread on different
 * streams are ordered like a context's own (the stream of a later call waits, on the device, for the stream of the
 * earlier one; no allocation: the event exists since the library looked the array's address up); calls that overlap
 * from two host threads, or under graph capture, race on it. ffmoe_last_live_experts does not see these calls. */
#define FFMOE_STATIC_SCRATCH_BYTES (3u << 20)
int ffmoe_verify_static(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                        uint32_t t, const uint32_t *idx, const uint16_t *w, const uint16_t *residual,
                        uint16_t *y, char **err);

/* Same expert pass, but writes the un-weighted per-route rows bf16 partials[(token*top_k+rank)*d ...]
 * the way the reference's verify and prefill kernels hand them to the reduce
 * (Metal/Prefill/prefill.metal:1372-1374, Runtime/Supervisor/DeviceSupervisor.swift:14-17). */
int ffmoe_verify_partials(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x,
                          uint32_t x_stride, uint32_t t, const uint32_t *idx, const uint16_t *w,
                          uint16_t *partials, char **err);

/* Router and expert pass of one block in one call, for the decode loop that never shows the routes to
 * the host: the results of ffmoe_router followed by ffmoe_verify on the same stream, bit for bit, with the
 * selected routes also written to out_idx / out_w ([t][top_k], device). Replaces the pair
 * MoE.encodeRouterGemma4 + encodeRoutedPersistentGPUSlots (Kernels/MoE/MoE.swift:168-247,454-496), where
 * the GPU routes the persistent kernels without a host round trip.
 * When the expert fits the persistent kernels and the router rows are 8-byte aligned, the router logits, the
 * select and gate/up run as ONE launch (a decode step is two launches, a verify block three): the blocks
 * hand logits and routes to each other through epoch-stamped words in device memory. That is fast when every
 * block of the launch is resident at once - the grid is sized from the kernel's occupancy on a GPU this stream has
 * to itself - and correct either way: a wave that has waited FFMOE_DEFAULT_HANDOVER_TICKS for a word (other work
 * on the GPU keeps the block that makes it from running) stops waiting and computes what it waited for itself,
 * with the same arithmetic in the same order, so the call returns the same routes and rows, only later.
 * ffmoe_handover_giveups counts such waves.
 * y may be NULL (residual then too): the call ends with the down projection and leaves the routes' un-weighted fp32
 * rows in the context, for ffmoe_layer_tail_routed to combine in its load stage (one launch and one pass over the
 * rows less per layer); out_idx / out_w are written as usual. */
int ffmoe_route_verify(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *router_x,
                       uint32_t router_x_stride, const uint16_t *x, uint32_t x_stride, uint32_t t,
                       const uint16_t *residual, uint16_t *y, uint32_t *out_idx, uint16_t *out_w, char **err);

/* How long a wave of ffmoe_route_verify's one-launch form waits for a hand-over word before it computes the word's
 * content itself, in ticks of the GPU's constant 100 MHz clock (default FFMOE_DEFAULT_HANDOVER_TICKS = 1 ms); also
 * clears the count of waves that stopped waiting. Waits for the stream. No counterpart in the reference. The tests
 * set 0, which sends every wave that does not find its words at once down the self-sufficient path. */
#define FFMOE_DEFAULT_HANDOVER_TICKS 100000ull
int ffmoe_set_handover_timeout(ffmoe_ctx *ctx, void *stream, uint64_t ticks, char **err);

/* enabled = 0: ffmoe_route_verify runs the router as launches of its own in front of the expert pass (five launches
 * for a verify block, four for a decode step; same results bit for bit), in which no block waits for another: the
 * faster form for a host whose other streams or processes keep compute units of this GPU busy, where the one-launch
 * form's waves would wait out their bound before they help themselves. enabled != 0 (the default) restores the
 * one-launch form. Host state, takes effect with the next call. No counterpart in the reference. */
int ffmoe_set_one_launch_routing(ffmoe_ctx *ctx, int enabled, char **err);

/* Measurement hook, no counterpart in the reference: issues exactly the weight loads (tiles and scales) of the
 * decode / verify gate/up and down kernels for `n_live` experts of `layer` (spread over the layer's experts), in
 * those kernels' grids and order, with no routing, no token rows, no arithmetic and no output. Two launches; what
 * they take is what the memory system gives this access pattern, i.e. the ceiling the expert pass can be held
 * against (with ffmoe_set_profiling: slots FFMOE_K_PROBE_GATE_UP / FFMOE_K_PROBE_DOWN). 1 <= n_live <= n_experts;
 * needs a shape that fits the persistent kernels (d <= 2816, f <= 704). */
int ffmoe_probe_stream(ffmoe_ctx *ctx, void *stream, uint32_t layer, uint32_t n_live, char **err);

/* Number of distinct experts the last ffmoe_verify* call on `stream` ran (reads back 4 bytes; waits
 * for the stream). For reporting only. */
int ffmoe_last_live_experts(ffmoe_ctx *ctx, void *stream, uint32_t *n_live, char **err);

/* Waves of ffmoe_route_verify's one-launch form that stopped waiting for a hand-over word and computed it themselves,
 * since the context was created or ffmoe_set_handover_timeout was last called (reads back 4 bytes; waits for the
 * stream). The results of such calls are correct; a count that keeps growing says the GPU is shared and
 * ffmoe_set_one_launch_routing(ctx, 0) would serve this host better. No counterpart in the reference. */
int ffmoe_handover_giveups(ffmoe_ctx *ctx, void *stream, uint32_t *count, char **err);

/* ---- routed experts, prefill chunk (t <= max_tokens) ------------------------------------------- */

/* y[t] = bf16(sum_r w[t][r] * partial[t][r]) with partial = bf16(down_e(gelu_tanh(gate_e x[t]) * up_e x[t])),
 * e = idx[t][r], for a whole prefill chunk: the routes are sorted by expert ON THE GPU (no read-back of
 * the router output), each expert's pairs run as M-tiles of a grouped GEMM on the matrix units with
 * INT4 -> bf16 tiles dequantised into LDS, and the per-route rows are combined in rank order. Routes
 * whose weight is exactly zero are dropped. Replaces makeTokenExpertPairs + groupTokenExpertPairs
 * (Kernels/Prefill/MoE/PrefillRouter.swift:75-95, PrefillMoEGrouping.swift:49-110),
 * PrefillGroupedRoutedMoE.encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:275-326) and
 * PrefillMoE.encodeReduceTokenMajor, i.e. RealForwardRunner.swift:1520-1599 without the host wait. */
int ffmoe_prefill(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                  uint32_t t, const uint32_t *idx, const uint16_t *w, uint16_t *y, char **err);

/* The guest contract of RoutedPrefillGuest.runLayer (Runtime/Supervisor/DeviceSupervisor.swift:14-22):
 * for every pair of `pairs` (device array, any order; the reference passes them expert-sorted) write
 * the UN-weighted row bf16 partials[(token * top_k + rank) * d ...]; rows of other routes are left
 * untouched (the host zeroes `partials` first, RealForwardRunner.swift:1502-1506). `partials` is
 * 16-byte aligned. Replaces ANERoutedPrefillBackend.runLayer
 * (Runtime/Inference/ANERoutedPrefillBackend.swift:348-427). */
int ffmoe_prefill_pairs(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                        const ffmoe_pair *pairs, uint32_t n_pairs, uint32_t t, uint16_t *partials, char **err);

/* Pairs kept and M-tiles run by the last prefill call on `stream`, and pairs per expert (`counts`,
 * n_experts entries, may be NULL). Waits for the stream. For reporting (the reference's
 * prefillRouted* counters, RealForwardRunner.swift:171-203). */
int ffmoe_prefill_plan_stats(ffmoe_ctx *ctx, void *stream, uint32_t *n_pairs, uint32_t *n_tiles,
                             uint32_t *counts, char **err);

/* ---- weighted combine ------------------------------------------------------------------------- */

/* h2[t][c] = bf16(sum_r w[t][r] * partials[t][r][c]), fma in rank order.
 * Replaces PrefillMoE.encodeReduceTokenMajor (Kernels/Prefill/MoE/PrefillMoE.swift:11-32,
 * Metal/Prefill/prefill.metal:544-565). */
int ffmoe_reduce_token_major(ffmoe_ctx *ctx, void *stream, const uint16_t *partials,
                             const uint16_t *weights, uint16_t *h2, uint32_t t, uint32_t top_k,
                             uint32_t d, char **err);

/* ---- generic INT4 GEMV (reference layout: W uint8 [m][n/2], S/B bf16 [m][n/64]) ---------------- */

/* y[r][row] = bf16(sum_k (q*scale + bias)[row][k] * x[r][k]) for r < rows <= 16, weights read once.
 * Row r equals the rows == 1 result bit for bit. Replaces DequantInt4GEMV.encode / encodeRows
 * (Kernels/Quant/DequantInt4GEMV.swift:72-123,184-224) and the LM-head GEMV
 * (Metal/Sampling/logit.metal:614-667). `w` needs 2-byte alignment only; 16-byte aligned rows take
 * the wide-load path. y_f32 != 0 writes fp32 logits instead of bf16 (RowsTypes.f16ToF32). */
int ffmoe_gemv_int4(ffmoe_ctx *ctx, void *stream, const uint8_t *w, const uint16_t *scales,
                    const uint16_t *biases, const uint16_t *x, void *y, uint32_t m, uint32_t n,
                    uint32_t rows, uint32_t x_stride, uint32_t y_stride, int y_f32, char **err);

/* The same over the m weight rows listed in `ids` (device, uint32): output o of each input row is the
 * dot product with weight row ids[o]; fp32 out. The caller keeps every id inside the table.
 * Replaces DequantInt4GEMV.encodeRowsListed (Kernels/Quant/DequantInt4GEMV.swift:124-145), the
 * projection of the LM head's hot-vocabulary guess (Kernels/Fusions/LMHeadChainInt4.swift:171-177). */
int ffmoe_gemv_int4_listed(ffmoe_ctx *ctx, void *stream, const uint8_t *w, const uint16_t *scales,
                           const uint16_t *biases, const uint32_t *ids, const uint16_t *x, float *y, uint32_t m,
                           uint32_t n, uint32_t rows, uint32_t x_stride, uint32_t y_stride, char **err);

/* ---- resident INT4 matrix (LM head and other static weights) ------------------------------------ */

#define FFMOE_MATRIX_MAX_N 2816  /* K kept in registers: 4 waves x 11 groups of 64 */

typedef struct ffmoe_matrix ffmoe_matrix;

/* Re-tiles one weight in the reference layout (W uint8 [m][n/2] with 2-byte alignment, S/B bf16
 * [m][n/64]; host or device memory) into HBM once, as LMHeadChainInt4 keeps the head's table and
 * scratch for its lifetime (Kernels/Fusions/LMHeadChainInt4.swift:57-88). n must be a multiple of 64,
 * at most FFMOE_MATRIX_MAX_N; m is any count whose re-tiled form, ceil(m / 32) * (n / 64) KiB, stays below 4 GiB
 * (the reference's head tests use 4,099 rows; 262,144 x 2816 takes 352 MiB). with_greedy != 0
 * also allocates the scratch of ffmoe_matrix_greedy / _conf (per-block winners and softmax pairs, 128 KiB). Blocking; not a
 * hot-path call. */
int ffmoe_matrix_create(ffmoe_ctx *ctx, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                        uint32_t m, uint32_t n, int with_greedy, ffmoe_matrix **out, char **err);
/* The same for an 8-bit affine weight (W uint8 [m][n], one value per byte, S/B bf16 [m][n/64]: w = q s + b with
 * q = 0 .. 255, Metal/Quant/dequant_int8.metal:5-12): the form in which the reference's packs hold the shared expert
 * by default (Model.sharedExpertWeightBits, Runtime/Inference/Model.swift:13). The matrix then serves
 * ffmoe_matrix_gemv (not the greedy calls) and replaces DequantInt8GEMV.encode
 * (Kernels/Quant/DequantInt8GEMV.swift:26-56, kernel dequant_int8_gemv_simd, dequant_int8.metal:41-83) for 1 to 16
 * rows per call. Held as two 4-bit planes per 16-row tile (q = 16 h + l: the high nibbles with scale 16 s and the
 * bias, the low ones with scale s), so it takes m x n bytes + scales like the source and streams at the 4-bit
 * matrix's rate. */
int ffmoe_matrix_create_int8(ffmoe_ctx *ctx, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                             uint32_t m, uint32_t n, ffmoe_matrix **out, char **err);
/* The gate and up projections of an 8-bit gated FFN as ONE matrix (each W uint8 [f][n], S/B bf16 [f][n/64], host or
 * device memory, all six of the same kind), their rows interleaved 16 at a time: ffmoe_matrix_gemv on it then writes
 * y[r][i] = round16(gelu_tanh(round16(gate_i . x_r)) * round16(up_i . x_r)) for i < f - the activation row of the
 * shared expert in one pass over both projections, as the reference's fused kernel shared_int8_gate_up_act_simd makes it
 * (Metal/Quant/dequant_int8.metal:84-140, run by SharedExpertInt8.encodeFusedGateUpAct,
 * Kernels/MoE/SharedExpertInt8.swift:99-135), and bit for bit what two ffmoe_matrix_gemv calls on separate matrices
 * and ffmoe_gelu_mul leave. A ffmoe_matrix_create_int8 matrix of the down projection finishes the expert. */
int ffmoe_matrix_create_int8_glu(ffmoe_ctx *ctx, const uint8_t *gate_w, const uint16_t *gate_scales,
                                 const uint16_t *gate_biases, const uint8_t *up_w, const uint16_t *up_scales,
                                 const uint16_t *up_biases, uint32_t f, uint32_t n, ffmoe_matrix **out, char **err);
/* A matrix belongs to the context it was created on. Destroying that context first releases the matrix's
 * device memory; the handle then only accepts ffmoe_matrix_destroy (compute calls return FFMOE_ERR_INVALID). */
void ffmoe_matrix_destroy(ffmoe_matrix *mx);

/* y[r][row] = sum_g [ s_g * sum_k q_k x_k + b_g * sum_k x_k ] for r < rows <= 16 with the matrix read
 * once: DequantInt4GEMV.encodeRows on a static weight (Kernels/Quant/DequantInt4GEMV.swift:72-123) and
 * the head projection of LMHeadChainInt4.encodeGreedyRows (LMHeadChainInt4.swift:122-131). x bf16
 * [rows][x_stride], 16-byte aligned, stride a multiple of 8; y bf16 or (y_f32 != 0) fp32 [rows][y_stride]. */
int ffmoe_matrix_gemv(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows,
                      void *y, uint32_t y_stride, int y_f32, char **err);

/* out[i][k] = round16((q s + b) * out_scale) for weight row ids[i] of a 4-bit matrix, i < count (ids: uint32 in device
 * memory - e.g. the tokens ffmoe_matrix_greedy left - or NULL with count = 1 for the one row token_id): the embedding
 * lookup of a model whose head and embedding share one table, served from the head's resident copy. Replaces
 * EmbedLookupInt4.encode (Kernels/Quant/EmbedLookupInt4.swift:14-44, kernel embed_lookup_int4,
 * Metal/Quant/dequant_int4.metal:53-73; out_scale = sqrt(hidden size) there). Bit for bit the reference's
 * half((float(q) * s + b) * out_scale) in the context's activation type. An id >= M gives a row of zeros (the
 * reference reads past its table). out 16-byte aligned, stride a multiple of 8 and >= N. */
int ffmoe_matrix_rows(ffmoe_matrix *mx, void *stream, const uint32_t *ids, uint32_t count, uint32_t token_id,
                      float out_scale, uint16_t *out, uint32_t out_stride, char **err);

/* out[r][i] = round16(gelu_tanh(gate[r][i]) * up[r][i]) for `rows` rows of `count` values in the context's activation
 * type: gelu_mul_fp16 (Metal/Primitives/utility.metal:4-17, run by PrefillSharedExpert.encodeBatched,
 * Kernels/Prefill/MoE/PrefillSharedExpert.swift:78-91), and with two ffmoe_matrix_gemv calls in front and one behind
 * the 8-bit shared expert: SharedExpertInt8.encode (Kernels/MoE/SharedExpertInt8.swift:56-97; its fused kernel
 * shared_int8_gate_up_act_simd rounds gate and up to 16 bits before the activation just as the separate calls do,
 * dequant_int8.metal:131-136). Strides in elements, each at least `count`; `out` may be `gate` or `up` itself (same
 * pointer and stride), and no other overlap is allowed. */
int ffmoe_gelu_mul(ffmoe_ctx *ctx, void *stream, const uint16_t *gate, uint32_t gate_stride, const uint16_t *up,
                   uint32_t up_stride, uint16_t *out, uint32_t out_stride, uint32_t rows, uint32_t count, char **err);

/* Greedy token per row: the fp32 logits of the GEMV above and, as that kernel's epilogue (the logits are
 * never written out), the index of the largest finite logit,
 * ties to the lowest index, non-finite values never chosen (Metal/Sampling/logit.metal:689-720,916-921;
 * LMHeadChainInt4.encodeGreedyDecode / encodeGreedyRows, LMHeadChainInt4.swift:94-139,225-284). The
 * input rows are the already normalised hidden rows (the reference runs its RMSNorm operator first). */
int ffmoe_matrix_greedy(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows,
                        uint32_t *out_tokens, char **err);

/* ffmoe_matrix_greedy that also leaves each row's confidence: the chosen token's softmax probability over the finite
 * logits, each capped to softcap * tanh(logit / softcap) when softcap > 0 (0 disables the cap) - what
 * argmax_rows_f32 writes to rowsConfidence for the DFlash drafter (Metal/Sampling/logit.metal:946-1010,
 * LMHeadChainInt4.encodeGreedyRows with softcap, LMHeadChainInt4.swift:94-139,209-223). The token is chosen on the
 * uncapped logits, as there. out_conf fp32 [rows] (0 for a row without a finite logit). The softmax sums run in
 * this build's order (the reference's simd_sum leaves it open): a probability is comparable to 1e-5, not to the bit. */
int ffmoe_matrix_greedy_conf(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows,
                             float softcap, uint32_t *out_tokens, float *out_conf, char **err);

/* The greedy choice over rows of fp32 logits that are in memory already - the output of ffmoe_gemv_int4_listed for a
 * drafter's hot vocabulary: out_index[r] = position of the largest finite value of logits[r][0..count), ties to the
 * lowest position, 0xFFFFFFFF when none is finite; out_conf (may be NULL) as above. The caller maps a position
 * through its id list. Replaces argmax_rows_f32 as LMHeadChainInt4.encodeHotGreedyRows dispatches it
 * (LMHeadChainInt4.swift:144-186,209-223). */
int ffmoe_argmax_rows(ffmoe_ctx *ctx, void *stream, const float *logits, uint32_t stride, uint32_t rows, uint32_t count,
                      float softcap, uint32_t *out_index, float *out_conf, char **err);

/* How a row of fp32 logits picks its token when it is not the argmax: TokenSampling + the position key of
 * LMHeadChainInt4.RowSampling (Kernels/Fusions/LMHeadChainInt4.swift:183-190; SampleRowsParams,
 * Metal/Sampling/logit.metal:1025-1035). */
typedef struct ffmoe_sampling {
    float temperature;   /* > 0 */
    float top_p;         /* (0, 1]; applies only with top_k */
    uint32_t top_k;      /* 0 = no truncation, else 1...256 */
    uint32_t key_base;   /* position of row 0's token (row r draws for position key_base + key_offset[0] + r) */
    float softcap;       /* > 0: logits are capped to (-softcap, softcap) */
    uint64_t seed;
} ffmoe_sampling;

/* The sampled choice over rows of fp32 logits that are in memory (ffmoe_matrix_gemv's output, or the listed
 * projection's): per row one draw from the tempered softmax of the capped logits by the Gumbel-max rule,
 * argmax_i capped(logit_i) / T + G(seed, key, token_i), over the entries the truncation keeps - the top_k largest
 * capped logits (ties to the lower position), of those the shortest prefix whose T = 1 probability reaches top_p.
 * The noise G is a hash of (seed, the drawn token's position, token id) alone, so every producer that draws a
 * position draws the same noise. out_tokens[r] = the POSITION drawn (0xFFFFFFFF when no logit is finite), out_prob[r]
 * its probability among the survivors at temperature T. ids (device, may be NULL): entry i is token ids[i] (the
 * noise follows the token id; the position is returned, as in the reference). key_offset (device, may be NULL): one
 * uint32 added to key_base, for a base that lives on the GPU. Replaces sample_rows_f32 as
 * LMHeadChainInt4.encodeChoice dispatches it (Metal/Sampling/logit.metal:1010-1259,
 * Kernels/Fusions/LMHeadChainInt4.swift:192-223). The top_k set is found exactly (a radix select), where the
 * reference gathers the histogram's edge bin into at most 1,024 candidates. rows <= 16. */
int ffmoe_sample_rows(ffmoe_ctx *ctx, void *stream, const float *logits, uint32_t stride, uint32_t rows, uint32_t count,
                      const uint32_t *ids, const ffmoe_sampling *rule, const uint32_t *key_offset, uint32_t *out_tokens,
                      float *out_prob, char **err);

/* ---- dense (shared-expert) FFN ------------------------------------------------------------------ */

/* One projection in the reference layout: W uint8 [rows][cols/2], S/B bf16 [rows][cols/64]
 * (SharedExpertProjection: Kernels/MoE/SharedExpertInt8.swift, used by SharedExpertInt4.encode,
 * Kernels/MoE/SharedExpertInt4.swift:32-40). Host or device pointers, all three of the same kind. */
typedef struct {
    const uint8_t *w;
    const uint16_t *scales;
    const uint16_t *biases;
} ffmoe_projection;

/* Uploads one expert from three separate projections (gate, up [f][d]; down [d][f]) instead of a blob:
 * the form in which the reference holds its shared expert (TensorView triples from
 * Model.sharedExpertGate / Up / Down, bound per call by SharedExpertInt4.encode,
 * Kernels/MoE/SharedExpertInt4.swift:67-72). The layer counts as loaded once each of its experts has
 * been uploaded this way (or ffmoe_upload_layer ran). Blocking. */
int ffmoe_upload_expert_parts(ffmoe_ctx *ctx, uint32_t layer, uint32_t expert, const ffmoe_projection *gate,
                              const ffmoe_projection *up, const ffmoe_projection *down, int src_is_device,
                              char **err);

/* y[t] = down( bf16( gelu_tanh(gate x[t]) * (up x[t]) ) ) for every row, weight 1, no routing: the
 * shared expert. Needs a context created with n_experts = 1 and top_k = 1 (f = the shared width).
 * Rows <= 16 run the streaming kernels of ffmoe_verify; 17 to 384 rows the resident-matrix GEMV on the expert's arena
 * tiles, a grid row per 16 input rows (when d and f fit that kernel: <= FFMOE_MATRIX_MAX_N); more rows the grouped GEMMs
 * of ffmoe_prefill (the reference switches from its per-token GEMV loop to batched GEMMs at 32 tokens). Replaces
 * SharedExpertInt4.encode (Kernels/MoE/SharedExpertInt4.swift:32-89, kernel shared_gate_up_act_int4,
 * Metal/MoE/moe.metal:548-570) and PrefillSharedExpert.encodeBlock
 * (Kernels/Prefill/MoE/PrefillSharedExpert.swift:94-137). Gate and up stay fp32 in front of the
 * activation; the reference rounds them to FP16 there only to match its own unfused path bit for bit.
 * x bf16 [t][x_stride], y bf16 [t][d]; both 16-byte aligned. */
int ffmoe_dense_ffn(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                    uint32_t t, uint16_t *y, char **err);

/* ---- the steps either side of the MoE stage ------------------------------------------------------ */

#define FFMOE_ROW_MAX_D 4096  /* kFusedMaxD / kPrefillPostMaxD: Kernels/Prefill/Epilogues/PrefillLayerTail.swift:27 */

/* After attention and its output projection, for each of t rows:
 *   attn = rmsnorm(attn, w_post_attn); hidden += attn (in place);
 *   dense_x = rmsnorm(hidden, w_pre_ffn); routed_x = rmsnorm(hidden, w_pre_ffn2); router_x = rmsnorm(hidden)
 * every result rounded to bf16 where the reference rounds to FP16. dense_x feeds the shared expert
 * (ffmoe_dense_ffn), routed_x the routed experts, router_x the router. Replaces fused_post_attn_setup
 * (Metal/Fusions/fused.metal:210-296, Kernels/Fusions/FusedPostAttentionSetup.swift) for t = 1 and
 * prefill_post_attn_setup_block (Metal/Prefill/prefill.metal:243-318,
 * Kernels/Prefill/Epilogues/PrefillPostAttentionSetup.swift) for a block. All pointers are device memory;
 * rows are bf16 with strides in elements (>= d, any 2-byte alignment: 16-byte aligned rows take the fast
 * path, the bits are the same); weights are bf16 [d]; d is a multiple of 8, at most FFMOE_ROW_MAX_D.
 * Bytes outside the d used elements of a row are left alone. Needs no uploaded layer. */
int ffmoe_post_attn_setup(ffmoe_ctx *ctx, void *stream, uint16_t *hidden, uint32_t hidden_stride,
                          const uint16_t *attn, uint32_t attn_stride, uint16_t *dense_x, uint32_t dense_stride,
                          uint16_t *routed_x, uint32_t routed_stride, uint16_t *router_x, uint32_t router_stride,
                          const uint16_t *w_post_attn, const uint16_t *w_pre_ffn, const uint16_t *w_pre_ffn2,
                          uint32_t t, uint32_t d, float eps, char **err);

/* After the FFNs, for each of t rows (h1 = shared-expert output, h2 = combined routed output):
 *   h12 = h1 + rmsnorm(h2, w_postffn2); hidden = (hidden + rmsnorm(h12, w_postffn)) * layer_scalar
 * in place, every step rounded to bf16 as the reference rounds to FP16 (cpuReference,
 * Tests/.../Kernels/Fusions/FusedLayerTailTests.swift:96-110). Replaces prefill_layer_tail_block
 * (Metal/Prefill/prefill.metal:320-399, Kernels/Prefill/Epilogues/PrefillLayerTail.swift:11-51) and
 * FusedLayerTail.encode (Kernels/Fusions/FusedLayerTail.swift). Same pointer rules as above. */
int ffmoe_layer_tail(ffmoe_ctx *ctx, void *stream, const uint16_t *h2, uint32_t h2_stride, const uint16_t *h1,
                     uint32_t h1_stride, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2,
                     const uint16_t *w_postffn, uint32_t t, uint32_t d, float eps, float layer_scalar, char **err);

/* ffmoe_layer_tail on the rows the last ffmoe_route_verify(..., y = NULL, ...) call on this context and stream left
 * un-combined: h2 = the router-weighted combine of those rows under `route_w` (that call's out_w, [t][top_k]), made
 * while the tail loads its inputs instead of by a launch of its own, then the tail as above with d = the context's
 * hidden size. Bit for bit ffmoe_route_verify with y followed by ffmoe_layer_tail. This is the fusion of the routed
 * experts' weighted combine (Metal/Prefill/prefill.metal:544-565) into the layer tail (:320-399) for the decode /
 * verify block (t <= 16). */
int ffmoe_layer_tail_routed(ffmoe_ctx *ctx, void *stream, const uint16_t *route_w, const uint16_t *h1, uint32_t h1_stride,
                            uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2, const uint16_t *w_postffn,
                            uint32_t t, float eps, float layer_scalar, char **err);

/* The same for an 8-bit shared expert (each W uint8 [rows][cols], one value per byte; S/B as above; host or device
 * memory), the form in which the reference's packs hold it by default (SharedExpertInt8.encode,
 * Kernels/MoE/SharedExpertInt8.swift:56-135; Model.sharedExpertWeightBits, Runtime/Inference/Model.swift:13). Only on a
 * context with n_experts = 1 and top_k = 1, d and f multiples of 64 up to FFMOE_MATRIX_MAX_N. The layer is then kept as
 * a gated gate/up matrix and a down matrix of nibble planes (ffmoe_matrix_create_int8_glu / _int8) owned by the
 * context, and ffmoe_dense_ffn, ffmoe_route_verify_shared and ffmoe_layer_tail_routed_shared serve it like a 4-bit
 * layer: ffmoe_dense_ffn runs the two GEMV passes, a grid row per 16 rows, or from 192 rows on (when the context's
 * max_tokens reaches that) two dense GEMMs of rocBLAS on hi + lo rows of the weights, kept in the activation type for
 * that purpose (4 more bytes per weight; that form is not meant for stream capture: the library may allocate workspace
 * on its first call), with the same roundings (gate and up are rounded to 16 bits in front of the
 * activation, as the reference's fused kernel does, dequant_int8.metal:131-136). A layer is served in the width of
 * its latest upload: a later ffmoe_upload_layer / ffmoe_upload_expert_parts of the layer drops the 8-bit form. Blocking. */
int ffmoe_upload_expert_parts_int8(ffmoe_ctx *ctx, uint32_t layer, const ffmoe_projection *gate,
                                   const ffmoe_projection *up, const ffmoe_projection *down, char **err);

/* The expert work of one MoE block for a decode step / verify block (t <= 16) with the shared expert inside the
 * routed experts' two launches: ffmoe_route_verify(ctx, ..., y = NULL) on (router_x, x) and ffmoe_dense_ffn(shared, ...)
 * on shared_x in one call. `shared` is a context with n_experts = 1 and top_k = 1 (ffmoe_upload_expert_parts /
 * ffmoe_upload_layer) on the same device with the same hidden size and activation type. Some blocks of the gate/up
 * launch walk the shared expert's rows - they need no routes, so they stream while the others wait for theirs - and the
 * down launch takes the shared expert's K = f in chunks of 704 as extra experts (f <= 2816). Nothing is combined: the
 * routed rows stay un-weighted in `ctx`, the shared expert's chunk rows in `shared`, for
 * ffmoe_layer_tail_routed_shared. out_idx / out_w as in ffmoe_route_verify (same routes, bit for bit). The routed part
 * equals ffmoe_route_verify bit for bit; the shared expert's row is the same sum in another order (K in three
 * chunks instead of four interleaved slices), inside the 1e-2 / 0.9999 bar of the dense FFN. Shapes outside
 * (routed f > 704, d > 2816) are refused: run the two calls. This is the reference's schedule - shared expert beside
 * router + routed experts (Runtime/Inference/RealForwardRunner.swift:454-756; Kernels/MoE/SharedExpertInt4.swift:23-89
 * beside Kernels/MoE/MoE.swift:454-496) - as one pair of launches. */
int ffmoe_route_verify_shared(ffmoe_ctx *ctx, ffmoe_ctx *shared, void *stream, uint32_t layer, uint32_t shared_layer,
                              const uint16_t *router_x, uint32_t router_x_stride, const uint16_t *x, uint32_t x_stride,
                              const uint16_t *shared_x, uint32_t shared_x_stride, uint32_t t, uint32_t *out_idx,
                              uint16_t *out_w, char **err);

/* ffmoe_layer_tail_routed with h1 taken from the rows the last ffmoe_route_verify_shared(ctx, shared, ...) left in
 * `shared`: h1 = the chunk rows added in chunk order, rounded once to 16 bits (the dense FFN's output row); h2 and
 * the tail as in ffmoe_layer_tail_routed. */
int ffmoe_layer_tail_routed_shared(ffmoe_ctx *ctx, ffmoe_ctx *shared, void *stream, const uint16_t *route_w,
                                   uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2,
                                   const uint16_t *w_postffn, uint32_t t, float eps, float layer_scalar, char **err);

/* The layer tail with the two decode norms either side of it folded in: h1 arrives BEFORE its own norm
 * (w_postffn1, the shared expert's post-FFN-1 norm; h1 is left as found), and when w_next / normed are
 * given the norm of the new hidden row under w_next (the next layer's input norm) is written to normed.
 * Bit for bit ffmoe_rmsnorm(h1), ffmoe_layer_tail, ffmoe_rmsnorm(hidden). Replaces
 * FusedLayerTail.encodeWithNorms (Kernels/Fusions/FusedLayerTail.swift:74-117). */
int ffmoe_layer_tail_norms(ffmoe_ctx *ctx, void *stream, const uint16_t *h2, uint32_t h2_stride, const uint16_t *h1,
                           uint32_t h1_stride, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn1,
                           const uint16_t *w_postffn2, const uint16_t *w_postffn, const uint16_t *w_next,
                           uint16_t *normed, uint32_t normed_stride, uint32_t t, uint32_t d, float eps,
                           float layer_scalar, char **err);

/* out[r] = round((x[r] * rsqrt(mean(x[r]^2) + eps)) * w) for t rows; out may be x. Replaces
 * RMSNorm.encodeBF16W (kernel rmsnorm_bf16w), the operator the reference runs in front of the LM head
 * (Kernels/Fusions/LMHeadChainInt4.swift:165-170) and around the tail. Same pointer rules as above. */
int ffmoe_rmsnorm(ffmoe_ctx *ctx, void *stream, const uint16_t *x, uint32_t x_stride, const uint16_t *w,
                  uint16_t *out, uint32_t out_stride, uint32_t t, uint32_t d, float eps, char **err);

/* ---- activation type ------------------------------------------------------------------------- */

/* What the 16-bit values a caller hands over or gets back are: input rows, residual, route weights
 * (the router's output), outputs, per-route rows, the rows of the setup / tail / norm calls and the
 * 16-bit outputs of the GEMV calls. FFMOE_BF16 at creation. Norm weights, scales and biases of the
 * quantized tensors, per-expert scales and effective scales are bf16 in both (as in the reference's
 * checkpoints). FFMOE_FP16 reproduces the reference's text path: the router reads FP16 rows exactly, the
 * decode / verify kernels multiply FP16 rows with the INT4 weights on the FP16 matrix instruction and
 * round where the reference rounds to FP16 (activations, per-route rows, outputs). The prefill GEMMs
 * (ffmoe_prefill, ffmoe_prefill_pairs, ffmoe_dense_ffn beyond 16 rows) follow the reference's FP16 tiles
 * (Metal/Prefill/prefill.metal:581-598,685-702,723-777): FP16 rows against tile weights half(fma(q, scale, bias)), fp32
 * sums, and the activations between the two GEMMs FP16 with a power-of-two scale per pair and 64-wide block of the
 * intermediate size, so that values past FP16's range keep FP16's relative precision; the down GEMM brings a
 * pair's blocks to the pair's largest scale as it reads them and applies that scale to the pair's sums. In FFMOE_FP16 input rows must be 16-byte aligned with strides
 * that are multiples of 8 wherever a call accepts less otherwise (router, GEMV). Set it before the
 * first compute call; switching waits for the device. May allocate (once). */
int ffmoe_set_activation_dtype(ffmoe_ctx *ctx, int dtype, char **err);

/* ---- per-kernel timing ------------------------------------------------------------------------ */

/* Kernel slots of ffmoe_profile. */
enum {
    FFMOE_K_ROUTER_LOGITS = 0, FFMOE_K_ROUTER_TOPK, FFMOE_K_PLAN, FFMOE_K_GATE_UP, FFMOE_K_DOWN,
    FFMOE_K_COMBINE, FFMOE_K_PREFILL_SORT, FFMOE_K_PREFILL_GATE_UP, FFMOE_K_PREFILL_DOWN,
    FFMOE_K_PREFILL_COMBINE, FFMOE_K_GEMV, FFMOE_K_ARGMAX,
    FFMOE_K_EVENT_GAP, /* two event records with nothing between them: what an event pair adds to every slot above */
    FFMOE_K_ROUTE_GATE_UP, /* ffmoe_route_verify: router logits, select and gate/up in one launch */
    FFMOE_K_PROBE_GATE_UP, FFMOE_K_PROBE_DOWN, /* ffmoe_probe_stream: the weight loads of gate/up and of down alone */
    FFMOE_PROFILE_SLOTS = 16
};
typedef struct {
    double ms[FFMOE_PROFILE_SLOTS];          /* summed GPU time per kernel slot */
    uint64_t launches[FFMOE_PROFILE_SLOTS];
} ffmoe_profile;

/* While enabled, every compute call brackets each of its kernels with HIP events on the caller's
 * stream and WAITS for the call to finish, adding the elapsed times to the context's profile.
 * Replaces ANE_FIELDFARE_GPU_TRACE / makeTracedComputeEncoder
 * (Infrastructure/Metal/GPUTrace.swift:19-115) and the runner's cumulative nanosecond counters
 * (Runtime/Inference/RealForwardRunner.swift:171-203). */
int ffmoe_set_profiling(ffmoe_ctx *ctx, int enabled, char **err);
int ffmoe_get_profile(ffmoe_ctx *ctx, ffmoe_profile *out, int reset, char **err);

const char *ffmoe_version(void);

#ifdef __cplusplus
}
#endif
#endif
