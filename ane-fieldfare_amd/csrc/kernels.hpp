// Internal launch interface between the C ABI (api.hip) and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/fieldfare_moe.h"

namespace ffmoe {

// Geometry of one expert inside the HBM arena. Every expert occupies `expert_bytes`, split into four
// contiguous regions:
//   gu_tiles  [F/16][D/64] tiles of 1024 B: lane l (weight row 16*rb + l%16, k-quarter l/16) owns 16 B =
//             {gate k-half 0, gate k-half 1, up k-half 0, up k-half 1}, each dword eight nibbles
//   gu_scales [F/16][D/64][16] x {gate scale, gate bias, up scale, up bias} bf16
//   dn_tiles  [D/32][F/64] tiles of 1024 B: lane owns {row a half 0, row a half 1, row b half 0, row b half 1}
//             with a = 32*rbp + l%16 and b = a + 16
//   dn_scales [D/32][F/64][16] x {scale a, bias a, scale b, bias b} bf16
// A wave reads one tile with one 16-byte load per lane: 1 KiB contiguous.
struct ArenaGeom {
    uint32_t d, f;
    uint32_t gd;          // d / 64: groups along a gate/up row
    uint32_t gf;          // f / 64: groups along a down row
    uint32_t gu_rb;       // f / 16: gate/up row blocks
    uint32_t dn_rbp;      // d / 32: down row-block pairs
    size_t gu_tiles_off, gu_scales_off, dn_tiles_off, dn_scales_off;
    size_t expert_bytes;
};

ArenaGeom make_geom(uint32_t d, uint32_t f);

// Per-call routing plan of a decode / verify block, built on the GPU (no host round trip).
struct PlanSlot {
    uint32_t expert;
    uint32_t n;                               // routes of this expert, 1..16
    uint32_t routes[FFMOE_MAX_VERIFY_ROWS];   // route = token * top_k + rank
};
struct VerifyPlan {
    uint32_t n_live;
    uint32_t pad[3];
    PlanSlot slots[FFMOE_MAX_EXPERTS];
    // 1 when the route takes part: weight != 0, expert in range, among its expert's first 16 routes (a row that names
    // one expert several times can give an expert more than 16)
    uint32_t route_valid[FFMOE_MAX_VERIFY_ROWS * 8];
};

// Hand-over words of the launch that routes and runs gate/up in one go (skinny.hip): {epoch << 32 | payload},
// written and polled with device-coherent accesses. `epoch` starts at 1 over zeroed words and is advanced by the
// last launch of every call that used the words; `faults` counts polls that gave up.
struct RouteMail {
    uint32_t epoch, faults, pad[2];
    unsigned long long routes[FFMOE_MAX_VERIFY_ROWS * 8];                    // weight bits << 16 | expert
    unsigned long long logits[FFMOE_MAX_VERIFY_ROWS][FFMOE_MAX_EXPERTS];     // fp32 bits
};

// Per-kernel GPU timing with HIP events on the caller's stream, switched on by ffmoe_set_profiling.
// The counterpart of the reference's traced compute encoders (Infrastructure/Metal/GPUTrace.swift:19-115).
struct KernelTimer {
    bool on = false;
    hipEvent_t ev[14] = {};      // ev[0], ev[1]: an empty interval; ev[1] also opens the first kernel's interval
    int ids[14] = {};
    int n = 0;
    double ms[FFMOE_PROFILE_SLOTS] = {};
    uint64_t launches[FFMOE_PROFILE_SLOTS] = {};
    void begin(hipStream_t s) {
        n = 0;
        if (!on) return;
        (void)hipEventRecord(ev[0], s);
        ids[0] = FFMOE_K_EVENT_GAP;
        (void)hipEventRecord(ev[1], s);
        n = 1;
    }
    // call right after launching kernel `id`
    void mark(hipStream_t s, int id) {
        if (!on || n >= 13) return;
        ids[n] = id;
        (void)hipEventRecord(ev[++n], s);
    }
    // waits for the stream: profiling mode trades asynchrony for per-kernel times
    void finish() {
        if (!on || n <= 1) {
            n = 0;
            return;
        }
        (void)hipEventSynchronize(ev[n]);
        for (int i = 0; i < n; ++i) {
            float t = 0.f;
            if (hipEventElapsedTime(&t, ev[i], ev[i + 1]) == hipSuccess) {
                ms[ids[i]] += t;
                launches[ids[i]] += 1;
            }
        }
        n = 0;
    }
};

// Prefill: expert-sorted pairs and their M-tiles, built on the GPU.
struct PrefillTile {
    uint32_t expert, row_start, rows;     // rows [row_start, row_start + rows) of the sorted pair list
    uint32_t order;                       // the tile's number in row order (the tile list itself runs from the largest tile down)
};
struct PrefillPlan {
    uint32_t n_pairs, n_tiles, pad[2];
    uint32_t expert_count[FFMOE_MAX_EXPERTS];
    uint32_t expert_offset[FFMOE_MAX_EXPERTS + 1];
};
struct PrefillScratch {
    uint32_t *block_cnt;        // [sort blocks][E]: counts, then bases
    PrefillPlan *plan;
    PrefillTile *tiles;
    uint32_t max_tiles;
    uint32_t *sorted_token;     // [max pairs]
    uint32_t *sorted_out_row;   // [max pairs]: token * top_k + rank
    uint16_t *acts;             // [max pairs][F] bf16
    uint16_t *partials;         // [max pairs][D] 16-bit (used when the caller wants the combined output)
    float *act_scale;           // FP16 prefill: [act_blocks][F / 64][16] block scales of the activations, then [act_blocks][16] the pairs' largest (a context in FP16 mode; else null)
    uint32_t act_blocks;        // 16-pair blocks `acts` holds
};

struct RouterWeights {
    const void *w;          // bf16 [E][D] or float [E][D]
    int w_is_f32;
    const uint16_t *effective_scale;   // bf16 [D] or nullptr
    const uint16_t *per_expert_scale;  // bf16 [E] or nullptr
    const uint4 *w_frag = nullptr;     // bf16 weights in matrix-operand order (router.hip), or nullptr
    float w_norm_max = 0.0f;           // an upper bound of the largest 2-norm of an expert's row
};

// What launch_verify needs to make the routes itself (ffmoe_route_verify).
struct RouteFusion {
    RouterWeights rw;
    const uint16_t *router_x;
    uint32_t router_x_stride;
    float *logits;          // scratch of the two-launch router (used when the one-launch form does not apply)
    RouteMail *mail;
    unsigned long long poll_ticks;      // how long a wave waits for a hand-over word (wall_clock64 ticks, 100 MHz)
    bool one_launch;                    // false: the router runs as launches of its own in front of the expert pass
    uint32_t resident_blocks;           // blocks of the one-launch form the GPU holds at once (0: unknown, use the launches)
};

// The shared expert of the same MoE block (a dense FFN with its own input rows; SharedExpertInt4.swift:23-89), served by
// blocks of the routed experts' launches instead of launches of its own (ffmoe_route_verify_shared): some blocks of the
// gate/up launch walk its gate/up row blocks - they need no routes and start while the others wait for theirs -, and
// the down launch takes its K = f in chunks of kRing groups, one extra "expert" per chunk, whose un-weighted fp32 rows
// the layer tail adds up.
struct SharedExpert {
    const uint8_t *arena_layer;     // the one expert of the dense context's layer
    ArenaGeom g;                    // d as the routed experts'; f = 64 * gf
    const uint16_t *x;              // [t][x_stride]
    uint32_t x_stride;
    uint16_t *acts;                 // [t][g.f]
    float *partials;                // [chunks][t][g.d], chunk c = groups [kRing c, kRing c + kRing) of K
    // an 8-bit shared expert (all four set; arena_layer unused): the nibble-plane tiles and scales of its gated gate/up
    // matrix and of its down matrix as launch_matrix_repack lays them out (matrix.hip)
    const uint8_t *gu_tiles8 = nullptr, *gu_scales8 = nullptr, *dn_tiles8 = nullptr, *dn_scales8 = nullptr;
};
constexpr uint32_t kSharedChunkGroups = 11;      // = kRing of the streaming kernels
inline uint32_t shared_chunks(const ArenaGeom &g) { return (g.gf + kSharedChunkGroups - 1) / kSharedChunkGroups; }

// repack.hip
hipError_t launch_repack_layer(hipStream_t s, const uint8_t *blobs, size_t stride, ffmoe_offsets off,
                               uint32_t n_experts, ArenaGeom g, uint8_t *arena_layer);
hipError_t launch_dequant_expert(hipStream_t s, const uint8_t *arena_expert, ArenaGeom g, int which,
                                 uint16_t *out);

// router.hip
hipError_t launch_router(hipStream_t s, RouterWeights rw, const uint16_t *x, uint32_t x_stride, uint32_t t,
                         uint32_t n_experts, uint32_t d, uint32_t top_k, float *logits, uint32_t *out_idx,
                         uint16_t *out_w, KernelTimer *timer, bool f16 = false, bool want_logits = true,
                         float *scratch = nullptr);
// `frag`: E * d bf16 values, the weights in matrix-operand order (needs d % 32 == 0 and E % 16 == 0)
hipError_t launch_router_fragments(hipStream_t s, const uint16_t *w, uint32_t n_experts, uint32_t d, void *frag);

// skinny.hip
hipError_t launch_verify(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts,
                         uint32_t top_k, const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx,
                         const uint16_t *w, const uint16_t *residual, uint16_t *y, uint16_t *partials_bf16,
                         VerifyPlan *plan, uint16_t *acts, float *partials_f32, uint32_t n_cus, KernelTimer *timer,
                         bool f16 = false, const RouteFusion *route = nullptr, bool dense = false,
                         const SharedExpert *shared = nullptr);
uint32_t route_launch_resident_blocks(uint32_t n_cus);
// the two expert kernels' weight loads for n_live experts and nothing else (nothing is stored)
hipError_t launch_probe_stream(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts, uint32_t n_live,
                               uint32_t n_cus, KernelTimer *timer);
hipError_t launch_reduce_token_major(hipStream_t s, const uint16_t *partials, const uint16_t *weights,
                                     uint16_t *h2, uint32_t t, uint32_t top_k, uint32_t d, bool f16 = false);

// matrix.hip: resident two-stream tiling of a [M][N] INT4 matrix, its multi-row GEMV and the greedy choice.
// planes8: the weight is an 8-bit affine one, kept as two nibble planes per 16-row tile (csrc/matrix.hip)
size_t matrix_tiles_bytes(uint32_t m, uint32_t n, bool planes8 = false);
size_t matrix_scales_bytes(uint32_t m, uint32_t n, bool planes8 = false);
bool matrix_shape_ok(uint32_t n);
hipError_t launch_matrix_repack(hipStream_t s, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                                uint32_t m, uint32_t n, uint8_t *tiles_out, uint8_t *scales_out, bool planes8 = false);
hipError_t launch_matrix_gemv(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n,
                              const uint16_t *x, uint32_t x_stride, uint32_t rows, void *y, uint32_t y_stride,
                              bool y_f32, uint32_t n_cus, bool f16 = false, bool planes8 = false, int glu = 0);
hipError_t launch_matrix_rows(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n, const uint32_t *ids,
                              uint32_t token_id, uint32_t count, float out_scale, uint16_t *out, uint32_t out_stride, bool f16);
hipError_t launch_expand_planes8(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n, bool glu,
                                 uint16_t *out, bool f16);
hipError_t launch_hilo_epilogue(hipStream_t s, const float *sums, uint32_t rows, uint32_t width, bool gated, uint16_t *out,
                                uint32_t out_stride, bool f16);
hipError_t launch_gelu_mul(hipStream_t s, const uint16_t *gate, uint32_t gate_stride, const uint16_t *up, uint32_t up_stride,
                           uint16_t *out, uint32_t out_stride, uint32_t rows, uint32_t count, bool f16);
uint32_t greedy_segments(uint32_t m, uint32_t n_cus);
// the GEMV with the greedy choice as its epilogue: per-block winners, then one block per input row
hipError_t launch_matrix_greedy(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n,
                                const uint16_t *x, uint32_t x_stride, uint32_t rows, unsigned long long *partials,
                                uint32_t *out, uint32_t n_cus, bool f16, KernelTimer *timer, float softcap = 0.0f,
                                float *out_conf = nullptr);
// greedy choice (and the winner's softmax probability under the softcap) over rows of fp32 logits in memory
hipError_t launch_argmax_rows(hipStream_t s, const float *logits, uint32_t stride, uint32_t rows, uint32_t count, float softcap,
                              uint32_t *out, float *out_conf);

// prefill.hip: routes come from (idx, w) [t][top_k], or from an explicit pair list when `pairs` != nullptr.
// Writes y [t][d] (combined) when y != nullptr; un-weighted bf16 rows go to partials_out or to scratch.
hipError_t launch_prefill(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t n_experts, uint32_t top_k,
                          const uint16_t *x, uint32_t x_stride, uint32_t t, const uint32_t *idx, const uint16_t *w,
                          const ffmoe_pair *pairs, uint32_t n_pairs_in, uint16_t *y, uint16_t *partials_out,
                          PrefillScratch sc, KernelTimer *timer, bool f16 = false, bool dense = false);

// Test hook: the weight fragments of one expert's gate/up (or down) tiles as the grouped GEMM's matrix instructions
// read them from LDS: [N-block][group][fragment 0..15][lane] x 16 bytes, `prefill_dump_fragments` fragments in all.
// Fragment u = arena tile (u % 8) / 2 of the N-block, stream u % 2, k-half u / 8; lane l holds row l % 16 of the
// stream and k = 32 * (k-half) + 8 * (l / 16) .. + 7 of the group.
uint32_t prefill_dump_fragments(const ArenaGeom &g, bool gate_up);
hipError_t launch_prefill_dump_tiles(hipStream_t s, const uint8_t *arena_layer, ArenaGeom g, uint32_t expert, bool gate_up,
                                     PrefillScratch sc, void *dump, bool f16 = false);

// epilogue.hip: row-wise steps either side of the MoE stage
hipError_t launch_post_attn_setup(hipStream_t s, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *attn,
                                  uint32_t attn_stride, uint16_t *dense_x, uint32_t dense_stride, uint16_t *routed_x,
                                  uint32_t routed_stride, uint16_t *router_x, uint32_t router_stride,
                                  const uint16_t *w_post_attn, const uint16_t *w_pre_ffn, const uint16_t *w_pre_ffn2,
                                  uint32_t t, uint32_t d, float eps, bool f16 = false);
hipError_t launch_layer_tail(hipStream_t s, const uint16_t *h2, uint32_t h2_stride, const uint16_t *h1, uint32_t h1_stride,
                             uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2, const uint16_t *w_postffn,
                             uint32_t t, uint32_t d, float eps, float layer_scalar, const uint16_t *w_postffn1 = nullptr,
                             const uint16_t *w_next = nullptr, uint16_t *normed = nullptr, uint32_t normed_stride = 0,
                             bool f16 = false, const float *routed_partials = nullptr, const uint16_t *routed_w = nullptr,
                             const uint32_t *route_valid = nullptr, uint32_t top_k = 0, const float *shared_partials = nullptr,
                             uint32_t shared_chunks = 0);
hipError_t launch_rmsnorm(hipStream_t s, const uint16_t *x, uint32_t x_stride, const uint16_t *w, uint16_t *out,
                          uint32_t out_stride, uint32_t t, uint32_t d, float eps, bool f16 = false);

// gemv.hip
hipError_t launch_gemv_int4(hipStream_t s, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                            const uint16_t *x, void *y, uint32_t m, uint32_t n, uint32_t rows,
                            uint32_t x_stride, uint32_t y_stride, int y_f32, const uint32_t *ids = nullptr, bool f16 = false);

// sample.hip: the sampled choice over rows of fp32 logits (Gumbel-max draw, exact top-k, top-p prefix)
hipError_t launch_sample_rows(hipStream_t s, const float *logits, uint32_t stride, uint32_t rows, uint32_t count,
                              const uint32_t *ids, float temperature, float top_p, uint32_t top_k, uint32_t key_base,
                              float softcap, unsigned long long seed, const uint32_t *key_offset, uint32_t *out_tokens,
                              float *out_prob);

}  // namespace ffmoe
