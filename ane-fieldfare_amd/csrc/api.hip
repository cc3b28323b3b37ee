// C ABI of libfieldfare_moe_hip.so (declared in include/fieldfare_moe.h): context, HBM expert arena,
// argument validation and stream-ordered launches. No call here touches a CPU implementation of the
// math: without a working HIP device every entry point fails with FFMOE_ERR_RUNTIME.
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "kernels.hpp"

using namespace ffmoe;

struct ffmoe_layer {
    bool experts_loaded = false;
    std::vector<bool> part_loaded;  // experts uploaded one at a time (ffmoe_upload_expert_parts)
    void *router_w = nullptr;       // bf16 or float [E][D]
    int router_is_f32 = 0;
    uint16_t *effective_scale = nullptr;
    uint16_t *per_expert_scale = nullptr;
    void *router_frag = nullptr;    // bf16 router weights in matrix-operand order (the prefill router's approximate pass)
    float router_norm_max = 0.0f;   // upper bound of the largest 2-norm of an expert's router row
    // a dense context's layer held 8-bit (ffmoe_upload_expert_parts_int8): the gated gate/up matrix and the down matrix
    struct ffmoe_matrix *gate_up8 = nullptr, *down8 = nullptr;
    // the same weights as hi + lo rows of the activation type for the library GEMM that serves large row counts
    // ([4 f][d] and [2 d][f]); null when the context's max_tokens stays below the row count from which it is used
    uint16_t *gate_up8_hilo = nullptr, *down8_hilo = nullptr;
};

// From this many rows on an 8-bit dense layer goes through the library's dense GEMM on hi / lo rows instead of one
// streaming pass per 16 rows (measured at 2816 -> 2112 -> 2816: streaming 19 us at 32 rows + 8.8 us per 32 more, 42 us at
// 127; the GEMM form 50 us at 128, 58 at 192, 67 at 256, 100 at 1,024, 244 at 3,072).
constexpr uint32_t kGemm8MinRows = 192;
// Up to this many rows a 4-bit dense layer streams its arena tiles through the resident-matrix GEMV (a grid row per 16
// input rows) instead of running the grouped GEMMs.
constexpr uint32_t kDenseStreamMaxRows = 384;

// A resident matrix: the re-tiled copy of one [m][n] INT4 weight plus the scratch of its greedy choice.
struct ffmoe_matrix {
    ffmoe_ctx *ctx = nullptr;     // null once the owning context was destroyed (the device memory went with it)
    int device = 0;
    uint32_t m = 0, n = 0;
    bool planes8 = false;         // an 8-bit weight kept as two nibble planes (ffmoe_matrix_create_int8)
    bool glu = false;             // gate and up projections interleaved 16 rows at a time; m = the outputs of the gated product
    uint8_t *tiles = nullptr, *scales = nullptr;
    unsigned long long *partials = nullptr;   // [16][blocks of the GEMV grid]: per-block winners of the greedy choice
};

struct ffmoe_ctx {
    int device = 0;
    uint32_t n_cus = 0;       // compute units: sizes the persistent grids
    ffmoe_shape shape{};
    ArenaGeom geom{};
    uint8_t *arena = nullptr;
    size_t layer_bytes = 0;
    std::vector<ffmoe_layer> layers;
    // scratch (owned by the context, sized at creation; calls on one context must not overlap)
    float *logits = nullptr;         // [max(max_tokens,16)][E]
    VerifyPlan *plan = nullptr;
    uint16_t *acts = nullptr;        // [16*top_k][F]
    float *partials = nullptr;       // [16*top_k][D]
    RouteMail *mail = nullptr;       // hand-over words of ffmoe_route_verify's one-launch router + gate/up
    unsigned long long handover_ticks = FFMOE_DEFAULT_HANDOVER_TICKS;
    bool one_launch_routing = true;
    uint32_t route_resident_blocks = 0;     // occupancy of the one-launch routing kernel x compute units
    PrefillScratch pf{};
    uint32_t max_pairs = 0;
    // dense FFN (n_experts == 1, top_k == 1): every row routes to expert 0 with weight 1
    uint32_t *dense_idx = nullptr;   // [max(max_tokens,16)] zeros
    uint16_t *dense_w = nullptr;     // [max(max_tokens,16)] 1.0 in the activation type
    bool f16 = false;                // activations are FP16 (ffmoe_set_activation_dtype)
    // the 8-bit dense layers' GEMM form: the library handle and the fp32 sums [max_tokens][max(4 f, 2 d)]
    rocblas_handle blas = nullptr;
    float *gemm8_sums = nullptr;
    KernelTimer timer;
    std::vector<ffmoe_matrix *> matrices;   // resident matrices created on this context and not yet destroyed
    // the stream the scratch was last used on, and the event a call on another stream waits for (claim_scratch)
    hipStream_t scratch_stream = nullptr;
    bool scratch_claimed = false;
    hipEvent_t scratch_event = nullptr;
};

// ---- scratch of ffmoe_verify_static: device memory that exists from the moment the library is loaded ----------
// One array per GPU (every device holds its own copy of a __device__ variable), shared by every context and
// every call on that GPU, never allocated and never freed. Layout: the route plan, then the activation rows
// [16 * top_k][f] (16-bit), then the un-weighted fp32 down rows [16 * top_k][d].
constexpr size_t kStaticPlanBytes = 32768;
constexpr size_t kStaticScratchBytes = FFMOE_STATIC_SCRATCH_BYTES;
static_assert(sizeof(VerifyPlan) <= kStaticPlanBytes, "the route plan outgrew its share of the static scratch");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
void *g_scratch_addr[kMaxDevices] = {};     // device address of `scratch` per device (its host-side name is no address)
std::mutex g_scratch_mutex;
// the stream that used a device's array last and the event a call on another stream waits for (claim_static_scratch)
hipStream_t g_scratch_stream[kMaxDevices] = {};
bool g_scratch_claimed[kMaxDevices] = {};
hipEvent_t g_scratch_event[kMaxDevices] = {};

// With `device` current: look the array's address on that device up once.
hipError_t resolve_static_scratch(int device) {
    if (device < 0 || device >= kMaxDevices) return hipSuccess;      // such a device runs without the static entry point
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_addr[device]) return hipSuccess;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e == hipSuccess) {
        g_scratch_addr[device] = p;
        if (hipEventCreateWithFlags(&g_scratch_event[device], hipEventDisableTiming) != hipSuccess) {
            g_scratch_event[device] = nullptr;
            (void)hipGetLastError();
        }
    }
    return e;
}

// Stream hand-over of one piece of scratch: `last` used it, `s` wants it. With `s` or `last` under graph capture, or
// `last` gone, nothing is done. Returns whether `s` now owns it.
bool hand_over(hipStream_t last, bool claimed, hipEvent_t event, hipStream_t s) {
    hipStreamCaptureStatus now = hipStreamCaptureStatusNone, before = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &now) != hipSuccess || now != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return false;
    }
    if (claimed && event) {
        // the previous stream may be gone by now (its owner destroyed it): then there is nothing left to wait for
        if (hipStreamIsCapturing(last, &before) == hipSuccess && before == hipStreamCaptureStatusNone &&
            hipEventRecord(event, last) == hipSuccess)
            (void)hipStreamWaitEvent(s, event, 0);
        (void)hipGetLastError();
    }
    return true;
}

// The static array serves every context on its GPU: the same stream-to-stream ordering as a context's own scratch
// (claim_scratch below), kept per device. Allocates nothing: the event exists since the address was looked up.
void claim_static_scratch(int device, void *stream) {
    if (device < 0 || device >= kMaxDevices) return;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_claimed[device] && g_scratch_stream[device] == s) return;
    if (hand_over(g_scratch_stream[device], g_scratch_claimed[device], g_scratch_event[device], s)) {
        g_scratch_stream[device] = s;
        g_scratch_claimed[device] = true;
    }
}

int fail(char **err, int code, const char *fmt, ...) {
    if (err) {
        char buf[512];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        *err = strdup(buf);
    }
    return code;
}

#define FF_HIP(call)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) return fail(err, FFMOE_ERR_RUNTIME, "%s: %s", #call, hipGetErrorString(e_)); \
    } while (0)

int check_ctx(ffmoe_ctx *ctx, char **err) {
    if (!ctx) return fail(err, FFMOE_ERR_INVALID, "null context");
    FF_HIP(hipSetDevice(ctx->device));
    return FFMOE_OK;
}

// The context's scratch (plan, activation rows, un-weighted rows, hand-over words, sort tables) serves one stream at a
// time. Calls on the stream that used it last cost nothing here; a call that arrives on ANOTHER stream first makes that
// stream wait, on the device, for everything the previous stream has been given, so that two streams sharing a
// context run one call after the other instead of racing for the scratch. (Streams under graph capture are left
// alone: a capture orders its own nodes, and an event from outside may not enter it.) Host threads are a different
// matter: a context is for one host thread at a time.
void claim_scratch(ffmoe_ctx *ctx, void *stream) {
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (ctx->scratch_claimed && ctx->scratch_stream == s) return;
    if (hand_over(ctx->scratch_stream, ctx->scratch_claimed, ctx->scratch_event, s)) {
        ctx->scratch_stream = s;
        ctx->scratch_claimed = true;
    }
}

int check_layer(ffmoe_ctx *ctx, uint32_t layer, bool need_experts, bool need_router, char **err) {
    if (layer >= ctx->shape.n_layers)
        return fail(err, FFMOE_ERR_INVALID, "layer %u out of range (n_layers = %u)", layer, ctx->shape.n_layers);
    if (need_experts && !ctx->layers[layer].experts_loaded)
        return fail(err, FFMOE_ERR_NO_LAYER, "experts of layer %u were not uploaded", layer);
    if (need_router && !ctx->layers[layer].router_w)
        return fail(err, FFMOE_ERR_NO_LAYER, "router of layer %u was not uploaded", layer);
    return FFMOE_OK;
}

// A layer that was uploaded 8-bit and is now uploaded 4-bit loses its 8-bit matrices.
void drop_int8_form(ffmoe_layer &l) {
    ffmoe_matrix_destroy(l.gate_up8);
    ffmoe_matrix_destroy(l.down8);
    l.gate_up8 = l.down8 = nullptr;
    if (l.gate_up8_hilo) (void)hipFree(l.gate_up8_hilo);
    if (l.down8_hilo) (void)hipFree(l.down8_hilo);
    l.gate_up8_hilo = l.down8_hilo = nullptr;
}

// (Re)makes the hi / lo rows of an 8-bit layer in the context's activation type from its nibble planes. Blocking.
hipError_t expand_int8_layer(ffmoe_ctx *ctx, ffmoe_layer &l) {
    if (!l.gate_up8_hilo) return hipSuccess;
    hipError_t e = launch_expand_planes8(nullptr, l.gate_up8->tiles, l.gate_up8->scales, ctx->shape.f, ctx->shape.d, true,
                                         l.gate_up8_hilo, ctx->f16);
    if (e == hipSuccess)
        e = launch_expand_planes8(nullptr, l.down8->tiles, l.down8->scales, ctx->shape.d, ctx->shape.f, false, l.down8_hilo, ctx->f16);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    return e;
}

template <typename T>
int upload_vec(T **dst, const T *src, size_t count, char **err) {
    if (*dst) { (void)hipFree(*dst); *dst = nullptr; }
    if (!src) return FFMOE_OK;
    FF_HIP(hipMalloc(reinterpret_cast<void **>(dst), count * sizeof(T)));
    FF_HIP(hipMemcpy(*dst, src, count * sizeof(T), hipMemcpyHostToDevice));
    return FFMOE_OK;
}

}  // namespace

extern "C" {

const char *ffmoe_version(void) { return "fieldfare-moe-hip 0.1 (gfx950)"; }

int ffmoe_create(int device, const ffmoe_shape *shape, ffmoe_ctx **out, char **err) {
    if (!shape || !out) return fail(err, FFMOE_ERR_INVALID, "null argument");
    *out = nullptr;
    if (shape->d == 0 || shape->d % FFMOE_GROUP || shape->f == 0 || shape->f % FFMOE_GROUP)
        return fail(err, FFMOE_ERR_INVALID, "d = %u and f = %u must be positive multiples of %d", shape->d, shape->f,
                    FFMOE_GROUP);
    if (shape->n_experts == 0 || shape->n_experts > FFMOE_MAX_EXPERTS)
        return fail(err, FFMOE_ERR_INVALID, "n_experts = %u outside 1...%d", shape->n_experts, FFMOE_MAX_EXPERTS);
    if (shape->top_k == 0 || shape->top_k > 8 || shape->top_k > shape->n_experts)
        return fail(err, FFMOE_ERR_INVALID, "top_k = %u outside 1...8", shape->top_k);
    if (shape->n_layers == 0) return fail(err, FFMOE_ERR_INVALID, "n_layers must be positive");
    int count = 0;
    FF_HIP(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(err, FFMOE_ERR_INVALID, "device %d not present (%d visible)", device, count);
    FF_HIP(hipSetDevice(device));
    // a device on which the array has no address runs everything but ffmoe_verify_static, which then says so
    if (resolve_static_scratch(device) != hipSuccess) (void)hipGetLastError();

    ffmoe_ctx *ctx = new (std::nothrow) ffmoe_ctx();
    if (!ctx) return fail(err, FFMOE_ERR_ALLOC, "out of host memory");
    ctx->device = device;
    {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
        ctx->n_cus = (uint32_t)cus;
    }
    ctx->route_resident_blocks = route_launch_resident_blocks(ctx->n_cus);
    if (hipEventCreateWithFlags(&ctx->scratch_event, hipEventDisableTiming) != hipSuccess) {
        ctx->scratch_event = nullptr;      // without it calls on different streams are the caller's to order, as documented
        (void)hipGetLastError();
    }
    ctx->shape = *shape;
    ctx->geom = make_geom(shape->d, shape->f);
    // an expert's tile regions are addressed through buffer descriptors with 32-bit sizes and offsets
    if ((size_t)shape->d * shape->f >= ((size_t)1 << 32)) {
        delete ctx;
        return fail(err, FFMOE_ERR_INVALID, "d = %u x f = %u: an expert's gate/up tile region must stay below 4 GiB", shape->d,
                    shape->f);
    }
    ctx->layer_bytes = (size_t)shape->n_experts * ctx->geom.expert_bytes;
    ctx->layers.resize(shape->n_layers);
    const uint32_t router_rows = shape->max_tokens > FFMOE_MAX_VERIFY_ROWS ? shape->max_tokens : FFMOE_MAX_VERIFY_ROWS;
    const size_t routes = (size_t)FFMOE_MAX_VERIFY_ROWS * shape->top_k;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&ctx->arena), ctx->layer_bytes * shape->n_layers);
    // (the two-pass router lays its four parts out with the row count rounded up to 64)
    const size_t router_rows_padded = ((size_t)router_rows + 63) & ~(size_t)63;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->logits), 4 * router_rows_padded * ((size_t)shape->n_experts + 1) * sizeof(float));      // logits; or, for the two-pass prefill router, the four K parts' squared row norms and approximate logits
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->plan), sizeof(VerifyPlan));
    if (e == hipSuccess) e = hipMemset(ctx->plan, 0, sizeof(VerifyPlan));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->mail), sizeof(RouteMail));
    if (e == hipSuccess) e = hipMemset(ctx->mail, 0, sizeof(RouteMail));
    if (e == hipSuccess) {
        const uint32_t first_epoch = 1;      // zeroed words never carry it
        e = hipMemcpy(&ctx->mail->epoch, &first_epoch, sizeof first_epoch, hipMemcpyHostToDevice);
    }
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->acts), routes * shape->f * sizeof(uint16_t));
    // the un-weighted fp32 rows; a dense expert whose K exceeds a wave's ring leaves one set per chunk of K when it rides
    // along in another context's launches (ffmoe_route_verify_shared)
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->partials), routes * shape->d * sizeof(float) * std::max(1u, shared_chunks(ctx->geom)));
    // prefill scratch: sort tables, pair lists, activations and per-route rows for max_tokens tokens
    ctx->max_pairs = (shape->max_tokens > FFMOE_MAX_VERIFY_ROWS ? shape->max_tokens : FFMOE_MAX_VERIFY_ROWS) * shape->top_k;
    const size_t sort_blocks = (ctx->max_pairs + 255) / 256;
    ctx->pf.max_tiles = ctx->max_pairs / FFMOE_PREFILL_TILE_M + shape->n_experts + 1;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.block_cnt), sort_blocks * shape->n_experts * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.plan), sizeof(PrefillPlan));
    if (e == hipSuccess) e = hipMemset(ctx->pf.plan, 0, sizeof(PrefillPlan));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.tiles), (size_t)ctx->pf.max_tiles * sizeof(PrefillTile));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.sorted_token), (size_t)ctx->max_pairs * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.sorted_out_row), (size_t)ctx->max_pairs * sizeof(uint32_t));
    // activations in 16-pair blocks: an M-tile's blocks start at a block of their own (see prefill.hip)
    if (e == hipSuccess)
        e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.acts),
                      ((size_t)ctx->max_pairs / 16 + ctx->pf.max_tiles + 2) * 16 * shape->f * sizeof(uint16_t));
    ctx->pf.act_blocks = ctx->max_pairs / 16 + ctx->pf.max_tiles + 2;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.partials), (size_t)ctx->max_pairs * shape->d * sizeof(uint16_t));
    if (e == hipSuccess && shape->n_experts == 1 && shape->top_k == 1) {
        e = hipMalloc(reinterpret_cast<void **>(&ctx->dense_idx), (size_t)router_rows * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMemset(ctx->dense_idx, 0, (size_t)router_rows * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->dense_w), (size_t)router_rows * sizeof(uint16_t));
        if (e == hipSuccess) e = hipMemsetD16(reinterpret_cast<hipDeviceptr_t>(ctx->dense_w), 0x3F80, router_rows);
    }
    if (e != hipSuccess) {
        const size_t want = ctx->layer_bytes * shape->n_layers;      // read before the context is gone
        ffmoe_destroy(ctx);
        return fail(err, FFMOE_ERR_ALLOC, "failed to allocate the expert arena (%zu bytes) or scratch: %s", want,
                    hipGetErrorString(e));
    }
    *out = ctx;
    return FFMOE_OK;
}

void ffmoe_destroy(ffmoe_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipDeviceSynchronize();
    if (ctx->blas) (void)rocblas_destroy_handle(ctx->blas);
    if (ctx->gemm8_sums) (void)hipFree(ctx->gemm8_sums);
    for (auto &l : ctx->layers) {
        // the layer's own 8-bit matrices: nobody else holds their handles
        drop_int8_form(l);
        if (l.router_w) (void)hipFree(l.router_w);
        if (l.router_frag) (void)hipFree(l.router_frag);
        if (l.effective_scale) (void)hipFree(l.effective_scale);
        if (l.per_expert_scale) (void)hipFree(l.per_expert_scale);
    }
    if (ctx->arena) (void)hipFree(ctx->arena);
    if (ctx->logits) (void)hipFree(ctx->logits);
    if (ctx->plan) (void)hipFree(ctx->plan);
    if (ctx->mail) (void)hipFree(ctx->mail);
    if (ctx->acts) (void)hipFree(ctx->acts);
    if (ctx->partials) (void)hipFree(ctx->partials);
    if (ctx->pf.block_cnt) (void)hipFree(ctx->pf.block_cnt);
    if (ctx->pf.plan) (void)hipFree(ctx->pf.plan);
    if (ctx->pf.tiles) (void)hipFree(ctx->pf.tiles);
    if (ctx->pf.sorted_token) (void)hipFree(ctx->pf.sorted_token);
    if (ctx->pf.sorted_out_row) (void)hipFree(ctx->pf.sorted_out_row);
    if (ctx->pf.acts) (void)hipFree(ctx->pf.acts);
    if (ctx->pf.partials) (void)hipFree(ctx->pf.partials);
    if (ctx->pf.act_scale) (void)hipFree(ctx->pf.act_scale);
    if (ctx->dense_idx) (void)hipFree(ctx->dense_idx);
    if (ctx->dense_w) (void)hipFree(ctx->dense_w);
    // matrices that outlive their context lose their device memory here; the handles stay valid to destroy
    for (ffmoe_matrix *mx : ctx->matrices) {
        if (mx->tiles) (void)hipFree(mx->tiles);
        if (mx->scales) (void)hipFree(mx->scales);
        if (mx->partials) (void)hipFree(mx->partials);
        mx->tiles = mx->scales = nullptr;
        mx->partials = nullptr;
        mx->ctx = nullptr;
    }
    if (ctx->scratch_event) (void)hipEventDestroy(ctx->scratch_event);
    for (auto &ev : ctx->timer.ev)
        if (ev) (void)hipEventDestroy(ev);
    delete ctx;
}

size_t ffmoe_layer_arena_bytes(const ffmoe_ctx *ctx) { return ctx ? ctx->layer_bytes : 0; }

int ffmoe_upload_layer(ffmoe_ctx *ctx, uint32_t layer, const void *blobs, size_t stride,
                       const ffmoe_offsets *offsets, int src_is_device, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, false, false, err)) return rc;
    if (!blobs || !offsets) return fail(err, FFMOE_ERR_INVALID, "null argument");
    const ffmoe_shape &sh = ctx->shape;
    // every sub-tensor must lie inside one blob (the reference trusts its layout.json; a bad offset
    // here would send the re-tiling kernel out of bounds)
    const size_t gu_w = (size_t)sh.f * sh.d / 2, gu_s = (size_t)sh.f * (sh.d / FFMOE_GROUP) * 2;
    const size_t dn_w = (size_t)sh.d * sh.f / 2, dn_s = (size_t)sh.d * (sh.f / FFMOE_GROUP) * 2;
    const struct { uint32_t off; size_t len; const char *name; } parts[9] = {
        {offsets->gate_w, gu_w, "gate_w"}, {offsets->gate_s, gu_s, "gate_s"}, {offsets->gate_b, gu_s, "gate_b"},
        {offsets->up_w, gu_w, "up_w"},     {offsets->up_s, gu_s, "up_s"},     {offsets->up_b, gu_s, "up_b"},
        {offsets->down_w, dn_w, "down_w"}, {offsets->down_s, dn_s, "down_s"}, {offsets->down_b, dn_s, "down_b"}};
    for (const auto &p : parts)
        if ((size_t)p.off + p.len > stride)
            return fail(err, FFMOE_ERR_INVALID, "sub-tensor %s (offset %u, %zu bytes) exceeds the blob stride %zu", p.name,
                        p.off, p.len, stride);
    const uint8_t *src = static_cast<const uint8_t *>(blobs);
    uint8_t *staging = nullptr;
    if (!src_is_device) {
        const size_t bytes = stride * sh.n_experts;
        FF_HIP(hipMalloc(reinterpret_cast<void **>(&staging), bytes));
        hipError_t e = hipMemcpy(staging, blobs, bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(staging);
            return fail(err, FFMOE_ERR_RUNTIME, "copy of layer %u to the device failed: %s", layer, hipGetErrorString(e));
        }
        src = staging;
    }
    hipError_t e = launch_repack_layer(nullptr, src, stride, *offsets, sh.n_experts, ctx->geom,
                                       ctx->arena + (size_t)layer * ctx->layer_bytes);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (staging) (void)hipFree(staging);
    if (e != hipSuccess) return fail(err, FFMOE_ERR_RUNTIME, "re-tiling layer %u failed: %s", layer, hipGetErrorString(e));
    drop_int8_form(ctx->layers[layer]);
    ctx->layers[layer].experts_loaded = true;
    return FFMOE_OK;
}

int ffmoe_sample_rows(ffmoe_ctx *ctx, void *stream, const float *logits, uint32_t stride, uint32_t rows, uint32_t count,
                      const uint32_t *ids, const ffmoe_sampling *rule, const uint32_t *key_offset, uint32_t *out_tokens,
                      float *out_prob, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!logits || !rule || !out_tokens || !out_prob) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (rows == 0 || rows > FFMOE_MAX_VERIFY_ROWS) return fail(err, FFMOE_ERR_INVALID, "rows = %u outside 1...%d", rows, FFMOE_MAX_VERIFY_ROWS);
    if (count == 0 || stride < count) return fail(err, FFMOE_ERR_INVALID, "count must be positive and the stride at least the count");
    if (!(rule->temperature > 0.0f) || std::isinf(rule->temperature))
        return fail(err, FFMOE_ERR_INVALID, "temperature must be positive and finite (temperature 0 is the greedy choice: ffmoe_argmax_rows)");
    if (!(rule->softcap > 0.0f) || std::isinf(rule->softcap))
        return fail(err, FFMOE_ERR_INVALID, "the sampled choice caps its logits: softcap must be positive and finite");
    if (rule->top_k > 256) return fail(err, FFMOE_ERR_INVALID, "top_k = %u outside 0...256", rule->top_k);
    if (rule->top_k && !(rule->top_p > 0.0f && rule->top_p <= 1.0f)) return fail(err, FFMOE_ERR_INVALID, "top_p outside (0, 1]");
    FF_HIP(launch_sample_rows(static_cast<hipStream_t>(stream), logits, stride, rows, count, ids, rule->temperature, rule->top_p,
                              rule->top_k, rule->key_base, rule->softcap, rule->seed, key_offset, out_tokens, out_prob));
    return FFMOE_OK;
}

int ffmoe_upload_expert_parts(ffmoe_ctx *ctx, uint32_t layer, uint32_t expert, const ffmoe_projection *gate,
                              const ffmoe_projection *up, const ffmoe_projection *down, int src_is_device,
                              char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, false, false, err)) return rc;
    const ffmoe_shape &sh = ctx->shape;
    if (expert >= sh.n_experts) return fail(err, FFMOE_ERR_INVALID, "expert %u out of range", expert);
    const ffmoe_projection *proj[3] = {gate, up, down};
    for (const ffmoe_projection *p : proj)
        if (!p || !p->w || !p->scales || !p->biases) return fail(err, FFMOE_ERR_INVALID, "null projection");
    // stage the nine arrays as one blob in the order gate W/S/B, up W/S/B, down W/S/B, 16-byte aligned
    const size_t gu_w = (size_t)sh.f * sh.d / 2, gu_s = (size_t)sh.f * (sh.d / FFMOE_GROUP) * 2;
    const size_t dn_w = (size_t)sh.d * sh.f / 2, dn_s = (size_t)sh.d * (sh.f / FFMOE_GROUP) * 2;
    const size_t len[9] = {gu_w, gu_s, gu_s, gu_w, gu_s, gu_s, dn_w, dn_s, dn_s};
    const void *src[9] = {gate->w, gate->scales, gate->biases, up->w, up->scales, up->biases,
                          down->w, down->scales, down->biases};
    uint32_t off[9];
    size_t total = 0;
    for (int i = 0; i < 9; ++i) {
        off[i] = (uint32_t)total;
        total += (len[i] + 15) & ~(size_t)15;
    }
    uint8_t *staging = nullptr;
    FF_HIP(hipMalloc(reinterpret_cast<void **>(&staging), total));
    hipError_t e = hipSuccess;
    for (int i = 0; i < 9 && e == hipSuccess; ++i)
        e = hipMemcpy(staging + off[i], src[i], len[i], src_is_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice);
    const ffmoe_offsets offsets = {off[0], off[1], off[2], off[3], off[4], off[5], off[6], off[7], off[8]};
    if (e == hipSuccess)
        e = launch_repack_layer(nullptr, staging, total, offsets, 1, ctx->geom,
                                ctx->arena + (size_t)layer * ctx->layer_bytes + (size_t)expert * ctx->geom.expert_bytes);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    (void)hipFree(staging);
    if (e != hipSuccess)
        return fail(err, FFMOE_ERR_RUNTIME, "upload of expert %u of layer %u failed: %s", expert, layer, hipGetErrorString(e));
    ffmoe_layer &l = ctx->layers[layer];
    drop_int8_form(l);      // the layer is 4-bit from here on
    if (l.part_loaded.size() != sh.n_experts) l.part_loaded.assign(sh.n_experts, false);
    l.part_loaded[expert] = true;
    bool all = true;
    for (bool b : l.part_loaded) all = all && b;
    if (all) l.experts_loaded = true;
    return FFMOE_OK;
}

int ffmoe_upload_router_bf16(ffmoe_ctx *ctx, uint32_t layer, const uint16_t *w, const uint16_t *effective_scale,
                             const uint16_t *per_expert_scale, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, false, false, err)) return rc;
    if (!w) return fail(err, FFMOE_ERR_INVALID, "null router weights");
    ffmoe_layer &l = ctx->layers[layer];
    const size_t n = (size_t)ctx->shape.n_experts * ctx->shape.d;
    uint16_t *dw = nullptr;
    if (l.router_w) { (void)hipFree(l.router_w); l.router_w = nullptr; }
    if (int rc = upload_vec(&dw, w, n, err)) return rc;
    l.router_w = dw;
    l.router_is_f32 = 0;
    if (l.router_frag) { (void)hipFree(l.router_frag); l.router_frag = nullptr; }
    if (ctx->shape.d % 32 == 0 && ctx->shape.n_experts % 16 == 0) {
        // the prefill router's approximate pass reads the weights in matrix-operand order and bounds its error with
        // the largest row norm (rounded up)
        double worst = 0.0;
        for (uint32_t e = 0; e < ctx->shape.n_experts; ++e) {
            double sum = 0.0;
            for (uint32_t k = 0; k < ctx->shape.d; ++k) {
                const uint32_t bits = (uint32_t)w[(size_t)e * ctx->shape.d + k] << 16;
                float v;
                memcpy(&v, &bits, sizeof v);
                sum += (double)v * (double)v;
            }
            if (!(sum <= worst)) worst = sum;       // a NaN or infinite row makes the bound non-finite: every expert becomes a candidate
        }
        l.router_norm_max = (float)(std::sqrt(worst) * (1.0 + 1e-6));
        FF_HIP(hipMalloc(&l.router_frag, n * sizeof(uint16_t)));
        FF_HIP(launch_router_fragments(nullptr, dw, ctx->shape.n_experts, ctx->shape.d, l.router_frag));
        FF_HIP(hipDeviceSynchronize());
    }
    if (int rc = upload_vec(&l.effective_scale, effective_scale, ctx->shape.d, err)) return rc;
    return upload_vec(&l.per_expert_scale, per_expert_scale, ctx->shape.n_experts, err);
}

int ffmoe_upload_router_int8(ffmoe_ctx *ctx, uint32_t layer, const uint8_t *w, const uint16_t *scales,
                             const uint16_t *biases, const uint16_t *effective_scale,
                             const uint16_t *per_expert_scale, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, false, false, err)) return rc;
    if (!w || !scales || !biases) return fail(err, FFMOE_ERR_INVALID, "null router weights");
    ffmoe_layer &l = ctx->layers[layer];
    const uint32_t e_count = ctx->shape.n_experts, d = ctx->shape.d, groups = d / FFMOE_GROUP;
    // fp32(q * s + b): q * s is exact (8-bit x 8-bit significands), one rounding in the add
    std::vector<float> deq((size_t)e_count * d);
    for (uint32_t e = 0; e < e_count; ++e)
        for (uint32_t k = 0; k < d; ++k) {
            uint32_t sb = (uint32_t)scales[(size_t)e * groups + k / FFMOE_GROUP] << 16;
            uint32_t bb = (uint32_t)biases[(size_t)e * groups + k / FFMOE_GROUP] << 16;
            float s, b;
            memcpy(&s, &sb, 4);
            memcpy(&b, &bb, 4);
            const float prod = (float)w[(size_t)e * d + k] * s;
            deq[(size_t)e * d + k] = prod + b;
        }
    float *dw = nullptr;
    if (l.router_w) { (void)hipFree(l.router_w); l.router_w = nullptr; }
    if (int rc = upload_vec(&dw, deq.data(), deq.size(), err)) return rc;
    l.router_w = dw;
    l.router_is_f32 = 1;
    if (l.router_frag) { (void)hipFree(l.router_frag); l.router_frag = nullptr; }
    if (int rc = upload_vec(&l.effective_scale, effective_scale, d, err)) return rc;
    return upload_vec(&l.per_expert_scale, per_expert_scale, e_count, err);
}

int ffmoe_dequant_expert(ffmoe_ctx *ctx, void *stream, uint32_t layer, uint32_t expert, int which,
                         uint16_t *out_bf16, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, true, false, err)) return rc;
    if (expert >= ctx->shape.n_experts) return fail(err, FFMOE_ERR_INVALID, "expert %u out of range", expert);
    if (which < FFMOE_GATE || which > FFMOE_DOWN || !out_bf16) return fail(err, FFMOE_ERR_INVALID, "bad sub-tensor or null output");
    if (reinterpret_cast<uintptr_t>(out_bf16) % 16) return fail(err, FFMOE_ERR_INVALID, "output must be 16-byte aligned");
    const uint8_t *base = ctx->arena + (size_t)layer * ctx->layer_bytes + (size_t)expert * ctx->geom.expert_bytes;
    FF_HIP(launch_dequant_expert(static_cast<hipStream_t>(stream), base, ctx->geom, which, out_bf16));
    return FFMOE_OK;
}

int ffmoe_router(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *router_x, uint32_t x_stride,
                 uint32_t t, uint32_t *out_idx, uint16_t *out_w, float *out_logits, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, false, true, err)) return rc;
    if (!router_x || !out_idx || !out_w) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (t == 0) return fail(err, FFMOE_ERR_INVALID, "queryCount must be positive");
    if (x_stride < ctx->shape.d) return fail(err, FFMOE_ERR_INVALID, "hidden stride is too small");
    if (ctx->f16 && (reinterpret_cast<uintptr_t>(router_x) % 8 || x_stride % 4))
        return fail(err, FFMOE_ERR_INVALID, "FP16 router rows must be 8-byte aligned with a stride that is a multiple of 4");
    const uint32_t cap = ctx->shape.max_tokens > FFMOE_MAX_VERIFY_ROWS ? ctx->shape.max_tokens : FFMOE_MAX_VERIFY_ROWS;
    if (!out_logits && t > cap) return fail(err, FFMOE_ERR_INVALID, "t = %u exceeds max_tokens = %u", t, cap);
    const ffmoe_layer &l = ctx->layers[layer];
    RouterWeights rw{l.router_w, l.router_is_f32, l.effective_scale, l.per_expert_scale,
                     static_cast<const uint4 *>(l.router_frag), l.router_norm_max};
    claim_scratch(ctx, stream);
    FF_HIP(launch_router(static_cast<hipStream_t>(stream), rw, router_x, x_stride, t, ctx->shape.n_experts,
                         ctx->shape.d, ctx->shape.top_k, out_logits ? out_logits : ctx->logits, out_idx, out_w, &ctx->timer,
                         ctx->f16, out_logits != nullptr, ctx->logits));
    return FFMOE_OK;
}

// Scratch of one decode / verify call: the context's own allocations, or pieces of the static array.
struct VerifyScratch {
    VerifyPlan *plan;
    uint16_t *acts;
    float *partials;
};

static int verify_common(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                         uint32_t t, const uint32_t *idx, const uint16_t *w, const uint16_t *residual, uint16_t *y,
                         uint16_t *partials_bf16, char **err, const VerifyScratch *use = nullptr,
                         const RouteFusion *route = nullptr, bool dense = false, const SharedExpert *shared = nullptr,
                         ffmoe_ctx *shared_ctx = nullptr) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, true, route != nullptr, err)) return rc;
    if (!x || !idx || !w || (!y && !partials_bf16 && !route)) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (t == 0 || t > FFMOE_MAX_VERIFY_ROWS) return fail(err, FFMOE_ERR_INVALID, "rows = %u outside 1...%d", t, FFMOE_MAX_VERIFY_ROWS);
    if (x_stride < ctx->shape.d || x_stride % 8 || reinterpret_cast<uintptr_t>(x) % 16)
        return fail(err, FFMOE_ERR_INVALID, "x must be 16-byte aligned with a stride that is a multiple of 8 and >= d");
    if ((y && reinterpret_cast<uintptr_t>(y) % 8) || (residual && reinterpret_cast<uintptr_t>(residual) % 8))
        return fail(err, FFMOE_ERR_INVALID, "y and residual must be 8-byte aligned");
    const VerifyScratch own{ctx->plan, ctx->acts, ctx->partials};
    const VerifyScratch &sc = use ? *use : own;
    if (use) claim_static_scratch(ctx->device, stream); else claim_scratch(ctx, stream);
    if (shared_ctx) claim_scratch(shared_ctx, stream);
    FF_HIP(launch_verify(static_cast<hipStream_t>(stream), ctx->arena + (size_t)layer * ctx->layer_bytes, ctx->geom,
                         ctx->shape.n_experts, ctx->shape.top_k, x, x_stride, t, idx, w, residual, y, partials_bf16,
                         sc.plan, sc.acts, sc.partials, ctx->n_cus, &ctx->timer, ctx->f16, route, dense, shared));
    return FFMOE_OK;
}

int ffmoe_verify(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride, uint32_t t,
                 const uint32_t *idx, const uint16_t *w, const uint16_t *residual, uint16_t *y, char **err) {
    if (!y) return fail(err, FFMOE_ERR_INVALID, "null output");
    return verify_common(ctx, stream, layer, x, x_stride, t, idx, w, residual, y, nullptr, err);
}

int ffmoe_verify_static(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride, uint32_t t,
                        const uint32_t *idx, const uint16_t *w, const uint16_t *residual, uint16_t *y, char **err) {
    if (!ctx) return fail(err, FFMOE_ERR_INVALID, "null context");
    if (!y) return fail(err, FFMOE_ERR_INVALID, "null output");
    void *base = ctx->device >= 0 && ctx->device < kMaxDevices ? g_scratch_addr[ctx->device] : nullptr;
    if (!base) return fail(err, FFMOE_ERR_RUNTIME, "the static scratch has no address on device %d", ctx->device);
    const size_t routes = (size_t)FFMOE_MAX_VERIFY_ROWS * ctx->shape.top_k;
    const size_t acts_bytes = (routes * ctx->shape.f * sizeof(uint16_t) + 255) & ~(size_t)255;
    const size_t rows_bytes = routes * ctx->shape.d * sizeof(float);
    if (kStaticPlanBytes + acts_bytes + rows_bytes > kStaticScratchBytes)
        return fail(err, FFMOE_ERR_INVALID,
                    "d = %u, f = %u, top_k = %u need %zu bytes of scratch; the static array holds %zu (use ffmoe_verify)",
                    ctx->shape.d, ctx->shape.f, ctx->shape.top_k, kStaticPlanBytes + acts_bytes + rows_bytes, kStaticScratchBytes);
    uint8_t *p = static_cast<uint8_t *>(base);
    const VerifyScratch sc{reinterpret_cast<VerifyPlan *>(p), reinterpret_cast<uint16_t *>(p + kStaticPlanBytes),
                           reinterpret_cast<float *>(p + kStaticPlanBytes + acts_bytes)};
    // Nothing in the array has to start at zero: every call rewrites the plan it reads (all slot counts, the live
    // count and the live slots' route lists), and rows of the two buffers are read only where this call wrote them.
    return verify_common(ctx, stream, layer, x, x_stride, t, idx, w, residual, y, nullptr, err, &sc);
}

int ffmoe_route_verify(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *router_x, uint32_t router_x_stride,
                       const uint16_t *x, uint32_t x_stride, uint32_t t, const uint16_t *residual, uint16_t *y,
                       uint32_t *out_idx, uint16_t *out_w, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!router_x || !out_idx || !out_w) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (!y && residual) return fail(err, FFMOE_ERR_INVALID, "a residual needs y: without y the rows stay un-combined");
    if (router_x_stride < ctx->shape.d) return fail(err, FFMOE_ERR_INVALID, "hidden stride is too small");
    if (ctx->f16 && (reinterpret_cast<uintptr_t>(router_x) % 8 || router_x_stride % 4))
        return fail(err, FFMOE_ERR_INVALID, "FP16 router rows must be 8-byte aligned with a stride that is a multiple of 4");
    if (layer >= ctx->layers.size()) return fail(err, FFMOE_ERR_INVALID, "layer %u out of range", layer);
    const ffmoe_layer &l = ctx->layers[layer];
    const RouteFusion route{RouterWeights{l.router_w, l.router_is_f32, l.effective_scale, l.per_expert_scale}, router_x,
                            router_x_stride, ctx->logits, ctx->mail, ctx->handover_ticks, ctx->one_launch_routing,
                            ctx->route_resident_blocks};
    return verify_common(ctx, stream, layer, x, x_stride, t, out_idx, out_w, residual, y, nullptr, err, nullptr, &route);
}

int ffmoe_route_verify_shared(ffmoe_ctx *ctx, ffmoe_ctx *shared, void *stream, uint32_t layer, uint32_t shared_layer,
                              const uint16_t *router_x, uint32_t router_x_stride, const uint16_t *x, uint32_t x_stride,
                              const uint16_t *shared_x, uint32_t shared_x_stride, uint32_t t, uint32_t *out_idx,
                              uint16_t *out_w, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_ctx(shared, err)) return rc;
    if (!router_x || !out_idx || !out_w || !shared_x) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (!shared->dense_idx)
        return fail(err, FFMOE_ERR_INVALID, "the shared expert needs a context with n_experts = 1 and top_k = 1");
    if (shared == ctx) return fail(err, FFMOE_ERR_INVALID, "the shared expert lives in a context of its own");
    if (shared->device != ctx->device || shared->f16 != ctx->f16)
        return fail(err, FFMOE_ERR_INVALID, "the two contexts must share the device and the activation type");
    if (int rc = check_layer(shared, shared_layer, false, false, err)) return rc;
    const ffmoe_layer &shared_l = shared->layers[shared_layer];
    if (!shared_l.gate_up8)
        if (int rc = check_layer(shared, shared_layer, true, false, err)) return rc;
    const ArenaGeom &sg = shared->geom;
    if (sg.d != ctx->geom.d || ctx->geom.gf > kSharedChunkGroups || (ctx->geom.gd + 3) / 4 > kSharedChunkGroups ||
        shared_chunks(sg) > 4 || ctx->shape.top_k > 8)
        return fail(err, FFMOE_ERR_INVALID,
                    "the shared expert rides along when both have the same d <= 2816 and the routed experts' f <= 704 "
                    "(run ffmoe_dense_ffn and ffmoe_route_verify otherwise)");
    if (shared_x_stride < sg.d || shared_x_stride % 8 || reinterpret_cast<uintptr_t>(shared_x) % 16)
        return fail(err, FFMOE_ERR_INVALID, "shared_x must be 16-byte aligned with a stride that is a multiple of 8 and >= d");
    if (router_x_stride < ctx->shape.d) return fail(err, FFMOE_ERR_INVALID, "hidden stride is too small");
    if (ctx->f16 && (reinterpret_cast<uintptr_t>(router_x) % 8 || router_x_stride % 4))
        return fail(err, FFMOE_ERR_INVALID, "FP16 router rows must be 8-byte aligned with a stride that is a multiple of 4");
    if (layer >= ctx->layers.size()) return fail(err, FFMOE_ERR_INVALID, "layer %u out of range", layer);
    const ffmoe_layer &l = ctx->layers[layer];
    const RouteFusion route{RouterWeights{l.router_w, l.router_is_f32, l.effective_scale, l.per_expert_scale}, router_x,
                            router_x_stride, ctx->logits, ctx->mail, ctx->handover_ticks, ctx->one_launch_routing,
                            ctx->route_resident_blocks};
    SharedExpert sh{shared->arena + (size_t)shared_layer * shared->layer_bytes, sg, shared_x, shared_x_stride, shared->acts,
                    shared->partials};
    if (shared_l.gate_up8) {
        sh.gu_tiles8 = shared_l.gate_up8->tiles;
        sh.gu_scales8 = shared_l.gate_up8->scales;
        sh.dn_tiles8 = shared_l.down8->tiles;
        sh.dn_scales8 = shared_l.down8->scales;
    }
    return verify_common(ctx, stream, layer, x, x_stride, t, out_idx, out_w, nullptr, nullptr, nullptr, err, nullptr, &route,
                         false, &sh, shared);
}

int ffmoe_set_handover_timeout(ffmoe_ctx *ctx, void *stream, uint64_t ticks, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    FF_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    ctx->handover_ticks = ticks;
    FF_HIP(hipMemset(&ctx->mail->faults, 0, sizeof(uint32_t)));
    return FFMOE_OK;
}

int ffmoe_set_one_launch_routing(ffmoe_ctx *ctx, int enabled, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    ctx->one_launch_routing = enabled != 0;      // host state only: takes effect with the next call
    return FFMOE_OK;
}

int ffmoe_verify_partials(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                          uint32_t t, const uint32_t *idx, const uint16_t *w, uint16_t *partials, char **err) {
    if (!partials) return fail(err, FFMOE_ERR_INVALID, "null output");
    return verify_common(ctx, stream, layer, x, x_stride, t, idx, w, nullptr, nullptr, partials, err);
}

int ffmoe_last_live_experts(ffmoe_ctx *ctx, void *stream, uint32_t *n_live, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!n_live) return fail(err, FFMOE_ERR_INVALID, "null argument");
    FF_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    FF_HIP(hipMemcpy(n_live, &ctx->plan->n_live, sizeof(uint32_t), hipMemcpyDeviceToHost));
    return FFMOE_OK;
}

int ffmoe_probe_stream(ffmoe_ctx *ctx, void *stream, uint32_t layer, uint32_t n_live, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, true, false, err)) return rc;
    if (n_live == 0 || n_live > ctx->shape.n_experts)
        return fail(err, FFMOE_ERR_INVALID, "n_live = %u outside 1...%u", n_live, ctx->shape.n_experts);
    if ((ctx->geom.gd + 3) / 4 > 11 || ctx->geom.gf > 11)
        return fail(err, FFMOE_ERR_INVALID, "the stream probe covers the persistent kernels' shapes (d <= 2816, f <= 704)");
    // reads the arena only: no scratch of the context is touched
    FF_HIP(launch_probe_stream(static_cast<hipStream_t>(stream), ctx->arena + (size_t)layer * ctx->layer_bytes, ctx->geom,
                               ctx->shape.n_experts, n_live, ctx->n_cus, &ctx->timer));
    return FFMOE_OK;
}

int ffmoe_handover_giveups(ffmoe_ctx *ctx, void *stream, uint32_t *count, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!count) return fail(err, FFMOE_ERR_INVALID, "null argument");
    FF_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    FF_HIP(hipMemcpy(count, &ctx->mail->faults, sizeof(uint32_t), hipMemcpyDeviceToHost));
    return FFMOE_OK;
}

static int prefill_common(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride, uint32_t t,
                          const uint32_t *idx, const uint16_t *w, const ffmoe_pair *pairs, uint32_t n_pairs, uint16_t *y,
                          uint16_t *partials, char **err, bool dense = false) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, true, false, err)) return rc;
    if (!x) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (t == 0) return fail(err, FFMOE_ERR_INVALID, "queryCount must be positive");
    if ((size_t)t * ctx->shape.top_k > ctx->max_pairs)
        return fail(err, FFMOE_ERR_INVALID, "t = %u exceeds max_tokens = %u", t, ctx->shape.max_tokens);
    if (pairs && n_pairs > ctx->max_pairs)
        return fail(err, FFMOE_ERR_ALLOC, "prefill sorted route pairs exceed reusable capacity (%u > %u)", n_pairs, ctx->max_pairs);
    if (x_stride < ctx->shape.d || x_stride % 8 || reinterpret_cast<uintptr_t>(x) % 16)
        return fail(err, FFMOE_ERR_INVALID, "x must be 16-byte aligned with a stride that is a multiple of 8 and >= d");
    if ((y && reinterpret_cast<uintptr_t>(y) % 16) || (partials && reinterpret_cast<uintptr_t>(partials) % 16))
        return fail(err, FFMOE_ERR_INVALID, "outputs must be 16-byte aligned");
    claim_scratch(ctx, stream);
    FF_HIP(launch_prefill(static_cast<hipStream_t>(stream), ctx->arena + (size_t)layer * ctx->layer_bytes, ctx->geom,
                          ctx->shape.n_experts, ctx->shape.top_k, x, x_stride, t, idx, w, pairs, n_pairs, y, partials,
                          ctx->pf, &ctx->timer, ctx->f16, dense));
    return FFMOE_OK;
}

int ffmoe_prefill(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride, uint32_t t,
                  const uint32_t *idx, const uint16_t *w, uint16_t *y, char **err) {
    if (!idx || !w || !y) return fail(err, FFMOE_ERR_INVALID, "null argument");
    return prefill_common(ctx, stream, layer, x, x_stride, t, idx, w, nullptr, 0, y, nullptr, err);
}

int ffmoe_prefill_pairs(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride,
                        const ffmoe_pair *pairs, uint32_t n_pairs, uint32_t t, uint16_t *partials, char **err) {
    if (!partials) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (n_pairs == 0) return FFMOE_OK;
    if (!pairs) return fail(err, FFMOE_ERR_INVALID, "null argument");
    return prefill_common(ctx, stream, layer, x, x_stride, t, nullptr, nullptr, pairs, n_pairs, nullptr, partials, err);
}

int ffmoe_prefill_dump_tiles(ffmoe_ctx *ctx, void *stream, uint32_t layer, uint32_t expert, int gate_up, void *out,
                             size_t out_bytes, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, true, false, err)) return rc;
    if (expert >= ctx->shape.n_experts) return fail(err, FFMOE_ERR_INVALID, "expert %u out of range", expert);
    if (!out || reinterpret_cast<uintptr_t>(out) % 16) return fail(err, FFMOE_ERR_INVALID, "output must be a 16-byte aligned device pointer");
    const size_t need = (size_t)prefill_dump_fragments(ctx->geom, gate_up != 0) * 64 * sizeof(uint4);
    if (out_bytes < need) return fail(err, FFMOE_ERR_INVALID, "output holds %zu bytes, the fragments take %zu", out_bytes, need);
    claim_scratch(ctx, stream);
    FF_HIP(launch_prefill_dump_tiles(static_cast<hipStream_t>(stream), ctx->arena + (size_t)layer * ctx->layer_bytes, ctx->geom,
                                     expert, gate_up != 0, ctx->pf, out, ctx->f16));
    return FFMOE_OK;
}

int ffmoe_dense_ffn(ffmoe_ctx *ctx, void *stream, uint32_t layer, const uint16_t *x, uint32_t x_stride, uint32_t t,
                    uint16_t *y, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!ctx->dense_idx)
        return fail(err, FFMOE_ERR_INVALID, "the dense FFN needs a context with n_experts = 1 and top_k = 1");
    if (!y) return fail(err, FFMOE_ERR_INVALID, "null output");
    if (reinterpret_cast<uintptr_t>(y) % 16) return fail(err, FFMOE_ERR_INVALID, "y must be 16-byte aligned");
    if (int rc = check_layer(ctx, layer, false, false, err)) return rc;
    if (ctx->layers[layer].gate_up8) {
        // an 8-bit layer: the gated gate/up pass into the activation scratch, then the down pass
        const ffmoe_layer &l = ctx->layers[layer];
        const uint32_t cap = std::max<uint32_t>(ctx->shape.max_tokens, FFMOE_MAX_VERIFY_ROWS);
        if (!x || t == 0 || t > cap) return fail(err, FFMOE_ERR_INVALID, "rows = %u outside 1...%u", t, cap);
        if (x_stride < ctx->shape.d || x_stride % 8 || reinterpret_cast<uintptr_t>(x) % 16)
            return fail(err, FFMOE_ERR_INVALID, "x must be 16-byte aligned with a stride that is a multiple of 8 and >= d");
        hipStream_t s = static_cast<hipStream_t>(stream);
        claim_scratch(ctx, stream);
        if (t >= kGemm8MinRows && l.gate_up8_hilo) {
            // many rows: two dense GEMMs of the library on the hi / lo rows (fp32 sums), each followed by the pass that adds
            // a weight row's two columns and rounds as the streaming form does
            const uint32_t f = ctx->shape.f, d = ctx->shape.d;
            const rocblas_datatype dt = ctx->f16 ? rocblas_datatype_f16_r : rocblas_datatype_bf16_r;
            const float one = 1.0f, zero = 0.0f;
            auto gemm = [&](const uint16_t *w, uint32_t n_out, uint32_t k, const uint16_t *in, uint32_t in_stride) {
                // row-major sums[t][n_out] = in[t][k] . w[n_out][k]^T, i.e. column-major w^T in
                return rocblas_gemm_ex(ctx->blas, rocblas_operation_transpose, rocblas_operation_none, (rocblas_int)n_out, (rocblas_int)t,
                                       (rocblas_int)k, &one, w, dt, (rocblas_int)k, in, dt, (rocblas_int)in_stride, &zero,
                                       ctx->gemm8_sums, rocblas_datatype_f32_r, (rocblas_int)n_out, ctx->gemm8_sums,
                                       rocblas_datatype_f32_r, (rocblas_int)n_out, rocblas_datatype_f32_r, rocblas_gemm_algo_standard,
                                       0, 0);
            };
            if (rocblas_set_stream(ctx->blas, s) != rocblas_status_success) return fail(err, FFMOE_ERR_RUNTIME, "rocblas_set_stream failed");
            ctx->timer.begin(s);
            rocblas_status st = gemm(l.gate_up8_hilo, 4 * f, d, x, x_stride);
            if (st != rocblas_status_success) return fail(err, FFMOE_ERR_RUNTIME, "rocblas_gemm_ex (gate/up): status %d", (int)st);
            FF_HIP(launch_hilo_epilogue(s, ctx->gemm8_sums, t, f, true, ctx->pf.acts, f, ctx->f16));
            ctx->timer.mark(s, FFMOE_K_GATE_UP);
            st = gemm(l.down8_hilo, 2 * d, f, ctx->pf.acts, f);
            if (st != rocblas_status_success) return fail(err, FFMOE_ERR_RUNTIME, "rocblas_gemm_ex (down): status %d", (int)st);
            FF_HIP(launch_hilo_epilogue(s, ctx->gemm8_sums, t, d, false, y, d, ctx->f16));
            ctx->timer.mark(s, FFMOE_K_DOWN);
            ctx->timer.finish();
            return FFMOE_OK;
        }
        // two launches whatever the row count: a grid row per 16 input rows, each a pass of its own over the weights
        // (from the caches after the first); the activation rows of a block of more than 16 go to the prefill scratch
        uint16_t *acts = t <= FFMOE_MAX_VERIFY_ROWS ? ctx->acts : ctx->pf.acts;
        ctx->timer.begin(s);
        FF_HIP(launch_matrix_gemv(s, l.gate_up8->tiles, l.gate_up8->scales, ctx->shape.f, ctx->shape.d, x, x_stride, t, acts,
                                  ctx->shape.f, false, ctx->n_cus, ctx->f16, true, 1));
        ctx->timer.mark(s, FFMOE_K_GATE_UP);
        FF_HIP(launch_matrix_gemv(s, l.down8->tiles, l.down8->scales, ctx->shape.d, ctx->shape.f, acts, ctx->shape.f, t, y,
                                  ctx->shape.d, false, ctx->n_cus, ctx->f16, true, 0));
        ctx->timer.mark(s, FFMOE_K_DOWN);
        ctx->timer.finish();
        return FFMOE_OK;
    }
    // With one route per row at weight 1, the un-weighted bf16 row of route t is the output row t: the
    // down projection writes y itself and the combine pass has nothing to add.
    if (t <= FFMOE_MAX_VERIFY_ROWS)
        return verify_common(ctx, stream, layer, x, x_stride, t, ctx->dense_idx, ctx->dense_w, nullptr, nullptr, y, err, nullptr,
                             nullptr, true);
    if (t <= kDenseStreamMaxRows && matrix_shape_ok(ctx->shape.d) && matrix_shape_ok(ctx->shape.f) && ctx->shape.f % 16 == 0) {
        // 17 rows to a few hundred (a short prompt, a chunk's ragged end): below the row count at which the grouped GEMMs'
        // fixed cost (the weights' expansion per M-tile) is paid back, the resident-matrix GEMV streams the expert's arena
        // tiles as they lie - a gate/up tile's two streams are a gate and an up row block, a down tile is a plain 4-bit
        // matrix tile - with one grid row per 16 input rows: two launches.
        if (int rc = check_layer(ctx, layer, true, false, err)) return rc;
        const uint32_t cap = std::max<uint32_t>(ctx->shape.max_tokens, FFMOE_MAX_VERIFY_ROWS);
        if (!x || t > cap) return fail(err, FFMOE_ERR_INVALID, "t = %u exceeds max_tokens = %u", t, cap);
        if (x_stride < ctx->shape.d || x_stride % 8 || reinterpret_cast<uintptr_t>(x) % 16)
            return fail(err, FFMOE_ERR_INVALID, "x must be 16-byte aligned with a stride that is a multiple of 8 and >= d");
        const ArenaGeom &g = ctx->geom;
        const uint8_t *expert = ctx->arena + (size_t)layer * ctx->layer_bytes;
        hipStream_t s = static_cast<hipStream_t>(stream);
        claim_scratch(ctx, stream);
        ctx->timer.begin(s);
        FF_HIP(launch_matrix_gemv(s, expert + g.gu_tiles_off, expert + g.gu_scales_off, ctx->shape.f, ctx->shape.d, x, x_stride, t,
                                  ctx->pf.acts, ctx->shape.f, false, ctx->n_cus, ctx->f16, false, 2));
        ctx->timer.mark(s, FFMOE_K_GATE_UP);
        FF_HIP(launch_matrix_gemv(s, expert + g.dn_tiles_off, expert + g.dn_scales_off, ctx->shape.d, ctx->shape.f, ctx->pf.acts,
                                  ctx->shape.f, t, y, ctx->shape.d, false, ctx->n_cus, ctx->f16, false, 0));
        ctx->timer.mark(s, FFMOE_K_DOWN);
        ctx->timer.finish();
        return FFMOE_OK;
    }
    return prefill_common(ctx, stream, layer, x, x_stride, t, ctx->dense_idx, ctx->dense_w, nullptr, 0, nullptr, y, err, true);
}

int ffmoe_prefill_plan_stats(ffmoe_ctx *ctx, void *stream, uint32_t *n_pairs, uint32_t *n_tiles, uint32_t *counts,
                             char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    FF_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    PrefillPlan host;
    FF_HIP(hipMemcpy(&host, ctx->pf.plan, sizeof(PrefillPlan), hipMemcpyDeviceToHost));
    if (n_pairs) *n_pairs = host.n_pairs;
    if (n_tiles) *n_tiles = host.n_tiles;
    if (counts) memcpy(counts, host.expert_count, ctx->shape.n_experts * sizeof(uint32_t));
    return FFMOE_OK;
}

static int check_rows(uint32_t t, uint32_t d, const uint32_t *strides, int n_strides, char **err) {
    if (t == 0) return fail(err, FFMOE_ERR_INVALID, "queryCount must be positive");
    if (d == 0 || d > FFMOE_ROW_MAX_D || d % 8) return fail(err, FFMOE_ERR_INVALID, "D must be a multiple of 8 in 8...%d", FFMOE_ROW_MAX_D);
    for (int i = 0; i < n_strides; ++i)
        if (strides[i] < d) return fail(err, FFMOE_ERR_INVALID, "a row stride is too small");
    return FFMOE_OK;
}

int ffmoe_post_attn_setup(ffmoe_ctx *ctx, void *stream, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *attn,
                          uint32_t attn_stride, uint16_t *dense_x, uint32_t dense_stride, uint16_t *routed_x,
                          uint32_t routed_stride, uint16_t *router_x, uint32_t router_stride, const uint16_t *w_post_attn,
                          const uint16_t *w_pre_ffn, const uint16_t *w_pre_ffn2, uint32_t t, uint32_t d, float eps,
                          char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!hidden || !attn || !dense_x || !routed_x || !router_x || !w_post_attn || !w_pre_ffn || !w_pre_ffn2)
        return fail(err, FFMOE_ERR_INVALID, "null argument");
    const uint32_t strides[5] = {hidden_stride, attn_stride, dense_stride, routed_stride, router_stride};
    if (int rc = check_rows(t, d, strides, 5, err)) return rc;
    FF_HIP(launch_post_attn_setup(static_cast<hipStream_t>(stream), hidden, hidden_stride, attn, attn_stride, dense_x,
                                  dense_stride, routed_x, routed_stride, router_x, router_stride, w_post_attn, w_pre_ffn,
                                  w_pre_ffn2, t, d, eps, ctx->f16));
    return FFMOE_OK;
}

int ffmoe_layer_tail(ffmoe_ctx *ctx, void *stream, const uint16_t *h2, uint32_t h2_stride, const uint16_t *h1,
                     uint32_t h1_stride, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2,
                     const uint16_t *w_postffn, uint32_t t, uint32_t d, float eps, float layer_scalar, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!h2 || !h1 || !hidden || !w_postffn2 || !w_postffn) return fail(err, FFMOE_ERR_INVALID, "null argument");
    const uint32_t strides[3] = {h2_stride, h1_stride, hidden_stride};
    if (int rc = check_rows(t, d, strides, 3, err)) return rc;
    FF_HIP(launch_layer_tail(static_cast<hipStream_t>(stream), h2, h2_stride, h1, h1_stride, hidden, hidden_stride,
                             w_postffn2, w_postffn, t, d, eps, layer_scalar, nullptr, nullptr, nullptr, 0, ctx->f16));
    return FFMOE_OK;
}

int ffmoe_layer_tail_routed(ffmoe_ctx *ctx, void *stream, const uint16_t *route_w, const uint16_t *h1, uint32_t h1_stride,
                            uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn2, const uint16_t *w_postffn,
                            uint32_t t, float eps, float layer_scalar, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!route_w || !h1 || !hidden || !w_postffn2 || !w_postffn) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (t == 0 || t > FFMOE_MAX_VERIFY_ROWS) return fail(err, FFMOE_ERR_INVALID, "rows = %u outside 1...%d", t, FFMOE_MAX_VERIFY_ROWS);
    const uint32_t strides[2] = {h1_stride, hidden_stride};
    if (int rc = check_rows(t, ctx->shape.d, strides, 2, err)) return rc;
    claim_scratch(ctx, stream);      // the rows it combines are the context's
    FF_HIP(launch_layer_tail(static_cast<hipStream_t>(stream), nullptr, 0, h1, h1_stride, hidden, hidden_stride, w_postffn2,
                             w_postffn, t, ctx->shape.d, eps, layer_scalar, nullptr, nullptr, nullptr, 0, ctx->f16, ctx->partials,
                             route_w, ctx->plan->route_valid, ctx->shape.top_k));
    return FFMOE_OK;
}

int ffmoe_layer_tail_routed_shared(ffmoe_ctx *ctx, ffmoe_ctx *shared, void *stream, const uint16_t *route_w, uint16_t *hidden,
                                   uint32_t hidden_stride, const uint16_t *w_postffn2, const uint16_t *w_postffn, uint32_t t,
                                   float eps, float layer_scalar, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_ctx(shared, err)) return rc;
    if (!route_w || !hidden || !w_postffn2 || !w_postffn) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (!shared->dense_idx || shared == ctx || shared->geom.d != ctx->geom.d || shared->f16 != ctx->f16)
        return fail(err, FFMOE_ERR_INVALID, "the shared expert's context does not match (one expert, top_k = 1, same d and type)");
    if (t == 0 || t > FFMOE_MAX_VERIFY_ROWS) return fail(err, FFMOE_ERR_INVALID, "rows = %u outside 1...%d", t, FFMOE_MAX_VERIFY_ROWS);
    const uint32_t strides[1] = {hidden_stride};
    if (int rc = check_rows(t, ctx->shape.d, strides, 1, err)) return rc;
    claim_scratch(ctx, stream);
    claim_scratch(shared, stream);
    FF_HIP(launch_layer_tail(static_cast<hipStream_t>(stream), nullptr, 0, nullptr, 0, hidden, hidden_stride, w_postffn2,
                             w_postffn, t, ctx->shape.d, eps, layer_scalar, nullptr, nullptr, nullptr, 0, ctx->f16, ctx->partials,
                             route_w, ctx->plan->route_valid, ctx->shape.top_k, shared->partials, shared_chunks(shared->geom)));
    return FFMOE_OK;
}

int ffmoe_layer_tail_norms(ffmoe_ctx *ctx, void *stream, const uint16_t *h2, uint32_t h2_stride, const uint16_t *h1,
                           uint32_t h1_stride, uint16_t *hidden, uint32_t hidden_stride, const uint16_t *w_postffn1,
                           const uint16_t *w_postffn2, const uint16_t *w_postffn, const uint16_t *w_next, uint16_t *normed,
                           uint32_t normed_stride, uint32_t t, uint32_t d, float eps, float layer_scalar, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!h2 || !h1 || !hidden || !w_postffn1 || !w_postffn2 || !w_postffn) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if ((w_next == nullptr) != (normed == nullptr))
        return fail(err, FFMOE_ERR_INVALID, "the next layer's norm weight and its output go together");
    const uint32_t strides[4] = {h2_stride, h1_stride, hidden_stride, normed ? normed_stride : d};
    if (int rc = check_rows(t, d, strides, 4, err)) return rc;
    FF_HIP(launch_layer_tail(static_cast<hipStream_t>(stream), h2, h2_stride, h1, h1_stride, hidden, hidden_stride, w_postffn2,
                             w_postffn, t, d, eps, layer_scalar, w_postffn1, w_next, normed, normed_stride, ctx->f16));
    return FFMOE_OK;
}

int ffmoe_rmsnorm(ffmoe_ctx *ctx, void *stream, const uint16_t *x, uint32_t x_stride, const uint16_t *w, uint16_t *out,
                  uint32_t out_stride, uint32_t t, uint32_t d, float eps, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!x || !w || !out) return fail(err, FFMOE_ERR_INVALID, "null argument");
    const uint32_t strides[2] = {x_stride, out_stride};
    if (int rc = check_rows(t, d, strides, 2, err)) return rc;
    FF_HIP(launch_rmsnorm(static_cast<hipStream_t>(stream), x, x_stride, w, out, out_stride, t, d, eps, ctx->f16));
    return FFMOE_OK;
}

int ffmoe_set_activation_dtype(ffmoe_ctx *ctx, int dtype, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (dtype != FFMOE_BF16 && dtype != FFMOE_FP16) return fail(err, FFMOE_ERR_INVALID, "activation dtype %d is neither FFMOE_BF16 nor FFMOE_FP16", dtype);
    const bool f16 = dtype == FFMOE_FP16;
    if (f16 && !ctx->pf.act_scale) {
        // the FP16 prefill keeps its activations FP16 with a power-of-two scale per pair and 64-wide block of F
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&ctx->pf.act_scale), (size_t)ctx->pf.act_blocks * 16 * (ctx->geom.gf + 1) * sizeof(float));
        if (e != hipSuccess) return fail(err, FFMOE_ERR_ALLOC, "hipMalloc of the FP16 activation scales: %s", hipGetErrorString(e));
    }
    if (ctx->dense_w) {
        // the dense FFN's unit route weights follow the type
        const uint32_t cap = ctx->shape.max_tokens > FFMOE_MAX_VERIFY_ROWS ? ctx->shape.max_tokens : FFMOE_MAX_VERIFY_ROWS;
        FF_HIP(hipDeviceSynchronize());
        FF_HIP(hipMemsetD16(reinterpret_cast<hipDeviceptr_t>(ctx->dense_w), f16 ? 0x3C00 : 0x3F80, cap));
    }
    const bool changed = ctx->f16 != f16;
    ctx->f16 = f16;
    if (changed)
        for (auto &l : ctx->layers) FF_HIP(expand_int8_layer(ctx, l));      // the GEMM form's rows are of the activation type
    return FFMOE_OK;
}

int ffmoe_set_profiling(ffmoe_ctx *ctx, int enabled, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (enabled && !ctx->timer.ev[0])
        for (auto &ev : ctx->timer.ev) FF_HIP(hipEventCreate(&ev));
    ctx->timer.on = enabled != 0;
    return FFMOE_OK;
}

int ffmoe_get_profile(ffmoe_ctx *ctx, ffmoe_profile *out, int reset, char **err) {
    if (!ctx || !out) return fail(err, FFMOE_ERR_INVALID, "null argument");
    for (int i = 0; i < FFMOE_PROFILE_SLOTS; ++i) {
        out->ms[i] = ctx->timer.ms[i];
        out->launches[i] = ctx->timer.launches[i];
        if (reset) { ctx->timer.ms[i] = 0; ctx->timer.launches[i] = 0; }
    }
    return FFMOE_OK;
}

int ffmoe_reduce_token_major(ffmoe_ctx *ctx, void *stream, const uint16_t *partials, const uint16_t *weights,
                             uint16_t *h2, uint32_t t, uint32_t top_k, uint32_t d, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!partials || !weights || !h2) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (t == 0) return fail(err, FFMOE_ERR_INVALID, "queryCount must be positive");
    if (top_k == 0) return fail(err, FFMOE_ERR_INVALID, "topK must be positive");
    if (d == 0) return fail(err, FFMOE_ERR_INVALID, "D must be positive");
    FF_HIP(launch_reduce_token_major(static_cast<hipStream_t>(stream), partials, weights, h2, t, top_k, d, ctx->f16));
    return FFMOE_OK;
}

static int gemv_common(ffmoe_ctx *ctx, void *stream, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                       const uint32_t *ids, const uint16_t *x, void *y, uint32_t m, uint32_t n, uint32_t rows,
                       uint32_t x_stride, uint32_t y_stride, int y_f32, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!w || !scales || !biases || !x || !y) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (n == 0 || n % FFMOE_GROUP) return fail(err, FFMOE_ERR_INVALID, "N must be a multiple of %d", FFMOE_GROUP);
    if (reinterpret_cast<uintptr_t>(w) % 2) return fail(err, FFMOE_ERR_INVALID, "weights need a 2-aligned offset");
    if (m == 0) return fail(err, FFMOE_ERR_INVALID, "M must be positive");
    if (rows == 0 || rows > FFMOE_MAX_VERIFY_ROWS) return fail(err, FFMOE_ERR_INVALID, "rows=%u outside 1...%d", rows, FFMOE_MAX_VERIFY_ROWS);
    if (x_stride < n || y_stride < m) return fail(err, FFMOE_ERR_INVALID, "stride smaller than the row");
    ctx->timer.begin(static_cast<hipStream_t>(stream));
    if (ctx->f16 && (reinterpret_cast<uintptr_t>(x) % 16 || x_stride % 8))
        return fail(err, FFMOE_ERR_INVALID, "FP16 input rows must be 16-byte aligned with a stride that is a multiple of 8");
    FF_HIP(launch_gemv_int4(static_cast<hipStream_t>(stream), w, scales, biases, x, y, m, n, rows, x_stride, y_stride, y_f32, ids,
                            ctx->f16));
    ctx->timer.mark(static_cast<hipStream_t>(stream), FFMOE_K_GEMV);
    ctx->timer.finish();
    return FFMOE_OK;
}

int ffmoe_gemv_int4(ffmoe_ctx *ctx, void *stream, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                    const uint16_t *x, void *y, uint32_t m, uint32_t n, uint32_t rows, uint32_t x_stride,
                    uint32_t y_stride, int y_f32, char **err) {
    return gemv_common(ctx, stream, w, scales, biases, nullptr, x, y, m, n, rows, x_stride, y_stride, y_f32, err);
}

int ffmoe_gemv_int4_listed(ffmoe_ctx *ctx, void *stream, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                           const uint32_t *ids, const uint16_t *x, float *y, uint32_t m, uint32_t n, uint32_t rows,
                           uint32_t x_stride, uint32_t y_stride, char **err) {
    if (!ids) return fail(err, FFMOE_ERR_INVALID, "null argument");
    return gemv_common(ctx, stream, w, scales, biases, ids, x, y, m, n, rows, x_stride, y_stride, 1, err);
}

static int matrix_create_common(ffmoe_ctx *ctx, const uint8_t *w, const uint16_t *scales, const uint16_t *biases, uint32_t m,
                                uint32_t n, int with_greedy, bool planes8, ffmoe_matrix **out, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!w || !scales || !biases || !out) return fail(err, FFMOE_ERR_INVALID, "null argument");
    *out = nullptr;
    if (m == 0) return fail(err, FFMOE_ERR_INVALID, "M must be positive");
    if (n == 0 || !matrix_shape_ok(n))
        return fail(err, FFMOE_ERR_INVALID, "N = %u must be a multiple of %d and at most %d", n, FFMOE_GROUP,
                    FFMOE_MATRIX_MAX_N);
    if (!planes8 && reinterpret_cast<uintptr_t>(w) % 2) return fail(err, FFMOE_ERR_INVALID, "weights need a 2-aligned offset");
    // the kernels address the tile region through a buffer descriptor with 32-bit sizes and offsets
    if (matrix_tiles_bytes(m, n, planes8) >= ((size_t)1 << 32))
        return fail(err, FFMOE_ERR_INVALID, "M = %u x N = %u needs a tile region of %zu bytes; the limit is 4 GiB", m, n,
                    matrix_tiles_bytes(m, n, planes8));
    ffmoe_matrix *mx = new (std::nothrow) ffmoe_matrix();
    if (!mx) return fail(err, FFMOE_ERR_ALLOC, "out of host memory");
    mx->ctx = ctx;
    mx->device = ctx->device;
    mx->m = m;
    mx->n = n;
    mx->planes8 = planes8;
    const size_t w_bytes = planes8 ? (size_t)m * n : (size_t)m * n / 2, s_bytes = (size_t)m * (n / FFMOE_GROUP) * 2;
    uint8_t *stage = nullptr;
    auto cleanup = [&]() {
        if (stage) (void)hipFree(stage);
        if (mx->tiles) (void)hipFree(mx->tiles);
        if (mx->scales) (void)hipFree(mx->scales);
        if (mx->partials) (void)hipFree(mx->partials);
        delete mx;
    };
#define FF_MX(call)                                                                                   \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            cleanup();                                                                                \
            return fail(err, e_ == hipErrorOutOfMemory ? FFMOE_ERR_ALLOC : FFMOE_ERR_RUNTIME,         \
                        "%s: %s", #call, hipGetErrorString(e_));                                      \
        }                                                                                             \
    } while (0)
    FF_MX(hipMalloc(&mx->tiles, matrix_tiles_bytes(m, n, planes8)));
    FF_MX(hipMalloc(&mx->scales, matrix_scales_bytes(m, n, planes8)));
    if (with_greedy) {
        // per input row and block of the GEMV grid: the winner's key, then its softmax pair (8 bytes each)
        FF_MX(hipMalloc(&mx->partials, 2 * (size_t)FFMOE_MAX_VERIFY_ROWS * greedy_segments(m, ctx->n_cus) * sizeof(unsigned long long)));
    }
    // the source may live on the host (an mmap of the checkpoint) or on the device
    const uint8_t *dw = w;
    const uint16_t *ds = scales, *db = biases;
    hipPointerAttribute_t attr{};
    const bool on_device = hipPointerGetAttributes(&attr, w) == hipSuccess && attr.type == hipMemoryTypeDevice;
    (void)hipGetLastError();
    if (!on_device) {
        const size_t w_pad = (w_bytes + 15) / 16 * 16, s_pad = (s_bytes + 15) / 16 * 16;
        FF_MX(hipMalloc(&stage, w_pad + 2 * s_pad));
        FF_MX(hipMemcpy(stage, w, w_bytes, hipMemcpyHostToDevice));
        FF_MX(hipMemcpy(stage + w_pad, scales, s_bytes, hipMemcpyHostToDevice));
        FF_MX(hipMemcpy(stage + w_pad + s_pad, biases, s_bytes, hipMemcpyHostToDevice));
        dw = stage;
        ds = reinterpret_cast<const uint16_t *>(stage + w_pad);
        db = reinterpret_cast<const uint16_t *>(stage + w_pad + s_pad);
    }
    FF_MX(launch_matrix_repack(nullptr, dw, ds, db, m, n, mx->tiles, mx->scales, planes8));
    FF_MX(hipDeviceSynchronize());
#undef FF_MX
    if (stage) (void)hipFree(stage);
    ctx->matrices.push_back(mx);
    *out = mx;
    return FFMOE_OK;
}

int ffmoe_matrix_create(ffmoe_ctx *ctx, const uint8_t *w, const uint16_t *scales, const uint16_t *biases, uint32_t m,
                        uint32_t n, int with_greedy, ffmoe_matrix **out, char **err) {
    return matrix_create_common(ctx, w, scales, biases, m, n, with_greedy, false, out, err);
}

int ffmoe_matrix_create_int8(ffmoe_ctx *ctx, const uint8_t *w, const uint16_t *scales, const uint16_t *biases, uint32_t m,
                             uint32_t n, ffmoe_matrix **out, char **err) {
    return matrix_create_common(ctx, w, scales, biases, m, n, 0, true, out, err);
}

int ffmoe_matrix_create_int8_glu(ffmoe_ctx *ctx, const uint8_t *gate_w, const uint16_t *gate_scales, const uint16_t *gate_biases,
                                 const uint8_t *up_w, const uint16_t *up_scales, const uint16_t *up_biases, uint32_t f, uint32_t n,
                                 ffmoe_matrix **out, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!gate_w || !gate_scales || !gate_biases || !up_w || !up_scales || !up_biases || !out)
        return fail(err, FFMOE_ERR_INVALID, "null argument");
    *out = nullptr;
    if (f == 0 || f > (1u << 24)) return fail(err, FFMOE_ERR_INVALID, "F = %u outside 1...2^24", f);
    if (n == 0 || !matrix_shape_ok(n))
        return fail(err, FFMOE_ERR_INVALID, "N = %u must be a multiple of %d and at most %d", n, FFMOE_GROUP, FFMOE_MATRIX_MAX_N);
    // one source matrix on the device with the two projections' rows interleaved 16 at a time (rows past F stay zero)
    const uint32_t full = f / 16, rest = f % 16, rows2 = 32 * ((f + 15) / 16), groups = n / FFMOE_GROUP;
    const size_t w_bytes = (size_t)rows2 * n, s_bytes = (size_t)rows2 * groups * 2;
    const size_t w_pad = (w_bytes + 15) / 16 * 16, s_pad = (s_bytes + 15) / 16 * 16;
    uint8_t *stage = nullptr;
    hipPointerAttribute_t attr{};
    const bool on_device = hipPointerGetAttributes(&attr, gate_w) == hipSuccess && attr.type == hipMemoryTypeDevice;
    (void)hipGetLastError();
    const hipMemcpyKind kind = on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice;
    auto place = [&](uint8_t *dst, const void *src, size_t row_bytes, uint32_t half) -> hipError_t {
        hipError_t e = hipSuccess;
        if (full)
            e = hipMemcpy2D(dst + (size_t)half * 16 * row_bytes, 32 * row_bytes, src, 16 * row_bytes, 16 * row_bytes, full, kind);
        if (e == hipSuccess && rest)
            e = hipMemcpy(dst + ((size_t)32 * full + 16 * half) * row_bytes, static_cast<const uint8_t *>(src) + (size_t)full * 16 * row_bytes,
                          (size_t)rest * row_bytes, kind);
        return e;
    };
    hipError_t e = hipMalloc(&stage, w_pad + 2 * s_pad);
    if (e == hipSuccess) e = hipMemset(stage, 0, w_pad + 2 * s_pad);
    if (e == hipSuccess) e = place(stage, gate_w, n, 0);
    if (e == hipSuccess) e = place(stage, up_w, n, 1);
    if (e == hipSuccess) e = place(stage + w_pad, gate_scales, (size_t)groups * 2, 0);
    if (e == hipSuccess) e = place(stage + w_pad, up_scales, (size_t)groups * 2, 1);
    if (e == hipSuccess) e = place(stage + w_pad + s_pad, gate_biases, (size_t)groups * 2, 0);
    if (e == hipSuccess) e = place(stage + w_pad + s_pad, up_biases, (size_t)groups * 2, 1);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        if (stage) (void)hipFree(stage);
        return fail(err, e == hipErrorOutOfMemory ? FFMOE_ERR_ALLOC : FFMOE_ERR_RUNTIME, "staging the gate and up projections: %s",
                    hipGetErrorString(e));
    }
    const int rc = matrix_create_common(ctx, stage, reinterpret_cast<const uint16_t *>(stage + w_pad),
                                        reinterpret_cast<const uint16_t *>(stage + w_pad + s_pad), rows2, n, 0, true, out, err);
    (void)hipFree(stage);
    if (rc != FFMOE_OK) return rc;
    (*out)->glu = true;
    (*out)->m = f;
    return FFMOE_OK;
}

int ffmoe_upload_expert_parts_int8(ffmoe_ctx *ctx, uint32_t layer, const ffmoe_projection *gate, const ffmoe_projection *up,
                                   const ffmoe_projection *down, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (int rc = check_layer(ctx, layer, false, false, err)) return rc;
    if (!ctx->dense_idx)
        return fail(err, FFMOE_ERR_INVALID, "an 8-bit expert needs a context with n_experts = 1 and top_k = 1 (the shared expert's)");
    const ffmoe_projection *proj[3] = {gate, up, down};
    for (const ffmoe_projection *p : proj)
        if (!p || !p->w || !p->scales || !p->biases) return fail(err, FFMOE_ERR_INVALID, "null projection");
    const ffmoe_shape &sh = ctx->shape;
    if (!matrix_shape_ok(sh.d) || !matrix_shape_ok(sh.f))
        return fail(err, FFMOE_ERR_INVALID, "an 8-bit expert needs d and f that are multiples of %d and at most %d", FFMOE_GROUP,
                    FFMOE_MATRIX_MAX_N);
    ffmoe_matrix *gu = nullptr, *dn = nullptr;
    if (int rc = ffmoe_matrix_create_int8_glu(ctx, gate->w, gate->scales, gate->biases, up->w, up->scales, up->biases, sh.f, sh.d,
                                              &gu, err))
        return rc;
    if (int rc = ffmoe_matrix_create_int8(ctx, down->w, down->scales, down->biases, sh.d, sh.f, &dn, err)) {
        ffmoe_matrix_destroy(gu);
        return rc;
    }
    ffmoe_layer &l = ctx->layers[layer];
    drop_int8_form(l);
    l.gate_up8 = gu;
    l.down8 = dn;
    if (sh.max_tokens >= kGemm8MinRows) {
        // large row counts go through the library's dense GEMM on hi / lo rows of the activation type
        if (!ctx->blas && rocblas_create_handle(&ctx->blas) != rocblas_status_success) {
            ctx->blas = nullptr;
            drop_int8_form(l);
            return fail(err, FFMOE_ERR_RUNTIME, "rocblas_create_handle failed");
        }
        hipError_t e = hipSuccess;
        if (!ctx->gemm8_sums)
            e = hipMalloc(reinterpret_cast<void **>(&ctx->gemm8_sums),
                          (size_t)sh.max_tokens * std::max(4 * (size_t)sh.f, 2 * (size_t)sh.d) * sizeof(float));
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&l.gate_up8_hilo), (size_t)4 * sh.f * sh.d * sizeof(uint16_t));
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&l.down8_hilo), (size_t)2 * sh.d * sh.f * sizeof(uint16_t));
        if (e == hipSuccess) e = expand_int8_layer(ctx, l);
        if (e != hipSuccess) {
            drop_int8_form(l);
            return fail(err, e == hipErrorOutOfMemory ? FFMOE_ERR_ALLOC : FFMOE_ERR_RUNTIME, "the GEMM form of the 8-bit layer: %s",
                        hipGetErrorString(e));
        }
    }
    return FFMOE_OK;
}

int ffmoe_gelu_mul(ffmoe_ctx *ctx, void *stream, const uint16_t *gate, uint32_t gate_stride, const uint16_t *up,
                   uint32_t up_stride, uint16_t *out, uint32_t out_stride, uint32_t rows, uint32_t count, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!gate || !up || !out) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (rows == 0 || count == 0) return fail(err, FFMOE_ERR_INVALID, "rows and count must be positive");
    if (gate_stride < count || up_stride < count || out_stride < count) return fail(err, FFMOE_ERR_INVALID, "stride smaller than the row");
    if (rows > 65535u) return fail(err, FFMOE_ERR_INVALID, "rows = %u: at most 65535 per call", rows);
    FF_HIP(launch_gelu_mul(static_cast<hipStream_t>(stream), gate, gate_stride, up, up_stride, out, out_stride, rows, count, ctx->f16));
    return FFMOE_OK;
}

void ffmoe_matrix_destroy(ffmoe_matrix *mx) {
    if (!mx) return;
    if (mx->ctx) {      // still owned: release the device memory and leave the context's list
        (void)hipSetDevice(mx->device);
        (void)hipDeviceSynchronize();
        if (mx->tiles) (void)hipFree(mx->tiles);
        if (mx->scales) (void)hipFree(mx->scales);
        if (mx->partials) (void)hipFree(mx->partials);
        auto &list = mx->ctx->matrices;
        for (size_t i = 0; i < list.size(); ++i)
            if (list[i] == mx) {
                list.erase(list.begin() + (long)i);
                break;
            }
    }
    delete mx;
}

static int check_matrix_call(ffmoe_matrix *mx, const uint16_t *x, uint32_t x_stride, uint32_t rows, char **err) {
    if (!mx) return fail(err, FFMOE_ERR_INVALID, "null matrix");
    if (!mx->ctx) return fail(err, FFMOE_ERR_INVALID, "the matrix's context was destroyed");
    if (int rc = check_ctx(mx->ctx, err)) return rc;
    if (!x) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (rows == 0 || rows > FFMOE_MAX_VERIFY_ROWS)
        return fail(err, FFMOE_ERR_INVALID, "rows=%u outside 1...%d", rows, FFMOE_MAX_VERIFY_ROWS);
    if (x_stride < mx->n || x_stride % 8 || reinterpret_cast<uintptr_t>(x) % 16)
        return fail(err, FFMOE_ERR_INVALID, "x must be 16-byte aligned with a row stride that is a multiple of 8 and >= N");
    return FFMOE_OK;
}

int ffmoe_matrix_gemv(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows, void *y,
                      uint32_t y_stride, int y_f32, char **err) {
    if (int rc = check_matrix_call(mx, x, x_stride, rows, err)) return rc;
    if (!y) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (y_stride < mx->m) return fail(err, FFMOE_ERR_INVALID, "stride smaller than the row");
    ffmoe_ctx *ctx = mx->ctx;
    ctx->timer.begin(static_cast<hipStream_t>(stream));
    FF_HIP(launch_matrix_gemv(static_cast<hipStream_t>(stream), mx->tiles, mx->scales, mx->m, mx->n, x, x_stride, rows,
                              y, y_stride, y_f32 != 0, ctx->n_cus, ctx->f16, mx->planes8, mx->glu ? 1 : 0));
    ctx->timer.mark(static_cast<hipStream_t>(stream), FFMOE_K_GEMV);
    ctx->timer.finish();
    return FFMOE_OK;
}

int ffmoe_matrix_rows(ffmoe_matrix *mx, void *stream, const uint32_t *ids, uint32_t count, uint32_t token_id, float out_scale,
                      uint16_t *out, uint32_t out_stride, char **err) {
    if (!mx) return fail(err, FFMOE_ERR_INVALID, "null matrix");
    if (!mx->ctx) return fail(err, FFMOE_ERR_INVALID, "the matrix's context was destroyed");
    if (int rc = check_ctx(mx->ctx, err)) return rc;
    if (mx->planes8) return fail(err, FFMOE_ERR_INVALID, "rows are looked up in a 4-bit matrix (the reference's embedding table is 4-bit)");
    if (!out) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (count == 0 || count > 65535u) return fail(err, FFMOE_ERR_INVALID, "count = %u outside 1...65535", count);
    if (!ids && count != 1) return fail(err, FFMOE_ERR_INVALID, "without an id list the call looks up the one row token_id");
    if (out_stride < mx->n || out_stride % 8 || reinterpret_cast<uintptr_t>(out) % 16)
        return fail(err, FFMOE_ERR_INVALID, "out must be 16-byte aligned with a row stride that is a multiple of 8 and >= N");
    if (!std::isfinite(out_scale)) return fail(err, FFMOE_ERR_INVALID, "out_scale must be finite");
    FF_HIP(launch_matrix_rows(static_cast<hipStream_t>(stream), mx->tiles, mx->scales, mx->m, mx->n, ids, token_id, count, out_scale,
                              out, out_stride, mx->ctx->f16));
    return FFMOE_OK;
}

static int matrix_greedy_common(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows,
                                float softcap, uint32_t *out_tokens, float *out_conf, char **err) {
    if (int rc = check_matrix_call(mx, x, x_stride, rows, err)) return rc;
    if (!out_tokens) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (!mx->partials || mx->planes8) return fail(err, FFMOE_ERR_INVALID, "matrix was created without the greedy scratch");
    if (!(softcap >= 0.0f) || std::isinf(softcap)) return fail(err, FFMOE_ERR_INVALID, "softcap must be finite and >= 0 (0 disables it)");
    ffmoe_ctx *ctx = mx->ctx;
    hipStream_t s = static_cast<hipStream_t>(stream);
    claim_scratch(ctx, stream);      // the per-block winners go through the matrix's scratch
    ctx->timer.begin(s);
    FF_HIP(launch_matrix_greedy(s, mx->tiles, mx->scales, mx->m, mx->n, x, x_stride, rows, mx->partials, out_tokens,
                                ctx->n_cus, ctx->f16, &ctx->timer, softcap, out_conf));
    ctx->timer.finish();
    return FFMOE_OK;
}

int ffmoe_matrix_greedy(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows,
                        uint32_t *out_tokens, char **err) {
    return matrix_greedy_common(mx, stream, x, x_stride, rows, 0.0f, out_tokens, nullptr, err);
}

int ffmoe_matrix_greedy_conf(ffmoe_matrix *mx, void *stream, const uint16_t *x, uint32_t x_stride, uint32_t rows,
                             float softcap, uint32_t *out_tokens, float *out_conf, char **err) {
    if (!out_conf) return fail(err, FFMOE_ERR_INVALID, "null argument");
    return matrix_greedy_common(mx, stream, x, x_stride, rows, softcap, out_tokens, out_conf, err);
}

int ffmoe_argmax_rows(ffmoe_ctx *ctx, void *stream, const float *logits, uint32_t stride, uint32_t rows, uint32_t count,
                      float softcap, uint32_t *out_index, float *out_conf, char **err) {
    if (int rc = check_ctx(ctx, err)) return rc;
    if (!logits || !out_index) return fail(err, FFMOE_ERR_INVALID, "null argument");
    if (rows == 0 || count == 0) return fail(err, FFMOE_ERR_INVALID, "rows and count must be positive");
    if (stride < count) return fail(err, FFMOE_ERR_INVALID, "stride smaller than the row");
    if (!(softcap >= 0.0f) || std::isinf(softcap)) return fail(err, FFMOE_ERR_INVALID, "softcap must be finite and >= 0 (0 disables it)");
    hipStream_t s = static_cast<hipStream_t>(stream);
    ctx->timer.begin(s);
    FF_HIP(launch_argmax_rows(s, logits, stride, rows, count, softcap, out_index, out_conf));
    ctx->timer.mark(s, FFMOE_K_ARGMAX);
    ctx->timer.finish();
    return FFMOE_OK;
}

}  // extern "C"
