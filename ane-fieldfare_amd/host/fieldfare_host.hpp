// Host-side mirror of the reference's Swift operator surface for the routed-expert stage, written
// over the C ABI of include/fieldfare_moe.h only (no HIP types: a stream is an opaque void*).
//
// The reference's host code is Swift; this image has no Swift toolchain, so the mirror is C++17 with
// the same names, argument meaning and error behaviour. Shape misuse, a Swift `precondition` trap in
// the reference, throws std::invalid_argument here; resource failures throw FieldfareError carrying
// the library's message (the reference throws MetalError / PrefillGroupedRoutedMoEError).
//
//   reference type (file)                                              -> here
//   MoEExpertOffsets              Kernels/MoE/MoE.swift:4-29            -> ffmoe_offsets (C ABI)
//   PrefillTokenExpertPair        Kernels/Prefill/MoE/PrefillRouter.swift:5-21 -> PrefillTokenExpertPair
//   PrefillRouter.makeTokenExpertPairs            PrefillRouter.swift:75-95    -> PrefillRouter::makeTokenExpertPairs
//   PrefillMoEGrouping.groupTokenExpertPairs      PrefillMoEGrouping.swift:49-110 -> PrefillMoEGrouping::groupTokenExpertPairs
//   PrefillStreamedTileBinding    PrefillGroupedRoutedMoE.swift:121-166 -> PrefillStreamedTileBinding
//   MoE (router, decode phases)   Kernels/MoE/MoE.swift:31-507          -> MoE
//   PrefillRouter.encodeGemma4Block               PrefillRouter.swift:30-73    -> PrefillRouter::encodeGemma4Block
//   PrefillGroupedRoutedMoE       PrefillGroupedRoutedMoE.swift:183-448 -> PrefillGroupedRoutedMoE
//   PrefillMoE.encodeReduceTokenMajor             PrefillMoE.swift:11-32       -> PrefillMoE::encodeReduceTokenMajor
//   DequantInt4GEMV               Kernels/Quant/DequantInt4GEMV.swift   -> DequantInt4GEMV
//   activeRoutedExperts, prefillExpertUnionCap    Runtime/Inference/RealForwardRunner.swift:818-847,1952-1961 -> RouteTrimming
//   RoutedPrefillGuest, DeviceSupervisor, RuntimeFaultPolicy, GuestFault
//                                 Runtime/Supervisor/DeviceSupervisor.swift:5-125 -> same names
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <memory>
#include <optional>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/fieldfare_moe.h"

namespace fieldfare {

struct FieldfareError : std::runtime_error {
    int code;
    FieldfareError(int c, const std::string &m) : std::runtime_error(m), code(c) {}
};

inline void check(int rc, char *err) {
    if (rc == FFMOE_OK) return;
    std::string msg = err ? err : "(no message)";
    std::free(err);
    throw FieldfareError(rc, msg);
}

// One ffmoe_ctx. Plays the part of MetalContext + the resident expert store for the operators below.
class Context {
public:
    Context(int device, const ffmoe_shape &shape) : shape_(shape) {
        char *err = nullptr;
        check(ffmoe_create(device, &shape, &ctx_, &err), err);
    }
    ~Context() { ffmoe_destroy(ctx_); }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    ffmoe_ctx *raw() const { return ctx_; }
    const ffmoe_shape &shape() const { return shape_; }

    // FFMOE_BF16 (default) or FFMOE_FP16, the reference's text-path type: what every 16-bit row handed to or
    // returned by the operators below is. Set before the first encode call.
    void setActivationDtype(int dtype) {
        char *err = nullptr;
        if (dtype != FFMOE_BF16 && dtype != FFMOE_FP16) throw std::invalid_argument("activation dtype is FFMOE_BF16 or FFMOE_FP16");
        check(ffmoe_set_activation_dtype(ctx_, dtype, &err), err);
    }

    void uploadLayer(uint32_t layer, const void *blobs, size_t stride, const ffmoe_offsets &offsets, bool onDevice = false) {
        char *err = nullptr;
        check(ffmoe_upload_layer(ctx_, layer, blobs, stride, &offsets, onDevice ? 1 : 0, &err), err);
    }
    void uploadRouterBF16(uint32_t layer, const uint16_t *w, const uint16_t *effectiveScale = nullptr,
                          const uint16_t *perExpertScale = nullptr) {
        char *err = nullptr;
        check(ffmoe_upload_router_bf16(ctx_, layer, w, effectiveScale, perExpertScale, &err), err);
    }
    void uploadRouterInt8(uint32_t layer, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                          const uint16_t *effectiveScale = nullptr, const uint16_t *perExpertScale = nullptr) {
        char *err = nullptr;
        check(ffmoe_upload_router_int8(ctx_, layer, w, scales, biases, effectiveScale, perExpertScale, &err), err);
    }

private:
    ffmoe_ctx *ctx_ = nullptr;
    ffmoe_shape shape_;
};

// ---------------------------------------------------------------------------------------------------
// Pair building and grouping: pure host logic (no GPU).
// ---------------------------------------------------------------------------------------------------
struct PrefillTokenExpertPair {
    uint32_t token, expert, rank, weightBitsAndReserved;
    bool operator==(const PrefillTokenExpertPair &o) const {
        return token == o.token && expert == o.expert && rank == o.rank && weightBitsAndReserved == o.weightBitsAndReserved;
    }
};
static_assert(sizeof(PrefillTokenExpertPair) == sizeof(ffmoe_pair), "pairs cross the C ABI as they are");

struct PrefillMoEGroup {
    uint32_t expert, pairStart, pairCount;
    bool operator==(const PrefillMoEGroup &o) const { return expert == o.expert && pairStart == o.pairStart && pairCount == o.pairCount; }
};

struct PrefillMoETile {
    uint32_t groupStart, groupCount, pairStart, pairCount;
    bool operator==(const PrefillMoETile &o) const {
        return groupStart == o.groupStart && groupCount == o.groupCount && pairStart == o.pairStart && pairCount == o.pairCount;
    }
};

struct PrefillMoEGroupedRoutes {
    std::vector<PrefillTokenExpertPair> sortedPairs;
    std::vector<PrefillMoEGroup> groups;
    std::vector<PrefillMoETile> tiles;
};

struct PrefillMoEGroupingError : std::runtime_error {
    uint32_t expert;
    explicit PrefillMoEGroupingError(uint32_t e)
        : std::runtime_error("route expert " + std::to_string(e) + " is out of range"), expert(e) {}
};

struct PrefillMoEGrouping {
    // The contract of PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:49-110): the pairs ordered by
    // (expertSortKeys[expert] if given, expert, token, rank), one group per expert that has pairs, tiles of up to
    // tileExpertCount consecutive groups. Built as a bucket pass rather than one comparison sort over all pairs: the
    // experts are put in order once, every pair drops into its expert's bucket (two linear passes), and only the
    // inside of a bucket is sorted - a no-op for pairs that arrive token-major, as makeTokenExpertPairs emits them.
    static PrefillMoEGroupedRoutes groupTokenExpertPairs(const std::vector<PrefillTokenExpertPair> &pairs, int queryCount,
                                                         int topK, int numExperts, int tileExpertCount,
                                                         const std::vector<uint64_t> *expertSortKeys = nullptr) {
        if (!(queryCount >= 0 && topK > 0 && numExperts > 0 && tileExpertCount >= 1 && tileExpertCount <= 16))
            throw std::invalid_argument("groupTokenExpertPairs: bad arguments");
        if (pairs.size() > (size_t)queryCount * (size_t)topK) throw std::invalid_argument("more pairs than queryCount * topK");
        if (expertSortKeys && expertSortKeys->size() != (size_t)numExperts) throw std::invalid_argument("expertSortKeys count mismatch");
        std::vector<uint32_t> bucketSize((size_t)numExperts, 0);
        for (const auto &p : pairs) {
            if (p.expert >= (uint32_t)numExperts) throw PrefillMoEGroupingError(p.expert);
            ++bucketSize[p.expert];
        }
        // the experts in output order
        std::vector<uint32_t> order((size_t)numExperts);
        for (uint32_t e = 0; e < (uint32_t)numExperts; ++e) order[e] = e;
        if (expertSortKeys)
            std::stable_sort(order.begin(), order.end(),
                             [&](uint32_t x, uint32_t y) { return (*expertSortKeys)[x] < (*expertSortKeys)[y]; });
        // where each expert's bucket starts; a group per non-empty bucket
        PrefillMoEGroupedRoutes out;
        std::vector<uint32_t> cursor((size_t)numExperts, 0);
        uint32_t filled = 0;
        for (uint32_t e : order) {
            cursor[e] = filled;
            if (bucketSize[e]) out.groups.push_back({e, filled, bucketSize[e]});
            filled += bucketSize[e];
        }
        out.sortedPairs.resize(pairs.size());
        for (const auto &p : pairs) out.sortedPairs[cursor[p.expert]++] = p;
        auto position = [](const PrefillTokenExpertPair &p) { return ((uint64_t)p.token << 32) | p.rank; };
        for (const auto &g : out.groups) {
            auto first = out.sortedPairs.begin() + g.pairStart, last = first + g.pairCount;
            if (!std::is_sorted(first, last, [&](const auto &x, const auto &y) { return position(x) < position(y); }))
                std::sort(first, last, [&](const auto &x, const auto &y) { return position(x) < position(y); });
        }
        for (size_t at = 0; at < out.groups.size(); at += (size_t)tileExpertCount) {
            const size_t n = std::min((size_t)tileExpertCount, out.groups.size() - at);
            const PrefillMoEGroup &head = out.groups[at], &tail = out.groups[at + n - 1];
            out.tiles.push_back({(uint32_t)at, (uint32_t)n, head.pairStart, tail.pairStart + tail.pairCount - head.pairStart});
        }
        return out;
    }
};

// The reference's two lossy routing options, applied on the host to a block's routes between the router and the
// expert pass, as the reference does on its shared-memory route buffers (both are off by default there):
//   activeRoutedExperts < topK   RealForwardRunner.swift:1952-1961: only the first `active` ranks of a row run, their
//                                weights rescaled so that the row keeps the total of all topK weights;
//   prefillExpertUnionCap        RealForwardRunner.swift:818-847 (capExpertUnion): a block keeps the `cap` experts with
//                                the most routed weight (ties to the lower expert), each row's kept weights rescaled to
//                                the row's original total, the others set to zero.
// Weights are 16-bit patterns in the context's activation type: bf16 (the default) or FP16. A route whose weight is
// zero takes no part in ffmoe_verify / ffmoe_prefill, which is how the trimmed routes drop out of the expert pass.
struct RouteTrimming {
    enum class WeightType { bf16, fp16 };

    static float widen(uint16_t bits, WeightType type) {
        if (type == WeightType::fp16) {
            const uint32_t sign = (uint32_t)(bits & 0x8000u) << 16, exp = (bits >> 10) & 0x1Fu, man = bits & 0x3FFu;
            uint32_t u;
            if (exp == 0x1Fu) {
                u = sign | 0x7F800000u | (man << 13);                       // infinity, NaN
            } else if (exp != 0) {
                u = sign | ((exp + 112u) << 23) | (man << 13);
            } else if (man == 0) {
                u = sign;
            } else {                                                        // subnormal: man * 2^-24, exact in fp32
                float f = (float)man * 0x1p-24f;
                std::memcpy(&u, &f, sizeof u);
                u |= sign;
            }
            float f;
            std::memcpy(&f, &u, sizeof f);
            return f;
        }
        const uint32_t u = (uint32_t)bits << 16;
        float f;
        std::memcpy(&f, &u, sizeof f);
        return f;
    }
    static uint16_t narrow(float value, WeightType type) {
        uint32_t u;
        std::memcpy(&u, &value, sizeof u);
        if (type == WeightType::fp16) {
            // round to nearest even, as a conversion instruction does
            const uint32_t sign = (u >> 16) & 0x8000u, mag = u & 0x7FFFFFFFu;
            if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);                     // NaN
            if (mag >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);                    // rounds to 65520 or more: infinity
            if (mag < 0x33000001u) return (uint16_t)sign;                                 // at most half the smallest subnormal: zero
            if (mag < 0x38800000u) {                                                      // subnormal result: whole multiples of 2^-24
                float f;
                std::memcpy(&f, &mag, sizeof f);
                const float scaled = f * 0x1p24f;                                         // exact
                uint32_t q = (uint32_t)scaled;
                const float rest = scaled - (float)q;
                if (rest > 0.5f || (rest == 0.5f && (q & 1u))) ++q;
                return (uint16_t)(sign | q);
            }
            const uint32_t rounded = mag + 0xFFFu + ((mag >> 13) & 1u);
            return (uint16_t)(sign | ((rounded - 0x38000000u) >> 13));
        }
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);      // NaN stays NaN
        return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);                            // round to nearest even
    }

    // weights [rows][topK], in place: ranks >= active become zero, the others are rescaled by full / kept (left alone
    // when the kept weights add up to zero)
    static void keepActiveRanks(uint16_t *weights, int rows, int topK, int active, WeightType type = WeightType::bf16) {
        if (!(rows >= 0 && topK > 0 && active >= 1 && active <= topK)) throw std::invalid_argument("keepActiveRanks: bad arguments");
        if (active == topK) return;
        for (int row = 0; row < rows; ++row) {
            uint16_t *w = weights + (size_t)row * topK;
            float full = 0.0f, kept = 0.0f;
            for (int r = 0; r < topK; ++r) full += widen(w[r], type);
            for (int r = 0; r < active; ++r) kept += widen(w[r], type);
            if (kept != 0.0f)
                for (int r = 0; r < active; ++r) w[r] = narrow(widen(w[r], type) * full / kept, type);
            for (int r = active; r < topK; ++r) w[r] = 0;
        }
    }

    // ids, weights [rows][topK]; weights are changed in place. Returns the number of distinct experts before the cap.
    static int capExpertUnion(const uint32_t *ids, uint16_t *weights, int rows, int topK, int numExperts, int cap,
                              WeightType type = WeightType::bf16) {
        if (!(rows >= 0 && topK > 0 && numExperts > 0 && cap >= 1)) throw std::invalid_argument("capExpertUnion: bad arguments");
        const size_t count = (size_t)rows * topK;
        std::vector<float> mass((size_t)numExperts, 0.0f);
        std::vector<char> seen((size_t)numExperts, 0);
        int distinct = 0;
        for (size_t i = 0; i < count; ++i) {
            if (ids[i] >= (uint32_t)numExperts) throw std::invalid_argument("router wrote an expert past the expert count");
            if (!seen[ids[i]]) {
                seen[ids[i]] = 1;
                ++distinct;
            }
            const float w = widen(weights[i], type);
            mass[ids[i]] += w < 0.0f ? -w : w;
        }
        if (distinct <= cap) return distinct;
        std::vector<uint32_t> order;
        for (uint32_t e = 0; e < (uint32_t)numExperts; ++e)
            if (mass[e] > 0.0f) order.push_back(e);
        std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return mass[x] > mass[y]; });
        std::vector<char> retained((size_t)numExperts, 0);
        for (size_t i = 0; i < order.size() && i < (size_t)cap; ++i) retained[order[i]] = 1;
        for (int row = 0; row < rows; ++row) {
            uint16_t *w = weights + (size_t)row * topK;
            const uint32_t *id = ids + (size_t)row * topK;
            float original = 0.0f, kept = 0.0f;
            for (int r = 0; r < topK; ++r) original += widen(w[r], type);
            for (int r = 0; r < topK; ++r)
                if (retained[id[r]]) kept += widen(w[r], type);
            const float scale = kept != 0.0f ? original / kept : 0.0f;
            for (int r = 0; r < topK; ++r) w[r] = retained[id[r]] ? narrow(widen(w[r], type) * scale, type) : (uint16_t)0;
        }
        return distinct;
    }
};

struct PrefillGroupedRoutedMoEError : std::runtime_error {
    enum Kind { invalidStreamedTileBinding, allocationFailed } kind;
    PrefillGroupedRoutedMoEError(Kind k, const std::string &reason)
        : std::runtime_error((k == invalidStreamedTileBinding ? "invalid streamed tile binding: " : "failed to allocate ") + reason), kind(k) {}
};

// PrefillGroupedRoutedMoE.swift:121-166. With every expert resident in HBM a binding carries expert ids
// only (the reference also carries one TensorView per expert); the validation rules are the same.
struct PrefillStreamedTileBinding {
    std::vector<int> expertIDs;
    explicit PrefillStreamedTileBinding(std::vector<int> ids) : expertIDs(std::move(ids)) {
        using E = PrefillGroupedRoutedMoEError;
        if (expertIDs.empty()) throw E(E::invalidStreamedTileBinding, "tile binding must include at least one expert");
        if (expertIDs.size() > 16)
            throw E(E::invalidStreamedTileBinding, "tile binding has " + std::to_string(expertIDs.size()) + " experts; maximum is 16");
        std::set<int> seen;
        for (int e : expertIDs) {
            if (e < 0) throw E(E::invalidStreamedTileBinding, "expert id " + std::to_string(e) + " must be non-negative");
            if (!seen.insert(e).second) throw E(E::invalidStreamedTileBinding, "duplicate expert id " + std::to_string(e) + " in tile binding");
        }
    }
    static std::vector<int> expertIDsForTile(int tileIndex, const PrefillMoEGroupedRoutes &routes) {
        const auto &tile = routes.tiles.at(tileIndex);
        std::vector<int> ids;
        for (uint32_t g = tile.groupStart; g < tile.groupStart + tile.groupCount; ++g) ids.push_back((int)routes.groups[g].expert);
        return ids;
    }
};

// ---------------------------------------------------------------------------------------------------
// Operators. Every encode... enqueues on `stream` and returns; device pointers are caller-owned.
// ---------------------------------------------------------------------------------------------------
class PrefillRouter {
public:
    explicit PrefillRouter(Context &c) : c_(c) {}
    // PrefillRouter.swift:30-73
    void encodeGemma4Block(void *stream, uint32_t layer, const uint16_t *hidden, uint32_t *outIndices, uint16_t *outWeights,
                           uint32_t queryCount, uint32_t hiddenStrideElements) {
        if (queryCount == 0) throw std::invalid_argument("queryCount must be positive");
        if (hiddenStrideElements < c_.shape().d) throw std::invalid_argument("hidden stride is too small");
        char *err = nullptr;
        check(ffmoe_router(c_.raw(), stream, layer, hidden, hiddenStrideElements, queryCount, outIndices, outWeights, nullptr, &err), err);
    }
    // PrefillRouter.swift:75-95: token-major pairs; weights are 16-bit patterns
    static std::vector<PrefillTokenExpertPair> makeTokenExpertPairs(const std::vector<uint32_t> &indices,
                                                                    const std::vector<uint16_t> &weights, int queryCount, int topK) {
        if (queryCount < 0) throw std::invalid_argument("queryCount must be non-negative");
        if (topK < 0) throw std::invalid_argument("topK must be non-negative");
        if (indices.size() != (size_t)queryCount * topK) throw std::invalid_argument("indices count mismatch");
        if (weights.size() != (size_t)queryCount * topK) throw std::invalid_argument("weights count mismatch");
        std::vector<PrefillTokenExpertPair> pairs;
        pairs.reserve(indices.size());
        for (int token = 0; token < queryCount; ++token)
            for (int rank = 0; rank < topK; ++rank) {
                const size_t i = (size_t)token * topK + rank;
                pairs.push_back({(uint32_t)token, indices[i], (uint32_t)rank, (uint32_t)weights[i]});
            }
        return pairs;
    }

private:
    Context &c_;
};

class MoE {
public:
    static constexpr int maxStreamedExperts = 8;
    static constexpr int maxRouterRows = 16;
    explicit MoE(Context &c) : c_(c) {}
    // MoE.encodeRouterGemma4 (MoE.swift:168-237): one hidden row
    void encodeRouterGemma4(void *stream, uint32_t layer, const uint16_t *hidden, uint32_t *outIndices, uint16_t *outWeights) {
        encodeRouterRowsGemma4(stream, layer, hidden, c_.shape().d, 1, outIndices, outWeights);
    }
    // MoE.encodeRouterRowsGemma4 (MoE.swift:249-300): rows <= 16 hidden rows of a block
    void encodeRouterRowsGemma4(void *stream, uint32_t layer, const uint16_t *hidden, uint32_t hiddenStrideElements, int rows,
                                uint32_t *outIndices, uint16_t *outWeights) {
        if (rows < 1 || rows > maxRouterRows) throw std::invalid_argument("rows outside 1...16");
        char *err = nullptr;
        check(ffmoe_router(c_.raw(), stream, layer, hidden, hiddenStrideElements, (uint32_t)rows, outIndices, outWeights, nullptr, &err), err);
    }
    // encodeRoutedPersistentPhase1U16Load + encodeRoutedPersistentPhase2Reduce, and the GPU-routed form
    // encodeGatherRoutedSlots + encodeRoutedPersistentGPUSlots (MoE.swift:312-496): the slots are the router's
    // `indices` on the device; no host read-back, no address table (every expert is resident).
    void encodeRoutedPersistentGPUSlots(void *stream, uint32_t layer, const uint16_t *x, const uint32_t *indices,
                                        const uint16_t *routingWeights, const uint16_t *residual, uint16_t *y) {
        char *err = nullptr;
        check(ffmoe_verify(c_.raw(), stream, layer, x, c_.shape().d, 1, indices, routingWeights, residual, y, &err), err);
    }
    // encodeRouterRowsGemma4 followed by the routed experts of the same rows, as the decode and verify loops
    // issue them back to back (RealForwardRunner.swift:1846-1923): one call, the routes also left on the device
    void encodeRouterAndRoutedExperts(void *stream, uint32_t layer, const uint16_t *routerHidden, uint32_t routerStrideElements,
                                      const uint16_t *x, uint32_t xStrideElements, int rows, const uint16_t *residual, uint16_t *y,
                                      uint32_t *outIndices, uint16_t *outWeights) {
        if (rows < 1 || rows > maxRouterRows) throw std::invalid_argument("rows outside 1...16");
        char *err = nullptr;
        check(ffmoe_route_verify(c_.raw(), stream, layer, routerHidden, routerStrideElements, x, xStrideElements, (uint32_t)rows,
                                 residual, y, outIndices, outWeights, &err), err);
    }
    // The same pair with the shared expert of the block (SharedExpertInt4.encode on `sharedX`, which the runner issues
    // beside the routed experts: RealForwardRunner.swift:454-756) inside its two launches. Nothing is combined: the rows
    // stay on the device for FusedLayerTail::encodeRoutedShared, which needs `outWeights`.
    void encodeRouterRoutedAndSharedExperts(void *stream, Context &shared, uint32_t layer, uint32_t sharedLayer,
                                            const uint16_t *routerHidden, uint32_t routerStrideElements, const uint16_t *x,
                                            uint32_t xStrideElements, const uint16_t *sharedX, uint32_t sharedStrideElements,
                                            int rows, uint32_t *outIndices, uint16_t *outWeights) {
        if (rows < 1 || rows > maxRouterRows) throw std::invalid_argument("rows outside 1...16");
        char *err = nullptr;
        check(ffmoe_route_verify_shared(c_.raw(), shared.raw(), stream, layer, sharedLayer, routerHidden, routerStrideElements, x,
                                        xStrideElements, sharedX, sharedStrideElements, (uint32_t)rows, outIndices, outWeights, &err),
              err);
    }
    // Waves of the one-launch form that stopped waiting for another block and computed its part themselves (the results
    // are the same; a count above zero says the GPU is shared and the routing should run as launches of its own).
    uint32_t handoverGiveups(void *stream) {
        uint32_t n = 0;
        char *err = nullptr;
        check(ffmoe_handover_giveups(c_.raw(), stream, &n, &err), err);
        return n;
    }

private:
    Context &c_;
};

class PrefillGroupedRoutedMoE {
public:
    static constexpr int verifyMaxRows = 16;
    explicit PrefillGroupedRoutedMoE(Context &c) : c_(c) {}
    // encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:275-326): `sortedPairs` on the device, un-weighted rows out
    void encodeStreamedBatched(void *stream, uint32_t layer, const uint16_t *hidden, uint32_t hiddenStrideElements,
                               const PrefillTokenExpertPair *sortedPairs, uint32_t pairCount, uint32_t queryCount,
                               uint16_t *routePartials) {
        char *err = nullptr;
        check(ffmoe_prefill_pairs(c_.raw(), stream, layer, hidden, hiddenStrideElements,
                                  reinterpret_cast<const ffmoe_pair *>(sortedPairs), pairCount, queryCount, routePartials, &err), err);
    }
    // encodeVerifyBound / encodeVerifyRows (PrefillGroupedRoutedMoE.swift:331-448): rows <= 16, routes on the device
    void encodeVerifyBound(void *stream, uint32_t layer, const uint16_t *hidden, uint32_t hiddenStrideElements, int rows,
                           const uint32_t *routeIDs, const uint16_t *routeWeights, uint16_t *routePartials) {
        if (rows <= 0 || rows > verifyMaxRows) throw std::invalid_argument("rows outside 1...16");
        char *err = nullptr;
        check(ffmoe_verify_partials(c_.raw(), stream, layer, hidden, hiddenStrideElements, (uint32_t)rows, routeIDs, routeWeights,
                                    routePartials, &err), err);
    }
    // the whole prefill stage on the GPU: sort + experts + reduce, no host wait between router and experts
    void encodeGPURouted(void *stream, uint32_t layer, const uint16_t *hidden, uint32_t hiddenStrideElements, uint32_t queryCount,
                         const uint32_t *routeIDs, const uint16_t *routeWeights, uint16_t *h2) {
        char *err = nullptr;
        check(ffmoe_prefill(c_.raw(), stream, layer, hidden, hiddenStrideElements, queryCount, routeIDs, routeWeights, h2, &err), err);
    }

private:
    Context &c_;
};

class PrefillMoE {
public:
    explicit PrefillMoE(Context &c) : c_(c) {}
    // PrefillMoE.swift:11-32
    void encodeReduceTokenMajor(void *stream, const uint16_t *routePartials, const uint16_t *routeWeights, uint16_t *h2,
                                uint32_t queryCount, uint32_t topK, uint32_t d) {
        if (queryCount == 0) throw std::invalid_argument("queryCount must be positive");
        if (topK == 0) throw std::invalid_argument("topK must be positive");
        if (d == 0) throw std::invalid_argument("D must be positive");
        char *err = nullptr;
        check(ffmoe_reduce_token_major(c_.raw(), stream, routePartials, routeWeights, h2, queryCount, topK, d, &err), err);
    }

private:
    Context &c_;
};

class DequantInt4GEMV {
public:
    static constexpr int maxBatchRows = 16;
    enum class RowsTypes { bf16, bf16ToF32 };
    explicit DequantInt4GEMV(Context &c) : c_(c) {}
    // DequantInt4GEMV.encode (DequantInt4GEMV.swift:184-224)
    void encode(void *stream, const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const uint16_t *x, uint16_t *y,
                uint32_t m, uint32_t n) {
        encodeRows(stream, weights, scales, biases, x, y, m, n, 1, n, m, RowsTypes::bf16);
    }
    // DequantInt4GEMV.encodeRows (DequantInt4GEMV.swift:72-123)
    void encodeRows(void *stream, const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const uint16_t *x, void *y,
                    uint32_t m, uint32_t n, int rows, uint32_t xStrideElements, uint32_t yStrideElements, RowsTypes types) {
        if (rows <= 0 || rows > maxBatchRows) throw std::invalid_argument("rows outside 1...16");
        if (n % FFMOE_GROUP) throw std::invalid_argument("N must be a multiple of 64");
        char *err = nullptr;
        check(ffmoe_gemv_int4(c_.raw(), stream, weights, scales, biases, x, y, m, n, (uint32_t)rows, xStrideElements, yStrideElements,
                              types == RowsTypes::bf16ToF32 ? 1 : 0, &err), err);
    }
    // DequantInt4GEMV.encodeRowsListed (DequantInt4GEMV.swift:124-145): output o is weight row ids[o]; fp32 out
    void encodeRowsListed(void *stream, const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, const uint32_t *ids,
                          const uint16_t *x, float *y, uint32_t m, uint32_t n, int rows, uint32_t xStrideElements,
                          uint32_t yStrideElements) {
        if (rows <= 0 || rows > maxBatchRows) throw std::invalid_argument("rows outside 1...16");
        if (n % FFMOE_GROUP) throw std::invalid_argument("N must be a multiple of 64");
        char *err = nullptr;
        check(ffmoe_gemv_int4_listed(c_.raw(), stream, weights, scales, biases, ids, x, y, m, n, (uint32_t)rows, xStrideElements,
                                     yStrideElements, &err), err);
    }

private:
    Context &c_;
};

// LMHeadChainInt4 (Kernels/Fusions/LMHeadChainInt4.swift:57-139,225-284): owns the head's INT4 table for its
// lifetime - here the re-tiled resident copy - plus the scratch of the greedy choice, and returns greedy tokens for
// 1...maxGreedyRows normalised hidden rows with one pass over the table. The RMSNorm the Swift chain runs
// first is a separate operator there too (rms.encodeBF16W) and stays with the caller.
class LMHeadChainInt4 {
public:
    static constexpr int maxGreedyRows = 16;
    // weights uint8 [vocab][d/2], scales/biases bf16 [vocab][d/64], in host or device memory
    LMHeadChainInt4(Context &c, const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, uint32_t d, uint32_t vocab)
        : d_(d), vocab_(vocab) {
        if (d % 64) throw std::invalid_argument("d must be a multiple of 64");
        char *err = nullptr;
        check(ffmoe_matrix_create(c.raw(), weights, scales, biases, vocab, d, 1, &mx_, &err), err);
    }
    ~LMHeadChainInt4() { ffmoe_matrix_destroy(mx_); }
    LMHeadChainInt4(const LMHeadChainInt4 &) = delete;
    LMHeadChainInt4 &operator=(const LMHeadChainInt4 &) = delete;
    // encodeGreedyDecode (LMHeadChainInt4.swift:225-284): one row
    void encodeGreedyDecode(void *stream, const uint16_t *normedHidden, uint32_t *outToken) {
        encodeGreedyRows(stream, normedHidden, d_, 1, outToken);
    }
    // encodeGreedyRows (LMHeadChainInt4.swift:94-139)
    void encodeGreedyRows(void *stream, const uint16_t *normedHidden, uint32_t hiddenStrideElements, int rowCount,
                          uint32_t *outTokens) {
        if (rowCount <= 0 || rowCount > maxGreedyRows) throw std::invalid_argument("rowCount outside 1...16");
        char *err = nullptr;
        check(ffmoe_matrix_greedy(mx_, stream, normedHidden, hiddenStrideElements, (uint32_t)rowCount, outTokens, &err), err);
    }
    // fp32 logits of the same rows (rowsProjection.encodeRows with .f16ToF32, LMHeadChainInt4.swift:122-131)
    void encodeLogitsRows(void *stream, const uint16_t *normedHidden, uint32_t hiddenStrideElements, int rowCount, float *logits,
                          uint32_t logitsStrideElements) {
        if (rowCount <= 0 || rowCount > maxGreedyRows) throw std::invalid_argument("rowCount outside 1...16");
        char *err = nullptr;
        check(ffmoe_matrix_gemv(mx_, stream, normedHidden, hiddenStrideElements, (uint32_t)rowCount, logits, logitsStrideElements, 1,
                                &err), err);
    }
    // encodeGreedyRows with the chain's softcap and rowsConfidence (LMHeadChainInt4.swift:94-139 with `softcap`, the
    // probability of the chosen token that argmax_rows_f32 leaves for the drafter: logit.metal:946-1010)
    void encodeGreedyRowsWithConfidence(void *stream, const uint16_t *normedHidden, uint32_t hiddenStrideElements, int rowCount,
                                        float softcap, uint32_t *outTokens, float *rowsConfidence) {
        if (rowCount <= 0 || rowCount > maxGreedyRows) throw std::invalid_argument("rowCount outside 1...16");
        char *err = nullptr;
        check(ffmoe_matrix_greedy_conf(mx_, stream, normedHidden, hiddenStrideElements, (uint32_t)rowCount, softcap, outTokens,
                                       rowsConfidence, &err), err);
    }
    // encodeHotGreedyRows (LMHeadChainInt4.swift:143-178): the greedy choice among the `count` listed rows of the head
    // in the reference layout (weights / scales / biases / ids in DEVICE memory, as DequantInt4GEMV.encodeRowsListed takes them). outIndices
    // are positions in `ids`, as the reference's argmax leaves them; rowsLogits is the chain's [rowCount][count] scratch.
    static void encodeHotGreedyRows(Context &c, void *stream, const uint16_t *normedHidden, uint32_t hiddenStrideElements,
                                    int rowCount, const uint32_t *ids, uint32_t count, const uint8_t *weights,
                                    const uint16_t *scales, const uint16_t *biases, uint32_t d, float softcap, float *rowsLogits,
                                    uint32_t *outIndices, float *rowsConfidence) {
        if (rowCount <= 0 || rowCount > maxGreedyRows || count == 0) throw std::invalid_argument("rowCount outside 1...16 or an empty table");
        char *err = nullptr;
        check(ffmoe_gemv_int4_listed(c.raw(), stream, weights, scales, biases, ids, normedHidden, rowsLogits, count, d,
                                     (uint32_t)rowCount, hiddenStrideElements, count, &err), err);
        check(ffmoe_argmax_rows(c.raw(), stream, rowsLogits, count, (uint32_t)rowCount, count, softcap, outIndices, rowsConfidence,
                                &err), err);
    }
    // TokenSampling + RowSampling (LMHeadChainInt4.swift:183-190): how a row picks its token when it is not the argmax
    struct RowSampling {
        float temperature = 1.0f, topP = 1.0f;
        uint32_t topK = 0;            // 0: no truncation
        uint64_t seed = 0;
        uint32_t keyBase = 0;         // position of row 0's token
        const uint32_t *keyOffset = nullptr;   // device: one uint32 added to keyBase, or null
    };
    // encodeChoice with a sampling rule (LMHeadChainInt4.swift:192-216): the draw over `count` fp32 logits per row that
    // are in device memory (encodeLogitsRows' output, or the listed projection's with `ids`); outIndices are positions
    static void encodeSampledChoice(Context &c, void *stream, const float *rowsLogits, uint32_t logitsStrideElements, int rowCount,
                                    uint32_t count, const uint32_t *ids, float softcap, const RowSampling &sampling,
                                    uint32_t *outIndices, float *rowsConfidence) {
        if (rowCount <= 0 || rowCount > maxGreedyRows) throw std::invalid_argument("rowCount outside 1...16");
        const ffmoe_sampling rule{sampling.temperature, sampling.topP, sampling.topK, sampling.keyBase, softcap, sampling.seed};
        char *err = nullptr;
        check(ffmoe_sample_rows(c.raw(), stream, rowsLogits, logitsStrideElements, (uint32_t)rowCount, count, ids, &rule,
                                sampling.keyOffset, outIndices, rowsConfidence, &err), err);
    }
    // EmbedLookupInt4.encode (Kernels/Quant/EmbedLookupInt4.swift:14-44) on the chain's table - the model ties its
    // embedding to the head, so the resident copy serves both: out[d] = round16((q s + b) * outScale) of row tokenId.
    void encodeEmbedLookup(void *stream, uint32_t tokenId, float outScale, uint16_t *out) {
        char *err = nullptr;
        check(ffmoe_matrix_rows(mx_, stream, nullptr, 1, tokenId, outScale, out, d_, &err), err);
    }
    // the same for `count` token ids in device memory (the tokens a greedy call left): rows of outStrideElements values
    void encodeEmbedLookupRows(void *stream, const uint32_t *tokenIds, int count, float outScale, uint16_t *out,
                               uint32_t outStrideElements) {
        if (count <= 0) throw std::invalid_argument("count must be positive");
        char *err = nullptr;
        check(ffmoe_matrix_rows(mx_, stream, tokenIds, (uint32_t)count, 0, outScale, out, outStrideElements, &err), err);
    }
    uint32_t vocab() const { return vocab_; }

private:
    ffmoe_matrix *mx_ = nullptr;
    uint32_t d_, vocab_;
};

// PrefillFinalRowHeadInt4 (Kernels/Prefill/Epilogues/PrefillFinalRowHead.swift:4-66): the head's logits for ONE row of
// a prefill block - the last prompt token's -, the final norm applied to that row where it lies. The Swift class binds
// the head's table on every call and owns the normed row's buffer; here the table is the resident copy a
// LMHeadChainInt4-style constructor makes, and the caller passes the normed row's scratch (d values, 16-byte aligned).
class PrefillFinalRowHeadInt4 {
public:
    PrefillFinalRowHeadInt4(Context &c, int maxD, const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, uint32_t d,
                            uint32_t vocab)
        : c_(c), d_(d), vocab_(vocab) {
        if (maxD <= 0) throw std::invalid_argument("maxD must be positive");
        if ((int)d > maxD) throw std::invalid_argument("d=" + std::to_string(d) + " exceeds maxD=" + std::to_string(maxD));
        if (d % FFMOE_GROUP) throw std::invalid_argument("d must be a multiple of 64");
        char *err = nullptr;
        check(ffmoe_matrix_create(c.raw(), weights, scales, biases, vocab, d, 0, &mx_, &err), err);
    }
    ~PrefillFinalRowHeadInt4() { ffmoe_matrix_destroy(mx_); }
    PrefillFinalRowHeadInt4(const PrefillFinalRowHeadInt4 &) = delete;
    PrefillFinalRowHeadInt4 &operator=(const PrefillFinalRowHeadInt4 &) = delete;
    // encodeLogits (PrefillFinalRowHead.swift:19-65): logits [vocab] in the activation type
    void encodeLogits(void *stream, const uint16_t *hiddenBlock, int row, int rowStrideElements, const uint16_t *normWeight,
                      uint16_t *normed, uint16_t *logits, float rmsEps) {
        if (row < 0) throw std::invalid_argument("row must be non-negative");
        if (rowStrideElements < (int)d_) throw std::invalid_argument("row stride must cover d");
        char *err = nullptr;
        check(ffmoe_rmsnorm(c_.raw(), stream, hiddenBlock + (size_t)row * rowStrideElements, (uint32_t)rowStrideElements, normWeight,
                            normed, d_, 1, d_, rmsEps, &err), err);
        check(ffmoe_matrix_gemv(mx_, stream, normed, d_, 1, logits, vocab_, 0, &err), err);
    }

private:
    Context &c_;
    ffmoe_matrix *mx_ = nullptr;
    uint32_t d_, vocab_;
};

// ---------------------------------------------------------------------------------------------------
// Shared expert (Kernels/MoE/SharedExpertInt4.swift, Kernels/Prefill/MoE/PrefillSharedExpert.swift): the dense
// INT4 FFN every token passes through. The Swift operators bind the three projections on every call; here
// they are uploaded once per layer into a context of one expert (n_experts = top_k = 1, f = the shared
// width) and the calls name the layer.
// ---------------------------------------------------------------------------------------------------
struct SharedExpertProjection {   // weights uint8 [rows][cols/2], scales/biases bf16 [rows][cols/64]
    const uint8_t *weights;
    const uint16_t *scales, *biases;
    uint32_t rows, cols;
};

struct SharedExpertError : std::runtime_error {
    enum Kind { unsupportedWeightBits, dimensionMismatch, scratchTooSmall } kind;
    SharedExpertError(Kind k, const std::string &m) : std::runtime_error(m), kind(k) {}
};

class SharedExpertInt4 {
public:
    explicit SharedExpertInt4(Context &dense) : c_(dense) {
        if (dense.shape().n_experts != 1 || dense.shape().top_k != 1)
            throw std::invalid_argument("the shared expert needs a context with n_experts = 1 and top_k = 1");
    }
    // the guard of SharedExpertInt4.encode (SharedExpertInt4.swift:41-46), then the upload
    void load(uint32_t layer, const SharedExpertProjection &gate, const SharedExpertProjection &up,
              const SharedExpertProjection &down, bool onDevice = false) {
        const ffmoe_shape &sh = c_.shape();
        if (gate.rows != up.rows || gate.cols != up.cols || down.rows != gate.cols || down.cols != gate.rows ||
            gate.rows != sh.f || gate.cols != sh.d)
            throw SharedExpertError(SharedExpertError::dimensionMismatch,
                                    "SharedExpert dimension mismatch: gate=(" + std::to_string(gate.rows) + "," +
                                        std::to_string(gate.cols) + ") up=(" + std::to_string(up.rows) + "," +
                                        std::to_string(up.cols) + ") down=(" + std::to_string(down.rows) + "," +
                                        std::to_string(down.cols) + ")");
        const ffmoe_projection g{gate.weights, gate.scales, gate.biases}, u{up.weights, up.scales, up.biases},
            dn{down.weights, down.scales, down.biases};
        char *err = nullptr;
        check(ffmoe_upload_expert_parts(c_.raw(), layer, 0, &g, &u, &dn, onDevice ? 1 : 0, &err), err);
    }
    // encode (SharedExpertInt4.swift:32-89): one row; the activation scratch is the context's
    void encode(void *stream, uint32_t layer, const uint16_t *x, uint16_t *y) {
        char *err = nullptr;
        check(ffmoe_dense_ffn(c_.raw(), stream, layer, x, c_.shape().d, 1, y, &err), err);
    }

protected:
    Context &c_;
};

// DequantInt8GEMV (Kernels/Quant/DequantInt8GEMV.swift:7-56): y = W x with W 8-bit affine (uint8 [m][n], scales / biases
// bf16 [m][n/64]). The Swift operator binds the weight on every call; here the weight is re-tiled once and owned, and a
// call takes 1...16 rows of x with one pass over it.
class DequantInt8GEMV {
public:
    static constexpr int maxBatchRows = 16;
    DequantInt8GEMV(Context &c, const uint8_t *weights, const uint16_t *scales, const uint16_t *biases, uint32_t m, uint32_t n)
        : m_(m), n_(n) {
        if (n % FFMOE_GROUP) throw std::invalid_argument("N must be a multiple of 64");
        char *err = nullptr;
        check(ffmoe_matrix_create_int8(c.raw(), weights, scales, biases, m, n, &mx_, &err), err);
    }
    ~DequantInt8GEMV() { ffmoe_matrix_destroy(mx_); }
    DequantInt8GEMV(const DequantInt8GEMV &) = delete;
    DequantInt8GEMV &operator=(const DequantInt8GEMV &) = delete;
    // encode (DequantInt8GEMV.swift:25-56): one row
    void encode(void *stream, const uint16_t *x, uint16_t *y) { encodeRows(stream, x, y, 1, n_, m_); }
    void encodeRows(void *stream, const uint16_t *x, uint16_t *y, int rows, uint32_t xStrideElements, uint32_t yStrideElements) {
        if (rows <= 0 || rows > maxBatchRows) throw std::invalid_argument("rows outside 1...16");
        char *err = nullptr;
        check(ffmoe_matrix_gemv(mx_, stream, x, xStrideElements, (uint32_t)rows, y, yStrideElements, 0, &err), err);
    }
    uint32_t m() const { return m_; }
    uint32_t n() const { return n_; }

private:
    ffmoe_matrix *mx_ = nullptr;
    uint32_t m_, n_;
};

// SharedExpertInt8 (Kernels/MoE/SharedExpertInt8.swift:40-135): y = down(gelu_tanh(gate(x)) * up(x)) with the three
// projections 8-bit affine, the form in which the packs hold the shared expert by default. Same shape as
// SharedExpertInt4 above: a dense context of one expert, load() once per layer (the layer is kept as a gated gate/up
// matrix and a down matrix of nibble planes), calls name the layer, and the activation scratch the Swift caller
// passes is the context's.
class SharedExpertInt8 {
public:
    explicit SharedExpertInt8(Context &dense) : c_(dense) {
        if (dense.shape().n_experts != 1 || dense.shape().top_k != 1)
            throw std::invalid_argument("the shared expert needs a context with n_experts = 1 and top_k = 1");
    }
    // the guards of SharedExpertInt8.encode (SharedExpertInt8.swift:63-70), then the upload; host or device pointers
    void load(uint32_t layer, const SharedExpertProjection &gate, const SharedExpertProjection &up,
              const SharedExpertProjection &down) {
        if (gate.rows != up.rows || gate.cols != up.cols)
            throw SharedExpertError(SharedExpertError::dimensionMismatch,
                                    "gate/up shapes differ: gate=(" + std::to_string(gate.rows) + "," + std::to_string(gate.cols) +
                                        ") up=(" + std::to_string(up.rows) + "," + std::to_string(up.cols) + ")");
        if (down.rows != gate.cols || down.cols != gate.rows)
            throw SharedExpertError(SharedExpertError::dimensionMismatch,
                                    "down expected (" + std::to_string(gate.cols) + "," + std::to_string(gate.rows) + "), got (" +
                                        std::to_string(down.rows) + "," + std::to_string(down.cols) + ")");
        if (gate.rows != c_.shape().f || gate.cols != c_.shape().d)
            throw SharedExpertError(SharedExpertError::dimensionMismatch,
                                    "SharedExpert dimension mismatch: expected gate/up=(" + std::to_string(c_.shape().f) + "," +
                                        std::to_string(c_.shape().d) + ")");
        const ffmoe_projection g{gate.weights, gate.scales, gate.biases}, u{up.weights, up.scales, up.biases},
            dn{down.weights, down.scales, down.biases};
        char *err = nullptr;
        check(ffmoe_upload_expert_parts_int8(c_.raw(), layer, &g, &u, &dn, &err), err);
    }
    // encode (SharedExpertInt8.swift:56-97): one row
    void encode(void *stream, uint32_t layer, const uint16_t *x, uint16_t *y) {
        char *err = nullptr;
        check(ffmoe_dense_ffn(c_.raw(), stream, layer, x, c_.shape().d, 1, y, &err), err);
    }

protected:
    Context &c_;
};

// SharedExpertRuntime (SharedExpertInt4.swift:92-130): picks the implementation by weight width. `dense` is the
// one-expert context both take.
class SharedExpertRuntime {
public:
    SharedExpertRuntime(Context &dense, int weightBits) : c_(dense) {
        if (weightBits == 4) int4_.reset(new SharedExpertInt4(dense));
        else if (weightBits == 8) int8_.reset(new SharedExpertInt8(dense));
        else
            throw SharedExpertError(SharedExpertError::unsupportedWeightBits,
                                    "SharedExpert unsupported weight bits: " + std::to_string(weightBits));
    }
    int weightBits() const { return int4_ ? 4 : 8; }
    void load(uint32_t layer, const SharedExpertProjection &gate, const SharedExpertProjection &up,
              const SharedExpertProjection &down) {
        if (int4_) int4_->load(layer, gate, up, down);
        else int8_->load(layer, gate, up, down);
    }
    void encode(void *stream, uint32_t layer, const uint16_t *x, uint16_t *y) {
        if (int4_) int4_->encode(stream, layer, x, y);
        else int8_->encode(stream, layer, x, y);
    }

protected:
    Context &c_;

private:
    std::unique_ptr<SharedExpertInt4> int4_;
    std::unique_ptr<SharedExpertInt8> int8_;
};

// PrefillSharedExpert (PrefillSharedExpert.swift:19-33,94-137): a block of rows in either weight width (the Swift
// class defaults to 8 bits). The Swift class loops its single-row operator below 32 tokens and batches the 4-bit
// form above; here rows <= 16 stream the weights once for all rows, a few hundred rows stream them once per 16 rows, and
// more rows run the grouped GEMMs (4 bits, from 385 rows) or the library's dense GEMMs (8 bits, from 192 rows).
class PrefillSharedExpert : public SharedExpertRuntime {
public:
    static constexpr int batchedMinimumTokens = 17;
    explicit PrefillSharedExpert(Context &dense, int weightBits = 4) : SharedExpertRuntime(dense, weightBits) {}
    void encodeBlock(void *stream, uint32_t layer, const uint16_t *x, uint16_t *y, int queryCount, int d, int intermediate,
                     int xStrideElements, int yStrideElements) {
        if (queryCount < 0) throw std::invalid_argument("queryCount must be non-negative");
        if (d <= 0) throw std::invalid_argument("d must be positive");
        if (intermediate <= 0) throw std::invalid_argument("intermediate must be positive");
        if (xStrideElements < d) throw std::invalid_argument("x stride is too small");
        if (yStrideElements < d) throw std::invalid_argument("y stride is too small");
        if ((uint32_t)d != c_.shape().d || (uint32_t)intermediate != c_.shape().f)
            throw SharedExpertError(SharedExpertError::dimensionMismatch,
                                    "SharedExpert dimension mismatch: expected gate/up=(" + std::to_string(c_.shape().f) + "," +
                                        std::to_string(c_.shape().d) + ")");
        if (yStrideElements != d) throw std::invalid_argument("y rows must be contiguous");
        if (queryCount == 0) return;
        char *err = nullptr;
        check(ffmoe_dense_ffn(c_.raw(), stream, layer, x, (uint32_t)xStrideElements, (uint32_t)queryCount, y, &err), err);
    }
};

// ---------------------------------------------------------------------------------------------------
// The steps either side of the MoE stage. PrefillPostAttentionSetup / PrefillLayerTail
// (Kernels/Prefill/Epilogues/) take blocks of rows; FusedPostAttentionSetup / FusedLayerTail
// (Kernels/Fusions/) are their one-row decode forms. Same preconditions as the Swift classes.
// ---------------------------------------------------------------------------------------------------
class PrefillPostAttentionSetup {
public:
    explicit PrefillPostAttentionSetup(Context &c) : c_(c) {}
    void encode(void *stream, uint16_t *hidden, const uint16_t *attn, uint16_t *denseX, uint16_t *routedX, uint16_t *routerX,
                const uint16_t *postAttnWeight, const uint16_t *preFFNWeight, const uint16_t *preFFN2Weight, uint32_t queryCount,
                uint32_t d, uint32_t hiddenStrideElements, uint32_t attnStrideElements, uint32_t denseStrideElements,
                uint32_t routedStrideElements, uint32_t routerStrideElements, float eps) {
        if (queryCount == 0) throw std::invalid_argument("queryCount must be positive");
        if (d == 0 || d > FFMOE_ROW_MAX_D) throw std::invalid_argument("D must be in 1...4096");
        char *err = nullptr;
        check(ffmoe_post_attn_setup(c_.raw(), stream, hidden, hiddenStrideElements, attn, attnStrideElements, denseX,
                                    denseStrideElements, routedX, routedStrideElements, routerX, routerStrideElements, postAttnWeight,
                                    preFFNWeight, preFFN2Weight, queryCount, d, eps, &err), err);
    }

protected:
    Context &c_;
};

class FusedPostAttentionSetup : public PrefillPostAttentionSetup {
public:
    using PrefillPostAttentionSetup::PrefillPostAttentionSetup;
    void encode(void *stream, uint16_t *hidden, const uint16_t *attn, uint16_t *denseX, uint16_t *routedX, uint16_t *routerX,
                const uint16_t *postAttnWeight, const uint16_t *preFFNWeight, const uint16_t *preFFN2Weight, uint32_t d, float eps) {
        PrefillPostAttentionSetup::encode(stream, hidden, attn, denseX, routedX, routerX, postAttnWeight, preFFNWeight, preFFN2Weight,
                                          1, d, d, d, d, d, d, eps);
    }
};

class PrefillLayerTail {
public:
    explicit PrefillLayerTail(Context &c) : c_(c) {}
    // encode (PrefillLayerTail.swift:11-51)
    void encode(void *stream, const uint16_t *h2, const uint16_t *h1, uint16_t *hidden, const uint16_t *postFFN2Weight,
                const uint16_t *postFFNWeight, uint32_t queryCount, uint32_t d, uint32_t h2StrideElements, uint32_t h1StrideElements,
                uint32_t hiddenStrideElements, float eps, float layerScalar) {
        if (queryCount == 0) throw std::invalid_argument("queryCount must be positive");
        if (d == 0 || d > FFMOE_ROW_MAX_D) throw std::invalid_argument("D must be in 1...4096");
        if (h2StrideElements < d) throw std::invalid_argument("h2 stride is too small");
        if (h1StrideElements < d) throw std::invalid_argument("h1 stride is too small");
        if (hiddenStrideElements < d) throw std::invalid_argument("hidden stride is too small");
        char *err = nullptr;
        check(ffmoe_layer_tail(c_.raw(), stream, h2, h2StrideElements, h1, h1StrideElements, hidden, hiddenStrideElements, postFFN2Weight,
                               postFFNWeight, queryCount, d, eps, layerScalar, &err), err);
    }

protected:
    Context &c_;
};

class FusedLayerTail : public PrefillLayerTail {
public:
    using PrefillLayerTail::PrefillLayerTail;
    static constexpr bool fusesNorms = true;
    void encode(void *stream, const uint16_t *h2, const uint16_t *h1, uint16_t *hidden, const uint16_t *postFFN2Weight,
                const uint16_t *postFFNWeight, uint32_t d, float eps, float layerScalar) {
        PrefillLayerTail::encode(stream, h2, h1, hidden, postFFN2Weight, postFFNWeight, 1, d, d, d, d, eps, layerScalar);
    }
    // The tail on the rows MoE::encodeRouterAndRoutedExperts left un-combined (y = nullptr there): the routed experts'
    // weighted combine (prefill.metal:544-565) happens while this launch loads its inputs
    void encodeRouted(void *stream, const uint16_t *routeWeights, const uint16_t *h1, uint16_t *hidden, const uint16_t *postFFN2Weight,
                      const uint16_t *postFFNWeight, int rows, float eps, float layerScalar) {
        char *err = nullptr;
        const uint32_t d = c_.shape().d;
        check(ffmoe_layer_tail_routed(c_.raw(), stream, routeWeights, h1, d, hidden, d, postFFN2Weight, postFFNWeight, (uint32_t)rows,
                                      eps, layerScalar, &err), err);
    }
    // ... and on the rows MoE::encodeRouterRoutedAndSharedExperts left in the two contexts (h1 = the shared expert's row)
    void encodeRoutedShared(void *stream, Context &shared, const uint16_t *routeWeights, uint16_t *hidden,
                            const uint16_t *postFFN2Weight, const uint16_t *postFFNWeight, int rows, float eps, float layerScalar) {
        char *err = nullptr;
        check(ffmoe_layer_tail_routed_shared(c_.raw(), shared.raw(), stream, routeWeights, hidden, c_.shape().d, postFFN2Weight,
                                             postFFNWeight, (uint32_t)rows, eps, layerScalar, &err), err);
    }
    // encodeWithNorms (FusedLayerTail.swift:74-117): h1 before its post-FFN-1 norm; nextInputNorm / nextNormed
    // may both be null (no next layer)
    void encodeWithNorms(void *stream, const uint16_t *h2, const uint16_t *h1, uint16_t *hidden, const uint16_t *postFFN1Weight,
                         const uint16_t *postFFN2Weight, const uint16_t *postFFNWeight, const uint16_t *nextInputNorm,
                         uint16_t *nextNormed, uint32_t d, float eps, float layerScalar) {
        if (d == 0 || d > FFMOE_ROW_MAX_D) throw std::invalid_argument("D > 4096 exceeds the fused-tail row limit");
        if ((nextInputNorm == nullptr) != (nextNormed == nullptr))
            throw std::invalid_argument("nextInputNorm and nextNormed go together");
        char *err = nullptr;
        check(ffmoe_layer_tail_norms(c_.raw(), stream, h2, d, h1, d, hidden, d, postFFN1Weight, postFFN2Weight, postFFNWeight,
                                     nextInputNorm, nextNormed, d, 1, d, eps, layerScalar, &err), err);
    }
};

// RMSNorm.encodeBF16W: rows of x normalised under a bf16 weight; `out` may be `x`
class RMSNorm {
public:
    explicit RMSNorm(Context &c) : c_(c) {}
    void encodeBF16W(void *stream, const uint16_t *x, const uint16_t *weight, uint16_t *out, uint32_t d, float eps, uint32_t rows = 1,
                     uint32_t xStrideElements = 0, uint32_t outStrideElements = 0) {
        char *err = nullptr;
        check(ffmoe_rmsnorm(c_.raw(), stream, x, xStrideElements ? xStrideElements : d, weight, out,
                            outStrideElements ? outStrideElements : d, rows, d, eps, &err), err);
    }

private:
    Context &c_;
};

// ---------------------------------------------------------------------------------------------------
// Guest plugin and supervisor (Runtime/Supervisor/DeviceSupervisor.swift:5-125).
// ---------------------------------------------------------------------------------------------------
enum class RuntimeFaultPolicy { failClosed, failoverHost };   // reference: .failClosed / .failoverMetal

struct CancellationError : std::runtime_error {
    CancellationError() : std::runtime_error("cancelled") {}
};

// Routed top-k prefill for one layer on a rail other than the host's. On return every routed (token, rank)
// row named by `pairs` has been written to `partials`; on throw the guest has drained its own work, so the
// host may overwrite `partials` at once.
struct RoutedPrefillGuest {
    virtual ~RoutedPrefillGuest() = default;
    virtual void runLayer(int layer, const uint16_t *hidden, uint16_t *partials, const PrefillMoEGroupedRoutes &routes,
                          const PrefillTokenExpertPair *pairsOnDevice) = 0;
    virtual std::string profile() const { return "{}"; }
};

// The guest that runs routed prefill on this library's kernels (stands where ANERoutedPrefillBackend stood).
class HipRoutedPrefillGuest : public RoutedPrefillGuest {
public:
    HipRoutedPrefillGuest(Context &c, void *stream, uint32_t queryCount, uint32_t hiddenStrideElements,
                          std::function<void(void *)> synchronize)
        : moe_(c), stream_(stream), queryCount_(queryCount), stride_(hiddenStrideElements), sync_(std::move(synchronize)) {}
    void runLayer(int layer, const uint16_t *hidden, uint16_t *partials, const PrefillMoEGroupedRoutes &routes,
                  const PrefillTokenExpertPair *pairsOnDevice) override {
        moe_.encodeStreamedBatched(stream_, (uint32_t)layer, hidden, stride_, pairsOnDevice, (uint32_t)routes.sortedPairs.size(),
                                   queryCount_, partials);
        if (sync_) sync_(stream_);   // the contract: rows are written when runLayer returns
        ++layers_;
    }
    std::string profile() const override { return "{\"layers_run\": " + std::to_string(layers_) + "}"; }

private:
    PrefillGroupedRoutedMoE moe_;
    void *stream_;
    uint32_t queryCount_, stride_;
    std::function<void(void *)> sync_;
    int layers_ = 0;
};

struct GuestFault {
    enum class Action { failedClosed, evictedToHost };
    int layer;
    std::string message;
    Action action;
    bool operator==(const GuestFault &o) const { return layer == o.layer && message == o.message && action == o.action; }
};

class DeviceSupervisor {
public:
    DeviceSupervisor(int guestLayers, RuntimeFaultPolicy policy, std::shared_ptr<RoutedPrefillGuest> guest)
        : guestLayers_(guest ? guestLayers : 0), faultPolicy_(policy), guest_(std::move(guest)) {}
    int guestLayers() const { return guestLayers_; }
    RuntimeFaultPolicy faultPolicy() const { return faultPolicy_; }
    bool evicted() const { return evicted_; }
    const std::vector<GuestFault> &faults() const { return faults_; }
    // nullptr when the layer is the host's: never admitted again after an eviction
    RoutedPrefillGuest *routedPrefill(int layer) const { return (!evicted_ && layer < guestLayers_) ? guest_.get() : nullptr; }
    // true: the guest completed. false: evicted, the host must run the layer. failClosed rethrows; cancellation
    // always propagates (DeviceSupervisor.swift:94-109).
    bool supervise(int layer, const std::function<void()> &body) {
        try {
            body();
            return true;
        } catch (const CancellationError &) {
            throw;
        } catch (const std::exception &e) {
            const bool closed = faultPolicy_ == RuntimeFaultPolicy::failClosed;
            faults_.push_back({layer, e.what(), closed ? GuestFault::Action::failedClosed : GuestFault::Action::evictedToHost});
            if (closed) throw;
            evicted_ = true;
            return false;
        }
    }

private:
    int guestLayers_;
    RuntimeFaultPolicy faultPolicy_;
    std::shared_ptr<RoutedPrefillGuest> guest_;
    bool evicted_ = false;
    std::vector<GuestFault> faults_;
};

}  // namespace fieldfare
