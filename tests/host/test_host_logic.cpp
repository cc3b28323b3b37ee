// Host-logic tests of the C++ operator mirror (no GPU): exact expected arrays restated from the reference's
// PrefillMoEGroupingTests.swift, PrefillRouterTests.swift:12-22, PrefillGroupedRoutedMoETests+Binding.swift and
// the fault policy of DeviceSupervisorFailoverTests.swift:19-81, and the packed-experts layout cases of
// GTurboFormatCodecTests.swift:47-66,136-183 and ModelLoaderTests.swift:56-90,204-241; the two route-trimming options of
// RealForwardRunner.swift:818-847,1952-1961 on hand-computed rows (the reference has no test of its own for them).
#include <cstdio>
#include <cstring>

#include "../../ane-fieldfare_amd/host/fieldfare_host.hpp"
#include "../../ane-fieldfare_amd/host/packed_experts.hpp"

using namespace fieldfare;

static int failures = 0;
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) { std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } \
    } while (0)

static PrefillTokenExpertPair pr(uint32_t t, uint32_t e, uint32_t r, uint32_t bits) { return {t, e, r, bits}; }

static void groupingSortsPairsAndBuildsOffsetsCountsAndTiles() {
    std::vector<PrefillTokenExpertPair> pairs = {pr(0, 3, 0, 10), pr(0, 1, 1, 11), pr(0, 4, 2, 12), pr(1, 1, 0, 13), pr(1, 3, 1, 14),
                                                 pr(1, 2, 2, 15), pr(2, 4, 0, 16), pr(2, 3, 1, 17), pr(2, 1, 2, 18), pr(3, 5, 0, 19),
                                                 pr(3, 1, 1, 20), pr(3, 4, 2, 21)};
    std::reverse(pairs.begin(), pairs.end());
    auto g = PrefillMoEGrouping::groupTokenExpertPairs(pairs, 4, 3, 6, 2);
    const uint32_t experts[] = {1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5};
    const uint32_t tr[][2] = {{0, 1}, {1, 0}, {2, 2}, {3, 1}, {1, 2}, {0, 0}, {1, 1}, {2, 1}, {0, 2}, {2, 0}, {3, 2}, {3, 0}};
    const uint32_t bits[] = {11, 13, 18, 20, 15, 10, 14, 17, 12, 16, 21, 19};
    EXPECT(g.sortedPairs.size() == 12);
    for (size_t i = 0; i < 12; ++i) {
        EXPECT(g.sortedPairs[i].expert == experts[i]);
        EXPECT(g.sortedPairs[i].token == tr[i][0] && g.sortedPairs[i].rank == tr[i][1]);
        EXPECT(g.sortedPairs[i].weightBitsAndReserved == bits[i]);
    }
    const std::vector<PrefillMoEGroup> groups = {{1, 0, 4}, {2, 4, 1}, {3, 5, 3}, {4, 8, 3}, {5, 11, 1}};
    EXPECT(g.groups == groups);
    const std::vector<PrefillMoETile> tiles = {{0, 2, 0, 5}, {2, 2, 5, 6}, {4, 1, 11, 1}};
    EXPECT(g.tiles == tiles);
}

static void groupingCanOrderTilesByExpertSortKeys() {
    std::vector<PrefillTokenExpertPair> pairs = {pr(0, 1, 0, 10), pr(0, 2, 1, 20), pr(1, 3, 0, 30), pr(1, 1, 1, 11), pr(2, 2, 0, 21), pr(2, 3, 1, 31)};
    const std::vector<uint64_t> keys = {0, 30, 10, 20};
    auto g = PrefillMoEGrouping::groupTokenExpertPairs(pairs, 3, 2, 4, 2, &keys);
    EXPECT(g.groups.size() == 3 && g.groups[0].expert == 2 && g.groups[1].expert == 3 && g.groups[2].expert == 1);
    const uint32_t experts[] = {2, 2, 3, 3, 1, 1};
    for (size_t i = 0; i < 6; ++i) EXPECT(g.sortedPairs[i].expert == experts[i]);
    const std::vector<PrefillMoETile> tiles = {{0, 2, 0, 4}, {2, 1, 4, 2}};
    EXPECT(g.tiles == tiles);
}

static void groupingRejectsInvalidMetadataBeforeKernelUse() {
    bool threw = false;
    try {
        PrefillMoEGrouping::groupTokenExpertPairs({pr(0, 2, 0, 1)}, 1, 1, 2, 1);
    } catch (const PrefillMoEGroupingError &e) {
        threw = e.expert == 2 && std::strcmp(e.what(), "route expert 2 is out of range") == 0;
    }
    EXPECT(threw);
}

static void tokenExpertPairsAreTokenMajor() {
    const std::vector<uint16_t> w = {0x2E66, 0x3266, 0x34CD, 0x3666, 0x3800, 0x38CD};   // fp16 0.1 .. 0.6
    auto pairs = PrefillRouter::makeTokenExpertPairs({3, 1, 2, 4, 0, 5}, w, 2, 3);
    const uint32_t tok[] = {0, 0, 0, 1, 1, 1}, rank[] = {0, 1, 2, 0, 1, 2}, ex[] = {3, 1, 2, 4, 0, 5};
    for (size_t i = 0; i < 6; ++i)
        EXPECT(pairs[i].token == tok[i] && pairs[i].rank == rank[i] && pairs[i].expert == ex[i] && pairs[i].weightBitsAndReserved == w[i]);
    bool threw = false;
    try { PrefillRouter::makeTokenExpertPairs({1, 2}, w, 2, 3); } catch (const std::invalid_argument &) { threw = true; }
    EXPECT(threw);
}

static void streamedTileBinding() {
    bool dup = false;
    try { PrefillStreamedTileBinding b({3, 3}); } catch (const PrefillGroupedRoutedMoEError &e) {
        dup = e.kind == PrefillGroupedRoutedMoEError::invalidStreamedTileBinding && std::string(e.what()).find("duplicate") != std::string::npos;
    }
    EXPECT(dup);
    bool empty = false, many = false, neg = false;
    try { PrefillStreamedTileBinding b(std::vector<int>{}); } catch (const PrefillGroupedRoutedMoEError &) { empty = true; }
    try { PrefillStreamedTileBinding b(std::vector<int>{0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16}); } catch (const PrefillGroupedRoutedMoEError &) { many = true; }
    try { PrefillStreamedTileBinding b({-1}); } catch (const PrefillGroupedRoutedMoEError &) { neg = true; }
    EXPECT(empty && many && neg);
    // streamedTilePlanningNeverExceedsDefaultSlotCount
    std::vector<PrefillTokenExpertPair> pairs;
    for (uint32_t i = 0; i < 24; ++i) pairs.push_back(pr(i / 8, std::min(i, 19u), i % 8, 0));
    auto routes = PrefillMoEGrouping::groupTokenExpertPairs(pairs, 3, 8, 128, 16);
    auto first = PrefillStreamedTileBinding::expertIDsForTile(0, routes), second = PrefillStreamedTileBinding::expertIDsForTile(1, routes);
    EXPECT(first.size() == 16 && second.size() == 4);
    for (int i = 0; i < 16; ++i) EXPECT(first[i] == i);
    for (int i = 0; i < 4; ++i) EXPECT(second[i] == 16 + i);
}

struct FaultAtLayerGuest : RoutedPrefillGuest {
    int faultLayer, calls = 0;
    bool poison;
    FaultAtLayerGuest(int l, bool p) : faultLayer(l), poison(p) {}
    void runLayer(int layer, const uint16_t *, uint16_t *partials, const PrefillMoEGroupedRoutes &, const PrefillTokenExpertPair *) override {
        ++calls;
        if (layer == faultLayer) {
            if (poison && partials) partials[0] = 0x7FC0;   // a NaN the host has to clear before its own run
            throw std::runtime_error("injected guest fault at layer " + std::to_string(layer));
        }
    }
};

static void supervisorPolicies() {
    PrefillMoEGroupedRoutes routes;
    {   // no guest: every layer is the host's
        DeviceSupervisor s(30, RuntimeFaultPolicy::failoverHost, nullptr);
        EXPECT(s.guestLayers() == 0 && s.routedPrefill(0) == nullptr);
    }
    {   // failover: the faulting layer is re-run by the host, the guest never comes back
        auto guest = std::make_shared<FaultAtLayerGuest>(2, true);
        DeviceSupervisor s(4, RuntimeFaultPolicy::failoverHost, guest);
        uint16_t partials[4] = {0, 0, 0, 0};
        int hostLayers = 0;
        for (int layer = 0; layer < 6; ++layer) {
            bool done = false;
            if (auto *g = s.routedPrefill(layer)) done = s.supervise(layer, [&] { g->runLayer(layer, nullptr, partials, routes, nullptr); });
            if (!done) { std::memset(partials, 0, sizeof partials); ++hostLayers; }
        }
        EXPECT(guest->calls == 3 && hostLayers == 4 && s.evicted());
        EXPECT(s.faults().size() == 1 && s.faults()[0].layer == 2 && s.faults()[0].action == GuestFault::Action::evictedToHost);
        EXPECT(s.faults()[0].message == "injected guest fault at layer 2");
        EXPECT(s.routedPrefill(0) == nullptr && partials[0] == 0);
    }
    {   // fail-closed rethrows and records
        auto guest = std::make_shared<FaultAtLayerGuest>(0, false);
        DeviceSupervisor s(4, RuntimeFaultPolicy::failClosed, guest);
        bool threw = false;
        try { s.supervise(0, [&] { guest->runLayer(0, nullptr, nullptr, routes, nullptr); }); } catch (const std::runtime_error &) { threw = true; }
        EXPECT(threw && !s.evicted() && s.faults().size() == 1 && s.faults()[0].action == GuestFault::Action::failedClosed);
    }
    {   // cancellation always propagates and is not a fault
        DeviceSupervisor s(4, RuntimeFaultPolicy::failoverHost, std::make_shared<FaultAtLayerGuest>(-1, false));
        bool cancelled = false;
        try { s.supervise(1, [] { throw CancellationError(); }); } catch (const CancellationError &) { cancelled = true; }
        EXPECT(cancelled && !s.evicted() && s.faults().empty());
    }
}

// FormatFixture.layout (GTurboFormatCodecTests.swift:47-66) as the JSON its encoder writes: one layer, two
// experts of one 16 KiB stride, one tensor "gate" {offset 0, size 32, U32, [8, 8], bits 4}.
static std::string fixtureLayoutJson(bool explicitIDs, bool explicitRanks, const std::string &file = "layer_00.bin",
                                     const std::string &tensor = "{\"offset\":0,\"size\":32,\"dtype\":\"U32\",\"shape\":[8,8],\"bits\":4}") {
    std::string experts;
    for (int e = 0; e < 2; ++e) {
        experts += e ? "," : "";
        experts += "{";
        if (explicitIDs) experts += "\"expert\":" + std::to_string(e) + ",";
        if (explicitRanks) experts += "\"physicalRank\":" + std::to_string(e) + ",";
        experts += "\"offset\":" + std::to_string(e * 16384) + ",\"size\":16384,\"tensors\":{\"gate\":" + tensor + "}}";
    }
    return "{\"expertStride\":16384,\"numLayers\":1,\"expertsPerLayer\":2,\"layers\":[{\"layer\":0,\"file\":\"" + file +
           "\",\"experts\":[" + experts + "]}]}";
}

static bool rejects(const std::string &json, const char *needle) {
    try {
        PackedExpertsLayoutReader::decode(json);
    } catch (const GTurboFormatError &e) {
        return std::string(e.what()).find(needle) != std::string::npos;
    }
    return false;
}

static void packedExpertsLayoutCodec() {
    // roundTripPreservesIdentityFallback (GTurboFormatCodecTests.swift:137-141): positional ids and ranks
    for (int mode = 0; mode < 4; ++mode) {
        const auto layout = PackedExpertsLayoutReader::decode(fixtureLayoutJson(mode & 1, mode & 2));
        EXPECT(layout.expertStride == 16384 && layout.numLayers == 1 && layout.expertsPerLayer == 2);
        EXPECT(layout.layers.size() == 1 && layout.layers[0].file == "layer_00.bin" && layout.layers[0].experts.size() == 2);
        for (int e = 0; e < 2; ++e) {
            const ExpertEntry &ex = layout.expert(0, e);
            EXPECT(ex.expert == e && ex.physicalRank == e && ex.offset == (uint64_t)e * 16384 && ex.size == 16384);
            const SubTensorEntry &t = ex.subTensors.at("gate");
            EXPECT(t.offset == 0 && t.size == 32 && t.dtype == "U32" && t.shape == std::vector<uint32_t>({8, 8}) && t.bits == 4);
        }
        EXPECT(layout.routedExpertPhysicalOffsets(0) == std::vector<uint64_t>({0, 16384}));
    }
    // rejectsSlashBearingLayerBasename (:143-152)
    EXPECT(rejects(fixtureLayoutJson(true, true, "nested/layer.bin"), "expected basename"));
    EXPECT(rejects(fixtureLayoutJson(true, true, "../layer.bin"), "non-canonical path"));
    EXPECT(rejects(fixtureLayoutJson(true, true, "/layer.bin"), "unsafe relative path"));
    EXPECT(rejects(fixtureLayoutJson(true, true, "Layout.JSON"), "reserved packed-expert filename"));
    // rejectsTensorOutsideExpertBlob (:167-181): offset stride - 8, size 16
    EXPECT(rejects(fixtureLayoutJson(true, true, "layer_00.bin", "{\"offset\":16376,\"size\":16,\"dtype\":\"U32\",\"shape\":[1],\"bits\":4}"),
                   "range exceeds expert blob"));
    // the validator's other guards (GTurboPackedExpertsLayoutV1.swift:73-160)
    EXPECT(rejects(fixtureLayoutJson(true, true, "layer_00.bin", "{\"offset\":0,\"size\":32,\"dtype\":\"F32\",\"shape\":[8,8]}"), "invalid dtype or shape"));
    EXPECT(rejects(fixtureLayoutJson(true, true, "layer_00.bin", "{\"offset\":0,\"size\":32,\"dtype\":\"U32\",\"shape\":[8,0]}"), "invalid dtype or shape"));
    EXPECT(rejects(fixtureLayoutJson(true, true, "layer_00.bin", "{\"offset\":0,\"size\":32,\"dtype\":\"U32\",\"shape\":[8,8],\"bits\":33}"), "invalid dtype or shape"));
    EXPECT(rejects("{\"expertStride\":1000,\"numLayers\":1,\"expertsPerLayer\":2,\"layers\":[]}", "invalid dimensions or stride"));
    EXPECT(rejects("{\"expertStride\":16384,\"numLayers\":2,\"expertsPerLayer\":2,\"layers\":[]}", "invalid dimensions or stride"));
    {   // ids must be all explicit or all positional; offsets must follow the physical rank
        std::string mixed = fixtureLayoutJson(true, false);
        mixed.replace(mixed.find("\"expert\":1,"), 11, "");
        EXPECT(rejects(mixed, "either all explicit or all positional"));
        std::string moved = fixtureLayoutJson(true, true);
        moved.replace(moved.find("\"offset\":16384"), 14, "\"offset\":32768");
        EXPECT(rejects(moved, "offset or size does not match physical rank"));
        std::string dup = fixtureLayoutJson(true, true);
        dup.replace(dup.find("\"expert\":1"), 10, "\"expert\":0");
        EXPECT(rejects(dup, "duplicate or invalid expert mapping"));
    }
    {   // two tensors that overlap
        const std::string two = "{\"expertStride\":16384,\"numLayers\":1,\"expertsPerLayer\":1,\"layers\":[{\"layer\":0,\"file\":\"l.bin\",\"experts\":["
                                "{\"offset\":0,\"size\":16384,\"tensors\":{\"gate\":{\"offset\":0,\"size\":32,\"dtype\":\"U32\",\"shape\":[8,8]},"
                                "\"gate_scales\":{\"offset\":16,\"size\":32,\"dtype\":\"BF16\",\"shape\":[8,2]}}}]}]}";
        EXPECT(rejects(two, "overlapping ranges gate and gate_scales"));
    }
    {   // truncated and malformed documents
        bool truncated = false;
        try { PackedExpertsLayoutReader::decode("{\"expertStride\":16384,"); } catch (const GTurboFormatError &e) { truncated = e.kind == GTurboFormatError::truncated; }
        EXPECT(truncated);
        EXPECT(rejects("[1,2]", "expected an object"));
        bool overflow = false;
        try { PackedExpertsLayoutReader::decode("{\"expertStride\":99999999999999999999999}"); } catch (const GTurboFormatError &e) { overflow = e.kind == GTurboFormatError::overflow; }
        EXPECT(overflow);
    }
    {   // a permuted layer: logical expert 0 at physical rank 1; experts come back sorted by logical id, and the
        // nine routed offsets are read from expert 0 (Model.routedExpertOffsets, ModelExpertIO.swift:11-30)
        auto tensors = [](int base) {
            const char *roles[9] = {"gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"};
            std::string t = "{";
            for (int i = 0; i < 9; ++i) {
                t += i ? "," : "";
                t += std::string("\"") + roles[i] + "\":{\"offset\":" + std::to_string(base + 64 * i) + ",\"size\":64,\"dtype\":\"" +
                     (i % 3 == 0 ? "U32" : "BF16") + "\",\"shape\":[4,4]}";
            }
            return t + "}";
        };
        const std::string json = "{\"expertStride\":16384,\"numLayers\":1,\"expertsPerLayer\":2,\"layers\":[{\"layer\":0,\"file\":\"layer_00.bin\",\"experts\":["
                                 "{\"expert\":1,\"physicalRank\":0,\"offset\":0,\"size\":16384,\"tensors\":" + tensors(0) + "},"
                                 "{\"expert\":0,\"physicalRank\":1,\"offset\":16384,\"size\":16384,\"tensors\":" + tensors(128) + "}]}]}";
        const auto layout = PackedExpertsLayoutReader::decode(json);
        EXPECT(layout.expert(0, 0).physicalRank == 1 && layout.expert(0, 1).physicalRank == 0);
        EXPECT(layout.routedExpertPhysicalOffsets(0) == std::vector<uint64_t>({16384, 0}));
        const ffmoe_offsets o = layout.routedExpertOffsets(0);
        EXPECT(o.gate_w == 128 && o.gate_s == 192 && o.gate_b == 256 && o.up_w == 320 && o.down_b == 128 + 64 * 8);
    }
}

static uint16_t bf(float v) { return RouteTrimming::narrow(v, RouteTrimming::WeightType::bf16); }
static float fl(uint16_t b) { return RouteTrimming::widen(b, RouteTrimming::WeightType::bf16); }

static void routeTrimming() {
    // activeRoutedExperts (RealForwardRunner.swift:1952-1961): the first two ranks carry the row's whole weight
    {
        uint16_t w[8] = {bf(0.5f), bf(0.25f), bf(0.125f), bf(0.125f), bf(0.25f), bf(0.25f), bf(0.25f), bf(0.25f)};
        RouteTrimming::keepActiveRanks(w, 2, 4, 2);
        // row 0: full 1.0, kept 0.75: 0.5 / 0.75 and 0.25 / 0.75, rounded to bf16; row 1: kept 0.5 of 1.0
        EXPECT(w[0] == bf(0.5f * 1.0f / 0.75f) && w[1] == bf(0.25f * 1.0f / 0.75f) && w[2] == 0 && w[3] == 0);
        EXPECT(w[4] == bf(0.5f) && w[5] == bf(0.5f) && w[6] == 0 && w[7] == 0);
        uint16_t same[4] = {bf(0.4f), bf(0.3f), bf(0.2f), bf(0.1f)}, keep[4];
        std::memcpy(keep, same, sizeof keep);
        RouteTrimming::keepActiveRanks(same, 1, 4, 4);                 // all ranks active: nothing changes
        EXPECT(std::memcmp(same, keep, sizeof keep) == 0);
        uint16_t zero[2] = {0, bf(1.0f)};
        RouteTrimming::keepActiveRanks(zero, 1, 2, 1);                 // the kept weights add up to zero: left alone, the rest dropped
        EXPECT(zero[0] == 0 && zero[1] == 0);
        bool threw = false;
        try { RouteTrimming::keepActiveRanks(zero, 1, 2, 3); } catch (const std::invalid_argument &) { threw = true; }
        EXPECT(threw);
    }
    // prefillExpertUnionCap (capExpertUnion, RealForwardRunner.swift:828-847): three rows, top 2, five experts in use
    {
        const uint32_t ids[6] = {0, 1, 2, 1, 3, 4};
        uint16_t w[6] = {bf(0.75f), bf(0.25f), bf(0.5f), bf(0.5f), bf(0.5f), bf(0.5f)};
        // routed weight per expert: 0: 0.75, 1: 0.75, 2: 0.5, 3: 0.5, 4: 0.5 -> cap 3 keeps 0, 1 (tie: both in) and 2 (the lowest of the tie)
        const int before = RouteTrimming::capExpertUnion(ids, w, 3, 2, 8, 3);
        EXPECT(before == 5);
        EXPECT(w[0] == bf(0.75f) && w[1] == bf(0.25f));               // row 0 keeps both: scale 1
        EXPECT(w[2] == bf(0.5f) && w[3] == bf(0.5f));                 // row 1 keeps both
        EXPECT(w[4] == 0 && w[5] == 0);                               // row 2 lost both: nothing kept, scale 0
        uint16_t w2[4] = {bf(0.75f), bf(0.25f), bf(0.25f), bf(0.75f)};
        const uint32_t ids2[4] = {5, 6, 6, 7};
        // 5: 0.75, 6: 0.5, 7: 0.75 -> cap 2 keeps 5 and 7; each row's kept weight is rescaled to the row's total
        EXPECT(RouteTrimming::capExpertUnion(ids2, w2, 2, 2, 8, 2) == 3);
        EXPECT(w2[0] == bf(1.0f) && w2[1] == 0 && w2[2] == 0 && w2[3] == bf(1.0f));
        uint16_t w3[2] = {bf(0.5f), bf(0.5f)};
        const uint32_t ids3[2] = {1, 2};
        EXPECT(RouteTrimming::capExpertUnion(ids3, w3, 1, 2, 4, 2) == 2 && w3[0] == bf(0.5f) && w3[1] == bf(0.5f));   // within the cap: untouched
        bool threw = false;
        const uint32_t bad[2] = {1, 9};
        try { RouteTrimming::capExpertUnion(bad, w3, 1, 2, 4, 1); } catch (const std::invalid_argument &) { threw = true; }
        EXPECT(threw);
    }
    // FP16 patterns go through the same arithmetic
    {
        const auto h = RouteTrimming::WeightType::fp16;
        uint16_t w[2] = {RouteTrimming::narrow(0.75f, h), RouteTrimming::narrow(0.25f, h)};
        RouteTrimming::keepActiveRanks(w, 1, 2, 1, h);
        EXPECT(RouteTrimming::widen(w[0], h) == 1.0f && w[1] == 0);
        EXPECT(fl(bf(1.0f)) == 1.0f && bf(1.0f) == 0x3F80 && RouteTrimming::narrow(1.0f, h) == 0x3C00);
        // every FP16 pattern that is a number survives widen -> narrow; midpoints go to the even neighbour
        int bad = 0;
        for (uint32_t b = 0; b < 0x10000u; ++b) {
            if ((b & 0x7C00u) == 0x7C00u && (b & 0x3FFu)) continue;      // NaN
            bad += RouteTrimming::narrow(RouteTrimming::widen((uint16_t)b, h), h) != b;
        }
        EXPECT(bad == 0);
        EXPECT(RouteTrimming::narrow(65520.0f, h) == 0x7C00 && RouteTrimming::narrow(65519.0f, h) == 0x7BFF);
        EXPECT(RouteTrimming::narrow(1.0f + 0x1p-11f, h) == 0x3C00 && RouteTrimming::narrow(1.0f + 3 * 0x1p-11f, h) == 0x3C02);
        EXPECT(RouteTrimming::narrow(0x1p-25f, h) == 0 && RouteTrimming::narrow(0x1.8p-24f, h) == 2 && RouteTrimming::narrow(0x1p-24f, h) == 1);
    }
}

int main() {
    routeTrimming();
    groupingSortsPairsAndBuildsOffsetsCountsAndTiles();
    groupingCanOrderTilesByExpertSortKeys();
    groupingRejectsInvalidMetadataBeforeKernelUse();
    tokenExpertPairsAreTokenMajor();
    streamedTileBinding();
    supervisorPolicies();
    packedExpertsLayoutCodec();
    std::printf(failures ? "%d FAILURES\n" : "host logic ok\n", failures);
    return failures ? 1 : 0;
}
