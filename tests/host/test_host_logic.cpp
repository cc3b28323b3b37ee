// Host-logic tests of the C++ operator mirror (no GPU): exact expected arrays restated from the reference's
// PrefillMoEGroupingTests.swift, PrefillRouterTests.swift:12-22, PrefillGroupedRoutedMoETests+Binding.swift and
// the fault policy of DeviceSupervisorFailoverTests.swift:19-81.
#include <cstdio>
#include <cstring>

#include "../../ane-fieldfare_amd/host/fieldfare_host.hpp"

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

int main() {
    groupingSortsPairsAndBuildsOffsetsCountsAndTiles();
    groupingCanOrderTilesByExpertSortKeys();
    groupingRejectsInvalidMetadataBeforeKernelUse();
    tokenExpertPairsAreTokenMajor();
    streamedTileBinding();
    supervisorPolicies();
    std::printf(failures ? "%d FAILURES\n" : "host logic ok\n", failures);
    return failures ? 1 : 0;
}
