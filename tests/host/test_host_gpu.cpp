// GPU test of the C++ operator mirror: the reference's call sequence for one prefill layer
// (RealForwardRunner.swift:1487-1599) and one decode layer (:1846-1923) driven through the mirrored
// classes, checked against the CPU oracle. Built with hipcc, run by tests/test_host_cpp.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>

#include "../../ane-fieldfare_amd/host/fieldfare_host.hpp"
#include "../../ane-fieldfare_amd/host/packed_experts.hpp"
#include "../../oracle/ffmoe_oracle.h"

using namespace fieldfare;

static int failures = 0;
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) { std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } \
    } while (0)
#define HIP(x)                                                                                   \
    do {                                                                                         \
        hipError_t e_ = (x);                                                                     \
        if (e_ != hipSuccess) { std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); return 2; } \
    } while (0)

template <typename T>
static T *toDevice(const std::vector<T> &v) {
    T *p = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&p), v.size() * sizeof(T)) != hipSuccess) return nullptr;
    (void)hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice);
    return p;
}
template <typename T>
static std::vector<T> toHost(const T *p, size_t n) {
    std::vector<T> v(n);
    (void)hipMemcpy(v.data(), p, n * sizeof(T), hipMemcpyDeviceToHost);
    return v;
}

static void errorStats(const std::vector<uint16_t> &got, const std::vector<float> &ref, double &rel, double &cosine) {
    double maxd = 0, maxr = 0, dot = 0, ng = 0, nr = 0;
    for (size_t i = 0; i < ref.size(); ++i) {
        const double g = ffo_bf16_to_float(got[i]), r = ref[i];
        maxd = std::fmax(maxd, std::fabs(g - r));
        maxr = std::fmax(maxr, std::fabs(r));
        dot += g * r; ng += g * g; nr += r * r;
    }
    rel = maxd / std::fmax(maxr, 1e-6);
    cosine = dot / std::sqrt(ng * nr);
}

struct FaultingGuest : RoutedPrefillGuest {
    void runLayer(int, const uint16_t *, uint16_t *, const PrefillMoEGroupedRoutes &, const PrefillTokenExpertPair *) override {
        throw std::runtime_error("injected guest fault");
    }
};

int main() {
    const int d = 128, f = 64, E = 16, K = 8, T = 40;
    // synthetic experts: uniform weights quantised with the reference quantiser, blob layout of makeBlob
    // (MoEFusedFFNTests.swift:221-257)
    const size_t guW = (size_t)f * d / 2, guS = (size_t)f * (d / 64) * 2, dnW = (size_t)d * f / 2, dnS = (size_t)d * (f / 64) * 2;
    ffmoe_offsets off{};
    uint32_t cur = 0;
    auto take = [&](size_t n) { uint32_t o = cur; cur += (uint32_t)n; return o; };
    off.gate_w = take(guW); off.gate_s = take(guS); off.gate_b = take(guS);
    off.up_w = take(guW);   off.up_s = take(guS);   off.up_b = take(guS);
    off.down_w = take(dnW); off.down_s = take(dnS); off.down_b = take(dnS);
    const size_t stride = cur;
    std::vector<uint8_t> pool(stride * E);
    uint64_t rng = 0x5EED;
    auto fill = [&](uint8_t *blob, uint32_t wOff, uint32_t sOff, uint32_t bOff, int rows, int cols) {
        std::vector<float> row(cols);
        for (int r = 0; r < rows; ++r) {
            ffo_splitmix64_fill_uniform(&rng, -0.4f, 0.4f, row.data(), cols);
            ffo_quantize_int4_affine(row.data(), cols, blob + wOff + (size_t)r * cols / 2,
                                     reinterpret_cast<uint16_t *>(blob + sOff) + (size_t)r * (cols / 64),
                                     reinterpret_cast<uint16_t *>(blob + bOff) + (size_t)r * (cols / 64));
        }
    };
    for (int e = 0; e < E; ++e) {
        uint8_t *blob = pool.data() + e * stride;
        fill(blob, off.gate_w, off.gate_s, off.gate_b, f, d);
        fill(blob, off.up_w, off.up_s, off.up_b, f, d);
        fill(blob, off.down_w, off.down_s, off.down_b, d, f);
    }
    std::vector<uint16_t> router((size_t)E * d), x((size_t)T * d);
    for (auto &v : router) v = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, -0.05f, 0.05f));
    for (auto &v : x) v = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, -1.0f, 1.0f));

    ffmoe_shape shape{(uint32_t)d, (uint32_t)f, (uint32_t)E, (uint32_t)K, 1, 64};
    Context ctx(0, shape);
    ctx.uploadLayer(0, pool.data(), stride, off);
    ctx.uploadRouterBF16(0, router.data());
    hipStream_t stream;
    HIP(hipStreamCreate(&stream));

    uint16_t *dx = toDevice(x);
    uint32_t *dIdx = nullptr;
    uint16_t *dW = nullptr, *dPartials = nullptr, *dH2 = nullptr, *dH2b = nullptr;
    HIP(hipMalloc(reinterpret_cast<void **>(&dIdx), (size_t)T * K * 4));
    HIP(hipMalloc(reinterpret_cast<void **>(&dW), (size_t)T * K * 2));
    HIP(hipMalloc(reinterpret_cast<void **>(&dPartials), (size_t)T * K * d * 2));
    HIP(hipMalloc(reinterpret_cast<void **>(&dH2), (size_t)T * d * 2));
    HIP(hipMalloc(reinterpret_cast<void **>(&dH2b), (size_t)T * d * 2));

    // --- prefill layer, host-routed through the guest (the reference's sequence) ---
    PrefillRouter prefillRouter(ctx);
    PrefillGroupedRoutedMoE grouped(ctx);
    PrefillMoE prefillMoE(ctx);
    prefillRouter.encodeGemma4Block(stream, 0, dx, dIdx, dW, T, d);
    HIP(hipStreamSynchronize(stream));                       // the reference's waitForCompletion(cb)
    auto idx = toHost(dIdx, (size_t)T * K);
    auto w = toHost(dW, (size_t)T * K);
    auto pairs = PrefillRouter::makeTokenExpertPairs(idx, w, T, K);
    auto routes = PrefillMoEGrouping::groupTokenExpertPairs(pairs, T, K, E, 16);
    PrefillTokenExpertPair *dPairs = toDevice(routes.sortedPairs);
    auto sync = [](void *s) { (void)hipStreamSynchronize(static_cast<hipStream_t>(s)); };
    DeviceSupervisor supervisor(1, RuntimeFaultPolicy::failoverHost,
                                std::make_shared<HipRoutedPrefillGuest>(ctx, stream, T, d, sync));
    HIP(hipMemsetAsync(dPartials, 0, (size_t)T * K * d * 2, stream));   // the host zeroes partials first
    bool done = false;
    if (auto *guest = supervisor.routedPrefill(0))
        done = supervisor.supervise(0, [&] { guest->runLayer(0, dx, dPartials, routes, dPairs); });
    EXPECT(done && !supervisor.evicted());
    prefillMoE.encodeReduceTokenMajor(stream, dPartials, dW, dH2, T, K, d);
    HIP(hipStreamSynchronize(stream));
    auto h2 = toHost(dH2, (size_t)T * d);

    std::vector<float> wf(w.size()), ref((size_t)T * d);
    for (size_t i = 0; i < w.size(); ++i) wf[i] = ffo_bf16_to_float(w[i]);
    ffo_offsets ooff;
    std::memcpy(&ooff, &off, sizeof ooff);
    ffo_moe_experts(pool.data(), stride, &ooff, d, f, x.data(), d, T, K, FFO_BF16, idx.data(), wf.data(), ref.data(), 0);
    double rel, cosine;
    errorStats(h2, ref, rel, cosine);
    std::printf("prefill via guest: rel err %.2e cosine %.6f\n", rel, cosine);
    EXPECT(rel <= 1e-2 && cosine >= 0.9999);
    // router indices are the oracle's
    std::vector<float> logits(E), ow(K);
    std::vector<uint32_t> oidx(K);
    for (int t = 0; t < T; ++t) {
        ffo_router_logits_pinned(router.data(), 0, x.data() + (size_t)t * d, FFO_BF16, nullptr, E, d, logits.data());
        ffo_topk_softmax(logits.data(), E, K, nullptr, oidx.data(), ow.data());
        EXPECT(std::memcmp(oidx.data(), idx.data() + (size_t)t * K, K * 4) == 0);
    }

    // --- the same layer GPU-routed: bit-identical to the host-routed result ---
    grouped.encodeGPURouted(stream, 0, dx, d, T, dIdx, dW, dH2b);
    HIP(hipStreamSynchronize(stream));
    EXPECT(toHost(dH2b, (size_t)T * d) == h2);

    // --- a faulting guest under failover: the host clears the rows and runs the layer itself ---
    DeviceSupervisor failing(1, RuntimeFaultPolicy::failoverHost, std::make_shared<FaultingGuest>());
    done = failing.supervise(0, [&] { failing.routedPrefill(0)->runLayer(0, dx, dPartials, routes, dPairs); });
    EXPECT(!done && failing.evicted() && failing.faults().size() == 1 && failing.routedPrefill(0) == nullptr);
    HIP(hipMemsetAsync(dPartials, 0, (size_t)T * K * d * 2, stream));
    grouped.encodeStreamedBatched(stream, 0, dx, d, dPairs, (uint32_t)routes.sortedPairs.size(), T, dPartials);
    prefillMoE.encodeReduceTokenMajor(stream, dPartials, dW, dH2b, T, K, d);
    HIP(hipStreamSynchronize(stream));
    EXPECT(toHost(dH2b, (size_t)T * d) == h2);

    // --- decode layer: router + GPU slots ---
    MoE moe(ctx);
    moe.encodeRouterGemma4(stream, 0, dx, dIdx, dW);
    moe.encodeRoutedPersistentGPUSlots(stream, 0, dx, dIdx, dW, nullptr, dH2b);
    HIP(hipStreamSynchronize(stream));
    auto y1 = toHost(dH2b, d);
    auto idx1 = toHost(dIdx, K);
    auto w1 = toHost(dW, K);
    std::vector<float> w1f(K), ref1(d);
    for (int i = 0; i < K; ++i) w1f[i] = ffo_bf16_to_float(w1[i]);
    ffo_moe_experts(pool.data(), stride, &ooff, d, f, x.data(), d, 1, K, FFO_BF16, idx1.data(), w1f.data(), ref1.data(), 0);
    errorStats(y1, ref1, rel, cosine);
    std::printf("decode: rel err %.2e cosine %.6f\n", rel, cosine);
    EXPECT(rel <= 1e-2 && cosine >= 0.9999);
    bool threw = false;
    try { moe.encodeRouterRowsGemma4(stream, 0, dx, d, 17, dIdx, dW); } catch (const std::invalid_argument &) { threw = true; }
    EXPECT(threw);

    // --- DequantInt4GEMV on one expert's gate matrix (reference layout, device copy of the blob) ---
    uint8_t *dPool = toDevice(pool);
    uint16_t *dY = nullptr;
    HIP(hipMalloc(reinterpret_cast<void **>(&dY), f * 2));
    DequantInt4GEMV gemv(ctx);
    gemv.encode(stream, dPool + off.gate_w, reinterpret_cast<uint16_t *>(dPool + off.gate_s),
                reinterpret_cast<uint16_t *>(dPool + off.gate_b), dx, dY, f, d);
    HIP(hipStreamSynchronize(stream));
    auto yg = toHost(dY, f);
    std::vector<float> xf(d), refg(f);
    for (int i = 0; i < d; ++i) xf[i] = ffo_bf16_to_float(x[i]);
    ffo_gemv_int4_ref(pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                      reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), f, d, xf.data(), refg.data());
    errorStats(yg, refg, rel, cosine);
    EXPECT(rel <= 1e-2);

    // --- PrefillFinalRowHeadInt4: row 2 of the block through a norm and the same 64-row "head": the oracle's normed row
    // bit for bit, and logits of its dequantised rows ---
    {
        std::vector<uint16_t> normW(d);
        for (auto &v : normW) v = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, 0.5f, 1.5f));
        uint16_t *dNormW = toDevice(normW), *dNormed = nullptr, *dLogits16 = nullptr;
        HIP(hipMalloc(reinterpret_cast<void **>(&dNormed), (size_t)d * 2));
        HIP(hipMalloc(reinterpret_cast<void **>(&dLogits16), (size_t)f * 2));
        PrefillFinalRowHeadInt4 finalRow(ctx, 256, pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                                         reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), d, f);
        bool threwStride = false, threwMaxD = false;
        try { finalRow.encodeLogits(stream, dx, 2, d - 1, dNormW, dNormed, dLogits16, 1e-6f); }
        catch (const std::invalid_argument &) { threwStride = true; }
        EXPECT(threwStride);
        try {
            PrefillFinalRowHeadInt4 small(ctx, 64, pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                                          reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), d, f);
        } catch (const std::invalid_argument &) { threwMaxD = true; }
        EXPECT(threwMaxD);
        finalRow.encodeLogits(stream, dx, 2, d, dNormW, dNormed, dLogits16, 1e-6f);
        HIP(hipStreamSynchronize(stream));
        std::vector<uint16_t> refNormed(d);
        ffo_rmsnorm(x.data() + (size_t)2 * d, normW.data(), refNormed.data(), d, 1e-6f, FFO_BF16);
        EXPECT(toHost(dNormed, (size_t)d) == refNormed);
        std::vector<float> xr(d), refLogits(f);
        for (int i = 0; i < d; ++i) xr[i] = ffo_bf16_to_float(refNormed[i]);
        ffo_gemv_int4_ref(pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                          reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), f, d, xr.data(), refLogits.data());
        double relF = 0, cosF = 0;
        errorStats(toHost(dLogits16, (size_t)f), refLogits, relF, cosF);
        EXPECT(relF <= 1e-2 && cosF >= 0.9999);
        HIP(hipFree(dNormW)); HIP(hipFree(dNormed)); HIP(hipFree(dLogits16));
    }

    // --- LMHeadChainInt4 over the same matrix as a 64-token "vocabulary": greedy token == CPU argmax ---
    {
        LMHeadChainInt4 head(ctx, pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                             reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), d, f);
        uint32_t *dTok = nullptr;
        HIP(hipMalloc(reinterpret_cast<void **>(&dTok), 4 * sizeof(uint32_t)));
        head.encodeGreedyRows(stream, dx, d, 3, dTok);
        HIP(hipStreamSynchronize(stream));
        auto tok = toHost(dTok, 3);
        for (int r = 0; r < 3; ++r) {
            std::vector<float> xr(d), ref(f);
            for (int i = 0; i < d; ++i) xr[i] = ffo_bf16_to_float(x[(size_t)r * d + i]);
            ffo_gemv_int4_ref(pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                              reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), f, d, xr.data(), ref.data());
            uint32_t best = 0;
            for (int i = 1; i < f; ++i)
                if (ref[i] > ref[best]) best = i;
            EXPECT(tok[r] == best);
        }
        bool threwRows = false;
        try { head.encodeGreedyRows(stream, dx, d, 17, dTok); } catch (const std::invalid_argument &) { threwRows = true; }
        EXPECT(threwRows);
        // the tied embedding: the rows of the three greedy tokens, and row 5 by value, from the same resident table
        {
            uint16_t *dEmb = nullptr;
            HIP(hipMalloc(reinterpret_cast<void **>(&dEmb), (size_t)4 * d * 2));
            const float outScale = std::sqrt((float)d);
            head.encodeEmbedLookupRows(stream, dTok, 3, outScale, dEmb, d);
            head.encodeEmbedLookup(stream, 5, outScale, dEmb + (size_t)3 * d);
            HIP(hipStreamSynchronize(stream));
            auto emb = toHost(dEmb, (size_t)4 * d);
            std::vector<float> rowF(d);
            for (int r = 0; r < 4; ++r) {
                const uint32_t id = r < 3 ? tok[r] : 5u;
                ffo_dequantize_int4_affine(pool.data() + off.gate_w + (size_t)id * d / 2,
                                           reinterpret_cast<uint16_t *>(pool.data() + off.gate_s) + (size_t)id * d / 64,
                                           reinterpret_cast<uint16_t *>(pool.data() + off.gate_b) + (size_t)id * d / 64, d, rowF.data());
                for (int i = 0; i < d; ++i) EXPECT(emb[(size_t)r * d + i] == ffo_bf16_bits(rowF[i] * outScale));
            }
            HIP(hipFree(dEmb));
        }
        // the same choice with the winner's probability (softmax of the row's logits, no softcap): same tokens, and
        // the probability the fp64 softmax of the CPU logits gives
        float *dConf = nullptr, *dLogits = nullptr;
        uint32_t *dTok2 = nullptr, *dIds = nullptr;
        HIP(hipMalloc(reinterpret_cast<void **>(&dConf), 4 * sizeof(float)));
        HIP(hipMalloc(reinterpret_cast<void **>(&dTok2), 4 * sizeof(uint32_t)));
        head.encodeGreedyRowsWithConfidence(stream, dx, d, 3, 0.0f, dTok2, dConf);
        HIP(hipStreamSynchronize(stream));
        EXPECT(toHost(dTok2, 3) == tok);
        auto conf = toHost(dConf, 3);
        // the hot-vocabulary form over eight listed rows of the table: position of the best listed row
        const std::vector<uint32_t> ids = {60, 5, 33, 9, 17, 41, 2, 50};
        dIds = toDevice(ids);
        HIP(hipMalloc(reinterpret_cast<void **>(&dLogits), 3 * ids.size() * sizeof(float)));
        // (the listed projection reads the table where it lies: the device copy of the blob)
        LMHeadChainInt4::encodeHotGreedyRows(ctx, stream, dx, d, 3, dIds, (uint32_t)ids.size(), dPool + off.gate_w,
                                             reinterpret_cast<uint16_t *>(dPool + off.gate_s),
                                             reinterpret_cast<uint16_t *>(dPool + off.gate_b), d, 0.0f, dLogits, dTok2, dConf);
        HIP(hipStreamSynchronize(stream));
        auto hot = toHost(dTok2, 3);
        for (int r = 0; r < 3; ++r) {
            std::vector<float> xr(d), ref(f);
            for (int i = 0; i < d; ++i) xr[i] = ffo_bf16_to_float(x[(size_t)r * d + i]);
            ffo_gemv_int4_ref(pool.data() + off.gate_w, reinterpret_cast<uint16_t *>(pool.data() + off.gate_s),
                              reinterpret_cast<uint16_t *>(pool.data() + off.gate_b), f, d, xr.data(), ref.data());
            double sum = 0;
            for (int i = 0; i < f; ++i) sum += std::exp((double)ref[i] - (double)ref[tok[r]]);
            EXPECT(std::fabs(conf[r] - 1.0 / sum) <= 2e-3 * (1.0 / sum) + 1e-6);
            uint32_t best = 0;
            for (size_t i = 1; i < ids.size(); ++i)
                if (ref[ids[i]] > ref[ids[best]]) best = (uint32_t)i;
            EXPECT(hot[r] == best);
        }
        // the sampled choice over the same listed logits: top_k = 1 keeps the best listed row alone, whatever the noise
        LMHeadChainInt4::RowSampling sampling;
        sampling.topK = 1;
        sampling.seed = 0x5EED;
        sampling.keyBase = 40;
        LMHeadChainInt4::encodeSampledChoice(ctx, stream, dLogits, (uint32_t)ids.size(), 3, (uint32_t)ids.size(), dIds, 30.0f,
                                             sampling, dTok2, dConf);
        HIP(hipStreamSynchronize(stream));
        EXPECT(toHost(dTok2, 3) == hot);
        EXPECT(toHost(dConf, 3) == std::vector<float>(3, 1.0f));
        HIP(hipFree(dConf));
        HIP(hipFree(dTok2));
        HIP(hipFree(dIds));
        HIP(hipFree(dLogits));
        HIP(hipFree(dTok));
    }

    // --- shared expert: expert 3's projections as the dense FFN, one row and a 40-row block ---
    {
        ffmoe_shape denseShape{(uint32_t)d, (uint32_t)f, 1, 1, 1, 64};
        Context dense(0, denseShape);
        const uint8_t *blob = pool.data() + 3 * stride;
        auto u16 = [&](uint32_t o) { return reinterpret_cast<const uint16_t *>(blob + o); };
        const SharedExpertProjection gate{blob + off.gate_w, u16(off.gate_s), u16(off.gate_b), (uint32_t)f, (uint32_t)d};
        const SharedExpertProjection up{blob + off.up_w, u16(off.up_s), u16(off.up_b), (uint32_t)f, (uint32_t)d};
        const SharedExpertProjection down{blob + off.down_w, u16(off.down_s), u16(off.down_b), (uint32_t)d, (uint32_t)f};
        PrefillSharedExpert shared(dense);
        bool threwDims = false;
        try { shared.load(0, gate, down, down); } catch (const SharedExpertError &e) { threwDims = e.kind == SharedExpertError::dimensionMismatch; }
        EXPECT(threwDims);
        bool threwBits = false;
        try { SharedExpertRuntime bad(dense, 6); } catch (const SharedExpertError &e) { threwBits = e.kind == SharedExpertError::unsupportedWeightBits; }
        EXPECT(threwBits);
        shared.load(0, gate, up, down);
        ffo_offsets fo{off.gate_w, off.gate_s, off.gate_b, off.up_w, off.up_s, off.up_b, off.down_w, off.down_s, off.down_b};
        std::vector<float> refAll((size_t)T * d), xr(d);
        for (int r = 0; r < T; ++r) {
            for (int i = 0; i < d; ++i) xr[i] = ffo_bf16_to_float(x[(size_t)r * d + i]);
            ffo_run_ffn(blob, &fo, d, f, xr.data(), refAll.data() + (size_t)r * d);
        }
        shared.encode(stream, 0, dx, dH2);
        shared.encodeBlock(stream, 0, dx, dH2b, T, d, f, d, d);
        HIP(hipStreamSynchronize(stream));
        double relS = 0, cosS = 0;
        errorStats(toHost(dH2, (size_t)d), std::vector<float>(refAll.begin(), refAll.begin() + d), relS, cosS);
        EXPECT(relS <= 1e-2 && cosS >= 0.9999);
        errorStats(toHost(dH2b, (size_t)T * d), refAll, relS, cosS);
        EXPECT(relS <= 1e-2 && cosS >= 0.9999);

        // the same block with FP16 rows in and out (the reference's text-path type): the bf16 inputs above are
        // exactly representable in FP16, so the reference rows are the same
        Context dense16(0, denseShape);
        bool threwType = false;
        try { dense16.setActivationDtype(5); } catch (const std::invalid_argument &) { threwType = true; }
        EXPECT(threwType);
        dense16.setActivationDtype(FFMOE_FP16);
        PrefillSharedExpert shared16(dense16);
        shared16.load(0, gate, up, down);
        std::vector<uint16_t> xh((size_t)T * d);
        for (size_t i = 0; i < xh.size(); ++i) {
            const _Float16 h = (_Float16)ffo_bf16_to_float(x[i]);
            std::memcpy(&xh[i], &h, 2);
        }
        uint16_t *dxh = toDevice(xh);
        shared16.encodeBlock(stream, 0, dxh, dH2b, T, d, f, d, d);
        shared16.encode(stream, 0, dxh, dH2);
        HIP(hipStreamSynchronize(stream));
        auto asBf16Ref = [&](const std::vector<uint16_t> &halfBits, const std::vector<float> &ref, double &rel, double &cosine) {
            double maxd = 0, maxr = 0, dot = 0, ng = 0, nr = 0;
            for (size_t i = 0; i < ref.size(); ++i) {
                _Float16 h;
                std::memcpy(&h, &halfBits[i], 2);
                const double g = (float)h, r = ref[i];
                maxd = std::fmax(maxd, std::fabs(g - r));
                maxr = std::fmax(maxr, std::fabs(r));
                dot += g * r; ng += g * g; nr += r * r;
            }
            rel = maxd / std::fmax(maxr, 1e-6);
            cosine = dot / std::sqrt(ng * nr);
        };
        asBf16Ref(toHost(dH2b, (size_t)T * d), refAll, relS, cosS);
        EXPECT(relS <= 1e-2 && cosS >= 0.9999);
        asBf16Ref(toHost(dH2, (size_t)d), std::vector<float>(refAll.begin(), refAll.begin() + d), relS, cosS);
        EXPECT(relS <= 1e-2 && cosS >= 0.9999);
        HIP(hipFree(dxh));
    }

    // --- the 8-bit shared expert (SharedExpertInt8, the packs' default form): 1 row and a 40-row block against the
    // dequantised rows in double with the operator's 16-bit roundings (gate, up, activation), and its guards ---
    {
        struct Proj8 { std::vector<uint8_t> w; std::vector<uint16_t> s, b; std::vector<float> deq; };
        auto make8 = [&](int rows, int cols) {
            Proj8 p;
            p.w.resize((size_t)rows * cols); p.s.resize((size_t)rows * cols / 64); p.b.resize(p.s.size()); p.deq.resize(p.w.size());
            std::vector<float> row(cols);
            for (int r = 0; r < rows; ++r) {
                ffo_splitmix64_fill_uniform(&rng, -0.08f, 0.08f, row.data(), (size_t)cols);
                ffo_quantize_int8_affine(row.data(), cols, &p.w[(size_t)r * cols], &p.s[(size_t)r * cols / 64], &p.b[(size_t)r * cols / 64]);
                ffo_dequantize_int8_affine(&p.w[(size_t)r * cols], &p.s[(size_t)r * cols / 64], &p.b[(size_t)r * cols / 64], cols,
                                           &p.deq[(size_t)r * cols]);
            }
            return p;
        };
        const Proj8 g8 = make8(f, d), u8 = make8(f, d), d8 = make8(d, f);
        const SharedExpertProjection gate{g8.w.data(), g8.s.data(), g8.b.data(), (uint32_t)f, (uint32_t)d};
        const SharedExpertProjection up{u8.w.data(), u8.s.data(), u8.b.data(), (uint32_t)f, (uint32_t)d};
        const SharedExpertProjection down{d8.w.data(), d8.s.data(), d8.b.data(), (uint32_t)d, (uint32_t)f};
        std::vector<float> ref8((size_t)T * d), act(f);
        for (int r = 0; r < T; ++r) {
            for (int j = 0; j < f; ++j) {
                double ga = 0, ua = 0;
                for (int i = 0; i < d; ++i) {
                    const double xi = ffo_bf16_to_float(x[(size_t)r * d + i]);
                    ga += (double)g8.deq[(size_t)j * d + i] * xi;
                    ua += (double)u8.deq[(size_t)j * d + i] * xi;
                }
                const float gr = ffo_bf16_to_float(ffo_bf16_bits((float)ga)), ur = ffo_bf16_to_float(ffo_bf16_bits((float)ua));
                act[j] = ffo_bf16_to_float(ffo_bf16_bits(ffo_gelu_tanh(gr) * ur));
            }
            for (int i = 0; i < d; ++i) {
                double ya = 0;
                for (int j = 0; j < f; ++j) ya += (double)d8.deq[(size_t)i * f + j] * act[j];
                ref8[(size_t)r * d + i] = (float)ya;
            }
        }
        ffmoe_shape dense8Shape{(uint32_t)d, (uint32_t)f, 1, 1, 2, 64};
        Context dense8(0, dense8Shape);
        PrefillSharedExpert shared8(dense8, 8);
        EXPECT(shared8.weightBits() == 8);
        bool threwDims = false, threwUnloaded = false, threwRouted = false;
        try { shared8.encode(stream, 1, dx, dH2); } catch (const FieldfareError &e) { threwUnloaded = e.code == FFMOE_ERR_NO_LAYER; }
        EXPECT(threwUnloaded);
        try { shared8.load(1, gate, up, up); } catch (const SharedExpertError &e) { threwDims = e.kind == SharedExpertError::dimensionMismatch; }
        EXPECT(threwDims);
        try { SharedExpertInt8 onRouted(ctx); } catch (const std::invalid_argument &) { threwRouted = true; }
        EXPECT(threwRouted);
        shared8.load(1, gate, up, down);
        shared8.encode(stream, 1, dx, dH2);
        shared8.encodeBlock(stream, 1, dx, dH2b, T, d, f, d, d);
        HIP(hipStreamSynchronize(stream));
        double rel8 = 0, cos8 = 0;
        const std::vector<uint16_t> row0 = toHost(dH2, (size_t)d);
        errorStats(row0, std::vector<float>(ref8.begin(), ref8.begin() + d), rel8, cos8);
        EXPECT(rel8 <= 1e-2 && cos8 >= 0.9999);
        const std::vector<uint16_t> block = toHost(dH2b, (size_t)T * d);
        errorStats(block, ref8, rel8, cos8);
        EXPECT(rel8 <= 1e-2 && cos8 >= 0.9999);
        EXPECT(std::equal(row0.begin(), row0.end(), block.begin()));       // row 0 of the block is the single-row call's
        // DequantInt8GEMV on the down projection: rows of the activation scratch are not exposed, so feed it x's first f values
        DequantInt8GEMV down8(ctx, d8.w.data(), d8.s.data(), d8.b.data(), (uint32_t)d, (uint32_t)f);
        EXPECT(down8.m() == (uint32_t)d && down8.n() == (uint32_t)f);
        down8.encodeRows(stream, dx, dH2b, 3, (uint32_t)d, (uint32_t)d);
        HIP(hipStreamSynchronize(stream));
        std::vector<float> refDown((size_t)3 * d);
        for (int r = 0; r < 3; ++r)
            for (int i = 0; i < d; ++i) {
                double acc = 0;
                for (int j2 = 0; j2 < f; ++j2) acc += (double)d8.deq[(size_t)i * f + j2] * ffo_bf16_to_float(x[(size_t)r * d + j2]);
                refDown[(size_t)r * d + i] = (float)acc;
            }
        errorStats(toHost(dH2b, (size_t)3 * d), refDown, rel8, cos8);
        EXPECT(rel8 <= 1e-2 && cos8 >= 0.9999);
        bool threwRows8 = false;
        try { down8.encodeRows(stream, dx, dH2b, 17, (uint32_t)d, (uint32_t)d); } catch (const std::invalid_argument &) { threwRows8 = true; }
        EXPECT(threwRows8);
    }

    // --- post-attention setup and layer tail through the mirrored classes: a 5-row block against the oracle's
    // rows, bit for bit, and the one-row forms against row 0 ---
    {
        const int R = 5;
        auto draw = [&](size_t n, float lo, float hi) {
            std::vector<uint16_t> v(n);
            for (auto &b : v) b = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, lo, hi));
            return v;
        };
        auto hid = draw((size_t)R * d, -2.f, 2.f), att = draw((size_t)R * d, -1.f, 1.f), h2v = draw((size_t)R * d, -1.f, 1.f),
             h1v = draw((size_t)R * d, -3.f, 3.f);
        std::vector<std::vector<uint16_t>> wts;
        for (int i = 0; i < 5; ++i) wts.push_back(draw(d, 0.5f, 1.5f));
        std::vector<uint16_t> refH = hid, refDense((size_t)R * d), refRouted((size_t)R * d), refRouter((size_t)R * d);
        for (int r = 0; r < R; ++r)
            ffo_post_attn_setup(refH.data() + (size_t)r * d, att.data() + (size_t)r * d, refDense.data() + (size_t)r * d,
                                refRouted.data() + (size_t)r * d, refRouter.data() + (size_t)r * d, wts[0].data(), wts[1].data(),
                                wts[2].data(), d, 1e-6f, FFO_BF16);
        std::vector<uint16_t> refT = refH;
        for (int r = 0; r < R; ++r)
            ffo_layer_tail(h2v.data() + (size_t)r * d, h1v.data() + (size_t)r * d, refT.data() + (size_t)r * d, wts[3].data(),
                           wts[4].data(), d, 1e-6f, 0.875f, FFO_BF16);
        uint16_t *dHid = toDevice(hid), *dAtt = toDevice(att), *dH2v = toDevice(h2v), *dH1v = toDevice(h1v);
        uint16_t *dWt[5];
        for (int i = 0; i < 5; ++i) dWt[i] = toDevice(wts[i]);
        uint16_t *dOut[3];
        for (auto &p : dOut) HIP(hipMalloc(reinterpret_cast<void **>(&p), (size_t)R * d * 2));
        PrefillPostAttentionSetup setup(ctx);
        PrefillLayerTail tail(ctx);
        setup.encode(stream, dHid, dAtt, dOut[0], dOut[1], dOut[2], dWt[0], dWt[1], dWt[2], R, d, d, d, d, d, d, 1e-6f);
        HIP(hipStreamSynchronize(stream));
        EXPECT(toHost(dHid, (size_t)R * d) == refH && toHost(dOut[0], (size_t)R * d) == refDense);
        EXPECT(toHost(dOut[1], (size_t)R * d) == refRouted && toHost(dOut[2], (size_t)R * d) == refRouter);
        tail.encode(stream, dH2v, dH1v, dHid, dWt[3], dWt[4], R, d, d, d, d, 1e-6f, 0.875f);
        HIP(hipStreamSynchronize(stream));
        EXPECT(toHost(dHid, (size_t)R * d) == refT);
        // decode forms on row 0
        uint16_t *dRow = toDevice(std::vector<uint16_t>(hid.begin(), hid.begin() + d));
        FusedPostAttentionSetup setup1(ctx);
        FusedLayerTail tail1(ctx);
        setup1.encode(stream, dRow, dAtt, dOut[0], dOut[1], dOut[2], dWt[0], dWt[1], dWt[2], d, 1e-6f);
        tail1.encode(stream, dH2v, dH1v, dRow, dWt[3], dWt[4], d, 1e-6f, 0.875f);
        HIP(hipStreamSynchronize(stream));
        EXPECT(toHost(dRow, (size_t)d) == std::vector<uint16_t>(refT.begin(), refT.begin() + d));
        // encodeWithNorms on row 0 equals RMSNorm(h1), encode, RMSNorm(hidden) bit for bit and leaves h1 alone
        {
            RMSNorm norm(ctx);
            uint16_t *sepHid = toDevice(std::vector<uint16_t>(hid.begin(), hid.begin() + d));
            uint16_t *fusHid = toDevice(std::vector<uint16_t>(hid.begin(), hid.begin() + d));
            const std::vector<uint16_t> h1Before = toHost(dH1v, (size_t)d);
            norm.encodeBF16W(stream, dH1v, dWt[0], dOut[0], d, 1e-6f);
            tail1.encode(stream, dH2v, dOut[0], sepHid, dWt[3], dWt[4], d, 1e-6f, 0.875f);
            norm.encodeBF16W(stream, sepHid, dWt[1], dOut[1], d, 1e-6f);
            tail1.encodeWithNorms(stream, dH2v, dH1v, fusHid, dWt[0], dWt[3], dWt[4], dWt[1], dOut[2], d, 1e-6f, 0.875f);
            HIP(hipStreamSynchronize(stream));
            EXPECT(toHost(fusHid, (size_t)d) == toHost(sepHid, (size_t)d));
            EXPECT(toHost(dOut[2], (size_t)d) == toHost(dOut[1], (size_t)d));
            EXPECT(toHost(dH1v, (size_t)d) == h1Before);
            bool threwPair = false;
            try { tail1.encodeWithNorms(stream, dH2v, dH1v, fusHid, dWt[0], dWt[3], dWt[4], dWt[1], nullptr, d, 1e-6f, 1.f); }
            catch (const std::invalid_argument &) { threwPair = true; }
            EXPECT(threwPair);
            HIP(hipFree(sepHid));
            HIP(hipFree(fusHid));
        }
        bool threwStride = false;
        try { tail.encode(stream, dH2v, dH1v, dHid, dWt[3], dWt[4], R, d, d - 8, d, d, 1e-6f, 1.f); } catch (const std::invalid_argument &) { threwStride = true; }
        EXPECT(threwStride);
        for (auto p : {dHid, dAtt, dH2v, dH1v, dRow, dOut[0], dOut[1], dOut[2]}) HIP(hipFree(p));
        for (auto p : dWt) HIP(hipFree(p));
    }

    // --- packed experts: a two-layer checkpoint directory written as ModelLoaderTests.swift:204-241 writes its
    // toy one (16 KiB stride, layout.json with explicit ids), layer 1 with reversed physical ranks; after
    // uploadPackedExperts every expert expands to the same bf16 weights as the directly uploaded blobs ---
    {
        char tmpl[] = "/tmp/ffmoe_ckpt_XXXXXX";
        const char *dir = mkdtemp(tmpl);
        EXPECT(dir != nullptr);
        const std::string root = dir ? dir : "/tmp";
        EXPECT(std::system(("mkdir -p " + root + "/packed_experts").c_str()) == 0);
        const uint64_t ckStride = 16384;
        EXPECT(stride <= ckStride);
        auto tensorsJson = [&]() {
            const char *roles[9] = {"gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases"};
            const uint32_t offs[9] = {off.gate_w, off.gate_s, off.gate_b, off.up_w, off.up_s, off.up_b, off.down_w, off.down_s, off.down_b};
            const size_t sizes[9] = {guW, guS, guS, guW, guS, guS, dnW, dnS, dnS};
            std::string t = "{";
            for (int i = 0; i < 9; ++i) {
                const bool wt = i % 3 == 0;
                const int rows = i < 6 ? f : d, cols = i < 6 ? d : f;
                t += (i ? "," : "") + std::string("\"") + roles[i] + "\":{\"offset\":" + std::to_string(offs[i]) + ",\"size\":" + std::to_string(sizes[i]) +
                     ",\"dtype\":\"" + (wt ? "U32" : "BF16") + "\",\"shape\":[" + std::to_string(rows) + "," + std::to_string(wt ? cols : cols / 64) + "]" +
                     (wt ? ",\"bits\":4" : "") + "}";
            }
            return t + "}";
        };
        std::string layersJson;
        for (int L = 0; L < 2; ++L) {
            std::vector<uint8_t> payload(ckStride * E, 0);
            std::string expertsJson;
            for (int e = 0; e < E; ++e) {
                const int rank = L == 0 ? e : E - 1 - e;
                std::memcpy(payload.data() + (size_t)rank * ckStride, pool.data() + (size_t)e * stride, stride);
                expertsJson += (e ? "," : "") + std::string("{\"expert\":") + std::to_string(e) + ",\"physicalRank\":" + std::to_string(rank) +
                               ",\"offset\":" + std::to_string((uint64_t)rank * ckStride) + ",\"size\":" + std::to_string(ckStride) + ",\"tensors\":" + tensorsJson() + "}";
            }
            const std::string file = "layer_0" + std::to_string(L) + ".bin";
            std::ofstream(root + "/packed_experts/" + file, std::ios::binary).write(reinterpret_cast<const char *>(payload.data()), (std::streamsize)payload.size());
            layersJson += (L ? "," : "") + std::string("{\"layer\":") + std::to_string(L) + ",\"file\":\"" + file + "\",\"experts\":[" + expertsJson + "]}";
        }
        std::ofstream(root + "/packed_experts/layout.json") << "{\"expertStride\":" << ckStride << ",\"numLayers\":2,\"expertsPerLayer\":" << E
                                                             << ",\"layers\":[" << layersJson << "]}";
        const PackedExpertsLayout layout = PackedExpertsLayoutReader::read(root);
        EXPECT(layout.numLayers == 2 && layout.expertsPerLayer == E && layout.expert(1, 0).physicalRank == E - 1);
        ffmoe_shape ckShape{(uint32_t)d, (uint32_t)f, (uint32_t)E, (uint32_t)K, 2, 64};
        Context ck(0, ckShape);
        EXPECT(uploadPackedExperts(ck, root, layout) == 2 * ckStride * E);
        uint16_t *dA = nullptr, *dB = nullptr;
        HIP(hipMalloc(reinterpret_cast<void **>(&dA), (size_t)f * d * 2));
        HIP(hipMalloc(reinterpret_cast<void **>(&dB), (size_t)f * d * 2));
        int mismatches = 0;
        for (int L = 0; L < 2; ++L)
            for (int e = 0; e < E; ++e)
                for (int which = 0; which < 3; ++which) {
                    char *err = nullptr;
                    check(ffmoe_dequant_expert(ctx.raw(), stream, 0, (uint32_t)e, which, dA, &err), err);
                    check(ffmoe_dequant_expert(ck.raw(), stream, (uint32_t)L, (uint32_t)e, which, dB, &err), err);
                    HIP(hipStreamSynchronize(stream));
                    if (toHost(dA, (size_t)f * d) != toHost(dB, (size_t)f * d)) ++mismatches;
                }
        EXPECT(mismatches == 0);
        // a layer file shorter than the layout says, and a shape the context does not have
        bool threwSize = false;
        EXPECT(truncate((root + "/packed_experts/layer_01.bin").c_str(), (off_t)(ckStride * (E - 1))) == 0);
        try { uploadPackedExperts(ck, root, layout); } catch (const MappedExpertLayerError &e) { threwSize = e.kind == MappedExpertLayerError::sizeMismatch; }
        EXPECT(threwSize);
        bool threwShape = false;
        ffmoe_shape other{(uint32_t)d, (uint32_t)(2 * f), (uint32_t)E, (uint32_t)K, 2, 64};
        Context wrong(0, other);
        try { uploadPackedExperts(wrong, root, layout); } catch (const GTurboFormatError &) { threwShape = true; }
        EXPECT(threwShape);
        HIP(hipFree(dA));
        HIP(hipFree(dB));
        EXPECT(std::system(("rm -rf " + root).c_str()) == 0);
    }

    // --- the MoE block of a 5-row verify step three ways: the separate operators (router + routed experts, shared
    // expert, tail); the routed rows left un-combined for the tail; the shared expert inside the routed experts'
    // launches as well. Same routes; the same hidden rows bit for bit (first two) and to the shared row's rounding ---
    {
        const int R = 5;
        ffmoe_shape denseShape{(uint32_t)d, (uint32_t)f, 1, 1, 1, 16};
        Context dense(0, denseShape);
        const uint8_t *blob = pool.data() + 3 * stride;
        auto u16 = [&](uint32_t o) { return reinterpret_cast<const uint16_t *>(blob + o); };
        PrefillSharedExpert shared(dense);
        shared.load(0, SharedExpertProjection{blob + off.gate_w, u16(off.gate_s), u16(off.gate_b), (uint32_t)f, (uint32_t)d},
                    SharedExpertProjection{blob + off.up_w, u16(off.up_s), u16(off.up_b), (uint32_t)f, (uint32_t)d},
                    SharedExpertProjection{blob + off.down_w, u16(off.down_s), u16(off.down_b), (uint32_t)d, (uint32_t)f});
        std::vector<uint16_t> hid((size_t)R * d), w3(d), w4(d);
        for (auto &b : hid) b = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, -2.f, 2.f));
        for (auto &b : w3) b = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, 0.5f, 1.5f));
        for (auto &b : w4) b = ffo_bf16_bits(ffo_splitmix64_uniform(&rng, 0.5f, 1.5f));
        uint16_t *dHidA = toDevice(hid), *dHidB = toDevice(hid), *dHidC = toDevice(hid), *dW3 = toDevice(w3), *dW4 = toDevice(w4);
        uint16_t *dY = nullptr, *dH1 = nullptr, *dWA = nullptr, *dWB = nullptr, *dWC = nullptr;
        uint32_t *dIA = nullptr, *dIB = nullptr, *dIC = nullptr;
        for (auto p : {&dY, &dH1}) HIP(hipMalloc(reinterpret_cast<void **>(p), (size_t)R * d * 2));
        for (auto p : {&dWA, &dWB, &dWC}) HIP(hipMalloc(reinterpret_cast<void **>(p), (size_t)R * K * 2));
        for (auto p : {&dIA, &dIB, &dIC}) HIP(hipMalloc(reinterpret_cast<void **>(p), (size_t)R * K * 4));
        MoE block(ctx);
        PrefillLayerTail tail(ctx);
        FusedLayerTail fused(ctx);
        block.encodeRouterAndRoutedExperts(stream, 0, dx, d, dx, d, R, nullptr, dY, dIA, dWA);
        shared.encodeBlock(stream, 0, dx, dH1, R, d, f, d, d);
        tail.encode(stream, dY, dH1, dHidA, dW3, dW4, R, d, d, d, d, 1e-6f, 0.875f);
        block.encodeRouterAndRoutedExperts(stream, 0, dx, d, dx, d, R, nullptr, nullptr, dIB, dWB);
        fused.encodeRouted(stream, dWB, dH1, dHidB, dW3, dW4, R, 1e-6f, 0.875f);
        block.encodeRouterRoutedAndSharedExperts(stream, dense, 0, 0, dx, d, dx, d, dx, d, R, dIC, dWC);
        fused.encodeRoutedShared(stream, dense, dWC, dHidC, dW3, dW4, R, 1e-6f, 0.875f);
        HIP(hipStreamSynchronize(stream));
        EXPECT(toHost(dIA, (size_t)R * K) == toHost(dIB, (size_t)R * K) && toHost(dIA, (size_t)R * K) == toHost(dIC, (size_t)R * K));
        EXPECT(toHost(dWA, (size_t)R * K) == toHost(dWB, (size_t)R * K) && toHost(dWA, (size_t)R * K) == toHost(dWC, (size_t)R * K));
        const auto hA = toHost(dHidA, (size_t)R * d), hB = toHost(dHidB, (size_t)R * d), hC = toHost(dHidC, (size_t)R * d);
        EXPECT(hA == hB);
        std::vector<float> refA(hA.size());
        for (size_t i = 0; i < hA.size(); ++i) refA[i] = ffo_bf16_to_float(hA[i]);
        double relC, cosC;
        errorStats(hC, refA, relC, cosC);
        EXPECT(relC <= 1e-2 && cosC >= 0.9999);
        EXPECT(hA != hid);
        EXPECT(block.handoverGiveups(stream) == 0);
        for (auto p : {dHidA, dHidB, dHidC, dW3, dW4, dY, dH1, dWA, dWB, dWC}) HIP(hipFree(p));
        for (auto p : {dIA, dIB, dIC}) HIP(hipFree(p));
    }

    std::printf(failures ? "%d FAILURES\n" : "host gpu ok\n", failures);
    return failures ? 1 : 0;
}
