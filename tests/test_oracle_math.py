"""Pins the oracle's GEMV, activation, router select, FFN, combine and host grouping logic against
library routines in fp64, brute force, invariants and the reference tests' exact expected arrays."""
import numpy as np
import pytest
import torch


def _rel(actual, ref):
    # RelError.compute, Tests/Support/Validation/Tolerance/RelError.swift:7-16
    return float(np.abs(actual - ref).max() / max(np.abs(ref).max(), 1e-6))


def _deq64(oracle, W, S, B):
    q = np.stack([W & 15, W >> 4], -1).reshape(W.shape[0], -1).astype(np.float64)
    s = np.repeat(oracle.bf16_to_float(S).astype(np.float64), 64, axis=1)
    b = np.repeat(oracle.bf16_to_float(B).astype(np.float64), 64, axis=1)
    return q * s + b


def test_gemv_special_inputs_and_fp64(oracle):
    # shapes of DequantInt4SmallBatchTests.swift:66-73, same seed derivation
    m, n = 300, 2112
    rng = oracle.seed_tree_key(0xD8, f"int4-small-batch-m{m}-n{n}-r3-off0")
    rows = rng.uniform(-0.5, 0.5, m * n).reshape(m, n)
    W, S, B = oracle.quantize_int4(rows)
    deq = oracle.dequantize_int4(W, S, B)
    # quantisation error bound: half a step of the bf16-rounded scale (plus its rounding)
    step = np.repeat(oracle.bf16_to_float(S), 64, axis=1)
    assert np.all(np.abs(deq - rows) <= 0.5 * step * 1.02 + 1e-6)
    # one-hot x picks a single dequantised weight exactly (pins row/column indexing)
    for k in (0, 1, 63, 64, 65, 1055, n - 1):
        x = np.zeros(n, np.float32)
        x[k] = 1.0
        assert np.array_equal(oracle.gemv_int4_ref(W, S, B, x), deq[:, k])
    # general x against a float64 BLAS product
    x = rng.uniform(-1.0, 1.0, n)
    y = oracle.gemv_int4_ref(W, S, B, x)
    y64 = _deq64(oracle, W, S, B) @ x.astype(np.float64)
    assert _rel(y, y64.astype(np.float32)) < 1e-5
    # linearity in x
    x2 = rng.uniform(-1.0, 1.0, n)
    y2 = oracle.gemv_int4_ref(W, S, B, x2)
    y12 = oracle.gemv_int4_ref(W, S, B, (x + x2).astype(np.float32))
    assert _rel(y12, y + y2) < 1e-5


def test_int4_dot_matches_gemv_and_factored_form(oracle):
    rng = np.random.default_rng(5)
    pool = oracle.random_pool(rng, 2, 128, 64)
    x = rng.normal(0, 1, 128).astype(np.float32)
    for which, rows in (("gate", 64), ("up", 64)):
        W, S, B = pool.sub(1, which)
        y = oracle.gemv_int4_ref(W, S, B, x)
        got = np.array([oracle.int4_dot(pool, 1, which, r, x) for r in range(rows)], np.float32)
        assert np.array_equal(got, y)     # same arithmetic: (q*s+b)*x summed left to right
        # factored form s*sum(q x) + b*sum(x) (moe.metal:323-378) agrees within fp32 noise
        q = np.stack([W & 15, W >> 4], -1).reshape(rows, -1).astype(np.float64)
        s = oracle.bf16_to_float(S).astype(np.float64)
        b = oracle.bf16_to_float(B).astype(np.float64)
        xs = x.astype(np.float64).reshape(-1, 64)
        fact = (s * (q.reshape(rows, -1, 64) * xs).sum(-1) + b * xs.sum(-1)).sum(-1)
        assert _rel(got, fact.astype(np.float32)) < 1e-5
    xd = rng.normal(0, 1, 64).astype(np.float32)
    W, S, B = pool.sub(0, "down")
    got = np.array([oracle.int4_dot(pool, 0, "down", r, xd) for r in range(128)], np.float32)
    assert np.array_equal(got, oracle.gemv_int4_ref(W, S, B, xd))


def test_gelu_tanh_vs_torch(oracle):
    x = np.concatenate([np.linspace(-12, 12, 4001), [0.0, -0.0, 1e-8, -30.0, 30.0]]).astype(np.float32)
    ref = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    got = oracle.gelu_tanh(x)
    assert np.abs(got - ref).max() < 2e-6
    assert oracle.gelu_tanh([0.0])[0] == 0.0
    assert oracle.gelu_tanh([30.0])[0] == 30.0 and oracle.gelu_tanh([-30.0])[0] == 0.0


def test_topk_against_full_sort(oracle):
    rng = np.random.default_rng(7)
    for _ in range(200):
        e = int(rng.choice([8, 16, 100, 128, 256]))
        logits = rng.normal(0, 1, e).astype(np.float32)
        if rng.random() < 0.5:                      # force exact ties
            logits[rng.integers(0, e, 6)] = logits[rng.integers(0, e)]
        idx, w = oracle.topk_softmax(logits, 8)
        # RouterTopKTests.swift:55-63: sort by (score desc, index asc), take 8
        order = sorted(range(e), key=lambda i: (-float(logits[i]), i))[:8]
        assert list(idx) == order
        s = logits[order].astype(np.float64)
        ref = np.exp(s - s[0]) / np.exp(s - s[0]).sum()
        assert np.abs(w - ref).max() < 1e-6
        assert abs(w.sum() - 1.0) < 1e-6 and np.all(np.diff(w) <= 0)


def test_topk_special_cases(oracle):
    # all-equal scores -> indices 0..7, equal weights
    idx, w = oracle.topk_softmax(np.zeros(128, np.float32), 8)
    assert list(idx) == list(range(8)) and np.allclose(w, 0.125)
    # fewer than 8 candidates: -inf and NaN are never taken; missing slots = (index 0, weight 0)
    logits = np.full(128, -np.inf, np.float32)
    logits[[5, 77, 9]] = [1.0, 3.0, 1.0]
    logits[3] = np.nan
    idx, w = oracle.topk_softmax(logits, 8)
    assert list(idx) == [77, 5, 9, 0, 0, 0, 0, 0]
    assert np.all(w[3:] == 0) and abs(w[:3].sum() - 1) < 1e-6
    # per-expert scale multiplies the softmax weight of the chosen expert (moe.metal:235)
    pes = oracle.bf16_bits(np.linspace(0.6, 1.4, 128).astype(np.float32))
    logits = np.arange(128, dtype=np.float32) * 0.1
    idx, w = oracle.topk_softmax(logits, 8, pes)
    idx0, w0 = oracle.topk_softmax(logits, 8)
    assert list(idx) == list(range(127, 119, -1))
    assert np.allclose(w, w0 * oracle.bf16_to_float(pes)[idx], rtol=1e-6)
    # generic top_k (prefill kernel, prefill.metal:499-541)
    idx3, w3 = oracle.topk_softmax(logits, 3)
    assert list(idx3) == [127, 126, 125] and abs(w3.sum() - 1) < 1e-6


def test_router_reference_test_restated(oracle):
    # RouterTopKTests.swift:17-44: 16 experts x 128, INT8-affine weights, ordering by full sort
    g = oracle.SplitMix64(0xA5B6_1234)
    weights = np.stack([g.uniform(-0.05, 0.05, 128) + np.float32(e) * np.float32(0.01) for e in range(16)])
    hidden = g.uniform(-1.0, 1.0, 128)
    inv = np.float32(1.0) / np.sqrt(np.float32(128))
    es = g.uniform(0.5, 1.5, 128) * inv
    pes = g.uniform(0.6, 1.4, 16)
    P, S, B = oracle.quantize_int8(weights)
    Wdeq = oracle.dequantize_int8(P, S, B)
    # the kernel sees fp16 hidden and bf16 effective scale / per-expert scale
    xb = oracle.bits16(hidden, oracle.FP16)
    esb, pesb = oracle.bf16_bits(es), oracle.bf16_bits(pes)
    logits = oracle.router_logits_pinned(Wdeq, xb, oracle.FP16, esb)
    ref = Wdeq.astype(np.float64) @ (oracle.from_bits16(xb, oracle.FP16).astype(np.float64) * oracle.bf16_to_float(esb))
    assert np.abs(logits - ref).max() < 1e-5
    idx, w = oracle.topk_softmax(logits, 8, pesb)
    # the Swift reference: fp32 inputs (no 16-bit rounding), sort, softmax, times expertScale
    ref32 = Wdeq.astype(np.float64) @ (hidden.astype(np.float64) * es.astype(np.float64))
    order = sorted(range(16), key=lambda i: (-ref32[i], i))[:8]
    assert list(idx) == order
    ex = np.exp(ref32[order] - ref32[order[0]])
    assert np.abs(w - ex / ex.sum() * pes[order]).max() < 5e-3


def test_router_pinned_order_definition(oracle):
    # the pinned order equals an explicit numpy evaluation of the same tree, and a fp64 dot within noise
    rng = np.random.default_rng(11)
    e, d = 128, 2816
    Wb = oracle.bf16_bits(rng.normal(0, 0.02, (e, d)).astype(np.float32))
    xb = oracle.bf16_bits(rng.normal(0, 1, d).astype(np.float32))
    got = oracle.router_logits_pinned(Wb, xb)
    W = oracle.bf16_to_float(Wb).astype(np.float64)
    x = oracle.bf16_to_float(xb).astype(np.float64)
    assert np.abs(got - W @ x).max() < 2e-5
    # sub-accumulator s of lane l: fp32 chain over k = 1024 i + 256 s + 4 l + j. bf16*bf16 products are
    # exact in fp32, so fma == mul+add here.
    Wf, xf = oracle.bf16_to_float(Wb), oracle.bf16_to_float(xb)
    sub = np.zeros((4, e, 64), np.float32)
    for i in range((d + 1023) // 1024):
        for s in range(4):
            for j in range(4):
                ks = 1024 * i + 256 * s + 4 * np.arange(64) + j
                ok = ks < d
                term = np.zeros((e, 64), np.float32)
                term[:, ok] = Wf[:, ks[ok]] * xf[ks[ok]]
                sub[s] = np.where(ok[None, :], (term + sub[s]).astype(np.float32), sub[s])
    p = ((sub[0] + sub[1]).astype(np.float32) + (sub[2] + sub[3]).astype(np.float32)).astype(np.float32)
    for m in (32, 16, 8, 4, 2, 1):
        p = (p + p[:, np.arange(64) ^ m]).astype(np.float32)
    assert np.array_equal(got, p[:, 0])


def test_ffn_and_layer_vs_torch_fp64(oracle):
    rng = np.random.default_rng(3)
    d, f, e, t = 128, 64, 16, 5
    pool = oracle.random_pool(rng, e, d, f)
    router = oracle.bf16_bits(rng.normal(0, 0.02, (e, d)).astype(np.float32))
    xb = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
    idx, w, y = oracle.moe_layer(pool, router, xb, 8)
    x64 = torch.from_numpy(oracle.bf16_to_float(xb).astype(np.float64))
    R = torch.from_numpy(oracle.bf16_to_float(router).astype(np.float64))
    logits = x64 @ R.T
    top = torch.topk(logits, 8, dim=1)
    assert np.array_equal(idx, top.indices.numpy().astype(np.uint32))
    wref = torch.softmax(top.values, dim=1).numpy()
    assert np.abs(w - wref).max() < 2 ** -8          # weights are rounded to bf16
    yref = np.zeros((t, d))
    for tok in range(t):
        for r in range(8):
            ex = int(idx[tok, r])
            G = torch.from_numpy(_deq64(oracle, *pool.sub(ex, "gate")))
            U = torch.from_numpy(_deq64(oracle, *pool.sub(ex, "up")))
            D = torch.from_numpy(_deq64(oracle, *pool.sub(ex, "down")))
            act = torch.nn.functional.gelu(G @ x64[tok], approximate="tanh") * (U @ x64[tok])
            yref[tok] += float(w[tok, r]) * (D @ act).numpy()
    assert _rel(y, yref.astype(np.float32)) < 1e-4
    # run_ffn alone and moe_experts agree with the layer composition
    y2 = oracle.moe_experts(pool, xb, idx, w)
    assert np.array_equal(y, y2)


def test_streamed_routed_reference_test_restated(oracle):
    # MoEFusedFFNTests.swift:17-46: D=128, F=64, K=8, SeedTree(0x2D3).key("production-routed-moe")
    g = oracle.seed_tree_key(0x2D3, "production-routed-moe")
    gates, ups, downs = [], [], []
    for _ in range(8):
        gates.append(g.uniform(-0.4, 0.4, 64 * 128).reshape(64, 128))
        ups.append(g.uniform(-0.4, 0.4, 64 * 128).reshape(64, 128))
        downs.append(g.uniform(-0.4, 0.4, 128 * 64).reshape(128, 64))
    x = g.uniform(-0.5, 0.5, 128).astype(np.float16).astype(np.float32)
    residual = g.uniform(-0.5, 0.5, 128).astype(np.float16).astype(np.float32)
    rw = (np.float32(0.04) + np.arange(8, dtype=np.float32) * np.float32(0.015)).astype(np.float16).astype(np.float32)
    pool = oracle.pool_from_float(gates, ups, downs)
    # blob layout of makeBlob (MoEFusedFFNTests.swift:221-257): nine tightly packed sub-tensors
    assert pool.offsets.as_tuple() == (0, 4096, 4352, 4608, 8704, 8960, 9216, 13312, 13568) and pool.stride == 13824
    y = oracle.apply_streamed_routed(pool, list(range(8)), x, residual, rw)
    ref = residual.astype(np.float64).copy()
    for k in range(8):
        G, U, D = (_deq64(oracle, *pool.sub(k, n)) for n in ("gate", "up", "down"))
        act = torch.nn.functional.gelu(torch.from_numpy(G @ x.astype(np.float64)), approximate="tanh").numpy() * (U @ x.astype(np.float64))
        ref += float(rw[k]) * (D @ act)
    assert _rel(y, ref.astype(np.float32)) < 1e-5
    # top_k = 5 ignores the other slots (MoEFusedFFNTests.swift:150-219)
    y5 = oracle.apply_streamed_routed(pool, list(range(5)), x, residual, rw[:5])
    ref5 = residual.astype(np.float64).copy()
    for k in range(5):
        ref5 += float(rw[k]) * oracle.run_ffn(pool, k, x).astype(np.float64)
    assert _rel(y5, ref5.astype(np.float32)) < 1e-6


def test_reduce_token_major(oracle):
    # PrefillMoETests.swift:10-20,46-64
    g = oracle.SplitMix64(0x4D0E_2026)
    rows, k, d = 3, 8, 64
    partials = g.uniform(-2.0, 2.0, rows * k * d).astype(np.float16)
    weights = g.uniform(-1.0, 1.0, rows * k).astype(np.float16)
    h2 = oracle.reduce_token_major(partials.view(np.uint16).reshape(rows, k, d), oracle.FP16,
                                   weights.view(np.uint16), oracle.FP16)
    ref = (weights.astype(np.float64).reshape(rows, k, 1) * partials.astype(np.float64).reshape(rows, k, d)).sum(1)
    assert np.abs(h2.view(np.float16).astype(np.float64) - ref).max() <= 2e-3
    # one-hot weights reproduce the selected partial bit for bit
    onehot = np.zeros((rows, k), np.float16)
    onehot[:, 5] = 1
    h = oracle.reduce_token_major(partials.view(np.uint16).reshape(rows, k, d), oracle.FP16, onehot.view(np.uint16), oracle.FP16)
    assert np.array_equal(h, partials.view(np.uint16).reshape(rows, k, d)[:, 5, :])
    # bf16 data, fp32 partials
    pf = g.uniform(-2.0, 2.0, rows * k * d).reshape(rows, k, d)
    wb = oracle.bf16_bits(g.uniform(0.0, 1.0, rows * k))
    hb = oracle.reduce_token_major(pf, oracle.F32, wb, oracle.BF16)
    refb = (oracle.bf16_to_float(wb).astype(np.float64).reshape(rows, k, 1) * pf).sum(1)
    assert np.abs(oracle.bf16_to_float(hb) - refb).max() <= np.abs(refb).max() * 2 ** -8


def test_pairs_are_token_major(oracle):
    # PrefillRouterTests.swift:12-22
    w = np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6], np.float16)
    pairs = oracle.make_token_expert_pairs([3, 1, 2, 4, 0, 5], w.view(np.uint16), 2, 3)
    assert list(pairs["token"]) == [0, 0, 0, 1, 1, 1]
    assert list(pairs["rank"]) == [0, 1, 2, 0, 1, 2]
    assert list(pairs["expert"]) == [3, 1, 2, 4, 0, 5]
    assert np.array_equal(pairs["weight_bits"].astype(np.uint16).view(np.float16), w)


def _pair(token, expert, rank, bits):
    return (token, expert, rank, bits)


def test_grouping_exact_arrays(oracle):
    # PrefillMoEGroupingTests.swift:5-50
    raw = [_pair(0, 3, 0, 10), _pair(0, 1, 1, 11), _pair(0, 4, 2, 12), _pair(1, 1, 0, 13), _pair(1, 3, 1, 14),
           _pair(1, 2, 2, 15), _pair(2, 4, 0, 16), _pair(2, 3, 1, 17), _pair(2, 1, 2, 18), _pair(3, 5, 0, 19),
           _pair(3, 1, 1, 20), _pair(3, 4, 2, 21)][::-1]
    pairs = np.array(raw, oracle.PAIR_DTYPE)
    sp, groups, tiles = oracle.group_token_expert_pairs(pairs, 6, 2)
    assert list(sp["expert"]) == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert [[int(p["token"]), int(p["rank"])] for p in sp] == [[0, 1], [1, 0], [2, 2], [3, 1], [1, 2], [0, 0], [1, 1],
                                                               [2, 1], [0, 2], [2, 0], [3, 2], [3, 0]]
    assert list(sp["weight_bits"]) == [11, 13, 18, 20, 15, 10, 14, 17, 12, 16, 21, 19]
    assert groups == [(1, 0, 4), (2, 4, 1), (3, 5, 3), (4, 8, 3), (5, 11, 1)]
    assert tiles == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]


def test_grouping_sort_keys_and_errors(oracle):
    # PrefillMoEGroupingTests.swift:52-96
    raw = [_pair(0, 1, 0, 10), _pair(0, 2, 1, 20), _pair(1, 3, 0, 30), _pair(1, 1, 1, 11), _pair(2, 2, 0, 21),
           _pair(2, 3, 1, 31)]
    sp, groups, tiles = oracle.group_token_expert_pairs(np.array(raw, oracle.PAIR_DTYPE), 4, 2, [0, 30, 10, 20])
    assert [g[0] for g in groups] == [2, 3, 1]
    assert list(sp["expert"]) == [2, 2, 3, 3, 1, 1]
    assert tiles == [(0, 2, 0, 4), (2, 1, 4, 2)]
    with pytest.raises(ValueError, match="route expert 2 is out of range"):
        oracle.group_token_expert_pairs(np.array([_pair(0, 2, 0, 1)], oracle.PAIR_DTYPE), 2, 1)
    # PrefillGroupedRoutedMoETests+Binding.swift:21-40: tiles never exceed 16 experts
    raw = [_pair(i // 8, min(i, 19), i % 8, 0) for i in range(24)]
    sp, groups, tiles = oracle.group_token_expert_pairs(np.array(raw, oracle.PAIR_DTYPE), 128, 16)
    assert [g[0] for g in groups[tiles[0][0]:tiles[0][0] + tiles[0][1]]] == list(range(16))
    assert [g[0] for g in groups[tiles[1][0]:tiles[1][0] + tiles[1][1]]] == list(range(16, 20))


def test_route_partials_reference_test_restated(oracle):
    # PrefillGroupedRoutedMoETests+Execution.swift:9-97 with syntheticRows (…Tests.swift:100-109)
    d = f = 64
    rows, top_k = 3, 2

    def synthetic(nrows, ncols, expert, role):
        r = np.arange(nrows, dtype=np.float32)[:, None]
        c = np.arange(ncols, dtype=np.float32)[None, :]
        return (np.float32(expert + 1) * np.float32(0.001) + np.float32(role + 1) * np.float32(0.003)
                + ((r % 7) - 3) * np.float32(0.0004) + ((c % 11) - 5) * np.float32(0.0002)).astype(np.float32)

    pool = oracle.pool_from_float([synthetic(f, d, e, 0) for e in range(16)], [synthetic(f, d, e, 1) for e in range(16)],
                                  [synthetic(d, f, e, 2) for e in range(16)])
    raw = [(0, 2, 0), (0, 0, 1), (1, 1, 0), (1, 2, 1), (2, 0, 0), (2, 1, 1)]
    pairs = np.array([(t, e, r, 0) for t, e, r in raw], oracle.PAIR_DTYPE)
    sp, groups, tiles = oracle.group_token_expert_pairs(pairs, 16, 16)
    hidden = (((np.arange(rows * d) % 17) - 8).astype(np.float32) * np.float32(0.01)).astype(np.float16)
    out = oracle.route_partials(pool, sp, hidden.view(np.uint16), d, rows, top_k, oracle.FP16, fill=-99.0)
    x64 = hidden.astype(np.float64).reshape(rows, d)
    for t, e, r in raw:
        G, U, D = (_deq64(oracle, *pool.sub(e, n)) for n in ("gate", "up", "down"))
        act = torch.nn.functional.gelu(torch.from_numpy(G @ x64[t]), approximate="tanh").numpy() * (U @ x64[t])
        ref = D @ act
        got = out[t, r].view(np.float16).astype(np.float64)
        assert np.abs(got - ref).max() <= 0.0015


def _rms_norm_ref64(x, w, eps):
    """RmsNormRef.apply (Tests/Support/Validation/Reference/Primitives/RmsNorm.swift:9-41) in float64."""
    x = np.asarray(x, np.float64)
    return x * np.asarray(w, np.float64) / np.sqrt((x * x).mean() + eps)


def test_layer_tail_against_cpu_reference_restated(oracle):
    # fusedLayerTailNorms_matchSeparateDispatchesAndReference (FusedLayerTailTests.swift:15-61): same seed and
    # draw order (h2, h1, hidden, four weight vectors, the scalar); cpuReference (:96-110) restated in float64
    # with its roundings; the reference's bound on FP16 data is 4e-3 relative, bf16 carries 2^-9 per rounding
    d, eps = 2816, 1e-6
    for dtype, bound in ((oracle.FP16, 4e-3), (oracle.BF16, 2e-2)):
        rng = oracle.SplitMix64(0x7A11_0001)
        h2 = oracle.bits16(rng.uniform(-1, 1, d), dtype)
        h1 = oracle.bits16(rng.uniform(-3, 3, d), dtype)
        hidden = oracle.bits16(rng.uniform(-2, 2, d), dtype)
        weights = [oracle.bf16_bits(rng.uniform(0.5, 1.5, d)) for _ in range(4)]
        scalar = float(rng.uniform(0.75, 1.25, 1)[0])
        r16 = lambda v: oracle.from_bits16(oracle.bits16(np.asarray(v, np.float32), dtype), dtype).astype(np.float64)
        w2, w1 = oracle.bf16_to_float(weights[1]), oracle.bf16_to_float(weights[2])
        h2n = r16(_rms_norm_ref64(oracle.from_bits16(h2, dtype), w2, eps))
        h12 = r16(oracle.from_bits16(h1, dtype).astype(np.float64) + h2n)
        h12n = r16(_rms_norm_ref64(h12, w1, eps))
        ref = r16(r16(oracle.from_bits16(hidden, dtype).astype(np.float64) + h12n) * r16(scalar))
        got = oracle.from_bits16(oracle.layer_tail(h2, h1, hidden, weights[1], weights[2], scalar, eps, dtype)[0], dtype)
        assert np.abs(got - ref).max() / np.abs(ref).max() < bound
        # almost every element agrees to the bit; the rest are one rounding step apart
        assert (got == ref).mean() > 0.95


def test_rmsnorm_against_float64_and_tail_with_norms_chain(oracle):
    # the plain norm against RmsNormRef in float64 (every element within one rounding step), the closed form
    # for a constant row, and the reference test's full chain (cpuReference, FusedLayerTailTests.swift:96-110,
    # with the post-FFN-1 norm in front and the next layer's norm behind) restated in float64
    d, eps = 2816, 1e-6
    for dtype, ulp in ((oracle.FP16, 2.0 ** -10), (oracle.BF16, 2.0 ** -7)):
        rng = oracle.SplitMix64(0x7A11_0001)
        h2 = oracle.bits16(rng.uniform(-1, 1, d), dtype)
        h1 = oracle.bits16(rng.uniform(-3, 3, d), dtype)
        hidden = oracle.bits16(rng.uniform(-2, 2, d), dtype)
        weights = [oracle.bf16_bits(rng.uniform(0.5, 1.5, d)) for _ in range(4)]
        scalar = float(rng.uniform(0.75, 1.25, 1)[0])
        f = lambda bits: oracle.from_bits16(bits, dtype).astype(np.float64)
        wf = [oracle.bf16_to_float(w).astype(np.float64) for w in weights]
        got = f(oracle.rmsnorm(h1, weights[0], eps, dtype)[0])
        ref = _rms_norm_ref64(f(h1), wf[0], eps)
        assert np.all(np.abs(got - ref) <= np.abs(ref) * ulp)
        r16 = lambda v: f(oracle.bits16(np.asarray(v, np.float32), dtype))
        h1n = r16(ref)
        h2n = r16(_rms_norm_ref64(f(h2), wf[1], eps))
        h12n = r16(_rms_norm_ref64(r16(h1n + h2n), wf[2], eps))
        new_hidden = r16(r16(f(hidden) + h12n) * r16(scalar))
        normed = r16(_rms_norm_ref64(new_hidden, wf[3], eps))
        o_hidden = oracle.layer_tail(h2, oracle.rmsnorm(h1, weights[0], eps, dtype), hidden, weights[1], weights[2], scalar, eps, dtype)
        o_normed = f(oracle.rmsnorm(o_hidden, weights[3], eps, dtype)[0])
        bound = 4e-3 if dtype == oracle.FP16 else 2e-2
        assert np.abs(f(o_hidden[0]) - new_hidden).max() / np.abs(new_hidden).max() < bound
        assert np.abs(o_normed - normed).max() / np.abs(normed).max() < bound
    # a constant row c with unit weight normalises to sign(c) (eps = 0), whatever c
    for c in (0.37, -5.0, 1024.0):
        row = oracle.bf16_bits(np.full(256, c, np.float32))
        out = oracle.bf16_to_float(oracle.rmsnorm(row, oracle.bf16_bits(np.ones(256, np.float32)), 0.0)[0])
        assert np.array_equal(out, np.full(256, np.sign(c), np.float32))
    # scaling the row by a power of two leaves the result unchanged (eps = 0); the weight scales it linearly
    g = np.random.default_rng(5)
    row = oracle.bf16_bits(g.uniform(-1, 1, 512).astype(np.float32))
    w = oracle.bf16_bits(g.uniform(0.5, 1.5, 512).astype(np.float32))
    base = oracle.rmsnorm(row, w, 0.0)
    row4 = oracle.bf16_bits(oracle.bf16_to_float(row) * 4.0)
    assert np.array_equal(oracle.rmsnorm(row4, w, 0.0), base)
    w2 = oracle.bf16_bits(oracle.bf16_to_float(w) * 2.0)
    assert np.array_equal(oracle.bf16_to_float(oracle.rmsnorm(row, w2, 0.0)), oracle.bf16_to_float(base) * 2.0)


def test_post_attn_setup_against_primitive_chain(oracle):
    # fusedPostAttentionSetup_matchesPrimitiveChainBitwise_realShape (FusedPostAttentionSetupTests.swift:11-100):
    # the chain norm(attn) -> hidden += -> three norms of hidden, the router's with a unit weight; same seed
    d, eps = 2816, 1e-6
    rng = oracle.SplitMix64(0x9057_A77E)
    hidden = oracle.bf16_bits(rng.uniform(-1, 1, d))
    attn = oracle.bf16_bits(rng.uniform(-1, 1, d))
    w_post, w_pre, w_pre2 = (oracle.bf16_bits(rng.uniform(0.5, 1.5, d)) for _ in range(3))
    new_hidden, dense, routed, router = oracle.post_attn_setup(hidden, attn, w_post, w_pre, w_pre2, eps)
    r16 = lambda v: oracle.bf16_to_float(oracle.bf16_bits(np.asarray(v, np.float32))).astype(np.float64)
    an = r16(_rms_norm_ref64(oracle.bf16_to_float(attn), oracle.bf16_to_float(w_post), eps))
    h = r16(oracle.bf16_to_float(hidden).astype(np.float64) + an)
    close = lambda got, ref: (np.abs(oracle.bf16_to_float(got[0]) - ref).max() / np.abs(ref).max() < 1e-2
                              and (oracle.bf16_to_float(got[0]) == ref).mean() > 0.95)
    assert close(new_hidden, h)
    hf = oracle.bf16_to_float(new_hidden[0])
    assert close(dense, r16(_rms_norm_ref64(hf, oracle.bf16_to_float(w_pre), eps)))
    assert close(routed, r16(_rms_norm_ref64(hf, oracle.bf16_to_float(w_pre2), eps)))
    assert close(router, r16(_rms_norm_ref64(hf, np.ones(d), eps)))
    # what the arithmetic fixes: router_x has unit RMS; unit weights make the three outputs the same bits;
    # zero attention leaves hidden alone; scaling hidden and attn by 2 leaves the normalised outputs alone
    assert abs(np.sqrt((oracle.bf16_to_float(router[0]).astype(np.float64) ** 2).mean()) - 1.0) < 2e-3
    ones = oracle.bf16_bits(np.ones(d, np.float32))
    _, a, b, c = oracle.post_attn_setup(hidden, attn, w_post, ones, ones, eps)
    assert np.array_equal(a, b) and np.array_equal(b, c)
    h0, *_ = oracle.post_attn_setup(hidden, np.zeros(d, np.uint16), w_post, w_pre, w_pre2, eps)
    assert np.array_equal(h0[0], hidden)
    two = lambda bits: oracle.bf16_bits(2.0 * oracle.bf16_to_float(bits))
    _, d2, r2, q2 = oracle.post_attn_setup(two(new_hidden[0]), np.zeros(d, np.uint16), w_post, w_pre, w_pre2, 0.0)
    _, d1, r1, q1 = oracle.post_attn_setup(new_hidden[0], np.zeros(d, np.uint16), w_post, w_pre, w_pre2, 0.0)
    assert np.array_equal(d1, d2) and np.array_equal(r1, r2) and np.array_equal(q1, q2)


def test_layer_tail_invariants(oracle):
    d, eps = 512, 1e-6
    rng = oracle.SplitMix64(0x7A11_B10C)
    h2, h1, hidden = (oracle.bf16_bits(rng.uniform(-1, 1, d)) for _ in range(3))
    w2, w1 = (oracle.bf16_bits(rng.uniform(0.5, 1.5, d)) for _ in range(2))
    base = oracle.layer_tail(h2, h1, hidden, w2, w1, 1.0, eps)
    # a power-of-two scalar only shifts exponents; a scalar is rounded to 16 bits before use
    assert np.array_equal(oracle.bf16_to_float(oracle.layer_tail(h2, h1, hidden, w2, w1, 2.0, eps)), 2.0 * oracle.bf16_to_float(base))
    assert np.array_equal(oracle.layer_tail(h2, h1, hidden, w2, w1, 1.0 + 2.0 ** -10, eps), base)
    # rows are independent: a block equals its rows one at a time (PrefillLayerTailTests.swift:11-118)
    blk = oracle.layer_tail(np.stack([h2, h1]), np.stack([h1, h2]), np.stack([hidden, hidden]), w2, w1, 0.9, eps)
    assert np.array_equal(blk[0], oracle.layer_tail(h2, h1, hidden, w2, w1, 0.9, eps)[0])
    assert np.array_equal(blk[1], oracle.layer_tail(h1, h2, hidden, w2, w1, 0.9, eps)[0])


def test_greedy_choice_rows_against_closed_forms(oracle):
    # the choice: first maximum among the finite values; the confidence: scipy's softmax of the (capped) finite values
    from scipy.special import softmax
    rng = np.random.default_rng(31)
    rows = rng.normal(0, 4, (6, 513)).astype(np.float32)
    rows[1, 17] = rows[1, 311] = rows[1].max() + 1.0           # a tie: the lower position wins (LMHeadChainInt4Tests.swift:100-116)
    rows[2, :5] = [np.inf, -np.inf, np.nan, 1e30, -1e30]        # non-finite values never win and carry no probability
    rows[3, :] = np.nan                                        # no candidate at all
    rows[4, :] = -7.25                                         # all equal: position 0, probability 1 / V
    for cap in (0.0, 30.0, 2.0):
        tok, conf = oracle.greedy_choice_rows(rows, cap)
        for r in range(6):
            finite = np.isfinite(rows[r])
            if not finite.any():
                assert tok[r] == 0xFFFFFFFF and conf[r] == 0.0
                continue
            want = int(np.argmax(np.where(finite, rows[r], -np.inf)))      # numpy's argmax returns the first maximum
            assert tok[r] == want
            v = rows[r][finite].astype(np.float64)
            p = softmax(cap * np.tanh(v / cap) if cap > 0 else v)
            assert abs(conf[r] - p[np.flatnonzero(finite).tolist().index(want)]) <= 1e-12
        assert tok[1] == 17 and tok[4] == 0 and abs(conf[4] - 1 / 513) < 1e-12
    # a cap far below the spread flattens the distribution: the winner's probability falls towards 1 / V
    _, c0 = oracle.greedy_choice_rows(rows[:1], 0.0)
    _, c2 = oracle.greedy_choice_rows(rows[:1], 0.5)
    assert c2[0] < c0[0]


def test_sample_gumbel_is_one_splitmix64_step(oracle):
    """The noise hash is SplitMix64 (pinned to its published vectors in test_oracle_codecs.py) stepped once from the
    state seed ^ key * 0x9E3779B97F4A7C15 ^ token * 0xD1B54A32D192ED03; its top 24 bits make the uniform."""
    mask = (1 << 64) - 1
    for seed, key, tok in ((0, 0, 0), (0x1234_5678_9ABC_DEF0, 7, 262143), (mask, 0xFFFFFFFF, 0xFFFFFFFF), (42, 1000, 17)):
        state = (seed ^ ((key * 0x9E3779B97F4A7C15) & mask) ^ ((tok * 0xD1B54A32D192ED03) & mask)) & mask
        z = oracle.SplitMix64(state).next()
        u = (np.float64(z >> 40) + 0.5) / 16777216.0
        want = -np.log(-np.log(u))
        got = float(oracle.sample_gumbel(seed, key, [tok])[0])
        assert 0.0 < u < 1.0 and abs(got - want) <= 4e-6 * max(1.0, abs(want)), (seed, key, tok, got, want)


def test_sample_rows_draws_from_the_truncated_tempered_softmax(oracle):
    """The draw's law, by counting: over 30,000 positions the frequencies of the drawn entries match the softmax of
    capped(logit) / T over the survivors (chi-square well inside its 99.9 % bound), and nothing outside the
    survivors is ever drawn. Survivors by brute force: sort by (value descending, index ascending), first top_k, then
    the shortest prefix whose T = 1 mass over ALL entries reaches top_p."""
    logits = np.array([2.0, -1.0, 0.5, 2.0, 1.5, -3.0, 0.0, 1.9], np.float32)
    cap = 30.0
    capped = cap * np.tanh(logits.astype(np.float64) / cap)
    n = 30000
    rows = np.tile(logits, (n, 1))
    for temperature, top_k, top_p in ((1.0, 0, 1.0), (0.7, 0, 1.0), (1.3, 5, 1.0), (0.9, 6, 0.8)):
        tokens, prob, _ = oracle.sample_rows(rows, temperature, top_p, top_k, key_base=1000, softcap=cap, seed=0xC0FFEE)
        order = sorted(range(len(logits)), key=lambda i: (-capped[i], i))
        if 0 < top_k < len(logits):
            p1 = np.exp(capped) / np.exp(capped).sum()
            kept, cum = [], 0.0
            for i in order[:top_k]:
                kept.append(i)
                cum += p1[i]
                if cum >= top_p:
                    break
        else:
            kept = order
        law = np.zeros(len(logits))
        law[kept] = np.exp(capped[kept] / temperature)
        law /= law.sum()
        seen = np.bincount(tokens, minlength=len(logits)).astype(np.float64)
        assert seen[law == 0].sum() == 0
        chi2 = (((seen - n * law) ** 2)[law > 0] / (n * law[law > 0])).sum()
        assert chi2 < 30.0, (temperature, top_k, top_p, chi2)        # 99.9 % point of chi-square with 7 degrees: 24.3
        # the reported probability is the law's value at the drawn entry
        assert np.allclose(prob, law[tokens], rtol=1e-5)


def test_sample_rows_special_cases(oracle):
    rng = np.random.default_rng(8)
    rows = rng.normal(0, 3, (5, 300)).astype(np.float32)
    rows[1, 40] = rows[1, 200] = rows[1].max() + 2.0
    rows[2, :4] = [np.inf, np.nan, -np.inf, 1e30]
    rows[3, :] = -np.inf
    greedy, _ = oracle.greedy_choice_rows(rows, 25.0)
    # top_k = 1 keeps the largest capped logit alone (ties: the lower position); a vanishing temperature does the same
    # (an exact tie survives a vanishing temperature: the noise, not the position, breaks it)
    for kwargs in (dict(temperature=1.0, top_k=1, top_p=1.0), dict(temperature=1e-4, top_k=0, top_p=1.0)):
        tokens, prob, _ = oracle.sample_rows(rows, key_base=3, softcap=25.0, seed=99, **kwargs)
        untied = [0, 2, 3, 4]
        assert np.array_equal(tokens[untied], greedy[untied]), kwargs
        assert tokens[1] == 40 if kwargs["top_k"] == 1 else tokens[1] in (40, 200)
        assert prob[3] == 0.0 and np.all(prob[[0, 1, 2, 4]] > 0.0)
    # the noise follows the token id, not the position: a permuted table with ids draws the same TOKEN
    perm = rng.permutation(300).astype(np.uint32)
    base, _, _ = oracle.sample_rows(rows[:1], 0.8, 1.0, 0, key_base=11, softcap=25.0, seed=5)
    listed, _, _ = oracle.sample_rows(rows[:1, perm], 0.8, 1.0, 0, key_base=11, softcap=25.0, seed=5, ids=perm)
    assert perm[listed[0]] == base[0]
    # and the key is the row's position: row r with base b draws what row 0 draws with base b + r
    two, _, _ = oracle.sample_rows(np.stack([rows[0], rows[0]]), 0.8, 1.0, 0, key_base=20, softcap=25.0, seed=5)
    one, _, _ = oracle.sample_rows(rows[:1], 0.8, 1.0, 0, key_base=21, softcap=25.0, seed=5)
    off, _, _ = oracle.sample_rows(rows[:1], 0.8, 1.0, 0, key_base=20, softcap=25.0, seed=5, key_offset=1)
    assert two[1] == one[0] == off[0]
