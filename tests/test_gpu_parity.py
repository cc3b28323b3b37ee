"""HIP kernels against the CPU oracle, through the C ABI (ctypes). Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import REAL, REAL_STRIDE, bf16_tensor, bits_of, cosine, make_layer, rel_err, to_ff_offsets

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch


@pytest.fixture(scope="module")
def ff():
    import fieldfare_moe
    fieldfare_moe.lib()       # raises when the HIP library is not built: no fallback
    return fieldfare_moe


@pytest.fixture(scope="module")
def small(oracle, ff, torch):
    d, f, e = 128, 64, 16
    rng, pool, router = make_layer(oracle, 11, d, f, e, align=1)
    ctx = ff.Context(d, f, e, 8, n_layers=2, max_tokens=64)
    ctx.upload_layer(1, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(1, router)
    yield dict(rng=rng, pool=pool, router=router, ctx=ctx, d=d, f=f, e=e)
    ctx.close()


@pytest.fixture(scope="module")
def real(oracle, ff, torch):
    rng, pool, router = make_layer(oracle, 0, REAL["d"], REAL["f"], REAL["n_experts"], stride=REAL_STRIDE)
    ctx = ff.Context(REAL["d"], REAL["f"], REAL["n_experts"], 8, n_layers=1, max_tokens=4096)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    yield dict(rng=rng, pool=pool, router=router, ctx=ctx, **REAL)
    ctx.close()


def test_library_reports_version(ff):
    assert b"gfx950" in ff.lib().ffmoe_version()


def test_missing_layer_is_an_error(small, ff, torch):
    ctx = small["ctx"]
    x = torch.zeros((1, small["d"]), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((1, 8), dtype=torch.int32, device="cuda")
    w = torch.zeros((1, 8), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ff.FieldfareError, match="layer 0 were not uploaded"):
        ctx.verify(0, x, idx, w)
    with pytest.raises(ff.FieldfareError, match="outside 1...16"):
        ctx.verify(1, torch.zeros((17, small["d"]), dtype=torch.bfloat16, device="cuda"),
                   torch.zeros((17, 8), dtype=torch.int32, device="cuda"),
                   torch.zeros((17, 8), dtype=torch.bfloat16, device="cuda"))


def test_dequant_bit_exact_adversarial(oracle, ff, torch):
    # every nibble value against the adversarial scale/bias set of MPPPrefillInt4QMMTests.swift:26-37
    d, f, e = 128, 64, 2
    L = oracle.lib()
    scales = [L.ffo_bf16_bits(0.001), L.ffo_bf16_bits(-0.0015), 0x0001, 0x8001]
    biases = [L.ffo_bf16_bits(-0.01), L.ffo_bf16_bits(0.006), 0x0001, 0x8001]
    parts = []
    for ex in range(e):
        triple = []
        for role, (rows, cols) in enumerate(((f, d), (f, d), (d, f))):
            n = rows * cols // 2
            W = ((np.arange(n) * 37 + 0x29 + 11 * role + 5 * ex) & 0xFF).astype(np.uint8).reshape(rows, cols // 2)
            S = np.array([[scales[(r + g) % 4] for g in range(cols // 64)] for r in range(rows)], np.uint16)
            B = np.array([[biases[(r * 3 + g) % 4] for g in range(cols // 64)] for r in range(rows)], np.uint16)
            triple.append((W, S, B))
        parts.append(tuple(triple))
    pool = oracle.pool_from_parts(parts, d, f, align=2)
    ctx = ff.Context(d, f, e, 2, n_layers=1, max_tokens=16)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    for ex in range(e):
        for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
            got = bits_of(ctx.dequant_expert(0, ex, which))
            want = oracle.dequantize_int4_bf16(*pool.sub(ex, name))
            assert np.array_equal(got, want), (ex, name)
    ctx.close()


def test_prefill_lds_tile_bit_exact_adversarial(oracle, ff, torch):
    # The tile the grouped GEMM's matrix instructions read from LDS (copied out by the kernel itself, fragment
    # by fragment, with the read indexing of the multiply loop) against bf16(fma(q, s, b)): every nibble value,
    # the adversarial scale/bias set incl. bf16 subnormals and negative scales (MPPPrefillInt4QMMTests.swift:26-37,
    # tile definition :190-192). Shapes: tiles that fill N-blocks exactly and ones that leave a ragged last block.
    L = oracle.lib()
    scales = [L.ffo_bf16_bits(0.001), L.ffo_bf16_bits(-0.0015), 0x0001, 0x8001, L.ffo_bf16_bits(0.0123)]
    biases = [L.ffo_bf16_bits(-0.01), L.ffo_bf16_bits(0.006), 0x0001, 0x8001, L.ffo_bf16_bits(-0.0984)]
    for d, f, e in ((128, 64, 2), (192, 320, 3)):
        parts = []
        for ex in range(e):
            triple = []
            for role, (rows, cols) in enumerate(((f, d), (f, d), (d, f))):
                n = rows * cols // 2
                W = ((np.arange(n) * 37 + 0x29 + 11 * role + 5 * ex) & 0xFF).astype(np.uint8).reshape(rows, cols // 2)
                S = np.array([[scales[(r + g + ex) % 5] for g in range(cols // 64)] for r in range(rows)], np.uint16)
                B = np.array([[biases[(r * 3 + g) % 5] for g in range(cols // 64)] for r in range(rows)], np.uint16)
                triple.append((W, S, B))
            parts.append(tuple(triple))
        pool = oracle.pool_from_parts(parts, d, f, align=2)
        ctx = ff.Context(d, f, e, 2, n_layers=1, max_tokens=16)
        ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
        for ex in range(e):
            for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
                got = bits_of(ctx.prefill_tiles(0, ex, which))
                want = oracle.dequantize_int4_bf16(*pool.sub(ex, name))
                assert got.shape == want.shape
                assert np.array_equal(got, want), (d, f, ex, name)
        ctx.close()


def test_prefill_lds_tile_bit_exact_real_shape(real, oracle, ff):
    for ex in (0, 127):
        for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
            got = bits_of(real["ctx"].prefill_tiles(0, ex, which))
            want = oracle.dequantize_int4_bf16(*real["pool"].sub(ex, name))
            assert np.array_equal(got, want), (ex, name)
            # and the standalone expansion kernel holds the same bits
            assert np.array_equal(got, bits_of(real["ctx"].dequant_expert(0, ex, which)))


def test_dequant_bit_exact_real_shape(real, oracle, ff):
    # device-resident source blobs take the same re-tiling path as host blobs; spot-check experts
    for ex in (0, 63, 127):
        for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
            got = bits_of(real["ctx"].dequant_expert(0, ex, which))
            want = oracle.dequantize_int4_bf16(*real["pool"].sub(ex, name))
            assert np.array_equal(got, want), (ex, name)


def test_upload_from_device_memory_matches_host_upload(small, oracle, ff, torch):
    pool = small["pool"]
    ctx = small["ctx"]
    dev = torch.from_numpy(pool.bytes).cuda()
    ctx.upload_layer(0, dev, pool.stride, to_ff_offsets(ff, pool.offsets))
    for ex in (0, 15):
        assert torch.equal(ctx.dequant_expert(0, ex, ff.DOWN), ctx.dequant_expert(1, ex, ff.DOWN))


def test_upload_rejects_out_of_range_offsets(small, ff):
    pool = small["pool"]
    bad = to_ff_offsets(ff, pool.offsets)
    bad.down_b = pool.stride - 8
    with pytest.raises(ff.FieldfareError, match="down_b"):
        small["ctx"].upload_layer(0, pool.bytes, pool.stride, bad)


@pytest.mark.parametrize("t", [1, 3, 16])
def test_router_logits_and_topk_bit_exact(real, oracle, torch, t):
    rng = np.random.default_rng(100 + t)
    xb = oracle.bf16_bits(rng.normal(0, 1, (t, real["d"])).astype(np.float32))
    idx, w, logits = real["ctx"].router(0, bf16_tensor(torch, xb), want_logits=True)
    logits = logits.cpu().numpy()
    min_gap = np.inf
    for tok in range(t):
        ref = oracle.router_logits_pinned(real["router"], xb[tok])
        assert np.array_equal(logits[tok].view(np.uint32), ref.view(np.uint32)), f"token {tok}: logits differ in bits"
        ridx, rw = oracle.topk_softmax(ref, 8)
        assert np.array_equal(idx[tok].cpu().numpy().astype(np.uint32), ridx)
        got_w = oracle.bf16_to_float(bits_of(w[tok]))
        # expf differs by ulps between libm and the GPU; the weights are rounded to bf16 (8 bits)
        assert np.abs(got_w - rw).max() <= np.abs(rw).max() * 2 ** -7
        s = np.sort(ref)[::-1]
        min_gap = min(min_gap, s[7] - s[8])
    print(f"T={t}: min 8th/9th logit gap {min_gap:.3e}")


def test_router_reference_int8_case(oracle, ff, torch):
    # RouterTopKTests.swift:17-44 restated: INT8-affine router, effective scale, per-expert scale.
    g = oracle.SplitMix64(0xA5B6_1234)
    weights = np.stack([g.uniform(-0.05, 0.05, 128) + np.float32(e) * np.float32(0.01) for e in range(16)])
    hidden = g.uniform(-1.0, 1.0, 128)
    es = g.uniform(0.5, 1.5, 128) * (np.float32(1.0) / np.sqrt(np.float32(128)))
    pes = g.uniform(0.6, 1.4, 16)
    P, S, B = oracle.quantize_int8(weights)
    ctx = ff.Context(128, 64, 16, 8, n_layers=1, max_tokens=16)
    esb, pesb = oracle.bf16_bits(es), oracle.bf16_bits(pes)
    ctx.upload_router_int8(0, P, S, B, esb, pesb)
    xb = oracle.bf16_bits(hidden)
    idx, w, logits = ctx.router(0, bf16_tensor(torch, xb[None, :]), want_logits=True)
    Wdeq = oracle.dequantize_int8(P, S, B)
    ref = oracle.router_logits_pinned(Wdeq, xb, oracle.BF16, esb)
    assert np.array_equal(logits[0].cpu().numpy().view(np.uint32), ref.view(np.uint32))
    ridx, rw = oracle.topk_softmax(ref, 8, pesb)
    assert np.array_equal(idx[0].cpu().numpy().astype(np.uint32), ridx)
    # the Swift test's own bar: indices equal to the fp32 full-sort reference, weights within 5e-3
    ref64 = Wdeq.astype(np.float64) @ (hidden.astype(np.float64) * es.astype(np.float64))
    order = sorted(range(16), key=lambda i: (-ref64[i], i))[:8]
    assert list(ridx) == order
    ex = np.exp(ref64[order] - ref64[order[0]])
    assert np.abs(oracle.bf16_to_float(bits_of(w[0])) - ex / ex.sum() * pes[order]).max() < 5e-3
    ctx.close()


def test_router_strided_rows_and_special_scores(small, oracle, torch):
    # stride = D + 13 with sentinels between rows (PrefillRouterTests.swift:24-87)
    d, e = small["d"], small["e"]
    rng = np.random.default_rng(5)
    stride = d + 13
    buf = np.full((3, stride), -31.0, np.float32)
    buf[:, :d] = rng.normal(0, 1, (3, d))
    xb = oracle.bf16_bits(buf)
    x = bf16_tensor(torch, xb)[:, :d]
    assert x.stride(0) == stride
    idx, w = small["ctx"].router(1, x)
    for tok in range(3):
        ridx, _ = oracle.topk_softmax(oracle.router_logits_pinned(small["router"], xb[tok, :d]), 8)
        assert np.array_equal(idx[tok].cpu().numpy().astype(np.uint32), ridx)


@pytest.mark.parametrize("t,d,e,pad,kind", [
    (37, 320, 13, 0, "bf16"),      # ragged token and expert tiles, d not a multiple of 256
    (64, 1344, 20, 13, "bf16"),    # stride d + 13: rows only 2-byte aligned
    (130, 1088, 128, 8, "int8"),   # fp32 router weights with effective and per-expert scales
    (17, 64, 1, 0, "bf16"),        # a single expert, top-1
])
def test_router_prefill_tiles_bit_exact(oracle, ff, torch, t, d, e, pad, kind):
    # more than 16 rows take the tiled logits kernel; every logit must still match the pinned order
    rng = np.random.default_rng(t * 1000 + d)
    k = min(8, e)
    ctx = ff.Context(d, 64, e, k, n_layers=1, max_tokens=t)
    W = rng.normal(0, 0.2, (e, d)).astype(np.float32)
    esb = pesb = None
    if kind == "int8":
        P, S, B = oracle.quantize_int8(W)
        esb = oracle.bf16_bits(rng.uniform(0.5, 1.5, d).astype(np.float32))
        pesb = oracle.bf16_bits(rng.uniform(0.6, 1.4, e).astype(np.float32))
        ctx.upload_router_int8(0, P, S, B, esb, pesb)
        Wref = oracle.dequantize_int8(P, S, B)
    else:
        Wref = oracle.bf16_bits(W)
        ctx.upload_router_bf16(0, Wref)
    buf = np.full((t, d + pad), 7.5, np.float32)
    buf[:, :d] = rng.normal(0, 1, (t, d))
    xb = oracle.bf16_bits(buf)
    x = bf16_tensor(torch, xb)[:, :d]
    idx, w, logits = ctx.router(0, x, want_logits=True)
    logits = logits.cpu().numpy()
    for tok in range(t):
        ref = oracle.router_logits_pinned(Wref, xb[tok, :d], oracle.BF16, esb)
        assert np.array_equal(logits[tok].view(np.uint32), ref.view(np.uint32)), f"token {tok}"
        ridx, rw = oracle.topk_softmax(ref, k, pesb)
        assert np.array_equal(idx[tok].cpu().numpy().astype(np.uint32), ridx)
        assert np.abs(oracle.bf16_to_float(bits_of(w[tok])) - rw).max() <= np.abs(rw).max() * 2 ** -7
    ctx.close()


def _run_verify_case(case, oracle, torch, t, seed, mode="fused"):
    d, e = case["d"], case["n_experts"] if "n_experts" in case else case["e"]
    rng = np.random.default_rng(seed)
    xb = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
    x = bf16_tensor(torch, xb)
    idx, w = case["ctx"].router(0 if "n_experts" in case else 1, x)
    layer = 0 if "n_experts" in case else 1
    idx_np = idx.cpu().numpy().astype(np.uint32)
    w_f = oracle.bf16_to_float(bits_of(w))
    ref = oracle.moe_experts(case["pool"], xb, idx_np, w_f)
    if mode == "fused":
        y = case["ctx"].verify(layer, x, idx, w)
        got = oracle.bf16_to_float(bits_of(y))
    else:
        partials = case["ctx"].verify_partials(layer, x, idx, w)
        got = oracle.bf16_to_float(bits_of(case["ctx"].reduce_token_major(partials, w)))
    return got, ref, case["ctx"].last_live_experts(), len(np.unique(idx_np))


@pytest.mark.parametrize("t", [1, 2, 5, 16])
def test_verify_small_shape(small, oracle, torch, t):
    got, ref, live, distinct = _run_verify_case(small, oracle, torch, t, 40 + t)
    assert live == distinct
    assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999


@pytest.mark.parametrize("d,f,t", [(3072, 64, 1), (3072, 64, 6), (128, 2880, 6), (128, 2880, 1)])
def test_verify_shapes_beyond_the_register_ring(oracle, ff, torch, d, f, t):
    # hidden > 2816: gate/up takes the one-shot grid behind the plan kernel; intermediate > 704: the down
    # projection splits K over the waves of a block (<= 2816) - routed experts, not only the dense form
    e, k = 8, 4
    rng, pool, router = make_layer(oracle, 1000 + d + t, d, f, e, align=1)
    ctx = ff.Context(d, f, e, k, n_layers=1, max_tokens=16)
    try:
        ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
        ctx.upload_router_bf16(0, router)
        xb = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
        x = bf16_tensor(torch, xb)
        idx, w = ctx.router(0, x)
        idx_np = idx.cpu().numpy().astype(np.uint32)
        for tok in range(t):
            ridx, _ = oracle.topk_softmax(oracle.router_logits_pinned(router, xb[tok]), k)
            assert np.array_equal(idx_np[tok], ridx)
        ref = oracle.moe_experts(pool, xb, idx_np, oracle.bf16_to_float(bits_of(w)))
        got = oracle.bf16_to_float(bits_of(ctx.verify(0, x, idx, w)))
        assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999
        assert ctx.last_live_experts() == len(np.unique(idx_np))
        partials = ctx.verify_partials(0, x, idx, w)
        got = oracle.bf16_to_float(bits_of(ctx.reduce_token_major(partials, w)))
        assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999
    finally:
        ctx.close()


@pytest.mark.parametrize("t,mode", [(1, "fused"), (16, "fused"), (16, "partials"), (7, "fused")])
def test_verify_real_shape(real, oracle, torch, t, mode):
    # layer outputs: max rel err <= 1e-2 and cosine >= 0.9999 against the fp32 reference composition
    got, ref, live, distinct = _run_verify_case(real, oracle, torch, t, 70 + t, mode)
    assert live == distinct
    r, c = rel_err(got, ref), cosine(got, ref)
    print(f"T={t} {mode}: live experts {live}, rel err {r:.2e}, cosine {c:.6f}")
    assert r <= 1e-2 and c >= 0.9999


def test_verify_matches_mirror_rounding_tightly(small, oracle, torch):
    # mirror mode: activation rounded to bf16, fp32 partials, rank-ordered fma, one final rounding
    t = 4
    rng = np.random.default_rng(9)
    xb = oracle.bf16_bits(rng.normal(0, 1, (t, small["d"])).astype(np.float32))
    x = bf16_tensor(torch, xb)
    idx, w = small["ctx"].router(1, x)
    pairs = oracle.make_token_expert_pairs(idx.cpu().numpy(), bits_of(w), t, 8)
    partial = oracle.route_partials(small["pool"], pairs, xb, small["d"], t, 8, oracle.F32)
    # route_partials in F32 mode keeps the activation unrounded; allow for that single rounding
    want = oracle.bf16_to_float(oracle.reduce_token_major(partial, oracle.F32, bits_of(w), oracle.BF16))
    got = oracle.bf16_to_float(bits_of(small["ctx"].verify(1, x, idx, w)))
    assert rel_err(got, want) <= 2 ** -6


def test_verify_residual_zero_weights_and_bad_indices(small, oracle, torch):
    d = small["d"]
    rng = np.random.default_rng(21)
    t = 3
    xb = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
    x = bf16_tensor(torch, xb)
    idx, w = small["ctx"].router(1, x)
    idx_np = idx.cpu().numpy().astype(np.uint32).copy()
    w_bits = bits_of(w).copy()
    # zero weights are skipped (RealForwardRunner.swift:1528-1530), also when the index is garbage
    w_bits[0, 7] = 0
    w_bits[1, 3] = 0x8000          # negative zero
    idx_np[1, 3] = 9999
    idx_np[2, 5] = 4_000_000_000   # out of range with a non-zero weight: ignored, contributes nothing
    w_f = oracle.bf16_to_float(w_bits)
    idx_ref = idx_np.copy()
    w_ref = w_f.copy()
    w_ref[2, 5] = 0
    idx_ref[1, 3] = 0
    idx_ref[2, 5] = 0
    resid = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
    ref = oracle.moe_experts(small["pool"], xb, idx_ref, w_ref) + oracle.bf16_to_float(resid)
    y = small["ctx"].verify(1, x, torch.from_numpy(idx_np.view(np.int32)).cuda(), bf16_tensor(torch, w_bits),
                            residual=bf16_tensor(torch, resid))
    got = oracle.bf16_to_float(bits_of(y))
    assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999


def test_streamed_routed_reference_case(oracle, ff, torch):
    # MoEFusedFFNTests.swift:17-146 restated with bf16 activations: D=128, F=64, K=8, residual, fixed routing weights
    g = oracle.seed_tree_key(0x2D3, "production-routed-moe")
    gates, ups, downs = [], [], []
    for _ in range(8):
        gates.append(g.uniform(-0.4, 0.4, 64 * 128).reshape(64, 128))
        ups.append(g.uniform(-0.4, 0.4, 64 * 128).reshape(64, 128))
        downs.append(g.uniform(-0.4, 0.4, 128 * 64).reshape(128, 64))
    xb = oracle.bf16_bits(g.uniform(-0.5, 0.5, 128))
    rb = oracle.bf16_bits(g.uniform(-0.5, 0.5, 128))
    wb = oracle.bf16_bits(np.float32(0.04) + np.arange(8, dtype=np.float32) * np.float32(0.015))
    pool = oracle.pool_from_float(gates, ups, downs)
    ctx = ff.Context(128, 64, 8, 8, n_layers=1, max_tokens=16)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    expected = oracle.apply_streamed_routed(pool, list(range(8)), oracle.bf16_to_float(xb), oracle.bf16_to_float(rb),
                                            oracle.bf16_to_float(wb))
    idx = torch.arange(8, dtype=torch.int32, device="cuda")[None, :].contiguous()
    y = ctx.verify(0, bf16_tensor(torch, xb[None, :]), idx, bf16_tensor(torch, wb[None, :]),
                   residual=bf16_tensor(torch, rb[None, :]))
    got = oracle.bf16_to_float(bits_of(y))[0]
    assert rel_err(got, expected) < 1e-2          # Tolerance.fp16ChainedReduction
    # fewer routed experts (top_k = 5 of the reference test): slots past 5 carry weight zero and add nothing
    wb5 = wb.copy()
    wb5[5:] = 0
    exp5 = oracle.apply_streamed_routed(pool, list(range(5)), oracle.bf16_to_float(xb), oracle.bf16_to_float(rb),
                                        oracle.bf16_to_float(wb[:5]))
    y5 = ctx.verify(0, bf16_tensor(torch, xb[None, :]), idx, bf16_tensor(torch, wb5[None, :]),
                    residual=bf16_tensor(torch, rb[None, :]))
    assert rel_err(oracle.bf16_to_float(bits_of(y5))[0], exp5) < 1e-2
    ctx.close()


def test_reduce_token_major_bit_exact(small, oracle, torch):
    g = oracle.SplitMix64(0x4D0E_2026)      # PrefillMoETests.swift:10-20
    rows, k, d = 3, 8, 64
    pb = oracle.bf16_bits(g.uniform(-2.0, 2.0, rows * k * d)).reshape(rows, k, d)
    wb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * k)).reshape(rows, k)
    want = oracle.reduce_token_major(pb, oracle.BF16, wb, oracle.BF16)
    got = bits_of(small["ctx"].reduce_token_major(bf16_tensor(torch, pb), bf16_tensor(torch, wb)))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,rows,off", [(300, 2112, 3, 0), (301, 2816, 4, 2), (264, 8192, 7, 0), (256, 2112, 12, 0),
                                          (384, 2816, 13, 0), (1408, 2816, 1, 0), (64, 128, 1, 0)])
def test_gemv_int4_reference_shapes(small, oracle, torch, m, n, rows, off):
    # DequantInt4SmallBatchTests.swift:66-119 shapes (incl. the 2-byte weight offset), config 1, and
    # StreamingKernelIntegrationTests.swift:84-161 (64 x 128)
    g = oracle.seed_tree_key(0xD8 + rows, f"int4-small-batch-m{m}-n{n}-r{rows}-off{off}")
    W, S, B = oracle.quantize_int4(g.uniform(-0.5, 0.5, m * n).reshape(m, n))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * n)).reshape(rows, n)
    raw = np.concatenate([np.zeros(off, np.uint8), W.ravel()])
    Wd = torch.from_numpy(raw).cuda()
    Sd = torch.from_numpy(S.view(np.int16)).cuda()
    Bd = torch.from_numpy(B.view(np.int16)).cuda()
    x = bf16_tensor(torch, xb)
    y = small["ctx"].gemv_int4(Wd, Sd, Bd, x, w_byte_offset=off)
    got = oracle.bf16_to_float(bits_of(y))
    for r in range(rows):
        ref = oracle.gemv_int4_ref(W, S, B, oracle.bf16_to_float(xb[r]))
        assert rel_err(got[r], ref) < 1e-2, f"row {r}"       # bf16 output: 8-bit significand
    y32 = small["ctx"].gemv_int4(Wd, Sd, Bd, x, f32_out=True, w_byte_offset=off).cpu().numpy()
    for r in range(rows):
        ref = oracle.gemv_int4_ref(W, S, B, oracle.bf16_to_float(xb[r]))
        assert rel_err(y32[r], ref) < 5e-3                   # Tolerance.fp16Reduction on the unrounded sum
    # row r of a multi-row call is the single-row GEMV bit for bit (matchesSingleRowGEMVBitwise)
    for r in range(rows):
        single = small["ctx"].gemv_int4(Wd, Sd, Bd, x[r:r + 1], f32_out=True, w_byte_offset=off).cpu().numpy()[0]
        assert np.array_equal(single.view(np.uint32), y32[r].view(np.uint32)), f"row {r} differs from the GEMV"


@pytest.mark.parametrize("which,t", [("small", 1), ("small", 3), ("small", 8), ("small", 9), ("real", 1), ("real", 4),
                                     ("real", 8), ("real", 16)])
def test_route_verify_equals_router_then_verify(small, real, oracle, torch, which, t):
    # one call against the two calls: routes,
    # weights and outputs bit for bit; the routes are the oracle's
    fx = small if which == "small" else real
    ctx, d, layer = fx["ctx"], fx["d"], 1 if which == "small" else 0
    g = oracle.seed_tree_key(0x207E, f"route-verify-{which}-{t}")
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    rb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    res = oracle.bf16_bits(g.uniform(-0.5, 0.5, t * d)).reshape(t, d)
    x, router_x, residual = bf16_tensor(torch, xb), bf16_tensor(torch, rb), bf16_tensor(torch, res)
    idx2, w2 = ctx.router(layer, router_x)
    y2 = ctx.verify(layer, x, idx2, w2, residual=residual)
    y1, idx1, w1 = ctx.route_verify(layer, router_x, x, residual=residual)
    assert np.array_equal(idx1.cpu().numpy(), idx2.cpu().numpy())
    assert np.array_equal(bits_of(w1), bits_of(w2))
    assert np.array_equal(bits_of(y1), bits_of(y2))
    got = idx1.cpu().numpy().astype(np.uint32)
    for r in range(t):
        ref_idx, _ = oracle.topk_softmax(oracle.router_logits_pinned(fx["router"], rb[r]), 8)
        assert np.array_equal(got[r], ref_idx), f"row {r}"


@pytest.mark.parametrize("t", [1, 5, 16])
def test_route_verify_is_correct_when_no_hand_over_arrives(real, oracle, torch, t):
    """The waves of route_verify's one-launch form wait for each other's words with a bounded poll. With the bound
    set to zero from the host every wave that does not find its words at once stops waiting and computes them itself
    (the row's logits for a selecting block, logits + select + weights of its rows for every other wave): the launch
    ends normally, such waves are counted, and routes, weights and rows equal router + verify bit for bit - the
    routes being the oracle's."""
    ctx, d = real["ctx"], real["d"]
    g = oracle.seed_tree_key(0x207E, f"route-verify-timeout-{t}")
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    rb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    x, router_x = bf16_tensor(torch, xb), bf16_tensor(torch, rb)
    idx2, w2 = ctx.router(0, router_x)
    y2 = ctx.verify(0, x, idx2, w2)
    try:
        ctx.set_handover_timeout(0)
        y1, idx1, w1 = ctx.route_verify(0, router_x, x)
        torch.cuda.synchronize()            # the launch ended
        assert ctx.handover_giveups() > 0
    finally:
        ctx.set_handover_timeout(100_000)
    assert ctx.handover_giveups() == 0
    assert np.array_equal(idx1.cpu().numpy(), idx2.cpu().numpy())
    assert np.array_equal(bits_of(w1), bits_of(w2))
    assert np.array_equal(bits_of(y1), bits_of(y2))
    got = idx1.cpu().numpy().astype(np.uint32)
    for r in range(t):
        ref_idx, _ = oracle.topk_softmax(oracle.router_logits_pinned(real["router"], rb[r]), 8)
        assert np.array_equal(got[r], ref_idx), f"row {r}"
    assert ctx.last_live_experts() == len(np.unique(got))
    # with the bound back, nobody gives up and the bits are the same again
    y3, idx3, w3 = ctx.route_verify(0, router_x, x)
    assert np.array_equal(bits_of(y3), bits_of(y2)) and np.array_equal(idx3.cpu().numpy(), idx2.cpu().numpy())
    assert ctx.handover_giveups() == 0


@pytest.mark.parametrize("t", [1, 16])
def test_route_verify_with_the_router_as_its_own_launches(real, oracle, torch, t):
    """set_one_launch_routing(False): the same call runs the router in front of the expert pass (the timer's router
    slots fill, the one-launch slot stays empty) and gives the bits of the one-launch form."""
    ctx, d = real["ctx"], real["d"]
    g = oracle.seed_tree_key(0x207E, f"route-verify-split-{t}")
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    x = bf16_tensor(torch, xb)
    y1, idx1, w1 = ctx.route_verify(0, x, x)
    try:
        ctx.set_one_launch_routing(False)
        ctx.set_profiling(True)
        ctx.profile(reset=True)
        y2, idx2, w2 = ctx.route_verify(0, x, x)
        prof = ctx.profile(reset=True)
    finally:
        ctx.set_profiling(False)
        ctx.set_one_launch_routing(True)
    assert prof["router_logits"][1] == 1 and prof["router_topk"][1] == 1 and prof["gate_up"][1] == 1
    assert prof.get("route_gate_up", (0.0, 0))[1] == 0
    assert np.array_equal(idx1.cpu().numpy(), idx2.cpu().numpy())
    assert np.array_equal(bits_of(w1), bits_of(w2))
    assert np.array_equal(bits_of(y1), bits_of(y2))
    ctx.set_profiling(True)
    ctx.profile(reset=True)
    ctx.route_verify(0, x, x)
    prof = ctx.profile(reset=True)
    ctx.set_profiling(False)
    assert prof["route_gate_up"][1] == 1 and prof.get("router_logits", (0.0, 0))[1] == 0


@pytest.mark.parametrize("which", ["small", "real"])
def test_decode_sized_blocks_equal_rows_of_a_larger_block(small, real, oracle, torch, which):
    # rows are independent of the block they arrive in: a block of two rows and a block of one row give the
    # bits of the same rows inside a three-row block, with and without a residual, with a skipped route
    fx = small if which == "small" else real
    ctx, d, layer = fx["ctx"], fx["d"], 1 if which == "small" else 0
    g = oracle.seed_tree_key(0xDEC0, f"decode-rows-{which}")
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, 3 * d)).reshape(3, d)
    res = oracle.bf16_bits(g.uniform(-0.5, 0.5, 3 * d)).reshape(3, d)
    x, residual = bf16_tensor(torch, xb), bf16_tensor(torch, res)
    idx, w = ctx.router(layer, x)
    w[1, 3] = 0.0                       # a skipped route inside the small blocks
    for resid in (None, residual):
        y3 = bits_of(ctx.verify(layer, x, idx, w, residual=resid))
        y2 = bits_of(ctx.verify(layer, x[:2], idx[:2], w[:2], residual=None if resid is None else resid[:2]))
        y1 = bits_of(ctx.verify(layer, x[2:3], idx[2:3], w[2:3], residual=None if resid is None else resid[2:3]))
        assert np.array_equal(y2, y3[:2])
        assert np.array_equal(y1[0], y3[2])
    # and the oracle on the small block
    w_np = oracle.bf16_to_float(bits_of(w[:2]))
    ref = oracle.moe_experts(fx["pool"], xb[:2], idx[:2].cpu().numpy().astype(np.uint32), w_np)
    got = oracle.bf16_to_float(bits_of(ctx.verify(layer, x[:2], idx[:2], w[:2])))
    assert rel_err(got, ref) < 1e-2 and cosine(got, ref) > 0.9999


def test_gemv_int4_listed_rows(small, oracle, torch):
    # encodeRowsListed (DequantInt4GEMV.swift:124-145): output o is weight row ids[o]; the hot-vocabulary
    # projection of LMHeadChainInt4.swift:171-177. Same arithmetic per row as the full GEMV: equal bits.
    ctx = small["ctx"]
    m, n, rows = 1031, 1408, 5
    g = oracle.seed_tree_key(0x11D5, "listed-gemv")
    W, S, B = oracle.quantize_int4(g.uniform(-0.5, 0.5, m * n).reshape(m, n))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * n)).reshape(rows, n)
    ids = np.array([7, 0, 1030, 512, 7, 64, 65, 1, 999], np.int32)          # unordered, with a repeat
    tW, tS, tB = torch.from_numpy(W).cuda(), torch.from_numpy(S.view(np.int16)).cuda(), torch.from_numpy(B.view(np.int16)).cuda()
    x = bf16_tensor(torch, xb)
    full = ctx.gemv_int4(tW, tS, tB, x, f32_out=True).cpu().numpy()
    listed = ctx.gemv_int4_listed(tW, tS, tB, torch.from_numpy(ids).cuda(), x).cpu().numpy()
    assert listed.shape == (rows, ids.size)
    assert np.array_equal(listed.view(np.uint32), full[:, ids].view(np.uint32))
    for r in range(rows):
        ref = oracle.gemv_int4_ref(W[ids], S[ids], B[ids], oracle.bf16_to_float(xb[r]))
        assert rel_err(listed[r], ref) < 5e-3


def test_expert_named_more_than_16_times_keeps_its_first_16_routes(small, oracle, torch):
    # The router never names an expert twice in a row, but ffmoe_verify takes any table: an expert's route list holds
    # 16 entries, further routes to it (in [row][rank] order) take no part - they add nothing, instead of whatever the
    # scratch rows held.
    ctx, d, t = small["ctx"], small["d"], 16
    rng = np.random.default_rng(991)
    xb = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
    x = bf16_tensor(torch, xb)
    idx_np = np.stack([rng.permutation(np.arange(1, small["e"]))[:8] for _ in range(t)]).astype(np.uint32)
    idx_np[idx_np == 5] = 6
    idx_np[:, 0] = 5
    idx_np[:, 3] = 5                      # expert 5: 32 routes, the first 16 are rows 0..7
    w_np = rng.random((t, 8)).astype(np.float32)
    w_np /= w_np.sum(1, keepdims=True)
    wb = oracle.bf16_bits(w_np)
    kept = oracle.bf16_to_float(wb).copy()
    kept[8:, 0] = 0.0
    kept[8:, 3] = 0.0
    idx = torch.from_numpy(idx_np.astype(np.int32)).cuda()
    w = bf16_tensor(torch, wb)
    # poison the scratch rows first: a block whose every route is live fills them all
    ctx.verify(1, x, *ctx.router(1, x))
    got = oracle.bf16_to_float(bits_of(ctx.verify(1, x, idx, w)))
    ref = oracle.moe_experts(small["pool"], xb, idx_np, kept)
    assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999, (rel_err(got, ref), cosine(got, ref))


@pytest.mark.parametrize("which,t,stride_pad", [("small", 1, 0), ("small", 7, 5), ("real", 1, 0), ("real", 16, 0), ("real", 16, 13)])
def test_layer_tail_routed_equals_route_verify_then_layer_tail(small, real, oracle, torch, which, t, stride_pad):
    """The routed experts' weighted combine folded into the layer tail (ffmoe_route_verify without y, then
    ffmoe_layer_tail_routed) against the separate calls: the new hidden rows bit for bit, padding untouched; and the
    separate calls' hidden rows are the oracle's layer tail on the combined rows."""
    fx = small if which == "small" else real
    ctx, d, layer = fx["ctx"], fx["d"], 1 if which == "small" else 0
    g = oracle.seed_tree_key(0x7A11, f"tail-routed-{which}-{t}-{stride_pad}")
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    x = bf16_tensor(torch, xb)
    h1 = np.full((t, d + stride_pad), oracle.bf16_bits(np.float32(-23.0)), np.uint16)
    hid = np.full((t, d + stride_pad), oracle.bf16_bits(np.float32(-25.0)), np.uint16)
    h1[:, :d] = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    hid[:, :d] = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    w2 = oracle.bf16_bits(g.uniform(0.5, 1.5, d))
    w1 = oracle.bf16_bits(g.uniform(0.5, 1.5, d))
    tw2, tw1 = bf16_tensor(torch, w2), bf16_tensor(torch, w1)
    th1 = bf16_tensor(torch, h1)
    # separate calls
    y, idx_a, w_a = ctx.route_verify(layer, x, x)
    hid_a = bf16_tensor(torch, hid)
    ctx.layer_tail(y, th1, hid_a, tw2, tw1, 0.875, 1e-6, d=d)
    want = hid.copy()
    want[:, :d] = oracle.layer_tail(bits_of(y), h1[:, :d], hid[:, :d], w2, w1, 0.875, 1e-6)
    assert np.array_equal(bits_of(hid_a), want)
    # the fused pair
    none, idx_b, w_b = ctx.route_verify(layer, x, x, combine=False)
    assert none is None
    hid_b = bf16_tensor(torch, hid)
    ctx.layer_tail_routed(w_b, th1, hid_b, tw2, tw1, 0.875, 1e-6)
    assert np.array_equal(idx_a.cpu().numpy(), idx_b.cpu().numpy()) and np.array_equal(bits_of(w_a), bits_of(w_b))
    assert np.array_equal(bits_of(hid_b), bits_of(hid_a))
    assert np.array_equal(bits_of(th1), h1)
    # the next call on the context is an ordinary one again (the epoch moved on with the un-combined call)
    y2, idx_c, _ = ctx.route_verify(layer, x, x)
    assert np.array_equal(bits_of(y2), bits_of(y)) and np.array_equal(idx_c.cpu().numpy(), idx_a.cpu().numpy())
    assert ctx.handover_giveups() == 0
