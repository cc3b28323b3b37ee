"""BASELINE.json config 5 under test: 30 resident layers at the model's shape (12.85 GB of INT4 experts, arena offsets
beyond 4 GiB), a 16-token verify block drawn as the benchmark draws it, an 8,192-token prefill chunk with Zipf(1.1)
routing, and the 262,144 x 2816 LM head with its greedy choice - each held against the CPU oracle on the deep layers.
Shapes follow Runtime/Inference/RealForwardRunner.swift:454-756 (30-layer verify loop) and
Kernels/Fusions/LMHeadChainInt4.swift:94-139,225-284 (head)."""
import numpy as np
import pytest

from helpers import bits_of, cosine, rel_err

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]

LAYERS = 30
DEEP = (11, 29)         # layer 11 starts 4.71 GB into the arena (past 4 GiB = 4.29 GB), layer 29 is the last
PREFILL_TOKENS = 8192


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch


@pytest.fixture(scope="module")
def ff():
    import fieldfare_moe
    fieldfare_moe.lib()
    return fieldfare_moe


@pytest.fixture(scope="module")
def model(oracle, ff, torch):
    """30 layers built on the GPU the way bench.py builds them; the deep layers' blobs are kept on the host for the oracle."""
    from fieldfare_moe import synthetic as syn
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    rng = np.random.default_rng(0)
    offsets, payload = syn.layout_offsets(syn.D, syn.F, align=16)
    o_offsets, o_payload = oracle.layout_offsets(syn.D, syn.F, align=16)
    assert payload == o_payload == syn.EXPERT_BYTES and o_offsets.as_tuple() == tuple(getattr(offsets, n) for n, _ in offsets._fields_)
    ctx = ff.Context(syn.D, syn.F, syn.E, syn.K, n_layers=LAYERS, max_tokens=PREFILL_TOKENS)
    assert ctx.layer_arena_bytes * DEEP[0] > 1 << 32, "the first deep layer must sit past 4 GiB of the arena"
    pools, routers = {}, []
    for layer in range(LAYERS):
        blob = syn.synth_layer_gpu(torch, gen, offsets)
        ctx.upload_layer(layer, blob.view(-1), syn.STRIDE, offsets)
        if layer in DEEP:
            pools[layer] = oracle.ExpertPool(blob.view(-1).cpu().numpy(), o_offsets, syn.STRIDE, syn.D, syn.F)
        del blob
        routers.append(syn.router_weights(rng))
        ctx.upload_router_bf16(layer, routers[-1])
    torch.cuda.empty_cache()
    yield dict(ctx=ctx, pools=pools, routers=routers, syn=syn, gen=gen)
    ctx.close()


@pytest.mark.parametrize("layer", DEEP)
def test_verify_block_on_deep_layers(model, oracle, torch, layer):
    syn, ctx = model["syn"], model["ctx"]
    rng = np.random.default_rng(1000 + layer)
    xb = syn.bf16_bits(syn.block_tokens(rng, 16))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    idx, w = ctx.router(layer, x)
    y = ctx.verify(layer, x, idx, w)
    idx_np = idx.cpu().numpy().astype(np.uint32)
    # the routes are the oracle's, bit for bit, and the block is config 3's: 40-60 distinct experts with overlap
    for tok in range(16):
        ridx, _ = oracle.topk_softmax(oracle.router_logits_pinned(model["routers"][layer], xb[tok]), 8)
        assert np.array_equal(idx_np[tok], ridx), (layer, tok)
    distinct = len(np.unique(idx_np))
    assert 40 <= distinct <= 60, distinct
    assert ctx.last_live_experts() == distinct
    per_expert = np.bincount(idx_np.ravel(), minlength=syn.E)
    assert per_expert.max() >= 4, "a block whose tokens share experts has some expert with several routes"
    ref = oracle.moe_experts(model["pools"][layer], xb, idx_np, oracle.bf16_to_float(bits_of(w)))
    got = oracle.bf16_to_float(bits_of(y))
    assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999, (layer, rel_err(got, ref), cosine(got, ref))
    # the call the benchmark times - router, select and gate/up in one launch - on the same block: routes, weights and
    # rows equal the two calls' bit for bit (so they are the oracle's routes and rows as well), and no wave of the
    # one-launch form had to help itself
    y1, idx1, w1 = ctx.route_verify(layer, x, x)
    assert np.array_equal(idx1.cpu().numpy(), idx.cpu().numpy())
    assert np.array_equal(bits_of(w1), bits_of(w))
    assert np.array_equal(bits_of(y1), bits_of(y))
    assert ctx.last_live_experts() == distinct and ctx.handover_giveups() == 0
    # a decode step (one row) of the same block through the same call
    y_one, idx_one, w_one = ctx.route_verify(layer, x[:1], x[:1])
    assert np.array_equal(idx_one.cpu().numpy(), idx.cpu().numpy()[:1]) and np.array_equal(bits_of(w_one), bits_of(w)[:1])
    ref_one = oracle.moe_experts(model["pools"][layer], xb[:1], idx_np[:1], oracle.bf16_to_float(bits_of(w))[:1])
    got_one = oracle.bf16_to_float(bits_of(y_one))
    assert rel_err(got_one, ref_one) <= 1e-2 and cosine(got_one, ref_one) >= 0.9999


@pytest.mark.parametrize("layer", DEEP)
def test_prefill_8192_zipf_on_deep_layers(model, oracle, ff, torch, layer):
    syn, ctx = model["syn"], model["ctx"]
    rng = np.random.default_rng(2000 + layer)
    idx_np, w_np = syn.zipf_routes(rng, PREFILL_TOKENS)
    wb = syn.bf16_bits(w_np)
    xb = syn.bf16_bits(rng.normal(0, 1, (PREFILL_TOKENS, syn.D)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    idx = torch.from_numpy(idx_np).cuda()
    w = torch.from_numpy(wb.view(np.int16)).cuda().view(torch.bfloat16)
    y = ctx.prefill(layer, x, idx, w)
    n_pairs, n_tiles, counts = ctx.prefill_stats()
    want_counts = np.bincount(idx_np.ravel(), minlength=syn.E)
    assert n_pairs == PREFILL_TOKENS * syn.K and np.array_equal(counts, want_counts)
    assert n_tiles == int(np.sum((want_counts + ff.PREFILL_TILE_M - 1) // ff.PREFILL_TILE_M))
    assert want_counts.max() > 10 * max(1, want_counts.min()), "Zipf routing: a few experts hold most pairs"
    # oracle on a sample of 32 tokens, among them the first and last rows of the chunk and tokens of the heaviest expert
    heavy = np.flatnonzero((idx_np == int(np.argmax(want_counts))).any(1))
    sample = np.unique(np.concatenate([[0, PREFILL_TOKENS - 1], heavy[:6], rng.choice(PREFILL_TOKENS, 24, replace=False)]))
    assert len(sample) >= 24
    ref = oracle.moe_experts(model["pools"][layer], xb[sample], idx_np[sample].astype(np.uint32), oracle.bf16_to_float(wb[sample]))
    got = oracle.bf16_to_float(bits_of(y[torch.from_numpy(sample).cuda()]))
    assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999, (layer, rel_err(got, ref), cosine(got, ref))


def test_dequant_last_expert_of_last_layer(model, oracle, ff):
    ctx, pool = model["ctx"], model["pools"][29]
    for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
        want = oracle.dequantize_int4_bf16(*pool.sub(127, name))
        assert np.array_equal(bits_of(ctx.dequant_expert(29, 127, which)), want), name
        assert np.array_equal(bits_of(ctx.prefill_tiles(29, 127, which)), want), name


def test_lm_head_262144_greedy(model, oracle, torch):
    syn, ctx = model["syn"], model["ctx"]
    W, S, B = syn.synth_matrix_gpu(torch, model["gen"], syn.VOCAB)
    head = ctx.matrix(W, S, B, greedy=True)
    Wh, Sh, Bh = W.cpu().numpy(), bits_of(S), bits_of(B)
    del W, S, B
    rng = np.random.default_rng(3000)
    xb = syn.bf16_bits(rng.normal(0, 1, (16, syn.D)).astype(np.float32))
    x = torch.from_numpy(xb.view(np.int16)).cuda().view(torch.bfloat16)
    tokens = head.greedy(x).cpu().numpy()
    logits = head.gemv(x, f32_out=True).cpu().numpy()
    # every row's choice is the first maximum of the GEMV's own fp32 logits
    assert np.array_equal(tokens, logits.argmax(1))
    # every row against the CPU reference (dequantise the row, then dot: DequantInt4GemvRef); the gap between the best
    # and the second-best logit says how much room the comparison had
    for row in range(16):
        ref = oracle.gemv_int4_ref(Wh, Sh, Bh, oracle.bf16_to_float(xb[row]))
        order = np.argsort(-ref, kind="stable")
        gap = float(ref[order[0]] - ref[order[1]])
        assert rel_err(logits[row], ref) <= 5e-3, (row, rel_err(logits[row], ref))
        err = float(np.abs(logits[row] - ref).max())
        if gap > 2 * err:       # the reference's winner is beyond what the two summation orders can differ by
            assert int(tokens[row]) == int(order[0]), (row, int(tokens[row]), int(order[0]), gap, err)
        else:
            assert ref[int(tokens[row])] >= ref[order[0]] - 2 * err, (row, gap, err)
        print(f"row {row}: token {int(order[0])}, top-2 logit gap {gap:.4f} ({gap / abs(float(ref[order[0]])):.2e} of the maximum)")
    head.close()
