"""A decode loop at a small shape, the way BASELINE.json config 5 runs it: blocks of 16 rows through every layer
(router + routed experts in the one call the benchmark times, the layer's output added to its input), then the INT4
LM head's greedy choice, whose tokens pick the next block's rows from an embedding table. Every layer of every block
is held against the CPU oracle on the rows the GPU fed it (routes bit for bit, rows within the 1e-2 / 0.9999 bar), and
every token against the oracle's argmax over the head (Kernels/Fusions/LMHeadChainInt4.swift:94-139), with the
reference tests' allowance where two logits are closer than the two summation orders can differ."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, cosine, make_layer, rel_err, to_ff_offsets

pytestmark = pytest.mark.gpu

D, F, E, K, LAYERS, VOCAB, BLOCKS, ROWS = 256, 128, 32, 8, 3, 1024, 16, 16


def test_decode_loop_small_shape(oracle):
    import torch
    import fieldfare_moe as ff
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    ctx = ff.Context(D, F, E, K, n_layers=LAYERS, max_tokens=64)
    pools, routers = [], []
    for layer in range(LAYERS):
        _, pool, router = make_layer(oracle, 500 + layer, D, F, E)
        ctx.upload_layer(layer, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
        ctx.upload_router_bf16(layer, router)
        pools.append(pool)
        routers.append(router)
    rng = np.random.default_rng(77)
    Wq, Sq, Bq = oracle.quantize_int4(rng.normal(0, 0.05, (VOCAB, D)).astype(np.float32))
    head = ctx.matrix(torch.from_numpy(Wq).cuda(), bf16_tensor(torch, Sq), bf16_tensor(torch, Bq), greedy=True)
    embed = oracle.bf16_bits(rng.normal(0, 1, (VOCAB, D)).astype(np.float32))
    tokens = rng.integers(0, VOCAB, ROWS)
    seen = []
    for block in range(BLOCKS):
        xb = embed[tokens]
        x = bf16_tensor(torch, xb)
        for layer in range(LAYERS):
            y, idx, w = ctx.route_verify(layer, x, x, residual=x)
            idx_np = idx.cpu().numpy().astype(np.uint32)
            for r in range(ROWS):
                ridx, _ = oracle.topk_softmax(oracle.router_logits_pinned(routers[layer], xb[r]), K)
                assert np.array_equal(idx_np[r], ridx), (block, layer, r)
            ref = oracle.moe_experts(pools[layer], xb, idx_np, oracle.bf16_to_float(bits_of(w))) + oracle.bf16_to_float(xb)
            got = oracle.bf16_to_float(bits_of(y))
            assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999, (block, layer, rel_err(got, ref))
            x, xb = y, bits_of(y)
        chosen = head.greedy(x).cpu().numpy().astype(np.int64)
        for r in range(ROWS):
            ref = oracle.gemv_int4_ref(Wq, Sq, Bq, oracle.bf16_to_float(xb[r]))
            best = int(np.argmax(ref))
            if int(chosen[r]) != best:      # only where the two leading logits are within the summation orders' reach
                assert ref[best] - ref[int(chosen[r])] <= 5e-3 * np.abs(ref).max(), (block, r, int(chosen[r]), best)
        tokens = chosen
        seen.append(chosen.copy())
    assert ctx.handover_giveups() == 0
    assert len({tuple(s_) for s_ in seen}) > 1, "the loop must move: the blocks' tokens differ"
    head.close()
    ctx.close()
