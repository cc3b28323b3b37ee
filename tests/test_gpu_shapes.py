"""Odd shapes through the C ABI against the CPU oracle: hidden / intermediate sizes that are not multiples of a
wave's K-slice, a single 64-wide group, expert counts that are not powers of two, fewer experts than top-k
slots, one route per token - for the router, the <= 16-row expert path and the grouped-GEMM path alike.
Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, cosine, make_layer, rel_err, to_ff_offsets

pytestmark = pytest.mark.gpu

#        d     f    e  k   t   prefill rows
SHAPES = [(64, 64, 1, 1, 1, 19),
          (64, 64, 2, 2, 16, 40),
          (192, 64, 5, 3, 7, 33),
          (320, 192, 9, 4, 16, 70),
          (704, 128, 17, 8, 3, 150),
          (1024, 320, 33, 8, 16, 257),
          (128, 704, 128, 8, 16, 64),
          (448, 448, 128, 1, 16, 300),
          (2816, 64, 8, 8, 1, 17),
          (1088, 1088, 3, 3, 5, 23),
          (256, 128, 256, 8, 16, 300),      # the most experts a context takes: selects over four key slots per lane
          (128, 64, 200, 4, 9, 100)]


@pytest.mark.parametrize("d,f,e,k,t,tp", SHAPES)
def test_shape(oracle, d, f, e, k, t, tp):
    import torch
    import fieldfare_moe as ff
    ff.lib()       # raises when the HIP library is not built: no fallback
    rng, pool, router = make_layer(oracle, 7000 + d + f + e, d, f, e, align=1)
    ctx = ff.Context(d, f, e, k, n_layers=1, max_tokens=max(tp, 16))
    try:
        ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
        ctx.upload_router_bf16(0, router)
        for rows, run in ((t, "verify"), (tp, "prefill")):
            xb = oracle.bf16_bits(rng.normal(0, 1, (rows, d)).astype(np.float32))
            x = bf16_tensor(torch, xb)
            idx, w = ctx.router(0, x)
            idx_np = idx.cpu().numpy().astype(np.uint32)
            for tok in range(0, rows, max(1, rows // 5)):
                ridx, _ = oracle.topk_softmax(oracle.router_logits_pinned(router, xb[tok]), k)
                assert np.array_equal(idx_np[tok], ridx), (run, tok)
            ref = oracle.moe_experts(pool, xb, idx_np, oracle.bf16_to_float(bits_of(w)))
            y = ctx.verify(0, x, idx, w) if run == "verify" else ctx.prefill(0, x, idx, w)
            got = oracle.bf16_to_float(bits_of(y))
            assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999, run
            if run == "verify":
                assert ctx.last_live_experts() == len(np.unique(idx_np))
                y2, idx2, _ = ctx.route_verify(0, x, x)
                assert np.array_equal(idx2.cpu().numpy().astype(np.uint32), idx_np)
                assert np.array_equal(bits_of(y2), bits_of(y)), "router + experts in one call differs from the two calls"
    finally:
        ctx.close()
