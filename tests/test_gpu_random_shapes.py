"""Shapes drawn at random (fixed seeds, so every run sees the same cases): ragged row counts, expert counts that are no
multiple of anything, top_k from 1 to 8, hidden and intermediate sizes from 128 up - through the router, the verify
block (both forms), the prefill chunk and the dense FFN, each against the CPU oracle to the bar of the fixed-shape
tests. Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, cosine, make_layer, rel_err, to_ff_offsets

pytestmark = pytest.mark.gpu


def _draw(seed, n_cases, dense):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < n_cases:
        d = 64 * int(rng.integers(2, 24))
        f = 64 * int(rng.integers(2, 30 if dense else 12))
        e = 1 if dense else int(rng.integers(1, 257))
        k = 1 if dense else int(rng.integers(1, min(8, e) + 1))
        t, tp = int(rng.integers(1, 17)), int(rng.integers(17, 700))
        if d * f * e > 24_000_000 or (dense and d * f > 1_500_000):
            continue
        if not dense and len(cases) % 3 == 0:
            # a shape the prefill router's two-pass form takes (d a multiple of 256, 16 ... 128 experts in sixteens)
            d, e = 256 * max(1, d // 256), 16 * max(1, min(8, e // 16))
            k = min(k, e)
        cases.append((len(cases), d, f, e, k, t, tp))
    return cases


@pytest.mark.parametrize("case,d,f,e,k,t,tp", _draw(2024, 24, False))
def test_random_routed_shapes(oracle, case, d, f, e, k, t, tp):
    import torch
    import fieldfare_moe as ff
    ff.lib()
    rng, pool, router = make_layer(oracle, 9000 + case, d, f, e, align=1)
    ctx = ff.Context(d, f, e, k, n_layers=1, max_tokens=max(tp, 16))
    try:
        ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
        ctx.upload_router_bf16(0, router)
        for rows, run in ((t, "verify"), (tp, "prefill")):
            xb = oracle.bf16_bits(rng.normal(0, 1, (rows, d)).astype(np.float32))
            x = bf16_tensor(torch, xb)
            idx, w = ctx.router(0, x)
            idx_np = idx.cpu().numpy().astype(np.uint32)
            for tok in range(0, rows, max(1, rows // 4)):
                want, _ = oracle.topk_softmax(oracle.router_logits_pinned(router, xb[tok]), k)
                assert np.array_equal(idx_np[tok], want), (run, tok)
            sel = np.arange(rows) if rows <= 48 else np.sort(rng.choice(rows, 32, replace=False))
            ref = oracle.moe_experts(pool, xb[sel], idx_np[sel], oracle.bf16_to_float(bits_of(w))[sel])
            y = ctx.verify(0, x, idx, w) if run == "verify" else ctx.prefill(0, x, idx, w)
            got = oracle.bf16_to_float(bits_of(y))[sel]
            assert rel_err(got, ref) <= 1e-2 and cosine(got, ref) >= 0.9999, (run, rel_err(got, ref), cosine(got, ref))
            if run == "verify":
                # router, select and gate/up in one launch: the same routes and rows bit for bit
                y2, idx2, w2 = ctx.route_verify(0, x, x)
                assert np.array_equal(idx2.cpu().numpy().astype(np.uint32), idx_np)
                assert np.array_equal(bits_of(w2), bits_of(w)) and np.array_equal(bits_of(y2), bits_of(y))
        assert ctx.handover_giveups() == 0
    finally:
        ctx.close()


@pytest.mark.parametrize("case,d,f,e,k,t,tp", _draw(2025, 12, True))
def test_random_dense_ffn_shapes(oracle, case, d, f, e, k, t, tp):
    import torch
    import fieldfare_moe as ff
    ff.lib()
    g = np.random.default_rng(7000 + case)
    scale = 0.4 if d < 1024 else 0.08
    parts = tuple(oracle.quantize_int4(g.uniform(-scale, scale, (r, c)).astype(np.float32)) for r, c in ((f, d), (f, d), (d, f)))
    (gW, gS, gB), (uW, uS, uB), (dW, dS, dB) = parts
    ctx = ff.Context(d, f, 1, 1, n_layers=1, max_tokens=max(tp, 16))
    try:
        ctx.upload_expert_parts(0, 0, *parts)
        for rows in (t, tp):
            xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, (rows, d)).astype(np.float32))
            sel = np.arange(rows) if rows <= 16 else np.sort(g.choice(rows, 16, replace=False))
            ref = []
            for row in xb[sel]:
                xr = oracle.bf16_to_float(row)
                act = oracle.gelu_tanh(oracle.gemv_int4_ref(gW, gS, gB, xr)) * oracle.gemv_int4_ref(uW, uS, uB, xr)
                ref.append(oracle.gemv_int4_ref(dW, dS, dB, oracle.bf16_to_float(oracle.bf16_bits(act))))
            ref = np.stack(ref)
            y = oracle.bf16_to_float(bits_of(ctx.dense_ffn(0, bf16_tensor(torch, xb))))[sel]
            assert rel_err(y, ref) <= 1e-2 and cosine(y, ref) >= 0.9999, (rows, rel_err(y, ref), cosine(y, ref))
    finally:
        ctx.close()
