"""The committed record tests/golden/moe_small.npz (written by tests/golden/make_golden.py): the CPU oracle must
still reproduce it, and the HIP path must match it through the C ABI - bit for bit where the work is integer or
pinned-order (dequantized weights, router logits, chosen experts), within the layer-output bar elsewhere."""
from pathlib import Path

import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, cosine, rel_err

GOLDEN = Path(__file__).parent / "golden" / "moe_small.npz"


@pytest.fixture(scope="module")
def gold():
    z = np.load(GOLDEN, allow_pickle=False)
    return {k: z[k] for k in z.files}


def _pool(oracle, gold):
    d, f = int(gold["dims"][0]), int(gold["dims"][1])
    offs = oracle.Offsets(*[int(v) for v in gold["pool_offsets"]])
    return oracle.ExpertPool(gold["pool_bytes"].copy(), offs, int(gold["pool_stride"]), d, f)


def test_oracle_reproduces_the_record(oracle, gold):
    d, f, e, k, t = (int(v) for v in gold["dims"])
    pool = _pool(oracle, gold)
    for tok in range(t):
        logits = oracle.router_logits_pinned(gold["router_bits"], gold["x_bits"][tok])
        assert np.array_equal(logits.view(np.uint32), gold["logits_bits"][tok])
        idx, w = oracle.topk_softmax(logits, k)
        assert np.array_equal(idx, gold["idx"][tok])
        # expf comes from the C library: allow it an ulp between builds
        assert np.allclose(w, gold["w_f32"][tok], rtol=1e-6, atol=0)
    for name in ("gate", "up", "down"):
        assert np.array_equal(oracle.dequantize_int4_bf16(*pool.sub(3, name)), gold[f"dequant_expert3_{name}"])
    y = oracle.moe_experts(pool, gold["x_bits"], gold["idx"], oracle.bf16_to_float(gold["w_bits"]))
    assert np.allclose(y, gold["y_f32"], rtol=1e-5, atol=1e-7)
    for r in range(gold["gemv_x_bits"].shape[0]):
        ref = oracle.gemv_int4_ref(gold["gemv_w"], gold["gemv_scales"], gold["gemv_biases"],
                                   oracle.bf16_to_float(gold["gemv_x_bits"][r]))
        assert np.allclose(ref, gold["gemv_y_f32"][r], rtol=1e-5, atol=1e-7)


def test_record_is_self_consistent(oracle, gold):
    # what the file itself fixes, without the oracle's kernels: the chosen experts are the eight largest
    # recorded logits (ties to the lower index), the weights are their softmax, and sum to one
    logits = gold["logits_bits"].view(np.float32)
    for tok in range(logits.shape[0]):
        order = sorted(range(logits.shape[1]), key=lambda i: (-logits[tok, i], i))[:8]
        assert list(gold["idx"][tok]) == order
        ex = np.exp(logits[tok, order].astype(np.float64) - logits[tok, order[0]])
        assert np.allclose(gold["w_f32"][tok], ex / ex.sum(), rtol=1e-5)
    assert np.array_equal(gold["w_bits"], oracle.bf16_bits(gold["w_f32"]))


@pytest.mark.gpu
def test_hip_path_matches_the_record(oracle, gold):
    import torch
    import fieldfare_moe as ff
    ff.lib()       # raises when the HIP library is not built: no fallback
    d, f, e, k, t = (int(v) for v in gold["dims"])
    ctx = ff.Context(d, f, e, k, n_layers=1, max_tokens=64)
    try:
        ctx.upload_layer(0, gold["pool_bytes"], int(gold["pool_stride"]),
                         ff.Offsets(*[int(v) for v in gold["pool_offsets"]]))
        ctx.upload_router_bf16(0, gold["router_bits"])
        for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
            assert np.array_equal(bits_of(ctx.dequant_expert(0, 3, which)), gold[f"dequant_expert3_{name}"]), name
        x = bf16_tensor(torch, gold["x_bits"])
        idx, w, logits = ctx.router(0, x, want_logits=True)
        assert np.array_equal(logits.cpu().numpy().view(np.uint32), gold["logits_bits"])
        assert np.array_equal(idx.cpu().numpy().astype(np.uint32), gold["idx"])
        got_w = oracle.bf16_to_float(bits_of(w))
        assert np.abs(got_w - gold["w_f32"]).max() <= np.abs(gold["w_f32"]).max() * 2 ** -7
        # the expert stage on the recorded routes and 16-bit weights, with and without the residual rows
        idx_rec = torch.from_numpy(gold["idx"].view(np.int32)).cuda()
        w_rec = bf16_tensor(torch, gold["w_bits"])
        got = oracle.bf16_to_float(bits_of(ctx.verify(0, x, idx_rec, w_rec)))
        assert rel_err(got, gold["y_f32"]) <= 1e-2 and cosine(got, gold["y_f32"]) >= 0.9999
        want_res = gold["y_f32"] + oracle.bf16_to_float(gold["residual_bits"])
        got = oracle.bf16_to_float(bits_of(ctx.verify(0, x, idx_rec, w_rec, residual=bf16_tensor(torch, gold["residual_bits"]))))
        assert rel_err(got, want_res) <= 1e-2 and cosine(got, want_res) >= 0.9999
        got = oracle.bf16_to_float(bits_of(ctx.prefill(0, x, idx_rec, w_rec)))
        assert rel_err(got, gold["y_f32"]) <= 1e-2 and cosine(got, gold["y_f32"]) >= 0.9999
        # the generic GEMV on the recorded matrix
        y = ctx.gemv_int4(torch.from_numpy(gold["gemv_w"]).cuda(), torch.from_numpy(gold["gemv_scales"].view(np.int16)).cuda(),
                          torch.from_numpy(gold["gemv_biases"].view(np.int16)).cuda(),
                          bf16_tensor(torch, gold["gemv_x_bits"]), f32_out=True).cpu().numpy()
        assert rel_err(y, gold["gemv_y_f32"]) < 5e-3
    finally:
        ctx.close()
