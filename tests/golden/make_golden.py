"""Writes tests/golden/moe_small.npz: one small quantized MoE layer, a 5-row block, and what the CPU oracle
makes of them. Nothing here reads or runs the reference; the oracle that computes the expected values is the
one the other tests pin against the reference tests' known answers.

    python tests/golden/make_golden.py

The file freezes inputs AND outputs, so a later change to the oracle or to a kernel that moves a result shows
up against a fixed record (tests/test_golden.py), not only as a disagreement between the two.

Shapes: hidden 128, intermediate 64, 16 experts, top-8, INT4 g64 blobs in the reference's per-expert layout
(gate W/S/B, up W/S/B, down W/S/B; Planning/RepackPlanner.swift:431-493), bf16 router [16][128].
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import oracle  # noqa: E402

D, F, E, K, T = 128, 64, 16, 8, 5
GEMV_M, GEMV_N, GEMV_ROWS = 24, 192, 3


def main():
    oracle.build()
    rng = np.random.default_rng(20260603)
    pool = oracle.random_pool(rng, E, D, F, align=1)
    router = oracle.bf16_bits(rng.normal(0, 0.05, (E, D)).astype(np.float32))
    x = oracle.bf16_bits(rng.normal(0, 1, (T, D)).astype(np.float32))
    residual = oracle.bf16_bits(rng.normal(0, 1, (T, D)).astype(np.float32))

    logits = np.stack([oracle.router_logits_pinned(router, x[t]) for t in range(T)])
    idx = np.zeros((T, K), np.uint32)
    w = np.zeros((T, K), np.float32)
    for t in range(T):
        idx[t], w[t] = oracle.topk_softmax(logits[t], K)
    w_bits = oracle.bf16_bits(w)
    # the expert stage takes the 16-bit routing weights the router hands over
    y = oracle.moe_experts(pool, x, idx, oracle.bf16_to_float(w_bits))

    deq = {}
    for name in ("gate", "up", "down"):
        deq[name] = oracle.dequantize_int4_bf16(*pool.sub(3, name))

    gw, gs, gb = oracle.quantize_int4(rng.uniform(-0.5, 0.5, (GEMV_M, GEMV_N)).astype(np.float32))
    gx = oracle.bf16_bits(rng.uniform(-1, 1, (GEMV_ROWS, GEMV_N)).astype(np.float32))
    gy = np.stack([oracle.gemv_int4_ref(gw, gs, gb, oracle.bf16_to_float(gx[r])) for r in range(GEMV_ROWS)])

    out = Path(__file__).with_name("moe_small.npz")
    np.savez_compressed(
        out,
        dims=np.array([D, F, E, K, T], np.uint32),
        pool_bytes=pool.bytes, pool_stride=np.uint64(pool.stride),
        pool_offsets=np.array(pool.offsets.as_tuple(), np.uint64),
        router_bits=router, x_bits=x, residual_bits=residual,
        logits_bits=logits.view(np.uint32), idx=idx, w_f32=w, w_bits=w_bits, y_f32=y,
        dequant_expert3_gate=deq["gate"], dequant_expert3_up=deq["up"], dequant_expert3_down=deq["down"],
        gemv_w=gw, gemv_scales=gs, gemv_biases=gb, gemv_x_bits=gx, gemv_y_f32=gy)
    print(out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
