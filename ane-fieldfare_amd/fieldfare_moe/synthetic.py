"""Seeded synthetic workloads of the shape the benchmark configurations name: expert layers in the reference's
blob layout generated on the GPU, verify blocks whose tokens share experts, Zipf-routed prefill chunks and INT4
matrices. Used by bench.py and by the GPU tests of the whole-model sweep; needs torch and numpy only.
"""
from __future__ import annotations

import numpy as np

from . import GROUP, Offsets

D, F, E, K = 2816, 704, 128, 8           # Gemma-4-26B-A4B: hidden, routed intermediate, experts, top-k
VOCAB = 262144
STRIDE = 3_358_720                       # 205 x 16 KiB per expert blob (Planning/RepackPlanner.swift:431-493)
EXPERT_BYTES = 3_345_408                 # gate + up + down weights, scales and biases of one expert
TOKEN_CORRELATION = 0.45                 # shared component of a verify block's tokens -> 40-60 distinct experts


def layout_offsets(d: int, f: int, align: int = 16):
    """(Offsets, payload bytes) of one expert blob: gate W/S/B, up W/S/B, down W/S/B, each `align`-aligned
    (makeBlob, Tests/ANEFieldfareUpstreamTests/Kernels/MoE/MoEFusedFFNTests.swift:221-257)."""
    def up(v):
        return (v + align - 1) // align * align
    sizes = []
    for rows, cols in ((f, d), (f, d), (d, f)):
        sizes += [rows * cols // 2, rows * (cols // GROUP) * 2, rows * (cols // GROUP) * 2]
    offs, cur = [], 0
    for sz in sizes:
        cur = up(cur)
        offs.append(cur)
        cur += sz
    return Offsets(*offs), up(cur)


def bf16_bits(a) -> np.ndarray:
    """float array -> bf16 bit patterns (uint16), round to nearest even (Quantization.bf16Bits,
    Infrastructure/ModelIO/Quantization.swift:9-15); the inputs here hold no NaN."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_cuda(torch, a):
    """float array -> bf16 CUDA tensor of the same shape."""
    return torch.from_numpy(bf16_bits(a).view(np.int16)).cuda().view(torch.bfloat16)


def synth_layer_gpu(torch, gen, offsets: Offsets, d: int = D, f: int = F, n_experts: int = E, stride: int = STRIDE):
    """One layer of experts in the reference blob layout, generated on the GPU: q ~ U{0..15},
    scale = bf16(|N(0, 0.01)|), bias = bf16(-8 scale + N(0, 1e-3)). Returns uint8 [n_experts, stride]."""
    blob = torch.zeros((n_experts, stride), dtype=torch.uint8, device="cuda")
    offs = tuple(getattr(offsets, n) for n, _ in offsets._fields_)
    for i, (rows, cols) in enumerate(((f, d), (f, d), (d, f))):
        wo, so, bo = offs[3 * i:3 * i + 3]
        nw, ns = rows * cols // 2, rows * (cols // GROUP)
        blob[:, wo:wo + nw] = torch.randint(0, 256, (n_experts, nw), dtype=torch.uint8, device="cuda", generator=gen)
        s = (torch.randn((n_experts, ns), device="cuda", generator=gen) * 0.01).abs().to(torch.bfloat16)
        b = (-8.0 * s.float() + torch.randn((n_experts, ns), device="cuda", generator=gen) * 1e-3).to(torch.bfloat16)
        blob[:, so:so + 2 * ns] = s.view(torch.uint8).view(n_experts, 2 * ns)
        blob[:, bo:bo + 2 * ns] = b.view(torch.uint8).view(n_experts, 2 * ns)
    return blob


def synth_matrix_gpu(torch, gen, m: int, n: int = D):
    """INT4 g64 matrix [m][n] in the reference layout: (W uint8 [m][n/2], S bf16 [m][n/64], B bf16 [m][n/64])."""
    W = torch.randint(0, 256, (m, n // 2), dtype=torch.uint8, device="cuda", generator=gen)
    S = (torch.randn((m, n // GROUP), device="cuda", generator=gen) * 0.01).abs().to(torch.bfloat16)
    B = (-8.0 * S.float() + torch.randn((m, n // GROUP), device="cuda", generator=gen) * 1e-3).to(torch.bfloat16)
    return W, S, B


def block_tokens(rng: np.random.Generator, t: int, d: int = D) -> np.ndarray:
    """t token rows ~ N(0, 1) that share a common component, so that a 16-token block routes to about 40-60
    distinct experts with overlap (BASELINE config 3) instead of the ~80 of independent rows."""
    c = rng.normal(0, 1, d)
    n = rng.normal(0, 1, (t, d))
    return (np.sqrt(TOKEN_CORRELATION) * c + np.sqrt(1 - TOKEN_CORRELATION) * n).astype(np.float32)


def router_weights(rng: np.random.Generator, n_experts: int = E, d: int = D) -> np.ndarray:
    """bf16 bits [n_experts][d] ~ N(0, 0.02)."""
    return bf16_bits(rng.normal(0, 0.02, (n_experts, d)).astype(np.float32))


def zipf_routes(rng: np.random.Generator, t: int, n_experts: int = E, top_k: int = K, s: float = 1.1):
    """Imposed routing with Zipf(s) popularity over a permuted expert order: top_k distinct experts per token,
    weights uniform-random normalised to 1. Returns (idx int32 [t][top_k], w float32 [t][top_k])."""
    p = 1.0 / np.arange(1, n_experts + 1) ** s
    p /= p.sum()
    perm = rng.permutation(n_experts)
    idx = np.stack([perm[rng.choice(n_experts, top_k, replace=False, p=p)] for _ in range(t)]).astype(np.int32)
    w = rng.random((t, top_k)).astype(np.float32)
    return idx, w / w.sum(1, keepdims=True)
