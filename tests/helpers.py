"""Shared builders for the GPU parity tests: seeded synthetic layers in the reference blob layout."""
import numpy as np

REAL = dict(d=2816, f=704, n_experts=128, top_k=8)
REAL_STRIDE = 3_358_720     # 205 x 16 KiB, Planning/RepackPlanner.swift:431-493


def rel_err(actual, ref):
    """RelError.compute, Tests/Support/Validation/Tolerance/RelError.swift:7-16."""
    actual = np.asarray(actual, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(actual - ref).max() / max(np.abs(ref).max(), 1e-6))


def cosine(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))


def make_layer(oracle, seed, d, f, n_experts, stride=None, align=16):
    rng = np.random.default_rng(seed)
    pool = oracle.random_pool(rng, n_experts, d, f, stride=stride, align=align)
    router = oracle.bf16_bits(rng.normal(0, 0.02, (n_experts, d)).astype(np.float32))
    return rng, pool, router


def to_ff_offsets(ff, o):
    return ff.Offsets(*o.as_tuple())


def bf16_tensor(torch, bits, device="cuda"):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(device).view(torch.bfloat16)


def bits_of(t):
    import torch
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
