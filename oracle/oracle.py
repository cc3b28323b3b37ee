"""ctypes/numpy front end of the CPU oracle (oracle/ffmoe_oracle.c). TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the
product package never does. Every function forwards to the C restatement, whose comments cite the
reference file:line each one follows; the few pure-Python functions here restate host-side integer
logic of the reference and cite it themselves.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "libffmoe_oracle.so"

BF16, FP16, F32 = 0, 1, 2
GROUP = 64


NATIVE_FLAGS = "-O3 -march=native -ffp-contract=off -fno-fast-math -fopenmp -fPIC -std=c11"


def build(force: bool = False) -> Path:
    """Compile the C oracle with the Makefile beside it."""
    if force or not _LIB_PATH.exists():
        subprocess.run(["make", "-C", str(_DIR), "-B", "libffmoe_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def use_native_build(out_dir) -> str | None:
    """For the CPU baseline on the machine that runs it: compile the same source with -march=native into `out_dir`
    and make it the library this module calls (the in-tree build targets x86-64-v3 so that one file runs on every
    host it is carried to). Returns the flags used, or None when no compiler is there and the in-tree build stays.
    Same arithmetic either way: contraction and fast-math stay off."""
    global _lib, _LIB_PATH
    out = Path(out_dir) / "libffmoe_oracle_native.so"
    try:
        subprocess.run(["gcc", *NATIVE_FLAGS.split(), "-shared", "-o", str(out), str(_DIR / "ffmoe_oracle.c"), "-lm"],
                       check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=120)
    except (OSError, subprocess.SubprocessError):
        return None
    _LIB_PATH, _lib = out, None
    return NATIVE_FLAGS


class Offsets(C.Structure):
    """MoEExpertOffsets, Kernels/MoE/MoE.swift:4-29."""
    _fields_ = [(n, C.c_uint32) for n in
                ("gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)


PAIR_DTYPE = np.dtype([("token", "<u4"), ("expert", "<u4"), ("rank", "<u4"), ("weight_bits", "<u4")])

_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(str(_LIB_PATH))
        vp, u64p = C.c_void_p, C.POINTER(C.c_uint64)
        L.ffo_bf16_bits.restype = C.c_uint16
        L.ffo_bf16_bits.argtypes = [C.c_float]
        L.ffo_bf16_to_float.restype = C.c_float
        L.ffo_bf16_to_float.argtypes = [C.c_uint16]
        L.ffo_fp16_bits.restype = C.c_uint16
        L.ffo_fp16_bits.argtypes = [C.c_float]
        L.ffo_fp16_to_float.restype = C.c_float
        L.ffo_fp16_to_float.argtypes = [C.c_uint16]
        L.ffo_splitmix64_next.restype = C.c_uint64
        L.ffo_splitmix64_next.argtypes = [u64p]
        L.ffo_splitmix64_uniform.restype = C.c_float
        L.ffo_splitmix64_uniform.argtypes = [u64p, C.c_float, C.c_float]
        L.ffo_splitmix64_fill_uniform.restype = None
        L.ffo_splitmix64_fill_uniform.argtypes = [u64p, C.c_float, C.c_float, vp, C.c_size_t]
        L.ffo_seedtree_key.restype = C.c_uint64
        L.ffo_seedtree_key.argtypes = [C.c_uint64, C.c_char_p]
        for name in ("ffo_quantize_int4_affine", "ffo_quantize_int8_affine"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, C.c_int, vp, vp, vp]
        for name in ("ffo_dequantize_int4_affine", "ffo_dequantize_int4_bf16", "ffo_dequantize_int8_affine"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, vp, C.c_int, vp]
        L.ffo_gemv_int4_ref.restype = None
        L.ffo_gemv_int4_ref.argtypes = [vp, vp, vp, C.c_int, C.c_int, vp, vp]
        L.ffo_int4_dot.restype = C.c_float
        L.ffo_int4_dot.argtypes = [vp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int, vp]
        L.ffo_gelu_tanh.restype = C.c_float
        L.ffo_gelu_tanh.argtypes = [C.c_float]
        L.ffo_run_ffn.restype = None
        L.ffo_run_ffn.argtypes = [vp, C.POINTER(Offsets), C.c_int, C.c_int, vp, vp]
        L.ffo_apply_streamed_routed.restype = None
        L.ffo_apply_streamed_routed.argtypes = [vp, C.POINTER(Offsets), C.c_int, C.c_int, vp, vp, vp, C.c_int, vp]
        L.ffo_route_partials.restype = None
        L.ffo_route_partials.argtypes = [vp, C.c_size_t, vp, C.c_size_t, C.POINTER(Offsets), vp, C.c_size_t,
                                         C.c_int, C.c_int, C.c_int, C.c_int, vp, C.c_int]
        L.ffo_reduce_token_major.restype = None
        L.ffo_reduce_token_major.argtypes = [vp, C.c_int, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp]
        L.ffo_router_logits_pinned.restype = None
        L.ffo_router_logits_pinned.argtypes = [vp, C.c_int, vp, C.c_int, vp, C.c_int, C.c_int, vp]
        L.ffo_topk_softmax.restype = None
        L.ffo_topk_softmax.argtypes = [vp, C.c_int, C.c_int, vp, vp, vp]
        L.ffo_moe_layer.restype = None
        L.ffo_moe_layer.argtypes = [vp, C.c_size_t, C.POINTER(Offsets), C.c_int, C.c_int, C.c_int, vp, vp,
                                    C.c_size_t, C.c_int, C.c_int, C.c_int, vp, vp, vp, C.c_int]
        L.ffo_moe_experts.restype = None
        L.ffo_moe_experts.argtypes = [vp, C.c_size_t, C.POINTER(Offsets), C.c_int, C.c_int, vp, C.c_size_t,
                                      C.c_int, C.c_int, C.c_int, vp, vp, vp, C.c_int]
        L.ffo_post_attn_setup.restype = None
        L.ffo_post_attn_setup.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_float, C.c_int]
        L.ffo_rmsnorm.restype = None
        L.ffo_rmsnorm.argtypes = [vp, vp, vp, C.c_int, C.c_float, C.c_int]
        L.ffo_layer_tail.restype = None
        L.ffo_layer_tail.argtypes = [vp, vp, vp, vp, vp, C.c_int, C.c_float, C.c_float, C.c_int]
        L.ffo_max_threads.restype = C.c_int
        _lib = L
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


# ----------------------------------------------------------------------------- codecs
def bf16_bits(x) -> np.ndarray:
    """Vectorised Quantization.bf16Bits (Infrastructure/ModelIO/Quantization.swift:9-15)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    return (((u + 0x7FFF + lsb) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_to_float(b) -> np.ndarray:
    """Vectorised Quantization.bf16ToFloat (Quantization.swift:17-20)."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bits16(x, dtype: int) -> np.ndarray:
    if dtype == FP16:
        return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)
    return bf16_bits(x)


def from_bits16(b, dtype: int) -> np.ndarray:
    if dtype == FP16:
        return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)
    return bf16_to_float(b)


# ----------------------------------------------------------------------------- PRNG
class SplitMix64:
    """Tests/Support/Validation/PRNG/SplitMix64.swift:9-21."""

    def __init__(self, seed: int):
        self.state = C.c_uint64(seed & 0xFFFFFFFFFFFFFFFF)

    def next(self) -> int:
        return int(lib().ffo_splitmix64_next(C.byref(self.state)))

    def uniform(self, lo: float, hi: float, n: int | None = None):
        if n is None:
            return float(lib().ffo_splitmix64_uniform(C.byref(self.state), lo, hi))
        out = np.empty(n, dtype=np.float32)
        lib().ffo_splitmix64_fill_uniform(C.byref(self.state), lo, hi, _p(out), n)
        return out


def seed_tree_key(root: int, label: str) -> SplitMix64:
    """SeedTree.key, Tests/Support/Validation/PRNG/SeedTree.swift:12-19."""
    return SplitMix64(int(lib().ffo_seedtree_key(root, label.encode("utf-8"))))


# ----------------------------------------------------------------------------- quantisation
def quantize_int4(rows: np.ndarray):
    """Row-wise quantizeInt4Affine. rows float32 [M][N] -> (packed u8 [M][N/2], scales, biases u16 [M][N/64])."""
    rows = np.ascontiguousarray(rows, dtype=np.float32)
    m, n = rows.shape
    assert n % GROUP == 0
    packed = np.zeros((m, n // 2), np.uint8)
    s = np.zeros((m, n // GROUP), np.uint16)
    b = np.zeros((m, n // GROUP), np.uint16)
    L = lib()
    for r in range(m):
        L.ffo_quantize_int4_affine(_p(rows[r]), n, _p(packed[r]), _p(s[r]), _p(b[r]))
    return packed, s, b


def dequantize_int4(packed, s, b) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    s = np.ascontiguousarray(s, np.uint16)
    b = np.ascontiguousarray(b, np.uint16)
    m, nb = packed.shape
    out = np.empty((m, nb * 2), np.float32)
    L = lib()
    for r in range(m):
        L.ffo_dequantize_int4_affine(_p(packed[r]), _p(s[r]), _p(b[r]), nb * 2, _p(out[r]))
    return out


def dequantize_int4_bf16(packed, s, b) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    s = np.ascontiguousarray(s, np.uint16)
    b = np.ascontiguousarray(b, np.uint16)
    m, nb = packed.shape
    out = np.empty((m, nb * 2), np.uint16)
    L = lib()
    for r in range(m):
        L.ffo_dequantize_int4_bf16(_p(packed[r]), _p(s[r]), _p(b[r]), nb * 2, _p(out[r]))
    return out


def quantize_int8(rows: np.ndarray):
    rows = np.ascontiguousarray(rows, dtype=np.float32)
    m, n = rows.shape
    packed = np.zeros((m, n), np.uint8)
    s = np.zeros((m, n // GROUP), np.uint16)
    b = np.zeros((m, n // GROUP), np.uint16)
    for r in range(m):
        lib().ffo_quantize_int8_affine(_p(rows[r]), n, _p(packed[r]), _p(s[r]), _p(b[r]))
    return packed, s, b


def dequantize_int8(packed, s, b) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    m, n = packed.shape
    out = np.empty((m, n), np.float32)
    s = np.ascontiguousarray(s, np.uint16)
    b = np.ascontiguousarray(b, np.uint16)
    for r in range(m):
        lib().ffo_dequantize_int8_affine(_p(packed[r]), _p(s[r]), _p(b[r]), n, _p(out[r]))
    return out


def gemv_int4_ref(W, S, B, x) -> np.ndarray:
    """DequantInt4GemvRef.apply for one input vector x (float32 [N]) -> float32 [M]."""
    W = np.ascontiguousarray(W, np.uint8)
    S = np.ascontiguousarray(S, np.uint16)
    Bb = np.ascontiguousarray(B, np.uint16)
    x = np.ascontiguousarray(x, np.float32)
    m, nb = W.shape
    y = np.empty(m, np.float32)
    lib().ffo_gemv_int4_ref(_p(W), _p(S), _p(Bb), m, nb * 2, _p(x), _p(y))
    return y


def gemv_int8_ref(W, S, B, x) -> np.ndarray:
    """DequantInt8GemvRef.apply (Tests/Support/Validation/Reference/Quant/DequantInt8Gemv.swift:8-37) for one input
    vector: every row dequantised (Quantization.dequantizeInt8Affine), then a dot product - in float64 here, where the
    reference's vDSP_dotpr sums in fp32 (it is a tolerance reference there as well)."""
    rows = dequantize_int8(W, S, B).astype(np.float64)
    return (rows @ np.ascontiguousarray(x, np.float64)).astype(np.float32)


def gelu_tanh(x) -> np.ndarray:
    x = np.atleast_1d(np.asarray(x, np.float32))
    return np.array([lib().ffo_gelu_tanh(float(v)) for v in x.ravel()], np.float32).reshape(x.shape)


# ----------------------------------------------------------------------------- expert blobs
@dataclass
class ExpertPool:
    """`n` expert blobs of one layer, `stride` bytes apart, in the reference's byte layout:
    [gate W, S, B, up W, S, B, down W, S, B] (Planning/RepackPlanner.swift:431-493;
    makeBlob in MoEFusedFFNTests.swift:221-257)."""
    bytes: np.ndarray  # uint8 [n * stride]
    offsets: Offsets
    stride: int
    d: int
    f: int

    @property
    def n(self) -> int:
        return self.bytes.size // self.stride

    def sub(self, expert: int, which: str):
        """(W u8 [rows][cols/2], S u16 [rows][cols/64], B u16) views of one sub-tensor."""
        rows, cols = (self.f, self.d) if which in ("gate", "up") else (self.d, self.f)
        base = expert * self.stride
        o = self.offsets
        w_off, s_off, b_off = {"gate": (o.gate_w, o.gate_s, o.gate_b), "up": (o.up_w, o.up_s, o.up_b),
                               "down": (o.down_w, o.down_s, o.down_b)}[which]
        W = self.bytes[base + w_off: base + w_off + rows * cols // 2].reshape(rows, cols // 2)
        S = self.bytes[base + s_off: base + s_off + rows * (cols // GROUP) * 2].view(np.uint16).reshape(rows, -1)
        B = self.bytes[base + b_off: base + b_off + rows * (cols // GROUP) * 2].view(np.uint16).reshape(rows, -1)
        return W, S, B


def layout_offsets(d: int, f: int, align: int = 1):
    """Sub-tensor offsets and payload size of one expert blob."""
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


def pool_from_parts(parts, d: int, f: int, align: int = 1, stride: int | None = None) -> ExpertPool:
    """parts: per expert ((gW,gS,gB),(uW,uS,uB),(dW,dS,dB)) as numpy arrays."""
    offs, payload = layout_offsets(d, f, align)
    stride = stride or payload
    buf = np.zeros(len(parts) * stride, np.uint8)
    for e, triple in enumerate(parts):
        flat = [a for sub in triple for a in sub]
        for off, arr in zip(offs.as_tuple(), flat):
            raw = np.ascontiguousarray(arr).view(np.uint8).ravel()
            buf[e * stride + off: e * stride + off + raw.size] = raw
    return ExpertPool(buf, offs, stride, d, f)


def pool_from_float(gates, ups, downs, align: int = 1) -> ExpertPool:
    """Quantise float matrices per expert with quantizeInt4Affine and lay them out as makeBlob does."""
    f, d = gates[0].shape
    parts = [(quantize_int4(g), quantize_int4(u), quantize_int4(dn)) for g, u, dn in zip(gates, ups, downs)]
    return pool_from_parts(parts, d, f, align)


def random_pool(rng: np.random.Generator, n_experts: int, d: int, f: int, stride: int | None = None,
                align: int = 16) -> ExpertPool:
    """Synthetic experts in the form the benchmark configs state: q ~ U{0..15}, scale = bf16(|N(0, 0.01)|),
    bias = bf16(-8*scale + N(0, 1e-3))."""
    parts = []
    for _ in range(n_experts):
        triple = []
        for rows, cols in ((f, d), (f, d), (d, f)):
            W = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
            sc = np.abs(rng.normal(0, 0.01, size=(rows, cols // GROUP))).astype(np.float32)
            S = bf16_bits(sc)
            B = bf16_bits(-8.0 * bf16_to_float(S) + rng.normal(0, 1e-3, size=S.shape).astype(np.float32))
            triple.append((W, S, B))
        parts.append(tuple(triple))
    return pool_from_parts(parts, d, f, align, stride)


# ----------------------------------------------------------------------------- FFN / layer
def int4_dot(pool: ExpertPool, expert: int, which: str, row: int, x) -> float:
    o = pool.offsets
    w, s, b = {"gate": (o.gate_w, o.gate_s, o.gate_b), "up": (o.up_w, o.up_s, o.up_b),
               "down": (o.down_w, o.down_s, o.down_b)}[which]
    n = pool.d if which != "down" else pool.f
    x = np.ascontiguousarray(x, np.float32)
    return float(lib().ffo_int4_dot(_p(pool.bytes), expert * pool.stride, w, s, b, row, n, _p(x)))


def run_ffn(pool: ExpertPool, expert: int, x) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(pool.d, np.float32)
    base = pool.bytes[expert * pool.stride:]
    lib().ffo_run_ffn(_p(base), C.byref(pool.offsets), pool.d, pool.f, _p(x), _p(out))
    return out


def apply_streamed_routed(pool: ExpertPool, experts, x, residual, routing_w) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    residual = np.ascontiguousarray(residual, np.float32)
    routing_w = np.ascontiguousarray(routing_w, np.float32)
    ptrs = (C.c_void_p * len(experts))(*[pool.bytes.ctypes.data + e * pool.stride for e in experts])
    y = np.empty(pool.d, np.float32)
    lib().ffo_apply_streamed_routed(ptrs, C.byref(pool.offsets), pool.d, pool.f, _p(x), _p(residual),
                                    _p(routing_w), len(experts), _p(y))
    return y


def route_partials(pool: ExpertPool, pairs: np.ndarray, hidden_bits: np.ndarray, hidden_stride: int,
                   t: int, top_k: int, dtype: int, fill=None, threads: int = 0) -> np.ndarray:
    pairs = np.ascontiguousarray(pairs, PAIR_DTYPE)
    hidden_bits = np.ascontiguousarray(hidden_bits, np.uint16)
    if dtype == F32:
        out = np.zeros(t * top_k * pool.d, np.float32) if fill is None else np.full(t * top_k * pool.d, fill, np.float32)
    else:
        out = np.zeros(t * top_k * pool.d, np.uint16)
        if fill is not None:
            out[:] = bits16(np.float32(fill), dtype)
    lib().ffo_route_partials(_p(pairs), pairs.size, _p(pool.bytes), pool.stride, C.byref(pool.offsets),
                             _p(hidden_bits), hidden_stride, top_k, pool.d, pool.f, dtype, _p(out), threads)
    return out.reshape(t, top_k, pool.d)


def reduce_token_major(partials: np.ndarray, partial_dtype: int, weight_bits: np.ndarray, dtype: int) -> np.ndarray:
    t, k, d = partials.shape
    partials = np.ascontiguousarray(partials)
    weight_bits = np.ascontiguousarray(weight_bits, np.uint16)
    h2 = np.empty((t, d), np.uint16)
    lib().ffo_reduce_token_major(_p(partials), partial_dtype, _p(weight_bits), dtype, t, k, d, _p(h2))
    return h2


def router_logits_pinned(W, x_bits, dtype: int = BF16, es_bits=None) -> np.ndarray:
    """W: uint16 bf16 bits [E][D] or float32 [E][D]; x_bits uint16 [D]."""
    W = np.ascontiguousarray(W)
    is_f32 = 1 if W.dtype == np.float32 else 0
    e, d = W.shape
    x_bits = np.ascontiguousarray(x_bits, np.uint16)
    es = None if es_bits is None else np.ascontiguousarray(es_bits, np.uint16)
    out = np.empty(e, np.float32)
    lib().ffo_router_logits_pinned(_p(W), is_f32, _p(x_bits), dtype, None if es is None else _p(es), e, d, _p(out))
    return out


def topk_softmax(logits, top_k: int = 8, per_expert_scale_bits=None):
    logits = np.ascontiguousarray(logits, np.float32)
    pes = None if per_expert_scale_bits is None else np.ascontiguousarray(per_expert_scale_bits, np.uint16)
    idx = np.zeros(top_k, np.uint32)
    w = np.zeros(top_k, np.float32)
    lib().ffo_topk_softmax(_p(logits), logits.size, top_k, None if pes is None else _p(pes), _p(idx), _p(w))
    return idx, w


def greedy_choice_rows(logits, softcap: float = 0.0):
    """argmax_rows_f32 (Metal/Sampling/logit.metal:946-1010) on rows of fp32 logits [R][V]: per row the position of the
    largest finite value (ties to the lowest position; 0xFFFFFFFF when no value is finite) and that value's softmax
    probability over the finite values, each capped to softcap * tanh(v / softcap) when softcap > 0 (:978,1001-1002;
    0 when there is no winner). The sums run in float64 here; the kernel's float32 order is its own, so probabilities
    are compared to a tolerance."""
    logits = np.atleast_2d(np.asarray(logits, np.float32))
    tokens = np.empty(logits.shape[0], np.uint32)
    conf = np.zeros(logits.shape[0], np.float64)
    for r, row in enumerate(logits):
        finite = np.isfinite(row)
        if not finite.any():
            tokens[r] = 0xFFFFFFFF
            continue
        best = int(np.flatnonzero(finite & (row == row[finite].max()))[0])
        tokens[r] = best
        v = row[finite].astype(np.float64)
        c = softcap * np.tanh(v / softcap) if softcap > 0 else v
        cb = softcap * np.tanh(np.float64(row[best]) / softcap) if softcap > 0 else np.float64(row[best])
        conf[r] = np.exp(cb - c.max()) / np.exp(c - c.max()).sum()
    return tokens, conf


def sample_gumbel(seed: int, key: int, tokens) -> np.ndarray:
    """sample_gumbel (Metal/Sampling/logit.metal:1042-1051): standard Gumbel noise per token from one SplitMix64 step of
    the state seed ^ key * 0x9E3779B97F4A7C15 ^ token * 0xD1B54A32D192ED03; the output's top 24 bits (+ 0.5) / 2^24 are
    the uniform. float32 throughout, as the kernel computes it."""
    mask = (1 << 64) - 1
    out = np.empty(len(tokens), np.float32)
    for n, tok in enumerate(np.asarray(tokens, np.uint64)):
        z = (seed ^ ((key * 0x9E3779B97F4A7C15) & mask) ^ ((int(tok) * 0xD1B54A32D192ED03) & mask)) & mask
        z = (z + 0x9E3779B97F4A7C15) & mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        z ^= z >> 31
        u = np.float32((np.float32(z >> 40) + np.float32(0.5)) * np.float32(1.0 / 16777216.0))
        out[n] = -np.log(-np.log(u, dtype=np.float32), dtype=np.float32)
    return out


def sample_rows(logits, temperature: float, top_p: float, top_k: int, key_base: int, softcap: float, seed: int,
                ids=None, key_offset: int = 0):
    """sample_rows_f32 (Metal/Sampling/logit.metal:1010-1259) on rows of fp32 logits [R][V]: per row the position drawn by
    the Gumbel-max rule over the entries the truncation keeps, its probability among them, and - for tests - the gap
    between the winning and the second perturbed score (a draw whose gap is within float rounding may fall either
    way on another machine's log / tanh). Truncation as the kernel's: the top_k largest capped logits by (value
    descending, index ascending) when 0 < top_k < V, of those the shortest prefix whose T = 1 mass (relative to ALL
    finite entries) reaches top_p, the draw at temperature T over the survivors. The noise key of row r is key_base +
    key_offset + r; entry i's token is ids[i] when ids are given. Normalisers are summed in float64 here."""
    logits = np.atleast_2d(np.asarray(logits, np.float32))
    rows, count = logits.shape
    tokens = np.full(rows, 0xFFFFFFFF, np.uint32)
    prob = np.zeros(rows, np.float64)
    gap = np.full(rows, np.inf, np.float64)
    cap, inv_t = np.float32(softcap), np.float32(1.0) / np.float32(temperature)
    for r in range(rows):
        row = logits[r]
        finite = np.isfinite(row)
        if not finite.any():
            continue
        pos = np.flatnonzero(finite)
        c = (cap * np.tanh(row[pos] / cap, dtype=np.float32)).astype(np.float32)
        key = (key_base + key_offset + r) & 0xFFFFFFFF
        if 0 < top_k < count:
            order = np.lexsort((pos, -c.astype(np.float64)))[:top_k]          # value descending, then index ascending
            total1 = np.exp(c.astype(np.float64) - float(cap)).sum()
            cum, keep = 0.0, 0
            while keep < len(order):
                cum += float(np.exp(np.float32(c[order[keep]] - cap), dtype=np.float32)) / total1
                keep += 1
                if np.float32(cum) >= np.float32(top_p):
                    break
            order = order[:max(keep, 1)]
            pos, c = pos[order], c[order]
        tok = pos if ids is None else np.asarray(ids, np.uint32)[pos]
        g = (c * inv_t).astype(np.float32) + sample_gumbel(seed, key, tok)
        best = int(np.flatnonzero(g == g.max())[0])                           # ties: the first in (rank or index) order
        tokens[r] = pos[best]
        e = np.exp((c.astype(np.float64) - float(c.max())) * float(inv_t))
        prob[r] = e[best] / e.sum()
        if len(g) > 1:
            rest = np.delete(g, best)
            gap[r] = float(g[best]) - float(rest.max())
    return tokens, prob, gap


def moe_layer(pool: ExpertPool, router_w_bits, x_bits, top_k: int = 8, dtype: int = BF16, threads: int = 0):
    """Router + top-k + experts + combine in fp32-reference mode. Returns (idx [T][K], w f32 [T][K], y f32 [T][D])."""
    x_bits = np.ascontiguousarray(x_bits, np.uint16)
    router_w_bits = np.ascontiguousarray(router_w_bits, np.uint16)
    t, stride = x_bits.shape
    idx = np.zeros((t, top_k), np.uint32)
    w = np.zeros((t, top_k), np.float32)
    y = np.zeros((t, pool.d), np.float32)
    lib().ffo_moe_layer(_p(pool.bytes), pool.stride, C.byref(pool.offsets), router_w_bits.shape[0], pool.d, pool.f,
                        _p(router_w_bits), _p(x_bits), stride, t, top_k, dtype, _p(idx), _p(w), _p(y), threads)
    return idx, w, y


def moe_experts(pool: ExpertPool, x_bits, idx, w, dtype: int = BF16, threads: int = 0) -> np.ndarray:
    x_bits = np.ascontiguousarray(x_bits, np.uint16)
    idx = np.ascontiguousarray(idx, np.uint32)
    w = np.ascontiguousarray(w, np.float32)
    t, stride = x_bits.shape
    y = np.zeros((t, pool.d), np.float32)
    lib().ffo_moe_experts(_p(pool.bytes), pool.stride, C.byref(pool.offsets), pool.d, pool.f, _p(x_bits), stride,
                          t, idx.shape[1], dtype, _p(idx), _p(w), _p(y), threads)
    return y


def post_attn_setup(hidden_bits, attn_bits, w_post_attn, w_pre_ffn, w_pre_ffn2, eps: float = 1e-6, dtype: int = BF16):
    """Rows [T, D] of 16-bit patterns -> (hidden, dense_x, routed_x, router_x), each [T, D]; hidden is the updated copy."""
    hidden = np.array(hidden_bits, np.uint16, ndmin=2, copy=True)
    attn = np.ascontiguousarray(np.array(attn_bits, np.uint16, ndmin=2))
    ws = [np.ascontiguousarray(w, np.uint16) for w in (w_post_attn, w_pre_ffn, w_pre_ffn2)]
    t, d = hidden.shape
    outs = [np.empty((t, d), np.uint16) for _ in range(3)]
    for r in range(t):
        lib().ffo_post_attn_setup(_p(hidden[r]), _p(attn[r]), _p(outs[0][r]), _p(outs[1][r]), _p(outs[2][r]),
                                  _p(ws[0]), _p(ws[1]), _p(ws[2]), d, eps, dtype)
    return hidden, outs[0], outs[1], outs[2]


def rmsnorm(x_bits, w_bits, eps: float = 1e-6, dtype: int = BF16) -> np.ndarray:
    """Rows [T, D] of 16-bit patterns, bf16 weight [D] -> normalised rows."""
    x = np.ascontiguousarray(np.array(x_bits, np.uint16, ndmin=2))
    w = np.ascontiguousarray(w_bits, np.uint16)
    out = np.empty_like(x)
    for r in range(x.shape[0]):
        lib().ffo_rmsnorm(_p(x[r]), _p(w), _p(out[r]), x.shape[1], eps, dtype)
    return out


def layer_tail(h2_bits, h1_bits, hidden_bits, w_postffn2, w_postffn, layer_scalar: float, eps: float = 1e-6,
               dtype: int = BF16) -> np.ndarray:
    """Rows [T, D] of 16-bit patterns -> the updated hidden rows."""
    hidden = np.array(hidden_bits, np.uint16, ndmin=2, copy=True)
    h2 = np.ascontiguousarray(np.array(h2_bits, np.uint16, ndmin=2))
    h1 = np.ascontiguousarray(np.array(h1_bits, np.uint16, ndmin=2))
    w2, w1 = np.ascontiguousarray(w_postffn2, np.uint16), np.ascontiguousarray(w_postffn, np.uint16)
    t, d = hidden.shape
    for r in range(t):
        lib().ffo_layer_tail(_p(h2[r]), _p(h1[r]), _p(hidden[r]), _p(w2), _p(w1), d, eps, layer_scalar, dtype)
    return hidden


def max_threads() -> int:
    return int(lib().ffo_max_threads())


# ----------------------------------------------------------------------------- host integer logic
def make_token_expert_pairs(indices, weight_bits, query_count: int, top_k: int) -> np.ndarray:
    """PrefillRouter.makeTokenExpertPairs, Kernels/Prefill/MoE/PrefillRouter.swift:75-95 (token-major)."""
    indices = np.asarray(indices, np.uint32).reshape(query_count, top_k)
    weight_bits = np.asarray(weight_bits, np.uint16).reshape(query_count, top_k)
    pairs = np.zeros(query_count * top_k, PAIR_DTYPE)
    pairs["token"] = np.repeat(np.arange(query_count, dtype=np.uint32), top_k)
    pairs["rank"] = np.tile(np.arange(top_k, dtype=np.uint32), query_count)
    pairs["expert"] = indices.ravel()
    pairs["weight_bits"] = weight_bits.ravel()
    return pairs


def group_token_expert_pairs(pairs: np.ndarray, num_experts: int, tile_expert_count: int, sort_keys=None):
    """PrefillMoEGrouping.groupTokenExpertPairs, Kernels/Prefill/MoE/PrefillMoEGrouping.swift:49-110.
    Returns (sorted_pairs, groups [(expert, pairStart, pairCount)], tiles [(groupStart, groupCount, pairStart, pairCount)])."""
    pairs = np.asarray(pairs, PAIR_DTYPE)
    bad = pairs["expert"][pairs["expert"] >= num_experts]
    if bad.size:
        raise ValueError(f"route expert {int(bad[0])} is out of range")
    items = [tuple(int(v) for v in p) for p in pairs]
    if sort_keys is None:
        key = lambda p: (p[1], p[0], p[2])
    else:
        key = lambda p: (int(sort_keys[p[1]]), p[1], p[0], p[2])
    items.sort(key=key)
    sorted_pairs = np.array(items, PAIR_DTYPE) if items else np.zeros(0, PAIR_DTYPE)
    groups, i = [], 0
    while i < len(items):
        e, start = items[i][1], i
        while i < len(items) and items[i][1] == e:
            i += 1
        groups.append((e, start, i - start))
    tiles, gs = [], 0
    while gs < len(groups):
        ge = min(len(groups), gs + tile_expert_count)
        first, last = groups[gs], groups[ge - 1]
        tiles.append((gs, ge - gs, first[1], last[1] + last[2] - first[1]))
        gs = ge
    return sorted_pairs, groups, tiles
