"""ctypes binding of libfieldfare_moe_hip.so (the C ABI in include/fieldfare_moe.h).

PyTorch is used for device memory and streams only: every method takes torch CUDA tensors, passes
their raw device pointers through the C ABI, and enqueues on torch's current stream. There is no CPU
or eager fallback: a missing library raises at import of the symbols, a missing GPU at Context().
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

_PKG = Path(__file__).resolve().parent.parent
LIB_PATH = _PKG / "libfieldfare_moe_hip.so"
CSRC = _PKG / "csrc"

OK = 0
GATE, UP, DOWN = 0, 1, 2
GROUP = 64
MAX_VERIFY_ROWS = 16
PREFILL_TILE_M = 256      # FFMOE_PREFILL_TILE_M


class FieldfareError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"ffmoe status {code}: {message}")
        self.code = code
        self.message = message


class Shape(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("d", "f", "n_experts", "top_k", "n_layers", "max_tokens")]


class Offsets(C.Structure):
    """MoEExpertOffsets (Kernels/MoE/MoE.swift:4-29)."""
    _fields_ = [(n, C.c_uint32) for n in
                ("gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b")]


BF16, FP16 = 0, 1     # FFMOE_BF16, FFMOE_FP16

EXPORTS = [
    "ffmoe_version", "ffmoe_create", "ffmoe_destroy", "ffmoe_layer_arena_bytes", "ffmoe_upload_layer",
    "ffmoe_upload_router_bf16", "ffmoe_upload_router_int8", "ffmoe_dequant_expert", "ffmoe_router",
    "ffmoe_verify", "ffmoe_verify_partials", "ffmoe_last_live_experts", "ffmoe_handover_giveups", "ffmoe_probe_stream", "ffmoe_reduce_token_major",
    "ffmoe_gemv_int4", "ffmoe_set_profiling", "ffmoe_get_profile", "ffmoe_prefill", "ffmoe_prefill_pairs",
    "ffmoe_prefill_plan_stats", "ffmoe_matrix_create", "ffmoe_matrix_destroy", "ffmoe_matrix_gemv",
    "ffmoe_matrix_greedy", "ffmoe_matrix_greedy_conf", "ffmoe_argmax_rows", "ffmoe_upload_expert_parts", "ffmoe_dense_ffn", "ffmoe_post_attn_setup",
    "ffmoe_layer_tail", "ffmoe_layer_tail_routed", "ffmoe_route_verify", "ffmoe_set_handover_timeout", "ffmoe_set_one_launch_routing", "ffmoe_gemv_int4_listed",
    "ffmoe_layer_tail_norms", "ffmoe_rmsnorm", "ffmoe_set_activation_dtype", "ffmoe_prefill_dump_tiles",
    "ffmoe_verify_static", "ffmoe_route_verify_shared", "ffmoe_layer_tail_routed_shared", "ffmoe_sample_rows",
    "ffmoe_matrix_create_int8", "ffmoe_matrix_create_int8_glu", "ffmoe_gelu_mul", "ffmoe_upload_expert_parts_int8", "ffmoe_matrix_rows",
]

PROFILE_SLOTS = 16
KERNEL_NAMES = ["router_logits", "router_topk", "plan", "gate_up", "down", "combine", "prefill_sort",
                "prefill_gate_up", "prefill_down", "prefill_combine", "gemv", "argmax", "event_gap", "route_gate_up",
                "probe_gate_up", "probe_down"]


class Projection(C.Structure):
    """SharedExpertProjection: W uint8 [rows][cols/2], S/B bf16 [rows][cols/64] (Kernels/MoE/SharedExpertInt4.swift:32-40)."""
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p)]


class Sampling(C.Structure):
    """ffmoe_sampling: TokenSampling + the position key of LMHeadChainInt4.RowSampling (LMHeadChainInt4.swift:183-190)."""
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("top_k", C.c_uint32), ("key_base", C.c_uint32),
                ("softcap", C.c_float), ("seed", C.c_uint64)]


class Profile(C.Structure):
    _fields_ = [("ms", C.c_double * PROFILE_SLOTS), ("launches", C.c_uint64 * PROFILE_SLOTS)]


class Matrix:
    """ffmoe_matrix: the LM head (or any static INT4 weight) kept re-tiled in HBM."""

    def __init__(self, ctx, W, S, B, greedy: bool, w_byte_offset: int = 0, int8: bool = False, up=None):
        """`up` = (W, S, B) of an up projection makes W, S, B the gate of a gated 8-bit pair: gemv then returns
        round16(gelu_tanh(gate x) * up x)."""
        import numpy as np
        self.ctx, self.L = ctx, ctx.L
        self.m, self.n = int(S.shape[0]), int(S.shape[1]) * GROUP
        self.int8 = int8 or up is not None
        keep = []

        def raw(a, off=0):
            if isinstance(a, np.ndarray):
                a = np.ascontiguousarray(a)
                keep.append(a)
                return C.c_void_p(a.ctypes.data + off)
            keep.append(a)
            return C.c_void_p(a.data_ptr() + off)

        h, err = C.c_void_p(), C.c_char_p()
        if up is not None:
            _check(self.L.ffmoe_matrix_create_int8_glu(ctx._h, raw(W), raw(S), raw(B), raw(up[0]), raw(up[1]), raw(up[2]), self.m,
                                                       self.n, C.byref(h), C.byref(err)), err)
        elif int8:
            _check(self.L.ffmoe_matrix_create_int8(ctx._h, raw(W, w_byte_offset), raw(S), raw(B), self.m, self.n,
                                                   C.byref(h), C.byref(err)), err)
        else:
            _check(self.L.ffmoe_matrix_create(ctx._h, raw(W, w_byte_offset), raw(S), raw(B), self.m, self.n, int(greedy),
                                              C.byref(h), C.byref(err)), err)
        self._h = h

    def gemv(self, x, f32_out: bool = False, out=None):
        import torch
        rows = x.shape[0]
        y = torch.empty((rows, self.m), dtype=torch.float32 if f32_out else self.ctx.act, device=x.device) if out is None else out
        err = C.c_char_p()
        _check(self.L.ffmoe_matrix_gemv(self._h, _stream(), _ptr(x), _row_stride(x), rows, _ptr(y), _row_stride(y),
                                        int(f32_out), C.byref(err)), err)
        return y

    def rows(self, ids, out_scale: float = 1.0, out=None):
        """Dequantised rows `ids` (an int or an int32 / uint32 CUDA tensor) times out_scale: [count, N] of the activation type."""
        import torch
        single = isinstance(ids, int)
        count = 1 if single else int(ids.shape[0])
        y = torch.empty((count, self.n), dtype=self.ctx.act, device="cuda") if out is None else out
        err = C.c_char_p()
        _check(self.L.ffmoe_matrix_rows(self._h, _stream(), None if single else _ptr(ids), count, ids if single else 0,
                                        out_scale, _ptr(y), _row_stride(y), C.byref(err)), err)
        return y

    def greedy(self, x):
        import torch
        rows = x.shape[0]
        out = torch.empty((rows,), dtype=torch.int32, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_matrix_greedy(self._h, _stream(), _ptr(x), _row_stride(x), rows, _ptr(out), C.byref(err)),
               err)
        return out

    def greedy_conf(self, x, softcap: float = 0.0):
        """(tokens int32 [rows], confidence fp32 [rows]): the greedy choice and its softmax probability under the softcap."""
        import torch
        rows = x.shape[0]
        out = torch.empty((rows,), dtype=torch.int32, device=x.device)
        conf = torch.empty((rows,), dtype=torch.float32, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_matrix_greedy_conf(self._h, _stream(), _ptr(x), _row_stride(x), rows, softcap, _ptr(out), _ptr(conf),
                                               C.byref(err)), err)
        return out, conf

    def close(self):
        if self._h:
            self.L.ffmoe_matrix_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


HASH_PATH = LIB_PATH.with_suffix(".so.srchash")


def source_hash() -> str:
    """Digest of everything the library is compiled from (kernels, headers, Makefile, the C header)."""
    import hashlib
    h = hashlib.sha256()
    files = sorted(p for p in CSRC.iterdir() if p.suffix in (".hip", ".hpp") or p.name == "Makefile")
    for p in files + [_PKG.parent / "include" / "fieldfare_moe.h"]:
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()


def is_stale() -> bool:
    """True when no library is built or the sources changed since it was (file times do not survive a copy of the tree,
    so the build leaves a digest of its sources beside the library)."""
    return not (LIB_PATH.exists() and HASH_PATH.exists() and HASH_PATH.read_text().strip() == source_hash())


def build(force: bool = True) -> Path:
    """Compile the library for gfx950 with the Makefile in csrc/ (hipcc cross-compiles without a GPU). `force` recompiles
    every source; otherwise make rebuilds what its dependencies say changed. A failed build raises with the compiler's
    messages."""
    cmd = ["make", "-C", str(CSRC), "-j8"] + (["-B"] if force else [])
    run = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if run.returncode != 0:
        raise RuntimeError(f"building {LIB_PATH.name} failed ({' '.join(cmd)}):\n{run.stdout[-6000:]}")
    HASH_PATH.write_text(source_hash() + "\n")
    return LIB_PATH


def ensure_built() -> Path:
    """Load what is built in-tree; compile only when nothing is, or when the sources are newer than the library."""
    if is_stale():
        build(force=not LIB_PATH.exists())
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise FileNotFoundError(f"{LIB_PATH} is not built; run __graft_entry__.build() (there is no fallback path)")
    if is_stale():
        raise RuntimeError(f"{LIB_PATH} was built from other sources than the ones in {CSRC}; run __graft_entry__.build() "
                           "or fieldfare_moe.ensure_built()")
    # torch ships its own HIP runtime: it has to be in the process before this library resolves
    # libamdhip64, or two runtimes end up loaded and the second one finds no device
    import torch  # noqa: F401
    L = C.CDLL(str(LIB_PATH))
    vp, u32, sz, i32 = C.c_void_p, C.c_uint32, C.c_size_t, C.c_int
    errp = C.POINTER(C.c_char_p)
    L.ffmoe_version.restype = C.c_char_p
    L.ffmoe_create.argtypes = [i32, C.POINTER(Shape), C.POINTER(vp), errp]
    L.ffmoe_destroy.argtypes = [vp]
    L.ffmoe_destroy.restype = None
    L.ffmoe_layer_arena_bytes.argtypes = [vp]
    L.ffmoe_layer_arena_bytes.restype = sz
    L.ffmoe_upload_layer.argtypes = [vp, u32, vp, sz, C.POINTER(Offsets), i32, errp]
    L.ffmoe_upload_router_bf16.argtypes = [vp, u32, vp, vp, vp, errp]
    L.ffmoe_upload_router_int8.argtypes = [vp, u32, vp, vp, vp, vp, vp, errp]
    L.ffmoe_dequant_expert.argtypes = [vp, vp, u32, u32, i32, vp, errp]
    L.ffmoe_prefill_dump_tiles.argtypes = [vp, vp, u32, u32, i32, vp, sz, errp]
    L.ffmoe_router.argtypes = [vp, vp, u32, vp, u32, u32, vp, vp, vp, errp]
    L.ffmoe_verify.argtypes = [vp, vp, u32, vp, u32, u32, vp, vp, vp, vp, errp]
    L.ffmoe_verify_static.argtypes = [vp, vp, u32, vp, u32, u32, vp, vp, vp, vp, errp]
    L.ffmoe_verify_partials.argtypes = [vp, vp, u32, vp, u32, u32, vp, vp, vp, errp]
    L.ffmoe_route_verify.argtypes = [vp, vp, u32, vp, u32, vp, u32, u32, vp, vp, vp, vp, errp]
    L.ffmoe_set_handover_timeout.argtypes = [vp, vp, C.c_uint64, errp]
    L.ffmoe_set_one_launch_routing.argtypes = [vp, C.c_int, errp]
    L.ffmoe_last_live_experts.argtypes = [vp, vp, C.POINTER(u32), errp]
    L.ffmoe_handover_giveups.argtypes = [vp, vp, C.POINTER(u32), errp]
    L.ffmoe_probe_stream.argtypes = [vp, vp, u32, u32, errp]
    L.ffmoe_reduce_token_major.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32, errp]
    L.ffmoe_gemv_int4.argtypes = [vp, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, i32, errp]
    L.ffmoe_layer_tail_norms.argtypes = [vp, vp, vp, u32, vp, u32, vp, u32, vp, vp, vp, vp, vp, u32, u32, u32, C.c_float,
                                         C.c_float, errp]
    L.ffmoe_set_activation_dtype.argtypes = [vp, C.c_int, errp]
    L.ffmoe_rmsnorm.argtypes = [vp, vp, vp, u32, vp, vp, u32, u32, u32, C.c_float, errp]
    L.ffmoe_gemv_int4_listed.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, errp]
    L.ffmoe_set_profiling.argtypes = [vp, i32, errp]
    L.ffmoe_get_profile.argtypes = [vp, C.POINTER(Profile), i32, errp]
    L.ffmoe_prefill.argtypes = [vp, vp, u32, vp, u32, u32, vp, vp, vp, errp]
    L.ffmoe_prefill_pairs.argtypes = [vp, vp, u32, vp, u32, vp, u32, u32, vp, errp]
    L.ffmoe_prefill_plan_stats.argtypes = [vp, vp, C.POINTER(u32), C.POINTER(u32), vp, errp]
    L.ffmoe_matrix_create.argtypes = [vp, vp, vp, vp, u32, u32, i32, C.POINTER(vp), errp]
    L.ffmoe_matrix_create_int8.argtypes = [vp, vp, vp, vp, u32, u32, C.POINTER(vp), errp]
    L.ffmoe_matrix_rows.argtypes = [vp, vp, vp, u32, u32, C.c_float, vp, u32, errp]
    L.ffmoe_matrix_create_int8_glu.argtypes = [vp, vp, vp, vp, vp, vp, vp, u32, u32, C.POINTER(vp), errp]
    L.ffmoe_gelu_mul.argtypes = [vp, vp, vp, u32, vp, u32, vp, u32, u32, u32, errp]
    L.ffmoe_matrix_destroy.argtypes = [vp]
    L.ffmoe_matrix_destroy.restype = None
    L.ffmoe_matrix_gemv.argtypes = [vp, vp, vp, u32, u32, vp, u32, i32, errp]
    L.ffmoe_matrix_greedy.argtypes = [vp, vp, vp, u32, u32, vp, errp]
    L.ffmoe_matrix_greedy_conf.argtypes = [vp, vp, vp, u32, u32, C.c_float, vp, vp, errp]
    L.ffmoe_argmax_rows.argtypes = [vp, vp, vp, u32, u32, u32, C.c_float, vp, vp, errp]
    L.ffmoe_upload_expert_parts.argtypes = [vp, u32, u32, C.POINTER(Projection), C.POINTER(Projection),
                                            C.POINTER(Projection), i32, errp]
    L.ffmoe_upload_expert_parts_int8.argtypes = [vp, u32, C.POINTER(Projection), C.POINTER(Projection), C.POINTER(Projection), errp]
    L.ffmoe_dense_ffn.argtypes = [vp, vp, u32, vp, u32, u32, vp, errp]
    L.ffmoe_post_attn_setup.argtypes = [vp, vp, vp, u32, vp, u32, vp, u32, vp, u32, vp, u32, vp, vp, vp, u32, u32,
                                        C.c_float, errp]
    L.ffmoe_layer_tail.argtypes = [vp, vp, vp, u32, vp, u32, vp, u32, vp, vp, u32, u32, C.c_float, C.c_float, errp]
    L.ffmoe_layer_tail_routed.argtypes = [vp, vp, vp, vp, u32, vp, u32, vp, vp, u32, C.c_float, C.c_float, errp]
    L.ffmoe_sample_rows.argtypes = [vp, vp, vp, u32, u32, u32, vp, C.POINTER(Sampling), vp, vp, vp, errp]
    L.ffmoe_route_verify_shared.argtypes = [vp, vp, vp, u32, u32, vp, u32, vp, u32, vp, u32, u32, vp, vp, errp]
    L.ffmoe_layer_tail_routed_shared.argtypes = [vp, vp, vp, vp, vp, u32, vp, vp, u32, C.c_float, C.c_float, errp]
    _lib = L
    return L


def _check(code: int, err: C.c_char_p):
    if code != OK:
        msg = err.value.decode() if err.value else "(no message)"
        raise FieldfareError(code, msg)


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _row_stride(t):
    """Row stride in elements; a single-row tensor may report any stride for its size-1 dimension."""
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class Context:
    """One ffmoe_ctx: the HBM expert arena of `n_layers` layers plus scratch, on one GPU."""

    def __init__(self, d: int, f: int, n_experts: int, top_k: int = 8, n_layers: int = 1, max_tokens: int = 4096,
                 device: int = 0, act_dtype: str = "bf16"):
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("no HIP device visible: the fieldfare MoE kernels have no CPU fallback")
        if act_dtype not in ("bf16", "fp16"):
            raise ValueError("act_dtype is 'bf16' or 'fp16'")
        self.L = lib()
        self.shape = Shape(d, f, n_experts, top_k, n_layers, max_tokens)
        self.device = device
        self.act = torch.bfloat16 if act_dtype == "bf16" else torch.float16    # type of every 16-bit row in and out
        self._h = C.c_void_p()
        err = C.c_char_p()
        _check(self.L.ffmoe_create(device, C.byref(self.shape), C.byref(self._h), C.byref(err)), err)
        if act_dtype == "fp16":
            _check(self.L.ffmoe_set_activation_dtype(self._h, FP16, C.byref(err)), err)

    def set_act_dtype(self, act_dtype: str):
        """Switch the type of every 16-bit row in and out ('bf16' or 'fp16'); waits for the device."""
        import torch
        if act_dtype not in ("bf16", "fp16"):
            raise ValueError("act_dtype is 'bf16' or 'fp16'")
        err = C.c_char_p()
        _check(self.L.ffmoe_set_activation_dtype(self._h, FP16 if act_dtype == "fp16" else BF16, C.byref(err)), err)
        self.act = torch.bfloat16 if act_dtype == "bf16" else torch.float16

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            self.L.ffmoe_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def layer_arena_bytes(self) -> int:
        return int(self.L.ffmoe_layer_arena_bytes(self._h))

    # -- per-kernel timing -----------------------------------------------------------------------
    def set_profiling(self, enabled: bool):
        err = C.c_char_p()
        _check(self.L.ffmoe_set_profiling(self._h, int(enabled), C.byref(err)), err)

    def profile(self, reset: bool = True) -> dict:
        """{kernel: (total ms, launches)} accumulated while profiling was enabled."""
        p = Profile()
        err = C.c_char_p()
        _check(self.L.ffmoe_get_profile(self._h, C.byref(p), int(reset), C.byref(err)), err)
        return {KERNEL_NAMES[i]: (p.ms[i], int(p.launches[i])) for i in range(PROFILE_SLOTS) if p.launches[i]}

    # -- weights ---------------------------------------------------------------------------------
    def upload_layer(self, layer: int, blobs, stride: int, offsets: Offsets):
        """`blobs`: torch uint8 tensor (CPU or CUDA) or numpy uint8 array holding n_experts blobs."""
        import numpy as np
        import torch
        err = C.c_char_p()
        if isinstance(blobs, np.ndarray):
            assert blobs.dtype == np.uint8 and blobs.flags["C_CONTIGUOUS"]
            p, on_dev = C.c_void_p(blobs.ctypes.data), 0
        else:
            assert blobs.dtype == torch.uint8 and blobs.is_contiguous()
            p, on_dev = C.c_void_p(blobs.data_ptr()), int(blobs.is_cuda)
        _check(self.L.ffmoe_upload_layer(self._h, layer, p, stride, C.byref(offsets), on_dev, C.byref(err)), err)

    def upload_expert_parts(self, layer: int, expert: int, gate, up, down, int8: bool = False):
        """One expert from three (W uint8, S bf16 bits, B bf16 bits) triples: all numpy arrays or all CUDA tensors.
        int8: the triples hold 8-bit weights (W uint8 [rows, cols]); dense contexts only, expert 0."""
        import numpy as np
        keep, kinds = [], set()

        def proj(triple):
            ptrs = []
            for a in triple:
                if isinstance(a, np.ndarray):
                    a = np.ascontiguousarray(a)
                    ptrs.append(a.ctypes.data)
                    kinds.add(0)
                else:
                    assert a.is_contiguous()
                    ptrs.append(a.data_ptr())
                    kinds.add(int(a.is_cuda))
                keep.append(a)
            return Projection(*ptrs)

        g, u, dn = proj(gate), proj(up), proj(down)
        assert len(kinds) == 1, "all nine arrays must live on the same side"
        err = C.c_char_p()
        if int8:
            assert expert == 0
            _check(self.L.ffmoe_upload_expert_parts_int8(self._h, layer, C.byref(g), C.byref(u), C.byref(dn), C.byref(err)), err)
            return
        _check(self.L.ffmoe_upload_expert_parts(self._h, layer, expert, C.byref(g), C.byref(u), C.byref(dn),
                                                kinds.pop(), C.byref(err)), err)

    def upload_router_bf16(self, layer: int, w_bits, effective_scale_bits=None, per_expert_scale_bits=None):
        """numpy uint16 arrays (bf16 bit patterns), host side."""
        import numpy as np
        err = C.c_char_p()
        keep = [np.ascontiguousarray(a, np.uint16) if a is not None else None
                for a in (w_bits, effective_scale_bits, per_expert_scale_bits)]
        ptrs = [C.c_void_p(a.ctypes.data) if a is not None else None for a in keep]
        _check(self.L.ffmoe_upload_router_bf16(self._h, layer, *ptrs, C.byref(err)), err)

    def upload_router_int8(self, layer: int, w_u8, scale_bits, bias_bits, effective_scale_bits=None,
                           per_expert_scale_bits=None):
        import numpy as np
        err = C.c_char_p()
        keep = [np.ascontiguousarray(w_u8, np.uint8)] + [
            np.ascontiguousarray(a, np.uint16) if a is not None else None
            for a in (scale_bits, bias_bits, effective_scale_bits, per_expert_scale_bits)]
        ptrs = [C.c_void_p(a.ctypes.data) if a is not None else None for a in keep]
        _check(self.L.ffmoe_upload_router_int8(self._h, layer, *ptrs, C.byref(err)), err)

    def dequant_expert(self, layer: int, expert: int, which: int):
        import torch
        rows, cols = (self.shape.d, self.shape.f) if which == DOWN else (self.shape.f, self.shape.d)
        out = torch.empty((rows, cols), dtype=torch.bfloat16, device=f"cuda:{self.device}")
        err = C.c_char_p()
        _check(self.L.ffmoe_dequant_expert(self._h, _stream(), layer, expert, which, _ptr(out), C.byref(err)), err)
        return out

    def prefill_tiles(self, layer: int, expert: int, which: int):
        """The 16-bit weights of one sub-tensor as the grouped GEMM's matrix instructions read them from LDS, put
        back into [rows][cols] order: a CUDA tensor of the context's activation type - bf16(fma(q, s, b)), or
        half(fma(q, s, b)) for a context in FP16 mode (ffmoe_prefill_dump_tiles)."""
        import torch
        d, f = self.shape.d, self.shape.f
        gate_up = which != DOWN
        tiles, groups = (f // 16, d // GROUP) if gate_up else (d // 32, f // GROUP)
        nblocks = (tiles + 3) // 4
        raw = torch.empty((nblocks, groups, 2, 4, 2, 4, 16, 8), dtype=self.act, device=f"cuda:{self.device}")
        err = C.c_char_p()
        _check(self.L.ffmoe_prefill_dump_tiles(self._h, _stream(), layer, expert, int(gate_up), _ptr(raw),
                                               raw.numel() * 2, C.byref(err)), err)
        # raw[nb, g, khalf, tile, stream, kq, r, e]: fragment u = 8 khalf + 2 tile + stream, lane = 16 kq + r
        t = raw.permute(0, 3, 4, 6, 1, 2, 5, 7)          # nb, tile, stream, r, g, khalf, kq, e
        t = t.reshape(nblocks * 4, 2, 16, groups * GROUP)[:tiles]
        if gate_up:
            return t[:, 0 if which == GATE else 1].reshape(f, d).contiguous()
        return t.reshape(d, f).contiguous()              # down rows 32 tile + 16 stream + r

    # -- router ----------------------------------------------------------------------------------
    def router(self, layer: int, router_x, want_logits: bool = False):
        """router_x: bf16 [T, stride>=d] CUDA tensor (rows may be strided). Returns (idx i32 [T,K], w bf16 [T,K][, logits])."""
        import torch
        assert router_x.dtype == self.act and router_x.is_cuda and router_x.stride(1) == 1
        t = router_x.shape[0]
        k, e = self.shape.top_k, self.shape.n_experts
        idx = torch.empty((t, k), dtype=torch.int32, device=router_x.device)
        w = torch.empty((t, k), dtype=self.act, device=router_x.device)
        logits = torch.empty((t, e), dtype=torch.float32, device=router_x.device) if want_logits else None
        err = C.c_char_p()
        _check(self.L.ffmoe_router(self._h, _stream(), layer, _ptr(router_x), _row_stride(router_x), t, _ptr(idx), _ptr(w),
                                   _ptr(logits), C.byref(err)), err)
        return (idx, w, logits) if want_logits else (idx, w)

    # -- routed experts --------------------------------------------------------------------------
    def verify(self, layer: int, x, idx, w, residual=None, out=None):
        """Decode step (T = 1) or verify block (T <= 16): fused experts + weighted combine. x bf16 [T, stride]."""
        import torch
        t = x.shape[0]
        y = out if out is not None else torch.empty((t, self.shape.d), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_verify(self._h, _stream(), layer, _ptr(x), _row_stride(x), t, _ptr(idx), _ptr(w), _ptr(residual),
                                   _ptr(y), C.byref(err)), err)
        return y

    def route_verify(self, layer: int, router_x, x, residual=None, out=None, combine: bool = True):
        """Router + expert pass of a block of <= 16 rows in one call. Returns (y, idx, w); combine=False leaves the
        routes' rows un-combined in the context (y is None) for layer_tail_routed."""
        import torch
        t, k = x.shape[0], self.shape.top_k
        y = None if not combine else out if out is not None else torch.empty((t, self.shape.d), dtype=self.act, device=x.device)
        idx = torch.empty((t, k), dtype=torch.int32, device=x.device)
        w = torch.empty((t, k), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_route_verify(self._h, _stream(), layer, _ptr(router_x), _row_stride(router_x), _ptr(x), _row_stride(x),
                                         t, _ptr(residual), _ptr(y), _ptr(idx), _ptr(w), C.byref(err)), err)
        return y, idx, w

    def route_verify_shared(self, shared: "Context", layer: int, shared_layer: int, router_x, x, shared_x):
        """route_verify(..., combine=False) with the shared expert (the dense context `shared`, on shared_x) inside the
        same two launches. Returns (idx, w); the rows stay in the two contexts for layer_tail_routed_shared."""
        import torch
        t, k = x.shape[0], self.shape.top_k
        idx = torch.empty((t, k), dtype=torch.int32, device=x.device)
        w = torch.empty((t, k), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_route_verify_shared(self._h, shared._h, _stream(), layer, shared_layer, _ptr(router_x),
                                                _row_stride(router_x), _ptr(x), _row_stride(x), _ptr(shared_x),
                                                _row_stride(shared_x), t, _ptr(idx), _ptr(w), C.byref(err)), err)
        return idx, w

    def verify_partials(self, layer: int, x, idx, w, partials=None):
        import torch
        t = x.shape[0]
        if partials is None:
            partials = torch.zeros((t, self.shape.top_k, self.shape.d), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_verify_partials(self._h, _stream(), layer, _ptr(x), _row_stride(x), t, _ptr(idx), _ptr(w),
                                            _ptr(partials), C.byref(err)), err)
        return partials

    def set_handover_timeout(self, ticks: int):
        """Ticks (100 MHz) a wave of route_verify's one-launch form waits for a hand-over word before it computes the
        word's content itself; clears the count handover_giveups() reports."""
        err = C.c_char_p()
        _check(self.L.ffmoe_set_handover_timeout(self._h, _stream(), ticks, C.byref(err)), err)

    def set_one_launch_routing(self, enabled: bool):
        """False: route_verify runs the router as launches of its own (no block waits for another)."""
        err = C.c_char_p()
        _check(self.L.ffmoe_set_one_launch_routing(self._h, int(bool(enabled)), C.byref(err)), err)

    def last_live_experts(self) -> int:
        n = C.c_uint32()
        err = C.c_char_p()
        _check(self.L.ffmoe_last_live_experts(self._h, _stream(), C.byref(n), C.byref(err)), err)
        return int(n.value)

    def probe_stream(self, layer: int, n_live: int):
        """The weight loads of the decode / verify expert kernels for n_live experts and nothing else (a timing probe)."""
        err = C.c_char_p()
        _check(self.L.ffmoe_probe_stream(self._h, _stream(), layer, n_live, C.byref(err)), err)

    def handover_giveups(self) -> int:
        """Waves of route_verify's one-launch form that stopped waiting for another block and helped themselves."""
        n = C.c_uint32()
        err = C.c_char_p()
        _check(self.L.ffmoe_handover_giveups(self._h, _stream(), C.byref(n), C.byref(err)), err)
        return int(n.value)

    def reduce_token_major(self, partials, weights):
        import torch
        t, k, d = partials.shape
        h2 = torch.empty((t, d), dtype=self.act, device=partials.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_reduce_token_major(self._h, _stream(), _ptr(partials), _ptr(weights), _ptr(h2), t, k, d,
                                               C.byref(err)), err)
        return h2

    # -- prefill ---------------------------------------------------------------------------------
    def prefill(self, layer: int, x, idx, w, out=None):
        import torch
        t = x.shape[0]
        y = out if out is not None else torch.empty((t, self.shape.d), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_prefill(self._h, _stream(), layer, _ptr(x), _row_stride(x), t, _ptr(idx), _ptr(w), _ptr(y),
                                    C.byref(err)), err)
        return y

    def dense_ffn(self, layer: int, x, out=None):
        """Shared expert: every row of x through expert 0 with weight 1 (context with n_experts = top_k = 1)."""
        import torch
        t = x.shape[0]
        y = out if out is not None else torch.empty((t, self.shape.d), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_dense_ffn(self._h, _stream(), layer, _ptr(x), _row_stride(x), t, _ptr(y), C.byref(err)), err)
        return y

    def prefill_pairs(self, layer: int, x, sorted_pairs, t: int, partials):
        """Guest contract: sorted_pairs int32 [n, 4] CUDA tensor of (token, expert, rank, weight bits)."""
        err = C.c_char_p()
        _check(self.L.ffmoe_prefill_pairs(self._h, _stream(), layer, _ptr(x), _row_stride(x), _ptr(sorted_pairs),
                                          sorted_pairs.shape[0], t, _ptr(partials), C.byref(err)), err)
        return partials

    def prefill_stats(self):
        """(pairs kept, M-tiles, pairs per expert) of the last prefill call."""
        import numpy as np
        n_pairs, n_tiles = C.c_uint32(), C.c_uint32()
        counts = np.zeros(self.shape.n_experts, np.uint32)
        err = C.c_char_p()
        _check(self.L.ffmoe_prefill_plan_stats(self._h, _stream(), C.byref(n_pairs), C.byref(n_tiles),
                                               C.c_void_p(counts.ctypes.data), C.byref(err)), err)
        return int(n_pairs.value), int(n_tiles.value), counts

    # -- steps either side of the MoE stage ------------------------------------------------------
    def post_attn_setup(self, hidden, attn, w_post_attn, w_pre_ffn, w_pre_ffn2, eps: float = 1e-6, d: int | None = None,
                        out=None):
        """hidden (updated in place), attn: bf16 CUDA tensors [t, >= d] (row stride = their second stride);
        returns (dense_x, routed_x, router_x), each [t, d] unless `out` gives three tensors to fill."""
        import torch
        t = hidden.shape[0]
        d = d or self.shape.d
        outs = out if out is not None else tuple(torch.empty((t, d), dtype=self.act, device=hidden.device) for _ in range(3))
        err = C.c_char_p()
        _check(self.L.ffmoe_post_attn_setup(self._h, _stream(), _ptr(hidden), _row_stride(hidden), _ptr(attn), _row_stride(attn),
                                            _ptr(outs[0]), _row_stride(outs[0]), _ptr(outs[1]), _row_stride(outs[1]),
                                            _ptr(outs[2]), _row_stride(outs[2]), _ptr(w_post_attn), _ptr(w_pre_ffn),
                                            _ptr(w_pre_ffn2), t, d, eps, C.byref(err)), err)
        return outs

    def layer_tail(self, h2, h1, hidden, w_postffn2, w_postffn, layer_scalar: float, eps: float = 1e-6, d: int | None = None):
        """hidden = (hidden + norm(h1 + norm(h2))) * layer_scalar, in place; bf16 CUDA tensors [t, >= d]."""
        t = hidden.shape[0]
        d = d or self.shape.d
        err = C.c_char_p()
        _check(self.L.ffmoe_layer_tail(self._h, _stream(), _ptr(h2), _row_stride(h2), _ptr(h1), _row_stride(h1), _ptr(hidden),
                                       _row_stride(hidden), _ptr(w_postffn2), _ptr(w_postffn), t, d, eps, layer_scalar,
                                       C.byref(err)), err)
        return hidden

    def layer_tail_routed(self, route_w, h1, hidden, w_postffn2, w_postffn, layer_scalar: float, eps: float = 1e-6):
        """layer_tail on the rows the last route_verify(..., combine=False) left un-combined (weights: that call's w)."""
        t = hidden.shape[0]
        err = C.c_char_p()
        _check(self.L.ffmoe_layer_tail_routed(self._h, _stream(), _ptr(route_w), _ptr(h1), _row_stride(h1), _ptr(hidden),
                                              _row_stride(hidden), _ptr(w_postffn2), _ptr(w_postffn), t, eps, layer_scalar,
                                              C.byref(err)), err)
        return hidden

    def layer_tail_routed_shared(self, shared: "Context", route_w, hidden, w_postffn2, w_postffn, layer_scalar: float,
                                 eps: float = 1e-6):
        """layer_tail on the rows the last route_verify_shared left in this context (routed) and in `shared` (h1)."""
        t = hidden.shape[0]
        err = C.c_char_p()
        _check(self.L.ffmoe_layer_tail_routed_shared(self._h, shared._h, _stream(), _ptr(route_w), _ptr(hidden),
                                                     _row_stride(hidden), _ptr(w_postffn2), _ptr(w_postffn), t, eps,
                                                     layer_scalar, C.byref(err)), err)
        return hidden

    def layer_tail_norms(self, h2, h1, hidden, w_postffn1, w_postffn2, w_postffn, layer_scalar: float, w_next=None,
                         eps: float = 1e-6, d: int | None = None):
        """The tail with h1 taken before its post-FFN-1 norm; with w_next also returns the next layer's input norm."""
        import torch
        t = hidden.shape[0]
        d = d or self.shape.d
        normed = torch.empty((t, d), dtype=self.act, device=hidden.device) if w_next is not None else None
        err = C.c_char_p()
        _check(self.L.ffmoe_layer_tail_norms(self._h, _stream(), _ptr(h2), _row_stride(h2), _ptr(h1), _row_stride(h1), _ptr(hidden),
                                             _row_stride(hidden), _ptr(w_postffn1), _ptr(w_postffn2), _ptr(w_postffn), _ptr(w_next),
                                             _ptr(normed), d, t, d, eps, layer_scalar, C.byref(err)), err)
        return normed

    def rmsnorm(self, x, w, eps: float = 1e-6, d: int | None = None, out=None):
        import torch
        t = x.shape[0]
        d = d or self.shape.d
        y = out if out is not None else torch.empty((t, d), dtype=self.act, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_rmsnorm(self._h, _stream(), _ptr(x), _row_stride(x), _ptr(w), _ptr(y), _row_stride(y), t, d, eps,
                                    C.byref(err)), err)
        return y

    # -- generic GEMV ----------------------------------------------------------------------------
    def matrix(self, W, S, B, greedy: bool = False, w_byte_offset: int = 0):
        """Resident re-tiled copy of W uint8 [M, N/2], S/B bf16 bits [M, N/64] (numpy arrays or tensors)."""
        return Matrix(self, W, S, B, greedy, w_byte_offset)

    def matrix_int8(self, W, S, B):
        """Resident copy of an 8-bit affine weight: W uint8 [M, N], S/B bf16 bits [M, N/64] (numpy arrays or tensors)."""
        return Matrix(self, W, S, B, False, 0, int8=True)

    def matrix_int8_glu(self, gate, up):
        """Gate and up projections (each a (W, S, B) triple as matrix_int8 takes them) as one gated matrix."""
        return Matrix(self, gate[0], gate[1], gate[2], False, 0, up=up)

    def gelu_mul(self, gate, up, out=None):
        """out = round16(gelu_tanh(gate) * up), rows of the activation type (2-D tensors of one shape)."""
        import torch
        rows, count = gate.shape
        out = torch.empty((rows, count), dtype=gate.dtype, device=gate.device) if out is None else out
        err = C.c_char_p()
        _check(self.L.ffmoe_gelu_mul(self._h, _stream(), _ptr(gate), _row_stride(gate), _ptr(up), _row_stride(up), _ptr(out),
                                     _row_stride(out), rows, count, C.byref(err)), err)
        return out

    def argmax_rows(self, logits, count: int | None = None, softcap: float = 0.0, want_conf: bool = True):
        """Greedy position per row of fp32 logits [rows, >= count] (int32, -1 when no value is finite) and, with
        want_conf, the winner's softmax probability under the softcap."""
        import torch
        rows = logits.shape[0]
        count = count or logits.shape[1]
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        conf = torch.empty((rows,), dtype=torch.float32, device=logits.device) if want_conf else None
        err = C.c_char_p()
        _check(self.L.ffmoe_argmax_rows(self._h, _stream(), _ptr(logits), _row_stride(logits), rows, count, softcap, _ptr(out),
                                        _ptr(conf), C.byref(err)), err)
        return (out, conf) if want_conf else out

    def sample_rows(self, logits, temperature: float, softcap: float, seed: int, key_base: int = 0, top_k: int = 0,
                    top_p: float = 1.0, ids=None, key_offset=None, count: int | None = None):
        """The sampled choice per row of fp32 logits [rows, >= count]: (position int32 [-1: nothing finite], probability)."""
        import torch
        rows = logits.shape[0]
        count = count or logits.shape[1]
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
        prob = torch.empty((rows,), dtype=torch.float32, device=logits.device)
        rule = Sampling(temperature, top_p, top_k, key_base, softcap, seed)
        err = C.c_char_p()
        _check(self.L.ffmoe_sample_rows(self._h, _stream(), _ptr(logits), _row_stride(logits), rows, count, _ptr(ids),
                                        C.byref(rule), _ptr(key_offset), _ptr(out), _ptr(prob), C.byref(err)), err)
        return out, prob

    def gemv_int4_listed(self, W, S, B, ids, x):
        """GEMV over the weight rows listed in `ids` (int32 CUDA tensor [m]): y fp32 [R, m], y[:, o] = row ids[o]."""
        import torch
        m, n, rows = ids.shape[0], S.shape[1] * GROUP, x.shape[0]
        y = torch.empty((rows, m), dtype=torch.float32, device=x.device)
        err = C.c_char_p()
        _check(self.L.ffmoe_gemv_int4_listed(self._h, _stream(), _ptr(W), _ptr(S), _ptr(B), _ptr(ids), _ptr(x), _ptr(y), m, n,
                                             rows, _row_stride(x), m, C.byref(err)), err)
        return y

    def gemv_int4(self, W, S, B, x, f32_out: bool = False, w_byte_offset: int = 0):
        """W uint8 [M, N/2] (optionally starting `w_byte_offset` bytes into a larger buffer), S/B bf16-bit
        int16/uint16 tensors [M, N/64], x bf16 [R, stride]. Returns y [R, M]."""
        import torch
        m, n = S.shape[0], S.shape[1] * GROUP
        rows = x.shape[0]
        y = torch.empty((rows, m), dtype=torch.float32 if f32_out else self.act, device=x.device)
        err = C.c_char_p()
        wp = C.c_void_p(W.data_ptr() + w_byte_offset)
        _check(self.L.ffmoe_gemv_int4(self._h, _stream(), wp, _ptr(S), _ptr(B), _ptr(x), _ptr(y), m, n, rows,
                                      _row_stride(x), m, int(f32_out), C.byref(err)), err)
        return y
