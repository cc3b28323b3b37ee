"""ffmoe_verify_static (the entry point that allocates nothing: its scratch is a fixed array in the library image)
against ffmoe_verify, through the C ABI, bit for bit: two calls in a row, the second on a smaller block, so that
what the first call left in the shared array is there when the second runs."""
import ctypes as C

import numpy as np
import pytest

from helpers import REAL, REAL_STRIDE, bf16_tensor, bits_of, make_layer, to_ff_offsets

pytestmark = pytest.mark.gpu


def _call(fn, ctx, torch, layer, x, idx, w, residual, y):
    err = C.c_char_p()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = fn(ctx._h, stream, layer, C.c_void_p(x.data_ptr()), x.stride(0) if x.shape[0] > 1 else x.shape[1], x.shape[0],
            C.c_void_p(idx.data_ptr()), C.c_void_p(w.data_ptr()), C.c_void_p(residual.data_ptr()) if residual is not None else None,
            C.c_void_p(y.data_ptr()), C.byref(err))
    assert rc == 0, (rc, err.value)


@pytest.mark.parametrize("shape", ["small", "real"])
def test_static_scratch_verify_equals_verify(oracle, shape):
    import torch
    import fieldfare_moe as ff
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    L = ff.lib()
    if shape == "small":
        d, f, e, stride = 256, 128, 32, None
    else:
        d, f, e, stride = REAL["d"], REAL["f"], REAL["n_experts"], REAL_STRIDE
    rng, pool, router = make_layer(oracle, 77, d, f, e, stride=stride)
    ctx = ff.Context(d, f, e, 8, n_layers=1, max_tokens=64)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    # a second context of the same shape: the call under test runs on `ctx`, whose own scratch a verify on a
    # throw-away block has filled with unrelated rows just before (so a static call that read or wrote the context's
    # allocations instead of the array would give other bits)
    junk = bf16_tensor(torch, oracle.bf16_bits(rng.normal(0, 3, (16, d)).astype(np.float32)))

    def sentinel(c):
        ji, jw = c.router(0, junk)
        c.verify(0, junk, ji, jw)
        torch.cuda.synchronize()
    for t, with_residual in ((16, True), (5, False), (1, True)):     # in a row; each smaller than the one before
        xb = oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))
        x = bf16_tensor(torch, xb)
        idx, w = ctx.router(0, x)
        residual = bf16_tensor(torch, oracle.bf16_bits(rng.normal(0, 1, (t, d)).astype(np.float32))) if with_residual else None
        y_ref = torch.full((t, d), float("nan"), dtype=torch.bfloat16, device="cuda")
        y_new = torch.full((t, d), float("nan"), dtype=torch.bfloat16, device="cuda")
        _call(L.ffmoe_verify, ctx, torch, 0, x, idx, w, residual, y_ref)
        torch.cuda.synchronize()
        # the context's own scratch must play no part in the static call: fill it with a pattern that would show
        sentinel(ctx)
        free_before = torch.cuda.mem_get_info()[0]
        _call(L.ffmoe_verify_static, ctx, torch, 0, x, idx, w, residual, y_new)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the static call changed the free device memory"
        assert np.array_equal(bits_of(y_new), bits_of(y_ref)), (shape, t)
        # and the pair is right, not merely equal: the oracle's fp32 layer on the same routes
        w_np = oracle.bf16_to_float(bits_of(w))
        ref = oracle.moe_experts(pool, xb, idx.cpu().numpy().astype(np.uint32), w_np)
        if residual is not None:
            ref = ref + oracle.bf16_to_float(bits_of(residual))
        got = oracle.bf16_to_float(bits_of(y_new))
        assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max(), (shape, t)
    ctx.close()


def test_static_scratch_rejects_shapes_beyond_its_size(oracle):
    import torch
    import fieldfare_moe as ff
    L = ff.lib()
    d = 6144           # 16 * 8 un-weighted fp32 rows of this width alone take 3 MiB
    ctx = ff.Context(d, 2048, 8, 8, n_layers=1, max_tokens=16)
    x = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((1, 8), dtype=torch.int32, device="cuda")
    w = torch.zeros((1, 8), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    err = C.c_char_p()
    rc = L.ffmoe_verify_static(ctx._h, None, 0, C.c_void_p(x.data_ptr()), d, 1, C.c_void_p(idx.data_ptr()),
                               C.c_void_p(w.data_ptr()), None, C.c_void_p(y.data_ptr()), C.byref(err))
    assert rc == -1 and b"static array holds" in err.value, (rc, err.value)
    ctx.close()
