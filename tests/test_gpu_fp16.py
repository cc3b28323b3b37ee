"""A context in FP16 mode (FFMOE_FP16, the reference's text-path activation type) through the C ABI against
the CPU oracle run with dtype = FP16: router, decode / verify, prefill, per-route rows, GEMV, the steps
either side. Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import REAL, REAL_STRIDE, bits_of, cosine, make_layer, rel_err, to_ff_offsets

pytestmark = pytest.mark.gpu
EPS = 1e-6


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch


@pytest.fixture(scope="module")
def ff():
    import fieldfare_moe
    fieldfare_moe.lib()
    return fieldfare_moe


def f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_float(bits):
    return np.ascontiguousarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


def f16_tensor(torch, bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.float16)


def bf16_tensor(torch, bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.bfloat16)


@pytest.fixture(scope="module")
def small(oracle, ff, torch):
    d, f, e = 128, 64, 16
    rng, pool, router = make_layer(oracle, 11, d, f, e, align=16)
    ctx = ff.Context(d, f, e, 8, n_layers=1, max_tokens=512, act_dtype="fp16")
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    yield dict(pool=pool, router=router, ctx=ctx, d=d, f=f, e=e)
    ctx.close()


@pytest.fixture(scope="module")
def real(oracle, ff, torch):
    rng, pool, router = make_layer(oracle, 0, REAL["d"], REAL["f"], REAL["n_experts"], stride=REAL_STRIDE)
    ctx = ff.Context(REAL["d"], REAL["f"], REAL["n_experts"], 8, n_layers=1, max_tokens=256, act_dtype="fp16")
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    yield dict(pool=pool, router=router, ctx=ctx, **REAL)
    ctx.close()


def test_unknown_dtype_is_an_error(ff, torch):
    ctx = ff.Context(128, 64, 4, 2, n_layers=1, max_tokens=16)
    import ctypes as C
    err = C.c_char_p()
    assert ctx.L.ffmoe_set_activation_dtype(ctx._h, 7, C.byref(err)) == -1 and b"neither" in err.value
    ctx.close()
    with pytest.raises(ValueError):
        ff.Context(128, 64, 4, 2, act_dtype="fp32")


@pytest.mark.parametrize("which,t", [("small", 1), ("small", 16), ("small", 37), ("real", 16), ("real", 130)])
def test_router_fp16_rows_bit_exact(small, real, oracle, torch, which, t):
    # FP16 rows widen to fp32 exactly: the logits keep the pinned order bit for bit, the routes are the
    # oracle's, the weights are FP16 roundings of the same softmax
    fx = small if which == "small" else real
    rng = np.random.default_rng(500 + t)
    xb = f16_bits(rng.normal(0, 1, (t, fx["d"])))
    idx, w, logits = fx["ctx"].router(0, f16_tensor(torch, xb), want_logits=True)
    assert w.dtype == torch.float16
    logits = logits.cpu().numpy()
    for tok in range(t):
        ref = oracle.router_logits_pinned(fx["router"], xb[tok], oracle.FP16)
        assert np.array_equal(logits[tok].view(np.uint32), ref.view(np.uint32)), f"token {tok}"
        ridx, rw = oracle.topk_softmax(ref, 8)
        assert np.array_equal(idx[tok].cpu().numpy().astype(np.uint32), ridx)
        assert np.abs(f16_float(bits_of(w[tok])) - rw).max() <= np.abs(rw).max() * 2 ** -10


def _routes(oracle, fx, xb):
    idx, w = [], []
    for row in xb:
        ridx, rw = oracle.topk_softmax(oracle.router_logits_pinned(fx["router"], row, oracle.FP16), 8)
        idx.append(ridx)
        w.append(rw)
    return np.stack(idx).astype(np.uint32), f16_bits(np.stack(w))


@pytest.mark.parametrize("which,t", [("small", 1), ("small", 5), ("small", 16), ("real", 1), ("real", 16)])
def test_verify_fp16_against_oracle(small, real, oracle, torch, which, t):
    # decode / verify block: FP16 rows times INT4 weights on the FP16 matrix instruction, activations and
    # outputs rounded to FP16 where the reference rounds (moe.metal:496, 627-636)
    fx = small if which == "small" else real
    rng = np.random.default_rng(900 + t)
    xb = f16_bits(rng.uniform(-0.5, 0.5, (t, fx["d"])))
    idx, wb = _routes(oracle, fx, xb)
    ref = oracle.moe_experts(fx["pool"], xb, idx, f16_float(wb), oracle.FP16)
    ti, tw = torch.from_numpy(idx.astype(np.int32)).cuda(), f16_tensor(torch, wb)
    y = fx["ctx"].verify(0, f16_tensor(torch, xb), ti, tw)
    assert y.dtype == torch.float16
    yf = f16_float(bits_of(y))
    assert rel_err(yf, ref) < 1e-2 and cosine(yf, ref) > 0.9999
    # the one-call form selects the same routes from the same rows
    y1, idx1, w1 = fx["ctx"].route_verify(0, f16_tensor(torch, xb), f16_tensor(torch, xb))
    assert np.array_equal(idx1.cpu().numpy().astype(np.uint32), idx)
    assert rel_err(f16_float(bits_of(y1)), ref) < 1e-2
    # per-route rows: un-weighted, FP16
    parts = fx["ctx"].verify_partials(0, f16_tensor(torch, xb), ti, tw)
    assert parts.dtype == torch.float16
    pf = f16_float(bits_of(parts)).reshape(t, 8, fx["d"])
    comb = (pf * f16_float(wb)[:, :, None]).sum(axis=1)
    assert rel_err(comb, ref) < 1e-2


@pytest.mark.parametrize("which,t", [("small", 40), ("small", 300), ("real", 64)])
def test_prefill_fp16_against_oracle(small, real, oracle, torch, which, t):
    # prefill chunk in FP16 mode: rows rounded to bf16 once for the GEMMs, FP16 rows out
    fx = small if which == "small" else real
    rng = np.random.default_rng(1300 + t)
    xb = f16_bits(rng.uniform(-0.5, 0.5, (t, fx["d"])))
    idx, wb = _routes(oracle, fx, xb)
    ref = oracle.moe_experts(fx["pool"], xb, idx, f16_float(wb), oracle.FP16, threads=8)
    y = fx["ctx"].prefill(0, f16_tensor(torch, xb), torch.from_numpy(idx.astype(np.int32)).cuda(), f16_tensor(torch, wb))
    assert y.dtype == torch.float16
    yf = f16_float(bits_of(y))
    assert rel_err(yf, ref) < 1e-2 and cosine(yf, ref) > 0.9999
    # the first rows through the streaming kernels agree to the same bar
    head = f16_float(bits_of(fx["ctx"].verify(0, f16_tensor(torch, xb[:8]), torch.from_numpy(idx[:8].astype(np.int32)).cuda(),
                                             f16_tensor(torch, wb[:8]))))
    assert rel_err(head, yf[:8]) < 1e-2


def test_gemv_and_resident_matrix_fp16(ff, oracle, torch):
    # DequantInt4GEMV with FP16 rows in and out (the reference's own types, dequant_int4.metal:152-169)
    m, n, rows = 520, 256, 5
    rng = np.random.default_rng(77)
    W, S, B = oracle.quantize_int4(rng.uniform(-0.4, 0.4, (m, n)).astype(np.float32))
    xb = f16_bits(rng.uniform(-1, 1, (rows, n)))
    ref = np.stack([oracle.gemv_int4_ref(W, S, B, f16_float(r)) for r in xb])
    ctx = ff.Context(256, 64, 2, 2, n_layers=1, max_tokens=16, act_dtype="fp16")
    dW, dS, dB = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (W, S.view(np.int16), B.view(np.int16)))
    y = ctx.gemv_int4(dW, dS, dB, f16_tensor(torch, xb))
    assert y.dtype == torch.float16
    assert np.abs(f16_float(bits_of(y)) - ref).max() <= np.abs(ref).max() * 2 ** -9
    y32 = ctx.gemv_int4(dW, dS, dB, f16_tensor(torch, xb), f32_out=True).cpu().numpy()
    assert np.abs(y32 - ref).max() <= np.abs(ref).max() * 1e-4
    mx = ff.Matrix(ctx, W, S, B, greedy=True)
    ym = mx.gemv(f16_tensor(torch, xb), f32_out=True).cpu().numpy()
    assert np.abs(ym - ref).max() <= np.abs(ref).max() * 1e-4
    assert mx.gemv(f16_tensor(torch, xb)).dtype == torch.float16
    assert np.array_equal(mx.greedy(f16_tensor(torch, xb)).cpu().numpy().astype(np.int64), ref.argmax(axis=1))
    mx.close()
    ctx.close()


def test_dense_ffn_fp16(ff, oracle, torch):
    # shared expert in FP16 mode, streaming (<= 16 rows) and batched
    d, f = 256, 192
    g = oracle.seed_tree_key(0x5EED, "shared-ffn-fp16")
    parts = tuple(oracle.quantize_int4(g.uniform(-0.4, 0.4, r * c).reshape(r, c)) for r, c in ((f, d), (f, d), (d, f)))
    pool = oracle.pool_from_parts([parts], d, f, align=16)
    ctx = ff.Context(d, f, 1, 1, n_layers=1, max_tokens=64, act_dtype="fp16")
    ctx.upload_expert_parts(0, 0, *parts)
    for t in (1, 16, 40):
        xb = f16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
        ref = np.stack([oracle.run_ffn(pool, 0, f16_float(row)) for row in xb])
        y = ctx.dense_ffn(0, f16_tensor(torch, xb))
        assert y.dtype == torch.float16
        yf = f16_float(bits_of(y))
        assert rel_err(yf, ref) < 1e-2 and cosine(yf, ref) > 0.9999
    ctx.close()


def test_row_steps_fp16_bit_exact(ff, oracle, torch):
    # the norms around the MoE stage with FP16 rows (the reference's own type there): every rounding to FP16,
    # bit for bit the oracle's; FusedLayerTailTests.swift:15-93 with its own FP16 data
    d = 2816
    ctx = ff.Context(d, 64, 2, 2, n_layers=1, max_tokens=16, act_dtype="fp16")
    rng = oracle.SplitMix64(0x7A11_0001)
    h2 = f16_bits(rng.uniform(-1, 1, d))[None, :]
    h1 = f16_bits(rng.uniform(-3, 3, d))[None, :]
    hidden = f16_bits(rng.uniform(-2, 2, d))[None, :]
    w = [oracle.bf16_bits(rng.uniform(0.5, 1.5, d)) for _ in range(4)]
    scalar = float(rng.uniform(0.75, 1.25, 1)[0])
    tw = [bf16_tensor(torch, x) for x in w]
    ref_h1n = oracle.rmsnorm(h1, w[0], EPS, oracle.FP16)
    ref_hidden = oracle.layer_tail(h2, ref_h1n, hidden, w[1], w[2], scalar, EPS, oracle.FP16)
    ref_normed = oracle.rmsnorm(ref_hidden, w[3], EPS, oracle.FP16)
    assert np.array_equal(bits_of(ctx.rmsnorm(f16_tensor(torch, h1), tw[0], EPS, d=d)), ref_h1n)
    th = f16_tensor(torch, hidden)
    normed = ctx.layer_tail_norms(f16_tensor(torch, h2), f16_tensor(torch, h1), th, tw[0], tw[1], tw[2], scalar, w_next=tw[3],
                                  eps=EPS, d=d)
    assert normed.dtype == torch.float16
    assert np.array_equal(bits_of(th), ref_hidden) and np.array_equal(bits_of(normed), ref_normed)
    th2 = f16_tensor(torch, hidden)
    ctx.layer_tail(f16_tensor(torch, h2), f16_tensor(torch, ref_h1n), th2, tw[1], tw[2], scalar, EPS, d=d)
    assert np.array_equal(bits_of(th2), ref_hidden)
    # post-attention setup, three rows
    g = np.random.default_rng(3)
    hid = f16_bits(g.uniform(-2, 2, (3, d)))
    att = f16_bits(g.uniform(-1, 1, (3, d)))
    ref = oracle.post_attn_setup(hid, att, w[0], w[1], w[2], EPS, oracle.FP16)
    thid = f16_tensor(torch, hid)
    outs = ctx.post_attn_setup(thid, f16_tensor(torch, att), tw[0], tw[1], tw[2], EPS, d=d)
    assert np.array_equal(bits_of(thid), ref[0])
    for got, want in zip(outs, ref[1:]):
        assert got.dtype == torch.float16 and np.array_equal(bits_of(got), want)
    ctx.close()


def test_guest_pairs_and_reduce_fp16(small, oracle, torch):
    # the guest seam in FP16 mode (RoutedPrefillGuest.runLayer: sorted pairs in, un-weighted FP16 rows out), then
    # prefill_moe_reduce_token_major on those rows: the GPU reduce is bit-exact against the oracle's reduce of
    # the same rows and equals the fused call
    t = 45
    rng = np.random.default_rng(21)
    xb = f16_bits(rng.normal(0, 1, (t, small["d"])))
    x = f16_tensor(torch, xb)
    ctx = small["ctx"]
    idx, w = ctx.router(0, x)
    pairs = oracle.make_token_expert_pairs(idx.cpu().numpy(), bits_of(w), t, 8)
    want_partials = oracle.route_partials(small["pool"], pairs, xb, small["d"], t, 8, oracle.FP16)
    partials = torch.zeros((t, 8, small["d"]), dtype=torch.float16, device="cuda")
    raw = np.stack([pairs["token"], pairs["expert"], pairs["rank"], pairs["weight_bits"]], 1).astype(np.uint32)
    ctx.prefill_pairs(0, x, torch.from_numpy(raw.view(np.int32)).cuda(), t, partials)
    assert rel_err(f16_float(bits_of(partials)), f16_float(want_partials)) <= 1e-2
    h2 = bits_of(ctx.reduce_token_major(partials, w))
    assert np.array_equal(h2, oracle.reduce_token_major(bits_of(partials), oracle.FP16, bits_of(w), oracle.FP16))
    assert np.array_equal(h2, bits_of(ctx.prefill(0, x, idx, w)))
