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
    # prefill chunk in FP16 mode: FP16 rows against FP16 tiles, block-scaled FP16 activations, FP16 rows out
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


def test_prefill_fp16_tiles_are_half_of_fma(small, real, oracle, ff, torch):
    """The tile weights the FP16 prefill's matrix instructions read from LDS (copied out by the kernel itself) are the
    reference's FP16 tile weights half(fma(q, scale, bias)) (prefill_mma_dequant32, prefill.metal:581-590), bit for bit:
    q * scale is exact in fp32, so numpy's float32 product-and-sum rounded to float16 is that value."""
    for fx, experts in ((small, (0, 15)), (real, (3,))):
        for ex in experts:
            for which, name in ((ff.GATE, "gate"), (ff.UP, "up"), (ff.DOWN, "down")):
                got = fx["ctx"].prefill_tiles(0, ex, which)
                assert got.dtype == torch.float16
                W, S, B = fx["pool"].sub(ex, name)
                rows, half_cols = W.shape
                q = np.empty((rows, half_cols * 2), np.float32)
                q[:, 0::2] = W & 0xF
                q[:, 1::2] = W >> 4
                sc = np.repeat(oracle.bf16_to_float(S), 64, axis=1)
                bi = np.repeat(oracle.bf16_to_float(B), 64, axis=1)
                want = (q * sc + bi).astype(np.float32).astype(np.float16).view(np.uint16)
                assert np.array_equal(bits_of(got), want), (ex, name)


def test_prefill_fp16_keeps_activations_past_half_range(oracle, ff, torch):
    """Inputs large enough that gelu(gate) * up passes FP16's largest value (65,504) while the layer's outputs stay
    inside it: the block-scaled FP16 activations (prefill.metal:593-598,685-702) carry them, so the rows are finite and
    within the usual bar of the fp32 reference; stored as plain FP16 the activations would be infinite."""
    d, f, e, t = 128, 64, 4, 48
    g = oracle.seed_tree_key(0xF16, "prefill-fp16-range")
    gates = [g.uniform(-0.5, 0.5, f * d).reshape(f, d) for _ in range(e)]
    ups = [g.uniform(-0.5, 0.5, f * d).reshape(f, d) for _ in range(e)]
    downs = [g.uniform(-0.004, 0.004, d * f).reshape(d, f) for _ in range(e)]
    pool = oracle.pool_from_float(gates, ups, downs, align=16)
    ctx = ff.Context(d, f, e, 2, n_layers=1, max_tokens=64, act_dtype="fp16")
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    xb = f16_bits(g.uniform(-1.0, 1.0, t * d).reshape(t, d) * 160.0)
    idx = np.stack([np.array([r % e, (r + 1) % e], np.uint32) for r in range(t)])
    w = np.full((t, 2), 0.5, np.float32)
    # the reference in float64 (the oracle's FP16 mode stores the activations as plain FP16: infinite here)
    x = f16_float(xb)
    ref = np.zeros((t, d), np.float64)
    peak = 0.0
    for r in range(t):
        for k in range(2):
            ex = int(idx[r, k])
            gw_, uw_, dw_ = (oracle.dequantize_int4(*pool.sub(ex, name)).astype(np.float64) for name in ("gate", "up", "down"))
            act = oracle.gelu_tanh((gw_ @ x[r]).astype(np.float32)).astype(np.float64) * (uw_ @ x[r])
            peak = max(peak, float(np.abs(act).max()))
            ref[r] += 0.5 * (dw_ @ act)
    ref = ref.astype(np.float32)
    assert peak > 2 * 65504.0 and np.abs(ref).max() < 3e4, (peak, np.abs(ref).max())
    y = ctx.prefill(0, f16_tensor(torch, xb), torch.from_numpy(idx.astype(np.int32)).cuda(), f16_tensor(torch, f16_bits(w)))
    yf = f16_float(bits_of(y))
    assert np.isfinite(yf).all()
    assert rel_err(yf, ref) < 1e-2 and cosine(yf, ref) > 0.9999, (rel_err(yf, ref), cosine(yf, ref))
    ctx.close()


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


def test_prefill_router_fp16_fast_form_equals_pinned_form(oracle, ff, torch):
    """FP16 rows through the two-pass prefill router (every value enters the approximate pass as two bf16 halves):
    routes and weights bit for bit those of the form that computes every pinned logit, which is held against the oracle
    - on rows with exact ties between experts, rows one bf16 step of a weight apart, rows at both ends of the FP16
    range, FP16 subnormals, zero and constant rows, and rows with non-finite values."""
    d, e, k, t = 2816, 128, 8, 80
    rng = np.random.default_rng(91)
    router = rng.normal(0, 0.02, (e, d)).astype(np.float32)
    router[5] = router[3]
    router[64] = router[3]
    bits = oracle.bf16_bits(router)
    bits[7] = bits[6]
    bits[7, 17] ^= 1
    x = rng.normal(0, 1, (t, d)).astype(np.float32)
    x[1] *= 2e3                                 # near the top of the FP16 range
    x[2] *= 1e-6                                # FP16 subnormals
    x[3] = 0.0
    x[4, :] = x[4, 0]
    x[5, 100] = np.inf
    x[6, 5] = np.nan
    x[7] = 60000.0                              # squares overflow fp32 sums nowhere near, the norm is large
    wf = oracle.bf16_to_float(bits)
    x[8] = wf[3] * 50
    front = [20, 30, 40, 50, 60, 70, 80]
    x[9] = 50.0 * (1.5 * wf[front].sum(axis=0) + wf[6])      # experts 6 and 7 as eighth and ninth, a few fp32 steps apart
    xb = f16_bits(x)
    ctx = ff.Context(d, 64, e, k, n_layers=1, max_tokens=128, act_dtype="fp16")
    ctx.upload_router_bf16(0, bits)
    xt = f16_tensor(torch, xb)
    idx_fast, w_fast = ctx.router(0, xt)
    idx_ref, w_ref, logits = ctx.router(0, xt, want_logits=True)
    torch.cuda.synchronize()
    assert w_fast.dtype == torch.float16
    assert np.array_equal(idx_fast.cpu().numpy(), idx_ref.cpu().numpy())
    assert np.array_equal(bits_of(w_fast), bits_of(w_ref))
    got = logits.cpu().numpy()
    for tok in (0, 1, 2, 3, 4, 8, 9, t - 1):
        want = oracle.router_logits_pinned(bits, xb[tok], oracle.FP16)
        assert np.array_equal(got[tok].view(np.uint32), want.view(np.uint32)), tok
        o_idx, _ = oracle.topk_softmax(want, k)
        assert np.array_equal(idx_fast.cpu().numpy()[tok].astype(np.uint32), o_idx), tok
    ctx.close()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("d,f,e,fs,t", [(128, 64, 16, 1472, 5), (2816, 704, 128, 2112, 16), (2816, 704, 128, 2112, 1)])
def test_shared_expert_inside_the_routed_launches_fp16(oracle, ff, torch, d, f, e, fs, t, bits):
    """FP16 rows through ffmoe_route_verify_shared + ffmoe_layer_tail_routed_shared against the separate FP16 calls
    (ffmoe_route_verify, ffmoe_dense_ffn, ffmoe_layer_tail): the same routes bit for bit, the new hidden rows to the
    rounding of the shared expert's row (its K is summed in chunks). The shared expert 4-bit and 8-bit."""
    _, pool, router = make_layer(oracle, 5, d, f, e, align=16)
    ctx = ff.Context(d, f, e, 8, n_layers=1, max_tokens=16, act_dtype="fp16")
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    g = np.random.default_rng(d + fs + t)
    scale = 0.4 if d < 1024 else 0.08
    quantize = oracle.quantize_int4 if bits == 4 else oracle.quantize_int8
    parts = tuple(quantize(g.uniform(-scale, scale, (r, c)).astype(np.float32)) for r, c in ((fs, d), (fs, d), (d, fs)))
    shared = ff.Context(d, fs, 1, 1, n_layers=1, max_tokens=16, act_dtype="fp16")
    shared.upload_expert_parts(0, 0, *parts, int8=bits == 8)
    x, rx, sx = (f16_tensor(torch, f16_bits(g.uniform(-1.0, 1.0, (t, d)))) for _ in range(3))
    hid = f16_bits(g.uniform(-1.0, 1.0, (t, d)))
    tw2, tw1 = (bf16_tensor(torch, oracle.bf16_bits(g.uniform(0.5, 1.5, d).astype(np.float32))) for _ in range(2))
    y, idx_a, w_a = ctx.route_verify(0, rx, x)
    h1 = shared.dense_ffn(0, sx)
    hid_a = f16_tensor(torch, hid)
    ctx.layer_tail(y, h1, hid_a, tw2, tw1, 0.875, 1e-6, d=d)
    idx_b, w_b = ctx.route_verify_shared(shared, 0, 0, rx, x, sx)
    hid_b = f16_tensor(torch, hid)
    ctx.layer_tail_routed_shared(shared, w_b, hid_b, tw2, tw1, 0.875, 1e-6)
    assert hid_b.dtype == torch.float16 and w_b.dtype == torch.float16
    assert np.array_equal(idx_a.cpu().numpy(), idx_b.cpu().numpy()) and np.array_equal(bits_of(w_a), bits_of(w_b))
    got, want = f16_float(bits_of(hid_b)), f16_float(bits_of(hid_a))
    assert rel_err(got, want) < 1e-2 and cosine(got, want) > 0.9999, (rel_err(got, want), cosine(got, want))
    assert ctx.handover_giveups() == 0
    ctx.close()
    shared.close()


def test_int8_dense_layer_at_many_rows_follows_the_activation_type(oracle, ff, torch):
    """The 8-bit dense layer's GEMM form (192 rows and more) keeps hi / lo rows of the weights in the activation type:
    uploaded under bf16, the context is switched to FP16 and back - each time the rows are made again from the nibble
    planes - and the 200-row call agrees with the streaming form of the same type (16 rows per matrix call)."""
    d, fs, t = 192, 1472, 200
    g = np.random.default_rng(21)
    parts = tuple(oracle.quantize_int8(g.uniform(-0.4, 0.4, (r, c)).astype(np.float32)) for r, c in ((fs, d), (fs, d), (d, fs)))
    dense = ff.Context(d, fs, 1, 1, n_layers=1, max_tokens=256)
    dense.upload_expert_parts(0, 0, *parts, int8=True)
    xv = g.uniform(-1.0, 1.0, (t, d)).astype(np.float32)
    seen = {}
    for act in ("bf16", "fp16", "bf16"):
        dense.set_act_dtype(act)
        x = f16_tensor(torch, f16_bits(xv)) if act == "fp16" else bf16_tensor(torch, oracle.bf16_bits(xv))
        y = dense.dense_ffn(0, x)
        assert y.dtype == (torch.float16 if act == "fp16" else torch.bfloat16)
        gate_up, down = dense.matrix_int8_glu(parts[0], parts[1]), dense.matrix_int8(*parts[2])
        want = torch.cat([down.gemv(gate_up.gemv(x[r0:r0 + 16])) for r0 in range(0, t, 16)])
        yf, wf = y.float().cpu().numpy(), want.float().cpu().numpy()
        # one rounding step at the largest element: 2^-8 of it in bf16, 2^-11 in FP16
        assert rel_err(yf, wf) < (2e-3 if act == "fp16" else 1e-2) and cosine(yf, wf) > 0.99999, (act, rel_err(yf, wf), cosine(yf, wf))
        assert np.mean(bits_of(y) == bits_of(want)) > (0.4 if act == "fp16" else 0.75)       # FP16 rows show three more bits of the sum's order
        if act in seen:
            assert torch.equal(y.view(torch.int16), seen[act].view(torch.int16))        # back to bf16: the same rows again
        seen[act] = y
        gate_up.close()
        down.close()
    dense.close()
