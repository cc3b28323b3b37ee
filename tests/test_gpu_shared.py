"""Dense (shared-expert) FFN through the C ABI against the CPU oracle: the single-row operator, its
multi-row and batched forms, and the upload from separate projections. Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, cosine, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available()
    return torch


@pytest.fixture(scope="module")
def ff():
    import fieldfare_moe
    fieldfare_moe.lib()
    return fieldfare_moe


def _reference_rows(oracle, parts, x_bits):
    """SharedExpertInt4Tests.swift:24-31 per row: dequant GEMV for gate and up, the activation rounded
    to 16 bits once, dequant GEMV for down."""
    (gW, gS, gB), (uW, uS, uB), (dW, dS, dB) = parts
    out = []
    for row in x_bits:
        x = oracle.bf16_to_float(row)
        g = oracle.gemv_int4_ref(gW, gS, gB, x)
        u = oracle.gemv_int4_ref(uW, uS, uB, x)
        act = oracle.bf16_to_float(oracle.bf16_bits(oracle.gelu_tanh(g) * u))
        out.append(oracle.gemv_int4_ref(dW, dS, dB, act))
    return np.stack(out)


def _context(ff, parts, d, f, max_tokens):
    ctx = ff.Context(d, f, 1, 1, n_layers=1, max_tokens=max_tokens)
    ctx.upload_expert_parts(0, 0, *parts)
    return ctx


def test_shared_expert_matches_affine_reference(ff, oracle, torch):
    # sharedExpertInt4MatchesAffineReference (SharedExpertInt4Tests.swift:13-50): same seed and draw order
    d, f = 128, 64
    rng = oracle.seed_tree_key(0x604, "shared-expert-int4")
    x = rng.uniform(-0.4, 0.4, d)
    gate = np.stack([rng.uniform(-0.4, 0.4, d) for _ in range(f)])
    up = np.stack([rng.uniform(-0.4, 0.4, d) for _ in range(f)])
    down = np.stack([rng.uniform(-0.4, 0.4, f) for _ in range(d)])
    parts = (oracle.quantize_int4(gate), oracle.quantize_int4(up), oracle.quantize_int4(down))
    xb = oracle.bf16_bits(x)[None, :]
    ref = _reference_rows(oracle, parts, xb)
    ctx = _context(ff, parts, d, f, 16)
    y = oracle.bf16_to_float(bits_of(ctx.dense_ffn(0, bf16_tensor(torch, xb))))
    # Tolerance.quantInt4 * 4 (Tolerances.swift:16) is the reference's FP16 bound; bf16 outputs carry 2^-9
    assert rel_err(y, ref) < 1e-2
    assert cosine(y, ref) > 0.9999
    ctx.close()


@pytest.mark.parametrize("d,f,t", [(128, 64, 5), (256, 192, 16), (2816, 2112, 1), (2816, 2112, 16), (3072, 192, 5),
                                   (192, 3072, 5), (3072, 2880, 16)])
def test_shared_expert_rows(ff, oracle, torch, d, f, t):
    # rows <= 16: the streaming kernels; (2816, 2112) is the model's shared expert. A hidden size above 2816 or an
    # intermediate size above 2816 is more than a wave's register ring holds: those take the one-shot grids
    g = oracle.seed_tree_key(0x5EED, f"shared-ffn-d{d}-f{f}-t{t}")
    scale = 0.4 if d < 1024 else 0.08
    parts = tuple(oracle.quantize_int4(g.uniform(-scale, scale, r * c).reshape(r, c)) for r, c in ((f, d), (f, d), (d, f)))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    ref = _reference_rows(oracle, parts, xb)
    ctx = _context(ff, parts, d, f, 16)
    x = bf16_tensor(torch, xb)
    y = bits_of(ctx.dense_ffn(0, x))
    yf = oracle.bf16_to_float(y)
    assert rel_err(yf, ref) < 1e-2
    assert cosine(yf, ref) > 0.9999
    # a row of a block equals the same row run alone, bit for bit
    for r in range(0, t, max(1, t // 3)):
        single = bits_of(ctx.dense_ffn(0, x[r:r + 1]))
        assert np.array_equal(single[0], y[r]), f"row {r}"
    ctx.close()


@pytest.mark.parametrize("d,f,t", [(128, 64, 17), (2816, 2112, 32), (256, 192, 23), (2816, 2112, 100), (192, 1472, 256),
                                   (64, 64, 255), (128, 64, 384), (3072, 192, 20)])
def test_shared_expert_17_to_384_rows_stream_the_arena_tiles(ff, oracle, torch, d, f, t):
    # a short prompt or a chunk's ragged end: the resident-matrix GEMV on the expert's arena tiles, a grid row per 16 input
    # rows ((3072, 192): wider than that kernel's ring, the grouped GEMMs take it). Rows against the reference; a row of
    # the block against the row run alone (the <= 16-row kernels: the same sums in another order, so to a rounding step);
    # the block split anywhere gives the same rows bit for bit.
    g = oracle.seed_tree_key(0x5EED, f"shared-ffn-stream-d{d}-f{f}-t{t}")
    scale = 0.4 if d < 1024 else 0.08
    parts = tuple(oracle.quantize_int4(g.uniform(-scale, scale, r * c).reshape(r, c)) for r, c in ((f, d), (f, d), (d, f)))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    ctx = _context(ff, parts, d, f, max(256, t))
    x = bf16_tensor(torch, xb)
    y = bits_of(ctx.dense_ffn(0, x))
    sel = sorted({0, 15, 16, t // 2, t - 1})
    ref = _reference_rows(oracle, parts, xb[sel])
    yf = oracle.bf16_to_float(y[sel])
    assert rel_err(yf, ref) < 1e-2 and cosine(yf, ref) > 0.9999, (rel_err(yf, ref), cosine(yf, ref))
    alone = np.stack([bits_of(ctx.dense_ffn(0, x[r:r + 1]))[0] for r in sel])
    af = oracle.bf16_to_float(alone)
    assert rel_err(yf, af) < 1e-2 and (d > 2816 or np.mean(alone == y[sel]) > 0.9)     # (the GEMMs round the weights to bf16)
    if d <= 2816:
        cut = 17 + (t - 17) // 2
        assert np.array_equal(bits_of(ctx.dense_ffn(0, x[:cut])), y[:cut])
        if t - cut > 16:
            assert np.array_equal(bits_of(ctx.dense_ffn(0, x[cut:])), y[cut:])
    ctx.close()


@pytest.mark.parametrize("d,f,t", [(128, 64, 40), (256, 192, 300), (2816, 2112, 64), (512, 640, 700)])
def test_shared_expert_batched(ff, oracle, torch, d, f, t):
    # more than 16 rows: the grouped GEMMs ((512, 640, 700): three M-tiles against ten and four N-blocks, so that the
    # one-expert block map has tiles, N-blocks past the first eight and empty block slots all at once). 64 rows of U(-2, 2) at the model's shape restate
    # batchedIsNoLessAccurateThanPerToken (PrefillSharedExpertBatchedTests.swift:47-101), whose reference is
    # MoeRef.runFFN per token and whose bound is a relative L2 error below 5e-3 on FP16 outputs.
    g = oracle.seed_tree_key(0x5EED, f"shared-ffn-batched-d{d}-f{f}-t{t}")
    scale = 0.4 if d < 1024 else 0.05
    parts = tuple(oracle.quantize_int4(g.uniform(-scale, scale, r * c).reshape(r, c)) for r, c in ((f, d), (f, d), (d, f)))
    xb = oracle.bf16_bits(g.uniform(-2.0, 2.0, t * d)).reshape(t, d)
    pool = oracle.pool_from_parts([parts], d, f, align=16)
    ref = np.stack([oracle.run_ffn(pool, 0, oracle.bf16_to_float(row)) for row in xb])
    ctx = _context(ff, parts, d, f, max(t, 64))
    yf = oracle.bf16_to_float(bits_of(ctx.dense_ffn(0, bf16_tensor(torch, xb))))
    l2 = float(np.sqrt(((yf - ref) ** 2).sum() / (ref ** 2).sum()))
    assert l2 < 5e-3
    assert rel_err(yf, ref) < 1e-2
    assert cosine(yf, ref) > 0.9999
    # the streaming path on the first rows agrees with the GEMM path to the same bar
    head = oracle.bf16_to_float(bits_of(ctx.dense_ffn(0, bf16_tensor(torch, xb[:8]))))
    assert rel_err(head, yf[:8]) < 1e-2
    ctx.close()


def test_parts_upload_equals_blob_upload(ff, oracle, torch):
    # the same expert through ffmoe_upload_expert_parts (host and device sources) and through a blob
    d, f = 256, 128
    rng = np.random.default_rng(11)
    pool = oracle.random_pool(rng, 2, d, f, align=16)
    blob = ff.Context(d, f, 2, 2, n_layers=1, max_tokens=16)
    blob.upload_layer(0, pool.bytes, pool.stride, ff.Offsets(*pool.offsets.as_tuple()))
    host = ff.Context(d, f, 2, 2, n_layers=1, max_tokens=16)
    dev = ff.Context(d, f, 2, 2, n_layers=1, max_tokens=16)
    x = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((1, 2), dtype=torch.int32, device="cuda")
    w = torch.ones((1, 2), dtype=torch.bfloat16, device="cuda")
    for e in range(2):
        parts = tuple(pool.sub(e, which) for which in ("gate", "up", "down"))
        if e == 0:
            # one of two experts uploaded: the layer is not ready yet
            host.upload_expert_parts(0, 1, *tuple(pool.sub(1, which) for which in ("gate", "up", "down")))
            with pytest.raises(ff.FieldfareError, match="not uploaded"):
                host.verify(0, x, idx, w)
        host.upload_expert_parts(0, e, *parts)
        dev.upload_expert_parts(0, e, *tuple(tuple(torch.from_numpy(np.ascontiguousarray(a).view(np.uint8)).cuda()
                                                   for a in tr) for tr in parts))
    for e in range(2):
        for which in (0, 1, 2):
            ref = bits_of(blob.dequant_expert(0, e, which))
            assert np.array_equal(bits_of(host.dequant_expert(0, e, which)), ref)
            assert np.array_equal(bits_of(dev.dequant_expert(0, e, which)), ref)
    for c in (blob, host, dev):
        c.close()


def test_dense_ffn_argument_errors(ff, oracle, torch):
    routed = ff.Context(128, 64, 4, 2, n_layers=1, max_tokens=16)
    x = torch.zeros((1, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ff.FieldfareError, match="n_experts = 1"):
        routed.dense_ffn(0, x)
    routed.close()
    dense = ff.Context(128, 64, 1, 1, n_layers=1, max_tokens=32)
    with pytest.raises(ff.FieldfareError, match="not uploaded"):
        dense.dense_ffn(0, x)
    parts = tuple(oracle.quantize_int4(np.zeros((r, c), np.float32)) for r, c in ((64, 128), (64, 128), (128, 64)))
    dense.upload_expert_parts(0, 0, *parts)
    with pytest.raises(ff.FieldfareError, match="exceeds max_tokens"):
        dense.dense_ffn(0, torch.zeros((33, 128), dtype=torch.bfloat16, device="cuda"))
    assert float(dense.dense_ffn(0, x).abs().max()) == 0.0
    dense.close()


@pytest.mark.parametrize("d,f,e,fs,t,mode", [
    (128, 64, 16, 192, 5, "one_launch"),          # shared K in one short chunk
    (128, 64, 16, 1472, 16, "one_launch"),        # 23 groups: chunks of 11, 11 and 1
    (128, 64, 16, 1472, 3, "router_launches"),    # the router as launches of its own: the plain gate/up kernel hosts the blocks
    (128, 64, 16, 1472, 7, "no_hand_over"),       # every wave gives up waiting at once and routes for itself
    (2816, 704, 128, 2112, 1, "one_launch"),      # the model's shapes: decode step
    (2816, 704, 128, 2112, 16, "one_launch"),     # verify block
    (2816, 704, 128, 2112, 6, "router_launches"),
])
def test_shared_expert_inside_the_routed_launches(ff, oracle, torch, d, f, e, fs, t, mode):
    """ffmoe_route_verify_shared + ffmoe_layer_tail_routed_shared against the separate calls (ffmoe_route_verify,
    ffmoe_dense_ffn, ffmoe_layer_tail): same routes bit for bit; the new hidden rows agree to the rounding of the
    shared expert's row (its K is summed in chunks instead of interleaved slices), and with the shared expert's rows
    zeroed out of the comparison - a shared expert of zero weights - bit for bit. Padding stays untouched."""
    from helpers import make_layer, to_ff_offsets
    rng, pool, router = make_layer(oracle, 5, d, f, e, align=16)
    ctx = ff.Context(d, f, e, 8, n_layers=1, max_tokens=16)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    g = oracle.seed_tree_key(0x5A4E, f"shared-inside-d{d}-fs{fs}-t{t}-{mode}")
    scale = 0.4 if d < 1024 else 0.08
    parts = tuple(oracle.quantize_int4(g.uniform(-scale, scale, r * c).reshape(r, c)) for r, c in ((fs, d), (fs, d), (d, fs)))
    zero_parts = tuple(oracle.quantize_int4(np.zeros((r, c), np.float32)) for r, c in ((fs, d), (fs, d), (d, fs)))
    shared = ff.Context(d, fs, 1, 1, n_layers=2, max_tokens=16)
    shared.upload_expert_parts(0, 0, *zero_parts)
    shared.upload_expert_parts(1, 0, *parts)
    pad = 8
    xb, rxb, sxb = (oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d) for _ in range(3))
    x, rx, sx = bf16_tensor(torch, xb), bf16_tensor(torch, rxb), bf16_tensor(torch, sxb)
    hid = np.full((t, d + pad), oracle.bf16_bits(np.float32(-25.0)), np.uint16)
    hid[:, :d] = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    tw2, tw1 = (bf16_tensor(torch, oracle.bf16_bits(g.uniform(0.5, 1.5, d))) for _ in range(2))
    if mode == "router_launches":
        ctx.set_one_launch_routing(False)
    if mode == "no_hand_over":
        ctx.set_handover_timeout(0)
    for layer_s in (0, 1):
        y, idx_a, w_a = ctx.route_verify(0, rx, x)
        h1 = shared.dense_ffn(layer_s, sx)
        hid_a = bf16_tensor(torch, hid)
        ctx.layer_tail(y, h1, hid_a, tw2, tw1, 0.875, 1e-6, d=d)
        idx_b, w_b = ctx.route_verify_shared(shared, 0, layer_s, rx, x, sx)
        hid_b = bf16_tensor(torch, hid)
        ctx.layer_tail_routed_shared(shared, w_b, hid_b, tw2, tw1, 0.875, 1e-6)
        assert np.array_equal(idx_a.cpu().numpy(), idx_b.cpu().numpy()) and np.array_equal(bits_of(w_a), bits_of(w_b))
        got, want = bits_of(hid_b), bits_of(hid_a)[:, :d]
        assert np.array_equal(got[:, d:], hid[:, d:])
        if layer_s == 0:
            assert float(h1.abs().max()) == 0.0
            assert np.array_equal(got[:, :d], want)
        else:
            gf, wf = oracle.bf16_to_float(got[:, :d]), oracle.bf16_to_float(want)
            assert rel_err(gf, wf) < 1e-2 and cosine(gf, wf) > 0.9999, (rel_err(gf, wf), cosine(gf, wf))
            assert np.mean(got[:, :d] == want) > 0.8
    # the shared expert's row itself: with the routed rows' norm weight at zero the tail is hidden + norm(h1) scaled
    zero = torch.zeros_like(tw2)
    one = torch.ones_like(tw1)
    hid0 = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    ctx.route_verify_shared(shared, 0, 1, rx, x, sx)
    ctx.layer_tail_routed_shared(shared, w_b, hid0, zero, one, 1.0, 1e-6)
    ref = _reference_rows(oracle, parts, sxb)
    ref_bits = oracle.bf16_bits(ref.astype(np.float32))
    want0 = oracle.layer_tail(np.zeros((t, d), np.uint16), ref_bits, np.zeros((t, d), np.uint16), bits_of(zero), bits_of(one), 1.0, 1e-6)
    g0, w0 = oracle.bf16_to_float(bits_of(hid0)), oracle.bf16_to_float(want0)
    assert rel_err(g0, w0) < 1e-2 and cosine(g0, w0) > 0.9999, (rel_err(g0, w0), cosine(g0, w0))
    if mode == "no_hand_over":
        assert ctx.handover_giveups() > 0
    elif mode == "one_launch":
        assert ctx.handover_giveups() == 0
    # ordinary calls on both contexts afterwards
    y2, idx_c, _ = ctx.route_verify(0, rx, x)
    assert np.array_equal(bits_of(y2), bits_of(y)) and np.array_equal(idx_c.cpu().numpy(), idx_a.cpu().numpy())
    assert np.array_equal(bits_of(shared.dense_ffn(1, sx)), bits_of(h1))
    ctx.close()
    shared.close()


def test_route_verify_shared_argument_errors(ff, oracle, torch):
    ctx = ff.Context(128, 64, 4, 2, n_layers=1, max_tokens=16)
    other = ff.Context(128, 64, 4, 2, n_layers=1, max_tokens=16)
    wide = ff.Context(256, 64, 1, 1, n_layers=1, max_tokens=16)
    x = torch.zeros((2, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ff.FieldfareError, match="n_experts = 1"):
        ctx.route_verify_shared(other, 0, 0, x, x, x)
    with pytest.raises(ff.FieldfareError, match="not uploaded"):
        ctx.route_verify_shared(wide, 0, 0, x, x, x)
    parts = tuple(oracle.quantize_int4(np.zeros((r, c), np.float32)) for r, c in ((64, 256), (64, 256), (256, 64)))
    wide.upload_expert_parts(0, 0, *parts)
    with pytest.raises(ff.FieldfareError, match="same d"):
        ctx.route_verify_shared(wide, 0, 0, x, x, x)
    for c in (ctx, other, wide):
        c.close()


def _int8_parts(oracle, g, d, fs, scale):
    return tuple(oracle.quantize_int8(g.uniform(-scale, scale, r * c).reshape(r, c)) for r, c in ((fs, d), (fs, d), (d, fs)))


def _int8_reference_rows(oracle, parts, x_bits):
    """SharedExpertInt8Tests.swift:33-41 per row: DequantInt8GemvRef for gate and up, the activation rounded to 16 bits
    once, DequantInt8GemvRef for down (float64 tanh: the single-precision form cancels below about -4)."""
    (gW, gS, gB), (uW, uS, uB), (dW, dS, dB) = parts
    out = []
    for row in x_bits:
        x = oracle.bf16_to_float(row)
        g64 = oracle.gemv_int8_ref(gW, gS, gB, x).astype(np.float64)
        u = oracle.gemv_int8_ref(uW, uS, uB, x)
        act = (0.5 * g64 * (1.0 + np.tanh(0.7978845608028654 * (g64 + 0.044715 * g64 ** 3)))).astype(np.float32) * u
        out.append(oracle.gemv_int8_ref(dW, dS, dB, oracle.bf16_to_float(oracle.bf16_bits(act))))
    return np.stack(out)


@pytest.mark.parametrize("d,fs,t", [(128, 64, 1), (128, 192, 16), (192, 1472, 5), (2816, 2112, 16), (128, 64, 40), (128, 64, 191),
                                    (192, 1472, 200), (2816, 2112, 256), (64, 64, 192)])
def test_dense_ffn_on_an_int8_layer(ff, oracle, torch, d, fs, t):
    # the 8-bit shared expert as a layer of the dense context: ffmoe_dense_ffn equals the gated matrix + down matrix calls
    # bit for bit (it runs the same two kernels, a grid row per 16 rows) and follows the reference's rows; from 192 rows on
    # it runs the library's dense GEMM on hi / lo rows of the weights instead, which sums in another order: the same rows
    # to the rounding of a sum
    g = oracle.seed_tree_key(0x1A8, f"dense-int8-d{d}-fs{fs}-t{t}")
    parts = _int8_parts(oracle, g, d, fs, 0.4 if d < 1024 else 0.08)
    dense = ff.Context(d, fs, 1, 1, n_layers=2, max_tokens=max(t, 16))
    x = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ff.FieldfareError, match="not uploaded"):
        dense.dense_ffn(1, x)
    dense.upload_expert_parts(1, 0, *parts, int8=True)
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    xt = bf16_tensor(torch, xb)
    y = dense.dense_ffn(1, xt)
    gate_up, down = dense.matrix_int8_glu(parts[0], parts[1]), dense.matrix_int8(*parts[2])
    want = torch.cat([down.gemv(gate_up.gemv(xt[r0:r0 + 16])) for r0 in range(0, t, 16)])
    if t < 192:
        assert torch.equal(y.view(torch.int16), want.view(torch.int16))
    else:
        yf, wf = y.float().cpu().numpy(), want.float().cpu().numpy()
        # one bf16 step at the largest element is 2^-8 of it
        assert rel_err(yf, wf) < 1e-2 and cosine(yf, wf) > 0.99999 and np.mean(bits_of(y) == bits_of(want)) > 0.75, (
            rel_err(yf, wf), cosine(yf, wf), np.mean(bits_of(y) == bits_of(want)))
    if d * fs <= 192 * 1472 or t <= 16 or t >= 192:
        rows = slice(0, min(t, 4) if d > 1024 or t > 40 else t)
        ref = _int8_reference_rows(oracle, parts, xb[rows])
        got = oracle.bf16_to_float(bits_of(y))[rows]
        assert rel_err(got, ref) < 1e-2 and cosine(got, ref) > 0.9999, (rel_err(got, ref), cosine(got, ref))
    with pytest.raises(ff.FieldfareError, match="outside"):
        dense.dense_ffn(1, torch.zeros((max(t, 16) + 1, d), dtype=torch.bfloat16, device="cuda"))
    # the layer is served in the width of its latest upload
    parts4 = tuple(oracle.quantize_int4(np.zeros((r, c), np.float32)) for r, c in ((fs, d), (fs, d), (d, fs)))
    dense.upload_expert_parts(1, 0, *parts4)
    assert float(dense.dense_ffn(1, xt).abs().max()) == 0.0
    dense.upload_expert_parts(1, 0, *parts, int8=True)
    assert torch.equal(dense.dense_ffn(1, xt).view(torch.int16), y.view(torch.int16))
    routed = ff.Context(128, 64, 4, 2, n_layers=1, max_tokens=16)
    with pytest.raises(ff.FieldfareError, match="n_experts = 1"):
        routed.upload_expert_parts(0, 0, *_int8_parts(oracle, g, 128, 64, 0.4), int8=True)
    for c in (gate_up, down, dense, routed):
        c.close()


@pytest.mark.parametrize("d,f,e,fs,t,mode", [
    (128, 64, 16, 192, 5, "one_launch"),
    (128, 64, 16, 1472, 16, "one_launch"),        # 23 groups: chunks of 11, 11 and 1, two down slots each
    (128, 64, 16, 1472, 3, "router_launches"),
    (128, 64, 16, 1472, 7, "no_hand_over"),
    (2816, 704, 128, 2112, 1, "one_launch"),      # the model's shapes: decode step
    (2816, 704, 128, 2112, 16, "one_launch"),     # verify block
    (2816, 704, 128, 2112, 6, "router_launches"),
])
def test_int8_shared_expert_inside_the_routed_launches(ff, oracle, torch, d, f, e, fs, t, mode):
    """ffmoe_route_verify_shared + ffmoe_layer_tail_routed_shared with the shared expert held 8-bit, against the separate
    calls (ffmoe_route_verify, ffmoe_dense_ffn on the 8-bit layer, ffmoe_layer_tail): same routes bit for bit; the new
    hidden rows agree to the rounding of the shared expert's row (its K is summed in chunks there), bit for bit with a
    shared expert of zero weights; the shared expert's own row follows the reference. A 4-bit layer of the same dense
    context is served side by side."""
    from helpers import make_layer, to_ff_offsets
    rng, pool, router = make_layer(oracle, 5, d, f, e, align=16)
    ctx = ff.Context(d, f, e, 8, n_layers=1, max_tokens=16)
    ctx.upload_layer(0, pool.bytes, pool.stride, to_ff_offsets(ff, pool.offsets))
    ctx.upload_router_bf16(0, router)
    g = oracle.seed_tree_key(0x5A4F, f"shared8-inside-d{d}-fs{fs}-t{t}-{mode}")
    parts = _int8_parts(oracle, g, d, fs, 0.4 if d < 1024 else 0.08)
    zero_parts = tuple(oracle.quantize_int8(np.zeros((r, c), np.float32)) for r, c in ((fs, d), (fs, d), (d, fs)))
    parts4 = tuple(oracle.quantize_int4(g.uniform(-0.1, 0.1, r * c).reshape(r, c)) for r, c in ((fs, d), (fs, d), (d, fs)))
    shared = ff.Context(d, fs, 1, 1, n_layers=3, max_tokens=16)
    shared.upload_expert_parts(0, 0, *zero_parts, int8=True)
    shared.upload_expert_parts(1, 0, *parts, int8=True)
    shared.upload_expert_parts(2, 0, *parts4)
    pad = 8
    xb, rxb, sxb = (oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d) for _ in range(3))
    x, rx, sx = bf16_tensor(torch, xb), bf16_tensor(torch, rxb), bf16_tensor(torch, sxb)
    hid = np.full((t, d + pad), oracle.bf16_bits(np.float32(-25.0)), np.uint16)
    hid[:, :d] = oracle.bf16_bits(g.uniform(-1.0, 1.0, t * d)).reshape(t, d)
    tw2, tw1 = (bf16_tensor(torch, oracle.bf16_bits(g.uniform(0.5, 1.5, d))) for _ in range(2))
    if mode == "router_launches":
        ctx.set_one_launch_routing(False)
    if mode == "no_hand_over":
        ctx.set_handover_timeout(0)
    for layer_s in (0, 1, 2):
        y, idx_a, w_a = ctx.route_verify(0, rx, x)
        h1 = shared.dense_ffn(layer_s, sx)
        hid_a = bf16_tensor(torch, hid)
        ctx.layer_tail(y, h1, hid_a, tw2, tw1, 0.875, 1e-6, d=d)
        idx_b, w_b = ctx.route_verify_shared(shared, 0, layer_s, rx, x, sx)
        hid_b = bf16_tensor(torch, hid)
        ctx.layer_tail_routed_shared(shared, w_b, hid_b, tw2, tw1, 0.875, 1e-6)
        assert np.array_equal(idx_a.cpu().numpy(), idx_b.cpu().numpy()) and np.array_equal(bits_of(w_a), bits_of(w_b))
        got, want = bits_of(hid_b), bits_of(hid_a)[:, :d]
        assert np.array_equal(got[:, d:], hid[:, d:])
        if layer_s == 0:
            assert float(h1.abs().max()) == 0.0
            assert np.array_equal(got[:, :d], want)
        else:
            gf, wf = oracle.bf16_to_float(got[:, :d]), oracle.bf16_to_float(want)
            assert rel_err(gf, wf) < 1e-2 and cosine(gf, wf) > 0.9999, (layer_s, rel_err(gf, wf), cosine(gf, wf))
            assert np.mean(got[:, :d] == want) > 0.8
    # the shared expert's row itself: with the routed rows' norm weight at zero the tail is hidden + norm(h1) scaled
    zero = torch.zeros_like(tw2)
    one = torch.ones_like(tw1)
    hid0 = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    _, w_c = ctx.route_verify_shared(shared, 0, 1, rx, x, sx)
    ctx.layer_tail_routed_shared(shared, w_c, hid0, zero, one, 1.0, 1e-6)
    rows = slice(0, min(t, 3) if d > 1024 else t)
    ref_bits = oracle.bf16_bits(_int8_reference_rows(oracle, parts, sxb[rows]).astype(np.float32))
    n_ref = ref_bits.shape[0]
    want0 = oracle.layer_tail(np.zeros((n_ref, d), np.uint16), ref_bits, np.zeros((n_ref, d), np.uint16), bits_of(zero), bits_of(one),
                              1.0, 1e-6)
    g0, w0 = oracle.bf16_to_float(bits_of(hid0))[rows], oracle.bf16_to_float(want0)
    assert rel_err(g0, w0) < 1e-2 and cosine(g0, w0) > 0.9999, (rel_err(g0, w0), cosine(g0, w0))
    if mode == "no_hand_over":
        assert ctx.handover_giveups() > 0
    elif mode == "one_launch":
        assert ctx.handover_giveups() == 0
    ctx.close()
    shared.close()
