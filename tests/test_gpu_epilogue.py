"""Post-attention setup and layer tail through the C ABI: bit-exact against the CPU oracle (which pins this
build's summation order), on the reference tests' seeds, strides and sentinels. Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of

pytestmark = pytest.mark.gpu

D = 2816          # ArchConfig.gemma4_26B_A4B.hiddenSize
EPS = 1e-6


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available()
    return torch


@pytest.fixture(scope="module")
def ctx(torch):
    import fieldfare_moe as ff
    ff.lib()
    c = ff.Context(128, 64, 4, 2, n_layers=1, max_tokens=16)
    yield c
    c.close()


def _block(oracle, rng, rows, stride, used, sentinel):
    """makeBlock (PrefillLayerTailTests.swift:120-133): sentinel-filled rows with `used` drawn values each."""
    out = np.full((rows, stride), oracle.bf16_bits(np.float32(sentinel)), np.uint16)
    for r in range(rows):
        out[r, :used] = oracle.bf16_bits(rng.uniform(-1.0, 1.0, used))
    return out


def _strided(torch, bits):
    """A CUDA bf16 tensor whose rows sit `bits.shape[1]` elements apart, plus the view of its used columns."""
    return bf16_tensor(torch, bits)


def test_layer_tail_block_matches_rows_and_oracle(ctx, oracle, torch):
    # blockLayerTailMatchesRepeatedFusedRows (PrefillLayerTailTests.swift:11-118): 3 rows, strides D + 9 / 13 / 17,
    # sentinels -21 / -23 / -25, same seed; whole-stride equality also proves the padding was left alone
    rows = 3
    rng = oracle.SplitMix64(0x7A11_B10C)
    h2 = _block(oracle, rng, rows, D + 9, D, -21.0)
    h1 = _block(oracle, rng, rows, D + 13, D, -23.0)
    hidden = _block(oracle, rng, rows, D + 17, D, -25.0)
    w2 = oracle.bf16_bits(rng.uniform(0.5, 1.5, D))
    w1 = oracle.bf16_bits(rng.uniform(0.5, 1.5, D))
    scalar = float(rng.uniform(0.75, 1.25, 1)[0])
    ref = hidden.copy()
    ref[:, :D] = oracle.layer_tail(h2[:, :D], h1[:, :D], hidden[:, :D], w2, w1, scalar, EPS)
    th2, th1, th = (_strided(torch, a) for a in (h2, h1, hidden))
    tw2, tw1 = bf16_tensor(torch, w2), bf16_tensor(torch, w1)
    ctx.layer_tail(th2, th1, th, tw2, tw1, scalar, EPS, d=D)
    assert np.array_equal(bits_of(th), ref)
    assert np.array_equal(bits_of(th2), h2) and np.array_equal(bits_of(th1), h1)
    # one row at a time gives the same bits as the block
    for r in range(rows):
        one = _strided(torch, hidden[r:r + 1])
        ctx.layer_tail(th2[r:r + 1], th1[r:r + 1], one, tw2, tw1, scalar, EPS, d=D)
        assert np.array_equal(bits_of(one)[0], ref[r])
    # 16-byte aligned rows (the fast path) give the same bits as the 2-byte aligned ones
    ah2, ah1, ah = (bf16_tensor(torch, np.ascontiguousarray(a[:, :D])) for a in (h2, h1, hidden))
    ctx.layer_tail(ah2, ah1, ah, tw2, tw1, scalar, EPS, d=D)
    assert np.array_equal(bits_of(ah), ref[:, :D])


def test_post_attn_setup_matches_oracle(ctx, oracle, torch):
    # the reference's real-shape case (FusedPostAttentionSetupTests.swift:11-30: seed, ranges) as row 0 of a
    # 3-row block with odd strides and sentinels (PrefillPostAttentionSetupTests.swift uses the same layout)
    rows = 3
    rng = oracle.SplitMix64(0x9057_A77E)
    hidden = _block(oracle, rng, rows, D + 11, D, -31.0)
    attn = _block(oracle, rng, rows, D + 7, D, -33.0)
    w_post, w_pre, w_pre2 = (oracle.bf16_bits(rng.uniform(0.5, 1.5, D)) for _ in range(3))
    ref_h, ref_dense, ref_routed, ref_router = oracle.post_attn_setup(hidden[:, :D], attn[:, :D], w_post, w_pre, w_pre2, EPS)
    sent = oracle.bf16_bits(np.float32(-35.0))
    outs = [np.full((rows, D + 3 + 2 * i), sent, np.uint16) for i in range(3)]
    th, ta = _strided(torch, hidden), _strided(torch, attn)
    touts = tuple(_strided(torch, o) for o in outs)
    tw = [bf16_tensor(torch, w) for w in (w_post, w_pre, w_pre2)]
    ctx.post_attn_setup(th, ta, *tw, eps=EPS, d=D, out=touts)
    exp_h = hidden.copy()
    exp_h[:, :D] = ref_h
    assert np.array_equal(bits_of(th), exp_h)
    assert np.array_equal(bits_of(ta), attn)
    for got, ref, o in zip(touts, (ref_dense, ref_routed, ref_router), outs):
        exp = o.copy()
        exp[:, :D] = ref
        assert np.array_equal(bits_of(got), exp)
    # aligned rows, allocated outputs: same bits
    ah, aa = (bf16_tensor(torch, np.ascontiguousarray(a[:, :D])) for a in (hidden, attn))
    dense, routed, router = ctx.post_attn_setup(ah, aa, *tw, eps=EPS, d=D)
    assert np.array_equal(bits_of(ah), ref_h)
    assert np.array_equal(bits_of(dense), ref_dense) and np.array_equal(bits_of(routed), ref_routed)
    assert np.array_equal(bits_of(router), ref_router)


@pytest.mark.parametrize("d,rows", [(64, 1), (128, 16), (4096, 5), (2816, 300)])
def test_setup_and_tail_shapes(ctx, oracle, torch, d, rows):
    g = oracle.seed_tree_key(0xE91, f"epilogue-d{d}-r{rows}")
    mk = lambda lo, hi: oracle.bf16_bits(g.uniform(lo, hi, rows * d)).reshape(rows, d)
    hidden, attn, h2, h1 = mk(-2, 2), mk(-1, 1), mk(-1, 1), mk(-3, 3)
    ws = [oracle.bf16_bits(g.uniform(0.5, 1.5, d)) for _ in range(5)]
    tw = [bf16_tensor(torch, w) for w in ws]
    ref_h, ref_dense, ref_routed, ref_router = oracle.post_attn_setup(hidden, attn, ws[0], ws[1], ws[2], EPS)
    th = bf16_tensor(torch, hidden)
    dense, routed, router = ctx.post_attn_setup(th, bf16_tensor(torch, attn), tw[0], tw[1], tw[2], eps=EPS, d=d)
    assert np.array_equal(bits_of(th), ref_h)
    assert np.array_equal(bits_of(dense), ref_dense) and np.array_equal(bits_of(routed), ref_routed)
    assert np.array_equal(bits_of(router), ref_router)
    ref_t = oracle.layer_tail(h2, h1, ref_h, ws[3], ws[4], 0.875, EPS)
    ctx.layer_tail(bf16_tensor(torch, h2), bf16_tensor(torch, h1), th, tw[3], tw[4], 0.875, EPS, d=d)
    assert np.array_equal(bits_of(th), ref_t)


def test_epilogue_argument_errors(ctx, torch):
    import fieldfare_moe as ff
    x = torch.zeros((2, 136), dtype=torch.bfloat16, device="cuda")
    w = torch.ones((136,), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ff.FieldfareError, match="multiple of 8"):
        ctx.layer_tail(x, x, x.clone(), w, w, 1.0, d=100)
    with pytest.raises(ff.FieldfareError, match="multiple of 8"):
        ctx.post_attn_setup(x.clone(), x, w, w, w, d=4104)
    with pytest.raises(ff.FieldfareError, match="stride is too small"):
        ctx.layer_tail(torch.zeros((2, 64), dtype=torch.bfloat16, device="cuda"), x, x.clone(), w, w, 1.0, d=136)


def test_layer_tail_with_norms_equals_separate_steps(ctx, oracle, torch):
    # fusedLayerTailNorms_matchSeparateDispatchesAndReference (FusedLayerTailTests.swift:15-93): same seed and
    # ranges; the fused call equals rmsnorm(h1) -> tail -> rmsnorm(hidden) bit for bit, on the GPU and in the
    # oracle, and leaves h1 as it found it
    rng = oracle.SplitMix64(0x7A11_0001)
    h2 = oracle.bf16_bits(rng.uniform(-1, 1, D))[None, :]
    h1 = oracle.bf16_bits(rng.uniform(-3, 3, D))[None, :]
    hidden = oracle.bf16_bits(rng.uniform(-2, 2, D))[None, :]
    w = [oracle.bf16_bits(rng.uniform(0.5, 1.5, D)) for _ in range(4)]      # post 1, post 2, post, next input
    scalar = float(rng.uniform(0.75, 1.25, 1)[0])
    tw = [bf16_tensor(torch, x) for x in w]
    # separate steps on the GPU
    h1n = ctx.rmsnorm(bf16_tensor(torch, h1), tw[0], EPS, d=D)
    sep_hidden = bf16_tensor(torch, hidden)
    ctx.layer_tail(bf16_tensor(torch, h2), h1n, sep_hidden, tw[1], tw[2], scalar, EPS, d=D)
    sep_normed = ctx.rmsnorm(sep_hidden, tw[3], EPS, d=D)
    # the oracle's chain
    ref_h1n = oracle.rmsnorm(h1, w[0], EPS)
    ref_hidden = oracle.layer_tail(h2, ref_h1n, hidden, w[1], w[2], scalar, EPS)
    ref_normed = oracle.rmsnorm(ref_hidden, w[3], EPS)
    assert np.array_equal(bits_of(h1n), ref_h1n)
    assert np.array_equal(bits_of(sep_hidden), ref_hidden) and np.array_equal(bits_of(sep_normed), ref_normed)
    # fused
    th1, fused_hidden = bf16_tensor(torch, h1), bf16_tensor(torch, hidden)
    normed = ctx.layer_tail_norms(bf16_tensor(torch, h2), th1, fused_hidden, tw[0], tw[1], tw[2], scalar, w_next=tw[3], eps=EPS, d=D)
    assert np.array_equal(bits_of(fused_hidden), ref_hidden) and np.array_equal(bits_of(normed), ref_normed)
    assert np.array_equal(bits_of(th1), h1)
    # without a next layer; several rows; rows that are only 2-byte aligned
    rows = 3
    blk = lambda lo, hi, stride: np.concatenate([oracle.bf16_bits(rng.uniform(lo, hi, rows * D)).reshape(rows, D),
                                                 np.full((rows, stride - D), 0xC1A8, np.uint16)], axis=1)
    bh2, bh1, bhid = blk(-1, 1, D + 9), blk(-3, 3, D + 13), blk(-2, 2, D + 17)
    ref = oracle.layer_tail(bh2[:, :D], oracle.rmsnorm(bh1[:, :D], w[0], EPS), bhid[:, :D], w[1], w[2], scalar, EPS)
    tb = bf16_tensor(torch, bhid)
    assert ctx.layer_tail_norms(bf16_tensor(torch, bh2), bf16_tensor(torch, bh1), tb, tw[0], tw[1], tw[2], scalar, eps=EPS, d=D) is None
    exp = bhid.copy()
    exp[:, :D] = ref
    assert np.array_equal(bits_of(tb), exp)


def test_rmsnorm_rows_in_place_and_unit_rms(ctx, oracle, torch):
    g = oracle.seed_tree_key(0x2A5, "rmsnorm")
    for d, rows in ((64, 1), (2816, 16), (4096, 3)):
        xb = oracle.bf16_bits(g.uniform(-4, 4, rows * d)).reshape(rows, d)
        wb = oracle.bf16_bits(g.uniform(0.5, 1.5, d))
        x = bf16_tensor(torch, xb)
        out = ctx.rmsnorm(x, bf16_tensor(torch, wb), EPS, d=d)
        ref = oracle.rmsnorm(xb, wb, EPS)
        assert np.array_equal(bits_of(out), ref)
        ctx.rmsnorm(x, bf16_tensor(torch, wb), EPS, d=d, out=x)               # in place
        assert np.array_equal(bits_of(x), ref)
        unit = oracle.bf16_to_float(bits_of(ctx.rmsnorm(bf16_tensor(torch, xb), bf16_tensor(torch, oracle.bf16_bits(np.ones(d, np.float32))), 0.0, d=d)))
        assert np.allclose(np.sqrt((unit.astype(np.float64) ** 2).mean(axis=1)), 1.0, atol=3e-3)


@pytest.mark.parametrize("act", ["fp16", "bf16"])
def test_rmsnorm_reference_case_hidden_size(oracle, torch, act):
    import fieldfare_moe as ff
    # rmsNorm_matchesReference_hiddenSize (RMSNormTests.swift:19-45): same seed, label and draw order (x, then the bf16
    # weight), FP16 rows as there (and bf16 rows), against the un-rounded norm within Tolerance.fp16Reduction = 5e-3
    d = 2816
    rng = oracle.seed_tree_key(0xD4, f"rmsnorm-d{d}-weighted=true")
    xv = rng.uniform(-1.0, 1.0, d).astype(np.float32)
    wb = oracle.bf16_bits(rng.uniform(0.5, 1.5, d))
    c = ff.Context(128, 64, 16, 8, n_layers=1, max_tokens=16, act_dtype=act)
    if act == "fp16":
        x = torch.from_numpy(xv.astype(np.float16)[None, :]).cuda()
        x64 = xv.astype(np.float16).astype(np.float64)
    else:
        x = bf16_tensor(torch, oracle.bf16_bits(xv)[None, :])
        x64 = oracle.bf16_to_float(oracle.bf16_bits(xv)).astype(np.float64)
    out = c.rmsnorm(x, bf16_tensor(torch, wb), 1e-6, d=d)
    got = out.float().cpu().numpy()[0].astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean() + 1e-6) * oracle.bf16_to_float(wb).astype(np.float64)
    rel = np.abs(got - ref).max() / np.abs(ref).max()
    assert rel < 5e-3, rel
    c.close()
