"""Resident INT4 matrix (LM head): re-tiling, multi-row GEMV and greedy choice against the CPU oracle,
through the C ABI. Run on the GPU box: pytest -m gpu."""
import numpy as np
import pytest

from helpers import bf16_tensor, bits_of, rel_err

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


@pytest.fixture(scope="module")
def ctx(ff, torch):
    c = ff.Context(128, 64, 16, 8, n_layers=1, max_tokens=16)
    yield c
    c.close()


def _i16(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


@pytest.mark.parametrize("m,n,rows,off,src", [(300, 2112, 3, 0, "host"), (301, 2816, 4, 2, "device"),
                                              (256, 2112, 12, 0, "device"), (384, 2816, 13, 0, "host"),
                                              (1408, 2816, 1, 0, "device"), (1408, 2816, 16, 0, "device"),
                                              (64, 128, 1, 0, "host"), (4099, 2816, 4, 0, "device")])
def test_matrix_gemv_reference_shapes(ctx, oracle, torch, m, n, rows, off, src):
    # DequantInt4SmallBatchTests.swift:66-119 shapes (incl. the 2-byte weight offset), config 1 (1408 x 2816),
    # StreamingKernelIntegrationTests.swift:84-161 (64 x 128) and the 4,099-row head of
    # LMHeadChainInt4Tests.swift:118-160; the weight comes from host memory or from device memory
    g = oracle.seed_tree_key(0xE1 + rows, f"matrix-m{m}-n{n}-r{rows}-off{off}")
    W, S, B = oracle.quantize_int4(g.uniform(-0.5, 0.5, m * n).reshape(m, n))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * n)).reshape(rows, n)
    raw = np.concatenate([np.zeros(off, np.uint8), W.ravel()])
    if src == "device":
        mx = ctx.matrix(torch.from_numpy(raw).cuda(), _i16(torch, S), _i16(torch, B), w_byte_offset=off)
    else:
        mx = ctx.matrix(raw, S, B, w_byte_offset=off)
    x = bf16_tensor(torch, xb)
    y16 = bits_of(mx.gemv(x))
    y32 = mx.gemv(x, f32_out=True).cpu().numpy()
    for r in range(rows):
        ref = oracle.gemv_int4_ref(W, S, B, oracle.bf16_to_float(xb[r]))
        assert rel_err(y32[r], ref) < 5e-3, f"row {r}"         # Tolerance.fp16Reduction on the unrounded sum
        assert rel_err(oracle.bf16_to_float(y16[r]), ref) < 1e-2, f"row {r}"
        # the 16-bit output is the rounding of the fp32 output
        assert np.array_equal(y16[r], oracle.bf16_bits(y32[r]))
    # row r of a multi-row call equals the single-row call bit for bit (matchesSingleRowGEMVBitwise)
    for r in range(rows):
        single = mx.gemv(x[r:r + 1], f32_out=True).cpu().numpy()[0]
        assert np.array_equal(single.view(np.uint32), y32[r].view(np.uint32)), f"row {r}"
    mx.close()


def test_matrix_equals_raw_layout_gemv(ctx, oracle, torch):
    # the same weight through the reference-layout GEMV and through the resident tiles
    m, n, rows = 512, 1408, 5
    g = oracle.SplitMix64(77)
    W, S, B = oracle.quantize_int4(g.uniform(-0.4, 0.4, m * n).reshape(m, n))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * n)).reshape(rows, n)
    x = bf16_tensor(torch, xb)
    mx = ctx.matrix(W, S, B)
    a = mx.gemv(x, f32_out=True).cpu().numpy()
    b = ctx.gemv_int4(torch.from_numpy(W).cuda(), _i16(torch, S), _i16(torch, B), x, f32_out=True).cpu().numpy()
    assert rel_err(a, b) < 1e-4
    mx.close()


def _cpu_greedy(oracle, W, S, B, x_f32):
    # cpuGreedy of LMHeadChainInt4Tests.swift:10-39 after its RMSNorm: first strictly larger dot wins
    return int(np.argmax(oracle.gemv_int4_ref(W, S, B, x_f32)))


def test_greedy_matches_cpu_reference(ctx, oracle, torch):
    # rawGreedyMatchesCPUReference (LMHeadChainInt4Tests.swift:77-100): d = 64, v = 1024, same seed
    d, v = 64, 1024
    rng = oracle.SplitMix64(0x1A4E_4EAD_2026_0603)
    hidden = rng.uniform(-1.0, 1.0, d)
    rng.uniform(0.5, 1.5, d)                                # the norm weights of the Swift test: drawn, not used here
    W, S, B = oracle.quantize_int4(np.stack([rng.uniform(-1.0, 1.0, d) for _ in range(v)]))
    xb = oracle.bf16_bits(hidden)
    mx = ctx.matrix(W, S, B, greedy=True)
    got = int(mx.greedy(bf16_tensor(torch, xb[None, :]))[0])
    logits = oracle.gemv_int4_ref(W, S, B, oracle.bf16_to_float(xb))
    order = np.argsort(-logits)
    assert logits[order[0]] - logits[order[1]] > 1e-4       # the case is not a near-tie
    assert got == order[0] == _cpu_greedy(oracle, W, S, B, oracle.bf16_to_float(xb))
    mx.close()


def test_greedy_ties_and_non_finite(ctx, oracle, torch):
    # tiesResolveToLowestIndex (LMHeadChainInt4Tests.swift:102-116): rows 17 and 311 carry the same weights
    d, v = 64, 1024
    hidden = np.array([0.2 + (i % 5) * 0.02 for i in range(d)], np.float32)
    rows = np.full((v, d), -0.25, np.float32)
    rows[17] = rows[311] = 1.0
    W, S, B = oracle.quantize_int4(rows)
    x = bf16_tensor(torch, oracle.bf16_bits(hidden)[None, :])
    mx = ctx.matrix(W, S, B, greedy=True)
    assert int(mx.greedy(x)[0]) == 17
    mx.close()
    # a row whose logit is +inf or NaN never wins (logit.metal:916-921): scale = +inf makes row 5 non-finite
    S2, B2 = S.copy(), B.copy()
    S2[5, 0] = 0x7F80
    S2[9, 0] = 0x7FC0
    mx = ctx.matrix(W, S2, B2, greedy=True)
    logits = mx.gemv(x, f32_out=True).cpu().numpy()[0]
    assert not np.isfinite(logits[5]) and not np.isfinite(logits[9])
    assert int(mx.greedy(x)[0]) == 17
    mx.close()


def test_greedy_rows_large_head(ctx, oracle, torch):
    # decode's shape (D = 2816) against a 4,099-row head with a tied pair, four rows at once
    # (checkAndHotGuessMatchSingleRowHead, LMHeadChainInt4Tests.swift:118-160)
    d, v, rows = 2816, 4099, 4
    rng = oracle.SplitMix64(0xC4EC_4EAD)
    Wf = rng.uniform(-1.0, 1.0, v * d).reshape(v, d)
    Wf[4001] = Wf[1203]                                     # a tied pair: the lower index must win when it leads
    W, S, B = oracle.quantize_int4(Wf)
    xb = oracle.bf16_bits(rng.uniform(-1.0, 1.0, rows * d)).reshape(rows, d)
    xb[2] = oracle.bf16_bits(oracle.dequantize_int4(W[1203:1204], S[1203:1204], B[1203:1204])[0])   # row 2 points at the pair
    mx = ctx.matrix(W, S, B, greedy=True)
    got = mx.greedy(bf16_tensor(torch, xb)).cpu().numpy()
    for r in range(rows):
        logits = oracle.gemv_int4_ref(W, S, B, oracle.bf16_to_float(xb[r]))
        order = np.argsort(-logits, kind="stable")
        if order[0] in (1203, 4001):
            assert got[r] == 1203
        else:
            assert logits[order[0]] - logits[order[1]] > 1e-3 * abs(logits[order[0]])
            assert got[r] == order[0]
    assert got[2] == 1203
    mx.close()


def test_matrix_argument_errors(ctx, ff, oracle, torch):
    W, S, B = oracle.quantize_int4(np.zeros((32, 64), np.float32))
    with pytest.raises(ff.FieldfareError, match="at most"):
        big = np.zeros((32, 2880 // 2), np.uint8)
        ctx.matrix(big, np.zeros((32, 45), np.uint16), np.zeros((32, 45), np.uint16))
    mx = ctx.matrix(W, S, B)
    x = torch.zeros((1, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ff.FieldfareError, match="greedy scratch"):
        mx.greedy(x)
    with pytest.raises(ff.FieldfareError, match="outside 1...16"):
        mx.gemv(torch.zeros((17, 64), dtype=torch.bfloat16, device="cuda"))
    mx.close()


@pytest.mark.parametrize("softcap", [0.0, 30.0, 1.5])
def test_argmax_rows_choice_and_confidence(ctx, oracle, torch, softcap):
    # argmax_rows_f32 (logit.metal:946-1010): first maximum among the finite values, 0xFFFFFFFF without one; the
    # winner's probability under the softcap against the float64 restatement (the sums' order is the kernel's own)
    rng = np.random.default_rng(41)
    rows = rng.normal(0, 4, (7, 4099)).astype(np.float32)
    rows[1, 17] = rows[1, 311] = rows[1].max() + 1.0
    rows[2, :5] = [np.inf, -np.inf, np.nan, 1e30, -1e30]
    rows[3, :] = np.nan
    rows[4, :] = -7.25
    rows[5, 4098] = 99.0                                       # the winner in the last position
    padded = np.full((7, 4099 + 5), 1e9, np.float32)           # a row stride beyond the count: the padding is not looked at
    padded[:, :4099] = rows
    want_tok, want_conf = oracle.greedy_choice_rows(rows, softcap)
    tok, conf = ctx.argmax_rows(torch.from_numpy(padded).cuda()[:, :4099], softcap=softcap)
    assert np.array_equal(tok.cpu().numpy().astype(np.uint32), want_tok)
    assert np.abs(conf.cpu().numpy() - want_conf).max() <= 1e-5 + 1e-4 * want_conf.max()
    only = ctx.argmax_rows(torch.from_numpy(padded).cuda()[:, :4099], softcap=softcap, want_conf=False)
    assert np.array_equal(only.cpu().numpy().astype(np.uint32), want_tok)


def test_greedy_conf_and_hot_vocabulary_choice(ctx, oracle, torch):
    # LMHeadChainInt4.encodeGreedyRows with its confidence output, and encodeHotGreedyRows (LMHeadChainInt4.swift:
    # 94-186): the choice over the listed rows of the head, mapped back through the list, equals the full head's
    # whenever the list holds the full head's winner; positions follow the list's order
    m, n, rows = 4099, 2816, 5
    g = oracle.seed_tree_key(0x1A4E, "head-conf")
    W, S, B = oracle.quantize_int4(g.uniform(-0.5, 0.5, m * n).reshape(m, n))
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * n)).reshape(rows, n)
    x = bf16_tensor(torch, xb)
    Wd, Sd, Bd = torch.from_numpy(W).cuda(), _i16(torch, S), _i16(torch, B)
    head = ctx.matrix(Wd, Sd, Bd, greedy=True)
    logits = head.gemv(x, f32_out=True).cpu().numpy()
    plain = head.greedy(x).cpu().numpy()
    for cap in (0.0, 30.0):
        tok, conf = head.greedy_conf(x, softcap=cap)
        want_tok, want_conf = oracle.greedy_choice_rows(logits, cap)
        assert np.array_equal(tok.cpu().numpy().astype(np.uint32), want_tok) and np.array_equal(tok.cpu().numpy(), plain)
        assert np.abs(conf.cpu().numpy() - want_conf).max() <= 1e-5 + 1e-4 * want_conf.max()
    # hot vocabulary: 512 listed rows in a shuffled order that hold every row's winner
    rng = np.random.default_rng(5)
    ids = np.unique(np.concatenate([plain.astype(np.int64), rng.choice(m, 512, replace=False)]))
    rng.shuffle(ids)
    ids_d = torch.from_numpy(ids.astype(np.int32)).cuda()
    listed = ctx.gemv_int4_listed(Wd, Sd, Bd, ids_d, x)
    pos, conf = ctx.argmax_rows(listed)
    pos = pos.cpu().numpy()
    assert np.array_equal(ids[pos], plain)
    want_pos, want_conf = oracle.greedy_choice_rows(listed.cpu().numpy(), 0.0)
    assert np.array_equal(pos.astype(np.uint32), want_pos)
    assert np.abs(conf.cpu().numpy() - want_conf).max() <= 1e-5 + 1e-4 * want_conf.max()
    head.close()


def _assert_draws(tok, prob, want_tok, want_prob, gap, what):
    """Positions equal wherever the oracle's winning margin is beyond float rounding of the log / tanh the two machines
    evaluate (a closer call may fall either way); nearly all rows must be of the first kind."""
    tok = tok.cpu().numpy().astype(np.uint32)
    clear = gap > 1e-4
    assert clear.mean() >= 0.9, (what, gap)
    assert np.array_equal(tok[clear], want_tok[clear]), (what, tok, want_tok, gap)
    p = prob.cpu().numpy().astype(np.float64)
    same = tok == want_tok
    assert (np.abs(p[same] - want_prob[same]) <= 1e-5 + 2e-3 * want_prob[same]).all(), (what, p, want_prob)


@pytest.mark.parametrize("count,temperature,top_k,top_p", [(4099, 1.0, 0, 1.0), (4099, 0.7, 0, 1.0), (300, 1.3, 0, 1.0),
                                                           (4099, 1.0, 64, 1.0), (4099, 0.8, 40, 0.9), (4099, 1.0, 256, 0.95),
                                                           (300, 1.0, 256, 0.5), (200, 1.0, 256, 0.9), (70000, 0.9, 50, 0.9)])
def test_sample_rows_draw_and_probability(ctx, oracle, torch, count, temperature, top_k, top_p):
    """ffmoe_sample_rows against the restated sample_rows_f32 (logit.metal:1010-1259): same drawn position and
    probability per row, without truncation and with top_k / top_p; rows with ties at the top_k edge (equal values:
    the lower positions survive), non-finite entries, fewer finite entries than top_k, nothing finite at all; a
    row stride beyond the count."""
    rng = np.random.default_rng(count + top_k)
    rows = rng.normal(0, 4, (16, count)).astype(np.float32)
    rows[1] = np.round(rows[1])                               # many equal values: the edge of the top_k set is a tie
    rows[2, :5] = [np.inf, -np.inf, np.nan, 1e30, -1e30]
    rows[3, :] = np.nan
    rows[4, 30:] = -np.inf                                     # 30 finite entries
    rows[5, :] = 2.5                                           # all equal: the lowest top_k positions survive
    padded = np.full((16, count + 3), 1e9, np.float32)
    padded[:, :count] = rows
    logits = torch.from_numpy(padded).cuda()[:, :count]
    want_tok, want_prob, gap = oracle.sample_rows(rows, temperature, top_p, top_k, key_base=100, softcap=30.0, seed=0xFEED_F00D)
    tok, prob = ctx.sample_rows(logits, temperature, 30.0, 0xFEED_F00D, key_base=100, top_k=top_k, top_p=top_p)
    assert tok.cpu().numpy()[3] == -1 and float(prob[3]) == 0.0
    _assert_draws(tok, prob, want_tok, want_prob, gap, (count, temperature, top_k, top_p))


def test_sample_rows_ids_key_offset_and_position_keys(ctx, oracle, torch):
    # the noise follows the token id (ids) and the position (key_base + key_offset[0] + row)
    rng = np.random.default_rng(77)
    count = 1000
    rows = rng.normal(0, 3, (8, count)).astype(np.float32)
    ids = rng.permutation(50000)[:count].astype(np.uint32)
    logits = torch.from_numpy(rows).cuda()
    tids = torch.from_numpy(ids.astype(np.int32)).cuda()
    koff = torch.tensor([12345], dtype=torch.int32, device="cuda")
    for top_k, top_p in ((0, 1.0), (32, 0.9)):
        want_tok, want_prob, gap = oracle.sample_rows(rows, 0.9, top_p, top_k, key_base=7, softcap=30.0, seed=3, ids=ids, key_offset=12345)
        tok, prob = ctx.sample_rows(logits, 0.9, 30.0, 3, key_base=7, top_k=top_k, top_p=top_p, ids=tids, key_offset=koff)
        _assert_draws(tok, prob, want_tok, want_prob, gap, ("ids", top_k))
        # without the ids the draws differ (other noise), with the offset folded into the base they are the same
        tok2, _ = ctx.sample_rows(logits, 0.9, 30.0, 3, key_base=7 + 12345, top_k=top_k, top_p=top_p, ids=tids)
        assert np.array_equal(tok2.cpu().numpy(), tok.cpu().numpy())
    # the same position drawn as row 3 of a block and as row 0 of a later call: the same token
    blk, _ = ctx.sample_rows(logits[:4], 1.0, 30.0, 9, key_base=50)
    one, _ = ctx.sample_rows(logits[3:4], 1.0, 30.0, 9, key_base=53)
    assert int(blk[3]) == int(one[0])


def test_sample_rows_full_vocabulary_row(ctx, oracle, torch):
    # a 262,144-entry row (the LM head's), top-64 / top-p 0.9 and the plain draw
    rng = np.random.default_rng(5)
    rows = rng.normal(0, 3, (2, 262144)).astype(np.float32)
    logits = torch.from_numpy(rows).cuda()
    for top_k, top_p in ((64, 0.9), (0, 1.0)):
        want_tok, want_prob, gap = oracle.sample_rows(rows, 0.8, top_p, top_k, key_base=1, softcap=30.0, seed=17)
        tok, prob = ctx.sample_rows(logits, 0.8, 30.0, 17, key_base=1, top_k=top_k, top_p=top_p)
        _assert_draws(tok, prob, want_tok, want_prob, gap, ("vocab", top_k))


def test_sample_rows_argument_errors(ctx, ff, torch):
    logits = torch.zeros((2, 64), dtype=torch.float32, device="cuda")
    for kwargs, match in ((dict(temperature=0.0, softcap=30.0), "temperature"), (dict(temperature=1.0, softcap=0.0), "softcap"),
                          (dict(temperature=1.0, softcap=30.0, top_k=257), "top_k"),
                          (dict(temperature=1.0, softcap=30.0, top_k=8, top_p=0.0), "top_p")):
        with pytest.raises(ff.FieldfareError, match=match):
            ctx.sample_rows(logits, kwargs["temperature"], kwargs["softcap"], 1, top_k=kwargs.get("top_k", 0), top_p=kwargs.get("top_p", 1.0))


# ---- the 8-bit affine matrix and the 8-bit shared expert built from it ------------------------------------------

def _shared_int8(ctx, parts):
    (gW, gS, gB), (uW, uS, uB), (dW, dS, dB) = parts
    return ctx.matrix_int8(gW, gS, gB), ctx.matrix_int8(uW, uS, uB), ctx.matrix_int8(dW, dS, dB)


def _shared_int8_rows(ctx, mats, x):
    gate, up, down = mats
    return down.gemv(ctx.gelu_mul(gate.gemv(x), up.gemv(x)))


def _shared_int8_reference(oracle, parts, x_rows, widen, narrow):
    """SharedExpertInt8Tests.swift:33-41: DequantInt8GemvRef for gate and up, gelu_pytorch_tanh(gate) * up rounded to 16
    bits once, DequantInt8GemvRef for down."""
    (gW, gS, gB), (uW, uS, uB), (dW, dS, dB) = parts
    out = []
    for row in x_rows:
        x = widen(row)
        g, u = oracle.gemv_int8_ref(gW, gS, gB, x), oracle.gemv_int8_ref(uW, uS, uB, x)
        g64 = g.astype(np.float64)
        act = (0.5 * g64 * (1.0 + np.tanh(0.7978845608028654 * (g64 + 0.044715 * g64 ** 3)))).astype(np.float32) * u
        out.append(oracle.gemv_int8_ref(dW, dS, dB, widen(narrow(act))))
    return np.stack(out)


@pytest.mark.parametrize("act", ["bf16", "fp16"])
def test_shared_expert_int8_matches_reference(ff, oracle, torch, act):
    # sharedExpertInt8_matchesReference (SharedExpertInt8Tests.swift:19-72): same seed, draw order, shapes and reference;
    # the reference's bound is Tolerance.quantInt8 * 4 = 4e-3 on FP16 outputs, bf16 outputs carry 2^-9 on top
    d, f = 128, 64
    rng = oracle.seed_tree_key(0x601, "shared-expert-int8")
    x = rng.uniform(-0.4, 0.4, d)
    gate = np.stack([rng.uniform(-0.4, 0.4, d) for _ in range(f)])
    up = np.stack([rng.uniform(-0.4, 0.4, d) for _ in range(f)])
    down = np.stack([rng.uniform(-0.4, 0.4, f) for _ in range(d)])
    parts = (oracle.quantize_int8(gate), oracle.quantize_int8(up), oracle.quantize_int8(down))
    c = ff.Context(128, 64, 16, 8, n_layers=1, max_tokens=16, act_dtype=act)
    if act == "fp16":
        widen = lambda b: np.ascontiguousarray(b, np.uint16).view(np.float16).astype(np.float32)
        narrow = lambda v: np.ascontiguousarray(v, np.float32).astype(np.float16).view(np.uint16)
        xt = torch.from_numpy(narrow(x)[None, :].view(np.int16)).cuda().view(torch.float16)
    else:
        widen, narrow = oracle.bf16_to_float, oracle.bf16_bits
        xt = bf16_tensor(torch, narrow(x)[None, :])
    ref = _shared_int8_reference(oracle, parts, narrow(x)[None, :], widen, narrow)
    mats = _shared_int8(c, parts)
    y = widen(bits_of(_shared_int8_rows(c, mats, xt)))
    assert rel_err(y, ref) < (4e-3 if act == "fp16" else 1e-2), rel_err(y, ref)
    for m_ in mats:
        m_.close()
    c.close()


@pytest.mark.parametrize("act", ["bf16", "fp16"])
@pytest.mark.parametrize("f,d,rows", [(64, 128, 1), (2112, 2816, 16), (100, 192, 5), (8, 64, 16), (33, 704, 3)])
def test_int8_gated_matrix_equals_separate_calls(ff, oracle, torch, act, f, d, rows):
    # the fused gate / up / activation pass (shared_int8_gate_up_act_simd, dequant_int8.metal:84-140) against the three
    # separate calls, bit for bit: F a multiple of 16 and not, one row to sixteen, sources on the host and on the device
    g = np.random.default_rng(f * 131 + d + rows)
    gate = oracle.quantize_int8(g.uniform(-0.4, 0.4, (f, d)).astype(np.float32))
    up = oracle.quantize_int8(g.uniform(-0.4, 0.4, (f, d)).astype(np.float32))
    c = ff.Context(128, 64, 16, 8, n_layers=1, max_tokens=16, act_dtype=act)
    xv = g.uniform(-0.5, 0.5, (rows, d)).astype(np.float32)
    x = (torch.from_numpy(xv.astype(np.float16)).cuda() if act == "fp16" else bf16_tensor(torch, oracle.bf16_bits(xv)))
    mg, mu = c.matrix_int8(*gate), c.matrix_int8(*up)
    want = c.gelu_mul(mg.gemv(x), mu.gemv(x))
    fused = c.matrix_int8_glu(gate, up)
    assert fused.m == f
    got = fused.gemv(x)
    assert got.shape == (rows, f) and torch.equal(got.view(torch.int16), want.view(torch.int16))
    on_device = lambda t: tuple(torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in t)
    fused_dev = c.matrix_int8_glu(on_device(gate), on_device(up))
    assert torch.equal(fused_dev.gemv(x).view(torch.int16), want.view(torch.int16))
    # fp32 out: the un-rounded product of the two rounded projections
    g32 = fused.gemv(x, f32_out=True)
    step = 2.0 ** -11 if act == "fp16" else 2.0 ** -8
    assert g32.dtype == torch.float32 and ((g32 - want.float()).abs() <= step * g32.abs() + 1e-6).all()
    with pytest.raises(ff.FieldfareError):
        fused.greedy(x)
    for m_ in (mg, mu, fused, fused_dev):
        m_.close()
    c.close()


def test_int8_matrix_block_equals_repeated_single_rows(ctx, oracle, torch):
    # blockSharedExpertMatchesRepeatedScalarRows (PrefillSharedExpertTests.swift:15-82): four rows with an input stride of
    # 144 and an output stride of 137 over sentinels - the block call equals the four single-row calls bit for bit,
    # padding included (here per projection: every stage of the expert is such a call)
    import ctypes as C
    rows, d, f, xs, ys = 4, 128, 64, 144, 137
    rng = oracle.seed_tree_key(0xC0FFEE, "prefill-shared-expert")
    sentinel = oracle.bf16_bits(np.float32(-7.25))
    xb = np.full((rows, xs), sentinel, np.uint16)
    for r in range(rows):
        xb[r, :d] = oracle.bf16_bits(rng.uniform(-0.35, 0.35, d))
    W, S, B = oracle.quantize_int8(np.stack([rng.uniform(-0.4, 0.4, d) for _ in range(f)]))
    mx = ctx.matrix_int8(W, S, B)
    x = bf16_tensor(torch, xb)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def run(first, count):
        y = bf16_tensor(torch, np.full((rows, ys), sentinel, np.uint16))
        err = C.c_char_p()
        for r in (range(first, first + count) if count == 1 else [first]):
            n = 1 if count == 1 else count
            rc = ctx.L.ffmoe_matrix_gemv(mx._h, stream, C.c_void_p(x.data_ptr() + r * xs * 2), xs, n,
                                         C.c_void_p(y.data_ptr() + r * ys * 2), ys, 0, C.byref(err))
            assert rc == 0, err.value
        return y

    block = run(0, rows)
    single = bf16_tensor(torch, np.full((rows, ys), sentinel, np.uint16))
    for r in range(rows):
        single[r] = run(r, 1)[r]
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(block), bits_of(single))
    assert np.array_equal(bits_of(block)[:, f:], np.full((rows, ys - f), sentinel, np.uint16))
    ref = np.stack([oracle.gemv_int8_ref(W, S, B, oracle.bf16_to_float(xb[r, :d])) for r in range(rows)])
    assert rel_err(oracle.bf16_to_float(bits_of(block)[:, :f]), ref) < 1e-2
    mx.close()


@pytest.mark.parametrize("m,n,rows", [(2112, 2816, 1), (2112, 2816, 16), (2816, 2112, 16), (300, 2112, 3), (17, 64, 5)])
def test_int8_matrix_gemv_shapes(ctx, ff, oracle, torch, m, n, rows):
    # the 26B-A4B shared expert's projections (gate / up 2112 x 2816, down 2816 x 2112: DequantInt8GEMV.swift:12-19) and
    # ragged row counts; fp32 outputs against the float64 reference, 16-bit outputs = their rounding, row r of a block
    # = the single-row call bit for bit; q = 0 and q = 255 in every group exercise both nibble planes' ends
    g = oracle.seed_tree_key(0xE8 + rows, f"matrix8-m{m}-n{n}-r{rows}")
    W, S, B = oracle.quantize_int8(g.uniform(-0.5, 0.5, m * n).reshape(m, n))
    assert W.min() == 0 and W.max() == 255
    xb = oracle.bf16_bits(g.uniform(-1.0, 1.0, rows * n)).reshape(rows, n)
    mx = ctx.matrix_int8(torch.from_numpy(W).cuda(), _i16(torch, S), _i16(torch, B)) if rows % 2 else ctx.matrix_int8(W, S, B)
    x = bf16_tensor(torch, xb)
    y32 = mx.gemv(x, f32_out=True).cpu().numpy()
    y16 = bits_of(mx.gemv(x))
    for r in range(rows):
        ref = oracle.gemv_int8_ref(W, S, B, oracle.bf16_to_float(xb[r]))
        assert rel_err(y32[r], ref) < 1e-3, (r, rel_err(y32[r], ref))        # Tolerance.quantInt8
        assert np.array_equal(y16[r], oracle.bf16_bits(y32[r]))
        single = mx.gemv(x[r:r + 1], f32_out=True).cpu().numpy()[0]
        assert np.array_equal(single.view(np.uint32), y32[r].view(np.uint32)), f"row {r}"
    with pytest.raises(ff.FieldfareError, match="greedy"):
        mx.greedy(x)
    mx.close()


def test_gelu_mul_and_int8_argument_errors(ctx, ff, oracle, torch):
    g = np.random.default_rng(3)
    a, b = (oracle.bf16_bits(g.normal(0, 2, (5, 200)).astype(np.float32)) for _ in range(2))
    a[0, :4] = oracle.bf16_bits(np.array([0.0, -0.0, 30.0, -30.0], np.float32))
    out = bits_of(ctx.gelu_mul(bf16_tensor(torch, a), bf16_tensor(torch, b)))
    x = oracle.bf16_to_float(a).astype(np.float64)
    want = 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3))) * oracle.bf16_to_float(b)
    # the tanh form in float64 (utility.metal:4-17 states it in single precision, where 1 + tanh cancels for inputs
    # below about -4): the kernels' form, x / (1 + exp(-2 * inner)), has no cancellation and follows it to a bf16 step
    assert (np.abs(oracle.bf16_to_float(out) - want) <= 2.0 ** -7 * np.abs(want) + 1e-7).all()
    near = np.abs(x) <= 3.0                            # and the single-precision oracle where that one is accurate
    want32 = oracle.gelu_tanh(oracle.bf16_to_float(a)) * oracle.bf16_to_float(b)
    assert (np.abs(oracle.bf16_to_float(out) - want32)[near] <= 2.0 ** -7 * np.abs(want32)[near] + 1e-7).all()
    ga = bf16_tensor(torch, a)
    assert ctx.gelu_mul(ga, bf16_tensor(torch, b), out=ga) is ga and (bits_of(ga) == out).all()   # in place, over the gate
    W, S, B = oracle.quantize_int8(g.uniform(-1, 1, (8, 100 * 64)).astype(np.float32))
    with pytest.raises(ff.FieldfareError, match="at most"):
        ctx.matrix_int8(W, S, B)                       # N beyond what a wave's register ring holds


def test_final_row_head_matches_scalar_offset_path(ctx, oracle, torch):
    # finalRowHeadLogitsMatchesScalarOffsetPath (PrefillFinalRowHeadTests.swift:31-127): row 3 of a five-row block with a
    # row stride of d + 17 values, norm then head. Same seed, label, draw order and shapes. The block path norms the row
    # where it lies (the 2-byte aligned offset the stride gives) and projects through the resident head; the scalar path
    # norms a copy of the row and projects through the reference-layout GEMV. The reference allows 1e-3 / 1e-4 between
    # them (held here on the fp32 logits); the normed row is the oracle's bit for bit and the logits those of its
    # dequantised rows.
    rows, sel, d, vocab = 5, 3, 128, 96
    stride = d + 17
    rng = oracle.seed_tree_key(0xB501, "prefill-final-row-head")
    hid = np.zeros((rows, stride), np.float32)
    for r in range(rows):
        hid[r, :d] = rng.uniform(-1.0, 1.0, d)
    hb = oracle.bf16_bits(hid)
    nb = oracle.bf16_bits(rng.uniform(0.5, 1.5, d))
    W, S, B = oracle.quantize_int4(np.stack([rng.uniform(-0.5, 0.5, d) for _ in range(vocab)]))
    block = bf16_tensor(torch, hb)
    norm_w = bf16_tensor(torch, nb)
    head = ctx.matrix(W, S, B)
    normed = ctx.rmsnorm(block[sel:sel + 1], norm_w, 1e-6, d=d)                 # read at offset 3 * 145 values
    logits_block = head.gemv(normed, f32_out=True)
    row_copy = block[sel, :d].clone()[None, :]
    Wt, St, Bt = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (W, S.view(np.int16), B.view(np.int16)))
    normed_copy = ctx.rmsnorm(row_copy, norm_w, 1e-6, d=d)
    assert torch.equal(normed.view(torch.int16), normed_copy.view(torch.int16))
    logits_scalar = ctx.gemv_int4(Wt, St, Bt, normed_copy, f32_out=True)
    a, b = logits_block.cpu().numpy()[0], logits_scalar.cpu().numpy()[0]
    assert np.abs(a - b).max() <= 1e-3 and rel_err(a, b) <= 1e-4            # the reference's two bounds
    ref_normed = oracle.rmsnorm(hb[sel:sel + 1, :d], nb, 1e-6)
    assert np.array_equal(bits_of(normed), ref_normed)
    ref = oracle.gemv_int4_ref(W, S, B, oracle.bf16_to_float(ref_normed[0]))
    assert rel_err(a, ref) < 5e-3                                           # Tolerance.fp16Reduction
    head.close()


@pytest.mark.parametrize("act", ["fp16", "bf16"])
def test_embedding_rows_from_the_resident_table(ff, oracle, torch, act):
    # embedLookupInt4_withSqrtDScale_matchesReference (EmbedLookupTests.swift:24-62): same seed, label, table (16 x 128),
    # token 9 and scale sqrt(128); FP16 out as there (and bf16). The reference allows Tolerance.quantInt4; the kernel's
    # expression half((q * s + b) * out_scale) is pinned bit for bit.
    V, D = 16, 128
    rng = oracle.seed_tree_key(0x131, "embed-lookup-int4-table")
    W, S, B = oracle.quantize_int4(np.stack([rng.uniform(-1.0, 1.0, D) for _ in range(V)]))
    c = ff.Context(128, 64, 16, 8, n_layers=1, max_tokens=16, act_dtype=act)
    dtype = oracle.FP16 if act == "fp16" else oracle.BF16
    table = c.matrix(W, S, B)
    scale = np.float32(np.sqrt(np.float32(D)))
    deq = oracle.dequantize_int4(W, S, B)
    want = oracle.bits16(deq * scale, dtype)
    got = bits_of(table.rows(9, float(scale)))
    assert got.shape == (1, D) and np.array_equal(got[0], want[9])
    # a list of ids in device memory: every row, a repeat, and one past the table (a row of zeros)
    ids = torch.tensor(list(range(V)) + [3, V + 5], dtype=torch.int32, device="cuda")
    rows = bits_of(table.rows(ids, float(scale)))
    assert np.array_equal(rows[:V], want) and np.array_equal(rows[V], want[3]) and not rows[V + 1].any()
    assert np.array_equal(bits_of(table.rows(ids, 1.0))[:V], oracle.bits16(deq, dtype))
    table.close()
    # a tall table with an odd row count and the model's width: rows either side of every tile boundary, into a padded output
    g = np.random.default_rng(11)
    m, n = 1000 + 7, 2816
    W, S, B = oracle.quantize_int4(g.uniform(-1.0, 1.0, (m, n)).astype(np.float32))
    table = c.matrix(W, S, B, greedy=True)
    pick = np.array([0, 15, 16, 31, 32, 47, 48, 63, 64, 500, 991, 992, 1005, 1006], np.int32)
    out = torch.full((len(pick), n + 8), -3.0, dtype=c.act, device="cuda")
    table.rows(torch.from_numpy(pick).cuda(), 53.0, out=out)
    want = oracle.bits16(oracle.dequantize_int4(W[pick], S[pick], B[pick]) * np.float32(53.0), dtype)
    got = bits_of(out)
    assert np.array_equal(got[:, :n], want) and (out[:, n:].float() == -3.0).all()
    # the tokens of a greedy choice feed the lookup without leaving the device
    x = torch.from_numpy(g.uniform(-1, 1, (4, n)).astype(np.float32)).cuda().to(c.act)
    tok = table.greedy(x)
    emb = bits_of(table.rows(tok, 1.0))
    t_host = tok.cpu().numpy()
    assert np.array_equal(emb, oracle.bits16(oracle.dequantize_int4(W[t_host], S[t_host], B[t_host]), dtype))
    with pytest.raises(ff.FieldfareError, match="4-bit"):
        m8 = c.matrix_int8(*oracle.quantize_int8(g.uniform(-1, 1, (16, 64)).astype(np.float32)))
        m8.rows(0)
    with pytest.raises(ff.FieldfareError, match="aligned"):
        table.rows(0, out=torch.empty((1, n + 8), dtype=c.act, device="cuda")[:, 1:n + 1])
    table.close()
    c.close()
