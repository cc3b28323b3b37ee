"""Pins the oracle's codecs, PRNG, quantiser and dequantiser against closed forms, independent
library implementations and the reference's own known-answer tests (CPU only)."""
import numpy as np
import pytest
import torch


def test_bf16_roundtrip_all_patterns(oracle):
    # every bf16 pattern widens and re-encodes to itself (NaN payloads included: no NaN special case,
    # Quantization.swift:9-15), except NaNs whose rounding add carries into the exponent: none do
    # because the low 16 bits are zero after widening.
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.bf16_to_float(bits)
    assert np.array_equal(oracle.bf16_bits(f), bits)
    L = oracle.lib()
    for b in (0x0000, 0x0001, 0x8001, 0x3F80, 0x7F7F, 0xFF80, 0x4300):
        assert L.ffo_bf16_bits(L.ffo_bf16_to_float(b)) == b


def test_bf16_rne_ties_and_torch(oracle):
    L = oracle.lib()
    # exact halfway cases: low 16 bits == 0x8000 round to even
    for hi in (0x3F80, 0x3F81, 0x4000, 0xC001, 0x0001):
        x = np.array([(hi << 16) | 0x8000], np.uint32).view(np.float32)[0]
        expect = hi + (hi & 1)
        assert L.ffo_bf16_bits(float(x)) == expect
        just_below = np.array([(hi << 16) | 0x7FFF], np.uint32).view(np.float32)[0]
        just_above = np.array([(hi << 16) | 0x8001], np.uint32).view(np.float32)[0]
        assert L.ffo_bf16_bits(float(just_below)) == hi
        assert L.ffo_bf16_bits(float(just_above)) == hi + 1
    # independent implementation: torch's float32 -> bfloat16 cast is RNE
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.normal(0, 1, 200000), rng.normal(0, 1e-30, 1000), rng.normal(0, 1e30, 1000)]).astype(np.float32)
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.bf16_bits(x), t)
    c = np.array([L.ffo_bf16_bits(float(v)) for v in x[:5000]], np.uint16)
    assert np.array_equal(c, t[:5000])


def test_fp16_codec_matches_numpy(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 7):
        v = L.ffo_fp16_to_float(b)
        if np.isnan(ref[b]):
            assert np.isnan(v)
        else:
            assert v == ref[b]
            assert L.ffo_fp16_bits(v) == b
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.normal(0, 1, 20000), rng.normal(0, 1e-6, 5000), rng.normal(0, 3e4, 5000),
                        [65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.99e-8, 0.0, -0.0]]).astype(np.float32)
    ref_bits = x.astype(np.float16).view(np.uint16)
    got = np.array([L.ffo_fp16_bits(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, ref_bits)


def test_splitmix64_published_vector(oracle):
    # SplitMix64 reference outputs for seed 1234567 (Vigna's splitmix64.c test vector)
    g = oracle.SplitMix64(1234567)
    assert [g.next() for _ in range(5)] == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                            4593380528125082431, 16408922859458223821]
    g = oracle.SplitMix64(0)
    assert g.next() == 0xE220A8397B1DCDAF
    # uniform: 24-bit mantissa in [lo, hi)
    g = oracle.SplitMix64(42)
    h = oracle.SplitMix64(42)
    u = g.uniform(-2.0, 3.0, 1000)
    manual = np.array([np.float32(-2.0) + np.float32(5.0) * (np.float32(h.next() >> 40) / np.float32(1 << 24)) for _ in range(1000)], np.float32)
    assert np.array_equal(u, manual)
    assert u.min() >= -2.0 and u.max() < 3.0


def test_seedtree_is_fnv1a_xor_root(oracle):
    # FNV-1a 64 of "a" is 0xAF63DC4C8601EC8C (published test value); empty label = offset basis
    L = oracle.lib()
    assert L.ffo_seedtree_key(0, b"a") == 0xAF63DC4C8601EC8C
    assert L.ffo_seedtree_key(0, b"") == 0xCBF29CE484222325
    assert L.ffo_seedtree_key(0x2D3, b"a") == 0xAF63DC4C8601EC8C ^ 0x2D3
    assert L.ffo_seedtree_key(0, b"foobar") == 0x85944171F73967E8


def test_nibble_order_literal_bytes(oracle):
    # Metal/Quant/dequant_int4.metal:7-12: byte k low nibble = element 2k, high nibble = element 2k+1.
    # A representable ramp (scale 0.5, bias -4) must quantise to q = 0..15 exactly, four times over.
    q = np.tile(np.arange(16), 4)
    row = (-4.0 + 0.5 * q).astype(np.float32)[None, :]
    packed, s, b = oracle.quantize_int4(row)
    assert packed.shape == (1, 32)
    assert list(packed[0][:8]) == [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]
    assert np.array_equal(packed[0], np.tile(packed[0][:8], 4))
    assert oracle.bf16_to_float(s)[0, 0] == 0.5 and oracle.bf16_to_float(b)[0, 0] == -4.0
    assert np.array_equal(oracle.dequantize_int4(packed, s, b), row)
    # as a little-endian uint32, nibble j = (w >> 4j) & 0xF (dequant_int4.metal:278)
    w = packed[0][:4].view("<u4")[0]
    assert [(int(w) >> (4 * j)) & 0xF for j in range(8)] == list(range(8))


def test_quantize_known_answer_ramp(oracle):
    # QuantizationAffineTests.swift:7-26
    row = np.concatenate([0.10 + np.arange(64, dtype=np.float32) * np.float32(0.01),
                          -0.50 - np.arange(64, dtype=np.float32) * np.float32(0.005)]).astype(np.float32)[None, :]
    packed, s, b = oracle.quantize_int4(row)
    assert packed.shape[1] == 64 and s.shape[1] == 2 and b.shape[1] == 2
    r = oracle.dequantize_int4(packed, s, b)
    assert np.abs(r - row).max() < 0.025
    # scale ~ range/15, bias = group min, both rounded to bf16
    sf, bf = oracle.bf16_to_float(s)[0], oracle.bf16_to_float(b)[0]
    assert abs(sf[0] - 0.63 / 15) < 0.63 / 15 * 2 ** -7 and abs(sf[1] - 0.315 / 15) < 0.315 / 15 * 2 ** -7
    assert abs(bf[0] - 0.10) <= 0.10 * 2 ** -8 and abs(bf[1] + 0.815) <= 0.815 * 2 ** -8
    # q is monotone along a monotone ramp and spans 0..15
    q0 = np.stack([packed[0, :32] & 15, packed[0, :32] >> 4], 1).ravel()
    assert q0[0] == 0 and q0[-1] == 15 and np.all(np.diff(q0.astype(int)) >= 0)


def test_quantize_constant_group_and_clamp(oracle):
    row = np.full((1, 64), 0.37, np.float32)
    packed, s, b = oracle.quantize_int4(row)
    assert oracle.bf16_to_float(s)[0, 0] == 1.0
    assert np.all(packed == 0)            # (w - bias) / 1 rounds to 0
    # int8 variant: 255 levels
    row8 = np.linspace(-1, 1, 64, dtype=np.float32)[None, :]
    p8, s8, b8 = oracle.quantize_int8(row8)
    # the bf16-rounded scale may exceed range/255, so the top code can fall a step or two short
    assert p8.min() == 0 and 252 <= p8.max() <= 255
    assert np.abs(oracle.dequantize_int8(p8, s8, b8) - row8).max() < 2 / 255


def test_dequant_closed_form_adversarial(oracle):
    # adversarial scales/biases of MPPPrefillInt4QMMTests.swift:26-37, incl. bf16 subnormals 0x0001/0x8001
    L = oracle.lib()
    scales = [L.ffo_bf16_bits(0.001), L.ffo_bf16_bits(-0.0015), 0x0001, 0x8001]
    biases = [L.ffo_bf16_bits(-0.01), L.ffo_bf16_bits(0.006), 0x0001, 0x8001]
    n = 64 * 16
    packed = ((np.arange(n // 2) * 37 + 0x29) & 0xFF).astype(np.uint8)[None, :]
    S = np.array([[scales[g % 4] for g in range(16)]], np.uint16)
    B = np.array([[biases[(g // 4) % 4] for g in range(16)]], np.uint16)
    got = oracle.dequantize_int4(packed, S, B)[0]
    got16 = oracle.dequantize_int4_bf16(packed, S, B)[0]
    # closed form in float64: q*s is exact (<= 12 significant bits), so fp32(q*s + b) == fp32 of the fp64 sum
    q = np.stack([packed[0] & 15, packed[0] >> 4], 1).ravel().astype(np.float64)
    s64 = np.repeat(oracle.bf16_to_float(S[0]).astype(np.float64), 64)
    b64 = np.repeat(oracle.bf16_to_float(B[0]).astype(np.float64), 64)
    exact = (q * s64 + b64)
    assert np.array_equal(got, exact.astype(np.float32))
    # and fma(q, s, b) (Metal, tensorops.metal:267) is the same fp32 value as q*s + b (Swift)
    fma = np.array([np.float32(np.float64(qq) * ss + bb) for qq, ss, bb in zip(q, s64, b64)], np.float32)
    assert np.array_equal(got, fma)
    # 16-bit tile value = RNE bf16 of that; torch cast as the independent rounding
    t = torch.from_numpy(got.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got16, t)
