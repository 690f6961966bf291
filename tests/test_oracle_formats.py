"""Pins the number-format half of the CPU oracle: the reference's own known-answer vectors
(tests/golden/ptx_cvt_kat.json, from ptx/src/test/spirv_run/mod.rs:321-329), the OCP definitions
written out independently as closed forms, and a brute-force nearest-value search for the encoders."""
import json
import os

import numpy as np
import pytest

import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden")
KAT = json.load(open(os.path.join(GOLD, "ptx_cvt_kat.json")))
L = oracle.lib()


def test_kat_e4m3_encode():
    a, b = KAT["e4m3x2_from_f32"]["in"]
    assert (L.oracle_encode_e4m3(a) << 8) | L.oracle_encode_e4m3(b) == KAT["e4m3x2_from_f32"]["out"]


def test_kat_e5m2_encode():
    a, b = KAT["e5m2x2_from_f32"]["in"]
    assert (L.oracle_encode_e5m2(a) << 8) | L.oracle_encode_e5m2(b) == KAT["e5m2x2_from_f32"]["out"]


def test_kat_bf16_encode():
    a, b = KAT["bf16x2_from_f32"]["in"]
    assert (L.oracle_encode_bf16(a) << 16) | L.oracle_encode_bf16(b) == KAT["bf16x2_from_f32"]["out"]


@pytest.mark.parametrize("name", ["e4m3", "e5m2"])
def test_kat_fp8_decode_to_f16(name):
    k = KAT["f16x2_from_%sx2" % name]
    dec = getattr(L, "oracle_decode_" + name)
    hi, lo = dec(k["in"] >> 8), dec(k["in"] & 0xFF)
    # both values are exactly representable in f16: the f16 bit patterns must match
    got = (int(np.float16(hi).view(np.uint16)) << 16) | int(np.float16(lo).view(np.uint16))
    assert got == k["out"]


def _closed_form(code, ebits, mbits, bias, ieee_like):
    s = -1.0 if code >> (ebits + mbits) else 1.0
    e = (code >> mbits) & ((1 << ebits) - 1)
    m = code & ((1 << mbits) - 1)
    if ieee_like and e == (1 << ebits) - 1:
        return s * np.inf if m == 0 else np.nan
    if not ieee_like and e == (1 << ebits) - 1 and m == (1 << mbits) - 1:
        return np.nan
    if e == 0:
        return s * m * 2.0 ** (1 - bias - mbits)
    return s * (1 + m / 2.0 ** mbits) * 2.0 ** (e - bias)


def test_decode_tables_match_ocp_definition():
    for name, (eb, mb, bias, ieee) in {"e4m3": (4, 3, 7, False), "e5m2": (5, 2, 15, True)}.items():
        tab = oracle.decode_table(name)
        for c in range(256):
            want = _closed_form(c, eb, mb, bias, ieee)
            if np.isnan(want):
                assert np.isnan(tab[c]), (name, c)
            else:
                assert tab[c] == np.float32(want), (name, c, tab[c], want)
    # E4M3 extremes: max finite 448, min subnormal 2^-9; E5M2: 57344, 2^-16
    assert oracle.decode_table("e4m3")[0x7E] == 448.0 and oracle.decode_table("e4m3")[0x01] == 2.0 ** -9
    assert oracle.decode_table("e5m2")[0x7B] == 57344.0 and oracle.decode_table("e5m2")[0x01] == 2.0 ** -16
    e2m1 = oracle.decode_table("e2m1")
    assert list(e2m1[:8]) == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert list(e2m1[8:]) == [-0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    assert np.signbit(e2m1[8])
    ue = oracle.decode_table("ue8m0")
    assert np.isnan(ue[255]) and ue[127] == 1.0 and ue[0] == np.float32(2.0 ** -127) and ue[254] == np.float32(2.0 ** 127)
    assert all(ue[i + 1] == 2 * ue[i] for i in range(254))


def _nearest_even(values, x, maxv):
    """brute force: index of the representable value nearest to |x| (ties -> even code), saturating"""
    ax = min(abs(float(x)), maxv)
    d = np.abs(values.astype(np.float64) - ax)
    best = np.flatnonzero(d == d.min())
    if best.size > 1:
        best = [b for b in best if b % 2 == 0]
    return int(best[0])


@pytest.mark.parametrize("name,maxcode", [("e4m3", 0x7E), ("e5m2", 0x7B), ("e2m1", 0x7)])
def test_encoders_are_nearest_even_saturating(name, maxcode):
    tab = oracle.decode_table(name)
    pos = tab[: maxcode + 1]  # non-negative finite codes, increasing
    enc = getattr(L, "oracle_encode_" + name)
    sign = 0x8 if name == "e2m1" else 0x80
    rng = np.random.default_rng(7)
    maxv = float(pos[-1])
    xs = np.concatenate([
        rng.standard_normal(3000) * maxv / 3, rng.standard_normal(3000), rng.standard_normal(2000) * float(pos[1]) * 4,
        (pos[:-1].astype(np.float64) + pos[1:]) / 2,            # exact ties
        pos, [maxv * 1.5, 1e30, np.inf, 0.0],
    ]).astype(np.float32)
    for x in xs:
        for v in (x, -x):
            code = enc(float(v))
            want = _nearest_even(pos, v, maxv)
            if np.signbit(v):
                want |= sign
            assert code == want, (name, float(v), hex(code), hex(want))


def test_encoders_roundtrip_every_code():
    for name, n in (("e4m3", 256), ("e5m2", 256), ("e2m1", 16)):
        tab = oracle.decode_table(name)
        enc = getattr(L, "oracle_encode_" + name)
        for c in range(n):
            if np.isfinite(tab[c]):
                assert enc(float(tab[c])) == c, (name, c)


def test_bf16_rne_brute_force():
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.standard_normal(4000) * 100, rng.standard_normal(4000) * 1e-3]).astype(np.float32)
    # ties: mantissa low 16 bits exactly 0x8000
    ties = (rng.integers(0, 0x7F7F, 2000).astype(np.uint32) << 16 | 0x8000).view(np.float32)
    xs = np.concatenate([xs, ties])
    got = oracle.encode_bf16(xs)
    bits = xs.view(np.uint32).astype(np.uint64)
    lo, up = (bits >> 16), (bits >> 16) + 1
    rem = bits & 0xFFFF
    want = np.where(rem > 0x8000, up, np.where(rem < 0x8000, lo, np.where(lo & 1, up, lo))).astype(np.uint16)
    assert np.array_equal(got, want)


def test_f16_encode_matches_numpy():
    rng = np.random.default_rng(5)
    xs = np.concatenate([rng.standard_normal(5000) * 50, rng.standard_normal(5000) * 1e-4, [65504.0, 65519.9, 1e6, 6e-8, 0.0]]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.encode_f16(xs), want)


def test_mxfp4_quantizer_block_semantics():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((5, 96)).astype(np.float32)
    x[2, 32:64] = 0.0
    q, s = oracle.quantize_mxfp4(x)
    e2m1 = oracle.decode_table("e2m1")
    for r in range(5):
        for kb in range(3):
            blk = x[r, kb * 32:(kb + 1) * 32]
            mx = np.abs(blk).max()
            e = int(np.floor(np.log2(mx))) - 2 if mx > 0 else -127
            assert s[r, kb] == e + 127
            codes = q[r, kb * 16:(kb + 1) * 16]
            vals = np.empty(32, np.float32)
            vals[0::2] = e2m1[codes & 15]       # low nibble = even (lower) K index
            vals[1::2] = e2m1[codes >> 4]
            deq = vals * np.float32(2.0) ** e
            # the block maximum lands in [4, 8) before rounding: error bounded by half a step of 2 (or saturation 6)
            assert np.all(np.abs(deq - blk) <= np.float32(2.0) ** e * 2.0 + 1e-12)
            assert np.abs(vals).max() <= 6.0


def test_gelu_is_tanh_form():
    xs = np.linspace(-6, 6, 241, dtype=np.float32)
    want = 0.5 * xs.astype(np.float64) * (1 + np.tanh(np.sqrt(2 / np.pi) * (xs.astype(np.float64) + 0.044715 * xs.astype(np.float64) ** 3)))
    got = np.array([L.oracle_gelu(float(x)) for x in xs])
    assert np.max(np.abs(got - want)) < 1e-6
    assert abs(L.oracle_gelu(1.0) - 0.8411919906082768) < 1e-6   # textbook value of tanh-GELU(1)
