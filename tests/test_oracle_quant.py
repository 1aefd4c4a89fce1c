"""Pins the CPU oracle's quantise / pack / cast functions.

The reference's tests hold no stored golden vectors for this path (only seeds
and error bounds, tests/test_quantize_ops.cpp:161-300), so the oracle is pinned
by: hand-derived known answers (tests/golden/quant_kat.json), the reference
tests' own bounds and zero-input exactness, numpy/torch casts for the 16-bit
formats, and exact rational arithmetic on tiny inputs.
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(__file__), "golden", "quant_kat.json")


@pytest.fixture(scope="module")
def kat():
    with open(GOLD) as f:
        return json.load(f)


# ----------------------------------------------------------------------------- 16-bit casts
def test_f16_all_patterns_roundtrip(orc):
    bits = np.arange(65536, dtype=np.uint16)
    vals = orc.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(vals.view(np.uint32), ref.view(np.uint32))
    finite = np.isfinite(ref)
    back = orc.f32_to_f16_bits(vals)
    assert np.array_equal(back[finite], bits[finite])


def test_f32_to_f16_ties_and_neighbours(orc):
    # every midpoint between adjacent non-negative fp16 values, and its fp32 neighbours
    bits = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = bits.view(np.float16).astype(np.float64)
    hi = (bits + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0                                    # the value after the largest finite half
    mid = ((lo + hi) / 2).astype(np.float32)            # exactly representable in fp32
    cases = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)),
                            np.nextafter(mid, np.float32(-np.inf)), -mid])
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16).view(np.uint16)
    got = orc.f32_to_f16_bits(cases)
    assert np.array_equal(got, want)


def test_f32_to_f16_random_bit_patterns(orc):
    rng = np.random.default_rng(5)
    u = rng.integers(0, 2**32, size=1 << 21, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f32_to_f16_bits(x), want)


def test_bf16_matches_torch(orc):
    rng = np.random.default_rng(6)
    u = rng.integers(0, 2**32, size=1 << 21, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[~np.isnan(x)]
    # exact ties: xxxx8000 patterns
    ties = ((u[:4096] & np.uint32(0xFFFF0000)) | np.uint32(0x8000)).view(np.float32)
    ties = ties[~np.isnan(ties)]
    x = np.concatenate([x, ties, np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38], np.float32)])
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = orc.f32_to_bf16_bits(x)
    assert np.array_equal(got, want)
    back = orc.bf16_bits_to_f32(got)
    assert np.array_equal(back.view(np.uint32), got.astype(np.uint32) << 16)
    assert np.isnan(orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(np.array([np.nan], np.float32))))[0]


# ----------------------------------------------------------------------------- known answers
def test_kat_int8_per_tensor(orc, kat):
    for case in kat["int8_per_tensor"]:
        q, s = orc.quantize_int8_per_tensor(np.array(case["x"], np.float32))
        assert s[0] == np.float32(case["scale"]), case["why"]
        assert q.tolist() == case["q"], case["why"]


def test_kat_int8_per_channel(orc, kat):
    for case in kat["int8_per_channel"]:
        x = np.array(case["x"], np.float32).reshape(case["rows"], case["cols"])
        q, s = orc.quantize_int8_per_channel(x)
        assert s.tolist() == case["scales"], case["why"]
        assert q.reshape(-1).tolist() == case["q"], case["why"]


def test_kat_int4(orc, kat):
    for case in kat["int4_group"]:
        packed, scales = orc.quantize_to_int4(np.array(case["x"], np.float32), case["group"])
        assert scales.tolist() == case["scales_f16"], case["why"]
        assert packed.tolist() == case["packed"], case["why"]
    for case in kat["int4_decode"]:
        out = orc.dequantize_int4(np.array(case["packed"], np.uint8),
                                  np.array(case["scales_f16"], np.uint16), case["n"], case["group"])
        assert out.tolist() == case["out"], case["why"]


# ----------------------------------------------------------------------------- reference test bounds
def test_reference_bounds_int8_per_tensor(orc):
    # tests/test_quantize_ops.cpp:161-190: n=1024, U(-2.5,2.5); |x - deq(q(x))| <= max|x|/127 + 1e-6
    x = np.random.default_rng(11).uniform(-2.5, 2.5, 1024).astype(np.float32)
    q, s = orc.quantize_int8_per_tensor(x)
    d = orc.dequantize_int8_per_tensor(q, s)
    assert np.abs(x - d).max() <= np.abs(x).max() / 127 + 1e-6
    # the tight form: half a step
    assert np.abs(x - d).max() <= s[0] / 2 * (1 + 1e-6)
    assert np.abs(q).max() == 127 and q[np.argmax(np.abs(x))] in (127, -127)


def test_reference_bounds_int8_per_channel(orc):
    # tests/test_quantize_ops.cpp:192-230: [32,64], column c ~ U(+-(0.1+0.05c))
    rng = np.random.default_rng(22)
    x = np.stack([rng.uniform(-(0.1 + 0.05 * c), 0.1 + 0.05 * c, 32) for c in range(64)], 1)
    x = x.astype(np.float32)
    q, s = orc.quantize_int8_per_channel(x)
    d = orc.dequantize_int8_per_channel(q, s)
    assert np.abs(x - d).max() <= np.abs(x).max() / 127 + 1e-6
    assert np.all(np.abs(x - d) <= s[None, :] / 2 * (1 + 1e-6))
    assert np.array_equal(s, np.abs(x).max(0) / np.float32(127))   # IEEE division, one rounding


def test_reference_zero_input_exact(orc):
    # tests/test_quantize_ops.cpp:232-267: dequant of quantised zeros is exactly 0, scale 1.0
    z = np.zeros((8, 16), np.float32)
    q, s = orc.quantize_int8_per_tensor(z)
    assert s[0] == 1.0 and not q.any()
    assert not orc.dequantize_int8_per_tensor(q, s).any()
    q, s = orc.quantize_int8_per_channel(z)
    assert np.all(s == 1.0) and not q.any()
    p, sc = orc.quantize_to_int4(z, 128)
    assert not p.any() and not sc.any()
    assert not orc.dequantize_int4(p, sc, z.size, 128).any()


def test_reference_bounds_int4(orc):
    # tests/test_quantize_ops.cpp:269-300: n=512, group 128, U(-1,1); bound max|x|/7 + 1e-3
    x = np.random.default_rng(33).uniform(-1, 1, 512).astype(np.float32)
    p, sc = orc.quantize_to_int4(x, 128)
    d = orc.dequantize_int4(p, sc, 512, 128)
    assert np.abs(x - d).max() <= np.abs(x).max() / 7 + 1e-3
    assert p.size == 256 and sc.size == 4


# ----------------------------------------------------------------------------- exact arithmetic on tiny inputs
def _rne_int(fr):
    """Round a Fraction to the nearest integer, ties to even."""
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return fl


def _f32(fr):
    """Round a Fraction to the nearest binary32 (the inputs here never hit a tie)."""
    return np.float32(fr.numerator / fr.denominator)


def test_int8_codes_by_rational_arithmetic(orc):
    rng = np.random.default_rng(7)
    x = rng.normal(0, 0.02, 300).astype(np.float32)
    q, s = orc.quantize_int8_per_tensor(x)
    mx = max(Fraction(float(abs(v))) for v in x)
    scale = _f32(mx / 127)
    assert s[0] == scale
    inv = _f32(1 / Fraction(float(scale)))
    for xi, qi in zip(x, q):
        prod = Fraction(float(np.float32(Fraction(float(xi)) * Fraction(float(inv)))))
        prod = max(min(prod, Fraction(127)), Fraction(-127))
        assert qi == _rne_int(prod)


def test_int4_codes_by_rational_arithmetic(orc):
    rng = np.random.default_rng(8)
    n, G = 5 * 32 + 7, 32                               # ragged: short last group, odd length
    x = rng.normal(0, 0.02, n).astype(np.float32)
    packed, sc = orc.quantize_to_int4(x, G)
    assert packed.size == (n + 1) // 2 and sc.size == 6
    for g in range(6):
        seg = x[g * G:(g + 1) * G]
        mx = max(Fraction(float(abs(v))) for v in seg)
        scale = _f32(mx / 7)
        assert sc[g] == np.float16(scale).view(np.uint16)          # stored scale: fp16 RNE
        inv = _f32(1 / Fraction(float(scale)))
        for j, xi in enumerate(seg):
            prod = Fraction(float(np.float32(Fraction(float(xi)) * Fraction(float(inv)))))
            prod = max(min(prod, Fraction(7)), Fraction(-7))
            code = _rne_int(prod) & 0xF
            f = g * G + j
            nib = (packed[f // 2] >> (4 * (f & 1))) & 0xF
            assert nib == code
    assert packed[-1] >> 4 == 0                          # odd tail: high nibble stays zero


def test_int4_dequant_is_exact_product(orc):
    # code (<=4 bits) times an fp16 scale (11-bit significand) is exact in fp32
    rng = np.random.default_rng(9)
    packed = rng.integers(0, 256, 64, dtype=np.uint8)
    sc = rng.integers(0, 0x7c00, 4, dtype=np.uint16)     # any finite non-negative fp16
    out = orc.dequantize_int4(packed, sc, 128, 32)
    for f in range(128):
        nib = (int(packed[f // 2]) >> (4 * (f & 1))) & 0xF
        qv = nib - 16 if nib >= 8 else nib
        want = Fraction(qv) * Fraction(float(sc[f // 32:f // 32 + 1].view(np.float16)[0]))
        assert Fraction(float(out[f])) == want


def test_plain_int8_cast(orc):
    # src/caif_cuda_kernels_quant.cu:144-162: clamp to +-127 THEN round to nearest even
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.4, 300.0, -300.0, -127.5], np.float32)
    assert orc.convert_fp32_to_int8(x).tolist() == [0, 2, 2, 0, -2, 126, 127, 127, -127, -127]
    q = np.arange(-128, 128).astype(np.int8)
    assert np.array_equal(orc.convert_int8_to_fp32(q), q.astype(np.float32))
