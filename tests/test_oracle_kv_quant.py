"""Pins the oracle's f16 conversion and KV quantizer (CPU only).

Evidence used, none of it the oracle's own formula retyped:
  * numpy.float16 as an independent IEEE round-to-nearest-even converter;
  * the reference's known answers and invariants (src/kv_quant.rs:302-332);
  * an exact-rational (fractions.Fraction) derivation of scale, bias and codes;
  * grid inputs whose codes are known by construction.
"""
from fractions import Fraction

import numpy as np
import pytest

import oracle


def test_f16_to_f32_all_halves():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_round_to_nearest_even():
    rng = np.random.default_rng(11)
    # Random bit patterns cover every exponent, incl. half subnormals and overflow.
    x = rng.integers(0, 2**32, size=1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    # Plus every exact tie between neighbouring halves.
    h = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, ties, -ties, np.float32([65504, 65519.99, 65520, 1e9, 0, -0.0, 5.96e-8, 2.9e-8, 3e-8])])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.f32_to_f16_bits(x)
    assert np.array_equal(got, want)


def test_codes_pack_lowest_bits_first():
    # src/kv_quant.rs:319-332
    x = np.zeros(64, np.float32)
    x[63] = 1.0
    x[1] = 1.0
    data, _, _ = oracle.quantize(x, 8)
    assert len(data) == 16 and data[0] == 255 << 8 and data[15] == 255 << 24
    assert not data[1:15].any()
    data, _, _ = oracle.quantize(x, 4)
    assert len(data) == 8 and data[0] == 15 << 4 and data[7] == 15 << 28
    assert not data[1:7].any()


def test_round_trip_is_within_half_a_step():
    # src/kv_quant.rs:302-317
    x = oracle.noise(4 * 64, 1)
    x[64:128] = 0.37
    for bits in (8, 4):
        _, scales, _ = oracle.quantize(x, bits)
        y = oracle.round_trip(x, bits)
        step = oracle.f16_bits_to_f32(scales)[np.arange(x.size) // 64]
        slack = step / 2 + np.abs(x) * 1e-3 + 1e-6
        assert (np.abs(x - y) <= slack).all()
        # The constant group has scale 0 and comes back as half(0.37) exactly.
        assert scales[1] == 0
        assert (y[64:128] == np.float32(np.float16(0.37))).all()


def _exact_quantize(group, bits):
    """Scale, bias and codes from exact rational arithmetic + explicit roundings."""
    levels = (1 << bits) - 1
    lo, hi = min(group), max(group)

    # (hi - lo) / levels in f32: subtract rounds once, divide rounds once.
    diff = np.float32(hi) - np.float32(lo)
    quotient = np.float32(float(Fraction(float(diff)) / levels))  # correctly rounded f32 divide
    s16 = np.float16(quotient)
    z16 = np.float16(np.float32(lo))
    s, z = Fraction(float(s16)), Fraction(float(z16))
    inv = np.float32(float(1 / s)) if s > 0 else np.float32(0)
    codes = []
    for v in group:
        d = np.float32(float(Fraction(float(np.float32(v))) - z))
        t = np.float32(float(Fraction(float(d)) * Fraction(float(inv))))
        r = Fraction(float(t))
        fl = r.numerator // r.denominator
        frac = r - fl
        q = fl + (1 if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and fl % 2) else 0)
        codes.append(min(max(q, 0), levels))
    return s16.view(np.uint16), z16.view(np.uint16), codes


@pytest.mark.parametrize("bits", [8, 4])
def test_matches_exact_rational_derivation(bits):
    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.standard_normal(64 * 6).astype(np.float32),
        (rng.standard_normal(64) * 200).astype(np.float32),
        (rng.standard_normal(64) * 1e-4).astype(np.float32),
        np.full(64, -1.5, np.float32),
    ])
    data, scales, biases = oracle.quantize(x, bits)
    per_word = 32 // bits
    for g in range(x.size // 64):
        s, z, codes = _exact_quantize([float(v) for v in x[g * 64:(g + 1) * 64]], bits)
        assert scales[g] == s and biases[g] == z
        words = data[g * 2 * bits:(g + 1) * 2 * bits]
        got = [(int(words[i // per_word]) >> ((i % per_word) * bits)) & ((1 << bits) - 1) for i in range(64)]
        assert got == codes


@pytest.mark.parametrize("bits", [8, 4])
def test_grid_values_get_their_own_codes(bits):
    # Values z + k * s with a power-of-two s are exact everywhere: code i must be k_i.
    levels = (1 << bits) - 1
    rng = np.random.default_rng(3)
    k = rng.integers(0, levels + 1, size=64)
    k[0], k[1] = 0, levels
    s, z = 2.0 ** -5, -3.0
    x = (z + k * s).astype(np.float32)
    data, scales, biases = oracle.quantize(x, bits)
    assert np.float16(s).view(np.uint16) == scales[0] and np.float16(z).view(np.uint16) == biases[0]
    per_word = 32 // bits
    got = [(int(data[i // per_word]) >> ((i % per_word) * bits)) & levels for i in range(64)]
    assert got == list(k)
    assert np.array_equal(oracle.dequantize(data, scales, biases, bits), x)


def test_dequantize_is_scale_times_code_plus_bias():
    rng = np.random.default_rng(9)
    for bits in (8, 4):
        groups = 5
        data = rng.integers(0, 2**32, size=groups * 2 * bits, dtype=np.uint64).astype(np.uint32)
        scales = rng.uniform(0.001, 0.1, groups).astype(np.float16)
        biases = rng.uniform(-4, 0, groups).astype(np.float16)
        got = oracle.dequantize(data, scales.view(np.uint16), biases.view(np.uint16), bits)
        per_word = 32 // bits
        codes = np.array([[(int(data[g * 2 * bits + i // per_word]) >> ((i % per_word) * bits)) & ((1 << bits) - 1)
                           for i in range(64)] for g in range(groups)], np.float32)
        want = scales.astype(np.float32)[:, None] * codes + biases.astype(np.float32)[:, None]
        assert np.array_equal(got.reshape(groups, 64), want)


def test_nan_and_infinite_inputs_follow_rust_semantics():
    # f32::min/max skip NaN; clamp keeps NaN and `as u32` makes it 0 (src/kv_quant.rs:61-76).
    x = np.linspace(-1, 1, 64).astype(np.float32)
    x[7] = np.nan
    data, scales, biases = oracle.quantize(x, 8)
    assert biases[0] == np.float16(-1).view(np.uint16)
    assert (int(data[1]) >> 24) & 255 == 0  # value 7 is NaN -> code 0
    assert int(data[15]) >> 24 == 255


def test_round_trip_kinds():
    x = oracle.noise(512, 2)
    assert np.array_equal(oracle.round_trip(x, 16), x.astype(np.float16).astype(np.float32))
    y8 = oracle.round_trip(x, 8)
    assert np.array_equal(oracle.round_trip_as_half(x, 8), y8.astype(np.float16).astype(np.float32))
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros(63, np.float32), 8)
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros(64, np.float32), 16)
