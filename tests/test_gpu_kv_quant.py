"""kv_quantize / kv_dequantize / to_half on the GPU against the oracle: bit-exact.

Restates tests/kv_quant.rs (37 tokens at position 5, one token at position 41 through a
plan, dequantize of 9 tokens) with the bar raised from "<= 0.1 % of codes one step off"
to "no code differs", plus ragged and extreme inputs and the full-size append.
"""
import numpy as np
import pytest
import torch

from gpu_common import VALUES, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
KINDS = [saetta.KvBits.Eight, saetta.KvBits.Four]


def compare(rows, x, from_token, kind):
    bits = kind.value
    groups = x.size // 64
    first = from_token * rows.per_token
    words = kind.words_per_group()
    data = host(rows.data).view(np.uint32)[first * words:(first + groups) * words]
    scales = host(rows.scales).view(np.uint16)[first:first + groups]
    biases = host(rows.biases).view(np.uint16)[first:first + groups]
    wd, ws, wz = oracle.quantize(x, bits)
    assert np.array_equal(scales, ws), f"{kind} scales"
    assert np.array_equal(biases, wz), f"{kind} biases"
    assert np.array_equal(data, wd), f"{kind}: {(data != wd).sum()} code words differ"


@pytest.mark.parametrize("kind", KINDS)
def test_prefill_rows_match_cpu(kind):
    tokens = 37
    cache = saetta.QuantRows(kind, VALUES, 64)
    x = oracle.quant_rows(tokens)
    cache.encode(dev(x), 5, tokens)
    compare(cache, x, 5, kind)
    # Nothing outside rows 5..41 was touched.
    assert not host(cache.scales)[:5 * 8].any() and not host(cache.scales)[42 * 8:].any()


@pytest.mark.parametrize("kind", KINDS)
def test_decode_row_matches_cpu(kind):
    cache = saetta.QuantRows(kind, VALUES, 64)
    x = oracle.quant_rows(1)
    plan = saetta.Plan()
    cache.record(plan, dev(x))
    built = plan.build()
    plan.set_params(saetta.TokenParams(0, 41))
    built.run()
    compare(cache, x, 41, kind)
    # The same recorded launch serves another position.
    plan.set_params(saetta.TokenParams(0, 7))
    built.run()
    compare(cache, x, 7, kind)


@pytest.mark.parametrize("kind", KINDS)
def test_dequantize_matches_cpu(kind):
    tokens = 9
    cache = saetta.QuantRows(kind, VALUES, 64)
    x = oracle.quant_rows(tokens)
    out = torch.zeros(tokens * VALUES, dtype=torch.float16, device="cuda")
    cache.encode(dev(x), 0, tokens)
    cache.encode_dequantize(out, tokens)
    groups = tokens * cache.per_token
    want = oracle.dequantize(host(cache.data).view(np.uint32)[:groups * kind.words_per_group()],
                             host(cache.scales).view(np.uint16)[:groups],
                             host(cache.biases).view(np.uint16)[:groups], kind.value)
    assert np.array_equal(host(out).view(np.uint16), oracle.f32_to_f16_bits(want))


@pytest.mark.parametrize("kind", KINDS)
def test_extreme_groups_are_bit_exact(kind):
    rng = np.random.default_rng(17)
    g = []
    g.append(rng.standard_normal(64) * 1e-6)          # scale in the half subnormals
    g.append(rng.standard_normal(64) * 3e4)           # scale and bias near the half maximum
    g.append(rng.standard_normal(64) * 1e6)           # bias overflows to infinity
    g.append(np.full(64, 0.37))                       # constant: scale 0
    g.append(np.zeros(64))
    g.append(np.where(np.arange(64) % 2, 1e-30, -1e-30))
    nan = rng.standard_normal(64); nan[[3, 40]] = np.nan
    g.append(nan)
    g.append(np.full(64, np.nan))
    inf = rng.standard_normal(64); inf[5] = np.inf
    g.append(inf)
    ties = -1.0 + (np.arange(64) + 0.5) * (2.0 / 255)  # values halfway between codes
    g.append(ties)
    while len(g) % 8:
        g.append(rng.standard_normal(64) * 8)
    x = np.concatenate(g).astype(np.float32)
    tokens = x.size // VALUES
    cache = saetta.QuantRows(kind, VALUES, tokens + 1)
    cache.encode(dev(x), 1, tokens)
    compare(cache, x, 1, kind)


@pytest.mark.parametrize("kind", KINDS)
def test_outlier_channels_and_a_full_chunk(kind):
    # configs[3]/[2]: N(0,1) with 1 % of channels x8; a 4096-token append in one launch.
    rng = np.random.default_rng(23)
    tokens = 4096
    x = rng.standard_normal((tokens, VALUES)).astype(np.float32)
    x[:, rng.choice(VALUES, 5, replace=False)] *= 8
    cache = saetta.QuantRows(kind, VALUES, tokens)
    cache.encode(dev(x.reshape(-1)), 0, tokens)
    compare(cache, x.reshape(-1), 0, kind)
    # Round trip: |x - dequant| <= step / 2 (+ the bias rounding), src/kv_quant.rs:302-317.
    out = torch.empty(tokens * VALUES, dtype=torch.float16, device="cuda")
    cache.encode_dequantize(out, tokens)
    step = host(cache.scales).astype(np.float32).repeat(64)
    xf = x.reshape(-1)
    assert (np.abs(host(out).astype(np.float32) - xf) <= step / 2 + np.abs(xf) * 2e-3 + 1e-6).all()


def test_empty_and_rejected_arguments():
    cache = saetta.QuantRows(saetta.KvBits.Eight, VALUES, 4)
    x = dev(np.zeros(VALUES, np.float32))
    cache.encode(x, 0, 0)  # nothing to do, no launch
    with pytest.raises(ValueError):
        cache.encode(x, 4, 1)  # past the capacity
    with pytest.raises(ValueError):
        saetta.QuantRows(saetta.KvBits.Half, VALUES, 4)
    with pytest.raises(saetta.ffi.SaettaError):
        saetta.ffi.check(saetta.ffi.lib().saetta_kv_quantize(None, 5, x.data_ptr(), cache.c(),
                                                             saetta.ffi.KvQuantParamsC(8, 8), None, 0), "bits 5")


def test_to_half_rounds_to_nearest_even():
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.standard_normal(4099) * 100, [65519.9, 65520.0, 1e-8, -0.0, 2.0**-24 * 1.5]]).astype(np.float32)
    out = torch.zeros(x.size, dtype=torch.float16, device="cuda")
    saetta.to_half(dev(x), out)
    assert np.array_equal(host(out).view(np.uint16), oracle.f32_to_f16_bits(x))


@pytest.mark.parametrize("kind", KINDS)
def test_module_functions_match_cpu(kind):
    # quantize / dequantize / round_trip / round_trip_as_half of src/kv_quant.rs:54-125 as device functions.
    bits = kind.value
    x = oracle.quant_rows(11)
    data, scales, biases = saetta.quantize(dev(x), kind)
    wd, ws, wz = oracle.quantize(x, bits)
    assert np.array_equal(host(data).view(np.uint32), wd)
    assert np.array_equal(host(scales).view(np.uint16), ws) and np.array_equal(host(biases).view(np.uint16), wz)
    back = host(saetta.dequantize(data, scales, biases, kind))
    assert np.array_equal(back.view(np.uint32), oracle.dequantize(wd, ws, wz, bits).view(np.uint32))
    assert np.array_equal(host(saetta.round_trip(dev(x), kind)).view(np.uint32),
                          oracle.round_trip(x, bits).reshape(-1).view(np.uint32))
    as_half = host(saetta.round_trip_as_half(dev(x), kind)).astype(np.float32)
    assert np.array_equal(as_half, oracle.round_trip_as_half(x, bits).reshape(-1))
    # the half step bound of src/kv_quant.rs:302-317, on the device result
    step = host(scales).astype(np.float32).repeat(64)
    assert (np.abs(back - x.reshape(-1)) <= 0.5 * step + 2e-3 * np.abs(x.reshape(-1)).max()).all()
    assert saetta.test_slack(kind) == {8: 4.0, 4: 16.0}[bits] and saetta.test_slack(saetta.KvBits.Half) == 1.0
    half = host(saetta.round_trip(dev(x), saetta.KvBits.Half))
    assert np.array_equal(half, x.reshape(-1).astype(np.float16).astype(np.float32))
