"""Chunked causal prefill attention on the GPU against the oracle.

Restates tests/attention_prefill.rs (spread data; (pos, tokens) = (0,1), (0,7), (5,8), (70,100),
(1000,64), (0,300), (4093,37); finite and max abs diff < 2e-3) with the oracle's token-by-token
f32 CPU attention as the other side (src/prefill.rs:2489-2495 defines the chunk that way), over a
half cache and over 8/4-bit caches read in place; bar of this build: rel-RMS <= 1e-3.
"""
import math

import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
KINDS = [saetta.KvBits.Half, saetta.KvBits.Eight, saetta.KvBits.Four]
SHAPES = [(0, 1), (0, 7), (5, 8), (70, 100), (1000, 64), (0, 300), (4093, 37)]
REL_RMS = 1e-3
MAX_ABS = 2e-3  # tests/attention_prefill.rs:56-59


def make_cache(kind, k, v, capacity, chunk_from=None):
    """Cache holding k, v [n, 512].  Rows from chunk_from on are appended on the device
    (to_half / kv_quantize), the others come from the host; rows past n hold NaN patterns."""
    n = k.shape[0]
    first = n if chunk_from is None else chunk_from
    if kind is saetta.KvBits.Half:
        kc = torch.full((capacity, VALUES), float("nan"), dtype=torch.float16, device="cuda")
        vc = torch.full((capacity, VALUES), float("nan"), dtype=torch.float16, device="cuda")
        kc[:first], vc[:first] = dev(k[:first].astype(np.float16)), dev(v[:first].astype(np.float16))
        if first < n:
            saetta.to_half(dev(k[first:].reshape(-1)), kc[first:n].view(-1))
            saetta.to_half(dev(v[first:].reshape(-1)), vc[first:n].view(-1))
        kf = k.astype(np.float16).astype(np.float32)
        vf = v.astype(np.float16).astype(np.float32)
        return kc, vc, kf, vf
    bits = kind.value
    kc, vc = saetta.QuantRows(kind, VALUES, capacity), saetta.QuantRows(kind, VALUES, capacity)
    for c, x in ((kc, k), (vc, v)):
        c.scales[:], c.biases[:], c.data[:] = float("nan"), float("inf"), -1
        if first:
            data, scales, biases = oracle.quantize(x[:first], bits)
            c.data[:data.size] = dev(data.view(np.int32))
            c.scales[:scales.size] = dev(scales.view(np.float16))
            c.biases[:biases.size] = dev(biases.view(np.float16))
        if first < n:
            c.encode(dev(x[first:].reshape(-1)), first, n - first)  # quantize-on-append
    return kc, vc, oracle.round_trip_as_half(k, bits), oracle.round_trip_as_half(v, bits)


def run(kind, q16, kc, vc, qg, pos, tokens):
    out = torch.full((tokens, H, D), float("nan"), device="cuda")
    p = saetta.FlashParams(H, KV, pos, tokens, 1.0 / math.sqrt(D))
    if kind is saetta.KvBits.Half:
        saetta.attention_prefill.encode(saetta.attention_prefill.DEFAULT, dev(q16), kc, vc, dev(qg), out, p)
    else:
        saetta.attention_prefill.encode_quant(dev(q16), kc, vc, dev(qg), out, p)
    return host(out)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("pos,tokens", SHAPES)
def test_matches_cpu_on_spread_data(kind, pos, tokens):
    n = pos + tokens
    capacity = -(-n // 64) * 64 + 64
    q16 = oracle.spread(tokens * H * D, 1).reshape(tokens, H, D)
    k = oracle.spread(n * VALUES, 2).astype(np.float32).reshape(n, VALUES)
    v = oracle.spread(n * VALUES, 3).astype(np.float32).reshape(n, VALUES)
    qg = ((np.arange(tokens * H * 2 * D) % 7) - 3).astype(np.float32).reshape(tokens, H, 2 * D)
    kc, vc, kf, vf = make_cache(kind, k, v, capacity, chunk_from=pos)
    got = run(kind, q16, kc, vc, qg, pos, tokens)
    want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < MAX_ABS, f"{kind} pos {pos} tokens {tokens}"
    assert oracle.rel_rms(got, want) < REL_RMS


@pytest.mark.parametrize("kind", KINDS)
def test_gaussian_chunk_with_cached_prefix(kind):
    # configs[2] in shape, scaled to what the CPU finishes in seconds: bf16-exact N(0,1) q, a cached
    # prefix quantized on the host, the chunk's K/V quantized on the device, gate N(0,1).
    rng = np.random.default_rng(12)
    pos, tokens = 300, 200
    n = pos + tokens
    q = rng.standard_normal((tokens, H, D)).astype(np.float32)
    q16 = torch.from_numpy(q).to(torch.bfloat16).to(torch.float16).numpy()
    k = rng.standard_normal((n, VALUES)).astype(np.float32)
    v = rng.standard_normal((n, VALUES)).astype(np.float32)
    qg = rng.standard_normal((tokens, H, 2 * D)).astype(np.float32)
    kc, vc, kf, vf = make_cache(kind, k, v, n, chunk_from=pos)
    got = run(kind, q16, kc, vc, qg, pos, tokens)
    want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
    assert oracle.rel_rms(got, want) < REL_RMS
    assert np.abs(got - want).max() < MAX_ABS


def test_causality_at_full_size():
    # The 4096 + 4096 shape: a token's output must not change when later keys change, and the
    # first token of the chunk must equal single-token decode attention over pos + 1 keys.
    rng = np.random.default_rng(3)
    pos = tokens = 4096
    n = pos + tokens
    kind = saetta.KvBits.Eight
    gen = torch.Generator(device="cuda").manual_seed(5)
    kx = torch.randn(n, VALUES, generator=gen, device="cuda")
    vx = torch.randn(n, VALUES, generator=gen, device="cuda")
    q16 = torch.randn(tokens, H, D, generator=gen, device="cuda").to(torch.float16)
    qg = torch.randn(tokens, H, 2 * D, generator=gen, device="cuda")
    kc, vc = saetta.QuantRows(kind, VALUES, n), saetta.QuantRows(kind, VALUES, n)
    kc.encode(kx.view(-1), 0, n), vc.encode(vx.view(-1), 0, n)
    p = saetta.FlashParams(H, KV, pos, tokens, 1.0 / 16)
    out = torch.empty(tokens, H, D, device="cuda")
    saetta.attention_prefill.encode_quant(q16, kc, vc, qg, out, p)
    a = host(out).copy()
    assert np.isfinite(a).all()
    # overwrite the last 1000 tokens' keys and values: rows before them must stay bit-equal
    kc.encode(vx[-1000:].contiguous().view(-1), n - 1000, 1000)
    vc.encode(kx[-1000:].contiguous().view(-1), n - 1000, 1000)
    saetta.attention_prefill.encode_quant(q16, kc, vc, qg, out, p)
    b = host(out)
    assert np.array_equal(a[:tokens - 1000], b[:tokens - 1000])
    assert not np.array_equal(a[tokens - 1000:], b[tokens - 1000:])
    # token 0 of the chunk against decode attention (itself checked against the oracle)
    kc.encode(kx[-1000:].contiguous().view(-1), n - 1000, 1000)
    vc.encode(vx[-1000:].contiguous().view(-1), n - 1000, 1000)
    att = saetta.DecodeAttention(H, KV, D, n)
    one = torch.empty(H, D, device="cuda")
    plan = saetta.Plan()
    att.record_quant(plan, q16[0].float().contiguous(), kc, vc, qg[0].contiguous(), one)
    plan.set_params(saetta.TokenParams(0, pos))
    plan.build().run()
    assert oracle.rel_rms(a[0], host(one)) < REL_RMS
    # a sample of rows against the oracle
    groups = n * 8
    kf = oracle.dequantize(host(kc.data).view(np.uint32), host(kc.scales).view(np.uint16), host(kc.biases).view(np.uint16), 8)
    vf = oracle.dequantize(host(vc.data).view(np.uint32), host(vc.scales).view(np.uint16), host(vc.biases).view(np.uint16), 8)
    kf = kf.astype(np.float16).astype(np.float32)
    vf = vf.astype(np.float16).astype(np.float32)
    qh, qgh = host(q16).astype(np.float32), host(qg)
    # Workgroups take 16-token tiles heaviest first, the second half of the tiles in a second
    # round: rows from both rounds, tile edges included; every row covers both kv heads.
    for i in (0, 1, 15, 16, 777, 1234, 2047, 2048, 2500, 3333, 4080, 4095):
        want = oracle.attend(qh[i], kf, vf, pos + i + 1, q_and_gate=qgh[i], threads=8)
        assert oracle.rel_rms(a[i], want) < REL_RMS


def test_shape_and_argument_checks():
    q = torch.zeros(1, H, D, dtype=torch.float16, device="cuda")
    kc = torch.zeros(64, VALUES, dtype=torch.float16, device="cuda")
    qg = torch.zeros(1, H, 2 * D, device="cuda")
    out = torch.zeros(1, H, D, device="cuda")
    with pytest.raises(ValueError):
        saetta.attention_prefill.encode("attention_fa16", q, kc, kc, qg, out, saetta.FlashParams(H, KV, 0, 1, 0.0625))
    with pytest.raises(ValueError):
        saetta.attention_prefill.encode("attention_fa8", q, kc, kc, qg, out, saetta.FlashParams(H, 4, 0, 1, 0.0625))
    # zero tokens: nothing to do
    saetta.attention_prefill.encode("attention_fa8", q, kc, kc, qg, out, saetta.FlashParams(H, KV, 0, 0, 0.0625))


def test_spread_rows2_and_bench_mirror_the_reference():
    # spread (src/attention_prefill.rs:102-108) against the oracle's restatement
    got = host(saetta.attention_prefill.spread(5000, 3)).astype(np.float32)
    assert np.array_equal(got, oracle.spread(5000, 3).astype(np.float32))
    # encode_rows2 is the same computation as encode
    pos, tokens = 40, 24
    n = pos + tokens
    q16 = oracle.spread(tokens * H * D, 1).reshape(tokens, H, D)
    k = torch.from_numpy(oracle.spread(n * VALUES, 2)).cuda()
    v = torch.from_numpy(oracle.spread(n * VALUES, 3)).cuda()
    qg = dev(((np.arange(tokens * H * 2 * D) % 7) - 3).astype(np.float32))
    q = torch.from_numpy(q16).cuda()
    a, b = torch.empty(tokens, H, D, device="cuda"), torch.empty(tokens, H, D, device="cuda")
    p = saetta.FlashParams(H, KV, pos, tokens, 1 / 16)
    saetta.attention_prefill.encode("attention_fa4", q, k, v, qg, a, p)
    saetta.attention_prefill.encode_rows2(q, k, v, qg, b, p)
    assert torch.equal(a, b)
    # bench of both modules on toy sizes: shapes and sanity of what they report
    rows = saetta.attention_prefill.bench([100], 64, 2)
    assert rows[0]["context"] == 128 and rows[0]["last_TFLOP/s"] > 0 and rows[0]["mid_TFLOP/s"] > 0
    for bits in (saetta.KvBits.Half, saetta.KvBits.Eight):
        rows = saetta.bench([256, 1000], 2, 3, bits)
        assert [r["tokens"] for r in rows] == [256, 1000] and all(r["GB/s"] > 0 and r["reduce_ms"] > 0 for r in rows)


@pytest.mark.parametrize("pos,tokens", [(4096, 4096), (0, 1000), (37, 3001), (100, 9000)])
def test_equal_keys_give_running_means_at_full_size(pos, tokens):
    # A closed form for every one of the 4096 x 16 rows of the headline shape: with the same key in every cache
    # row all scores of a token are equal, so token i's output is the mean of the first pos + i + 1 value rows
    # (as the half values the cache is read through) times sigmoid(gate), whatever q is.  A key block skipped,
    # taken twice or masked at the wrong place, or a wrong merge of the two waves of a row group, moves it.
    # The other shapes are the other ways the tiles reach the workgroups (one workgroup per CU takes tiles until
    # none are left, the ones past its first by asking a counter): 126 tiles, fewer than workgroups; 376, between
    # one and two each; 1126, more than four each, the chunk and its position ragged against tiles and key blocks.
    n = pos + tokens
    kind = saetta.KvBits.Eight
    gen = torch.Generator(device="cuda").manual_seed(17)
    krow = torch.randn(VALUES, generator=gen, device="cuda") * 2.0
    kx = krow.repeat(n, 1).contiguous()
    vx = torch.randn(n, VALUES, generator=gen, device="cuda")
    vx[:, 7] += 2.0
    q16 = torch.randn(tokens, H, D, generator=gen, device="cuda").to(torch.float16)
    qg = torch.randn(tokens, H, 2 * D, generator=gen, device="cuda")
    kc, vc = saetta.QuantRows(kind, VALUES, n), saetta.QuantRows(kind, VALUES, n)
    kc.encode(kx.view(-1), 0, n), vc.encode(vx.view(-1), 0, n)
    p = saetta.FlashParams(H, KV, pos, tokens, 1.0 / 16)
    out = torch.full((tokens, H, D), float("nan"), device="cuda")
    saetta.attention_prefill.encode_quant(q16, kc, vc, qg, out, p)
    got = host(out)
    vf = oracle.dequantize(host(vc.data).view(np.uint32), host(vc.scales).view(np.uint16), host(vc.biases).view(np.uint16), 8)
    vf = vf.reshape(n, VALUES).astype(np.float16).astype(np.float64)
    sums = np.cumsum(vf[pos:], axis=0) + vf[:pos].sum(axis=0)          # [tokens, 512]
    assert np.isfinite(got).all()
    means = (sums / (pos + 1 + np.arange(tokens))[:, None]).reshape(tokens, KV, D)
    gate = 1.0 / (1.0 + np.exp(-host(qg).reshape(tokens, H, 2 * D)[:, :, D:].astype(np.float64)))
    want = np.repeat(means, H // KV, axis=1) * gate
    worst = np.abs(got - want).max()
    assert worst < 2e-5, worst


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("pos", [1, 2, 3, 5, 17, 30, 31])
def test_chunk_from_a_position_that_splits_a_row_group(kind, pos):
    # A chunk that starts at a position that is no multiple of 4, early in the cache: in the row group whose
    # tokens see 30 .. 33 keys some rows end inside key block 0 and others reach block 1, so the wave that
    # takes the odd blocks meets rows for which its first block is masked whole.
    rng = np.random.default_rng(600 + pos)
    tokens = 70
    n = pos + tokens
    k = rng.standard_normal((n, VALUES)).astype(np.float32)
    v = rng.standard_normal((n, VALUES)).astype(np.float32)
    q16 = rng.standard_normal((tokens, H, D)).astype(np.float16)
    qg = rng.standard_normal((tokens, H, 2 * D)).astype(np.float32)
    kc, vc, kf, vf = make_cache(kind, k, v, n + 9, chunk_from=pos)
    got = run(kind, q16, kc, vc, qg, pos, tokens)
    assert np.isfinite(got).all()
    want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
    assert oracle.rel_rms(got, want) < REL_RMS
    assert np.abs(got - want).max() < MAX_ABS
