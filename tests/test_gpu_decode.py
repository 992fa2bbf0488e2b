"""Decode and verify attention on the GPU against the oracle.

Restates tests/attention.rs (half cache at lengths 1,2,127,128,129,1000,4096; quantized
caches at 1,127,129,1000,1024; max abs error < 2e-5 against the f64 formula on the values
the cache stands for) and src/rows.rs:666-743 (m rows == m single-row decodes, < 1e-4),
plus the build's own bar: rel-RMS <= 1e-3 against the f32 CPU path (orc_attend).
"""
import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, cache_pair, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
KINDS = [saetta.KvBits.Half, saetta.KvBits.Eight, saetta.KvBits.Four]
REL_RMS = 1e-3      # tolerance stated for the path, vs the f32 CPU reference
MAX_ABS_F64 = 2e-5  # tests/attention.rs:91,198


def run_decode(att, kind, q, kc, vc, qg, length):
    out = torch.full((H, D), float("nan"), device="cuda")
    plan = saetta.Plan()
    if kind is saetta.KvBits.Half:
        att.record(plan, q, kc, vc, qg, out)
    else:
        att.record_quant(plan, q, kc, vc, qg, out)
    plan.set_params(saetta.TokenParams(0, length - 1))
    plan.build().run()
    return host(out)


@pytest.mark.parametrize("kind", KINDS)
def test_matches_cpu_at_several_lengths(kind):
    capacity = 4096 if kind is saetta.KvBits.Half else 1024
    lengths = [1, 2, 127, 128, 129, 1000, 4096] if kind is saetta.KvBits.Half else [1, 127, 129, 1000, 1024]
    # Big keys make the softmax peaky, which tests the max handling.
    k = (oracle.noise(capacity * VALUES, 1) * 4.0).reshape(capacity, VALUES)
    v = oracle.noise(capacity * VALUES, 2).reshape(capacity, VALUES)
    q = oracle.noise(H * D, 3)
    qg = oracle.noise(H * 2 * D, 4)
    kc, vc, kf, vf = cache_pair(k, v, kind, capacity, poison=False)
    att = saetta.DecodeAttention(H, KV, D, capacity)
    for length in lengths:
        got = run_decode(att, kind, dev(q), kc, vc, dev(qg), length)
        want64 = oracle.attention_f64(q, kf, vf, qg, length, threads=8)
        worst = np.abs(got - want64).max()
        assert worst < MAX_ABS_F64, f"{kind} len {length}: {worst}"
        want32 = oracle.attend(q, kf, vf, length, q_and_gate=qg, threads=8)
        assert oracle.rel_rms(got, want32) < REL_RMS


@pytest.mark.parametrize("kind", KINDS)
def test_rows_past_the_context_never_reach_the_output(kind):
    # hipMalloc'd caches are not zeroed: NaN scales, Inf biases and all-ones codes sit past kv_len.
    capacity, length = 640, 333
    rng = np.random.default_rng(4)
    k = rng.standard_normal((length, VALUES)).astype(np.float32)
    v = rng.standard_normal((length, VALUES)).astype(np.float32)
    q = rng.standard_normal(H * D).astype(np.float32)
    qg = rng.standard_normal(H * 2 * D).astype(np.float32)
    kc, vc, kf, vf = cache_pair(k, v, kind, capacity, poison=True)
    att = saetta.DecodeAttention(H, KV, D, capacity)
    got = run_decode(att, kind, dev(q), kc, vc, dev(qg), length)
    assert np.isfinite(got).all()
    assert np.abs(got - oracle.attention_f64(q, kf, vf, qg, length, threads=8)).max() < MAX_ABS_F64


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8])
def test_verify_rows_match_single_row_decodes(kind, m):
    # src/rows.rs:666-743: contexts 40 and 1024 (+ one that is not a multiple of anything).
    rng = np.random.default_rng(100 + m)
    for ctx in (40, 1024, 1500):
        capacity = -(-(ctx + saetta.MAX_ROWS) // 128) * 128
        tokens = ctx - 1 + m
        k = rng.standard_normal((tokens, VALUES)).astype(np.float32)
        v = rng.standard_normal((tokens, VALUES)).astype(np.float32)
        q = rng.standard_normal((m, H, D)).astype(np.float32)
        qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
        kc, vc, kf, vf = cache_pair(k, v, kind, capacity)
        rows = saetta.AttentionRows(H, KV, capacity, saetta.MAX_ROWS)
        out = torch.full((m, H, D), float("nan"), device="cuda")
        pos = ctx - 1
        params = [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)]
        plan = saetta.Plan()
        if kind is saetta.KvBits.Half:
            rows.record(plan, m, dev(q), kc, vc, dev(qg), out, params)
        else:
            rows.record_quant(plan, m, dev(q), kc, vc, dev(qg), out, params)
        plan.build().run()
        got = host(out)
        want64 = oracle.rows(q, kf, vf, pos, m, q_and_gate=qg, threads=8, f64=True)
        assert np.abs(got - want64).max() < MAX_ABS_F64, f"{kind} ctx {ctx} m {m}"
        # ... and equal to m single-row decodes on the GPU (the reference's own check, < 1e-4).
        att = saetta.DecodeAttention(H, KV, D, capacity)
        for r in range(m):
            one = run_decode(att, kind, dev(q[r]), kc, vc, dev(qg[r]), pos + r + 1)
            assert np.abs(one - got[r]).max() < 1e-4


@pytest.mark.parametrize("kind,m", [(saetta.KvBits.Eight, 2), (saetta.KvBits.Eight, 3), (saetta.KvBits.Eight, 4),
                                    (saetta.KvBits.Four, 1)])
def test_long_context_with_outlier_channels(kind, m):
    # configs[1] in full: 8-bit at 32768 + m rows for m = 2, 3, 4 (m = 1 at this size is in
    # test_large_cache_of_codes_one_row); 4-bit at 20000 with 1 % of channels x8; the new tokens are
    # quantized on the device into the rows after the context.
    rng = np.random.default_rng(8 + m)
    ctx = 32768 if kind is saetta.KvBits.Eight else 20000
    capacity = -(-(ctx + m) // 128) * 128
    k = rng.standard_normal((ctx + m, VALUES)).astype(np.float32)
    v = rng.standard_normal((ctx + m, VALUES)).astype(np.float32)
    if kind is saetta.KvBits.Four:
        ch = rng.choice(VALUES, 5, replace=False)
        k[:, ch] *= 8
        v[:, ch] *= 8
    q = rng.standard_normal((m, H, D)).astype(np.float32)
    qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
    kc, vc, kf, vf = cache_pair(k[:ctx], v[:ctx], kind, capacity)
    kc.encode(dev(k[ctx:].reshape(-1)), ctx, m)
    vc.encode(dev(v[ctx:].reshape(-1)), ctx, m)
    bits = kind.value
    kf = np.concatenate([kf, oracle.round_trip(k[ctx:], bits)])
    vf = np.concatenate([vf, oracle.round_trip(v[ctx:], bits)])
    rows = saetta.AttentionRows(H, KV, capacity, m)
    out = torch.full((m, H, D), float("nan"), device="cuda")
    plan = saetta.Plan()
    rows.record_quant(plan, m, dev(q), kc, vc, dev(qg), out, [saetta.TokenParams(0, ctx).as_tensor("cuda")] * m)
    plan.build().run()
    got = host(out)
    want = oracle.rows(q, kf, vf, ctx, m, q_and_gate=qg, threads=8)
    assert oracle.rel_rms(got, want) < REL_RMS
    want64 = oracle.rows(q, kf, vf, ctx, m, q_and_gate=qg, threads=8, f64=True)
    # Outlier channels carry values 8x larger: the absolute bound scales with them.
    assert np.abs(got - want64).max() < MAX_ABS_F64 * max(1.0, np.abs(want64).max())


def poison_from(cache, bits, token):
    """Everything from row `token` on as uninitialised memory might look: NaN scales, Inf biases,
    all-ones codes."""
    cache.scales[token * 8:] = float("nan")
    cache.biases[token * 8:] = float("inf")
    cache.data[token * 8 * 2 * bits:] = -1


def test_four_bit_150k_tokens_with_append():
    # configs[3] in full: one query token over 150 000 cached tokens of 4-bit codes with 1 % of the
    # channels scaled x8, capacity 150 016, the step's 4 new tokens quantized on the device into
    # the rows after them.  A one-row launch over 4-bit codes in a cache this large takes the
    # two-workgroups-per-CU kernel and 256 splits.  Then two shorter contexts in the same cache
    # (fewer blocks than splits; ragged iterations), the rows past them poisoned.
    kind, bits, ctx, new = saetta.KvBits.Four, 4, 150000, 4
    capacity = 150016
    rng = np.random.default_rng(150)
    k = rng.standard_normal((ctx + new, VALUES)).astype(np.float32)
    v = rng.standard_normal((ctx + new, VALUES)).astype(np.float32)
    ch = rng.choice(VALUES, 5, replace=False)
    k[:, ch] *= 8
    v[:, ch] *= 8
    q = rng.standard_normal(H * D).astype(np.float32)
    qg = rng.standard_normal(H * 2 * D).astype(np.float32)
    kc, vc, kf, vf = cache_pair(k[:ctx], v[:ctx], kind, capacity)
    kc.encode(dev(k[ctx:].reshape(-1)), ctx, new)
    vc.encode(dev(v[ctx:].reshape(-1)), ctx, new)
    # the appended rows are the oracle quantizer's rows, bit for bit
    for cache, x in ((kc, k), (vc, v)):
        data, scales, biases = oracle.quantize(x[ctx:], bits)
        assert np.array_equal(host(cache.data[ctx * 64:(ctx + new) * 64]).view(np.uint32), data.reshape(-1))
        assert np.array_equal(host(cache.scales[ctx * 8:(ctx + new) * 8]).view(np.uint16), scales.reshape(-1))
        assert np.array_equal(host(cache.biases[ctx * 8:(ctx + new) * 8]).view(np.uint16), biases.reshape(-1))
    kf = np.concatenate([kf, oracle.round_trip(k[ctx:], bits)])
    vf = np.concatenate([vf, oracle.round_trip(v[ctx:], bits)])
    att = saetta.DecodeAttention(H, KV, D, capacity)
    for length in (ctx + new, 70001, 1):
        poison_from(kc, bits, length), poison_from(vc, bits, length)
        got = run_decode(att, kind, dev(q), kc, vc, dev(qg), length)
        assert np.isfinite(got).all(), length
        want64 = oracle.attention_f64(q, kf, vf, qg, length, threads=8)
        worst = np.abs(got - want64).max()
        assert worst < MAX_ABS_F64 * max(1.0, np.abs(want64).max()), (length, worst)
        want32 = oracle.attend(q, kf, vf, length, q_and_gate=qg, threads=8)
        assert oracle.rel_rms(got, want32) < REL_RMS, length


@pytest.mark.parametrize("kind", [saetta.KvBits.Eight, saetta.KvBits.Four])
@pytest.mark.parametrize("capacity", [81920, 98304])
def test_register_kernels_one_row_over_codes(kind, capacity):
    # DecodeAttention.kernel = "attention_partial" (the reference's switch between its kernel
    # families, src/attention.rs:36-38) keeps one row over codes on the kernels that load the cache
    # into registers: one workgroup per CU up to 80k tokens of capacity, two per CU and 256 splits
    # above.  Same lengths and poisoned tails as for the kernel with loader waves.
    rng = np.random.default_rng(78)
    k = (rng.standard_normal((capacity, VALUES)) * 2.0).astype(np.float32)
    v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    q = rng.standard_normal(H * D).astype(np.float32)
    qg = rng.standard_normal(H * 2 * D).astype(np.float32)
    att = saetta.DecodeAttention(H, KV, D, capacity)
    att.kernel = "attention_partial"
    kc, vc, kf, vf = cache_pair(k, v, kind, capacity, poison=False)
    for length in [capacity, 50001, 33000, 4100, 100, 1]:
        poison_from(kc, kind.value, length), poison_from(vc, kind.value, length)
        got = run_decode(att, kind, dev(q), kc, vc, dev(qg), length)
        assert np.isfinite(got).all(), length
        worst = np.abs(got - oracle.attention_f64(q, kf, vf, qg, length, threads=8)).max()
        assert worst < MAX_ABS_F64, (length, worst)
    att.kernel = "attention_partial_simd"
    with pytest.raises(ValueError):
        run_decode(att, kind, dev(q), kc, vc, dev(qg), 10)


def test_one_plan_serves_every_position():
    # Context length enters only through TokenParams (src/plan.rs:1-11).
    capacity = 2048
    rng = np.random.default_rng(5)
    k = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    q, qg = rng.standard_normal(H * D).astype(np.float32), rng.standard_normal(H * 2 * D).astype(np.float32)
    kc, vc, kf, vf = cache_pair(k, v, saetta.KvBits.Eight, capacity)
    att = saetta.DecodeAttention(H, KV, D, capacity)
    out = torch.zeros(H, D, device="cuda")
    plan = saetta.Plan()
    att.record_quant(plan, dev(q), kc, vc, dev(qg), out)
    built = plan.build()
    for length in (2048, 5, 700):
        plan.set_params(saetta.TokenParams(0, length - 1))
        built.run()
        assert np.abs(host(out) - oracle.attention_f64(q, kf, vf, qg, length, threads=8)).max() < MAX_ABS_F64
    # kv_len beyond the capacity is clamped (kernels/attention.metal:37).
    plan.set_params(saetta.TokenParams(0, capacity + 50))
    built.run()
    assert np.abs(host(out) - oracle.attention_f64(q, kf, vf, qg, capacity, threads=8)).max() < MAX_ABS_F64
    # Plan::build_where: the reduce alone reproduces the output from the partials.
    out.zero_()
    plan.build_where(lambda name: name == "attention_reduce").run()
    assert np.abs(host(out) - oracle.attention_f64(q, kf, vf, qg, capacity, threads=8)).max() < MAX_ABS_F64


def test_shape_checks():
    with pytest.raises(ValueError):
        saetta.DecodeAttention(16, 2, 128, 1024)
    with pytest.raises(ValueError):
        saetta.DecodeAttention(16, 4, 256, 1024)
    with pytest.raises(ValueError):
        saetta.AttentionRows(16, 2, 1024, 9)


def test_capacity_must_be_whole_blocks():
    # The kernels read whole 16-token blocks; the reference's caches are multiples of 128 (KV_ALIGN).
    capacity = 1000
    z = torch.zeros(capacity * VALUES, dtype=torch.float16, device="cuda")
    q, qg, out = torch.zeros(H * D, device="cuda"), torch.zeros(H * 2 * D, device="cuda"), torch.zeros(H * D, device="cuda")
    att = saetta.DecodeAttention(H, KV, D, capacity)
    plan = saetta.Plan()
    att.record(plan, q, z, z, qg, out)
    plan.set_params(saetta.TokenParams(0, 10))
    with pytest.raises(saetta.ffi.SaettaError, match="multiple of 16"):
        plan.build().run()


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("kind", [saetta.KvBits.Eight, saetta.KvBits.Four])
def test_large_cache_of_codes_several_rows(kind, m):
    # Two to four rows over codes in a cache of 24k tokens and more whose longest share is one round of
    # 17 blocks (capacities up to 34816) run the keys-first kernel in one round, two rows to a tile; three
    # rows: the second tile's upper half repeats row 2.  Capacity 35072: a share can be 18 blocks, which
    # the same kernel takes in three rounds of 6.  Positions: the first tokens of a cache (row r sees r + 1
    # tokens: whole shares are empty for the earlier rows); one block per share; shares of a few
    # blocks; shares of 16 and of 17 blocks side by side; the whole capacity.  The rows past the last
    # token are poisoned.
    rng = np.random.default_rng(770 + m)
    q = rng.standard_normal((m, H, D)).astype(np.float32)
    qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
    for capacity in (34816, 24576, 35072):
        k = (rng.standard_normal((capacity, VALUES)) * 2.0).astype(np.float32)
        v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
        rows = saetta.AttentionRows(H, KV, capacity, m)
        for tokens in [m, 2049, 16400, 33000, capacity]:
            if tokens > capacity:
                continue
            pos = tokens - m
            kc, vc, kf, vf = cache_pair(k[:tokens], v[:tokens], kind, capacity, poison=True)
            out = torch.full((m, H, D), float("nan"), device="cuda")
            params = [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)]
            plan = saetta.Plan()
            rows.record_quant(plan, m, dev(q), kc, vc, dev(qg), out, params)
            plan.build().run()
            got = host(out)
            assert np.isfinite(got).all(), (capacity, tokens)
            want64 = oracle.rows(q, kf, vf, pos, m, q_and_gate=qg, threads=8, f64=True)
            worst = np.abs(got - want64).max()
            assert worst < MAX_ABS_F64, (capacity, tokens, worst)
            del kc, vc


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("kind", [saetta.KvBits.Eight, saetta.KvBits.Four])
def test_several_rows_in_caches_of_65536_and_131072_tokens(kind, m):
    # The reference's caches are 8192 * 2^k tokens (src/gpu_model.rs:390,406-416): a verify step at 32k
    # tokens runs in a cache of 65536.  The keys-first kernel sees the length when it runs: shares of up to
    # 17 blocks are one round whatever the capacity is, longer ones rounds of up to 8 blocks with the
    # maxima and sums carried from round to round.  Positions: the first tokens of a cache; a block per
    # share; shares of 16 and 17 blocks side by side (one round); 18 to 20 blocks (three rounds of 6 and
    # 7); 25 blocks (rounds of 7 and 4); the whole capacity (4 and 8 rounds of 8).  The rows past the last
    # token are poisoned.
    rng = np.random.default_rng(6500 + m)
    q = rng.standard_normal((m, H, D)).astype(np.float32)
    qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
    for capacity in (65536, 131072):
        k = (rng.standard_normal((capacity, VALUES)) * 2.0).astype(np.float32)
        v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
        rows = saetta.AttentionRows(H, KV, capacity, m)
        for tokens in [m, 2049, 33000, 38000, 50001, capacity]:
            pos = tokens - m
            kc, vc, kf, vf = cache_pair(k[:tokens], v[:tokens], kind, capacity, poison=True)
            out = torch.full((m, H, D), float("nan"), device="cuda")
            params = [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)]
            plan = saetta.Plan()
            rows.record_quant(plan, m, dev(q), kc, vc, dev(qg), out, params)
            plan.build().run()
            got = host(out)
            assert np.isfinite(got).all(), (capacity, tokens)
            want64 = oracle.rows(q, kf, vf, pos, m, q_and_gate=qg, threads=8, f64=True)
            worst = np.abs(got - want64).max()
            assert worst < MAX_ABS_F64, (capacity, tokens, worst)
            del kc, vc


@pytest.mark.parametrize("splits", [100, 64, 7])
def test_several_rows_with_fewer_splits(splits):
    # RowsAttentionParams.splits is an upper bound the caller may lower (src/rows.rs:344-367).  In a
    # cache of 24576 tokens: 100 splits are shares of 15 and 16 blocks, still one round of the
    # keys-first kernel; 64 splits are shares of 24 blocks (three rounds of 8) and 7 of 220 (28 rounds).
    rng = np.random.default_rng(4100 + splits)
    capacity, m, kind = 24576, 3, saetta.KvBits.Eight
    k = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    q = rng.standard_normal((m, H, D)).astype(np.float32)
    qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
    rows = saetta.AttentionRows(H, KV, capacity, m)
    rows.splits = splits
    for tokens in [capacity, 5000]:
        pos = tokens - m
        kc, vc, kf, vf = cache_pair(k[:tokens], v[:tokens], kind, capacity, poison=True)
        out = torch.full((m, H, D), float("nan"), device="cuda")
        plan = saetta.Plan()
        rows.record_quant(plan, m, dev(q), kc, vc, dev(qg), out, [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)])
        plan.build().run()
        got = host(out)
        assert np.isfinite(got).all(), tokens
        worst = np.abs(got - oracle.rows(q, kf, vf, pos, m, q_and_gate=qg, threads=8, f64=True)).max()
        assert worst < MAX_ABS_F64, (tokens, worst)
        del kc, vc


@pytest.mark.parametrize("capacity", [81920, 49152, 34816])
@pytest.mark.parametrize("kind", [saetta.KvBits.Eight, saetta.KvBits.Four])
def test_large_cache_of_codes_one_row(kind, capacity):
    # One row over codes in a cache of 24k tokens and more runs the kernel whose extra waves move the
    # codes into LDS, the keys first: a share of up to 17 blocks in one round, a longer one in rounds of up
    # to 8 blocks in alternate halves of LDS.  Lengths: less than one block; a single block per share;
    # shares of a few blocks; shares of 16 and of 17 blocks side by side (33000 tokens, and the whole of
    # 34816: every share has block 16); 18 blocks and more: three rounds of 6 (34817 tokens and up), odd
    # and even numbers of rounds, last rounds shorter than the others, up to five rounds at 81920.  The
    # rows past each length are poisoned.
    rng = np.random.default_rng(77)
    k = (rng.standard_normal((capacity, VALUES)) * 2.0).astype(np.float32)
    v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    q = rng.standard_normal(H * D).astype(np.float32)
    qg = rng.standard_normal(H * 2 * D).astype(np.float32)
    att = saetta.DecodeAttention(H, KV, D, capacity)
    for length in [1, 100, 2049, 8200, 16400, 33000, 34816, 34817, 50001, 81920]:
        if length > capacity:
            continue
        kc, vc, kf, vf = cache_pair(k[:length], v[:length], kind, capacity, poison=True)
        got = run_decode(att, kind, dev(q), kc, vc, dev(qg), length)
        assert np.isfinite(got).all(), length
        worst = np.abs(got - oracle.attention_f64(q, kf, vf, qg, length, threads=8)).max()
        assert worst < MAX_ABS_F64, (length, worst)
        del kc, vc


def test_four_bit_one_row_in_a_cache_of_131072_tokens():
    # One row over 4-bit codes in a cache of 131072 tokens: shares of up to 64 blocks, eight rounds in alternate
    # halves of LDS, each half refilled several times.  Lengths: a single token; shares of 35 blocks (an odd
    # number of rounds, the last one short); 120000 tokens; the whole capacity.  The rows past each length
    # are poisoned.
    rng = np.random.default_rng(131)
    capacity, kind = 131072, saetta.KvBits.Four
    k = (rng.standard_normal((capacity, VALUES)) * 2.0).astype(np.float32)
    v = rng.standard_normal((capacity, VALUES)).astype(np.float32)
    q = rng.standard_normal(H * D).astype(np.float32)
    qg = rng.standard_normal(H * 2 * D).astype(np.float32)
    att = saetta.DecodeAttention(H, KV, D, capacity)
    for length in [1, 70001, 120000, capacity]:
        kc, vc, kf, vf = cache_pair(k[:length], v[:length], kind, capacity, poison=True)
        got = run_decode(att, kind, dev(q), kc, vc, dev(qg), length)
        assert np.isfinite(got).all(), length
        worst = np.abs(got - oracle.attention_f64(q, kf, vf, qg, length, threads=8)).max()
        assert worst < MAX_ABS_F64, (length, worst)
        del kc, vc


@pytest.mark.parametrize("kind,ctx,m", [(saetta.KvBits.Eight, 32768, 1), (saetta.KvBits.Eight, 32768, 4),
                                        (saetta.KvBits.Eight, 131072, 1), (saetta.KvBits.Four, 150000, 1),
                                        (saetta.KvBits.Four, 32768, 3), (saetta.KvBits.Half, 4096, 2)])
def test_equal_keys_give_the_mean_of_the_values(kind, ctx, m):
    # A closed form that holds at any size and needs no attention code to check: when every key in the
    # cache is the same row, every token's score is the same number whatever q is, so row r's output is
    # the plain mean of the first pos + r + 1 value rows times sigmoid(gate).  A token counted twice, a
    # share dropped or a merge weighted wrongly moves the mean.  The mean is taken here in f64 over the
    # values the cache stands for.
    rng = np.random.default_rng(9000 + ctx % 1000 + m)
    tokens = ctx - 1 + m
    capacity = -(-tokens // 128) * 128
    k = np.tile((rng.standard_normal(VALUES) * 3.0).astype(np.float32), (tokens, 1))
    v = rng.standard_normal((tokens, VALUES)).astype(np.float32)
    v[:, 5] += 3.0  # a channel whose mean is far from zero
    q = rng.standard_normal((m, H, D)).astype(np.float32)
    qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
    kc, vc, kf, vf = cache_pair(k, v, kind, capacity, poison=True)
    out = torch.full((m, H, D), float("nan"), device="cuda")
    pos = ctx - 1
    plan = saetta.Plan()
    if m == 1:
        att = saetta.DecodeAttention(H, KV, D, capacity)
        if kind is saetta.KvBits.Half:
            att.record(plan, dev(q[0]), kc, vc, dev(qg[0]), out[0])
        else:
            att.record_quant(plan, dev(q[0]), kc, vc, dev(qg[0]), out[0])
        plan.set_params(saetta.TokenParams(0, pos))
    else:
        rows = saetta.AttentionRows(H, KV, capacity, m)
        params = [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)]
        if kind is saetta.KvBits.Half:
            rows.record(plan, m, dev(q), kc, vc, dev(qg), out, params)
        else:
            rows.record_quant(plan, m, dev(q), kc, vc, dev(qg), out, params)
    plan.build().run()
    got = host(out)
    sums = np.cumsum(vf[pos:tokens].astype(np.float64), axis=0) + vf[:pos].astype(np.float64).sum(axis=0)
    for r in range(m):
        mean = (sums[r] / (pos + r + 1)).reshape(KV, D)
        gate = 1.0 / (1.0 + np.exp(-qg[r].reshape(H, 2 * D)[:, D:].astype(np.float64)))
        want = np.repeat(mean, H // KV, axis=0) * gate
        worst = np.abs(got[r] - want).max()
        assert worst < MAX_ABS_F64, (kind, ctx, m, r, worst)


@pytest.mark.parametrize("kv_heads", [1, 4])
@pytest.mark.parametrize("kind", KINDS)
def test_other_head_counts(kind, kv_heads):
    # 8 and 32 q heads (1 and 4 kv heads): one row and three verify rows at a short and at a long context (the
    # register kernels, and for the codes at 32768 the loader kernels), against the f64 formula.  The model
    # has 16 / 2; the entry points take any kv head count with 8 q heads each.
    rng = np.random.default_rng(900 + kv_heads)
    heads, values = 8 * kv_heads, kv_heads * D
    for ctx in (300, 4000 if kind is saetta.KvBits.Half else 32768):
        m = 3
        capacity = -(-(ctx + m) // 128) * 128
        tokens = ctx - 1 + m
        k = rng.standard_normal((tokens, values)).astype(np.float32)
        v = rng.standard_normal((tokens, values)).astype(np.float32)
        q = rng.standard_normal((m, heads, D)).astype(np.float32)
        qg = rng.standard_normal((m, heads, 2 * D)).astype(np.float32)
        if kind is saetta.KvBits.Half:
            kc = torch.full((capacity, values), float("nan"), dtype=torch.float16, device="cuda")
            vc = torch.full((capacity, values), float("nan"), dtype=torch.float16, device="cuda")
            kc[:tokens], vc[:tokens] = dev(k.astype(np.float16)), dev(v.astype(np.float16))
            kf, vf = oracle.round_trip(k, 16), oracle.round_trip(v, 16)
        else:
            kc, vc = saetta.QuantRows(kind, values, capacity), saetta.QuantRows(kind, values, capacity)
            for c, x in ((kc, k), (vc, v)):
                c.scales[:], c.biases[:], c.data[:] = float("nan"), float("inf"), -1
                c.encode(dev(x.reshape(-1)), 0, tokens)
            bits = kind.value
            kf, vf = oracle.round_trip(k, bits), oracle.round_trip(v, bits)
        pos = ctx - 1
        rows = saetta.AttentionRows(heads, kv_heads, capacity, saetta.MAX_ROWS)
        out = torch.full((m, heads, D), float("nan"), device="cuda")
        params = [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)]
        plan = saetta.Plan()
        (rows.record if kind is saetta.KvBits.Half else rows.record_quant)(plan, m, dev(q), kc, vc, dev(qg), out, params)
        plan.build().run()
        want = oracle.rows(q, kf, vf, pos, m, heads=heads, kv_heads=kv_heads, q_and_gate=qg, threads=8, f64=True)
        assert np.abs(host(out) - want).max() < MAX_ABS_F64, (kind, kv_heads, ctx)
        att = saetta.DecodeAttention(heads, kv_heads, D, capacity)
        one = torch.full((heads, D), float("nan"), device="cuda")
        plan = saetta.Plan()
        (att.record if kind is saetta.KvBits.Half else att.record_quant)(plan, dev(q[0]), kc, vc, dev(qg[0]), one)
        plan.set_params(saetta.TokenParams(0, pos))
        plan.build().run()
        assert np.abs(host(one) - want[0]).max() < MAX_ABS_F64, (kind, kv_heads, ctx)
