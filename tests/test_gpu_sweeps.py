"""Seeded sweeps over shapes the other tests do not name: decode / verify over capacities, context
lengths, cache kinds and row counts against the f64 formula (the bar of tests/attention.rs), and
prefill chunks over positions, chunk lengths and cache kinds against the oracle's f32 CPU path (the
bar of tests/attention_prefill.rs).  The cases are drawn from fixed seeds, so every run sees the
same ones; rows past the context hold NaN patterns.
"""
import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, cache_pair, dev, host, oracle, saetta
from test_gpu_prefill import make_cache, run as run_prefill

pytestmark = pytest.mark.gpu
KINDS = [saetta.KvBits.Half, saetta.KvBits.Eight, saetta.KvBits.Four]
CAPACITIES = [128, 256, 1024, 4096, 8192, 16384, 24576, 24704, 32768, 34816, 34944, 40960, 61440, 65536, 81920]


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_decode_and_verify_sweep(seed):
    rng = np.random.default_rng(seed)
    done = 0
    while done < 40:
        kind = KINDS[rng.integers(3)]
        cap = CAPACITIES[rng.integers(len(CAPACITIES))]
        if kind is saetta.KvBits.Half and cap > 16384:
            continue
        m = int(rng.choice([1, 1, 1, 2, 3, 4, 5, 8]))
        ctx = int(rng.choice([1, 2, 15, 16, 17, 127, 129, cap - m, cap - m - 1, int(rng.integers(1, cap - m + 1)),
                              int(rng.integers(1, cap - m + 1))]))
        ctx = max(1, min(ctx, cap - m + 1))
        tokens = ctx - 1 + m
        k = (rng.standard_normal((tokens, VALUES)) * float(rng.choice([1.0, 2.0, 4.0]))).astype(np.float32)
        v = rng.standard_normal((tokens, VALUES)).astype(np.float32)
        q = rng.standard_normal((m, H, D)).astype(np.float32)
        qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
        kc, vc, kf, vf = cache_pair(k, v, kind, cap, poison=True)
        out = torch.full((m, H, D), float("nan"), device="cuda")
        pos = ctx - 1
        plan = saetta.Plan()
        if m == 1 and rng.integers(2):
            att = saetta.DecodeAttention(H, KV, D, cap)
            (att.record if kind is saetta.KvBits.Half else att.record_quant)(plan, dev(q[0]), kc, vc, dev(qg[0]), out[0])
            plan.set_params(saetta.TokenParams(0, pos))
        else:
            rows = saetta.AttentionRows(H, KV, cap, saetta.MAX_ROWS)
            params = [saetta.TokenParams(0, pos + r).as_tensor("cuda") for r in range(m)]
            (rows.record if kind is saetta.KvBits.Half else rows.record_quant)(plan, m, dev(q), kc, vc, dev(qg), out, params)
        plan.build().run()
        got = host(out)
        want = oracle.rows(q, kf, vf, pos, m, q_and_gate=qg, threads=8, f64=True)
        assert np.isfinite(got).all(), (seed, done, kind, cap, ctx, m)
        assert np.abs(got - want).max() < 2e-5, (seed, done, kind, cap, ctx, m)
        del kc, vc
        done += 1


@pytest.mark.parametrize("seed", [11, 12])
def test_prefill_sweep(seed):
    rng = np.random.default_rng(seed)
    for done in range(150):
        kind = KINDS[rng.integers(3)]
        pos = int(rng.choice([0, 0, 1, 15, 16, 31, 32, 33, 100, 511, 1000, int(rng.integers(0, 3000))]))
        tokens = int(rng.choice([1, 2, 3, 15, 16, 17, 31, 32, 33, 64, 100, 257, int(rng.integers(1, 400))]))
        n = pos + tokens
        capacity = n + int(rng.integers(0, 40))
        k = (rng.standard_normal((n, VALUES)) * float(rng.choice([1.0, 2.0]))).astype(np.float32)
        v = rng.standard_normal((n, VALUES)).astype(np.float32)
        q16 = rng.standard_normal((tokens, H, D)).astype(np.float16)
        qg = rng.standard_normal((tokens, H, 2 * D)).astype(np.float32)
        kc, vc, kf, vf = make_cache(kind, k, v, capacity, chunk_from=pos if rng.integers(2) else None)
        got = run_prefill(kind, q16, kc, vc, qg, pos, tokens)
        want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
        assert np.isfinite(got).all(), (seed, done, kind, pos, tokens, capacity)
        assert np.abs(got - want).max() < 2e-3 and oracle.rel_rms(got, want) < 1e-3, (seed, done, kind, pos, tokens, capacity)
