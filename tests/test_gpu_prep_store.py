"""The step before the scores in one launch: q/k RMSNorm + RoPE and the token's key and value into
the cache (half, 8-bit, 4-bit), against the oracle's rms_norm / rope / quantize.

Reference path: GpuAttention::record_store (src/gpu_layers.rs:370-411) = attention_prep{,_float}
(kernels/layers.metal:637-702) + two kv_quantize dispatches; CPU definition
src/cpu/attention.rs:110-138.  What is exact and what is not:
  * the codes, scales and biases are bit-exact against quantize() of the f32 key the kernel itself
    produced (k_back) and of v: the fused kernel quantizes as kv_quantize does;
  * q and the normed, rotated key are within 2e-6 relative of the CPU's (the sum of squares is
    added in another order; sin and cos are f64 on both sides);
  * with theta a power of two and the norm a no-op the rotation is the CPU's bit for bit.
"""
import math

import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
ROPE_DIMS, THETA, EPS = 64, 1e7, 1e-6
KINDS = [saetta.KvBits.Half, saetta.KvBits.Eight, saetta.KvBits.Four]


def make_cache(kind, capacity):
    if kind is saetta.KvBits.Half:
        return (torch.zeros(capacity, VALUES, dtype=torch.float16, device="cuda"),
                torch.zeros(capacity, VALUES, dtype=torch.float16, device="cuda"))
    return saetta.QuantRows(kind, VALUES, capacity), saetta.QuantRows(kind, VALUES, capacity)


def slot(cache, kind, token):
    """The stored row of a token: f16 [512] or (codes, scales, biases)."""
    if kind is saetta.KvBits.Half:
        return host(cache)[token]
    w = kind.words_per_group()
    return (host(cache.data).view(np.uint32)[token * 8 * w:(token + 1) * 8 * w],
            host(cache.scales).view(np.uint16)[token * 8:(token + 1) * 8],
            host(cache.biases).view(np.uint16)[token * 8:(token + 1) * 8])


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("pos", [0, 5, 1000, 32767])
def test_one_token(kind, pos):
    rng = np.random.default_rng(pos + kind.value)
    capacity = pos + 3
    qg = rng.standard_normal(H * 2 * D).astype(np.float32) * 3
    k = rng.standard_normal(KV * D).astype(np.float32) * 2
    v = rng.standard_normal(KV * D).astype(np.float32)
    qn = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kn = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    keys, values = make_cache(kind, capacity)
    q_out = torch.full((H * D,), float("nan"), device="cuda")
    k_back = torch.full((KV * D,), float("nan"), device="cuda")
    plan = saetta.Plan()
    p = saetta.PrepParams(H, KV, D, ROPE_DIMS, THETA, EPS)
    saetta.record_store(plan, dev(qg), dev(k), dev(v), dev(qn), dev(kn), q_out, keys, values, p, capacity, k_back=k_back)
    assert [name for name, _ in plan.ops] == ["attention_prep_store"]
    plan.set_params(saetta.TokenParams(0, pos))
    plan.build().run()
    torch.cuda.synchronize()
    wq, wk, wv = oracle.attention_prep(qg, k, v, qn, kn, H, KV, D, ROPE_DIMS, pos, THETA, EPS)
    gq, gk = host(q_out), host(k_back)
    # log2(theta) is carried as f32 (PrepParams): the angle of pair i is off by up to pos * 1.6e-8 rad
    tol = 2e-6 + pos * 2e-8
    assert np.abs(gq - wq).max() <= tol * np.abs(wq).max()
    assert np.abs(gk - wk).max() <= tol * np.abs(wk).max()
    if kind is saetta.KvBits.Half:
        assert np.array_equal(slot(keys, kind, pos), gk.astype(np.float16))
        assert np.array_equal(slot(values, kind, pos), v.astype(np.float16))
    else:
        for cache, x in ((keys, gk), (values, v)):
            data, scales, biases = slot(cache, kind, pos)
            wd, ws, wz = oracle.quantize(x, kind.value)
            assert np.array_equal(scales, ws) and np.array_equal(biases, wz)
            assert np.array_equal(data, wd)
    # nothing else in the cache was touched
    if kind is not saetta.KvBits.Half:
        other = host(keys.scales).view(np.uint16).copy()
        other[pos * 8:(pos + 1) * 8] = 0
        assert not other.any()


def test_rotation_is_the_cpus_when_log2_theta_is_exact():
    # theta = 2^23: PrepParams.log2_theta carries it exactly; unit norm weights and an input whose
    # mean square is 1 - eps up to rounding make the norm nearly the identity.
    theta, pos = float(2 ** 23), 777
    rng = np.random.default_rng(3)
    qg = rng.standard_normal(H * 2 * D).astype(np.float32)
    k = rng.standard_normal(KV * D).astype(np.float32)
    v = rng.standard_normal(KV * D).astype(np.float32)
    ones = np.ones(D, np.float32)
    keys, values = make_cache(saetta.KvBits.Half, pos + 1)
    q_out = torch.empty(H * D, device="cuda")
    k_back = torch.empty(KV * D, device="cuda")
    plan = saetta.Plan()
    saetta.record_store(plan, dev(qg), dev(k), dev(v), dev(ones), dev(ones), q_out, keys, values,
                        saetta.PrepParams(H, KV, D, ROPE_DIMS, theta, EPS), pos + 1, k_back=k_back)
    plan.set_params(saetta.TokenParams(0, pos))
    plan.build().run()
    wq, wk, _ = oracle.attention_prep(qg, k, v, ones, ones, H, KV, D, ROPE_DIMS, pos, theta, EPS)
    # the only difference left is the order of the sum of squares: a relative 1e-7 on the scale
    assert np.abs(host(q_out) - wq).max() <= 4e-7 * np.abs(wq).max()
    assert np.abs(host(k_back) - wk).max() <= 4e-7 * np.abs(wk).max()
    # dims past the rotary ones are only normed
    assert np.allclose(host(k_back).reshape(KV, D)[:, ROPE_DIMS:], wk.reshape(KV, D)[:, ROPE_DIMS:], rtol=4e-7, atol=0)


@pytest.mark.parametrize("kind", [saetta.KvBits.Eight, saetta.KvBits.Half])
def test_verify_rows_and_decode_after_store(kind):
    # m rows at positions pos..pos+m-1 in one launch, then attention over the cache it wrote:
    # the whole step of src/gpu_layers.rs:345-368 minus the projections.
    rng = np.random.default_rng(9)
    m, ctx = 3, 200
    capacity = 256
    # a context already in the cache (written token by token through the same op)
    keys, values = make_cache(kind, capacity)
    qn = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    kn = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    p = saetta.PrepParams(H, KV, D, ROPE_DIMS, THETA, EPS)
    kf, vf = np.zeros((ctx + m, VALUES), np.float32), np.zeros((ctx + m, VALUES), np.float32)
    bits = kind.value

    def stored(x):  # what a decode cache holds of x
        return x.astype(np.float16).astype(np.float32) if kind is saetta.KvBits.Half else oracle.round_trip(x, bits)

    step = 8
    for t0 in range(0, ctx, step):
        qg = rng.standard_normal((step, H, 2 * D)).astype(np.float32)
        k = rng.standard_normal((step, KV * D)).astype(np.float32)
        v = rng.standard_normal((step, KV * D)).astype(np.float32)
        q_out = torch.empty(step, H * D, device="cuda")
        k_back = torch.empty(step, KV * D, device="cuda")
        plan = saetta.Plan()
        saetta.record_store(plan, dev(qg), dev(k), dev(v), dev(qn), dev(kn), q_out, keys, values, p, capacity,
                            rows=step, k_back=k_back)
        plan.set_params(saetta.TokenParams(0, t0))
        plan.build().run()
        kb = host(k_back)
        for r in range(step):
            kf[t0 + r], vf[t0 + r] = stored(kb[r]), stored(v[r])
            wq, wk, _ = oracle.attention_prep(qg[r], k[r], v[r], qn, kn, H, KV, D, ROPE_DIMS, t0 + r, THETA, EPS)
            assert np.abs(kb[r] - wk).max() <= 1e-5 * np.abs(wk).max()
    # the verify step: m new tokens stored, then m rows of attention over ctx + r + 1 tokens
    qg = rng.standard_normal((m, H, 2 * D)).astype(np.float32)
    k = rng.standard_normal((m, KV * D)).astype(np.float32)
    v = rng.standard_normal((m, KV * D)).astype(np.float32)
    q = torch.empty(m, H, D, device="cuda")
    k_back = torch.empty(m, KV * D, device="cuda")
    out = torch.full((m, H, D), float("nan"), device="cuda")
    plan = saetta.Plan()
    dqg = dev(qg)
    saetta.record_store(plan, dqg, dev(k), dev(v), dev(qn), dev(kn), q, keys, values, p, capacity, rows=m, k_back=k_back)
    att = saetta.AttentionRows(H, KV, capacity, m)
    params = [plan.params] * m
    if kind is saetta.KvBits.Half:
        att.record(plan, m, q, keys, values, dqg, out, params)
    else:
        att.record_quant(plan, m, q, keys, values, dqg, out, params)
    plan.set_params(saetta.TokenParams(0, ctx))
    plan.build().run()
    kb = host(k_back)
    for r in range(m):
        kf[ctx + r], vf[ctx + r] = stored(kb[r]), stored(v[r])
    want = oracle.rows(host(q), kf, vf, ctx, m, q_and_gate=qg, threads=8, f64=True)
    assert np.abs(host(out) - want).max() < 2e-5


def test_rejected_arguments():
    keys, values = make_cache(saetta.KvBits.Eight, 8)
    z = torch.zeros(H * 2 * D, device="cuda")
    plan = saetta.Plan()
    saetta.record_store(plan, z, z, z, z, z, z, keys, values, saetta.PrepParams(H, KV, 128, 64, THETA, EPS), 8)
    with pytest.raises(saetta.ffi.SaettaError, match="head dim 256"):
        plan.build().run()
    with pytest.raises(ValueError):
        saetta.record_store(plan, z, z, z, z, z, z, keys, torch.zeros(8, VALUES, dtype=torch.float16, device="cuda"),
                            saetta.PrepParams(H, KV, D, 64, THETA, EPS), 8)
