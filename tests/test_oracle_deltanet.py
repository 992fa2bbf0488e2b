"""The oracle's Gated DeltaNet against the reference's golden vectors and against what the
mathematics fixes.

src/cpu/deltanet.rs:162-204 holds MLX outputs for six tokens; the same file, the same bounds
(outputs 1e-4, conv state 1e-5, recurrent state 1e-4).  The golden run pins the whole chain
(conv, SiLU, normalize_qk, gates, delta rule, gated RMSNorm, head -> key head map, projections);
the closed forms below pin the pieces one by one, so that a dropped term or a swapped index fails.
"""
import json
import os

import numpy as np

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "deltanet.json")


def close(got, want, tol):
    got, want = np.asarray(got, np.float64).reshape(-1), np.asarray(want, np.float64).reshape(-1)
    return np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max())


def test_layer_matches_mlx_over_six_tokens():
    f = json.load(open(GOLDEN))
    cfg = {k: f[k] for k in ("hidden", "k_heads", "v_heads", "k_dim", "v_dim", "kernel", "eps")}
    names = ["in_proj_qkv", "in_proj_z", "in_proj_b", "in_proj_a", "out_proj", "conv1d", "A_log", "dt_bias", "norm"]
    layer = oracle.DeltaNetLayer(cfg, {n: f[n] for n in names})
    for i, (x, want) in enumerate(zip(f["inputs"], f["outputs"])):
        assert close(layer.step(x), want, 1e-4), f"token {i}"
    assert close(layer.conv, f["conv_state"], 1e-5)
    assert close(layer.recurrent, f["state"], 1e-4)


def test_conv_is_a_causal_depthwise_filter_with_a_shifting_state():
    rng = np.random.default_rng(0)
    channels, kernel = 10, 4
    w = rng.standard_normal((channels, kernel)).astype(np.float32)
    xs = rng.standard_normal((7, channels)).astype(np.float32)
    state = np.zeros((kernel - 1, channels), np.float32)
    for t in range(7):
        got = oracle.deltanet_conv(w, xs[t], state, kernel)
        hist = np.concatenate([np.zeros((kernel, channels)), xs.astype(np.float64)])[t + 1:t + 1 + kernel]  # oldest first
        pre = (hist * w.T.astype(np.float64)).sum(0)
        assert close(got, pre / (1 + np.exp(-pre)), 1e-6)
        assert np.array_equal(state[-1], xs[t])
        if t >= 2:
            assert np.array_equal(state[0], xs[t - 2])


def step_f64(q, k, v, a, b, a_log, dt_bias, state, z, norm, kh, vh, dk, dv, eps):
    """The recurrence written from its definition in f64: S <- g S; d = (v - S k) beta; S += d k^T; y = S q."""
    q = q.reshape(kh, dk).astype(np.float64)
    k = k.reshape(kh, dk).astype(np.float64)
    q = q / np.sqrt((q * q).sum(1, keepdims=True) + eps) / np.sqrt(dk)
    k = k / np.sqrt((k * k).sum(1, keepdims=True) + eps)
    S = state.reshape(vh, dv, dk).astype(np.float64)
    y = np.zeros((vh, dv))
    for h in range(vh):
        x = float(a[h]) + float(dt_bias[h])
        g = np.exp(-np.exp(float(a_log[h])) * np.log1p(np.exp(x)))
        beta = 1 / (1 + np.exp(-float(b[h])))
        S[h] *= g
        d = (v.reshape(vh, dv)[h] - S[h] @ k[h * kh // vh]) * beta
        S[h] += np.outer(d, k[h * kh // vh])
        o = S[h] @ q[h * kh // vh]
        o = o / np.sqrt((o * o).mean() + eps) * norm
        zz = z.reshape(vh, dv)[h].astype(np.float64)
        y[h] = o * zz / (1 + np.exp(-zz))
    return y.reshape(-1), S.reshape(-1)


def test_step_matches_the_f64_recurrence_and_its_special_cases():
    rng = np.random.default_rng(1)
    kh, vh, dk, dv, eps = 2, 6, 16, 12, 1e-6
    state = (0.1 * rng.standard_normal(vh * dv * dk)).astype(np.float32)
    for _ in range(4):
        args = [rng.standard_normal(n).astype(np.float32) for n in (kh * dk, kh * dk, vh * dv, vh, vh, vh, vh)]
        z = rng.standard_normal(vh * dv).astype(np.float32)
        norm = (1 + 0.1 * rng.standard_normal(dv)).astype(np.float32)
        want_y, want_s = step_f64(*args, state, z, norm, kh, vh, dk, dv, eps)
        got_y = oracle.deltanet_step(*args, state, z, norm, kh, vh, dk, dv, eps)
        assert close(got_y, want_y, 2e-5) and close(state, want_s, 2e-5)
    # beta -> 1 (b large) and g -> 1 (a very negative): after the step S k = v exactly (the write
    # replaces what the key held), and reading with q = k returns v / sqrt(dk) before the norm
    q = rng.standard_normal(kh * dk).astype(np.float32)
    v = rng.standard_normal(vh * dv).astype(np.float32)
    state = (0.1 * rng.standard_normal(vh * dv * dk)).astype(np.float32)
    big, small = np.full(vh, 40, np.float32), np.full(vh, -40, np.float32)
    zero = np.zeros(vh, np.float32)
    oracle.deltanet_step(q, q, v, small, big, zero, zero, state, np.ones(vh * dv, np.float32), np.ones(dv, np.float32),
                         kh, vh, dk, dv, eps)
    kn = q.reshape(kh, dk).astype(np.float64)
    kn = kn / np.sqrt((kn * kn).sum(1, keepdims=True) + eps)
    S = state.reshape(vh, dv, dk).astype(np.float64)
    for h in range(vh):
        assert close(S[h] @ kn[h * kh // vh], v.reshape(vh, dv)[h], 1e-5)
    # g -> 0 (a large with A_log = 0): the old state is forgotten, S = beta v k^T
    state = rng.standard_normal(vh * dv * dk).astype(np.float32)
    oracle.deltanet_step(q, q, v, big, zero, zero, zero, state, np.ones(vh * dv, np.float32), np.ones(dv, np.float32),
                         kh, vh, dk, dv, eps)
    S = state.reshape(vh, dv, dk).astype(np.float64)
    for h in range(vh):
        assert close(S[h], 0.5 * np.outer(v.reshape(vh, dv)[h], kn[h * kh // vh]), 1e-5)
