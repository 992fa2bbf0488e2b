"""Pins the oracle's attention functions (CPU only).

Evidence: the reference's MLX golden vectors (attention.json, ops.json), torch's
float64 scaled_dot_product_attention as an independent library routine, and
closed forms (one key, equal keys, one dominating key).
"""
import json
import os

import numpy as np
import pytest
import torch

import oracle

H, KV, D = 16, 2, 256


def load(golden_dir, name):
    with open(os.path.join(golden_dir, name)) as f:
        return json.load(f)


def assert_close(got, want, tol):
    # src/cpu/testdata.rs:53-59: |g - w| <= tol * max(1, |w|)
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape
    assert (np.abs(got - want) <= tol * np.maximum(1.0, np.abs(want))).all()


def test_ops_match_mlx(golden_dir):
    # src/cpu/ops.rs:81-110
    f = load(golden_dir, "ops.json")
    x = np.float32(f["x"])
    assert_close(oracle.softmax(x), f["softmax"], 1e-6)
    assert_close(oracle.rms_norm(x, f["w"], 1e-6), f["rms_norm"], 1e-5)
    rope_in = np.float32(f["rope_in"])
    for pos, want in zip(f["rope_positions"], f["rope_out"]):
        got = np.concatenate([oracle.rope(rope_in[i:i + 16], 4, pos, 1e7) for i in range(0, 48, 16)])
        assert_close(got, want, 1e-4)


def test_attention_layer_matches_mlx_over_four_tokens(golden_dir):
    # src/cpu/attention.rs:188-221
    f = load(golden_dir, "attention.json")
    cfg = {k: f[k] for k in ("hidden", "heads", "kv_heads", "head_dim", "rope_dims", "rope_theta", "eps")}
    weights = {k: f[k] for k in ("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm")}
    layer = oracle.AttentionLayer(cfg, weights)
    for x, want in zip(f["inputs"], f["outputs"]):
        assert_close(layer.step(x), want, 1e-4)
    assert layer.len == 4


def sdpa64(q, k, v, lens, gate=None):
    """torch float64 SDPA with GQA expansion; row r of q sees lens[r] keys."""
    rows = q.shape[0]
    qt = torch.from_numpy(q.astype(np.float64)).permute(1, 0, 2)  # [H, rows, D]
    n = max(lens)
    kt = torch.from_numpy(k[:n].astype(np.float64)).permute(1, 0, 2).repeat_interleave(H // KV, 0)
    vt = torch.from_numpy(v[:n].astype(np.float64)).permute(1, 0, 2).repeat_interleave(H // KV, 0)
    mask = torch.arange(n)[None, :] < torch.tensor(lens)[:, None]
    out = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=mask[None])
    out = out.permute(1, 0, 2).numpy()
    if gate is not None:
        out = out / (1.0 + np.exp(-gate.astype(np.float64)))
    assert out.shape == (rows, H, D)
    return out


@pytest.fixture(scope="module")
def data():
    rng = np.random.default_rng(1)
    n = 300
    k = rng.standard_normal((n, KV, D)).astype(np.float32)
    v = rng.standard_normal((n, KV, D)).astype(np.float32)
    q = rng.standard_normal((5, H, D)).astype(np.float32)
    qg = rng.standard_normal((5, H, 2 * D)).astype(np.float32)
    return q, k, v, qg


@pytest.mark.parametrize("length", [1, 2, 127, 300])
def test_attend_matches_torch_sdpa(data, length):
    q, k, v, qg = data
    want = sdpa64(q[:1], k, v, [length], qg[:1, :, D:])[0]
    got = oracle.attend(q[0], k, v, length, q_and_gate=qg[0])
    assert np.abs(got - want).max() < 2e-6
    got64 = oracle.attention_f64(q[0], k, v, qg[0], length)
    assert np.abs(got64 - want).max() < 1e-12
    # without a gate
    want = sdpa64(q[:1], k, v, [length])[0]
    assert np.abs(oracle.attend(q[0], k, v, length) - want).max() < 4e-6
    assert np.abs(oracle.attention_f64(q[0], k, v, None, length) - want).max() < 1e-12


def test_head_to_kv_head_map_and_gate_slot():
    # Values of kv head 1 are 7, of kv head 0 are 3: heads 0-7 must see 3, heads 8-15 see 7.
    k = np.zeros((4, KV, D), np.float32)
    v = np.empty((4, KV, D), np.float32)
    v[:, 0], v[:, 1] = 3.0, 7.0
    q = np.ones((H, D), np.float32)
    out = oracle.attend(q, k, v, 4)
    assert np.allclose(out[:8], 3.0) and np.allclose(out[8:], 7.0)
    # The gate of head h is q_and_gate[h, D:], not [h, :D].
    qg = np.zeros((H, 2 * D), np.float32)
    qg[:, :D] = 50.0
    qg[3, D:] = -50.0
    out = oracle.attend(q, k, v, 4, q_and_gate=qg)
    assert np.allclose(np.delete(out, 3, 0)[:7], 1.5) and np.allclose(out[3], 0.0, atol=1e-20)
    out64 = oracle.attention_f64(q, k, v, qg, 4)
    assert np.allclose(np.delete(out64, 3, 0)[:7], 1.5) and np.allclose(out64[3], 0.0, atol=1e-20)


def test_closed_forms(data):
    q, k, v, _ = data
    # One key: the output is that value.
    assert np.allclose(oracle.attend(q[0], k, v, 1)[:8], v[0, 0], atol=1e-6)
    # Equal keys: the output is the mean of the values.
    k2 = np.repeat(k[:1], 50, 0)
    out = oracle.attend(q[0], k2, v, 50)
    assert np.allclose(out[8:], v[:50, 1].mean(0), atol=1e-5)
    # One dominating key (its score is far above the others): that value.
    k3 = k[:64].copy()
    k3[17, 0] = 40 * q[0, 2] / np.linalg.norm(q[0, 2])
    out = oracle.attend(q[0], k3, v, 64)
    assert np.allclose(out[2], v[17, 0], atol=1e-4)


def test_rows_are_single_tokens_with_growing_context(data):
    q, k, v, qg = data
    pos, m = 290, 4
    got = oracle.rows(q[:m], k, v, pos, m, q_and_gate=qg[:m])
    want = sdpa64(q[:m], k, v, [pos + r + 1 for r in range(m)], qg[:m, :, D:])
    assert np.abs(got - want).max() < 2e-6
    got64 = oracle.rows(q[:m], k, v, pos, m, q_and_gate=qg[:m], f64=True)
    assert np.abs(got64 - want).max() < 1e-12


def test_prefill_is_causal_over_the_chunk(data):
    q, k, v, qg = data
    pos, t = 100, 5
    got = oracle.prefill(q[:t], k, v, pos, t, q_and_gate=qg[:t], threads=2)
    want = sdpa64(q[:t], k, v, [pos + i + 1 for i in range(t)], qg[:t, :, D:])
    assert np.abs(got - want).max() < 2e-6
    # pos 0: the first token sees only itself.
    got = oracle.prefill(q[:t], k, v, 0, t)
    assert np.allclose(got[0, :8], v[0, 0], atol=1e-6)


def test_threads_do_not_change_bits(data):
    q, k, v, qg = data
    a = oracle.attend(q[0], k, v, 300, q_and_gate=qg[0], threads=1)
    b = oracle.attend(q[0], k, v, 300, q_and_gate=qg[0], threads=4)
    assert np.array_equal(a, b)


def test_reference_input_generators():
    x = oracle.noise(1000, 1)
    assert x.min() >= -1 and x.max() < 1 and abs(x.mean()) < 0.1
    # First value by hand: s = 1*a + c, take s >> 40.
    s = (6364136223846793005 + 1442695040888963407) % 2**64
    assert x[0] == np.float32(np.float32(s >> 40) / np.float32(1 << 23) - np.float32(1.0))
    sp = oracle.spread(10, 2).astype(np.float32)
    want = [np.float16(np.float32(((i * 7919 + 2 * 104729) % 1999)) / np.float32(500.0) - np.float32(2.0)) for i in range(10)]
    assert np.array_equal(sp, np.float32(want))
    r = oracle.quant_rows(2)
    assert (r[64:128] == -1.5).all() and np.abs(r[:64]).max() > 5 and np.abs(r[128:192]).max() <= 1
