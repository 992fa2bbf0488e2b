"""Gated DeltaNet decode step on the GPU (deltanet_conv + deltanet_step) against the oracle.

The oracle is pinned by the reference's MLX golden vectors at dims 8 (tests/test_oracle_deltanet.py);
here the kernels run the real shape (16 key / 32 value heads of 128, conv kernel 4, configs[4]) and
smaller value dims over several tokens, with the states carried along on both sides.  Dot products
are summed in another order than on the CPU: 2e-5 relative on y and the state, 2e-6 on the conv.
"""
import numpy as np
import pytest
import torch

from gpu_common import dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
K_DIM = 128


def run_tokens(k_heads, v_heads, v_dim, kernel, tokens, seed):
    rng = np.random.default_rng(seed)
    eps = 1e-6
    key, val = k_heads * K_DIM, v_heads * v_dim
    channels = 2 * key + val
    conv_w = (0.5 * rng.standard_normal((channels, kernel))).astype(np.float32)
    a_log = rng.uniform(-1, 1, v_heads).astype(np.float32)
    dt_bias = rng.standard_normal(v_heads).astype(np.float32)
    norm = (1 + 0.1 * rng.standard_normal(v_dim)).astype(np.float32)
    conv_cpu = np.zeros((kernel - 1, channels), np.float32)
    state_cpu = np.zeros(v_heads * v_dim * K_DIM, np.float32)
    conv_gpu, state_gpu = dev(conv_cpu.copy()), dev(state_cpu.copy())
    mixed, y = torch.empty(channels, device="cuda"), torch.empty(val, device="cuda")
    x_d, z_d = torch.empty(channels, device="cuda"), torch.empty(val, device="cuda")
    a_d, b_d = torch.empty(v_heads, device="cuda"), torch.empty(v_heads, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_conv(plan, x_d, dev(conv_w), conv_gpu, mixed, channels, kernel)
    saetta.deltanet_step(plan, mixed[:key], mixed[key:2 * key], mixed[2 * key:], a_d, b_d, dev(a_log), dev(dt_bias),
                         state_gpu, z_d, dev(norm), y, k_heads, v_heads, v_dim, eps)
    assert [n for n, _ in plan.ops] == ["deltanet_conv", "deltanet_step"]
    built = plan.build()
    for t in range(tokens):
        x = rng.standard_normal(channels).astype(np.float32)
        z = rng.standard_normal(val).astype(np.float32)
        a = rng.standard_normal(v_heads).astype(np.float32)
        b = rng.standard_normal(v_heads).astype(np.float32)
        for dst, src in ((x_d, x), (z_d, z), (a_d, a), (b_d, b)):
            dst.copy_(torch.from_numpy(src))
        built.run()
        want_mixed = oracle.deltanet_conv(conv_w, x, conv_cpu, kernel)
        want_y = oracle.deltanet_step(want_mixed[:key], want_mixed[key:2 * key], want_mixed[2 * key:], a, b, a_log,
                                      dt_bias, state_cpu, z, norm, k_heads, v_heads, K_DIM, v_dim, eps)
        assert np.abs(host(mixed) - want_mixed).max() <= 2e-6 * max(1.0, np.abs(want_mixed).max()), t
        assert np.array_equal(host(conv_gpu).reshape(kernel - 1, channels), conv_cpu), t
        assert np.abs(host(y) - want_y).max() <= 2e-5 * max(1.0, np.abs(want_y).max()), t
        assert np.abs(host(state_gpu) - state_cpu).max() <= 2e-5 * max(1.0, np.abs(state_cpu).max()), t


def test_real_shape_over_tokens():
    run_tokens(16, 32, 128, 4, 6, seed=1)


@pytest.mark.parametrize("v_dim", [1, 24, 33, 200, 256])
def test_other_value_dims(v_dim):
    run_tokens(2, 4, v_dim, 4, 3, seed=v_dim)


def test_step_with_vectors_apart():
    # q, k and v in buffers of their own take deltanet_step_kernel (one workgroup per value head);
    # as slices of the conv's output (the tests above) the same call runs the rows kernels.
    rng = np.random.default_rng(11)
    k_heads, v_heads, v_dim, eps = 16, 32, 128, 1e-6
    key, val = k_heads * K_DIM, v_heads * v_dim
    a_log = rng.uniform(-1, 1, v_heads).astype(np.float32)
    dt_bias = rng.standard_normal(v_heads).astype(np.float32)
    norm = (1 + 0.1 * rng.standard_normal(v_dim)).astype(np.float32)
    state_cpu = (0.1 * rng.standard_normal(v_heads * v_dim * K_DIM)).astype(np.float32)
    state_gpu = dev(state_cpu.copy())
    q, k = rng.standard_normal(key).astype(np.float32), rng.standard_normal(key).astype(np.float32)
    v, z = rng.standard_normal(val).astype(np.float32), rng.standard_normal(val).astype(np.float32)
    a, b = rng.standard_normal(v_heads).astype(np.float32), rng.standard_normal(v_heads).astype(np.float32)
    y = torch.empty(val, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_step(plan, dev(q), dev(k), dev(v), dev(a), dev(b), dev(a_log), dev(dt_bias), state_gpu, dev(z),
                         dev(norm), y, k_heads, v_heads, v_dim, eps)
    plan.build().run()
    want_y = oracle.deltanet_step(q, k, v, a, b, a_log, dt_bias, state_cpu, z, norm, k_heads, v_heads, K_DIM, v_dim, eps)
    assert np.abs(host(y) - want_y).max() <= 2e-5 * max(1.0, np.abs(want_y).max())
    assert np.abs(host(state_gpu) - state_cpu).max() <= 2e-5 * max(1.0, np.abs(state_cpu).max())


def test_conv_kernel_sizes_and_rejections():
    run_tokens(1, 1, 16, 2, 3, seed=5)
    run_tokens(1, 2, 16, 7, 9, seed=6)
    z = torch.zeros(4096, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_step(plan, z, z, z, z, z, z, z, torch.zeros(3 * 8 * 128, device="cuda"), z, z, z, 2, 3, 8, 1e-6)
    with pytest.raises(saetta.ffi.SaettaError, match="value heads"):
        plan.build().run()
    with pytest.raises(ValueError):
        saetta.deltanet_step(saetta.Plan(), z, z, z, z, z, z, z, torch.zeros(10, device="cuda"), z, z, z, 2, 4, 8, 1e-6)


@pytest.mark.parametrize("k_heads,v_heads,v_dim,kernel", [(16, 32, 128, 4), (2, 4, 24, 4), (1, 2, 200, 7), (1, 1, 1, 2)])
def test_token_call_matches_conv_then_step(k_heads, v_heads, v_dim, kernel):
    # saetta_deltanet_token: the same token step in two launches with the rows spread over more
    # workgroups; against the oracle over several tokens, states carried on both sides.
    rng = np.random.default_rng(v_dim + kernel)
    eps = 1e-6
    key, val = k_heads * K_DIM, v_heads * v_dim
    channels = 2 * key + val
    conv_w = (0.5 * rng.standard_normal((channels, kernel))).astype(np.float32)
    a_log = rng.uniform(-1, 1, v_heads).astype(np.float32)
    dt_bias = rng.standard_normal(v_heads).astype(np.float32)
    norm = (1 + 0.1 * rng.standard_normal(v_dim)).astype(np.float32)
    conv_cpu = np.zeros((kernel - 1, channels), np.float32)
    state_cpu = np.zeros(v_heads * v_dim * K_DIM, np.float32)
    conv_gpu, state_gpu = dev(conv_cpu.copy()), dev(state_cpu.copy())
    x_d, z_d, y = torch.empty(channels, device="cuda"), torch.empty(val, device="cuda"), torch.empty(val, device="cuda")
    a_d, b_d = torch.empty(v_heads, device="cuda"), torch.empty(v_heads, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_token(plan, x_d, dev(conv_w), conv_gpu, a_d, b_d, dev(a_log), dev(dt_bias), state_gpu, z_d,
                          dev(norm), y, k_heads, v_heads, v_dim, kernel, eps)
    built = plan.build(graph=True)
    for t in range(5):
        x = rng.standard_normal(channels).astype(np.float32)
        z = rng.standard_normal(val).astype(np.float32)
        a = rng.standard_normal(v_heads).astype(np.float32)
        b = rng.standard_normal(v_heads).astype(np.float32)
        for dst, src in ((x_d, x), (z_d, z), (a_d, a), (b_d, b)):
            dst.copy_(torch.from_numpy(src))
        built.run()
        m = oracle.deltanet_conv(conv_w, x, conv_cpu, kernel)
        want_y = oracle.deltanet_step(m[:key], m[key:2 * key], m[2 * key:], a, b, a_log, dt_bias, state_cpu, z, norm,
                                      k_heads, v_heads, K_DIM, v_dim, eps)
        assert np.array_equal(host(conv_gpu).reshape(kernel - 1, channels), conv_cpu), t
        assert np.abs(host(y) - want_y).max() <= 2e-5 * max(1.0, np.abs(want_y).max()), t
        assert np.abs(host(state_gpu) - state_cpu).max() <= 2e-5 * max(1.0, np.abs(state_cpu).max()), t
