"""Gated DeltaNet over several tokens in one launch (verify rows, prefill chunks) against the oracle.

The oracle runs the tokens one at a time (conv, then step), which is how the reference defines the
result (`record_rows`: "as m calls of record would", src/gpu_layers.rs:686-688; the chunked prefill
of src/prefill.rs:1433-1578 against the CPU layer).  Beyond that, properties the oracle is too slow
for: a 4096-token chunk equals the same tokens in uneven pieces bit for bit, snapshot t equals the
state a t + 1-token call leaves, and the first rows equal the single-token kernels'.
Tolerances as for the single-token kernels: 2e-6 on the conv, 2e-5 (relative to the largest value)
on y and the state; the sums run over 16 lanes of 8 values instead of the CPU's one after the other.
"""
import numpy as np
import pytest
import torch

from gpu_common import dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
K_DIM = 128
EPS = 1e-6


class Layer:
    def __init__(self, k_heads, v_heads, v_dim, kernel, seed):
        rng = np.random.default_rng(seed)
        self.k_heads, self.v_heads, self.v_dim, self.kernel = k_heads, v_heads, v_dim, kernel
        self.key, self.val = k_heads * K_DIM, v_heads * v_dim
        self.channels = 2 * self.key + self.val
        self.conv_w = (0.5 * rng.standard_normal((self.channels, kernel))).astype(np.float32)
        self.a_log = rng.uniform(-1, 1, v_heads).astype(np.float32)
        self.dt_bias = rng.standard_normal(v_heads).astype(np.float32)
        self.norm = (1 + 0.1 * rng.standard_normal(v_dim)).astype(np.float32)
        self.rng = rng

    def inputs(self, tokens):
        r = self.rng
        return (r.standard_normal((tokens, self.channels)).astype(np.float32),
                r.standard_normal((tokens, self.val)).astype(np.float32),
                r.standard_normal((tokens, self.v_heads)).astype(np.float32),
                r.standard_normal((tokens, self.v_heads)).astype(np.float32))

    def zero_state(self):
        return (torch.zeros(self.kernel - 1, self.channels, device="cuda"),
                torch.zeros(self.v_heads * self.v_dim * K_DIM, device="cuda"))

    def gpu_rows(self, x, z, a, b, conv, state, snapshots=False):
        """One call over all the tokens of x; returns mixed, y and the snapshots (or None)."""
        tokens = x.shape[0]
        xd, zd, ad, bd = (dev(np.ascontiguousarray(t)) for t in (x, z, a, b))
        mixed = torch.empty(tokens, self.channels, device="cuda")
        y = torch.empty(tokens, self.val, device="cuda")
        snaps = None
        if snapshots:
            snaps = (torch.full((tokens, self.kernel - 1, self.channels), 7.0, device="cuda"),
                     torch.full((tokens, self.v_heads * self.v_dim * K_DIM), 7.0, device="cuda"))
        plan = saetta.Plan()
        saetta.deltanet_conv_rows(plan, xd, dev(self.conv_w), conv, mixed, self.channels, self.kernel, tokens,
                                  snaps[0] if snapshots else None)
        saetta.deltanet_rows(plan, mixed, ad, bd, dev(self.a_log), dev(self.dt_bias), state, zd, dev(self.norm), y,
                             self.k_heads, self.v_heads, self.v_dim, tokens, EPS, snaps[1] if snapshots else None)
        assert [n for n, _ in plan.ops] == ["deltanet_conv_rows", "deltanet_rows"]
        plan.build().run()
        torch.cuda.synchronize()
        return mixed, y, snaps

    def cpu_rows(self, x, z, a, b, conv, state):
        """Token by token through the oracle; conv and state (numpy) are updated in place."""
        mixed, y, conv_after, state_after = [], [], [], []
        for t in range(x.shape[0]):
            m = oracle.deltanet_conv(self.conv_w, x[t], conv, self.kernel)
            y.append(oracle.deltanet_step(m[:self.key], m[self.key:2 * self.key], m[2 * self.key:], a[t], b[t],
                                          self.a_log, self.dt_bias, state, z[t], self.norm, self.k_heads,
                                          self.v_heads, K_DIM, self.v_dim, EPS))
            mixed.append(m)
            conv_after.append(conv.copy())
            state_after.append(state.copy())
        return np.stack(mixed), np.stack(y), np.stack(conv_after), np.stack(state_after)


def close(got, want, rel):
    return np.abs(got - want).max() <= rel * max(1.0, np.abs(want).max())


def check_against_oracle(layer, tokens, pieces, snapshots, tol=2e-5):
    x, z, a, b = layer.inputs(tokens)
    conv_cpu = np.zeros((layer.kernel - 1, layer.channels), np.float32)
    state_cpu = np.zeros(layer.v_heads * layer.v_dim * K_DIM, np.float32)
    want_mixed, want_y, want_conv, want_state = layer.cpu_rows(x, z, a, b, conv_cpu, state_cpu)
    conv, state = layer.zero_state()
    at = 0
    for n in pieces:
        s = slice(at, at + n)
        mixed, y, snaps = layer.gpu_rows(x[s], z[s], a[s], b[s], conv, state, snapshots)
        assert close(host(mixed), want_mixed[s], 2e-6), (at, n)
        assert close(host(y), want_y[s], tol), (at, n)
        if n:
            assert np.array_equal(host(conv), want_conv[at + n - 1]), (at, n)
            assert close(host(state), want_state[at + n - 1], tol), (at, n)
        if snapshots and n:
            assert np.array_equal(host(snaps[0]), want_conv[s])
            assert close(host(snaps[1]), want_state[s], 2e-5)
            # the last snapshot is the state itself
            assert np.array_equal(host(snaps[1][n - 1]), host(state))
        at += n
    assert at == tokens


def test_real_shape_verify_rows_with_snapshots():
    # configs[4]: 16 key / 32 value heads of 128, conv kernel 4; 1..4 rows as the verify step has
    layer = Layer(16, 32, 128, 4, seed=11)
    check_against_oracle(layer, 10, [1, 2, 3, 4], snapshots=True)


def test_real_shape_chunk_crosses_token_blocks():
    # 37 tokens: two full staged blocks of 16 and a ragged one
    layer = Layer(16, 32, 128, 4, seed=12)
    check_against_oracle(layer, 37, [37], snapshots=False)


def test_real_shape_longer_chunk_against_oracle():
    # From 128 tokens on a call without snapshots runs the delta rule in blocks of 64 tokens on the
    # matrix cores (products of f16 hi and lo parts: about 2^-21 relative per product, held to the same 2e-5 against the
    # oracle's f32 chain).  200 tokens at the real shape: three blocks and a ragged one, every
    # token's output and the last state against the oracle's token-by-token run; then a piece that
    # takes the token-by-token kernels (100) followed by one that takes the blocks (150), the state
    # carried from one to the other.
    layer = Layer(16, 32, 128, 4, seed=13)
    # (the memory the workspace and the outputs are taken from holds NaN patterns: whatever is read
    # before it is written shows)
    junk = [torch.full((32 << 20,), float("nan"), device="cuda") for _ in range(8)]
    del junk
    check_against_oracle(layer, 200, [200], snapshots=False)
    check_against_oracle(layer, 250, [100, 150], snapshots=False)


@pytest.mark.parametrize("scale", [1e-3, 1.0, 1e3])
def test_blocks_of_tokens_hold_values_and_states_far_from_one(scale):
    # The blocks' products take every operand as an f16 hi part and an f16 lo part: a value v (or a state entry) keeps
    # 22 bits while its lo part is a normal f16 (|v| above 2^-3), fewer below (the lo part of 1e-3 is 5e-7, a subnormal
    # with a step of 6e-8: 14 bits left), and nothing above 65504.  The delta rule is linear in (state, values) together,
    # so the state after the same tokens with both scaled by 1e-3 and by 1e3 is held to the oracle's f32 chain at that
    # scale, relative to the largest entry: 2e-5 at 1 and 1e3, 3e-4 at 1e-3 (measured 1e-4; a real layer's values are O(1)).
    # The output is normalised per head with eps = 1e-6 under the root: at scale 1 that eps mutes the heads whose output
    # nearly cancels, at 1e3 it does not, and what is left of such a head's output is its rounding (measured 3e-4 of the
    # largest output against 2e-5 at scale 1): held to 1e-3 there.
    layer = Layer(16, 32, 128, 4, seed=21)
    tokens = 200
    x, z, a, b = layer.inputs(tokens)
    mixed = np.tanh(x).astype(np.float32)  # what a convolution would hand over: q, k and v of every token
    mixed[:, 2 * layer.key:] *= scale
    state0 = (scale * 0.5 * layer.rng.standard_normal(layer.v_heads * layer.v_dim * K_DIM)).astype(np.float32)
    state_cpu = state0.copy()
    want_y = np.stack([oracle.deltanet_step(m[:layer.key], m[layer.key:2 * layer.key], m[2 * layer.key:], a[t], b[t],
                                            layer.a_log, layer.dt_bias, state_cpu, z[t], layer.norm, layer.k_heads,
                                            layer.v_heads, K_DIM, layer.v_dim, EPS).reshape(-1) for t, m in enumerate(mixed)])
    state = dev(state0)
    y = torch.empty(tokens, layer.val, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_rows(plan, dev(mixed), dev(a), dev(b), dev(layer.a_log), dev(layer.dt_bias), state, dev(z),
                         dev(layer.norm), y, layer.k_heads, layer.v_heads, layer.v_dim, tokens, EPS, None)
    plan.build().run()
    torch.cuda.synchronize()
    tol = 3e-4 if scale < 1 else 2e-5
    got = host(state).reshape(-1)
    assert np.isfinite(got).all()
    err = float(np.abs(got - state_cpu).max() / np.abs(state_cpu).max())
    assert err <= tol, (scale, err)
    assert close(host(y), want_y, 2e-5 if scale == 1.0 else 1e-3), scale


def test_blocks_of_tokens_other_value_dims():
    # value dims that are multiples of 16 take the blocks too; 24 keeps to the token-by-token kernels
    for v_dim, tokens in ((16, 130), (64, 192), (256, 129), (24, 140)):
        layer = Layer(2, 4, v_dim, 4, seed=v_dim)
        check_against_oracle(layer, tokens, [tokens], snapshots=False)


@pytest.mark.parametrize("k_heads,v_heads,v_dim,tokens", [(2, 2, 32, 130), (1, 4, 16, 200), (8, 8, 16, 128), (1, 3, 48, 150)])
def test_blocks_of_tokens_other_head_ratios(k_heads, v_heads, v_dim, tokens):
    # Two value heads per key head (the model's ratio) share a workgroup of the blocks' prepare kernel; any
    # other ratio takes one workgroup per value head.  Eight value heads and more are dealt to the XCDs by
    # head, fewer in launch order.
    layer = Layer(k_heads, v_heads, v_dim, 4, seed=100 * k_heads + v_heads)
    check_against_oracle(layer, tokens, [tokens], snapshots=False)


@pytest.mark.parametrize("v_dim,kernel,tokens", [(4, 2, 5), (24, 4, 17), (100, 7, 33), (256, 4, 16), (16, 16, 3)])
def test_other_shapes(v_dim, kernel, tokens):
    layer = Layer(2, 4, v_dim, kernel, seed=v_dim + kernel)
    check_against_oracle(layer, tokens, [tokens // 2, tokens - tokens // 2], snapshots=(v_dim <= 100))


def test_fewer_tokens_than_conv_taps_keep_the_older_state_rows():
    layer = Layer(1, 2, 8, 6, seed=3)
    check_against_oracle(layer, 7, [1, 2, 1, 3], snapshots=True)


def test_first_row_equals_the_single_token_kernels():
    layer = Layer(16, 32, 128, 4, seed=21)
    x, z, a, b = layer.inputs(1)
    conv, state = layer.zero_state()
    state.copy_(torch.randn_like(state) * 0.1)
    conv.copy_(torch.randn_like(conv))
    conv1, state1 = conv.clone(), state.clone()
    mixed, y, _ = layer.gpu_rows(x, z, a, b, conv, state)
    mixed1, y1 = torch.empty(layer.channels, device="cuda"), torch.empty(layer.val, device="cuda")
    key = layer.key
    plan = saetta.Plan()
    saetta.deltanet_conv(plan, dev(x[0]), dev(layer.conv_w), conv1, mixed1, layer.channels, layer.kernel)
    saetta.deltanet_step(plan, mixed1[:key], mixed1[key:2 * key], mixed1[2 * key:], dev(a[0]), dev(b[0]),
                         dev(layer.a_log), dev(layer.dt_bias), state1, dev(z[0]), dev(layer.norm), y1,
                         layer.k_heads, layer.v_heads, layer.v_dim, EPS)
    plan.build().run()
    assert torch.equal(mixed[0], mixed1) and torch.equal(conv, conv1)
    # the two step kernels add a row's 128 products in different orders
    assert close(host(y[0]), host(y1), 2e-5) and close(host(state), host(state1), 2e-5)


def test_full_chunk_against_oracle():
    # The whole 4096-token chunk of the real shape, one call (64 blocks of 64 tokens on the matrix cores),
    # against the oracle's token-by-token run: every token's output and the state after the last one.  The
    # blocks' f16 hi/lo products against the oracle's f32 chain over 4096 dependent steps: outputs to 2e-5,
    # the state to 1e-5 of the largest entry (measured 1.6e-6 and 6e-7: the decay keeps rounding from piling up).
    layer = Layer(16, 32, 128, 4, seed=77)
    tokens = 4096
    x, z, a, b = layer.inputs(tokens)
    conv_cpu = np.zeros((layer.kernel - 1, layer.channels), np.float32)
    state_cpu = np.zeros(layer.v_heads * layer.v_dim * K_DIM, np.float32)
    want_y = np.empty((tokens, layer.v_heads * layer.v_dim), np.float32)
    for t in range(tokens):
        m = oracle.deltanet_conv(layer.conv_w, x[t], conv_cpu, layer.kernel)
        want_y[t] = oracle.deltanet_step(m[:layer.key], m[layer.key:2 * layer.key], m[2 * layer.key:], a[t], b[t],
                                         layer.a_log, layer.dt_bias, state_cpu, z[t], layer.norm, layer.k_heads,
                                         layer.v_heads, K_DIM, layer.v_dim, EPS).reshape(-1)
    conv, state = layer.zero_state()
    _, y, _ = layer.gpu_rows(x, z, a, b, conv, state)
    assert close(host(y).reshape(tokens, -1), want_y, 2e-5)
    assert close(host(state).reshape(-1), state_cpu, 1e-5)
    assert np.array_equal(host(conv), conv_cpu)


def test_full_chunk_equals_uneven_pieces():
    # 4096 tokens at the real shape: what a prefill chunk is.  One call (64 blocks of 64 tokens on the
    # matrix cores) against the same tokens in uneven pieces: the short ones run token by token, the
    # long ones in blocks that start elsewhere.  The two ways differ by rounding only (f16 hi/lo
    # products against the f32 chain): the normalised outputs agree to 2e-5, the states to 1e-5 of
    # the largest entry (measured 1.1e-6 and 3e-7).  Short pieces alone (token by token throughout) agree
    # bit for bit.
    layer = Layer(16, 32, 128, 4, seed=31)
    tokens = 4096
    x, z, a, b = layer.inputs(tokens)
    conv, state = layer.zero_state()
    _, y, _ = layer.gpu_rows(x, z, a, b, conv, state)
    conv2, state2 = layer.zero_state()
    ys, at = [], 0
    for n in (1, 15, 16, 17, 1000, 3047):
        s = slice(at, at + n)
        ys.append(layer.gpu_rows(x[s], z[s], a[s], b[s], conv2, state2)[1])
        at += n
    assert at == tokens
    assert torch.equal(conv, conv2)
    assert float((torch.cat(ys) - y).abs().max()) <= 2e-5 * max(1.0, float(y.abs().max()))
    assert float((state - state2).abs().max()) <= 1e-5 * max(1.0, float(state.abs().max()))
    assert torch.isfinite(y).all() and float(y.abs().max()) > 0.1
    # decay keeps the state bounded: |g| < 1 and beta in (0, 1) with unit keys
    assert float(state.abs().max()) < 1e3
    # token by token throughout: any split gives the same bits
    conv3, state3 = layer.zero_state()
    conv4, state4 = layer.zero_state()
    whole = layer.gpu_rows(x[:100], z[:100], a[:100], b[:100], conv3, state3)[1]
    parts, at = [], 0
    for n in (1, 15, 16, 17, 51):
        s = slice(at, at + n)
        parts.append(layer.gpu_rows(x[s], z[s], a[s], b[s], conv4, state4)[1])
        at += n
    assert torch.equal(torch.cat(parts), whole) and torch.equal(state3, state4)


def test_rejections():
    z = torch.zeros(4096, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_rows(plan, z, z, z, z, z, torch.zeros(3 * 8 * 128, device="cuda"), z, z, z, 2, 3, 8, 1, EPS)
    with pytest.raises(saetta.ffi.SaettaError, match="value heads"):
        plan.build().run()
    plan = saetta.Plan()
    saetta.deltanet_rows(plan, z, z, z, z, z, torch.zeros(2 * 6 * 128, device="cuda"), z, z, z, 1, 2, 6, 1, EPS)
    with pytest.raises(saetta.ffi.SaettaError, match="multiple of 4"):
        plan.build().run()
    with pytest.raises(ValueError):
        saetta.deltanet_rows(saetta.Plan(), z, z, z, z, z, torch.zeros(10, device="cuda"), z, z, z, 2, 4, 8, 1, EPS)
    with pytest.raises(ValueError):
        saetta.deltanet_conv_rows(saetta.Plan(), z, z, z, z, 1024, 4, 8)
    plan = saetta.Plan()
    saetta.deltanet_conv_rows(plan, z, z, z, z, 16, 1, 2)
    with pytest.raises(saetta.ffi.SaettaError, match="kernel size"):
        plan.build().run()
