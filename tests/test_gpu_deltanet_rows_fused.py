"""Gated DeltaNet, up to 8 rows with conv and step in one call (the verify step), against the oracle.

The reference records this as one op (kernel deltanet_rows, GpuDeltaNet::record_rows with
DN_SIMDS = 0, src/gpu_layers.rs:737-757) and defines it by "as m calls of record would"
(src/gpu_layers.rs:686-688): the oracle runs the rows one at a time, conv then step.  Beside it,
the call must agree with the two-call path (deltanet_conv_rows + deltanet_rows) it stands in for.
Tolerances as for the other DeltaNet kernels: the conv state and its snapshots are copies and must
be exact; y, the state and its snapshots within 2e-5 of the largest value.
"""
import numpy as np
import pytest
import torch

from gpu_common import dev, host, oracle, saetta
from test_gpu_deltanet_rows import EPS, K_DIM, Layer, close

pytestmark = pytest.mark.gpu


def gpu_fused(layer, x, z, a, b, conv, state, snapshots):
    rows = x.shape[0]
    xd, zd, ad, bd = (dev(np.ascontiguousarray(t)) for t in (x, z, a, b))
    y = torch.full((rows, layer.val), float("nan"), device="cuda")
    snaps = (None, None)
    if snapshots:
        snaps = (torch.full((rows, layer.kernel - 1, layer.channels), 7.0, device="cuda"),
                 torch.full((rows, layer.v_heads * layer.v_dim * K_DIM), 7.0, device="cuda"))
    plan = saetta.Plan()
    saetta.deltanet_rows_fused(plan, xd, dev(layer.conv_w), conv, ad, bd, dev(layer.a_log), dev(layer.dt_bias), state,
                               zd, dev(layer.norm), y, layer.k_heads, layer.v_heads, layer.v_dim, layer.kernel, rows, EPS,
                               snaps[0], snaps[1])
    assert [n for n, _ in plan.ops] == ["deltanet_rows_fused"]
    plan.build().run()
    torch.cuda.synchronize()
    return y, snaps


def check(layer, pieces, snapshots):
    tokens = sum(pieces)
    x, z, a, b = layer.inputs(tokens)
    conv_cpu = np.zeros((layer.kernel - 1, layer.channels), np.float32)
    state_cpu = np.zeros(layer.v_heads * layer.v_dim * K_DIM, np.float32)
    _, want_y, want_conv, want_state = layer.cpu_rows(x, z, a, b, conv_cpu, state_cpu)
    conv, state = layer.zero_state()
    conv2, state2 = layer.zero_state()
    at = 0
    for n in pieces:
        s = slice(at, at + n)
        y, snaps = gpu_fused(layer, x[s], z[s], a[s], b[s], conv, state, snapshots)
        assert close(host(y), want_y[s], 2e-5), (at, n)
        assert np.array_equal(host(conv), want_conv[at + n - 1]), (at, n)
        assert close(host(state), want_state[at + n - 1], 2e-5), (at, n)
        if snapshots:
            assert np.array_equal(host(snaps[0]), want_conv[s])
            assert close(host(snaps[1]), want_state[s], 2e-5)
            assert np.array_equal(host(snaps[1][n - 1]), host(state))
        # the two-call path on the same rows
        _, y2, _ = layer.gpu_rows(x[s], z[s], a[s], b[s], conv2, state2)
        assert torch.equal(conv, conv2)
        assert close(host(y), host(y2), 2e-5) and close(host(state), host(state2), 2e-5)
        at += n


@pytest.mark.parametrize("snapshots", [False, True])
def test_real_shape_one_to_eight_rows(snapshots):
    # configs[4]: 16 key / 32 value heads of 128, conv kernel 4; every row count the call takes
    layer = Layer(16, 32, 128, 4, seed=41 + snapshots)
    check(layer, [1, 2, 3, 4, 5, 6, 7, 8], snapshots)


@pytest.mark.parametrize("v_dim,kernel", [(4, 2), (24, 4), (100, 7), (256, 4), (16, 16)])
def test_other_shapes(v_dim, kernel):
    # value dims that leave a workgroup's 16 rows ragged; 2, 7 and 16 taps
    layer = Layer(2, 4, v_dim, kernel, seed=v_dim + kernel)
    check(layer, [3, 8, 1], snapshots=(v_dim <= 100))


def test_fewer_rows_than_conv_taps_keep_the_older_state_rows():
    layer = Layer(1, 2, 8, 6, seed=5)
    check(layer, [1, 2, 1, 3], snapshots=True)


def test_no_rows_is_no_work():
    layer = Layer(1, 2, 8, 4, seed=6)
    conv, state = layer.zero_state()
    conv.fill_(3.0), state.fill_(2.0)
    z = torch.zeros(4096, device="cuda")
    plan = saetta.Plan()
    saetta.deltanet_rows_fused(plan, z, dev(layer.conv_w), conv, z, z, dev(layer.a_log), dev(layer.dt_bias), state, z,
                               dev(layer.norm), z, 1, 2, 8, 4, 0, EPS)
    plan.build().run()
    torch.cuda.synchronize()
    assert float(conv.min()) == 3.0 and float(state.min()) == 2.0


def test_rejections():
    z = torch.zeros(1 << 16, device="cuda")
    with pytest.raises(ValueError, match="up to 8"):
        saetta.deltanet_rows_fused(saetta.Plan(), z, z, z, z, z, z, z, z, z, z, z, 1, 2, 8, 4, 9, EPS)
    with pytest.raises(ValueError, match="both"):
        saetta.deltanet_rows_fused(saetta.Plan(), z, z, z, z, z, z, z, z, z, z, z, 1, 2, 8, 4, 2, EPS, conv_snaps=z)
    with pytest.raises(ValueError, match="too small"):
        saetta.deltanet_rows_fused(saetta.Plan(), z[:10], z, z, z, z, z, z, z, z, z, z, 1, 2, 8, 4, 2, EPS)
    plan = saetta.Plan()
    saetta.deltanet_rows_fused(plan, z, z, z, z, z, z, z, z, z, z, z, 2, 3, 8, 4, 2, EPS)
    with pytest.raises(saetta.ffi.SaettaError, match="value heads"):
        plan.build().run()
    plan = saetta.Plan()
    saetta.deltanet_rows_fused(plan, z, z, z, z, z, z, z, z, z, z, z, 1, 2, 8, 17, 2, EPS)
    with pytest.raises(saetta.ffi.SaettaError, match="kernel size"):
        plan.build().run()
