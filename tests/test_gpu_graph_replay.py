"""Plans replayed from a HIP graph (the counterpart of the reference's indirect command buffer,
src/plan.rs:229-235; tests/plan.rs:27-45 asks that serial == replay exactly).  A graph is replayed
several times, with eager work of the program between the replays and another position each time,
and every replay is checked against the same launches run eagerly."""
import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind,capacity", [(saetta.KvBits.Eight, 4096), (saetta.KvBits.Eight, 32768),
                                           (saetta.KvBits.Four, 4096), (saetta.KvBits.Half, 4096)])
def test_token_step_replays_bit_for_bit(kind, capacity):
    # one token of an attention layer: store (norm, rope, append) then decode, at the plan's position
    rng = np.random.default_rng(capacity + kind.value)
    qg, k, v = (dev(rng.standard_normal(n).astype(np.float32)) for n in (H * 2 * D, KV * D, KV * D))
    qn, kn = dev(np.ones(D, np.float32)), dev(np.ones(D, np.float32))
    cache = saetta.GpuKvCache.with_bits(H, KV, D, capacity, kind)
    fill = dev(oracle.noise(capacity * VALUES, 3).reshape(capacity, VALUES))
    if kind is saetta.KvBits.Half:
        cache.keys.copy_(fill.flatten().half()), cache.values.copy_(fill.flatten().half())
        keys, values = cache.keys, cache.values
    else:
        keys, values = cache.quant
        keys.encode(fill, 0, capacity), values.encode(fill, 0, capacity)
    q, out = torch.empty(H * D, device="cuda"), torch.empty(H * D, device="cuda")
    plan = saetta.Plan()
    saetta.record_store(plan, qg, k, v, qn, kn, q, keys, values, saetta.PrepParams(H, KV, D, 64, 1e7, 1e-6), capacity)
    if kind is saetta.KvBits.Half:
        cache.decode.record(plan, q, keys, values, qg, out)
    else:
        cache.decode.record_quant(plan, q, keys, values, qg, out)
    eager, graph = plan.build(), plan.build(graph=True)
    assert graph.graph is not None
    for pos in (0, 17, 1000, capacity - 1, 5):
        plan.set_params(saetta.TokenParams(0, pos))
        eager.run()
        want = out.clone()
        out.fill_(float("nan"))
        scratch = torch.randn(1 << 16, device="cuda").sum()  # the program's own eager work between replays
        graph.run()
        torch.cuda.synchronize()
        assert torch.equal(out, want), pos
        assert torch.isfinite(scratch)


def test_deltanet_rows_replay_advances_the_state_like_eager_runs():
    kh, vh, dv, kernel, m = 2, 4, 32, 4, 3
    key, val = kh * 128, vh * dv
    ch = 2 * key + val
    g = torch.Generator(device="cuda").manual_seed(5)

    def r(*n):
        return torch.randn(*n, generator=g, device="cuda")

    x, z, a, b = r(m, ch), r(m, val), r(m, vh), r(m, vh)
    w, alog, dtb, norm = 0.5 * r(ch * kernel), r(vh), r(vh), 1 + 0.1 * r(dv)

    def run(graph, replays):
        conv, st = torch.zeros((kernel - 1) * ch, device="cuda"), torch.zeros(vh * dv * 128, device="cuda")
        mixed, y = torch.empty(m, ch, device="cuda"), torch.empty(m, val, device="cuda")
        plan = saetta.Plan()
        saetta.deltanet_conv_rows(plan, x, w, conv, mixed, ch, kernel, m)
        saetta.deltanet_rows(plan, mixed, a, b, alog, dtb, st, z, norm, y, kh, vh, dv, m, 1e-6)
        built = plan.build(graph=graph)  # building a graph must not run the plan: the state would move
        assert not st.any()
        ys = []
        for _ in range(replays):
            built.run()
            torch.cuda.synchronize()
            ys.append(y.clone())
        return ys, conv, st

    want_y, want_conv, want_st = run(False, 4)
    got_y, got_conv, got_st = run(True, 4)
    for u, v in zip(got_y, want_y):
        assert torch.equal(u, v)
    assert torch.equal(got_conv, want_conv) and torch.equal(got_st, want_st)
    assert not torch.equal(want_y[0], want_y[1])  # the state did move between the runs


def test_serial_and_replay_agree_on_a_chain():
    # tests/plan.rs:27-45: 100 dependent ops each add 1, then one adds the token position, which the
    # device reads from the plan's TokenParams when it runs; run serially, then replayed from the
    # graph at another position.
    n = 1024
    data = torch.zeros(n, device="cuda")
    plan = saetta.Plan()
    for _ in range(100):
        plan.op("add_one", lambda s: data.add_(1.0))
    plan.op("add_position", lambda s: data.add_(plan.params[1]))
    assert len(plan) == 101 and plan.len() == 101 and not plan.is_empty() and saetta.Plan().is_empty()
    assert plan.kernels() == [("add_one", 100), ("add_position", 1)]
    built = plan.build(graph=True)
    plan.set_params(saetta.TokenParams(0, 7))
    assert plan.run_serial() > 0.0
    assert bool((data == 107.0).all())
    plan.set_params(saetta.TokenParams(0, 1000))
    wall, gpu_seconds = built.run_timed()
    assert bool((data == 1207.0).all())
    assert wall > 0.0 and 0.0 < gpu_seconds <= wall
    # commit does not wait; what it returns does
    built.commit().synchronize()
    assert bool((data == 2307.0).all())
    # only the ops of one kernel (Plan::build_where)
    plan.build_where(lambda k: k == "add_position").run()
    assert bool((data == 3307.0).all())
    two = plan.constant([1.5, 2.5])
    assert two.is_cuda and two.tolist() == [1.5, 2.5]
    # a captured plan replays on the current stream: naming another one is refused, not ignored
    other = torch.cuda.Stream()
    with pytest.raises(ValueError, match="current stream"):
        built.run(other)
    built.run(torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert bool((data == 4307.0 + 100.0).all())
