"""The entry point that allocates nothing: saetta_attn_decode_quant_static keeps its partials in a
buffer that is part of the library's code object.  Checked through the C ABI against
saetta_attn_decode_quant (same kernels, so bit for bit), on two calls in a row, the second with
a smaller input, the static buffer still holding the first call's partials."""
import ctypes
import math

import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
ffi = saetta.ffi


def ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def decode_both_ways(bits, capacity, length, seed):
    kind = {8: saetta.KvBits.Eight, 4: saetta.KvBits.Four}[bits]
    gen = torch.Generator(device="cuda").manual_seed(seed)
    keys, values = saetta.QuantRows(kind, VALUES, capacity), saetta.QuantRows(kind, VALUES, capacity)
    keys.encode(torch.randn(length * VALUES, generator=gen, device="cuda"), 0, length)
    values.encode(torch.randn(length * VALUES, generator=gen, device="cuda"), 0, length)
    q = torch.randn(H, D, generator=gen, device="cuda")
    qg = torch.randn(H, 2 * D, generator=gen, device="cuda")
    tp = saetta.TokenParams(0, length - 1).as_tensor("cuda")
    p = ffi.DecodeParamsC(H, KV, capacity, 1.0 / math.sqrt(D))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    lib = ffi.lib()
    # the existing entry point, with scratch of the caller's
    part_o = torch.empty(lib.saetta_part_o_bytes(H, capacity, 1) // 4, device="cuda")
    part_ml = torch.empty(lib.saetta_part_ml_bytes(H, capacity, 1) // 4, device="cuda")
    want = torch.full((H, D), float("nan"), device="cuda")
    ffi.check(lib.saetta_attn_decode_quant(stream, bits, ptr(q), keys.c(), values.c(), ptr(part_o), ptr(part_ml),
                                           ptr(qg), ptr(want), p, ptr(tp), ffi.STAGE_ALL), "attn_decode_quant")
    # the new one: no scratch arguments
    got = torch.full((H, D), float("nan"), device="cuda")
    ffi.check(lib.saetta_attn_decode_quant_static(stream, bits, ptr(q), keys.c(), values.c(), ptr(qg), ptr(got), p,
                                                  ptr(tp), ffi.STAGE_ALL), "attn_decode_quant_static")
    return host(got), host(want), (q, qg, keys, values)


def test_static_scratch_matches_the_callers_scratch_twice_in_a_row():
    ffi.check(ffi.lib().saetta_init(), "init")
    assert ffi.lib().saetta_static_scratch_bytes() == 4 * (256 * 16 * 256 + 256 * 16 * 2)
    # first call: a large cache (128 splits, the kernel with loader waves), 8-bit
    got, want, _ = decode_both_ways(8, 32896, 32769, 1)
    assert np.isfinite(got).all() and np.array_equal(got, want)
    # second call: a smaller input (8 splits, far fewer partial slots than the buffer now holds), 4-bit
    got, want, (q, qg, keys, values) = decode_both_ways(4, 1024, 777, 2)
    assert np.isfinite(got).all() and np.array_equal(got, want)
    # ... and the result is the oracle's
    n = 777 * 8
    kf = oracle.dequantize(host(keys.data[:n * 8]).view(np.uint32), host(keys.scales[:n]).view(np.uint16),
                           host(keys.biases[:n]).view(np.uint16), 4)
    vf = oracle.dequantize(host(values.data[:n * 8]).view(np.uint32), host(values.scales[:n]).view(np.uint16),
                           host(values.biases[:n]).view(np.uint16), 4)
    want64 = oracle.attention_f64(host(q).reshape(-1), kf, vf, host(qg).reshape(-1), 777, threads=8)
    assert np.abs(got - want64).max() < 2e-5
    # third: the largest number of splits a launch uses (256: 4-bit, above 136k tokens of capacity)
    got, want, _ = decode_both_ways(4, 150016, 150004, 3)
    assert np.isfinite(got).all() and np.array_equal(got, want)


def test_more_heads_than_the_static_scratch_holds_are_rejected():
    z = torch.zeros(16, device="cuda")
    rows = ffi.QuantRowsC(z.data_ptr(), z.data_ptr(), z.data_ptr())
    p = ffi.DecodeParamsC(32, 4, 1024, 1.0 / 16)
    rc = ffi.lib().saetta_attn_decode_quant_static(None, 8, ptr(z), rows, rows, ptr(z), ptr(z), p, ptr(z), ffi.STAGE_ALL)
    assert rc == -6 and b"static scratch" in ffi.lib().saetta_last_error()


def test_static_entry_allocates_nothing_replays_from_a_graph_and_splits_into_stages():
    # What the entry point is for: a call under stream capture (nothing may allocate there), replayed at
    # two positions against eager calls with scratch of the caller's; no device memory taken across the
    # calls; and the partial and the reduce stage as two calls, the partials waiting in the static buffer.
    lib = ffi.lib()
    ffi.check(lib.saetta_init(), "init")
    bits, capacity = 8, 32896
    gen = torch.Generator(device="cuda").manual_seed(11)
    keys, values = saetta.QuantRows(saetta.KvBits.Eight, VALUES, capacity), saetta.QuantRows(saetta.KvBits.Eight, VALUES, capacity)
    keys.encode(torch.randn(capacity * VALUES, generator=gen, device="cuda"), 0, capacity)
    values.encode(torch.randn(capacity * VALUES, generator=gen, device="cuda"), 0, capacity)
    q = torch.randn(H, D, generator=gen, device="cuda")
    qg = torch.randn(H, 2 * D, generator=gen, device="cuda")
    p = ffi.DecodeParamsC(H, KV, capacity, 1.0 / math.sqrt(D))
    part_o = torch.empty(lib.saetta_part_o_bytes(H, capacity, 1) // 4, device="cuda")
    part_ml = torch.empty(lib.saetta_part_ml_bytes(H, capacity, 1) // 4, device="cuda")
    got, want = torch.empty(H, D, device="cuda"), torch.empty(H, D, device="cuda")
    plan = saetta.Plan()
    plan.op("attention_static", lambda st: ffi.check(lib.saetta_attn_decode_quant_static(
        st, bits, ptr(q), keys.c(), values.c(), ptr(qg), ptr(got), p, ptr(plan.params), ffi.STAGE_ALL), "attn_decode_quant_static"))
    built = plan.build(graph=True)  # captured: a hipMalloc here would fail the capture
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (a first replay and a first eager call: what the runtime itself sets up on a first launch is not the call's)
    plan.set_params(saetta.TokenParams(0, 5))
    built.run()
    ffi.check(lib.saetta_attn_decode_quant(stream, bits, ptr(q), keys.c(), values.c(), ptr(part_o), ptr(part_ml), ptr(qg),
                                           ptr(want), p, ptr(plan.params), ffi.STAGE_ALL), "attn_decode_quant")
    host(got), host(want)
    free_before = torch.cuda.mem_get_info()[0]
    for position in (32768, 700, 20000):
        plan.set_params(saetta.TokenParams(0, position))
        got.fill_(float("nan"))
        built.run()
        ffi.check(lib.saetta_attn_decode_quant(stream, bits, ptr(q), keys.c(), values.c(), ptr(part_o), ptr(part_ml), ptr(qg),
                                               ptr(want), p, ptr(plan.params), ffi.STAGE_ALL), "attn_decode_quant")
        g, w = host(got), host(want)
        assert np.isfinite(g).all() and np.array_equal(g, w), position
    # the two stages as two calls (eager, on the stream)
    plan.set_params(saetta.TokenParams(0, 12345))
    got.fill_(float("nan"))
    for stage in (ffi.STAGE_PARTIAL, ffi.STAGE_REDUCE):
        ffi.check(lib.saetta_attn_decode_quant_static(stream, bits, ptr(q), keys.c(), values.c(), ptr(qg), ptr(got), p,
                                                      ptr(plan.params), stage), "attn_decode_quant_static")
    ffi.check(lib.saetta_attn_decode_quant(stream, bits, ptr(q), keys.c(), values.c(), ptr(part_o), ptr(part_ml), ptr(qg),
                                           ptr(want), p, ptr(plan.params), ffi.STAGE_ALL), "attn_decode_quant")
    assert np.array_equal(host(got), host(want))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the calls took device memory"


def test_no_bounded_wait_gave_up_in_this_process():
    # Collected last: the sticky status word of the device is still 0 after every kernel the tests of
    # this process have run (a wave whose bounded wait runs out leaves a code there).
    ffi.check(ffi.lib().saetta_init(), "init")
    torch.cuda.synchronize()
    assert saetta.device_status() == 0
