#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints ONE JSON line.  The default workload is the one the headline metric is
quoted on: decode attention for one query token over a 32768-token, 8-bit
group-quantized KV cache (16 q heads / 2 kv heads, head dim 256).  A "step" is
one decode token's attention over LAYERS independent layer caches back to
back on one stream (split-K partial kernel + reduce kernel per layer), as the
reference's own `bench-attention` does with `layers` distinct caches
(src/attention.rs:173-231): one layer is only 35.65 MB, which would sit in the
256 MB Infinity Cache if it were re-read.

value      = LAYERS * (ctx + 1) * 1088 B / wall time of a step, in GB/s: the
             algorithmic KV bytes (codes + scales + biases of keys and values,
             each read once for all 8 q heads of a kv head).
roofline   = the same bytes per launch of the partial kernel over that kernel's
             average duration, measured with HIP events on the launch stream,
             against 8 TB/s.
cpu_baseline = the CPU oracle (a C restatement of the reference's
             single-threaded f32 CPU attention) on one of the layers.

Other workloads (--workload): decode4_150k (4-bit, 150000 tokens), decode16_4k
(half cache, 4096 tokens: the reference's own CPU-runnable case), verify2..4
(2-4 query rows at 32k, 8-bit), prefill (4096-token chunk at position 4096),
deltanet (the Gated DeltaNet decode step over 30 layer states), deltanet_prefill
(conv + delta rule + gated norm of a 4096-token chunk of one layer), prep_store
(q/k norm + RoPE + KV store of one token, 32 layers), all (the default line with
the others under "other_workloads").
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

H, KV, D = 16, 2, 256
VALUES = KV * D
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0


# HBM bytes per launch of the dominant kernel from hardware counters (FETCH_SIZE and WRITE_SIZE of
# rocprofv3 --pmc, each scaled by what the same counter reads for a 256 MiB copy in the same run;
# the runs are summarised in profiles/*_hbm_traffic.txt).  Counters cannot be read inside this
# script, so the figures are carried here for the workloads they were measured on.
MEASURED_TRAFFIC = {"decode8_32k": 38.2e6, "prefill": 421.5e6, "decode4_150k": 88.9e6, "verify4": 45.0e6,
                    "deltanet_prefill": 664.1e6,  # (the three kernels of the chunk together)
                    "prefill_gemm": 2.18e9}       # (the 2 launches of a call together)


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def make_decode_workload(s, torch, ctx, bits, rows, layers, seed=1234):
    """LAYERS caches of ctx + rows tokens, quantized on the device from N(0,1)."""
    kind = {8: s.KvBits.Eight, 4: s.KvBits.Four, 16: s.KvBits.Half}[bits]
    # room for the query rows' tokens and for the 4 tokens the append timing writes at ctx .. ctx + 3
    capacity = (ctx + max(rows, 4) + 127) // 128 * 128
    gen = torch.Generator(device="cuda").manual_seed(seed)
    caches = []
    chunk = 8192
    for _ in range(layers if bits == 16 else 0):
        # a half cache: [capacity][kv heads][256] f16, the rows past the context left at zero
        k = torch.zeros(capacity, VALUES, dtype=torch.float16, device="cuda")
        v = torch.zeros(capacity, VALUES, dtype=torch.float16, device="cuda")
        k[:ctx + rows] = torch.randn(ctx + rows, VALUES, generator=gen, device="cuda").to(torch.float16)
        v[:ctx + rows] = torch.randn(ctx + rows, VALUES, generator=gen, device="cuda").to(torch.float16)
        caches.append((k, v))
    for _ in range(0 if bits == 16 else layers):
        k, v = s.QuantRows(kind, VALUES, capacity), s.QuantRows(kind, VALUES, capacity)
        for rows_q in (k, v):
            for start in range(0, ctx + rows, chunk):
                n = min(chunk, ctx + rows - start)
                x = torch.randn(n, VALUES, generator=gen, device="cuda")
                if bits == 4:
                    # 1 % of the channels scaled x8, as outlier channels (same channels everywhere).
                    x[:, [7, 101, 230, 333, 460]] *= 8.0
                rows_q.encode(x.reshape(-1), start, n)
        caches.append((k, v))
    q = torch.randn(rows, H, D, generator=gen, device="cuda")
    qg = torch.randn(rows, H, 2 * D, generator=gen, device="cuda")
    out = torch.empty(rows, H, D, device="cuda")
    return kind, capacity, caches, q, qg, out


def bench_decode(s, torch, args, ctx, bits, rows, layers, compact=False, workload=None):
    """compact: a short record for the default line's "other_workloads": no CPU timing loops (one oracle
    run on all cores for the parity figure), no reader floor.  workload: caches made before (with room for
    `rows` rows), for the records that share them."""
    import oracle  # only for the CPU-baseline leg below

    kind, capacity, caches, q, qg, out = workload or make_decode_workload(s, torch, ctx, bits, rows, layers)
    q, qg, out = q[:rows], qg[:rows], out[:rows]
    plan = s.Plan()
    half = bits == 16
    if rows == 1:
        att = s.DecodeAttention(H, KV, D, capacity)
        for k, v in caches:
            (att.record if half else att.record_quant)(plan, q[0], k, v, qg[0], out[0])
        plan.set_params(s.TokenParams(0, ctx))  # position ctx: sees ctx + 1 tokens
    else:
        att = s.AttentionRows(H, KV, capacity, rows)
        tp = s.TokenParams(0, ctx).as_tensor("cuda")
        for k, v in caches:
            (att.record if half else att.record_quant)(plan, rows, q, k, v, qg, out, [tp] * rows)
    graph = not args.no_graph
    built = plan.build(graph)
    partial_only = plan.build_where(lambda name: "partial" in name, graph)
    reduce_only = plan.build_where(lambda name: "reduce" in name, graph)
    bytes_per_token = {8: 1088, 4: 576, 16: 2048}[bits]
    layer_bytes = (ctx + rows) * bytes_per_token

    for _ in range(args.warmup):
        built.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        built.run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = layers * layer_bytes / (ms_per_step * 1e-3) / 1e9

    # Kernel durations with HIP events on the launch stream (torch's current stream is the
    # one every launch above went to): all partial launches of a step between two events.
    def kernel_us(b):
        ts = []
        for _ in range(max(5, args.steps)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            b.run()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / layers)
        return median(ts), min(ts)

    part_us, part_us_min = kernel_us(partial_only)
    red_us, _ = kernel_us(reduce_only)
    achieved = layer_bytes / (part_us * 1e-6) / 1e9

    # CPU baseline: the oracle's f32 attention on layer 0 (what the reference's CPU path does,
    # src/cpu/attention.rs:141-181), single thread and all threads the box gives us.
    import numpy as np
    k0, v0 = caches[0]
    n_tok = ctx + 1
    groups = n_tok * 8

    def deq(rows_q):
        return oracle.dequantize(rows_q.data[:groups * 2 * bits].cpu().numpy().view(np.uint32),
                                 rows_q.scales[:groups].cpu().numpy().view(np.uint16),
                                 rows_q.biases[:groups].cpu().numpy().view(np.uint16), bits)

    if half:
        kf, vf = k0[:n_tok].float().cpu().numpy().reshape(-1), v0[:n_tok].float().cpu().numpy().reshape(-1)
    else:
        kf, vf = deq(k0), deq(v0)
    qh, qgh = q[0].cpu().numpy(), qg[0].cpu().numpy()
    threads_all = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)

    def cpu_time(threads, budget_s):
        ts, spent = [], 0.0
        while spent < budget_s or len(ts) < 2:
            c0 = time.perf_counter()
            ref = oracle.attend(qh, kf, vf, n_tok, q_and_gate=qgh, threads=threads)
            ts.append(time.perf_counter() - c0)
            spent += ts[-1]
        return median(ts), ref

    if compact:
        cpu1 = cpun = None
        ref = oracle.attend(qh, kf, vf, n_tok, q_and_gate=qgh, threads=threads_all)
    else:
        cpu1, ref = cpu_time(1, 8.0)
        cpun, _ = cpu_time(threads_all, 4.0)
    # The GPU's answer for the same layer, checked against the oracle while we are here.
    check = s.Plan()
    if rows == 1:
        (att.record if half else att.record_quant)(check, q[0], k0, v0, qg[0], out[0])
        check.set_params(s.TokenParams(0, ctx))
    else:
        (att.record if half else att.record_quant)(check, rows, q, k0, v0, qg, out,
                                                    [s.TokenParams(0, ctx).as_tensor("cuda")] * rows)
    check.build().run()
    torch.cuda.synchronize()
    rel_rms = oracle.rel_rms(out[0].cpu().numpy(), ref)

    # Quantize-on-append of 4 new tokens into every layer's K and V caches (two launches per
    # layer, rows ctx .. ctx + 3; last, because it writes over the rows the check above read).
    import ctypes
    new_tokens = 4
    assert ctx + new_tokens <= capacity, "the appended rows must lie inside the caches"
    x_new = torch.randn(new_tokens, VALUES, device="cuda")
    append = s.Plan()
    for k, v in ([] if half else caches):
        for rows_q in (k, v):
            p = s.ffi.KvQuantParamsC(rows_q.per_token * new_tokens, rows_q.per_token)
            append.op(f"kv_quantize_{bits}", lambda st, c=rows_q.c(), p=p: s.ffi.check(
                s.ffi.lib().saetta_kv_quantize(st, bits, ctypes.c_void_p(x_new.data_ptr()), c, p, None, ctx), "kv_quantize"))
    append_us = kernel_us(append.build(graph))[0] if not half else 0.0

    name = f"decode attention, {bits}-bit KV, ctx {ctx}, {rows} query row(s), {layers} layer caches per step"
    if compact:
        return {"metric": f"decode attn HBM GB/s @{ctx // 1024}k ctx {bits}-bit KV, {rows} row(s)", "value": round(value, 1),
                "unit": "GB/s", "ms_per_step": round(ms_per_step, 4), "config": {"workload": name},
                "append_4_tokens_k_and_v_us_per_layer": None if half else round(append_us, 3),
                "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(achieved / HBM_PEAK_GBS, 4), "kernel": "attention_partial_kernel",
                             "avg_us": round(part_us, 3), "reduce_kernel_us": round(red_us, 3)},
                "parity_rel_rms_vs_oracle": float(f"{rel_rms:.3e}")}
    # The floor of a launch of this size: a plain read of the same bytes by 256 workgroups.
    reader, empty_us = reader_floor(s, torch, args, layer_bytes, layers) if not args.no_reader_floor else ({}, None)
    reader_us = min(reader.values()) if reader else None
    res = {
        "metric": f"decode attn HBM GB/s @{ctx // 1024}k ctx {bits}-bit KV",
        "value": round(value, 1),
        "unit": "GB/s",
        "ms_per_step": round(ms_per_step, 4),
        "dtype": "f16 cache, f16 MFMA, f32 accumulate" if half else "u8 codes, f16 MFMA, f32 accumulate",
        "config": {"workload": name, "heads": H, "kv_heads": KV, "head_dim": D, "ctx": ctx, "kv_bits": bits,
                   "rows": rows, "layers_per_step": layers, "bytes_per_layer": layer_bytes,
                   "append_4_tokens_k_and_v_us_per_layer": None if half else round(append_us, 3),
                   "inputs": "K, V, q, gate ~ N(0,1) from torch's device generator (Philox, seed 1234), not the "
                             "reference tests' LCG + Box-Muller stream; caches quantized on the device by the "
                             "library's quantizer" + ("; channels 7, 101, 230, 333, 460 of the 512 scaled x8 as "
                                                      "outlier channels" if bits == 4 else "")},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get({(32768, 8, 1): "decode8_32k", (150000, 4, 1): "decode4_150k",
                                                      (32768, 8, 4): "verify4"}.get((ctx, bits, rows))),
                     "kernel": "attention_partial_kernel", "avg_us": round(part_us, 3),
                     "min_us": round(part_us_min, 3), "reduce_kernel_us": round(red_us, 3),
                     "reader_us": reader_us, "reader_variants_us": reader, "empty_launch_us": empty_us,
                     "frac_of_reader": round(reader_us / part_us, 4) if reader_us else None},
        "cpu_baseline": {"value": round(layer_bytes / cpu1 / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                         "sample": f"one of the {layers} layer caches, full shape, median of repeats; "
                                   f"{cpu1 * 1e3:.1f} ms per layer",
                         "all_cores": {"value": round(layer_bytes / cpun / 1e9, 4), "cores": threads_all,
                                       "ms": round(cpun * 1e3, 2)}},
        "parity_rel_rms_vs_oracle": float(f"{rel_rms:.3e}"),
    }
    return res


_calib = None


def calib_lib(s):
    """The calibration kernels (a plain streaming read; the prefill kernel's MFMA streams alone): a library of
    their own beside the product's."""
    global _calib
    if _calib is None:
        import ctypes
        path = os.path.join(os.path.dirname(s.ffi.LIB_PATH), "libsaetta_calib.so")
        _calib = ctypes.CDLL(path)
        _calib.saetta_calib_read.restype = ctypes.c_int
        _calib.saetta_calib_read.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32,
                                             ctypes.c_uint32, ctypes.c_void_p]
        _calib.saetta_calib_mfma.restype = ctypes.c_int
        _calib.saetta_calib_mfma.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                             ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
    return _calib


def reader_floor(s, torch, args, nbytes, layers, workgroups=256):
    """How long one launch of `workgroups` workgroups takes to READ nbytes from HBM and do nothing
    else: `layers` buffers of their own (as the layer caches are), one launch each, replayed from a
    HIP graph and timed with events like the attention kernels.  Returns {variant: us per launch}
    and the time of an empty launch in the same setting (a read of 16 bytes per workgroup)."""
    import ctypes
    lib = calib_lib(s)
    nbytes = nbytes // 16 * 16
    bufs = [torch.full((nbytes // 4,), -1, dtype=torch.int32, device="cuda") for _ in range(layers)]
    sink = torch.zeros(1024, dtype=torch.int32, device="cuda")
    names = {0: "256 threads x 8 loads", 1: "512 x 4", 2: "1024 x 4", 3: "1024 x 2",
             4: "to LDS, 4 waves", 5: "to LDS, 8 waves", 6: "to LDS, 12 waves", 7: "to LDS, 16 waves"}

    def timed(variant, size):
        plan = s.Plan()
        for b in bufs:
            plan.op("calib_read", lambda st, b=b: s.ffi.check(lib.saetta_calib_read(
                st, ctypes.c_void_p(b.data_ptr()), size, workgroups, variant, ctypes.c_void_p(sink.data_ptr())), "calib_read"))
        built = plan.build(graph=not args.no_graph)
        for _ in range(args.warmup):
            built.run()
        ts = []
        for _ in range(max(5, args.steps)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            built.run()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / layers)
        return median(ts)

    # (the readers into LDS hold a workgroup's whole share there: 160 KB at most)
    fits_lds = -(-(nbytes // 1024) // workgroups) * 1024 <= 160 * 1024
    out = {names[v]: round(timed(v, nbytes), 3) for v in names if v < 4 or fits_lds}
    empty = round(timed(0, 16 * workgroups), 3)
    assert int(sink.sum().item()) == 0
    return out, empty


def mfma_floor(s, torch, args, steps=192, workgroups=256, nbytes=16 * 1024 * 1024 + 768 * 1024):
    """What rate of f16 MFMAs ONE launch shaped like the prefill attention kernel (a workgroup of 8 waves per CU,
    `steps` x 32 MFMAs per wave: 192 steps are the two tiles a workgroup takes at 4096 tokens behind 4096) sustains
    with nothing else to do, and at what shader clock: on operands that never change, on operands that change with
    every MFMA, and as the prefill kernel's own instruction streams (fragment reads from LDS, global -> LDS copies
    out of a buffer of the key and value images' size, a barrier per step) without the softmax.  The operands are
    N(0, 1) values in f16, like the keys and queries of the prefill workload.  Launches back to back, timed with
    events like the prefill kernel.  Returns {variant: {"TFLOP/s", "GHz", "us"}}."""
    import ctypes
    lib = calib_lib(s)
    gen = torch.Generator(device="cuda").manual_seed(7)
    operands = torch.randn(nbytes // 2, generator=gen, device="cuda").to(torch.float16)
    out = torch.zeros(2 * workgroups, dtype=torch.int64, device="cuda")
    sink = torch.zeros(workgroups, dtype=torch.float32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    names = {0: "operands that never change", 1: "operands that change with every MFMA",
             2: "the prefill kernel's streams (LDS fragment reads, copies, barrier), no softmax"}
    flops = workgroups * 8 * steps * 32 * 32768.0
    res = {}
    for v, name in names.items():
        def run():
            s.ffi.check(lib.saetta_calib_mfma(stream, v, steps, workgroups, ctypes.c_void_p(operands.data_ptr()), nbytes,
                                              ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(sink.data_ptr())), "calib_mfma")
        for _ in range(max(3, args.warmup)):
            run()
        ts, ghz = [], []
        for _ in range(max(5, args.steps)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            run()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
            c = out.view(workgroups, 2).double()
            ghz.append(float((c[:, 0] / (c[:, 1] * 10.0)).mean().item()))
        us = median(ts)
        res[name] = {"TFLOP/s": round(flops / (us * 1e-6) / 1e12, 1), "GHz": round(median(ghz), 3), "us": round(us, 1)}
    return res


def bench_mfma_floor(s, torch, args):
    variants = mfma_floor(s, torch, args)
    best = variants["the prefill kernel's streams (LDS fragment reads, copies, barrier), no softmax"]
    return {
        "metric": "f16 MFMA rate of the prefill kernel's streams alone, TFLOP/s",
        "value": best["TFLOP/s"], "unit": "TFLOP/s", "ms_per_step": round(best["us"] / 1e3, 4),
        "dtype": "f16 MFMA",
        "config": {"workload": "calibration: one launch of 256 workgroups of 8 waves, 192 steps of 32 "
                               "v_mfma_f32_32x32x16_f16 per wave, N(0,1) operands", "variants": variants},
        "roofline": {"bound": "mfma", "achieved": best["TFLOP/s"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(best["TFLOP/s"] / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "calib_mfma_stream_kernel", "avg_us": best["us"]},
        "cpu_baseline": None,
    }


def bench_reader_floor(s, torch, args, ctx=32768, layers=32):
    nbytes = (ctx + 1) * 1088
    variants, empty = reader_floor(s, torch, args, nbytes, layers)
    best = min(variants.values())
    return {
        "metric": "plain streaming read of one layer's KV bytes, GB/s",
        "value": round(nbytes / best / 1e3, 1), "unit": "GB/s", "ms_per_step": round(best * layers / 1e3, 4),
        "dtype": "u32x4 loads",
        "config": {"workload": f"calibration: one launch of 256 workgroups reads {nbytes} bytes and computes nothing, "
                               f"{layers} buffers per step", "us_per_launch": variants, "empty_launch_us": empty},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / best / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(nbytes / best / 1e3 / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "calib_read_kernel",
                     "avg_us": best},
        "cpu_baseline": None,
    }


def bench_prefill(s, torch, args, tokens=4096, pos=4096, bits=8, gemm=False):
    """gemm: the same chunk by AttGemm (src/attention_gemm.rs), block by block of 1024 keys with the block's
    probabilities written out and read back, instead of the flash kernel."""
    import numpy as np
    import oracle  # CPU-baseline leg only

    kind = {8: s.KvBits.Eight, 4: s.KvBits.Four}[bits]
    capacity = (pos + tokens + 127) // 128 * 128
    gen = torch.Generator(device="cuda").manual_seed(99)
    keys, values = s.QuantRows(kind, VALUES, capacity), s.QuantRows(kind, VALUES, capacity)
    knew = torch.randn(pos + tokens, VALUES, generator=gen, device="cuda")
    vnew = torch.randn(pos + tokens, VALUES, generator=gen, device="cuda")
    keys.encode(knew[:pos].reshape(-1), 0, pos)
    values.encode(vnew[:pos].reshape(-1), 0, pos)
    q = torch.randn(tokens, H, D, generator=gen, device="cuda").to(torch.bfloat16).to(torch.float16)
    qg = torch.randn(tokens, H, 2 * D, generator=gen, device="cuda")
    out = torch.empty(tokens, H, D, device="cuda")
    p = s.FlashParams(H, KV, pos, tokens, 1.0 / math.sqrt(D))
    kx, vx = knew[pos:].reshape(-1).contiguous(), vnew[pos:].reshape(-1).contiguous()
    att_gemm = s.attention_gemm.AttGemm(tokens, KV) if gemm else None
    # the key and value tile images of the flash kernel: allocated once, outside every timed region
    ws = None if gemm else torch.empty(s.attention_prefill.workspace_bytes(p), dtype=torch.uint8, device="cuda")

    def attention():
        if gemm:
            att_gemm.encode(q, None, None, (keys, values), qg, out, p)
        else:
            s.attention_prefill.encode_quant(q, keys, values, qg, out, p, workspace=ws)

    def step():
        # quantize-on-append of the chunk's K and V, then the attention over codes in place
        keys.encode(kx, pos, tokens)
        values.encode(vx, pos, tokens)
        attention()

    flops = 4.0 * H * D * (tokens * pos + tokens * (tokens + 1) / 2)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    ts = []
    for _ in range(max(3, args.steps)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        attention()
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e3)
    kern_us = median(ts)
    achieved = flops / (kern_us * 1e-6) / 1e12
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_F16_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4),
                "traffic": MEASURED_TRAFFIC.get("prefill") if (tokens, pos, bits, gemm) == (4096, 4096, 8, False) else None,
                "kernel": "attention_prefill_kernel", "avg_us": round(kern_us, 2)}
    if not gemm and not args.no_reader_floor:
        # what the kernel's own MFMA streams reach with no softmax, prologue or epilogue around them
        floor = mfma_floor(s, torch, args)
        stream_only = floor["the prefill kernel's streams (LDS fragment reads, copies, barrier), no softmax"]["TFLOP/s"]
        roofline["mfma_streams_alone"] = floor
        roofline["frac_of_streams_alone"] = round(achieved / stream_only, 4)
    if gemm:
        # What bounds this route is the scratch it writes and reads back.  Algorithmic bytes per query row: 2 B out
        # and 2 B in per key its 16-token tile sees (in whole tiles of 32 keys), and a maximum and a sum (8 B)
        # out and in per tile of 32 keys; per span of eight blocks of 1024 keys it touches, its q twice (one read
        # per part of the span's tiles: two at this chunk length) and 1 KB of output sums in and 1 KB out.
        nbytes = 0
        for t0 in range(0, tokens, 16):
            last_key = pos + min(t0 + 16, tokens) - 1
            rows = (min(t0 + 16, tokens) - t0) * H
            nbytes += rows * ((last_key // 32 + 1) * (32 * 4 + 16) + (last_key // 8192 + 1) * 3072)
        gbs = nbytes / (kern_us * 1e-6) / 1e9
        roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(gbs / HBM_PEAK_GBS, 4),
                    "traffic": MEASURED_TRAFFIC.get("prefill_gemm") if (tokens, pos, bits) == (4096, 4096, 8) else None,
                    "kernel": "attention_gemm_scores_kernel + attention_gemm_pv_kernel", "avg_us": round(kern_us, 2),
                    "bytes": nbytes, "mfma_TFLOPs": round(achieved, 2), "mfma_frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4)}
    # CPU baseline on a bounded sample: the last `sample` tokens of the chunk (the longest rows).
    sample = max(16, 512 * 8192 // (pos + tokens))  # 512 tokens at the headline shape: about 7 s on one core
    groups = (pos + tokens) * 8

    def deq(rows_q):
        x = oracle.dequantize(rows_q.data[:groups * 2 * bits].cpu().numpy().view(np.uint32),
                              rows_q.scales[:groups].cpu().numpy().view(np.uint16),
                              rows_q.biases[:groups].cpu().numpy().view(np.uint16), bits)
        return x.astype(np.float16).astype(np.float32)  # read through half, as prefill does

    kf, vf = deq(keys), deq(values)
    qs = q[tokens - sample:].float().cpu().numpy()
    qgs = qg[tokens - sample:].cpu().numpy()
    c0 = time.perf_counter()
    ref = oracle.prefill(qs, kf, vf, pos + tokens - sample, sample, q_and_gate=qgs, threads=1)
    cpu_s = time.perf_counter() - c0
    cpu_flops = 4.0 * H * D * sum(pos + tokens - sample + i + 1 for i in range(sample))
    rel_rms = oracle.rel_rms(out[tokens - sample:].cpu().numpy(), ref)
    return {
        "metric": "prefill-chunk attn TFLOP/s",
        "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "ms_per_step": round(ms_per_step, 4),
        "dtype": "f16 MFMA, f32 softmax state",
        "config": {"workload": f"causal prefill chunk of {tokens} tokens at position {pos}, {bits}-bit KV cache "
                               "read in place, chunk K/V quantized on append inside the step"
                               + (", attention as matrix products over blocks of 1024 keys (AttGemm)" if gemm else ""),
                   "heads": H, "kv_heads": KV, "head_dim": D, "flops": flops,
                   "timing": "value: wall time of steps (2 x kv_quantize of the chunk + prepare + attention); "
                             "roofline: median of event-timed prepare + attention calls"
                             + (f" ({2 * -(-(pos + tokens) // 8192)} launches: scores and pv per span of eight blocks of 1024 keys)" if gemm else ""),
                   "inputs": "q (through bf16), K, V, gate ~ N(0,1) from torch's device generator (Philox, seed 99)"},
        "roofline": roofline,
        "cpu_baseline": {"value": round(cpu_flops / cpu_s / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                         "sample": f"the last {sample} tokens of the chunk ({cpu_s:.2f} s)"},
        "parity_rel_rms_vs_oracle": float(f"{rel_rms:.3e}"),
    }


def bench_deltanet(s, torch, args, layers=30):
    """Gated DeltaNet decode step (conv + step) over `layers` layer states of their own, the model's
    shape: 16 key / 32 value heads of 128, conv kernel 4.  Algorithmic bytes per layer: the
    recurrent state read and written, 2 x 32 x 128 x 128 x 4 B."""
    import numpy as np
    import oracle  # parity check and CPU-baseline leg only

    kh, vh, dv, kernel, eps = 16, 32, 128, 4, 1e-6
    key, val = kh * 128, vh * dv
    ch = 2 * key + val
    gen = torch.Generator(device="cuda").manual_seed(7)

    def r(n, scale=1.0):
        return torch.randn(n, generator=gen, device="cuda") * scale

    x, z, a, b, alog, dtb, w = r(ch), r(val), r(vh), r(vh), r(vh), r(vh), r(ch * kernel, 0.5)
    norm = 1 + r(dv, 0.1)
    states = [(torch.zeros((kernel - 1) * ch, device="cuda"), r(vh * dv * 128, 0.1)) for _ in range(layers)]
    first_state = states[0][1].clone()
    mixed, y = torch.empty(ch, device="cuda"), torch.empty(val, device="cuda")

    def plan_of(which):
        plan = s.Plan()
        for conv, st in states:
            if which == "token":
                s.deltanet_token(plan, x, w, conv, a, b, alog, dtb, st, z, norm, y, kh, vh, dv, kernel, eps)
                continue
            if which != "step":
                s.deltanet_conv(plan, x, w, conv, mixed, ch, kernel)
            if which != "conv":
                s.deltanet_step(plan, mixed[:key], mixed[key:2 * key], mixed[2 * key:], a, b, alog, dtb, st, z, norm, y,
                                kh, vh, dv, eps)
        return plan.build(graph=not args.no_graph)

    # parity of one step against the oracle, before the states are run over many times
    one = s.Plan()
    s.deltanet_token(one, x, w, states[0][0], a, b, alog, dtb, states[0][1], z, norm, y, kh, vh, dv, kernel, eps)
    one.build().run()
    torch.cuda.synchronize()
    conv_cpu = np.zeros((kernel - 1, ch), np.float32)
    st_cpu = first_state.cpu().numpy().copy()
    c0 = time.perf_counter()
    m_cpu = oracle.deltanet_conv(w.cpu().numpy().reshape(ch, kernel), x.cpu().numpy(), conv_cpu, kernel)
    y_cpu = oracle.deltanet_step(m_cpu[:key], m_cpu[key:2 * key], m_cpu[2 * key:], a.cpu().numpy(), b.cpu().numpy(),
                                 alog.cpu().numpy(), dtb.cpu().numpy(), st_cpu, z.cpu().numpy(), norm.cpu().numpy(),
                                 kh, vh, 128, dv, eps)
    cpu_s = time.perf_counter() - c0
    rel = float(np.sqrt(((y.cpu().numpy() - y_cpu) ** 2).mean() / (y_cpu ** 2).mean()))

    def timed(built):
        for _ in range(args.warmup):
            built.run()
        ts = []
        for _ in range(max(5, args.steps)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            built.run()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / layers)
        return median(ts)

    both_us, step_us, token_us = timed(plan_of("both")), timed(plan_of("step")), timed(plan_of("token"))

    # The verify step of the same layers: 4 rows with the conv and delta states after every row
    # (what an MTP verify asks for), as one call of two launches and as the pair of calls for chunks.
    m = 4
    xm, zm, am, bm = r(m * ch), r(m * val), r(m * vh), r(m * vh)
    mixed_m, ym = torch.empty(m * ch, device="cuda"), torch.empty(m * val, device="cuda")
    csn, ssn = torch.empty(m * (kernel - 1) * ch, device="cuda"), torch.empty(m * vh * dv * 128, device="cuda")
    fused, pair = s.Plan(), s.Plan()
    for conv, st in states:
        s.deltanet_rows_fused(fused, xm, w, conv, am, bm, alog, dtb, st, zm, norm, ym, kh, vh, dv, kernel, m, eps, csn, ssn)
        s.deltanet_conv_rows(pair, xm, w, conv, mixed_m, ch, kernel, m, csn)
        s.deltanet_rows(pair, mixed_m, am, bm, alog, dtb, st, zm, norm, ym, kh, vh, dv, m, eps, ssn)
    verify_us = timed(fused.build(graph=not args.no_graph))
    verify_pair_us = timed(pair.build(graph=not args.no_graph))
    nbytes = 2.0 * vh * dv * 128 * 4
    achieved = nbytes / token_us / 1e3
    return {
        "metric": "Gated DeltaNet decode step, state GB/s",
        "value": round(nbytes / token_us / 1e3, 1),
        "unit": "GB/s",
        "ms_per_step": round(token_us * layers / 1e3, 4),
        "dtype": "f32",
        "config": {"workload": f"Gated DeltaNet, one token, conv + step (deltanet_token), {layers} layer states per step",
                   "k_heads": kh, "v_heads": vh, "k_dim": 128, "v_dim": dv, "conv_kernel": kernel, "bytes_per_layer": nbytes,
                   "conv_then_step_us": round(both_us, 3), "verify_4_rows_with_snapshots_us": round(verify_us, 3),
                   "verify_4_rows_as_conv_rows_then_rows_us": round(verify_pair_us, 3), "step_kernel_alone_us": round(step_us, 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "deltanet_rows_small_kernel + deltanet_rows_small_tail_kernel", "avg_us": round(token_us, 3)},
        "cpu_baseline": {"value": round(nbytes / cpu_s / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                         "sample": f"one layer, conv + step ({cpu_s * 1e3:.2f} ms)"},
        "parity_rel_rms_vs_oracle": float(f"{rel:.3e}"),
    }


def bench_prep_store(s, torch, args, layers=32, capacity=32896):
    """The step before the scores, once per layer: q/k norm + RoPE + the token's key and value into
    8-bit caches in one launch (attention_prep_store), beside the two kv_quantize launches the
    reference records after its own prep kernel.  Latency-bound: 21 KB in, 1.1 KB + 16 KB out."""
    import numpy as np
    import oracle  # parity check only

    gen = torch.Generator(device="cuda").manual_seed(5)
    qg = torch.randn(H * 2 * D, generator=gen, device="cuda")
    k, v = torch.randn(KV * D, generator=gen, device="cuda"), torch.randn(KV * D, generator=gen, device="cuda")
    qn, kn = 1 + 0.1 * torch.randn(D, generator=gen, device="cuda"), 1 + 0.1 * torch.randn(D, generator=gen, device="cuda")
    q, kb = torch.empty(H * D, device="cuda"), torch.empty(KV * D, device="cuda")
    caches = [(s.QuantRows(s.KvBits.Eight, VALUES, capacity), s.QuantRows(s.KvBits.Eight, VALUES, capacity))
              for _ in range(layers)]
    p = s.PrepParams(H, KV, D, 64, 1e7, 1e-6)
    pos = 32768

    def timed(plan):
        plan.set_params(s.TokenParams(0, pos))
        built = plan.build(graph=not args.no_graph)
        for _ in range(args.warmup):
            built.run()
        ts = []
        for _ in range(max(5, args.steps)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            built.run()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / layers)
        return median(ts)

    two = s.Plan()
    for kc, vc in caches:
        kc.record(two, k), vc.record(two, v)
    two_us = timed(two)
    fused = s.Plan()  # last: what it stores is checked below
    for i, (kc, vc) in enumerate(caches):
        s.record_store(fused, qg, k, v, qn, kn, q, kc, vc, p, capacity, k_back=kb if i == 0 else None)
    fused_us = timed(fused)
    # parity: q against the oracle's norm + rope, the stored codes against the oracle's quantizer
    want_q, _, _ = oracle.attention_prep(qg.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), qn.cpu().numpy(),
                                         kn.cpu().numpy(), H, KV, D, 64, pos, 1e7, 1e-6)
    torch.cuda.synchronize()
    rel = float(np.sqrt(((q.cpu().numpy() - want_q.reshape(-1)) ** 2).mean() / (want_q ** 2).mean()))
    data, scales, biases = oracle.quantize(kb.cpu().numpy().reshape(1, VALUES), 8)
    kc = caches[0][0]
    w0 = pos * 8 * 16
    codes_equal = bool((kc.data[w0:w0 + 8 * 16].cpu().numpy().view(np.uint32) == data.reshape(-1)).all())
    nbytes = 4.0 * (H * 2 * D + 2 * KV * D + 2 * D) + 4.0 * H * D + 2 * 8 * (64 + 4)
    return {
        "metric": "q/k norm + RoPE + KV store, launches per second of one layer",
        "value": round(1e6 / fused_us, 1),
        "unit": "layer-tokens/s",
        "ms_per_step": round(fused_us * layers / 1e3, 4),
        "dtype": "f32 in, u8 codes + f16 scales out",
        "config": {"workload": f"attention_prep_store, 8-bit caches, position {pos}, {layers} layers per step",
                   "bytes_per_layer": nbytes, "two_kv_quantize_launches_us": round(two_us, 3)},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / fused_us / 1e3, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(nbytes / fused_us / 1e3 / HBM_PEAK_GBS, 6), "traffic": None,
                     "kernel": "attention_prep_store_kernel", "avg_us": round(fused_us, 3)},
        "cpu_baseline": None,
        "parity_rel_rms_vs_oracle": float(f"{rel:.3e}"),
        "codes_equal_oracle": codes_equal,
    }


def bench_deltanet_prefill(s, torch, args, tokens=4096):
    """A prefill chunk of one Gated DeltaNet layer: deltanet_conv_rows + deltanet_rows over `tokens`
    tokens in order, the model's shape.  Algorithmic bytes of the rows launch: `mixed` and a, b read,
    o written, the gated norm's read of o and z and write of y, the state read and written.  The
    delta rule runs in blocks of 64 tokens on the matrix cores (deltanet_chunk.hip); its rate is
    also given in the token chain's own count (7 f32 flops per state value and token)."""
    import numpy as np
    import oracle  # parity check and CPU-baseline leg only

    kh, vh, dv, kernel, eps = 16, 32, 128, 4, 1e-6
    key, val = kh * 128, vh * dv
    ch = 2 * key + val
    gen = torch.Generator(device="cuda").manual_seed(9)

    def r(*n, scale=1.0):
        return torch.randn(*n, generator=gen, device="cuda") * scale

    x, z, a, b = r(tokens, ch), r(tokens, val), r(tokens, vh), r(tokens, vh)
    alog, dtb, w, norm = r(vh), r(vh), r(ch * kernel, scale=0.5), 1 + r(dv, scale=0.1)
    conv, st = torch.zeros((kernel - 1) * ch, device="cuda"), torch.zeros(vh * dv * 128, device="cuda")
    mixed, y = torch.empty(tokens, ch, device="cuda"), torch.empty(tokens, val, device="cuda")

    def plan_of(which, n=tokens):
        plan = s.Plan()
        if which != "rows":
            s.deltanet_conv_rows(plan, x, w, conv, mixed, ch, kernel, n)
        if which != "conv":
            s.deltanet_rows(plan, mixed, a, b, alog, dtb, st, z, norm, y, kh, vh, dv, n, eps)
        return plan.build(graph=not args.no_graph)

    # parity of the first tokens against the oracle (token by token), from zero states; 160 tokens:
    # a call of 128 tokens and more takes the blocks
    n_check = 160
    plan_of("both", n_check).run()
    torch.cuda.synchronize()
    conv_cpu, st_cpu = np.zeros((kernel - 1, ch), np.float32), np.zeros(vh * dv * 128, np.float32)
    xs, zs, as_, bs = (t[:n_check].cpu().numpy() for t in (x, z, a, b))
    wn, an, dn, nn = w.cpu().numpy().reshape(ch, kernel), alog.cpu().numpy(), dtb.cpu().numpy(), norm.cpu().numpy()
    c0 = time.perf_counter()
    want = []
    for t in range(n_check):
        m = oracle.deltanet_conv(wn, xs[t], conv_cpu, kernel)
        want.append(oracle.deltanet_step(m[:key], m[key:2 * key], m[2 * key:], as_[t], bs[t], an, dn, st_cpu, zs[t], nn,
                                         kh, vh, 128, dv, eps))
    cpu_s = (time.perf_counter() - c0) / n_check
    want = np.stack(want)
    rel = float(np.sqrt(((y[:n_check].cpu().numpy() - want) ** 2).mean() / (want ** 2).mean()))
    conv.zero_(), st.zero_()

    def timed(built):
        for _ in range(min(args.warmup, 2)):
            built.run()
        ts = []
        for _ in range(max(5, min(args.steps, 10))):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            built.run()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        return median(ts)

    both_us, rows_us = timed(plan_of("both")), timed(plan_of("rows"))
    rows_bytes = 4.0 * (tokens * ch + 2 * tokens * vh + 4 * tokens * val + 2 * vh * dv * 128)
    conv_bytes = 4.0 * 2 * tokens * ch
    flops = 7.0 * tokens * vh * dv * 128
    achieved = rows_bytes / rows_us / 1e3
    return {
        "metric": "Gated DeltaNet prefill chunk, tokens/s of one layer",
        "value": round(tokens / both_us * 1e6, 1),
        "unit": "tokens/s",
        "ms_per_step": round(both_us / 1e3, 4),
        "dtype": "f32",
        "config": {"workload": f"Gated DeltaNet, {tokens}-token chunk of one layer, conv + delta rule + gated norm",
                   "k_heads": kh, "v_heads": vh, "k_dim": 128, "v_dim": dv, "conv_kernel": kernel,
                   "bytes_rows_launch": rows_bytes, "bytes_conv_launch": conv_bytes},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get("deltanet_prefill") if (tokens, kh, vh, dv) == (4096, 16, 32, 128) else None,
                     "kernel": "deltanet_chunk_prepare_kernel + deltanet_chunk_chain_kernel + deltanet_gated_norm_wide_kernel",
                     "avg_us": round(rows_us, 1), "token_chain_TFLOPs": round(flops / rows_us / 1e6, 2)},
        "cpu_baseline": {"value": round(1.0 / cpu_s, 1), "unit": "tokens/s", "cores": 1, "kind": "port",
                         "sample": f"the first {n_check} tokens, conv + step each ({cpu_s * 1e3:.2f} ms per token)"},
        "parity_rel_rms_vs_oracle": float(f"{rel:.3e}"),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="default",
                    choices=["decode8_32k", "decode4_150k", "decode16_4k", "verify2", "verify3", "verify4", "prefill", "prefill_131k", "prefill_gemm", "prefill_gemm_131k", "deltanet",
                             "deltanet_prefill", "prep_store", "reader_floor", "mfma_floor", "default", "all"])
    ap.add_argument("--no-graph", action="store_true", help="launch from Python instead of replaying a HIP graph")
    ap.add_argument("--layers", type=int, default=0, help="layer caches per step (default 32; 12 at 150k)")
    ap.add_argument("--ctx", type=int, default=0, help="context length of the decode and verify workloads (default: the workload's own)")
    ap.add_argument("--no-reader-floor", action="store_true", help="skip the plain-read calibration of the decode workloads")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run a plain device copy of 256 MiB (three times): a kernel of known traffic for a "
                         "hardware-counter run of the same command to be scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    import __graft_entry__ as entry
    s = entry.load_package()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback)", file=sys.stderr)
        sys.exit(1)
    s.ffi.check(s.ffi.lib().saetta_init(), "init")
    if args.calibrate_copy:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    def one(workload):
        if workload == "decode8_32k":
            return bench_decode(s, torch, args, args.ctx or 32768, 8, 1, args.layers or 32)
        if workload == "decode4_150k":
            return bench_decode(s, torch, args, args.ctx or 150000, 4, 1, args.layers or 12)
        if workload == "decode16_4k":
            return bench_decode(s, torch, args, 4096, 16, 1, args.layers or 32)
        if workload.startswith("verify"):
            return bench_decode(s, torch, args, args.ctx or 32768, 8, int(workload[-1]), args.layers or 32)
        if workload == "deltanet":
            return bench_deltanet(s, torch, args)
        if workload == "deltanet_prefill":
            return bench_deltanet_prefill(s, torch, args)
        if workload == "prep_store":
            return bench_prep_store(s, torch, args)
        if workload == "reader_floor":
            return bench_reader_floor(s, torch, args)
        if workload == "mfma_floor":
            return bench_mfma_floor(s, torch, args)
        if workload == "prefill_131k":
            # the last 4096-token chunk of a 131072-token context: whether the one flash kernel holds up where
            # the reference switches to its multi-pass form (src/attention_gemm.rs)
            return bench_prefill(s, torch, args, tokens=4096, pos=131072 - 4096)
        if workload == "prefill_gemm":
            return bench_prefill(s, torch, args, gemm=True)
        if workload == "prefill_gemm_131k":
            return bench_prefill(s, torch, args, tokens=4096, pos=131072 - 4096, gemm=True)
        return bench_prefill(s, torch, args)

    if args.workload in ("default", "all"):
        # Both halves of the metric in one line: the decode record at the top level, the
        # prefill-chunk record (same keys) under "prefill"; then short records of the other
        # configurations: the verify step of 2, 3 and 4 rows over the same caches, 4-bit decode at
        # 150000 tokens with the 4-token append, the half cache at 4096 tokens, the Gated DeltaNet
        # decode step and prefill chunk.
        layers = args.layers or 32
        shared = make_decode_workload(s, torch, args.ctx or 32768, 8, 4, layers)
        res = bench_decode(s, torch, args, args.ctx or 32768, 8, 1, layers, workload=shared)
        res["metric"] = "decode attn HBM GB/s @32k ctx 8-bit KV; prefill-chunk attn TFLOP/s"
        other = {}
        for m in (2, 3, 4):
            other[f"verify{m}"] = bench_decode(s, torch, args, args.ctx or 32768, 8, m, layers, compact=True, workload=shared)
        del shared
        torch.cuda.empty_cache()
        res["prefill"] = one("prefill")
        torch.cuda.empty_cache()
        other["decode4_150k"] = bench_decode(s, torch, args, 150000, 4, 1, 12, compact=True)
        torch.cuda.empty_cache()
        other["decode16_4k"] = bench_decode(s, torch, args, 4096, 16, 1, 32, compact=True)
        for w in ["deltanet", "deltanet_prefill"]:
            torch.cuda.empty_cache()
            r = one(w)
            other[w] = {k: r[k] for k in ("metric", "value", "unit", "ms_per_step", "roofline", "parity_rel_rms_vs_oracle")}
            other[w]["config"] = {"workload": r["config"]["workload"]}
        res["other_workloads"] = other
    if args.workload == "all":
        for w in ["prefill_131k", "prefill_gemm", "prefill_gemm_131k", "prep_store"]:
            torch.cuda.empty_cache()
            r = one(w)
            res["other_workloads"][w] = {k: r[k] for k in ("metric", "value", "unit", "ms_per_step", "roofline",
                                                            "parity_rel_rms_vs_oracle")}
    elif args.workload != "default":
        res = one(args.workload)
    res.update({"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
                "scaling": "weak", "vs_baseline": None, "data": "synthetic"})
    print(json.dumps(res))


if __name__ == "__main__":
    main()
