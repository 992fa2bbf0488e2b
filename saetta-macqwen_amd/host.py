"""Host-side objects of the path, named as in the reference.

  kv_quant.rs           KvBits, GROUP, QuantRows (new / record / record_at / encode / encode_dequantize)
  plan.rs               TokenParams, Plan (params / op / constant / set_params / len / is_empty / run_serial /
                        kernels / build / build_where), Built (run / run_timed / commit)
  attention.rs          DecodeAttention (new / record / record_quant, pub kernel)
  rows.rs               MAX_ROWS, AttentionRows (new / record / record_quant)
  attention_prefill.rs  FlashParams, KERNELS, DEFAULT, KEY_BLOCK, encode
  attention_gemm.rs     KEYS, AttGemm (new / encode, pub fused, texp, stages), bench

A reference `View` (buffer + byte offset) is a torch tensor here (a slice is a
view with an offset); a Metal encoder is a HIP stream.  Shape violations raise
(the reference asserts); a failed launch raises SaettaError.
"""
import ctypes
import enum
import math
import time

import torch

from . import ffi

GROUP = 64      # src/kv_quant.rs:9
MAX_ROWS = 8    # src/rows.rs:9
DIM = 256
CHUNK = 128


class KvBits(enum.Enum):
    """src/kv_quant.rs:11-50."""
    Half = 16
    Eight = 8
    Four = 4

    @staticmethod
    def parse(s):
        return {"16": KvBits.Half, "8": KvBits.Eight, "4": KvBits.Four}.get(s)

    def bits(self):
        return self.value

    def words_per_group(self):
        return 2 * self.value

    def bytes_per_value(self):
        return 2.0 if self is KvBits.Half else self.value / 8.0 + 4.0 / GROUP


class TokenParams:
    """src/plan.rs:16-35."""

    def __init__(self, token, position):
        self.token, self.position, self.kv_len, self.pad = token, position, position + 1, 0

    def as_tensor(self, device):
        return torch.tensor([self.token, self.position, self.kv_len, self.pad], dtype=torch.int32,
                            device=device)


def _stream(stream=None):
    if isinstance(stream, ctypes.c_void_p):  # what a plan op is handed
        return stream
    s = stream if stream is not None else torch.cuda.current_stream()
    return ctypes.c_void_p(s.cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def device_status(clear=False):
    """The current device's sticky status word: 0 unless a kernel's bounded wait gave up, after which
    every call on the device raises (SAETTA_E_WAIT) until the word is cleared."""
    return int(ffi.lib().saetta_device_status(1 if clear else 0))


def _need(t, dtype, what):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous()):
        raise TypeError(f"{what}: expected a contiguous {dtype} tensor on the GPU")
    return t


class Plan:
    """A list of launches recorded once and run for every token (src/plan.rs:63-146).

    Per-token state lives in `params`, a TokenParams record in device memory
    that the kernels read when they run."""

    def __init__(self, device="cuda"):
        self.device = torch.device(device)
        self.params = torch.zeros(4, dtype=torch.int32, device=self.device)
        self.ops = []  # (kernel name, callable(stream))

    def op(self, kernel, launch):
        self.ops.append((kernel, launch))

    def set_params(self, tp):
        """Plan::set_params (src/plan.rs:144-146): a small async copy on the current stream."""
        host = torch.tensor([tp.token, tp.position, tp.kv_len, tp.pad], dtype=torch.int32).pin_memory()
        self.params.copy_(host, non_blocking=True)
        self._keep = host

    def __len__(self):
        return len(self.ops)

    def len(self):
        return len(self.ops)

    def is_empty(self):
        return not self.ops

    def constant(self, data):
        """Plan::constant (src/plan.rs:128-141): a device buffer holding `data`, for values that never
        change between tokens."""
        return torch.as_tensor(data).to(self.params.device)

    def run_serial(self, stream=None):
        """Plan::run_serial (src/plan.rs:157-168): every op launched one after the other on the
        stream, outside any graph, then a wait; the wall time in seconds."""
        start = time.perf_counter()
        s = _stream(stream)
        for _, launch in self.ops:
            launch(s)
        torch.cuda.synchronize()
        return time.perf_counter() - start

    def kernels(self):
        """Plan::kernels (src/plan.rs:171-181): each kernel name with how many ops use it, in order
        of first use."""
        out = {}
        for kernel, _ in self.ops:
            out[kernel] = out.get(kernel, 0) + 1
        return list(out.items())

    def build(self, graph=False):
        """Plan::build (src/plan.rs:229-235).  graph=True captures the launches into a HIP
        graph, the counterpart of the reference's indirect command buffer: one submission
        replays them all, and the position still comes from `params` at run time."""
        return Built(list(self.ops), graph)

    def build_where(self, keep, graph=False):
        """Plan::build_where (src/plan.rs:187-226): only the ops whose kernel passes `keep`."""
        return Built([(k, f) for k, f in self.ops if keep(k)], graph)


class Built:
    def __init__(self, ops, graph=False):
        self.ops = ops
        self.graph = None
        if graph and ops:
            # The library's one-time set-up (code objects, LDS limits) must not happen under capture;
            # the launches themselves are not run here: a plan may hold ops that advance a state.
            ffi.check(ffi.lib().saetta_init(), "init")
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                s = _stream()
                for _, launch in ops:
                    launch(s)
            self.graph = g

    def run(self, stream=None):
        """Enqueues the recorded launches (one graph launch, or one by one) and returns without
        waiting: the stream orders what follows, as for any torch op.  Built::commit
        (src/plan.rs:254-256) without the Pending; `run_timed` is the reference's waiting `run`."""
        if self.graph is not None:
            # a captured graph replays on torch's current stream: another stream is the caller's to make current
            if stream is not None and stream.cuda_stream != torch.cuda.current_stream().cuda_stream:
                raise ValueError("Built.run: a captured plan replays on the current stream; make the stream current instead of passing it")
            self.graph.replay()
            return
        s = _stream(stream)
        for _, launch in self.ops:
            launch(s)

    def run_timed(self, stream=None):
        """Built::run_timed (src/plan.rs:249-251): runs, waits, and returns (wall seconds, the
        GPU's own seconds between the first launch and the end of the last, from two events)."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start = time.perf_counter()
        e0.record()
        self.run(stream)
        e1.record()
        e1.synchronize()
        return time.perf_counter() - start, e0.elapsed_time(e1) * 1e-3

    def commit(self, stream=None):
        """Built::commit (src/plan.rs:254-256): `run` without the wait; the event returned waits
        for it (`.synchronize()`)."""
        self.run(stream)
        done = torch.cuda.Event()
        done.record()
        return done


class QuantRows:
    """Codes, scales and biases of one cache (src/kv_quant.rs:156-283)."""

    def __init__(self, bits, values, capacity, device="cuda"):
        if bits is KvBits.Half or values % GROUP:
            raise ValueError("QuantRows: bits must be Eight or Four and values a multiple of 64")
        self.bits = bits
        self.per_token = values // GROUP
        groups = self.per_token * capacity
        self.capacity = capacity
        self.data = torch.zeros(groups * bits.words_per_group(), dtype=torch.int32, device=device)
        self.scales = torch.zeros(groups, dtype=torch.float16, device=device)
        self.biases = torch.zeros(groups, dtype=torch.float16, device=device)

    def c(self):
        return ffi.QuantRowsC(self.data.data_ptr(), self.scales.data_ptr(), self.biases.data_ptr())

    def record(self, plan, x):
        self.record_at(plan, x, plan.params)

    def record_at(self, plan, x, params, parallel=False):
        _need(x, torch.float32, "QuantRows.record x")
        p = ffi.KvQuantParamsC(self.per_token, self.per_token)
        rows, bits = self.c(), self.bits.value

        def launch(s):
            ffi.check(ffi.lib().saetta_kv_quantize(s, bits, _ptr(x), rows, p, _ptr(params), 0), "kv_quantize")

        plan.op(f"kv_quantize_{bits}", launch)

    def encode(self, x, pos, tokens, stream=None):
        _need(x, torch.float32, "QuantRows.encode x")
        if pos + tokens > self.capacity or x.numel() < tokens * self.per_token * GROUP:
            raise ValueError("QuantRows.encode: tokens do not fit")
        p = ffi.KvQuantParamsC(self.per_token * tokens, self.per_token)
        ffi.check(ffi.lib().saetta_kv_quantize(_stream(stream), self.bits.value, _ptr(x), self.c(), p, None, pos),
                  "kv_quantize")

    def encode_dequantize(self, out, tokens, stream=None):
        _need(out, torch.float16, "QuantRows.encode_dequantize out")
        if out.numel() < tokens * self.per_token * GROUP:
            raise ValueError("QuantRows.encode_dequantize: out too small")
        p = ffi.KvQuantParamsC(self.per_token * tokens, self.per_token)
        ffi.check(ffi.lib().saetta_kv_dequantize(_stream(stream), self.bits.value, self.c(), _ptr(out), p),
                  "kv_dequantize")


def quantize(x, bits, stream=None):
    """quantize (src/kv_quant.rs:54-87) of a device f32 tensor whose length is a multiple of
    64: (codes int32 [groups * 2 * bits], scales f16 [groups], biases f16 [groups])."""
    _need(x, torch.float32, "quantize x")
    if bits is KvBits.Half or x.numel() % GROUP:
        raise ValueError("quantize: bits must be Eight or Four and the length a multiple of 64")
    rows = QuantRows(bits, GROUP, x.numel() // GROUP, device=x.device)
    rows.encode(x, 0, x.numel() // GROUP, stream)
    return rows.data, rows.scales, rows.biases


def dequantize(data, scales, biases, bits, stream=None):
    """dequantize (src/kv_quant.rs:90-105): f32 [groups * 64] = f32(s) * code + f32(z)."""
    _need(data, torch.int32, "dequantize data"), _need(scales, torch.float16, "dequantize scales")
    _need(biases, torch.float16, "dequantize biases")
    groups = scales.numel()
    if bits is KvBits.Half or data.numel() != groups * bits.words_per_group() or biases.numel() != groups:
        raise ValueError("dequantize: sizes do not match the bit width")
    out = torch.empty(groups * GROUP, dtype=torch.float32, device=data.device)
    rows = ffi.QuantRowsC(data.data_ptr(), scales.data_ptr(), biases.data_ptr())
    ffi.check(ffi.lib().saetta_kv_dequantize_f32(_stream(stream), bits.value, rows, _ptr(out),
                                                 ffi.KvQuantParamsC(groups, groups)), "kv_dequantize_f32")
    return out


def round_trip(x, bits, stream=None):
    """round_trip (src/kv_quant.rs:107-117): what a decode cache holds of x."""
    if bits is KvBits.Half:
        return x.to(torch.float16).to(torch.float32)
    return dequantize(*quantize(x, bits, stream), bits, stream)


def round_trip_as_half(x, bits, stream=None):
    """round_trip_as_half (src/kv_quant.rs:119-125): what prefill sees of x, f16."""
    if bits is KvBits.Half:
        return x.to(torch.float16)
    rows = QuantRows(bits, GROUP, x.numel() // GROUP, device=x.device)
    rows.encode(x, 0, x.numel() // GROUP, stream)
    out = torch.empty(x.numel(), dtype=torch.float16, device=x.device)
    rows.encode_dequantize(out, x.numel() // GROUP, stream)
    return out


def test_slack(bits):
    """test_slack (src/kv_quant.rs:127-135): how much looser a test bound is per cache kind."""
    return {KvBits.Half: 1.0, KvBits.Eight: 4.0, KvBits.Four: 16.0}[bits]


def to_half(x, out, stream=None):
    """to_half (kernels/prefill.metal:1428-1432)."""
    _need(x, torch.float32, "to_half x")
    _need(out, torch.float16, "to_half out")
    ffi.check(ffi.lib().saetta_to_half(_stream(stream), _ptr(x), _ptr(out), x.numel()), "to_half")


def _check_shape(heads, kv_heads, head_dim, what):
    if head_dim != DIM:
        raise ValueError(f"{what} is written for head dim 256")
    if heads != kv_heads * 8:
        raise ValueError(f"{what} needs 8 q heads per kv head")


class DecodeAttention:
    """Scratch and launches of one-token attention (src/attention.rs:28-171)."""

    def __init__(self, heads, kv_heads, head_dim, capacity, device="cuda"):
        _check_shape(heads, kv_heads, head_dim, "decode attention")
        self.heads, self.kv_heads, self.capacity = heads, kv_heads, capacity
        l = ffi.lib()
        self.part_o = torch.empty(l.saetta_part_o_bytes(heads, capacity, 1) // 4, dtype=torch.float32,
                                  device=device)
        self.part_ml = torch.empty(l.saetta_part_ml_bytes(heads, capacity, 1) // 4, dtype=torch.float32,
                                   device=device)
        # The reference switches between its two kernel families here (src/attention.rs:36-38).
        # "attention_partial_mma": the library picks, which for one row over codes in a large
        # cache is the kernel with loader waves; "attention_partial": the register kernels only.
        self.kernel = "attention_partial_mma"

    def _flags(self):
        if self.kernel not in ("attention_partial_mma", "attention_partial"):
            raise ValueError(f"no decode attention kernel {self.kernel}")
        return 0 if self.kernel == "attention_partial_mma" else ffi.STAGE_NO_LOADERS

    def _params(self):
        return ffi.DecodeParamsC(self.heads, self.kv_heads, self.capacity, 1.0 / math.sqrt(DIM))

    def record(self, plan, q, keys, values, q_and_gate, out):
        _need(q, torch.float32, "q"), _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
        _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        p, tp, po, pml, flags = self._params(), plan.params, self.part_o, self.part_ml, self._flags()

        def launch(stage):
            def f(s):
                ffi.check(ffi.lib().saetta_attn_decode(s, _ptr(q), _ptr(keys), _ptr(values), _ptr(po), _ptr(pml),
                                                       _ptr(q_and_gate), _ptr(out), p, _ptr(tp), stage | flags),
                          "attn_decode")
            return f

        plan.op(self.kernel, launch(ffi.STAGE_PARTIAL))
        plan.op("attention_reduce", launch(ffi.STAGE_REDUCE))

    def record_quant(self, plan, q, keys, values, q_and_gate, out):
        if keys.bits is KvBits.Half:
            raise ValueError("a half cache goes through record")
        _need(q, torch.float32, "q"), _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        p, tp, po, pml, bits = self._params(), plan.params, self.part_o, self.part_ml, keys.bits.value
        kc, vc, flags = keys.c(), values.c(), self._flags()

        def launch(stage):
            def f(s):
                ffi.check(ffi.lib().saetta_attn_decode_quant(s, bits, _ptr(q), kc, vc, _ptr(po), _ptr(pml),
                                                             _ptr(q_and_gate), _ptr(out), p, _ptr(tp), stage | flags),
                          "attn_decode_quant")
            return f

        plan.op(f"{self.kernel}_q{bits}", launch(ffi.STAGE_PARTIAL))
        plan.op("attention_reduce", launch(ffi.STAGE_REDUCE))


class PrepParams:
    """PrepParams (src/gpu_layers.rs:387-394)."""

    def __init__(self, heads, kv_heads, dim, rope_dims, rope_theta, eps):
        self.heads, self.kv_heads, self.dim, self.half_dims = heads, kv_heads, dim, rope_dims // 2
        self.log2_theta, self.eps = math.log2(rope_theta), eps

    def c(self):
        return ffi.PrepParamsC(self.heads, self.kv_heads, self.dim, self.half_dims, self.log2_theta, self.eps)


def record_store(plan, q_and_gate, k, v, q_norm, k_norm, q, keys, values, p, capacity, rows=1, k_back=None):
    """GpuAttention::record_store (src/gpu_layers.rs:370-411): q norm and RoPE into q, k norm and
    RoPE, then the token's key and value into the cache slot at the plan's position: as half
    (`keys`, `values` f16 tensors) or as codes (`keys`, `values` QuantRows), in one launch where the
    reference records attention_prep{,_float} and two kv_quantize dispatches.  k_back: an f32
    tensor that gets the normed, rotated key (what attention_prep_float leaves in k), or None."""
    for t, what in ((q_and_gate, "q_and_gate"), (k, "k"), (v, "v"), (q_norm, "q_norm"), (k_norm, "k_norm"), (q, "q")):
        _need(t, torch.float32, what)
    quant = isinstance(keys, QuantRows)
    if quant != isinstance(values, QuantRows):
        raise ValueError("record_store: keys and values must be the same kind of cache")
    none = ffi.QuantRowsC(None, None, None)
    if quant:
        bits, kh, vh, kq, vq = keys.bits.value, None, None, keys.c(), values.c()
    else:
        _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
        bits, kh, vh, kq, vq = 16, _ptr(keys), _ptr(values), none, none
    pc, tp = p.c(), plan.params
    kb = None if k_back is None else _ptr(k_back)

    def launch(s):
        ffi.check(ffi.lib().saetta_attn_prep_store(s, bits, _ptr(q_and_gate), _ptr(k), _ptr(v), _ptr(q_norm),
                                                   _ptr(k_norm), _ptr(q), kh, vh, kq, vq, kb, pc, rows, capacity,
                                                   _ptr(tp)), "attn_prep_store")

    plan.op("attention_prep_store", launch)


def deltanet_conv(plan, x, w, state, out, channels, kernel_size):
    """Records deltanet_conv (kernels/layers.metal:203-226; conv_step, src/cpu/deltanet.rs:117-131):
    depthwise causal conv1d + SiLU of one token; `state` [kernel_size - 1][channels] takes x in."""
    for t, what in ((x, "x"), (w, "w"), (state, "state"), (out, "out")):
        _need(t, torch.float32, what)
    if x.numel() < channels or w.numel() < channels * kernel_size or state.numel() < (kernel_size - 1) * channels:
        raise ValueError("deltanet_conv: buffers too small")
    p = ffi.ConvParamsC(channels, kernel_size)
    plan.op("deltanet_conv", lambda s: ffi.check(
        ffi.lib().saetta_deltanet_conv(s, _ptr(x), _ptr(w), _ptr(state), _ptr(out), p), "deltanet_conv"))


def deltanet_step(plan, q, k, v, a, b, a_log, dt_bias, state, z, norm_w, y, k_heads, v_heads, v_dim, eps):
    """Records deltanet_step (kernels/layers.metal:297-357): normalize_qk, the gates, the delta rule
    and the gated RMSNorm for every value head (src/cpu/deltanet.rs:86-112,133-155); key dim 128."""
    ts = (q, k, v, a, b, a_log, dt_bias, state, z, norm_w, y)
    for t in ts:
        _need(t, torch.float32, "deltanet_step buffer")
    if state.numel() < v_heads * v_dim * 128 or q.numel() < k_heads * 128 or v.numel() < v_heads * v_dim:
        raise ValueError("deltanet_step: buffers too small")
    p = ffi.StepParamsC(k_heads, v_heads, v_dim, eps)
    plan.op("deltanet_step", lambda s: ffi.check(
        ffi.lib().saetta_deltanet_step(s, *[_ptr(t) for t in ts], p), "deltanet_step"))


def deltanet_token(plan, x, w, conv_state, a, b, a_log, dt_bias, state, z, norm_w, y, k_heads, v_heads, v_dim,
                   kernel_size, eps):
    """Records one token of a Gated DeltaNet layer, conv and step (GpuDeltaNet::record,
    src/gpu_layers.rs:633-684) as one call of two launches: what deltanet_conv + deltanet_step give,
    without the conv output in between."""
    ts = (x, w, conv_state, a, b, a_log, dt_bias, state, z, norm_w, y)
    for t in ts:
        _need(t, torch.float32, "deltanet_token buffer")
    channels = 2 * k_heads * 128 + v_heads * v_dim
    if (x.numel() < channels or w.numel() < channels * kernel_size or conv_state.numel() < (kernel_size - 1) * channels
            or state.numel() < v_heads * v_dim * 128 or y.numel() < v_heads * v_dim or z.numel() < v_heads * v_dim):
        raise ValueError("deltanet_token: buffers too small")
    cp, sp = ffi.ConvParamsC(channels, kernel_size), ffi.StepParamsC(k_heads, v_heads, v_dim, eps)
    plan.op("deltanet_token", lambda s: ffi.check(
        ffi.lib().saetta_deltanet_token(s, *[_ptr(t) for t in ts], cp, sp), "deltanet_token"))


def deltanet_conv_rows(plan, x, w, state, out, channels, kernel_size, tokens, snaps=None):
    """Records the conv of `tokens` tokens in order (conv_rows2 + conv_state, kernels/prefill.metal:734-786;
    deltanet_conv_rows, kernels/layers.metal:510-544): x, out [tokens][channels]; with `snaps`
    ([tokens][kernel_size - 1][channels]) the state after each token goes there too."""
    for t, what in ((x, "x"), (w, "w"), (state, "state"), (out, "out")):
        _need(t, torch.float32, what)
    if snaps is not None:
        _need(snaps, torch.float32, "snaps")
        if snaps.numel() < tokens * (kernel_size - 1) * channels:
            raise ValueError("deltanet_conv_rows: snapshots too small")
    if (x.numel() < tokens * channels or out.numel() < tokens * channels or w.numel() < channels * kernel_size
            or state.numel() < (kernel_size - 1) * channels):
        raise ValueError("deltanet_conv_rows: buffers too small")
    p = ffi.ConvRowsParamsC(channels, kernel_size, tokens, int(snaps is not None))
    plan.op("deltanet_conv_rows", lambda s: ffi.check(
        ffi.lib().saetta_deltanet_conv_rows(s, _ptr(x), _ptr(w), _ptr(state), _ptr(out),
                                            _ptr(snaps) if snaps is not None else None, p), "deltanet_conv_rows"))


def deltanet_rows(plan, mixed, a, b, a_log, dt_bias, state, z, norm_w, y, k_heads, v_heads, v_dim, tokens, eps,
                  snaps=None):
    """Records the step of `tokens` tokens in order (delta_prep + delta_rows3 + gated norm,
    kernels/prefill.metal:788-1116, src/prefill.rs:1487-1578; deltanet_step_rows,
    GpuDeltaNet::record_rows, src/gpu_layers.rs:686-786): `mixed` [tokens][q | k | v] is the conv
    output; with `snaps` ([tokens][v_heads][v_dim][128]) the state after each token goes there too."""
    ts = (mixed, a, b, a_log, dt_bias, state, z, norm_w, y)
    for t in ts:
        _need(t, torch.float32, "deltanet_rows buffer")
    channels = 2 * k_heads * 128 + v_heads * v_dim
    if (mixed.numel() < tokens * channels or state.numel() < v_heads * v_dim * 128
            or y.numel() < tokens * v_heads * v_dim or z.numel() < tokens * v_heads * v_dim
            or a.numel() < tokens * v_heads or b.numel() < tokens * v_heads):
        raise ValueError("deltanet_rows: buffers too small")
    if snaps is not None:
        _need(snaps, torch.float32, "snaps")
        if snaps.numel() < tokens * v_heads * v_dim * 128:
            raise ValueError("deltanet_rows: snapshots too small")
    p = ffi.RowsStepParamsC(k_heads, v_heads, v_dim, tokens, eps, int(snaps is not None))
    # a prefill chunk runs in blocks of 64 tokens and keeps per-block matrices in a workspace, which the
    # recorded op owns (the reference's prefill works in buffers of its own, src/prefill.rs:1433-1578)
    need = ffi.lib().saetta_deltanet_rows_workspace_bytes(p)
    ws = torch.empty(need, dtype=torch.uint8, device=mixed.device) if need else None
    plan.op("deltanet_rows", lambda s: ffi.check(
        ffi.lib().saetta_deltanet_rows_ws(s, *[_ptr(t) for t in ts], _ptr(snaps) if snaps is not None else None, p,
                                          _ptr(ws) if ws is not None else None, need),
        "deltanet_rows"))


def deltanet_rows_fused(plan, x, w, conv_state, a, b, a_log, dt_bias, state, z, norm_w, y, k_heads, v_heads, v_dim,
                        kernel_size, rows, eps, conv_snaps=None, state_snaps=None):
    """Records up to 8 rows of a Gated DeltaNet layer, conv and step, as one call of two launches
    (kernel deltanet_rows, GpuDeltaNet::record_rows with DN_SIMDS = 0, src/gpu_layers.rs:737-757):
    x, z [rows][...] as for deltanet_conv_rows + deltanet_rows, which this equals; with the two
    snapshot buffers the conv and delta states after each row go there too."""
    ts = (x, w, conv_state, a, b, a_log, dt_bias, state, z, norm_w, y)
    for t in ts:
        _need(t, torch.float32, "deltanet_rows_fused buffer")
    if rows > MAX_ROWS:
        raise ValueError(f"deltanet_rows_fused: {rows} rows (up to {MAX_ROWS})")
    if (conv_snaps is None) != (state_snaps is None):
        raise ValueError("deltanet_rows_fused: both snapshot buffers or neither")
    channels = 2 * k_heads * 128 + v_heads * v_dim
    if (x.numel() < rows * channels or w.numel() < channels * kernel_size
            or conv_state.numel() < (kernel_size - 1) * channels or state.numel() < v_heads * v_dim * 128
            or y.numel() < rows * v_heads * v_dim or z.numel() < rows * v_heads * v_dim
            or a.numel() < rows * v_heads or b.numel() < rows * v_heads):
        raise ValueError("deltanet_rows_fused: buffers too small")
    if conv_snaps is not None:
        _need(conv_snaps, torch.float32, "conv_snaps")
        _need(state_snaps, torch.float32, "state_snaps")
        if conv_snaps.numel() < rows * (kernel_size - 1) * channels or state_snaps.numel() < rows * v_heads * v_dim * 128:
            raise ValueError("deltanet_rows_fused: snapshots too small")
    p = ffi.RowsFusedParamsC(k_heads, v_heads, v_dim, kernel_size, eps, rows, int(conv_snaps is not None))
    plan.op("deltanet_rows_fused", lambda s: ffi.check(
        ffi.lib().saetta_deltanet_rows_fused(s, *[_ptr(t) for t in ts],
                                             _ptr(conv_snaps) if conv_snaps is not None else None,
                                             _ptr(state_snaps) if state_snaps is not None else None, p),
        "deltanet_rows_fused"))


KV_ALIGN = 128  # src/gpu_layers.rs:199: the decode chunk, and a multiple of the prefill key block


class GpuKvCache:
    """GpuKvCache (src/gpu_layers.rs:183-293): the keys and values of one attention layer on the
    GPU, token p in row p, half values or codes with their scales and biases, plus the decode
    attention sized for the capacity.  `resize` moves to new buffers and copies every old row that
    fits; plans recorded with the old buffers must be recorded again, as in the reference."""

    def __init__(self, heads, kv_heads, head_dim, capacity, bits=KvBits.Half, device="cuda"):
        self.heads, self.kv_heads, self.head_dim, self.bits, self.device = heads, kv_heads, head_dim, bits, device
        self.capacity = -(-capacity // KV_ALIGN) * KV_ALIGN
        values = kv_heads * head_dim
        self.decode = DecodeAttention(heads, kv_heads, head_dim, self.capacity, device)
        if bits is KvBits.Half:
            self.quant = None
            self.keys = torch.zeros(self.capacity * values, dtype=torch.float16, device=device)
            self.values = torch.zeros(self.capacity * values, dtype=torch.float16, device=device)
        else:
            k, v = QuantRows(bits, values, self.capacity, device), QuantRows(bits, values, self.capacity, device)
            self.quant, self.keys, self.values = (k, v), k.data, v.data

    @classmethod
    def with_bits(cls, heads, kv_heads, head_dim, capacity, bits, device="cuda"):
        return cls(heads, kv_heads, head_dim, capacity, bits, device)

    def buffers(self):
        """Every buffer of the cache; each holds `capacity` rows of equal size (src/gpu_layers.rs:247-253)."""
        out = [self.keys, self.values]
        if self.quant:
            k, v = self.quant
            out += [k.scales, k.biases, v.scales, v.biases]
        return out

    def resize(self, capacity):
        capacity = -(-capacity // KV_ALIGN) * KV_ALIGN
        old, rows = self.capacity, min(self.capacity, capacity)
        moved = []
        for b in self.buffers():
            per_row = b.numel() // old
            new = torch.zeros(per_row * capacity, dtype=b.dtype, device=b.device)
            new[:per_row * rows].copy_(b[:per_row * rows])
            moved.append(new)
        torch.cuda.current_stream().synchronize()  # the reference waits for the blit as well
        self.keys, self.values = moved[0], moved[1]
        if self.quant:
            k, v = self.quant
            k.data, v.data = self.keys, self.values
            k.scales, k.biases, v.scales, v.biases = moved[2:6]
            k.capacity = v.capacity = capacity
        self.decode = DecodeAttention(self.heads, self.kv_heads, self.head_dim, capacity, self.device)
        self.capacity = capacity


class RowBackup:
    """RowBackup (src/gpu_cache.rs:196-283): a copy of KV rows from..from + n of every attention
    layer, for a short detour that writes over a long conversation; `restore` puts them back."""

    def __init__(self):
        self.copy = None

    def bytes(self):
        return sum(p.numel() * p.element_size() for p in self.copy[0]) if self.copy else 0

    @staticmethod
    def _parts(caches):
        return [(b, b.numel() // c.capacity) for c in caches for b in c.buffers()]

    def save(self, caches, start, n):
        self.copy = None
        if n == 0 or not caches:
            return
        if any(start + n > c.capacity for c in caches):
            raise ValueError("RowBackup.save: rows past the capacity")
        self.copy = ([b[start * row:(start + n) * row].clone() for b, row in self._parts(caches)], start, n)

    def restore(self, caches):
        if not self.copy:
            return
        parts, start, n = self.copy
        self.copy = None
        for (b, row), saved in zip(self._parts(caches), parts):
            b[start * row:(start + n) * row].copy_(saved)

    def clear(self):
        self.copy = None


def _median_ms(run, runs):
    """One warm-up, then the median of `runs` event-timed calls, in milliseconds."""
    ts = []
    for i in range(runs + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        run()
        e1.record()
        e1.synchronize()
        if i:
            ts.append(e0.elapsed_time(e1))
    ts.sort()
    return ts[len(ts) // 2]


def bench(lengths, layers, runs, bits=KvBits.Half, device="cuda"):
    """attention::bench (src/attention.rs:173-231): one token's attention over `layers` caches of
    their own, at each context length; same fill values, median of `runs` after a warm-up,
    bytes = layers * len * token * 2 (K, V) * bytes per value.  Returns one dict per length."""
    heads, kv = 16, 2
    capacity = -(-max(lengths) // CHUNK) * CHUNK
    token = kv * DIM
    i = torch.arange(capacity * token, device=device, dtype=torch.int64)
    fill = (((i * 7919) % 2000).to(torch.float32) / 1000.0 - 1.0)
    caches = []
    for _ in range(layers):
        if bits is KvBits.Half:
            caches.append((fill.to(torch.float16), fill.to(torch.float16)))
        else:
            k, v = QuantRows(bits, token, capacity, device), QuantRows(bits, token, capacity, device)
            k.encode(fill, 0, capacity), v.encode(fill, 0, capacity)
            caches.append((k, v))
    q = torch.full((heads * DIM,), 0.01, device=device)
    qg = torch.full((heads * 2 * DIM,), 0.5, device=device)
    out = torch.empty(heads * DIM, device=device)
    att = DecodeAttention(heads, kv, DIM, capacity, device)
    plan = Plan(device)
    for k, v in caches:
        (att.record if bits is KvBits.Half else att.record_quant)(plan, q, k, v, qg, out)
    built = plan.build(graph=True)
    reduce = plan.build_where(lambda name: name == "attention_reduce", graph=True)
    rows = []
    for n in lengths:
        plan.set_params(TokenParams(0, n - 1))
        ms, reduce_ms = _median_ms(built.run, runs), _median_ms(reduce.run, runs)
        nbytes = layers * n * token * 2 * bits.bytes_per_value()
        rows.append({"tokens": n, "ms": ms, "GB/s": nbytes / ms / 1e6, "reduce_ms": reduce_ms})
    return rows


class AttentionRows:
    """Verify attention for 1..8 rows (src/rows.rs:344-494)."""

    def __init__(self, heads, kv_heads, capacity, rows, device="cuda"):
        _check_shape(heads, kv_heads, DIM, "rows attention")
        if not 1 <= rows <= MAX_ROWS:
            raise ValueError(f"{rows} rows")
        self.heads, self.kv_heads, self.capacity, self.rows = heads, kv_heads, capacity, rows
        l = ffi.lib()
        self.splits = l.saetta_part_ml_bytes(heads, capacity, 1) // (heads * 8)
        self.part_o = torch.empty(l.saetta_part_o_bytes(heads, capacity, rows) // 4, dtype=torch.float32,
                                  device=device)
        self.part_ml = torch.empty(l.saetta_part_ml_bytes(heads, capacity, rows) // 4, dtype=torch.float32,
                                   device=device)

    def _params(self, m):
        return ffi.RowsParamsC(self.heads, self.kv_heads, self.capacity, 1.0 / math.sqrt(DIM), m, self.splits)

    def record(self, plan, m, q, keys, values, q_and_gate, out, params):
        if m > self.rows or len(params) < m:
            raise ValueError("AttentionRows.record: too many rows")
        _need(q, torch.float32, "q"), _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
        _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        p, tp, po, pml = self._params(m), params[0], self.part_o, self.part_ml

        def launch(stage):
            def f(s):
                ffi.check(ffi.lib().saetta_attn_rows(s, _ptr(q), _ptr(keys), _ptr(values), _ptr(po), _ptr(pml),
                                                     _ptr(q_and_gate), _ptr(out), p, _ptr(tp), stage), "attn_rows")
            return f

        plan.op("attention_partial_rows_chunks", launch(ffi.STAGE_PARTIAL))
        plan.op("attention_reduce_rows_chunks", launch(ffi.STAGE_REDUCE))

    def record_quant(self, plan, m, q, keys, values, q_and_gate, out, params):
        if m > self.rows or len(params) < m:
            raise ValueError("AttentionRows.record_quant: too many rows")
        if keys.bits is KvBits.Half:
            raise ValueError("a half cache goes through record")
        _need(q, torch.float32, "q"), _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        p, tp, po, pml, bits = self._params(m), params[0], self.part_o, self.part_ml, keys.bits.value
        kc, vc = keys.c(), values.c()

        def launch(stage):
            def f(s):
                ffi.check(ffi.lib().saetta_attn_rows_quant(s, bits, _ptr(q), kc, vc, _ptr(po), _ptr(pml),
                                                           _ptr(q_and_gate), _ptr(out), p, _ptr(tp), stage),
                          "attn_rows_quant")
            return f

        plan.op(f"attention_partial_rows_q{bits}", launch(ffi.STAGE_PARTIAL))
        plan.op("attention_reduce_rows", launch(ffi.STAGE_REDUCE))


def _workspace(t):
    if t is None:
        return None, 0
    _need(t, torch.uint8, "workspace")
    return _ptr(t), t.numel()


def _workspace_or_own(t, nbytes, like, stream):
    """The caller's workspace, or a tensor of this call's own from torch's allocator (which hands a
    block out again only behind the work queued on its stream): the library's own workspace, which a
    NULL pointer would select, is one per device and stream that stays for the life of the process."""
    if t is not None:
        return t
    t = torch.empty(nbytes, dtype=torch.uint8, device=like.device)
    if isinstance(stream, torch.cuda.Stream):
        t.record_stream(stream)
    return t


class FlashParams:
    """src/attention_prefill.rs:4-14."""

    def __init__(self, heads, kv_heads, pos, tokens, scale):
        self.heads, self.kv_heads, self.pos, self.tokens, self.scale = heads, kv_heads, pos, tokens, scale

    def c(self):
        return ffi.FlashParamsC(self.heads, self.kv_heads, self.pos, self.tokens, self.scale)


class attention_prefill:
    """Namespace of src/attention_prefill.rs."""
    KERNELS = ["attention_fa8", "attention_fa4"]
    DEFAULT = "attention_fa8"
    KEY_BLOCK = 16
    FlashParams = FlashParams

    @staticmethod
    def workspace_bytes(p):
        """Bytes of workspace a chunk with these FlashParams needs."""
        return ffi.lib().saetta_prefill_workspace_bytes(p.pos, p.tokens, p.kv_heads)

    @staticmethod
    def encode(kernel, q, keys, values, q_and_gate, out, p, stream=None, workspace=None):
        """encode (src/attention_prefill.rs:39-72).  `kernel` picks a tile size in
        the reference; the one gfx950 kernel serves both names.  `workspace` is a
        uint8 tensor of at least workspace_bytes(p) bytes, or None for one of this
        call's own (a caller that times the call, or records it, brings its own)."""
        if kernel not in attention_prefill.KERNELS:
            raise ValueError(f"no prefill attention kernel {kernel}")
        if p.heads != p.kv_heads * 8:
            raise ValueError(f"{kernel} needs 8 q heads per kv head")
        _need(q, torch.float16, "q"), _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
        _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        workspace = _workspace_or_own(workspace, attention_prefill.workspace_bytes(p), q, stream)
        ffi.check(ffi.lib().saetta_attn_prefill(_stream(stream), _ptr(q), _ptr(keys), _ptr(values),
                                                _ptr(q_and_gate), _ptr(out), p.c(), *_workspace(workspace)),
                  "attn_prefill")

    @staticmethod
    def encode_rows2(q, keys, values, q_and_gate, out, p, stream=None, workspace=None):
        """encode_rows2 (src/attention_prefill.rs:74-100): the reference's attention_rows2_half on
        the same buffers, its baseline in `bench`; here the same kernel as `encode`."""
        attention_prefill.encode(attention_prefill.DEFAULT, q, keys, values, q_and_gate, out, p, stream, workspace)

    @staticmethod
    def spread(n, seed, device="cuda"):
        """spread (src/attention_prefill.rs:102-108): half values in about -2 .. 2.  Test data,
        made on the host in IEEE f32 (one division, one subtraction, one rounding to half) and
        copied to the device."""
        import numpy as np
        i = np.arange(n, dtype=np.int64)
        x = ((i * 7919 + seed * 104729) % 1999).astype(np.float32) / np.float32(500.0) - np.float32(2.0)
        return torch.from_numpy(x.astype(np.float16)).to(device)

    @staticmethod
    def bench(contexts, chunk, layers, device="cuda"):
        """bench (src/attention_prefill.rs:110-176): a chunk of `chunk` tokens at the middle and at
        the end of a prefill of each context, best of 3 after a warm-up; TFLOP/s by the causal
        count 4 * heads * dim * (chunk * pos + chunk * (chunk + 1) / 2).  One dict per context."""
        heads, kv, dim = 16, 2, DIM
        rows = []
        for n in contexts:
            n = -(-n // chunk) * chunk
            capacity = -(-n // 64) * 64 + 64
            q = attention_prefill.spread(chunk * heads * dim, 1, device)
            k = attention_prefill.spread(capacity * kv * dim, 2, device)
            v = attention_prefill.spread(capacity * kv * dim, 3, device)
            g = ((torch.arange(chunk * heads * 2 * dim, device=device) % 7) - 3).to(torch.float32)
            out = torch.empty(chunk * heads * dim, dtype=torch.float32, device=device)
            chunks = n // chunk
            mid, last = (chunks // 2) * chunk, n - chunk

            def flops(pos):
                return 4.0 * heads * dim * (chunk * pos + chunk * (chunk + 1) / 2)

            def best_ms(pos):
                p = FlashParams(heads, kv, pos, chunk, 1.0 / math.sqrt(dim))
                ws = torch.empty(attention_prefill.workspace_bytes(p), dtype=torch.uint8, device=device)

                def run():
                    attention_prefill.encode(attention_prefill.DEFAULT, q, k, v, g, out, p, workspace=ws)

                run()
                best = float("inf")
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    run()
                    e1.record()
                    e1.synchronize()
                    best = min(best, e0.elapsed_time(e1))
                return best

            tm, tl = best_ms(mid), best_ms(last)
            rows.append({"context": n, "chunk": chunk, "last_ms": tl, "last_TFLOP/s": flops(last) / tl / 1e9,
                         "mid_TFLOP/s": flops(mid) / tm / 1e9, "prefill_attention_s": tm * 1e-3 * chunks * layers})
        return rows

    @staticmethod
    def encode_quant(q, keys, values, q_and_gate, out, p, stream=None, workspace=None):
        """The chunk over a quantized cache read in place (src/prefill.rs:1735-1776)."""
        if p.heads != p.kv_heads * 8:
            raise ValueError("prefill attention needs 8 q heads per kv head")
        _need(q, torch.float16, "q"), _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        workspace = _workspace_or_own(workspace, attention_prefill.workspace_bytes(p), q, stream)
        ffi.check(ffi.lib().saetta_attn_prefill_quant(_stream(stream), keys.bits.value, _ptr(q), keys.c(), values.c(),
                                                      _ptr(q_and_gate), _ptr(out), p.c(), *_workspace(workspace)),
                  "attn_prefill_quant")


class attention_gemm:
    """Namespace of src/attention_gemm.rs: prefill attention as matrix products over blocks of keys."""
    KEYS = 1024    # src/attention_gemm.rs:28
    # Query slices a chunk runs in unless SAETTA_AG_SLICES says otherwise.  The reference takes 2
    # (src/attention_gemm.rs:59-63) to halve a scratch that shares the machine's one memory with the model;
    # here one: 1.2 GB of scratch for a 4096-token chunk, and twice the workgroups per launch.
    SLICES = 1

    @staticmethod
    def slices():
        """SAETTA_AG_SLICES, as the reference reads it (src/attention_gemm.rs:83-89)."""
        import os
        try:
            n = int(os.environ.get("SAETTA_AG_SLICES", ""))
        except ValueError:
            n = 0
        return n if n > 0 else attention_gemm.SLICES

    class AttGemm:
        """AttGemm (src/attention_gemm.rs:95-364): the buffers of one block for slices of up to `slice`
        tokens of a chunk, and `encode`.  Only the reference's default variant exists here (`fused` and
        `texp` both true: the scores pass writes the probabilities relative to each tile's maximum and the
        tiles' sums, the pv pass scales a tile once); SAETTA_AG_FUSED=0 or SAETTA_AG_TEXP=0 raise.
        `stages` as in the reference's bench: 0 all passes, 1 or 2 scores only, 3 scores and pv and no
        outputs."""

        def __init__(self, chunk, kv_heads, device="cuda"):
            import os
            for name in ("SAETTA_AG_FUSED", "SAETTA_AG_TEXP"):
                if os.environ.get(name) == "0":
                    raise ValueError(f"{name}=0: only the fused variant with tile sums is built")
            self.slice = -(-chunk // attention_gemm.slices())
            self.rows_pad = -(-self.slice * 8 // 64) * 64
            self.chunk, self.kv_heads, self.device = chunk, kv_heads, device
            self.fused = self.texp = True
            self.stages = 0
            self._workspace = None

        def workspace_bytes(self, p):
            return ffi.lib().saetta_attn_gemm_workspace_bytes(p.pos, p.tokens, self.slice, p.kv_heads)

        def encode(self, q, keys, values, quant, q_and_gate, out, f, stream=None):
            """encode (src/attention_gemm.rs:144-188): the same as attention_prefill.encode on the same
            buffers; with `quant` = (QuantRows of the keys, QuantRows of the values) the cache is read from
            those 8- or 4-bit rows and `keys` and `values` are not read."""
            if f.heads != f.kv_heads * 8:
                raise ValueError("needs 8 q heads per kv head")
            if f.tokens > self.chunk or f.kv_heads != self.kv_heads:
                raise ValueError(f"AttGemm for chunks of {self.chunk} tokens and {self.kv_heads} kv heads")
            _need(q, torch.float16, "q"), _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
            if quant is None:
                _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
                bits = 16
                k = ffi.QuantRowsC(_ptr(keys), None, None)
                v = ffi.QuantRowsC(_ptr(values), None, None)
            else:
                if quant[0].bits is KvBits.Half or quant[0].bits is not quant[1].bits:
                    raise ValueError(f"no gemm attention for {quant[0].bits} rows")
                bits, k, v = quant[0].bits.value, quant[0].c(), quant[1].c()
            need = self.workspace_bytes(f)
            if self._workspace is None or self._workspace.numel() < need:
                self._workspace = torch.empty(need, dtype=torch.uint8, device=self.device)
            ffi.check(ffi.lib().saetta_attn_gemm(_stream(stream), bits, _ptr(q), k, v, _ptr(q_and_gate), _ptr(out),
                                                 f.c(), self.slice, self.stages, *_workspace(self._workspace)),
                      "attn_gemm")

    @staticmethod
    def bench(contexts, chunk, layers, device="cuda"):
        """bench (src/attention_gemm.rs:366-470): for each context the chunk of `chunk` tokens at its end and
        at its middle through attention_prefill.encode_rows2 and through AttGemm, best of 3 after a warm-up;
        the gemm passes of the last chunk one by one as differences of runs that stop early; the largest and
        the rms relative difference of the two outputs.  One dict per context."""
        heads, kv, dim = 16, 2, DIM
        gemm = attention_gemm.AttGemm(chunk, kv, device)
        rows = []
        for n in contexts:
            n = -(-n // chunk) * chunk
            capacity = -(-n // 64) * 64 + 64
            q = attention_prefill.spread(chunk * heads * dim, 1, device)
            k = attention_prefill.spread(capacity * kv * dim, 2, device)
            v = attention_prefill.spread(capacity * kv * dim, 3, device)
            g = ((torch.arange(chunk * heads * 2 * dim, device=device) % 7) - 3).to(torch.float32)
            want = torch.empty(chunk * heads * dim, dtype=torch.float32, device=device)
            got = torch.empty_like(want)
            chunks = n // chunk
            mid, last = (chunks // 2) * chunk, n - chunk
            ws = torch.empty(attention_prefill.workspace_bytes(FlashParams(heads, kv, last, chunk, 1.0)),
                             dtype=torch.uint8, device=device)

            def flops(pos):
                return 4.0 * heads * dim * (chunk * pos + chunk * (chunk + 1) / 2)

            def best_ms(gemm_kernel, pos):
                p = FlashParams(heads, kv, pos, chunk, 1.0 / math.sqrt(dim))

                def run():
                    if gemm_kernel:
                        gemm.encode(q, k, v, None, g, got, p)
                    else:
                        attention_prefill.encode_rows2(q, k, v, g, want, p, workspace=ws)

                run()
                best = float("inf")
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    run()
                    e1.record()
                    e1.synchronize()
                    best = min(best, e0.elapsed_time(e1))
                return best

            row = {"context": n, "chunk": chunk}
            for name, gemm_kernel in (("rows2", False), ("gemm", True)):
                tl, tm = best_ms(gemm_kernel, last), best_ms(gemm_kernel, mid)
                row[name] = {"last_ms": tl, "last_TFLOP/s": flops(last) / tl / 1e9, "mid_TFLOP/s": flops(mid) / tm / 1e9,
                             "prefill_attention_s": tm * 1e-3 * chunks * layers}
            prefix = [0.0] * 4
            for stage in (1, 2, 3):
                gemm.stages = stage
                prefix[stage] = best_ms(True, last)
            gemm.stages = 0
            whole = best_ms(True, last)
            row["stages"] = {"scores_ms": prefix[1], "scores_TFLOP/s": flops(last) / 2 / prefix[1] / 1e9,
                             "softmax_ms": prefix[2] - prefix[1], "pv_ms": prefix[3] - prefix[2],
                             "pv_TFLOP/s": flops(last) / 2 / max(prefix[3] - prefix[2], 1e-9) / 1e9,
                             "final_ms": whole - prefix[3]}
            # both outputs are now of the last chunk
            best_ms(False, last)
            diff = (want - got).double()
            row["rel_rms"] = float((diff.pow(2).sum() / want.double().pow(2).sum()).sqrt())
            row["max_abs"] = float(diff.abs().max())
            rows.append(row)
        return rows
