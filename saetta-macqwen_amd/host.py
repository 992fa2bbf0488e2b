"""Host-side objects of the path, named as in the reference.

  kv_quant.rs           KvBits, GROUP, QuantRows (new / record / record_at / encode / encode_dequantize)
  plan.rs               TokenParams, Plan (params / op / set_params / build), Built.run
  attention.rs          DecodeAttention (new / record / record_quant, pub kernel)
  rows.rs               MAX_ROWS, AttentionRows (new / record / record_quant)
  attention_prefill.rs  FlashParams, KERNELS, DEFAULT, KEY_BLOCK, encode

A reference `View` (buffer + byte offset) is a torch tensor here (a slice is a
view with an offset); a Metal encoder is a HIP stream.  Shape violations raise
(the reference asserts); a failed launch raises SaettaError.
"""
import ctypes
import enum
import math

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
    s = stream if stream is not None else torch.cuda.current_stream()
    return ctypes.c_void_p(s.cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


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
            # One eager run first: lazy one-time set-up must not happen under capture.
            self.run()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                s = _stream()
                for _, launch in ops:
                    launch(s)
            self.graph = g

    def run(self, stream=None):
        if self.graph is not None:
            self.graph.replay()
            return
        s = _stream(stream)
        for _, launch in self.ops:
            launch(s)


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
        # The reference switches between a vector and a matrix kernel here; this
        # build has one kernel per cache kind and keeps the field for callers.
        self.kernel = "attention_partial_mma"

    def _params(self):
        return ffi.DecodeParamsC(self.heads, self.kv_heads, self.capacity, 1.0 / math.sqrt(DIM))

    def record(self, plan, q, keys, values, q_and_gate, out):
        _need(q, torch.float32, "q"), _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
        _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        p, tp, po, pml = self._params(), plan.params, self.part_o, self.part_ml

        def launch(stage):
            def f(s):
                ffi.check(ffi.lib().saetta_attn_decode(s, _ptr(q), _ptr(keys), _ptr(values), _ptr(po), _ptr(pml),
                                                       _ptr(q_and_gate), _ptr(out), p, _ptr(tp), stage),
                          "attn_decode")
            return f

        plan.op(self.kernel, launch(ffi.STAGE_PARTIAL))
        plan.op("attention_reduce", launch(ffi.STAGE_REDUCE))

    def record_quant(self, plan, q, keys, values, q_and_gate, out):
        if keys.bits is KvBits.Half:
            raise ValueError("a half cache goes through record")
        _need(q, torch.float32, "q"), _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        p, tp, po, pml, bits = self._params(), plan.params, self.part_o, self.part_ml, keys.bits.value
        kc, vc = keys.c(), values.c()

        def launch(stage):
            def f(s):
                ffi.check(ffi.lib().saetta_attn_decode_quant(s, bits, _ptr(q), kc, vc, _ptr(po), _ptr(pml),
                                                             _ptr(q_and_gate), _ptr(out), p, _ptr(tp), stage),
                          "attn_decode_quant")
            return f

        plan.op(f"{self.kernel}_q{bits}", launch(ffi.STAGE_PARTIAL))
        plan.op("attention_reduce", launch(ffi.STAGE_REDUCE))


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
        uint8 tensor of at least workspace_bytes(p) bytes, or None to let the
        library use its own."""
        if kernel not in attention_prefill.KERNELS:
            raise ValueError(f"no prefill attention kernel {kernel}")
        if p.heads != p.kv_heads * 8:
            raise ValueError(f"{kernel} needs 8 q heads per kv head")
        _need(q, torch.float16, "q"), _need(keys, torch.float16, "keys"), _need(values, torch.float16, "values")
        _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        ffi.check(ffi.lib().saetta_attn_prefill(_stream(stream), _ptr(q), _ptr(keys), _ptr(values),
                                                _ptr(q_and_gate), _ptr(out), p.c(), *_workspace(workspace)),
                  "attn_prefill")

    @staticmethod
    def encode_quant(q, keys, values, q_and_gate, out, p, stream=None, workspace=None):
        """The chunk over a quantized cache read in place (src/prefill.rs:1735-1776)."""
        if p.heads != p.kv_heads * 8:
            raise ValueError("prefill attention needs 8 q heads per kv head")
        _need(q, torch.float16, "q"), _need(q_and_gate, torch.float32, "q_and_gate"), _need(out, torch.float32, "out")
        ffi.check(ffi.lib().saetta_attn_prefill_quant(_stream(stream), keys.bits.value, _ptr(q), keys.c(), values.c(),
                                                      _ptr(q_and_gate), _ptr(out), p.c(), *_workspace(workspace)),
                  "attn_prefill_quant")
