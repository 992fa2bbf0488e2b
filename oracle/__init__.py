"""ctypes front end of the CPU oracle (``saetta_oracle.c``).

TEST INFRASTRUCTURE ONLY: the product library never imports this package.
It is loaded by the tests, by the smoke check and by the benchmark's
CPU-baseline leg, always as the checker and never as the thing measured or
shipped.  Arrays are numpy; halves travel as ``uint16`` bit patterns or
``float16`` views of them.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")

GROUP = 64


def build():
    """Compiles the C restatement (gcc, a second or two)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    return lib


_lib = _load()

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_sz = ctypes.c_size_t
_int = ctypes.c_int
_opt_f32 = ctypes.c_void_p


def _sig(name, res, *args):
    fn = getattr(_lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


_f32_to_f16_array = _sig("orc_f32_to_f16_array", None, _f32p, _sz, _u16p)
_f16_to_f32_array = _sig("orc_f16_to_f32_array", None, _u16p, _sz, _f32p)
_quantize = _sig("orc_quantize", _int, _f32p, _sz, _int, _u32p, _u16p, _u16p)
_dequantize = _sig("orc_dequantize", _int, _u32p, _u16p, _u16p, _sz, _int, _f32p)
_round_trip = _sig("orc_round_trip", _int, _f32p, _sz, _int, _f32p)
_round_trip_as_half = _sig("orc_round_trip_as_half", _int, _f32p, _sz, _int, _f32p)
_softmax = _sig("orc_softmax", None, _f32p, _sz)
_rms_norm = _sig("orc_rms_norm", None, _f32p, _f32p, _sz, ctypes.c_float)
_rope = _sig("orc_rope", None, _f32p, _sz, _sz, ctypes.c_float)
_attend = _sig("orc_attend", _int, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _opt_f32, _sz, _f32p, _int)
_attention_f64 = _sig("orc_attention_f64", _int, _f32p, _f32p, _f32p, _opt_f32, _sz, _sz, _sz, _sz, _f64p, _int)
_rows = _sig("orc_rows", _int, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz, _opt_f32, _f32p, _int)
_rows_f64 = _sig("orc_rows_f64", _int, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz, _opt_f32, _f64p, _int)
_prefill = _sig("orc_prefill", _int, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz, _opt_f32, _f32p, _int)
_layer = _sig(
    "orc_attention_layer", _int, _f32p, _sz, _sz, _sz, _sz, _sz, ctypes.c_float, ctypes.c_float,
    _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _sz, _sz, _int, _f32p)
_dn_conv = _sig("orc_deltanet_conv", None, _f32p, _f32p, _f32p, _sz, _sz, _f32p)
_dn_step = _sig("orc_deltanet_step", None, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p,
                _sz, _sz, _sz, _sz, ctypes.c_float, _f32p)
_dn_layer = _sig("orc_deltanet_layer", None, _f32p, _sz, _sz, _sz, _sz, _sz, _sz, ctypes.c_float, _f32p, _f32p, _f32p,
                 _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p)
_noise = _sig("orc_noise", None, _f32p, _sz, ctypes.c_uint64)
_spread = _sig("orc_spread", None, _u16p, _sz, _sz)
_quant_rows = _sig("orc_quant_rows", None, _f32p, _sz, _sz)


def _c32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"oracle {what}: bad arguments (code {rc})")


# ----------------------------------------------------------------- f16 ----

def f32_to_f16_bits(x):
    x = _c32(x)
    out = np.empty(x.shape, np.uint16)
    _f32_to_f16_array(x.reshape(-1), x.size, out.reshape(-1))
    return out


def f16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    _f16_to_f32_array(h.reshape(-1), h.size, out.reshape(-1))
    return out


# ------------------------------------------------------------ quantizer ----

def words_per_group(bits):
    """KvBits::words_per_group."""
    return 2 * bits


def quantize(x, bits):
    """quantize(): (codes u32, scales u16 bits, biases u16 bits)."""
    x = _c32(x).reshape(-1)
    if x.size % GROUP or bits not in (8, 4):
        raise ValueError("quantize: length must be a multiple of 64 and bits 8 or 4")
    groups = x.size // GROUP
    data = np.empty(groups * words_per_group(bits), np.uint32)
    scales = np.empty(groups, np.uint16)
    biases = np.empty(groups, np.uint16)
    _check(_quantize(x, x.size, bits, data, scales, biases), "quantize")
    return data, scales, biases


def dequantize(data, scales, biases, bits):
    data = np.ascontiguousarray(data, np.uint32).reshape(-1)
    scales = np.ascontiguousarray(scales).view(np.uint16).reshape(-1)
    biases = np.ascontiguousarray(biases).view(np.uint16).reshape(-1)
    out = np.empty(scales.size * GROUP, np.float32)
    _check(_dequantize(data, scales, biases, scales.size, bits, out), "dequantize")
    return out


def round_trip(x, bits):
    x = _c32(x)
    out = np.empty_like(x)
    _check(_round_trip(x.reshape(-1), x.size, bits, out.reshape(-1)), "round_trip")
    return out


def round_trip_as_half(x, bits):
    x = _c32(x)
    out = np.empty_like(x)
    _check(_round_trip_as_half(x.reshape(-1), x.size, bits, out.reshape(-1)), "round_trip_as_half")
    return out


# ------------------------------------------------------------ small ops ----

def softmax(x):
    y = _c32(x).copy()
    _softmax(y, y.size)
    return y


def rms_norm(x, w, eps):
    y = _c32(x).copy()
    _rms_norm(y, _c32(w), y.size, eps)
    return y


def rope(head, dims, pos, theta):
    y = _c32(head).copy()
    _rope(y, dims, pos, theta)
    return y


def attention_prep(q_and_gate, k, v, q_norm, k_norm, heads, kv_heads, dim, rope_dims, pos, theta, eps):
    """What attention_at does to one token before the scores (src/cpu/attention.rs:110-138):
    q and k through rms_norm and rope per head, v as it is.  Returns (q, k, v) as f32
    [heads * dim], [kv_heads * dim], [kv_heads * dim]."""
    qg = _c32(q_and_gate).reshape(heads, 2 * dim)
    q = np.stack([rope(rms_norm(qg[h, :dim], q_norm, eps), rope_dims, pos, theta) for h in range(heads)])
    kk = _c32(k).reshape(kv_heads, dim)
    kk = np.stack([rope(rms_norm(kk[h], k_norm, eps), rope_dims, pos, theta) for h in range(kv_heads)])
    return q.reshape(-1), kk.reshape(-1), _c32(v).reshape(-1).copy()


# ------------------------------------------------------------ attention ----

def _shape(keys, heads, kv_heads, dim):
    keys = _c32(keys)
    return keys.reshape(-1, kv_heads, dim)


def attend(q, keys, values, length, heads=16, kv_heads=2, dim=256, q_and_gate=None, threads=1):
    """One token's attention in f32 as the reference CPU path: out [heads, dim]."""
    q = _c32(q).reshape(heads, dim)
    keys, values = _shape(keys, heads, kv_heads, dim), _shape(values, heads, kv_heads, dim)
    assert keys.shape[0] >= length and values.shape[0] >= length
    out = np.empty((heads, dim), np.float32)
    gate = None
    if q_and_gate is not None:
        q_and_gate = _c32(q_and_gate).reshape(heads, 2 * dim)
        gate = ctypes.c_void_p(q_and_gate.ctypes.data + dim * 4)
    _check(_attend(q, keys, values, length, heads, kv_heads, dim, gate, 2 * dim, out, threads), "attend")
    return out


def attention_f64(q, keys, values, q_and_gate, length, heads=16, kv_heads=2, dim=256, threads=1):
    q = _c32(q).reshape(heads, dim)
    keys, values = _shape(keys, heads, kv_heads, dim), _shape(values, heads, kv_heads, dim)
    assert keys.shape[0] >= length and values.shape[0] >= length
    if q_and_gate is not None:
        q_and_gate = _c32(q_and_gate).reshape(heads, 2 * dim)
    out = np.empty((heads, dim), np.float64)
    _check(_attention_f64(q, keys, values, _ptr(q_and_gate), length, heads, kv_heads, dim, out, threads),
           "attention_f64")
    return out


def rows(q, keys, values, pos, m, heads=16, kv_heads=2, dim=256, q_and_gate=None, threads=1, f64=False):
    """m verify rows: row r sees pos + r + 1 keys."""
    q = _c32(q).reshape(m, heads, dim)
    keys, values = _shape(keys, heads, kv_heads, dim), _shape(values, heads, kv_heads, dim)
    assert keys.shape[0] >= pos + m
    if q_and_gate is not None:
        q_and_gate = _c32(q_and_gate).reshape(m, heads, 2 * dim)
    out = np.empty((m, heads, dim), np.float64 if f64 else np.float32)
    fn = _rows_f64 if f64 else _rows
    _check(fn(q, keys, values, pos, m, heads, kv_heads, dim, _ptr(q_and_gate), out, threads), "rows")
    return out


def prefill(q, keys, values, pos, tokens, heads=16, kv_heads=2, dim=256, q_and_gate=None, threads=1):
    """A causal chunk: token i sees keys 0 ..= pos + i."""
    q = _c32(q).reshape(tokens, heads, dim)
    keys, values = _shape(keys, heads, kv_heads, dim), _shape(values, heads, kv_heads, dim)
    assert keys.shape[0] >= pos + tokens
    if q_and_gate is not None:
        q_and_gate = _c32(q_and_gate).reshape(tokens, heads, 2 * dim)
    out = np.empty((tokens, heads, dim), np.float32)
    _check(_prefill(q, keys, values, pos, tokens, heads, kv_heads, dim, _ptr(q_and_gate), out, threads),
           "prefill")
    return out


class AttentionLayer:
    """attention_at over a growing f32 cache, dense projections."""

    def __init__(self, cfg, weights, capacity=64, rounding=0):
        self.cfg = cfg
        self.w = {k: _c32(v).reshape(-1) for k, v in weights.items()}
        kvw = cfg["kv_heads"] * cfg["head_dim"]
        self.keys = np.zeros((capacity, kvw), np.float32)
        self.values = np.zeros((capacity, kvw), np.float32)
        self.len = 0
        self.rounding = rounding

    def step(self, x, pos=None):
        c, w = self.cfg, self.w
        x = _c32(x).reshape(-1)
        out = np.empty(c["hidden"], np.float32)
        rc = _layer(x, c["hidden"], c["heads"], c["kv_heads"], c["head_dim"], c["rope_dims"],
                    c["rope_theta"], c["eps"], w["q_proj"], w["k_proj"], w["v_proj"], w["o_proj"],
                    w["q_norm"], w["k_norm"], self.keys.reshape(-1), self.values.reshape(-1),
                    self.len, self.len if pos is None else pos, self.rounding, out)
        _check(rc, "attention_layer")
        self.len += 1
        return out


# ------------------------------------------------------------ Gated DeltaNet ----

def deltanet_conv(weight, x, state, kernel):
    """conv_step (src/cpu/deltanet.rs:117-131).  state [kernel-1][channels] is updated in place
    (pass a contiguous f32 array); returns the mixed, SiLU'd channels."""
    x = _c32(x).reshape(-1)
    assert state.dtype == np.float32 and state.flags.c_contiguous
    out = np.empty_like(x)
    _dn_conv(_c32(weight).reshape(-1), x, state.reshape(-1), x.size, kernel, out)
    return out


def deltanet_step(q, k, v, a, b, a_log, dt_bias, state, z, norm, k_heads, v_heads, k_dim, v_dim, eps):
    """normalize_qk, the gates, delta_rule and the gated RMSNorm (src/cpu/deltanet.rs:86-112,133-155).
    state [v_heads][v_dim][k_dim] is updated in place; returns y [v_heads * v_dim]."""
    assert state.dtype == np.float32 and state.flags.c_contiguous
    y = np.empty(v_heads * v_dim, np.float32)
    _dn_step(_c32(q).reshape(-1), _c32(k).reshape(-1), _c32(v).reshape(-1), _c32(a), _c32(b), _c32(a_log),
             _c32(dt_bias), state.reshape(-1), _c32(z).reshape(-1), _c32(norm), k_heads, v_heads, k_dim, v_dim, eps, y)
    return y


class DeltaNetLayer:
    """deltanet (src/cpu/deltanet.rs:69-114) with dense projections, state kept between tokens."""

    def __init__(self, cfg, weights):
        self.cfg = cfg
        self.w = {k: _c32(v).reshape(-1) for k, v in weights.items()}
        conv = 2 * cfg["k_heads"] * cfg["k_dim"] + cfg["v_heads"] * cfg["v_dim"]
        self.conv = np.zeros((cfg["kernel"] - 1) * conv, np.float32)
        self.recurrent = np.zeros(cfg["v_heads"] * cfg["v_dim"] * cfg["k_dim"], np.float32)

    def step(self, x):
        c, w = self.cfg, self.w
        out = np.empty(c["hidden"], np.float32)
        _dn_layer(_c32(x).reshape(-1), c["hidden"], c["k_heads"], c["v_heads"], c["k_dim"], c["v_dim"], c["kernel"],
                  c["eps"], w["in_proj_qkv"], w["in_proj_z"], w["in_proj_b"], w["in_proj_a"], w["out_proj"],
                  w["conv1d"], w["A_log"], w["dt_bias"], w["norm"], self.conv, self.recurrent, out)
        return out


# --------------------------------------------------- the reference's inputs ----

def noise(n, seed):
    out = np.empty(n, np.float32)
    _noise(out, n, seed)
    return out


def spread(n, seed):
    """Halves in about -2 .. 2, returned as float16."""
    out = np.empty(n, np.uint16)
    _spread(out, n, seed)
    return out.view(np.float16)


def quant_rows(tokens, values=512):
    out = np.empty(tokens * values, np.float32)
    _quant_rows(out, tokens, values)
    return out


def rel_rms(got, want):
    """sqrt(sum (g - w)^2 / sum w^2), the reference's rel_rms (src/gpu_verify.rs:374-378)."""
    got = np.asarray(got, np.float64).reshape(-1)
    want = np.asarray(want, np.float64).reshape(-1)
    return float(np.sqrt(((got - want) ** 2).sum() / (want ** 2).sum()))
