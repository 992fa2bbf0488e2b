"""ctypes binding of include/saetta_hip.h.  One function per exported symbol."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SAETTA_HIP_LIB") or os.path.join(_HERE, "lib", "libsaetta_hip.so")

# Every symbol include/saetta_hip.h declares; tests check the library exports each.
SYMBOLS = [
    "saetta_init", "saetta_last_error", "saetta_device_status", "saetta_kv_quantize", "saetta_kv_dequantize", "saetta_kv_dequantize_f32", "saetta_to_half", "saetta_attn_prep_store", "saetta_deltanet_conv", "saetta_deltanet_step", "saetta_deltanet_conv_rows", "saetta_deltanet_rows", "saetta_deltanet_rows_ws", "saetta_deltanet_rows_workspace_bytes", "saetta_deltanet_token", "saetta_deltanet_rows_fused",
    "saetta_part_o_bytes", "saetta_part_ml_bytes", "saetta_attn_decode", "saetta_attn_decode_quant",
    "saetta_attn_rows", "saetta_attn_rows_quant", "saetta_static_scratch_bytes", "saetta_attn_decode_quant_static", "saetta_prefill_workspace_bytes", "saetta_attn_prefill", "saetta_attn_prefill_quant",
    "saetta_attn_gemm_workspace_bytes", "saetta_attn_gemm",
]

STAGE_PARTIAL, STAGE_REDUCE, STAGE_ALL, STAGE_NO_LOADERS = 1, 2, 3, 4


class TokenParamsC(ctypes.Structure):
    _fields_ = [("token", ctypes.c_uint32), ("position", ctypes.c_uint32), ("kv_len", ctypes.c_uint32),
                ("pad", ctypes.c_uint32)]


class KvQuantParamsC(ctypes.Structure):
    _fields_ = [("groups", ctypes.c_uint32), ("per_token", ctypes.c_uint32)]


class DecodeParamsC(ctypes.Structure):
    _fields_ = [("heads", ctypes.c_uint32), ("kv_heads", ctypes.c_uint32), ("capacity", ctypes.c_uint32),
                ("scale", ctypes.c_float)]


class RowsParamsC(ctypes.Structure):
    _fields_ = [("heads", ctypes.c_uint32), ("kv_heads", ctypes.c_uint32), ("capacity", ctypes.c_uint32),
                ("scale", ctypes.c_float), ("rows", ctypes.c_uint32), ("splits", ctypes.c_uint32)]


class FlashParamsC(ctypes.Structure):
    _fields_ = [("heads", ctypes.c_uint32), ("kv_heads", ctypes.c_uint32), ("pos", ctypes.c_uint32),
                ("tokens", ctypes.c_uint32), ("scale", ctypes.c_float)]


class QuantRowsC(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("scales", ctypes.c_void_p), ("biases", ctypes.c_void_p)]


class SaettaError(RuntimeError):
    """A non-zero return of the C ABI (the reference panics in these places)."""


_lib = None


def lib():
    """Loads the library on first use; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SaettaError(f"{LIB_PATH} is missing: run __graft_entry__.build() (make -C csrc)")
        l = ctypes.CDLL(LIB_PATH)
        vp, u32, i32, sz = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int, ctypes.c_size_t
        l.saetta_init.restype, l.saetta_init.argtypes = i32, []
        l.saetta_last_error.restype, l.saetta_last_error.argtypes = ctypes.c_char_p, []
        l.saetta_device_status.restype, l.saetta_device_status.argtypes = u32, [i32]
        l.saetta_kv_quantize.restype = i32
        l.saetta_kv_quantize.argtypes = [vp, i32, vp, QuantRowsC, KvQuantParamsC, vp, u32]
        l.saetta_kv_dequantize.restype = i32
        l.saetta_kv_dequantize.argtypes = [vp, i32, QuantRowsC, vp, KvQuantParamsC]
        l.saetta_kv_dequantize_f32.restype = i32
        l.saetta_kv_dequantize_f32.argtypes = [vp, i32, QuantRowsC, vp, KvQuantParamsC]
        l.saetta_to_half.restype, l.saetta_to_half.argtypes = i32, [vp, vp, vp, sz]
        l.saetta_deltanet_conv.restype = i32
        l.saetta_deltanet_conv.argtypes = [vp, vp, vp, vp, vp, ConvParamsC]
        l.saetta_deltanet_step.restype = i32
        l.saetta_deltanet_step.argtypes = [vp] * 12 + [StepParamsC]
        l.saetta_deltanet_token.restype = i32
        l.saetta_deltanet_token.argtypes = [vp] * 12 + [ConvParamsC, StepParamsC]
        l.saetta_deltanet_rows_fused.restype = i32
        l.saetta_deltanet_rows_fused.argtypes = [vp] * 14 + [RowsFusedParamsC]
        l.saetta_deltanet_conv_rows.restype = i32
        l.saetta_deltanet_conv_rows.argtypes = [vp] * 6 + [ConvRowsParamsC]
        l.saetta_deltanet_rows.restype = i32
        l.saetta_deltanet_rows.argtypes = [vp] * 11 + [RowsStepParamsC]
        l.saetta_deltanet_rows_ws.restype = i32
        l.saetta_deltanet_rows_ws.argtypes = [vp] * 11 + [RowsStepParamsC, vp, ctypes.c_size_t]
        l.saetta_deltanet_rows_workspace_bytes.restype = ctypes.c_size_t
        l.saetta_deltanet_rows_workspace_bytes.argtypes = [RowsStepParamsC]
        l.saetta_attn_prep_store.restype = i32
        l.saetta_attn_prep_store.argtypes = [vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, QuantRowsC, QuantRowsC, vp,
                                             PrepParamsC, u32, u32, vp]
        l.saetta_part_o_bytes.restype, l.saetta_part_o_bytes.argtypes = sz, [u32, u32, u32]
        l.saetta_part_ml_bytes.restype, l.saetta_part_ml_bytes.argtypes = sz, [u32, u32, u32]
        l.saetta_attn_decode.restype = i32
        l.saetta_attn_decode.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, DecodeParamsC, vp, u32]
        l.saetta_attn_decode_quant.restype = i32
        l.saetta_attn_decode_quant.argtypes = [vp, i32, vp, QuantRowsC, QuantRowsC, vp, vp, vp, vp,
                                               DecodeParamsC, vp, u32]
        l.saetta_static_scratch_bytes.restype, l.saetta_static_scratch_bytes.argtypes = sz, []
        l.saetta_attn_decode_quant_static.restype = i32
        l.saetta_attn_decode_quant_static.argtypes = [vp, i32, vp, QuantRowsC, QuantRowsC, vp, vp, DecodeParamsC, vp, u32]
        l.saetta_attn_rows.restype = i32
        l.saetta_attn_rows.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, RowsParamsC, vp, u32]
        l.saetta_attn_rows_quant.restype = i32
        l.saetta_attn_rows_quant.argtypes = [vp, i32, vp, QuantRowsC, QuantRowsC, vp, vp, vp, vp,
                                             RowsParamsC, vp, u32]
        l.saetta_attn_prefill.restype = i32
        l.saetta_attn_prefill.argtypes = [vp, vp, vp, vp, vp, vp, FlashParamsC, vp, ctypes.c_size_t]
        l.saetta_prefill_workspace_bytes.restype = ctypes.c_size_t
        l.saetta_prefill_workspace_bytes.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]
        l.saetta_attn_prefill_quant.restype = i32
        l.saetta_attn_prefill_quant.argtypes = [vp, i32, vp, QuantRowsC, QuantRowsC, vp, vp, FlashParamsC, vp,
                                                ctypes.c_size_t]
        l.saetta_attn_gemm_workspace_bytes.restype = ctypes.c_size_t
        l.saetta_attn_gemm_workspace_bytes.argtypes = [ctypes.c_uint32] * 4
        l.saetta_attn_gemm.restype = i32
        l.saetta_attn_gemm.argtypes = [vp, i32, vp, QuantRowsC, QuantRowsC, vp, vp, FlashParamsC, u32, u32, vp,
                                       ctypes.c_size_t]
        _lib = l
    return _lib


class PrepParamsC(ctypes.Structure):
    _fields_ = [("heads", ctypes.c_uint32), ("kv_heads", ctypes.c_uint32), ("dim", ctypes.c_uint32),
                ("half_dims", ctypes.c_uint32), ("log2_theta", ctypes.c_float), ("eps", ctypes.c_float)]


class ConvParamsC(ctypes.Structure):
    _fields_ = [("channels", ctypes.c_uint32), ("kernel_size", ctypes.c_uint32)]


class StepParamsC(ctypes.Structure):
    _fields_ = [("k_heads", ctypes.c_uint32), ("v_heads", ctypes.c_uint32), ("v_dim", ctypes.c_uint32),
                ("eps", ctypes.c_float)]


class ConvRowsParamsC(ctypes.Structure):
    _fields_ = [("channels", ctypes.c_uint32), ("kernel_size", ctypes.c_uint32), ("tokens", ctypes.c_uint32),
                ("snapshots", ctypes.c_uint32)]


class RowsStepParamsC(ctypes.Structure):
    _fields_ = [("k_heads", ctypes.c_uint32), ("v_heads", ctypes.c_uint32), ("v_dim", ctypes.c_uint32),
                ("tokens", ctypes.c_uint32), ("eps", ctypes.c_float), ("snapshots", ctypes.c_uint32)]


class RowsFusedParamsC(ctypes.Structure):
    _fields_ = [("k_heads", ctypes.c_uint32), ("v_heads", ctypes.c_uint32), ("v_dim", ctypes.c_uint32),
                ("kernel_size", ctypes.c_uint32), ("eps", ctypes.c_float), ("rows", ctypes.c_uint32),
                ("snapshots", ctypes.c_uint32)]


def check(rc, what):
    if rc != 0:
        msg = lib().saetta_last_error().decode()
        raise SaettaError(f"{what}: {msg} (code {rc})")
