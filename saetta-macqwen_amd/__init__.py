"""MI355X (gfx950) attention hot path of saetta: Python front end.

The product is ``lib/libsaetta_hip.so`` (hand-written HIP kernels behind the
C ABI of ``include/saetta_hip.h``).  This package binds that ABI with ctypes
and mirrors, name for name, the host-side objects the reference keeps in
``src/kv_quant.rs``, ``src/attention.rs``, ``src/rows.rs`` and
``src/attention_prefill.rs``.  torch is used only to own device memory and
streams.  There is no CPU fallback: importing works anywhere (so the build can
be checked), every call needs the library and a gfx950 device.
"""
from . import ffi
from .host import (GROUP, KV_ALIGN, MAX_ROWS, AttentionRows, Built, DecodeAttention, FlashParams, GpuKvCache, KvBits,
                   Plan, RowBackup,
                   PrepParams, QuantRows, TokenParams, attention_gemm, attention_prefill, bench, deltanet_conv, deltanet_conv_rows, deltanet_rows, deltanet_rows_fused, deltanet_token,
                   deltanet_step, dequantize, device_status, quantize, round_trip,
                   record_store, round_trip_as_half, test_slack, to_half)

__all__ = ["ffi", "GROUP", "KV_ALIGN", "MAX_ROWS", "AttentionRows", "Built", "DecodeAttention", "FlashParams",
           "GpuKvCache", "KvBits", "RowBackup",
           "Plan", "PrepParams", "QuantRows", "TokenParams", "attention_gemm", "attention_prefill", "bench", "deltanet_conv", "deltanet_conv_rows",
           "deltanet_rows", "deltanet_rows_fused", "deltanet_token", "deltanet_step", "dequantize", "device_status", "quantize",
           "record_store", "round_trip", "round_trip_as_half", "test_slack", "to_half"]
