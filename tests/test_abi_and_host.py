"""CPU-only checks: the C ABI library loads and exports every symbol the header declares,
the parameter blocks have the reference's layout, arguments are rejected with clear errors,
and the host-side mirror of the reference's types behaves as the reference's do.  Nothing
here computes on a GPU; on a box without one the library must refuse to run, loudly."""
import ctypes
import os
import re
import subprocess

import pytest

import __graft_entry__ as entry

saetta = entry.load_package()
ffi = saetta.ffi
ROOT = entry.ROOT


def header_functions():
    text = open(os.path.join(ROOT, "include", "saetta_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(saetta_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(ffi.LIB_PATH), "build the library first: python __graft_entry__.py"
    declared = header_functions()
    assert declared == sorted(ffi.SYMBOLS)
    out = subprocess.run(["nm", "-D", "--defined-only", ffi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = set(re.findall(r" T (saetta_[a-z0-9_]+)", out))
    assert set(declared) <= exported
    lib = ctypes.CDLL(ffi.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name)


def test_header_is_plain_c():
    # The boundary is a C ABI: the header must compile as C99 on its own (a Rust, Go or C binding reads it).
    header = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "saetta_hip.h")
    done = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", header],
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    # ... and the parameter blocks the mirrors build by hand have the sizes the compiler gives them
    probe = ('#include "%s"\n#include <stdio.h>\nint main(void) { printf("%%zu %%zu %%zu %%zu %%zu\\n", '
             'sizeof(saetta_rows_fused_params), sizeof(saetta_rows_step_params), sizeof(saetta_conv_rows_params), '
             'sizeof(saetta_step_params), sizeof(saetta_conv_params)); return 0; }\n') % header
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        src, exe = os.path.join(d, "probe.c"), os.path.join(d, "probe")
        with open(src, "w") as f:
            f.write(probe)
        subprocess.run(["gcc", "-std=c99", src, "-o", exe], check=True)
        sizes = [int(x) for x in subprocess.run([exe], capture_output=True, text=True, check=True).stdout.split()]
    assert sizes == [ctypes.sizeof(ffi.RowsFusedParamsC), ctypes.sizeof(ffi.RowsStepParamsC), ctypes.sizeof(ffi.ConvRowsParamsC),
                     ctypes.sizeof(ffi.StepParamsC), ctypes.sizeof(ffi.ConvParamsC)]


def test_parameter_blocks_match_the_reference_layout():
    # TokenParams (src/plan.rs:16-35) is 4 x u32; DecodeParams 3 x u32 + f32 (src/attention.rs:19-26);
    # RowsAttentionParams adds rows, splits (src/rows.rs:307-317); FlashParams 4 x u32 + f32
    # (src/attention_prefill.rs:4-14); KvQuantParams 2 x u32 (src/kv_quant.rs:147-153).
    assert ctypes.sizeof(ffi.TokenParamsC) == 16
    assert ctypes.sizeof(ffi.DecodeParamsC) == 16 and ffi.DecodeParamsC.scale.offset == 12
    assert ctypes.sizeof(ffi.RowsParamsC) == 24 and ffi.RowsParamsC.rows.offset == 16
    assert ctypes.sizeof(ffi.FlashParamsC) == 20 and ffi.FlashParamsC.scale.offset == 16
    assert ctypes.sizeof(ffi.KvQuantParamsC) == 8
    assert ctypes.sizeof(ffi.QuantRowsC) == 24


def test_scratch_sizes_never_exceed_the_reference():
    lib = ffi.lib()
    for capacity in (1, 100, 128, 1024, 32896, 150016, 262144):
        chunks = -(-capacity // 128)
        for rows in (1, 4, 8):
            assert lib.saetta_part_o_bytes(16, capacity, rows) <= rows * chunks * 16 * 256 * 4
            assert lib.saetta_part_ml_bytes(16, capacity, rows) <= rows * chunks * 16 * 2 * 4
            assert lib.saetta_part_o_bytes(16, capacity, rows) == 128 * lib.saetta_part_ml_bytes(16, capacity, rows)


def test_bad_arguments_are_rejected_before_any_launch():
    lib = ffi.lib()
    rows = ffi.QuantRowsC(16, 16, 16)
    p = ffi.KvQuantParamsC(8, 8)
    assert lib.saetta_kv_quantize(None, 5, 16, rows, p, None, 0) == -1  # SAETTA_E_BITS
    assert b"bits 5" in lib.saetta_last_error()
    assert lib.saetta_kv_quantize(None, 8, None, rows, p, None, 0) == -3  # SAETTA_E_NULL
    assert lib.saetta_kv_quantize(None, 8, 12, rows, p, None, 0) == -4  # x not 16-byte aligned
    dp = ffi.DecodeParamsC(16, 4, 1024, 0.0625)
    assert lib.saetta_attn_decode_quant(None, 8, 16, rows, rows, 16, 16, 16, 16, dp, 16, 3) == -2
    assert b"8 q heads per kv head" in lib.saetta_last_error()
    rp = ffi.RowsParamsC(16, 2, 1024, 0.0625, 9, 8)
    assert lib.saetta_attn_rows_quant(None, 8, 16, rows, rows, 16, 16, 16, 16, rp, 16, 3) == -2
    assert b"9 rows" in lib.saetta_last_error()
    odd = ffi.DecodeParamsC(16, 2, 1000, 0.0625)
    assert lib.saetta_attn_decode_quant(None, 8, 16, rows, rows, 16, 16, 16, 16, odd, 16, 3) == -2
    assert b"multiple of 16" in lib.saetta_last_error()
    # Gated DeltaNet: heads must divide, v_dim a multiple of 4 for several tokens, snapshots need a buffer
    sp = ffi.RowsStepParamsC(2, 3, 8, 1, 1e-6, 0)
    assert lib.saetta_deltanet_rows(None, *([16] * 9), None, sp) == -2
    assert b"value heads" in lib.saetta_last_error()
    sp = ffi.RowsStepParamsC(1, 2, 6, 1, 1e-6, 0)
    assert lib.saetta_deltanet_rows(None, *([16] * 9), None, sp) == -2
    sp = ffi.RowsStepParamsC(1, 2, 8, 1, 1e-6, 1)
    assert lib.saetta_deltanet_rows(None, *([16] * 9), None, sp) == -3  # snapshots asked for, no buffer
    cp = ffi.ConvRowsParamsC(64, 1, 4, 0)
    assert lib.saetta_deltanet_conv_rows(None, 16, 16, 16, 16, None, cp) == -2
    assert b"kernel size" in lib.saetta_last_error()
    # ... the fused call takes up to 8 rows, conv kernels of 2..16 taps, and both snapshot buffers or neither
    fused = ffi.RowsFusedParamsC(1, 2, 8, 4, 1e-6, 9, 0)
    assert lib.saetta_deltanet_rows_fused(None, *([16] * 11), None, None, fused) == -2
    assert b"9 rows" in lib.saetta_last_error()
    fused = ffi.RowsFusedParamsC(1, 2, 8, 17, 1e-6, 2, 0)
    assert lib.saetta_deltanet_rows_fused(None, *([16] * 11), None, None, fused) == -2
    assert b"kernel size" in lib.saetta_last_error()
    fused = ffi.RowsFusedParamsC(1, 2, 8, 4, 1e-6, 2, 1)
    assert lib.saetta_deltanet_rows_fused(None, *([16] * 11), 16, None, fused) == -3
    fused = ffi.RowsFusedParamsC(1, 2, 8, 4, 1e-6, 2, 0)
    assert lib.saetta_deltanet_rows_fused(None, *([16] * 7), 12, *([16] * 3), None, None, fused) == -4  # the state's alignment
    token_c, token_s = ffi.ConvParamsC(100, 4), ffi.StepParamsC(1, 2, 8, 1e-6)
    assert lib.saetta_deltanet_token(None, *([16] * 11), token_c, token_s) == -2
    assert b"channels" in lib.saetta_last_error()
    fp = ffi.FlashParamsC(16, 2, 0, 1, 0.0625)
    assert lib.saetta_attn_prefill_quant(None, 16, 16, rows, rows, 16, 16, fp, None, 0) == -1
    assert lib.saetta_attn_prefill_quant(None, 8, 16, rows, rows, 16, 16, fp, 8, 1 << 30) == -4  # workspace alignment
    # 32 keys per image, one image per kv head and block, whole kilobytes each; behind them a 256-byte line
    # (the attention kernel's count of tiles handed out)
    one = lib.saetta_prefill_workspace_bytes(0, 32, 1) - 256
    assert one % 1024 == 0 and one >= 2 * 32 * 256 * 2
    assert lib.saetta_prefill_workspace_bytes(4096, 4096, 2) == one * 2 * 256 + 256
    assert lib.saetta_prefill_workspace_bytes(0, 33, 1) == 2 * one + 256
    with pytest.raises(ffi.SaettaError):
        ffi.check(-1, "demo")


def test_without_a_gpu_the_library_refuses_to_run():
    import torch
    if torch.cuda.is_available():
        pytest.skip("this box has a GPU")
    rc = ffi.lib().saetta_init()
    assert rc == -5  # SAETTA_E_DEVICE: there is no CPU fallback
    assert ffi.lib().saetta_last_error()


def test_kv_bits_mirror():
    # src/kv_quant.rs:11-50
    K = saetta.KvBits
    assert K.parse("16") is K.Half and K.parse("8") is K.Eight and K.parse("4") is K.Four and K.parse("2") is None
    assert [k.bits() for k in (K.Half, K.Eight, K.Four)] == [16, 8, 4]
    assert K.Eight.words_per_group() == 16 and K.Four.words_per_group() == 8
    assert K.Half.bytes_per_value() == 2.0
    assert K.Eight.bytes_per_value() == 1.0 + 4.0 / 64 and K.Four.bytes_per_value() == 0.5 + 4.0 / 64
    # bytes per token and kv head of 256: 272 at 8 bits, 144 at 4 (src/kv_quant.rs:3-4)
    assert K.Eight.bytes_per_value() * 256 == 272 and K.Four.bytes_per_value() * 256 == 144
    assert saetta.GROUP == 64 and saetta.MAX_ROWS == 8


def test_token_params_and_prefill_constants():
    tp = saetta.TokenParams(7, 41)
    assert (tp.token, tp.position, tp.kv_len, tp.pad) == (7, 41, 42, 0)  # src/plan.rs:26-34
    ap = saetta.attention_prefill
    assert ap.KERNELS == ["attention_fa8", "attention_fa4"] and ap.DEFAULT == "attention_fa8" and ap.KEY_BLOCK == 16
    p = saetta.FlashParams(16, 2, 5, 8, 0.0625).c()
    assert (p.heads, p.kv_heads, p.pos, p.tokens) == (16, 2, 5, 8)


def test_plan_records_and_filters_ops_without_a_device():
    plan = saetta.Plan.__new__(saetta.Plan)  # no device buffer: only the op list is exercised
    plan.ops = []
    ran = []
    plan.op("attention_partial_mma_q8", lambda s: ran.append("partial"))
    plan.op("attention_reduce", lambda s: ran.append("reduce"))
    built = plan.build_where(lambda name: name == "attention_reduce")
    assert [k for k, _ in built.ops] == ["attention_reduce"]
    assert [k for k, _ in plan.build().ops] == ["attention_partial_mma_q8", "attention_reduce"]
