"""Prefill attention as matrix products over blocks of 1024 keys (AttGemm, src/attention_gemm.rs) against
the oracle's token-by-token f32 CPU attention, to the bar of the flash kernel's tests (finite, max abs
diff < 2e-3 as tests/attention_prefill.rs:56-59, rel-RMS <= 1e-3), and against the flash kernel on the
same buffers, which is what the reference's own check of this path prints (src/attention_gemm.rs:451-467).
The reference holds no other test of it.  Shapes: the flash tests' and ones whose keys cross blocks of
1024, spans of eight blocks and whose tokens cross slices.
"""
import math

import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, dev, host, oracle, saetta
from test_gpu_prefill import KINDS, MAX_ABS, REL_RMS, make_cache, run as run_flash

pytestmark = pytest.mark.gpu
# (the last three cross spans of eight blocks, 8192 keys, which is what a pair of launches takes)
SHAPES = [(0, 1), (0, 7), (5, 8), (70, 100), (1000, 64), (0, 300), (4093, 37), (1020, 40), (2047, 2), (1024, 33),
          (990, 1100), (8100, 200), (8191, 2), (16380, 40)]


def run(kind, q16, kc, vc, qg, pos, tokens, chunk=None, stages=0, fill=float("nan")):
    if not torch.is_tensor(q16):
        q16, qg = dev(q16), dev(qg)
    out = torch.full((tokens, H, D), fill, device="cuda")
    p = saetta.FlashParams(H, KV, pos, tokens, 1.0 / math.sqrt(D))
    gemm = saetta.attention_gemm.AttGemm(chunk or tokens, KV)
    gemm.stages = stages
    if kind is saetta.KvBits.Half:
        gemm.encode(q16, kc, vc, None, qg, out, p)
    else:
        gemm.encode(q16, None, None, (kc, vc), qg, out, p)
    return host(out)


def spread_case(pos, tokens):
    n = pos + tokens
    q16 = oracle.spread(tokens * H * D, 1).reshape(tokens, H, D)
    k = oracle.spread(n * VALUES, 2).astype(np.float32).reshape(n, VALUES)
    v = oracle.spread(n * VALUES, 3).astype(np.float32).reshape(n, VALUES)
    qg = ((np.arange(tokens * H * 2 * D) % 7) - 3).astype(np.float32).reshape(tokens, H, 2 * D)
    return q16, k, v, qg


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("pos,tokens", SHAPES)
def test_matches_cpu_on_spread_data(kind, pos, tokens):
    n = pos + tokens
    q16, k, v, qg = spread_case(pos, tokens)
    kc, vc, kf, vf = make_cache(kind, k, v, -(-n // 64) * 64 + 64, chunk_from=pos)
    got = run(kind, q16, kc, vc, qg, pos, tokens)
    want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < MAX_ABS, f"{kind} pos {pos} tokens {tokens}"
    assert oracle.rel_rms(got, want) < REL_RMS


@pytest.mark.parametrize("slices", [1, 2, 3, 7])
@pytest.mark.parametrize("kind", KINDS)
def test_gaussian_chunk_in_slices(kind, slices, monkeypatch):
    # SAETTA_AG_SLICES (src/attention_gemm.rs:83-89): the chunk's tokens in that many slices, one after the
    # other through the same scratch; 1100 keys: two blocks, the second one ragged.
    monkeypatch.setenv("SAETTA_AG_SLICES", str(slices))
    rng = np.random.default_rng(40 + slices)
    pos, tokens = 870, 230
    n = pos + tokens
    q16 = rng.standard_normal((tokens, H, D)).astype(np.float16)
    k = (rng.standard_normal((n, VALUES)) * 2.0).astype(np.float32)
    v = rng.standard_normal((n, VALUES)).astype(np.float32)
    qg = rng.standard_normal((tokens, H, 2 * D)).astype(np.float32)
    kc, vc, kf, vf = make_cache(kind, k, v, n, chunk_from=pos)
    assert saetta.attention_gemm.AttGemm(tokens, KV).slice == -(-tokens // slices)
    got = run(kind, q16, kc, vc, qg, pos, tokens)
    want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
    assert np.abs(got - want).max() < MAX_ABS and oracle.rel_rms(got, want) < REL_RMS
    # a chunk shorter than the one the buffers were made for
    got = run(kind, q16[:100], kc, vc, qg[:100], pos, 100, chunk=tokens)
    assert np.abs(got - want[:100]).max() < MAX_ABS


def test_equal_keys_give_running_means():
    # A closed form for every row: with the same key in every cache row all scores of a token are equal, so
    # token i's output is the mean of the first pos + i + 1 value rows times sigmoid(gate), whatever q is.  A
    # tile of keys skipped, taken twice or masked at the wrong place, a block folded in with the wrong factor
    # or a slice at the wrong position moves it.  5000 keys: five blocks, the chunk's tokens across two of them.
    pos, tokens = 3000, 2000
    n = pos + tokens
    gen = torch.Generator(device="cuda").manual_seed(23)
    krow = torch.randn(VALUES, generator=gen, device="cuda") * 2.0
    kc = krow.repeat(n, 1).to(torch.float16).contiguous()
    vx = torch.randn(n, VALUES, generator=gen, device="cuda")
    vx[:, 7] += 2.0
    vc = vx.to(torch.float16)
    q16 = torch.randn(tokens, H, D, generator=gen, device="cuda").to(torch.float16)
    qg = torch.randn(tokens, H, 2 * D, generator=gen, device="cuda")
    got = run(saetta.KvBits.Half, q16, kc, vc, qg, pos, tokens)
    vf = host(vc).astype(np.float64)
    sums = np.cumsum(vf[pos:], axis=0) + vf[:pos].sum(axis=0)
    means = (sums / (pos + 1 + np.arange(tokens))[:, None]).reshape(tokens, KV, D)
    gate = 1.0 / (1.0 + np.exp(-host(qg).reshape(tokens, H, 2 * D)[:, :, D:].astype(np.float64)))
    want = np.repeat(means, H // KV, axis=1) * gate
    # the probabilities are f16 here (all equal to 1 before the division: exact), the values' sums f32
    assert np.abs(got - want).max() < 2e-5


@pytest.mark.parametrize("kind", [saetta.KvBits.Eight, saetta.KvBits.Four])
def test_full_size_chunk_against_the_flash_kernel(kind):
    # The 4096-token chunk at position 4096 over codes: every output against the flash kernel's on the same
    # buffers (the check the reference's bench prints, src/attention_gemm.rs:451-467).
    pos = tokens = 4096
    n = pos + tokens
    gen = torch.Generator(device="cuda").manual_seed(9)
    kx = torch.randn(n, VALUES, generator=gen, device="cuda")
    vx = torch.randn(n, VALUES, generator=gen, device="cuda")
    q16 = torch.randn(tokens, H, D, generator=gen, device="cuda").to(torch.float16)
    qg = torch.randn(tokens, H, 2 * D, generator=gen, device="cuda")
    kc, vc = saetta.QuantRows(kind, VALUES, n), saetta.QuantRows(kind, VALUES, n)
    kc.encode(kx.view(-1), 0, n), vc.encode(vx.view(-1), 0, n)
    want = run_flash(kind, host(q16), kc, vc, host(qg), pos, tokens)
    got = run(kind, q16, kc, vc, qg, pos, tokens)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < MAX_ABS
    assert oracle.rel_rms(got, want) < REL_RMS


def test_stages_stop_early_and_write_no_outputs():
    # AttGemm::stages (src/attention_gemm.rs:112-114, 296-327): the passes of a block one by one for the
    # bench; a run that stops early leaves `out` alone.
    pos, tokens = 100, 40
    q16, k, v, qg = spread_case(pos, tokens)
    kc, vc, _, _ = make_cache(saetta.KvBits.Eight, k, v, 192)
    for stages in (1, 2, 3):
        got = run(saetta.KvBits.Eight, q16, kc, vc, qg, pos, tokens, stages=stages, fill=7.0)
        assert (got == 7.0).all(), stages


def test_rejections(monkeypatch):
    pos, tokens = 10, 20
    q16, k, v, qg = spread_case(pos, tokens)
    kc, vc, _, _ = make_cache(saetta.KvBits.Half, k, v, 64)
    gemm = saetta.attention_gemm.AttGemm(tokens, KV)
    out = torch.zeros(tokens, H, D, device="cuda")
    with pytest.raises(ValueError, match="8 q heads"):
        gemm.encode(dev(q16), kc, vc, None, dev(qg), out, saetta.FlashParams(H, 4, pos, tokens, 1.0))
    with pytest.raises(ValueError, match="chunks of"):
        gemm.encode(dev(q16), kc, vc, None, dev(qg), out, saetta.FlashParams(H, KV, pos, tokens + 1, 1.0))
    monkeypatch.setenv("SAETTA_AG_FUSED", "0")
    with pytest.raises(ValueError, match="fused"):
        saetta.attention_gemm.AttGemm(tokens, KV)
    monkeypatch.delenv("SAETTA_AG_FUSED")
    # through the C ABI: a workspace too small, a stage that does not exist
    lib, ffi = saetta.ffi.lib(), saetta.ffi
    p = saetta.FlashParams(H, KV, pos, tokens, 1.0)
    need = lib.saetta_attn_gemm_workspace_bytes(pos, tokens, 0, KV)
    assert need > lib.saetta_prefill_workspace_bytes(pos, tokens, KV)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    rows = lambda t: ffi.QuantRowsC(t.data_ptr(), None, None)  # noqa: E731
    args = (None, 16, dev(q16).data_ptr(), rows(kc), rows(vc), dev(qg).data_ptr(), out.data_ptr(), p.c())
    assert lib.saetta_attn_gemm(*args, 0, 0, ws.data_ptr(), need - 1) != 0
    assert "workspace" in lib.saetta_last_error().decode()
    assert lib.saetta_attn_gemm(*args, 0, 4, ws.data_ptr(), need) != 0
    assert "stages" in lib.saetta_last_error().decode()
    assert lib.saetta_attn_gemm(*args, 0, 0, ws.data_ptr(), need) == 0
    want = host(out).copy()
    # no workspace: the library's own, grown on demand (not under capture)
    out.zero_()
    assert lib.saetta_attn_gemm(*args, 0, 0, None, 0) == 0
    assert np.array_equal(host(out), want)
    assert lib.saetta_attn_gemm(*args, 7, 0, None, 0) == 0  # three slices of 7, 7 and 6 tokens
    assert np.abs(host(out) - want).max() < 1e-6


@pytest.mark.parametrize("seed", [31, 32])
def test_sweep(seed, monkeypatch):
    rng = np.random.default_rng(seed)
    for done in range(80):
        kind = KINDS[rng.integers(3)]
        pos = int(rng.choice([0, 0, 1, 15, 31, 32, 33, 511, 1000, 1023, 1024, 1025, int(rng.integers(0, 3000))]))
        tokens = int(rng.choice([1, 2, 3, 15, 16, 17, 31, 32, 33, 64, 100, 257, int(rng.integers(1, 400))]))
        slices = int(rng.choice([1, 2, 2, 3, 5]))
        monkeypatch.setenv("SAETTA_AG_SLICES", str(slices))
        n = pos + tokens
        k = (rng.standard_normal((n, VALUES)) * float(rng.choice([1.0, 2.0]))).astype(np.float32)
        v = rng.standard_normal((n, VALUES)).astype(np.float32)
        q16 = rng.standard_normal((tokens, H, D)).astype(np.float16)
        qg = rng.standard_normal((tokens, H, 2 * D)).astype(np.float32)
        kc, vc, kf, vf = make_cache(kind, k, v, n + int(rng.integers(0, 40)), chunk_from=pos if rng.integers(2) else None)
        got = run(kind, q16, kc, vc, qg, pos, tokens)
        want = oracle.prefill(q16.astype(np.float32), kf, vf, pos, tokens, q_and_gate=qg, threads=8)
        assert np.isfinite(got).all(), (seed, done, kind, pos, tokens, slices)
        assert np.abs(got - want).max() < MAX_ABS and oracle.rel_rms(got, want) < REL_RMS, (seed, done, kind, pos, tokens, slices)


def test_replayed_from_a_graph_equals_the_eager_call():
    # The call only enqueues kernels once its buffers exist (made by a first eager call), so a plan can
    # capture it: three replays with other work and synchronizations between them, each against the eager
    # result, bit for bit (the same kernels in the same order on the same inputs).
    pos, tokens = 1500, 300
    q16, k, v, qg = spread_case(pos, tokens)
    kc, vc, _, _ = make_cache(saetta.KvBits.Eight, k, v, 1856)
    q, g = dev(q16), dev(qg)
    p = saetta.FlashParams(H, KV, pos, tokens, 1.0 / math.sqrt(D))
    gemm = saetta.attention_gemm.AttGemm(tokens, KV)
    eager = torch.empty(tokens, H, D, device="cuda")
    gemm.encode(q, None, None, (kc, vc), g, eager, p)
    out = torch.full((tokens, H, D), float("nan"), device="cuda")
    plan = saetta.Plan()
    plan.op("attention_gemm", lambda s: gemm.encode(q, None, None, (kc, vc), g, out, p, stream=s))
    built = plan.build(graph=True)
    for replay in range(3):
        out.fill_(float("nan"))
        built.run()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), replay
        junk = torch.randn(1 << 20, device="cuda").sum().item()  # eager work between the replays
        assert junk == junk


@pytest.mark.parametrize("kv_heads", [1, 4])
def test_other_head_counts_both_routes(kv_heads):
    # 8 and 32 q heads (1 and 4 kv heads) over a half cache, 1100 keys: the flash kernel and AttGemm against the
    # oracle.  (The model has 16 / 2; the entry points take any kv head count with 8 q heads each.)
    rng = np.random.default_rng(70 + kv_heads)
    heads, pos, tokens = 8 * kv_heads, 1000, 100
    n = pos + tokens
    q16 = rng.standard_normal((tokens, heads, D)).astype(np.float16)
    k16 = rng.standard_normal((n, kv_heads * D)).astype(np.float16)
    v16 = rng.standard_normal((n, kv_heads * D)).astype(np.float16)
    qg = rng.standard_normal((tokens, heads, 2 * D)).astype(np.float32)
    want = oracle.prefill(q16.astype(np.float32), k16.astype(np.float32), v16.astype(np.float32), pos, tokens,
                          heads=heads, kv_heads=kv_heads, q_and_gate=qg, threads=8)
    p = saetta.FlashParams(heads, kv_heads, pos, tokens, 1.0 / math.sqrt(D))
    q, kc, vc, g = dev(q16), dev(k16), dev(v16), dev(qg)
    flash = torch.full((tokens, heads, D), float("nan"), device="cuda")
    saetta.attention_prefill.encode(saetta.attention_prefill.DEFAULT, q, kc, vc, g, flash, p)
    gemm = torch.full((tokens, heads, D), float("nan"), device="cuda")
    saetta.attention_gemm.AttGemm(tokens, kv_heads).encode(q, kc, vc, None, g, gemm, p)
    for got in (host(flash), host(gemm)):
        assert np.isfinite(got).all()
        assert np.abs(got - want).max() < MAX_ABS and oracle.rel_rms(got, want) < REL_RMS


def test_bench_mirrors_the_reference():
    # bench (src/attention_gemm.rs:366-470) at a small shape: both kernels timed at the last and the middle
    # chunk, the passes one by one, and the two outputs compared as the reference prints them.
    assert saetta.attention_gemm.KEYS == 1024
    (row,) = saetta.attention_gemm.bench([3000], 512, 10)
    assert row["context"] == 3072 and row["chunk"] == 512
    for name in ("rows2", "gemm"):
        assert row[name]["last_ms"] > 0 and row[name]["last_TFLOP/s"] > 0 and row[name]["prefill_attention_s"] > 0
    assert set(row["stages"]) == {"scores_ms", "scores_TFLOP/s", "softmax_ms", "pv_ms", "pv_TFLOP/s", "final_ms"}
    assert row["stages"]["scores_ms"] > 0
    assert row["rel_rms"] < 1e-3 and row["max_abs"] < MAX_ABS
