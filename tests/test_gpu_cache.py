"""GpuKvCache (grow / shrink, src/gpu_layers.rs:183-293) and RowBackup (src/gpu_cache.rs:196-283)
of the host mirror: the rows a resize or a backup moves are the same bytes afterwards, and the
attention over a resized cache is the attention over the old one (re-recorded, as the reference
requires after a resize).  The reference's own checks: src/gpu_cache.rs tests (rows come back bit
for bit) and the resize contract in the doc comment of `resize`."""
import numpy as np
import pytest
import torch

from gpu_common import D, H, KV, VALUES, dev, host, oracle, saetta

pytestmark = pytest.mark.gpu
KINDS = [saetta.KvBits.Half, saetta.KvBits.Eight, saetta.KvBits.Four]


def fill(cache, x, start=0):
    """Rows start.. of both keys and values from x [tokens, 512] (values get -x)."""
    tokens = x.shape[0]
    if cache.bits is saetta.KvBits.Half:
        cache.keys[start * VALUES:(start + tokens) * VALUES] = dev(x.astype(np.float16)).flatten()
        cache.values[start * VALUES:(start + tokens) * VALUES] = dev((-x).astype(np.float16)).flatten()
    else:
        k, v = cache.quant
        k.encode(dev(x), start, tokens)
        v.encode(dev(-x), start, tokens)


def attend(cache, q, qg, length):
    out = torch.empty(H, D, device="cuda")
    plan = saetta.Plan()
    if cache.bits is saetta.KvBits.Half:
        cache.decode.record(plan, q, cache.keys, cache.values, qg, out)
    else:
        cache.decode.record_quant(plan, q, cache.quant[0], cache.quant[1], qg, out)
    plan.set_params(saetta.TokenParams(0, length - 1))
    plan.build().run()
    return host(out)


@pytest.mark.parametrize("kind", KINDS)
def test_resize_keeps_the_rows_and_the_attention(kind):
    cache = saetta.GpuKvCache.with_bits(H, KV, D, 200, kind)
    assert cache.capacity == 256 and len(cache.buffers()) == (2 if kind is saetta.KvBits.Half else 6)
    tokens = 150
    x = oracle.noise(tokens * VALUES, 5).reshape(tokens, VALUES)
    fill(cache, x)
    q, qg = dev(oracle.noise(H * D, 6)), dev(oracle.noise(H * 2 * D, 7))
    before = attend(cache, q, qg, tokens)
    rows_before = [host(b).copy() for b in cache.buffers()]

    cache.resize(1000)  # grow
    assert cache.capacity == 1024 and cache.decode.capacity == 1024
    for b, old in zip(cache.buffers(), rows_before):
        got = host(b)
        assert got.size == old.size * 4 and np.array_equal(got[:old.size], old) and not got[old.size:].any()
    # more splits over the same rows: the same sums in another order
    assert np.abs(attend(cache, q, qg, tokens) - before).max() < 2e-6
    if kind is not saetta.KvBits.Half:
        assert cache.quant[0].data.data_ptr() == cache.keys.data_ptr() and cache.quant[0].capacity == 1024
        fill(cache, x[:10], start=1000)  # the new rows take appends

    cache.resize(100)  # shrink: 128 rows stay
    assert cache.capacity == 128
    for b, old in zip(cache.buffers(), rows_before):
        assert np.array_equal(host(b), old[:old.size // 2])
    assert np.abs(attend(cache, q, qg, 128) - attend_reference(x[:128], q, qg, kind)).max() < 2e-5


def attend_reference(x, q, qg, kind):
    bits = {saetta.KvBits.Half: 16, saetta.KvBits.Eight: 8, saetta.KvBits.Four: 4}[kind]
    kf, vf = oracle.round_trip(x, bits), oracle.round_trip(-x, bits)
    return oracle.attention_f64(host(q), kf, vf, host(qg), x.shape[0], threads=4)


@pytest.mark.parametrize("kind", KINDS)
def test_row_backup_puts_the_rows_back(kind):
    caches = [saetta.GpuKvCache(H, KV, D, 256, kind) for _ in range(3)]
    for i, c in enumerate(caches):
        fill(c, oracle.noise(256 * VALUES, 10 + i).reshape(256, VALUES))
    want = [[host(b).copy() for b in c.buffers()] for c in caches]
    backup = saetta.RowBackup()
    assert backup.bytes() == 0
    backup.save(caches, 100, 12)
    per_token = {saetta.KvBits.Half: 2048, saetta.KvBits.Eight: 1088, saetta.KvBits.Four: 576}[kind]
    assert backup.bytes() == 3 * 12 * per_token
    for c in caches:  # the detour writes over the rows
        fill(c, oracle.noise(12 * VALUES, 99).reshape(12, VALUES), start=100)
    assert not np.array_equal(host(caches[0].keys), want[0][0])
    backup.restore(caches)
    assert backup.bytes() == 0
    for c, w in zip(caches, want):
        for b, old in zip(c.buffers(), w):
            assert np.array_equal(host(b), old)
    backup.restore(caches)  # nothing held: nothing happens
    backup.save(caches, 0, 0)
    assert backup.bytes() == 0
    with pytest.raises(ValueError):
        backup.save(caches, 250, 12)
    backup.save(caches, 5, 2)
    backup.clear()
    assert backup.bytes() == 0
