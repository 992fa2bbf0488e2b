"""Helpers of the GPU parity tests: the package, device tensors, quantized caches."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402
import oracle  # noqa: E402  (the checker)

saetta = entry.load_package()
H, KV, D = 16, 2, 256
VALUES = KV * D


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def bits_of(kind):
    return {saetta.KvBits.Eight: 8, saetta.KvBits.Four: 4, saetta.KvBits.Half: 16}[kind]


def quant_cache_from_host(x, kind, capacity):
    """A QuantRows filled with the ORACLE's codes of x [tokens, 512] (host-quantized cache)."""
    bits = bits_of(kind)
    rows = saetta.QuantRows(kind, VALUES, capacity)
    data, scales, biases = oracle.quantize(x, bits)
    rows.data[:data.size] = dev(data.view(np.int32))
    rows.scales[:scales.size] = dev(scales.view(np.float16))
    rows.biases[:biases.size] = dev(biases.view(np.float16))
    return rows


def cache_pair(k, v, kind, capacity, poison=True):
    """Keys/values caches of `kind` holding k, v [tokens, 512], and the f32 values the
    oracle sees.  Rows past the tokens are filled with NaN patterns (hipMalloc'd memory
    is not zeroed; nothing past the context may reach the output)."""
    bits = bits_of(kind)
    tokens = k.shape[0]
    if kind is saetta.KvBits.Half:
        kc = torch.full((capacity, VALUES), float("nan"), dtype=torch.float16, device="cuda")
        vc = torch.full((capacity, VALUES), float("nan"), dtype=torch.float16, device="cuda")
        if not poison:
            kc.zero_(), vc.zero_()
        kc[:tokens] = dev(k.astype(np.float16))
        vc[:tokens] = dev(v.astype(np.float16))
        return kc, vc, oracle.round_trip(k, 16), oracle.round_trip(v, 16)
    kc, vc = quant_cache_from_host(k, kind, capacity), quant_cache_from_host(v, kind, capacity)
    if poison:
        for c in (kc, vc):
            c.scales[tokens * 8:] = float("nan")
            c.biases[tokens * 8:] = float("inf")
            c.data[tokens * 8 * 2 * bits:] = -1
    return kc, vc, oracle.round_trip(k, bits), oracle.round_trip(v, bits)
