"""Writes tests/golden/alibi_golden.npz: attention with ALiBi's linear distance bias, spelt as an explicit
additive mask and computed by a library routine, torch.nn.functional.scaled_dot_product_attention on the
CPU in fp64.  A case is one sequence with `past` cached tokens and `n` new ones: query i sits at position
p = past + i, attends keys j <= p (and j > p - window when window > 0), and the mask holds
slope[h] * (j - p) there and -inf elsewhere.  The paged-attention oracle is held to these outputs with the
keys and values laid out in a paged cache (tests/test_oracle_cpu.py).

Nothing from the reference is imported or run.  Usage: python tests/golden/make_alibi_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

CASES = [
    # name, Hq, Hkv, D, past, n, window
    ("decode", 4, 2, 16, 37, 1, 0),
    ("chunk", 8, 2, 32, 20, 12, 0),
    ("prefill", 2, 2, 8, 0, 9, 0),
    ("window", 4, 1, 16, 50, 6, 17),
]


def slopes(Hq):
    """The geometric sequence of the ALiBi paper for a power-of-two head count: 2^(-8 h / Hq), h = 1..Hq."""
    return (2.0 ** (-8.0 * np.arange(1, Hq + 1) / Hq)).astype(np.float32)


def main():
    out = {}
    for idx, (name, Hq, Hkv, D, past, n, window) in enumerate(CASES):
        g = torch.Generator().manual_seed(4400 + idx)
        ctx = past + n
        q = torch.randn(1, Hq, n, D, generator=g, dtype=torch.float32)
        k = torch.randn(1, Hkv, ctx, D, generator=g, dtype=torch.float32)
        v = torch.randn(1, Hkv, ctx, D, generator=g, dtype=torch.float32)
        sl = torch.from_numpy(slopes(Hq))
        p = past + torch.arange(n)[:, None]
        j = torch.arange(ctx)[None, :]
        keep = j <= p
        if window > 0:
            keep &= j > p - window
        bias = sl.double()[:, None, None] * (j - p).double()[None]
        bias = torch.where(keep[None], bias, torch.full_like(bias, float("-inf")))
        o = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=bias[None], enable_gqa=True)
        out[name + "/q"], out[name + "/k"], out[name + "/v"] = q.numpy(), k.numpy(), v.numpy()
        out[name + "/slopes"] = sl.numpy()
        out[name + "/meta"] = np.array([Hq, Hkv, D, past, n, window], np.int32)
        out[name + "/out"] = o.float().numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "alibi_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
