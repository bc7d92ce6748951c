"""Writes tests/golden/sdpa_golden.npz: inputs and outputs of a library routine,
torch.nn.functional.scaled_dot_product_attention on the CPU in fp64, for the shapes the
reference's own SDPA test instantiates
(modules/nvidia_plugin/tests/functional/shared_tests_instances/single_layer_tests/
scaled_dot_product_attention.cpp:76-104) plus GQA and rectangular cases.

Nothing from the reference is imported or run.  Usage: python tests/golden/make_sdpa_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

CASES = [
    # name, B, Hq, Hkv, Lq, Lk, D
    ("ref_small", 1, 1, 1, 4, 4, 8),
    ("ref_medium", 1, 4, 4, 16, 16, 32),
    ("ref_llm", 1, 8, 8, 32, 32, 64),
    ("ref_3d", 1, 4, 4, 2, 2, 8),  # rank-3 [4,2,8]: leading dim is batch-like
    ("gqa", 2, 4, 2, 17, 17, 32),
    ("rect", 1, 4, 2, 5, 40, 64),
    ("long_row", 1, 2, 1, 3, 300, 16),
]

MASK_CASES = [
    # name, B, Hq, Hkv, Lq, Lk, D, mask shape, boolean
    ("float_full", 2, 4, 2, 9, 13, 16, (2, 4, 9, 13), False),
    ("float_2d", 1, 4, 4, 16, 16, 32, (16, 16), False),
    ("float_per_batch", 2, 2, 2, 5, 70, 8, (2, 1, 1, 70), False),
    ("bool_full", 1, 4, 2, 7, 33, 16, (1, 4, 7, 33), True),
    ("bool_keys", 3, 2, 1, 4, 20, 64, (3, 1, 1, 20), True),
]


def main():
    out = {}
    for idx, (name, B, Hq, Hkv, Lq, Lk, D) in enumerate(CASES):
        g = torch.Generator().manual_seed(4200 + idx)
        q = torch.randn(B, Hq, Lq, D, generator=g, dtype=torch.float32)
        k = torch.randn(B, Hkv, Lk, D, generator=g, dtype=torch.float32)
        v = torch.randn(B, Hkv, Lk, D, generator=g, dtype=torch.float32)
        out[name + "/q"], out[name + "/k"], out[name + "/v"] = q.numpy(), k.numpy(), v.numpy()
        for causal in (False, True):
            o = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=causal,
                                               enable_gqa=True)
            out["%s/out_causal%d" % (name, int(causal))] = o.float().numpy()
    # attention_mask input: float masks (added to the scaled scores) and boolean masks (True = take
    # part), full [B,Hq,Lq,Lk] and broadcast shapes; no row is masked out completely
    for idx, (name, B, Hq, Hkv, Lq, Lk, D, mshape, boolean) in enumerate(MASK_CASES):
        g = torch.Generator().manual_seed(4300 + idx)
        q = torch.randn(B, Hq, Lq, D, generator=g, dtype=torch.float32)
        k = torch.randn(B, Hkv, Lk, D, generator=g, dtype=torch.float32)
        v = torch.randn(B, Hkv, Lk, D, generator=g, dtype=torch.float32)
        if boolean:
            mask = torch.rand(*mshape, generator=g) < 0.6
            mask[..., 0] = True
            am = mask
        else:
            mask = 2.0 * torch.randn(*mshape, generator=g, dtype=torch.float32)
            am = mask.double()
        o = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=am, enable_gqa=True)
        out["mask_%s/q" % name], out["mask_%s/k" % name], out["mask_%s/v" % name] = q.numpy(), k.numpy(), v.numpy()
        out["mask_%s/mask" % name] = mask.numpy()
        out["mask_%s/out" % name] = o.float().numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sdpa_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
