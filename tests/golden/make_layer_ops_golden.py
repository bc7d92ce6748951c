"""Writes tests/golden/layer_ops_golden.npz: inputs and outputs of library routines for the
operators around attention - torch.nn.functional.rms_norm on the CPU in fp64, and the rotary
position embedding helpers of the transformers library (LLaMA's rotate-half form, GPT-J's
adjacent-pair form) in fp64, whole-head and partial (the first rotary_ndims elements of a head),
and torch's silu / gelu (erf and tanh forms) in fp64 for the gated MLP.

Nothing from the reference is imported or run.  Usage: python tests/golden/make_layer_ops_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F
from transformers.models.gptj.modeling_gptj import apply_rotary_pos_emb as gptj_rope
from transformers.models.llama.modeling_llama import apply_rotary_pos_emb as llama_rope

RMS_CASES = [("rms_small", 3, 16, 1e-6), ("rms_odd", 5, 37, 1e-5), ("rms_wide", 2, 1024, 1e-6)]
# name, tokens, heads, head_size, rotary_ndims, interleaved
ROPE_CASES = [("llama", 6, 3, 16, 16, False), ("llama_partial", 4, 2, 32, 8, False), ("gptj", 5, 2, 16, 16, True),
              ("gptj_partial", 3, 4, 24, 8, True)]


def angles(tokens, width, g):
    """Arbitrary angles (not a frequency ladder), so that every table entry matters."""
    return 6.0 * torch.rand(tokens, width, generator=g, dtype=torch.float64)


def main():
    out = {}
    for idx, (name, rows, hidden, eps) in enumerate(RMS_CASES):
        g = torch.Generator().manual_seed(5100 + idx)
        x = torch.randn(rows, hidden, generator=g, dtype=torch.float32) * 3.0
        w = torch.randn(hidden, generator=g, dtype=torch.float32)
        out[name + "/x"], out[name + "/gamma"], out[name + "/eps"] = x.numpy(), w.numpy(), np.float32(eps)
        out[name + "/out"] = F.rms_norm(x.double(), (hidden,), w.double(), eps).float().numpy()
    for idx, (name, T, H, S, rot, interleaved) in enumerate(ROPE_CASES):
        g = torch.Generator().manual_seed(5200 + idx)
        x = torch.randn(T, H, S, generator=g, dtype=torch.float32)
        xd = x.double()
        if interleaved:
            th = angles(T, rot // 2, g)
            cos, sin = th.cos(), th.sin()
            # GPT-J layout [batch, tokens, heads, head]; sin/cos [batch, tokens, rot/2]
            rotated = gptj_rope(xd[None, :, :, :rot], sin[None], cos[None])[0]
        else:
            th = angles(T, rot, g)  # both halves of a row carry their own angle
            cos, sin = th.cos(), th.sin()
            # LLaMA layout [batch, heads, tokens, head]; cos/sin [batch, tokens, rot]
            xq = xd[:, :, :rot].permute(1, 0, 2)[None]
            rotated = llama_rope(xq, xq, cos[None], sin[None])[0][0].permute(1, 0, 2)
        o = torch.cat([rotated, xd[:, :, rot:]], dim=-1)
        out[name + "/x"], out[name + "/cos"], out[name + "/sin"] = x.numpy(), cos.float().numpy(), sin.float().numpy()
        out[name + "/out"] = o.float().numpy()
    # activations of the gated MLP: silu with a beta, gelu in both of OpenVINO's modes
    g = torch.Generator().manual_seed(5300)
    x = 4.0 * torch.randn(257, generator=g, dtype=torch.float32)
    out["act/x"] = x.numpy()
    out["act/silu"] = F.silu(x.double()).float().numpy()
    out["act/silu_beta1p7"] = (x.double() * torch.sigmoid(1.7 * x.double())).float().numpy()
    out["act/gelu_erf"] = F.gelu(x.double()).float().numpy()
    out["act/gelu_tanh"] = F.gelu(x.double(), approximate="tanh").float().numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "layer_ops_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
