"""The quantisers of the reference's harness (benchmark.py:96-107), as torch ops on whatever device holds x."""
import torch


def quant_pertoken(x):
    """Per-row symmetric int8 (benchmark.py:96-100): scale = absmax / 127 in x's dtype, round-half-even."""
    scale = x.abs().amax(dim=-1) / 127
    return torch.round(x / scale.unsqueeze(-1)).to(torch.int8), scale


def quant_pertensor(x):
    """One scale per (batch, head) slice (benchmark.py:102-107)."""
    scale = x.abs().amax(dim=(-2, -1)) / 127
    return torch.round(x / scale[:, :, None, None]).to(torch.int8), scale
