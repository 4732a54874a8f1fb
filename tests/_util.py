"""Shared helpers of the parity tests."""
import torch

from oracle import na1d_oracle as O

TOL = {torch.bfloat16: 1e-2, torch.float16: 2e-3}   # rel-L2 bars of the parity contract


def make_inputs(B, T, C, W, seed, dtype, n=3, scale=None):
    """Seeded N(0,1) tensors rounded to `dtype` (CPU), q optionally pre-scaled in 16-bit."""
    return O.seeded_qkv(B, T, C, seed, dtype, n=n, scale_q=scale)


def seeded_scores(B, T, W, seed):
    g = torch.Generator().manual_seed(seed + 1000)
    return torch.randn(B, T, W, generator=g, dtype=torch.float32)


def dev(*ts):
    out = [None if t is None else t.cuda() for t in ts]
    return out if len(out) > 1 else out[0]
