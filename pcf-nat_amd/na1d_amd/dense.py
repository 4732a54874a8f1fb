"""Dense ("global") attention of the models' global layers: softmax(q k^T * scale + mask) v per head.

Replaces ``attn = (q * scale) @ k.transpose(-2, -1) + attn_mask; attn = softmax(attn); x = attn @ v`` of
models/PCF_NATransformer.py:215-221, with the mask of get_attn_mask_global (:406-414) derived in the kernel from
the per-sample valid length: no ``[N, H, T, T]`` tensor is ever written, in either direction.
"""
from __future__ import annotations

import torch

from . import _lib


class _GlobalAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, t_valid, num_heads, scale, dropout):
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        assert q.dtype == k.dtype == v.dtype
        assert q.dim() == 3 and q.shape == k.shape == v.shape, "q, k, v must all be [B, T, C]"
        B, T, C = q.shape
        assert B % num_heads == 0
        if t_valid is not None:
            assert t_valid.dtype == torch.int32 and t_valid.numel() == B // num_heads and t_valid.is_contiguous()
        out = torch.empty_like(q)
        lse = torch.empty(B, T, dtype=torch.float32, device=q.device)
        if _lib.call_global_forward(out, lse, q, k, v, t_valid, B, num_heads, T, C, scale, dropout) != 0:
            raise _lib.NA1DError("global attention covers head_dim <= 128, got %d" % C)
        ctx.save_for_backward(q, k, v, out, lse, t_valid)
        ctx.args = (num_heads, scale, dropout)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, t_valid = ctx.saved_tensors
        num_heads, scale, dropout = ctx.args
        B, T, C = q.shape
        dout = dout.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        if B * T:
            ws = torch.empty(_lib.global_backward_workspace_bytes(B, num_heads, T, C, q.dtype), dtype=torch.uint8,
                             device=q.device)
            _lib.call_global_backward(dq, dk, dv, q, k, v, out, dout, lse, t_valid, B, num_heads, T, C, scale, ws,
                                      dropout)
        return dq, dk, dv, None, None, None, None


def global_attention(q, k, v, num_heads, t_valid=None, scale=None, dropout_p=0.0, seed=None):
    """``softmax(q k^T * scale + mask) v`` over whole sequences.

    q, k, v: ``[N * num_heads, T, C]`` bf16/fp16, contiguous, head fastest inside a sample.
    t_valid: optional int32 ``[N]``; -100 is added wherever the query row or the key column is ``>= t_valid[n]``.
    scale defaults to ``C ** -0.5``.
    dropout_p, seed: attention dropout inside the kernels, as in :func:`na1d_amd.na1d_fused` (the window slot of the
    keep rule is the key's row index).
    """
    if scale is None:
        scale = q.shape[-1] ** -0.5
    dropout = None
    if dropout_p > 0.0:
        assert dropout_p < 1.0
        dropout = (float(dropout_p), int(torch.randint(0, 2 ** 62, (1,)).item()) if seed is None else int(seed))
    return _GlobalAttention.apply(q, k, v, t_valid, num_heads, float(scale), dropout)
