"""Fused NA1D: QK^T -> +rpb -> +mask -> softmax -> .V in one kernel each way.

Replaces the chain ``QK_Function -> + relative_position_bias -> + attn_mask ->
softmax -> AV_Function`` of models/PCF_NATransformer.py:141-150 (mask of
:87-99) without ever writing the ``[B, T, W]`` tensor.  The mask is derived in
the kernel from the per-sample valid length, so no mask tensor exists either.
"""
from __future__ import annotations

import torch

from . import _lib


class _FusedNA1D(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, rpb, t_valid, num_heads, win_size, left, scale, deterministic):
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        assert q.dtype == k.dtype == v.dtype
        assert q.dim() == 3 and q.shape == k.shape == v.shape, "q, k, v must all be [B, T, C]"
        B, T, C = q.shape
        assert B % num_heads == 0
        ctx.rpb_shape = None if rpb is None else rpb.shape
        if rpb is not None:
            rpb = rpb.detach().reshape(num_heads, win_size).to(torch.float32).contiguous()
        if t_valid is not None:
            assert t_valid.numel() == B // num_heads
            t_valid = t_valid.to(device=q.device, dtype=torch.int32).contiguous()
        out = torch.empty_like(q)
        lse = torch.empty((B, T), dtype=torch.float32, device=q.device)
        _lib.call_fused_forward(out, lse, q, k, v, rpb, t_valid, B, num_heads, T, C, win_size, left, scale)
        ctx.save_for_backward(q, k, v, out, lse, rpb, t_valid)
        ctx.geom = (num_heads, win_size, left, scale, deterministic)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, rpb, t_valid = ctx.saved_tensors
        num_heads, win_size, left, scale, deterministic = ctx.geom
        B, T, C = q.shape
        dout = dout.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        drpb = ws = None
        if rpb is not None and ctx.needs_input_grad[3]:
            drpb = torch.zeros((num_heads, win_size), dtype=torch.float32, device=q.device)
            if deterministic:   # fold the per-workgroup partial sums in a fixed order instead of with atomics
                nbytes = _lib.fused_backward_workspace_bytes(B, num_heads, T, C, win_size, left, q.dtype)
                if nbytes > 0:
                    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
        _lib.call_fused_backward(dq, dk, dv, drpb, q, k, v, out, dout, lse, rpb, t_valid,
                                 B, num_heads, T, C, win_size, left, scale, workspace=ws)
        if drpb is not None:
            drpb = drpb.view(ctx.rpb_shape)
        return dq, dk, dv, drpb, None, None, None, None, None, None


def na1d_fused(q, k, v, win_size, left, rpb=None, t_valid=None, num_heads=1, scale=1.0, deterministic=False):
    """Fused neighbourhood attention.

    q, k, v : contiguous ``[B, T, C]`` bf16/fp16, ``B = N * num_heads``.  ``q`` is
              used as given; ``scale`` multiplies the fp32 scores (pass the
              pre-scaled q of the reference model with ``scale=1``).
    rpb     : ``[num_heads, W]`` (any shape with that many elements), or None.
    t_valid : int tensor ``[N]`` of valid lengths (``T - padding``), or None.
    deterministic : the gradient of ``rpb`` is summed over workgroups with float
              atomics by default (fast, last bits vary from run to run); ``True``
              folds the partial sums in a fixed order through a scratch buffer.
              dq, dk, dv never use atomics.
    Returns ``[B, T, C]`` in q's dtype.  The gradient of ``rpb`` has rpb's shape.
    """
    return _FusedNA1D.apply(q, k, v, rpb, t_valid, num_heads, win_size, left, float(scale), bool(deterministic))


def na1d_fused_forward_lse(q, k, v, win_size, left, rpb=None, t_valid=None, num_heads=1, scale=1.0):
    """Inference-only variant that also returns the per-row log-sum-exp ``[B, T]``."""
    B, T, C = q.shape
    if rpb is not None:
        rpb = rpb.detach().reshape(num_heads, win_size).to(torch.float32).contiguous()
    if t_valid is not None:
        t_valid = t_valid.to(device=q.device, dtype=torch.int32).contiguous()
    out = torch.empty_like(q)
    lse = torch.empty((B, T), dtype=torch.float32, device=q.device)
    _lib.call_fused_forward(out, lse, q, k, v, rpb, t_valid, B, num_heads, T, C, win_size, left, float(scale))
    return out, lse
