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


class _FusedNA1DQKV(torch.autograd.Function):
    """Fused NA1D straight on the qkv projection's output ``[N, T, 3, H, C]`` -> ``[N, T, H*C]``."""

    @staticmethod
    def forward(ctx, qkv, rpb, t_valid, win_size, left, scale, deterministic):
        assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.is_contiguous()
        N, T, _, H, C = qkv.shape
        ctx.rpb_shape = None if rpb is None else rpb.shape
        if rpb is not None:
            rpb = rpb.detach().reshape(H, win_size).to(torch.float32).contiguous()
        if t_valid is not None:
            assert t_valid.numel() == N
            t_valid = t_valid.to(device=qkv.device, dtype=torch.int32).contiguous()
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))          # [N, H, T, C] views
        out = torch.empty((N, T, H, C), dtype=qkv.dtype, device=qkv.device)
        lse = torch.empty((N * H, T), dtype=torch.float32, device=qkv.device)
        st = _lib.call_fused_forward_strided(out.permute(0, 2, 1, 3), lse, q, k, v, rpb, t_valid, win_size, left, scale)
        ctx.strided = st == 0
        ctx.packed_out = None
        if not ctx.strided:      # shape outside the strided kernels: pack, as the reference does, and use the packed op
            qp, kp, vp = (z.contiguous().view(N * H, T, C) for z in (q, k, v))
            op = torch.empty_like(qp)
            _lib.call_fused_forward(op, lse, qp, kp, vp, rpb, t_valid, N * H, H, T, C, win_size, left, scale)
            out.copy_(op.view(N, H, T, C).permute(0, 2, 1, 3))
            ctx.packed_out = op          # the generic backward kernel reads it
        ctx.save_for_backward(qkv, lse, rpb, t_valid)
        ctx.geom = (win_size, left, scale, deterministic)
        return out.view(N, T, H * C)

    @staticmethod
    def backward(ctx, dout):
        qkv, lse, rpb, t_valid = ctx.saved_tensors
        win_size, left, scale, deterministic = ctx.geom
        N, T, _, H, C = qkv.shape
        dout = dout.contiguous().view(N, T, H, C)
        dqkv = torch.empty_like(qkv)
        drpb = ws = None
        if rpb is not None and ctx.needs_input_grad[1]:
            drpb = torch.zeros((H, win_size), dtype=torch.float32, device=qkv.device)
            if deterministic:
                nbytes = _lib.fused_backward_workspace_bytes(N * H, H, T, C, win_size, left, qkv.dtype)
                if nbytes > 0:
                    ws = torch.empty(nbytes, dtype=torch.uint8, device=qkv.device)
        q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
        if ctx.strided:
            dq, dk, dv = (dqkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            st = _lib.call_fused_backward_strided(dq, dk, dv, drpb, q, k, v, dout.permute(0, 2, 1, 3), lse, rpb, t_valid,
                                                  win_size, left, scale, workspace=ws)
            assert st == 0
        else:
            qp, kp, vp = (z.contiguous().view(N * H, T, C) for z in (q, k, v))
            gp = dout.permute(0, 2, 1, 3).contiguous().view(N * H, T, C)
            dqp, dkp, dvp = torch.empty_like(qp), torch.empty_like(kp), torch.empty_like(vp)
            _lib.call_fused_backward(dqp, dkp, dvp, drpb, qp, kp, vp, ctx.packed_out, gp, lse, rpb, t_valid, N * H, H, T, C,
                                     win_size, left, scale, workspace=ws)
            for i, z in enumerate((dqp, dkp, dvp)):
                dqkv[:, :, i].copy_(z.view(N, H, T, C).permute(0, 2, 1, 3))
        if drpb is not None:
            drpb = drpb.view(ctx.rpb_shape)
        return dqkv, drpb, None, None, None, None, None


def na1d_fused_qkv(qkv, win_size, left, rpb=None, t_valid=None, scale=1.0, deterministic=False):
    """Fused neighbourhood attention on a token-major qkv projection output.

    qkv : contiguous ``[N, T, 3, H, C]`` bf16/fp16 (the ``[N, T, 3*dim]`` output of the projection, viewed).
          The kernels read each head's rows in place and write ``[N, T, H*C]`` directly, so the head split
          and merge copies of the reference (models/MFA_NATransformer.py:127-138,150-151) do not exist; the
          gradient comes back as one ``[N, T, 3, H, C]`` tensor.  ``scale`` multiplies the fp32 scores (the
          reference multiplies q by it in 16 bit beforehand).
    Other arguments as in :func:`na1d_fused`.
    """
    return _FusedNA1DQKV.apply(qkv, rpb, t_valid, win_size, left, float(scale), bool(deterministic))
