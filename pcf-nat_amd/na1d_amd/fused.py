"""Fused NA1D: QK^T -> +rpb -> +mask -> softmax -> .V in one kernel each way.

Replaces the chain ``QK_Function -> + relative_position_bias -> + attn_mask ->
softmax -> AV_Function`` of models/PCF_NATransformer.py:141-150 (mask of
:87-99) without ever writing the ``[B, T, W]`` tensor.  The mask is derived in
the kernel from the per-sample valid length, so no mask tensor exists either.
"""
from __future__ import annotations

import torch

from . import _lib


def _residue(x4, r, d):
    """Rows r, r+d, r+2d, ... of a ``[N, H, T, C]`` view: the sub-sequence a dilated window lives in."""
    return x4[:, :, r::d]


def _residue_lengths(t_valid, r, d):
    """Valid length of that sub-sequence: rows r + d*t' < t_valid."""
    return None if t_valid is None else ((t_valid - r + d - 1) // d).clamp_(min=0).to(torch.int32)


def _strided_or_packed_forward(out4, lse, q4, k4, v4, rpb, t_valid, W, left, scale, dropout=None):
    """Forward on ``[N, H, T, C]`` views through the strided entry point, or - for shapes it does not cover -
    on packed copies through the packed one.  Returns the packed output when it had to be made.  ``dropout``:
    ``None`` or ``(p, seed, row_stride, row_offset, seq_rows)``."""
    if _lib.call_fused_forward_strided(out4, lse, q4, k4, v4, rpb, t_valid, W, left, scale, dropout=dropout) == 0:
        return None
    if dropout is not None and len(dropout) > 2 and tuple(dropout[2:4]) != (1, 0):
        raise _lib.NA1DError("attention dropout with dilated windows needs head_dim <= 128 (the packed entry points "
                             "name rows by their place in the tensor they are given)")
    N, H, T, C = q4.shape
    qp, kp, vp = (z.contiguous().view(N * H, T, C) for z in (q4, k4, v4))
    op = torch.empty_like(qp)
    _lib.call_fused_forward(op, lse, qp, kp, vp, rpb, t_valid, N * H, H, T, C, W, left, scale,
                            dropout=None if dropout is None else dropout[:2])
    out4.copy_(op.view(N, H, T, C))
    return op


def _strided_or_packed_backward(dq4, dk4, dv4, drpb, q4, k4, v4, packed_out, dout4, lse, rpb, t_valid, W, left, scale, ws,
                                dropout=None):
    if packed_out is None:
        st = _lib.call_fused_backward_strided(dq4, dk4, dv4, drpb, q4, k4, v4, dout4, lse, rpb, t_valid, W, left, scale,
                                              workspace=ws, dropout=dropout)
        assert st == 0
        return
    N, H, T, C = q4.shape
    qp, kp, vp, gp = (z.contiguous().view(N * H, T, C) for z in (q4, k4, v4, dout4))
    dqp, dkp, dvp = torch.empty_like(qp), torch.empty_like(kp), torch.empty_like(vp)
    _lib.call_fused_backward(dqp, dkp, dvp, drpb, qp, kp, vp, packed_out, gp, lse, rpb, t_valid, N * H, H, T, C, W, left,
                             scale, workspace=ws, dropout=None if dropout is None else dropout[:2])
    for dst, src in ((dq4, dqp), (dk4, dkp), (dv4, dvp)):
        dst.copy_(src.view(N, H, T, C))


def _deterministic_workspace_bytes(B, H, T, C, win_size, left, dilation, dtype):
    """Bytes of scratch for the fixed-order reduction of the bias gradient over every launch of one backward: with
    dilation d the residue classes have ceil(T/d) or floor(T/d) rows, and the shorter class can need the larger
    workspace (the split into workgroups is not monotonic in the length), so it is the maximum over both."""
    lengths = {-(-T // dilation)}
    if dilation > 1 and T % dilation and T // dilation > 0:
        lengths.add(T // dilation)
    return max(_lib.fused_backward_workspace_bytes(B, H, t, C, win_size, left, dtype) for t in lengths)


def _deterministic_workspace(B, H, T, C, win_size, left, like, dilation=1):
    """Scratch for the fixed-order reduction of the bias gradient.  The matrix-core backward kernels have that path;
    for head_dim > 128 (the generic kernels) the library would use float atomics, so the request is refused instead."""
    nbytes = _deterministic_workspace_bytes(B, H, T, C, win_size, left, dilation, like.dtype)
    if nbytes <= 0:
        raise _lib.NA1DError("deterministic=True: no fixed-order reduction of the bias gradient for head_dim %d "
                             "(it covers head_dim <= 128)" % C)
    return torch.empty(nbytes, dtype=torch.uint8, device=like.device)


class _FusedNA1D(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, rpb, t_valid, num_heads, win_size, left, scale, deterministic, dilation, dropout):
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        ctx.dropout = dropout
        assert q.dtype == k.dtype == v.dtype
        assert q.dim() == 3 and q.shape == k.shape == v.shape, "q, k, v must all be [B, T, C]"
        B, T, C = q.shape
        assert B % num_heads == 0 and dilation >= 1
        ctx.rpb_shape = None if rpb is None else rpb.shape
        if rpb is not None:
            rpb = rpb.detach().reshape(num_heads, win_size).to(torch.float32).contiguous()
        if t_valid is not None:
            assert t_valid.numel() == B // num_heads
            t_valid = t_valid.to(device=q.device, dtype=torch.int32).contiguous()
        out = torch.empty_like(q)
        ctx.geom = (num_heads, win_size, left, scale, deterministic, dilation)
        if dilation == 1:
            lse = torch.empty((B, T), dtype=torch.float32, device=q.device)
            _lib.call_fused_forward(out, lse, q, k, v, rpb, t_valid, B, num_heads, T, C, win_size, left, scale,
                                    dropout=dropout)
            ctx.save_for_backward(q, k, v, out, rpb, t_valid, lse)
            return out
        # Dilation d: slot j of row t is row t + (j - left) * d, so the rows of one residue class t mod d only
        # ever meet each other - d independent, undilated problems on every d-th row, read and written in place.
        shape4 = (B // num_heads, num_heads, T, C)
        q4, k4, v4, o4 = (z.view(shape4) for z in (q, k, v, out))
        lses, ctx.packed_outs = [], []
        for r in range(min(dilation, T)):
            qr = _residue(q4, r, dilation)
            lse = torch.empty((B, qr.shape[2]), dtype=torch.float32, device=q.device)
            ctx.packed_outs.append(_strided_or_packed_forward(
                _residue(o4, r, dilation), lse, qr, _residue(k4, r, dilation), _residue(v4, r, dilation), rpb,
                _residue_lengths(t_valid, r, dilation), win_size, left, scale,
                dropout=None if dropout is None else (*dropout, dilation, r, T)))     # rows named by their place in T
            lses.append(lse)
        ctx.save_for_backward(q, k, v, out, rpb, t_valid, *lses)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, rpb, t_valid, *lses = ctx.saved_tensors
        num_heads, win_size, left, scale, deterministic, dilation = ctx.geom
        B, T, C = q.shape
        dout = dout.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        drpb = ws = None
        if rpb is not None and ctx.needs_input_grad[3]:
            drpb = torch.zeros((num_heads, win_size), dtype=torch.float32, device=q.device)
            if deterministic:   # fold the per-workgroup partial sums in a fixed order instead of with atomics
                ws = _deterministic_workspace(B, num_heads, T, C, win_size, left, q, dilation)
        if dilation == 1:
            _lib.call_fused_backward(dq, dk, dv, drpb, q, k, v, out, dout, lses[0], rpb, t_valid,
                                     B, num_heads, T, C, win_size, left, scale, workspace=ws, dropout=ctx.dropout)
        else:
            shape4 = (B // num_heads, num_heads, T, C)
            views = [z.view(shape4) for z in (dq, dk, dv, q, k, v, dout)]
            for r, lse in enumerate(lses):
                a = [_residue(z, r, dilation) for z in views]
                _strided_or_packed_backward(a[0], a[1], a[2], drpb, a[3], a[4], a[5], ctx.packed_outs[r], a[6], lse, rpb,
                                            _residue_lengths(t_valid, r, dilation), win_size, left, scale, ws,
                                            dropout=None if ctx.dropout is None else (*ctx.dropout, dilation, r, T))
        if drpb is not None:
            drpb = drpb.view(ctx.rpb_shape)
        return dq, dk, dv, drpb, None, None, None, None, None, None, None, None


def na1d_fused(q, k, v, win_size, left, rpb=None, t_valid=None, num_heads=1, scale=1.0, deterministic=False,
               dilation=1, dropout_p=0.0, seed=None):
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
    dilation : window slot j of row t addresses row ``t + (j - left) * dilation`` (the reference computes this on
              the CPU only, models/PCF_NATransformer.py:101-116,158-170; its CUDA path asserts dilation == 1).
    dropout_p, seed : attention dropout inside the kernels (nn.Dropout(attn_drop) of models/PCF_NATransformer.py:71,149):
              each probability is kept with chance ``1 - dropout_p`` and scaled by ``1 / (1 - dropout_p)``.  The mask
              is a hash of (seed, sequence, row, window slot) that the backward recomputes; ``seed`` (a 64-bit int)
              defaults to a draw from torch's CPU generator.  Needs head_dim <= 128.  With ``dilation > 1`` the mask
              is still the one of (sequence, row, slot) of the whole operator: the launches on the residue classes
              name their rows by their place in the sequence.
    Returns ``[B, T, C]`` in q's dtype.  The gradient of ``rpb`` has rpb's shape.
    """
    dropout = None
    if dropout_p > 0.0:
        assert dropout_p < 1.0
        if seed is None:
            seed = int(torch.randint(0, 2 ** 62, (1,)).item())
        dropout = (float(dropout_p), int(seed))
    return _FusedNA1D.apply(q, k, v, rpb, t_valid, num_heads, win_size, left, float(scale), bool(deterministic),
                            int(dilation), dropout)


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
    def forward(ctx, qkv, rpb, t_valid, win_size, left, scale, deterministic, dilation, dropout):
        assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.is_contiguous() and dilation >= 1
        ctx.dropout = dropout
        N, T, _, H, C = qkv.shape
        ctx.rpb_shape = None if rpb is None else rpb.shape
        if rpb is not None:
            rpb = rpb.detach().reshape(H, win_size).to(torch.float32).contiguous()
        if t_valid is not None:
            assert t_valid.numel() == N
            t_valid = t_valid.to(device=qkv.device, dtype=torch.int32).contiguous()
        q4, k4, v4 = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))       # [N, H, T, C] views
        out = torch.empty((N, T, H, C), dtype=qkv.dtype, device=qkv.device)
        o4 = out.permute(0, 2, 1, 3)
        lses, ctx.packed_outs = [], []
        for r in range(min(dilation, T)):                                         # see _FusedNA1D.forward
            qr = _residue(q4, r, dilation)
            lse = torch.empty((N * H, qr.shape[2]), dtype=torch.float32, device=qkv.device)
            ctx.packed_outs.append(_strided_or_packed_forward(
                _residue(o4, r, dilation), lse, qr, _residue(k4, r, dilation), _residue(v4, r, dilation), rpb,
                _residue_lengths(t_valid, r, dilation), win_size, left, scale,
                dropout=None if dropout is None else (*dropout, dilation, r, T)))
            lses.append(lse)
        ctx.save_for_backward(qkv, rpb, t_valid, *lses)
        ctx.geom = (win_size, left, scale, deterministic, dilation)
        return out.view(N, T, H * C)

    @staticmethod
    def backward(ctx, dout):
        qkv, rpb, t_valid, *lses = ctx.saved_tensors
        win_size, left, scale, deterministic, dilation = ctx.geom
        N, T, _, H, C = qkv.shape
        g4 = dout.contiguous().view(N, T, H, C).permute(0, 2, 1, 3)
        dqkv = torch.empty_like(qkv)
        drpb = ws = None
        if rpb is not None and ctx.needs_input_grad[1]:
            drpb = torch.zeros((H, win_size), dtype=torch.float32, device=qkv.device)
            if deterministic:
                ws = _deterministic_workspace(N * H, H, T, C, win_size, left, qkv, dilation)
        views = [dqkv[:, :, i].permute(0, 2, 1, 3) for i in range(3)] + [qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3)]
        for r, lse in enumerate(lses):
            a = [_residue(z, r, dilation) for z in views]
            _strided_or_packed_backward(a[0], a[1], a[2], drpb, a[3], a[4], a[5], ctx.packed_outs[r],
                                        _residue(g4, r, dilation), lse, rpb, _residue_lengths(t_valid, r, dilation),
                                        win_size, left, scale, ws,
                                        dropout=None if ctx.dropout is None else (*ctx.dropout, dilation, r, T))
        if drpb is not None:
            drpb = drpb.view(ctx.rpb_shape)
        return dqkv, drpb, None, None, None, None, None, None, None


def na1d_fused_qkv(qkv, win_size, left, rpb=None, t_valid=None, scale=1.0, deterministic=False, dilation=1,
                   dropout_p=0.0, seed=None):
    """Fused neighbourhood attention on a token-major qkv projection output.

    qkv : contiguous ``[N, T, 3, H, C]`` bf16/fp16 (the ``[N, T, 3*dim]`` output of the projection, viewed).
          The kernels read each head's rows in place and write ``[N, T, H*C]`` directly, so the head split
          and merge copies of the reference (models/MFA_NATransformer.py:127-138,150-151) do not exist; the
          gradient comes back as one ``[N, T, 3, H, C]`` tensor.  ``scale`` multiplies the fp32 scores (the
          reference multiplies q by it in 16 bit beforehand).
    Other arguments as in :func:`na1d_fused`; with ``dropout_p`` the mask is the one :func:`na1d_fused` draws for the
    same seed on the split tensors (sequence n * H + h, row, slot).
    """
    dropout = None
    if dropout_p > 0.0:
        assert dropout_p < 1.0
        if seed is None:
            seed = int(torch.randint(0, 2 ** 62, (1,)).item())
        dropout = (float(dropout_p), int(seed))
    if dropout is None and dilation == 1 and not (torch.is_grad_enabled() and (qkv.requires_grad or (rpb is not None and rpb.requires_grad))):
        # inference: one library call, no views, no log-sum-exp
        assert qkv.dim() == 5 and qkv.shape[2] == 3 and qkv.is_contiguous()
        N, T, _, H, C = qkv.shape
        if rpb is not None:
            rpb = rpb.detach().reshape(H, win_size)
            if rpb.dtype != torch.float32 or not rpb.is_contiguous():
                rpb = rpb.to(torch.float32).contiguous()
        if t_valid is not None:
            assert t_valid.numel() == N
            t_valid = t_valid.to(device=qkv.device, dtype=torch.int32).contiguous()
        out = torch.empty((N, T, H * C), dtype=qkv.dtype, device=qkv.device)
        if N * T == 0 or _lib.call_fused_forward_qkv(out, None, qkv, rpb, t_valid, win_size, left, float(scale)) == 0:
            return out
    return _FusedNA1DQKV.apply(qkv, rpb, t_valid, win_size, left, float(scale), bool(deterministic), int(dilation),
                               dropout)
