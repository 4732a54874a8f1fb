"""Drop-in for the reference's operator API (na1d_tensorcore/nattn.py:32-137).

``getNA1dFunction(C, dilation, dtype)`` returns the two ``autograd.Function``
classes the models call as ``QK.apply(q * scale, k, win_size, left, dilation)``
and ``AV.apply(attn, v, win_size, left, dilation)``
(models/PCF_NATransformer.py:85,141,150).  Layouts, dtypes, saved tensors and
the 5-tuple backward returns are those of the reference; the kernels behind
them are the gfx950 HIP kernels of libna1d, launched on torch's current stream.
The library is prebuilt - nothing is compiled at import (the reference JITs at
import from a cwd-relative path, nattn.py:10-29).
"""
from __future__ import annotations

import torch

from . import _lib


def _check_qk(q, k, win_size, left):
    # nattn.py:35-37 asserts; ours also reject what the reference lets through silently
    assert q.is_contiguous()
    assert k.is_contiguous()
    assert q.dtype == k.dtype
    assert q.dim() == 3 and q.shape == k.shape, "q and k must both be [B, T, C]"


def _make_functions(dtype: torch.dtype, prefix: str):
    """Build the (QK, AV) pair for one 16-bit dtype."""

    class QK(torch.autograd.Function):
        # forward/backward of nattn.py:32-54 (bf16) and :80-102 (fp16)
        @staticmethod
        def forward(ctx, q, k, win_size, left, dilation=1):
            _check_qk(q, k, win_size, left)
            assert q.dtype == dtype, "this Function was built for %s" % dtype
            B, T, C = q.shape
            attn = torch.empty((B, T, win_size), dtype=torch.float32, device=q.device)
            _lib.call_unfused("na1d_qk_forward", attn, q, k, B, T, C, win_size, left, dtype)
            ctx.save_for_backward(q, k)
            ctx.win_size = win_size
            ctx.left = left
            return attn

        @staticmethod
        def backward(ctx, attn_gd):
            q, k = ctx.saved_tensors
            B, T, C = q.shape
            # the reference passes attn_gd as it arrives (nattn.py:46-54); its newer
            # packaging makes it contiguous first (ops_tc240_or_bigger.py:68) and so do we
            attn_gd = attn_gd.contiguous()
            q_gd = torch.empty(q.shape, dtype=q.dtype, device=attn_gd.device)
            _lib.call_unfused("na1d_q_backward", q_gd, attn_gd, k, B, T, C, ctx.win_size, ctx.left, dtype)
            k_gd = torch.empty(k.shape, dtype=k.dtype, device=attn_gd.device)
            _lib.call_unfused("na1d_k_backward", k_gd, attn_gd, q, B, T, C, ctx.win_size, ctx.left, dtype)
            return (q_gd, k_gd, None, None, None)

    class AV(torch.autograd.Function):
        # forward/backward of nattn.py:56-78 (bf16) and :104-126 (fp16)
        @staticmethod
        def forward(ctx, attn, v, win_size, left, dilation=1):
            assert attn.is_contiguous()
            assert v.is_contiguous()
            assert v.dtype == dtype, "this Function was built for %s" % dtype
            assert attn.dtype == torch.float32, "attn must be fp32 [B, T, win_size]"
            B, T, C = v.shape
            assert attn.shape == (B, T, win_size)
            result = torch.empty(v.shape, dtype=v.dtype, device=v.device)
            _lib.call_unfused("na1d_av_forward", result, attn, v, B, T, C, win_size, left, dtype)
            ctx.save_for_backward(attn, v)
            ctx.win_size = win_size
            ctx.left = left
            return result

        @staticmethod
        def backward(ctx, result_gd):
            result_gd = result_gd.contiguous()
            B, T, C = result_gd.shape
            attn, v = ctx.saved_tensors
            attn_gd = torch.empty(attn.shape, dtype=attn.dtype, device=result_gd.device)
            _lib.call_unfused("na1d_a_backward", attn_gd, result_gd, v, B, T, C, ctx.win_size, ctx.left, dtype)
            v_gd = torch.empty(v.shape, dtype=v.dtype, device=result_gd.device)
            _lib.call_unfused("na1d_v_backward", v_gd, attn, result_gd, B, T, C, ctx.win_size, ctx.left, dtype)
            return (attn_gd, v_gd, None, None, None)

    QK.__name__ = QK.__qualname__ = prefix + "_ANA1d_QK_Function"
    AV.__name__ = AV.__qualname__ = prefix + "_ANA1d_AV_Function"
    return QK, AV


bf16_ANA1d_QK_Function, bf16_ANA1d_AV_Function = _make_functions(torch.bfloat16, "bf16")
fp16_ANA1d_QK_Function, fp16_ANA1d_AV_Function = _make_functions(torch.float16, "fp16")


def getNA1dFunction(C, dilation, dtype):
    """nattn.py:128-137: same asserts, same return order ``(QK, AV)``."""
    assert C % 8 == 0
    assert dilation == 1
    if dtype == torch.bfloat16:
        return bf16_ANA1d_QK_Function, bf16_ANA1d_AV_Function
    elif dtype == torch.float16:
        return fp16_ANA1d_QK_Function, fp16_ANA1d_AV_Function
    else:
        assert False, "NA1D kernels exist for torch.bfloat16 and torch.float16 only"
