"""The NA1D operators as ``torch.library`` ops, so that ``torch.compile`` traces through them.

This is the second statement of the reference's operator boundary (its build for torch >= 2.4:
``extension_na/na_cuda/csrc_tc240_or_bigger/main.cpp:27-41`` declares twelve ops
``na_cuda::{bf16,fp16}_ana_{qk_forward,q_backward,k_backward,av_forward,attn_backward,v_backward}``
``(Tensor, Tensor, int N, int T, int C, int win_size, int left) -> Tensor``, callee allocating, and
``extension_na/na_cuda/ops_tc240_or_bigger.py:15-44,51-300`` gives them fake kernels, autograd formulas and the
wrappers ``ana_qk`` / ``ana_av``).  The same names, schemas and semantics are registered here on top of libna1d,
so code written against ``torch.ops.na_cuda.*`` runs unchanged; importing this module is what registers them.

Beyond the reference, the fused operator is registered the same way:
``na_cuda::na1d_fused_forward`` / ``na_cuda::na1d_fused_backward`` and the wrapper :func:`na1d_fused_op`.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import _lib

NAMESPACE = "na_cuda"
_SIG = "int N, int T, int C, int win_size, int left"

# op suffix -> (libna1d entry point, name of the two tensor arguments, which one is 16-bit, what comes back)
_UNFUSED = {
    "ana_qk_forward": ("na1d_qk_forward", ("query", "key"), 0, "scores"),
    "ana_q_backward": ("na1d_q_backward", ("attn_gd", "key"), 1, "rows"),
    "ana_k_backward": ("na1d_k_backward", ("attn_gd", "query"), 1, "rows"),
    "ana_av_forward": ("na1d_av_forward", ("attn", "value"), 1, "rows"),
    "ana_attn_backward": ("na1d_a_backward", ("result_gd", "value"), 0, "scores"),
    "ana_v_backward": ("na1d_v_backward", ("attn", "result_gd"), 1, "rows"),
}
_DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16}

_library = torch.library.Library(NAMESPACE, "FRAGMENT")   # kept alive for the life of the process


def _checked(a: Tensor, b: Tensor, half: int, dtype: torch.dtype, N: int, T: int, C: int, win_size: int, kind: str):
    """Argument contract shared by the real and the fake kernels; returns the output's (shape, dtype).  Layout is
    not part of it: a compiler backend may hand an op a tensor with other strides than the eager program had, so
    the real kernels pack what is not contiguous, as the reference's ops do (ops_tc240_or_bigger.py:68)."""
    x16, x32 = (a, b)[half], (a, b)[1 - half]
    torch._check(a.device == b.device, lambda: "NA1D operands must be on one device")
    torch._check(x16.dtype == dtype and tuple(x16.shape) == (N, T, C), lambda: "bad 16-bit operand")
    if kind == "rows":                                    # the other operand is the fp32 score tensor
        torch._check(x32.dtype == torch.float32 and tuple(x32.shape) == (N, T, win_size), lambda: "bad score tensor")
        return (N, T, C), dtype
    torch._check(x32.dtype == dtype and tuple(x32.shape) == (N, T, C), lambda: "bad second operand")
    return (N, T, win_size), torch.float32


def _define_unfused(prefix: str, dtype: torch.dtype, suffix: str):
    entry, (first, second), half, kind = _UNFUSED[suffix]
    name = "%s_%s" % (prefix, suffix)
    _library.define("%s(Tensor %s, Tensor %s, %s) -> Tensor" % (name, first, second, _SIG))

    def kernel(a, b, N, T, C, win_size, left):
        shape, out_dtype = _checked(a, b, half, dtype, N, T, C, win_size, kind)
        out = torch.empty(shape, dtype=out_dtype, device=a.device)
        _lib.call_unfused(entry, out, a.contiguous(), b.contiguous(), N, T, C, win_size, left, dtype)
        return out

    def fake(a, b, N, T, C, win_size, left):
        shape, out_dtype = _checked(a, b, half, dtype, N, T, C, win_size, kind)
        return torch.empty(shape, dtype=out_dtype, device=a.device)

    _library.impl(name, kernel, "CUDA")
    torch.library.register_fake("%s::%s" % (NAMESPACE, name), fake, lib=_library)


def _register_autograd(prefix: str):
    ops = getattr(torch.ops, NAMESPACE)
    q_bwd, k_bwd = getattr(ops, prefix + "_ana_q_backward"), getattr(ops, prefix + "_ana_k_backward")
    a_bwd, v_bwd = getattr(ops, prefix + "_ana_attn_backward"), getattr(ops, prefix + "_ana_v_backward")

    def setup(ctx, inputs, output):
        a, b, _N, _T, _C, ctx.win_size, ctx.left = inputs
        ctx.save_for_backward(a, b)

    def qk_backward(ctx, attn_gd):                       # nattn.py:46-54
        q, k = ctx.saved_tensors
        N, T, C = q.shape
        g = attn_gd.contiguous()
        return (q_bwd(g, k, N, T, C, ctx.win_size, ctx.left), k_bwd(g, q, N, T, C, ctx.win_size, ctx.left),
                None, None, None, None, None)

    def av_backward(ctx, result_gd):                     # nattn.py:69-78
        attn, v = ctx.saved_tensors
        N, T, C = v.shape
        g = result_gd.contiguous()
        return (a_bwd(g, v, N, T, C, ctx.win_size, ctx.left), v_bwd(attn, g, N, T, C, ctx.win_size, ctx.left),
                None, None, None, None, None)

    torch.library.register_autograd("%s::%s_ana_qk_forward" % (NAMESPACE, prefix), qk_backward, setup_context=setup,
                                    lib=_library)
    torch.library.register_autograd("%s::%s_ana_av_forward" % (NAMESPACE, prefix), av_backward, setup_context=setup,
                                    lib=_library)


for _prefix, _dtype in _DTYPES.items():
    for _suffix in _UNFUSED:
        _define_unfused(_prefix, _dtype, _suffix)
    _register_autograd(_prefix)


def _prefix_of(t: Tensor) -> str:
    for prefix, dtype in _DTYPES.items():
        if t.dtype == dtype:
            return prefix
    raise AssertionError("NA1D operands must be bf16 or fp16, got %s" % t.dtype)


def ana_qk(q: Tensor, k: Tensor, win_size: int, left: int) -> Tensor:
    """Band QK^T: fp32 ``[N, T, win_size]`` (ops_tc240_or_bigger.py:15-29)."""
    assert q.is_contiguous() and k.is_contiguous() and q.dtype == k.dtype
    N, T, C = q.shape
    return getattr(getattr(torch.ops, NAMESPACE), _prefix_of(q) + "_ana_qk_forward")(q, k, N, T, C, win_size, left)


def ana_av(attn: Tensor, v: Tensor, win_size: int, left: int) -> Tensor:
    """Band . V: ``[N, T, C]`` in v's dtype (ops_tc240_or_bigger.py:31-44)."""
    assert attn.is_contiguous() and v.is_contiguous() and attn.dtype == torch.float32
    N, T, C = v.shape
    return getattr(getattr(torch.ops, NAMESPACE), _prefix_of(v) + "_ana_av_forward")(attn, v, N, T, C, win_size, left)


# --------------------------------------------------------------------------- the fused operator
_library.define("na1d_fused_forward(Tensor q, Tensor k, Tensor v, Tensor? rpb, Tensor? t_valid, int num_heads, "
                "int win_size, int left, float scale) -> (Tensor, Tensor)")
_library.define("na1d_fused_backward(Tensor dout, Tensor q, Tensor k, Tensor v, Tensor out, Tensor lse, Tensor? rpb, "
                "Tensor? t_valid, int num_heads, int win_size, int left, float scale, bool want_drpb) "
                "-> (Tensor, Tensor, Tensor, Tensor)")


def _fused_contract(q, k, v, rpb, t_valid, num_heads, win_size):
    torch._check(q.dim() == 3 and q.shape == k.shape == v.shape, lambda: "q, k, v must all be [B, T, C]")
    torch._check(q.dtype == k.dtype == v.dtype and q.dtype in _DTYPES.values(), lambda: "q, k, v must be bf16 or fp16")
    torch._check(q.shape[0] % num_heads == 0, lambda: "B must be a multiple of num_heads")
    if rpb is not None:
        torch._check(rpb.dtype == torch.float32 and tuple(rpb.shape) == (num_heads, win_size),
                     lambda: "rpb must be fp32 [num_heads, win_size]")
    if t_valid is not None:
        torch._check(t_valid.dtype == torch.int32 and t_valid.numel() == q.shape[0] // num_heads,
                     lambda: "t_valid must be int32 [B / num_heads]")


def _fused_forward(q, k, v, rpb, t_valid, num_heads, win_size, left, scale):
    _fused_contract(q, k, v, rpb, t_valid, num_heads, win_size)
    B, T, C = q.shape
    q, k, v, rpb, t_valid = _packed(q, k, v, rpb, t_valid)
    out = torch.empty_like(q)
    lse = torch.empty((B, T), dtype=torch.float32, device=q.device)
    _lib.call_fused_forward(out, lse, q, k, v, rpb, t_valid, B, num_heads, T, C, win_size, left, scale)
    return out, lse


def _packed(*tensors):
    return tuple(None if t is None else t.contiguous() for t in tensors)


def _like(q):
    return torch.empty(q.shape, dtype=q.dtype, device=q.device)      # contiguous, whatever q's strides


def _fused_forward_fake(q, k, v, rpb, t_valid, num_heads, win_size, left, scale):
    _fused_contract(q, k, v, rpb, t_valid, num_heads, win_size)
    return _like(q), torch.empty(q.shape[:2], dtype=torch.float32, device=q.device)


def _fused_backward(dout, q, k, v, out, lse, rpb, t_valid, num_heads, win_size, left, scale, want_drpb):
    B, T, C = q.shape
    dout, q, k, v, out, lse, rpb, t_valid = _packed(dout, q, k, v, out, lse, rpb, t_valid)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    drpb = torch.zeros((num_heads, win_size) if want_drpb else (0,), dtype=torch.float32, device=q.device)
    _lib.call_fused_backward(dq, dk, dv, drpb if want_drpb else None, q, k, v, out, dout, lse, rpb,
                             t_valid, B, num_heads, T, C, win_size, left, scale)
    return dq, dk, dv, drpb


def _fused_backward_fake(dout, q, k, v, out, lse, rpb, t_valid, num_heads, win_size, left, scale, want_drpb):
    drpb = torch.empty((num_heads, win_size) if want_drpb else (0,), dtype=torch.float32, device=q.device)
    return _like(q), _like(k), _like(v), drpb


_library.impl("na1d_fused_forward", _fused_forward, "CUDA")
_library.impl("na1d_fused_backward", _fused_backward, "CUDA")
torch.library.register_fake(NAMESPACE + "::na1d_fused_forward", _fused_forward_fake, lib=_library)
torch.library.register_fake(NAMESPACE + "::na1d_fused_backward", _fused_backward_fake, lib=_library)


def _fused_setup(ctx, inputs, output):
    q, k, v, rpb, t_valid, ctx.num_heads, ctx.win_size, ctx.left, ctx.scale = inputs
    out, lse = output
    ctx.has_rpb, ctx.has_tv = rpb is not None, t_valid is not None
    ctx.save_for_backward(*[t for t in (q, k, v, out, lse, rpb, t_valid) if t is not None])


def _fused_autograd(ctx, dout, _dlse):
    saved = list(ctx.saved_tensors)
    q, k, v, out, lse = saved[:5]
    rest = saved[5:]
    rpb = rest.pop(0) if ctx.has_rpb else None
    t_valid = rest.pop(0) if ctx.has_tv else None
    want = ctx.has_rpb and ctx.needs_input_grad[3]
    dq, dk, dv, drpb = getattr(torch.ops, NAMESPACE).na1d_fused_backward(
        dout, q, k, v, out, lse, rpb, t_valid, ctx.num_heads, ctx.win_size, ctx.left, ctx.scale, want)
    return dq, dk, dv, (drpb if want else None), None, None, None, None, None


torch.library.register_autograd(NAMESPACE + "::na1d_fused_forward", _fused_autograd, setup_context=_fused_setup,
                                lib=_library)


def na1d_fused_op(q: Tensor, k: Tensor, v: Tensor, win_size: int, left: int, rpb: Optional[Tensor] = None,
                  t_valid: Optional[Tensor] = None, num_heads: int = 1, scale: float = 1.0) -> Tensor:
    """:func:`na1d_amd.na1d_fused` through the registered op (traceable by ``torch.compile``).  ``rpb`` is
    ``[num_heads, win_size]`` fp32 (reshape the model's ``[1, H, 1, W]`` parameter), ``t_valid`` int32 ``[N]``."""
    return getattr(torch.ops, NAMESPACE).na1d_fused_forward(q, k, v, rpb, t_valid, num_heads, win_size, left,
                                                            float(scale))[0]


# --------------------------------------------------------------------------- dense attention of the global layers
_library.define("global_attention_forward(Tensor q, Tensor k, Tensor v, Tensor? t_valid, int num_heads, float scale) "
                "-> (Tensor, Tensor)")
_library.define("global_attention_backward(Tensor dout, Tensor q, Tensor k, Tensor v, Tensor out, Tensor lse, "
                "Tensor? t_valid, int num_heads, float scale) -> (Tensor, Tensor, Tensor)")


def _dense_forward(q, k, v, t_valid, num_heads, scale):
    _fused_contract(q, k, v, None, t_valid, num_heads, 0)
    B, T, C = q.shape
    q, k, v, t_valid = _packed(q, k, v, t_valid)
    out = torch.empty_like(q)
    lse = torch.empty((B, T), dtype=torch.float32, device=q.device)
    torch._check(_lib.call_global_forward(out, lse, q, k, v, t_valid, B, num_heads, T, C, scale) == 0,
                 lambda: "dense attention covers head_dim <= 128")
    return out, lse


def _dense_forward_fake(q, k, v, t_valid, num_heads, scale):
    _fused_contract(q, k, v, None, t_valid, num_heads, 0)
    return _like(q), torch.empty(q.shape[:2], dtype=torch.float32, device=q.device)


def _dense_backward(dout, q, k, v, out, lse, t_valid, num_heads, scale):
    B, T, C = q.shape
    dout, q, k, v, out, lse, t_valid = _packed(dout, q, k, v, out, lse, t_valid)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if B * T:
        ws = torch.empty(_lib.global_backward_workspace_bytes(B, num_heads, T, C, q.dtype), dtype=torch.uint8,
                         device=q.device)
        _lib.call_global_backward(dq, dk, dv, q, k, v, out, dout, lse, t_valid, B, num_heads, T, C, scale, ws)
    return dq, dk, dv


def _dense_backward_fake(dout, q, k, v, out, lse, t_valid, num_heads, scale):
    return _like(q), _like(k), _like(v)


_library.impl("global_attention_forward", _dense_forward, "CUDA")
_library.impl("global_attention_backward", _dense_backward, "CUDA")
torch.library.register_fake(NAMESPACE + "::global_attention_forward", _dense_forward_fake, lib=_library)
torch.library.register_fake(NAMESPACE + "::global_attention_backward", _dense_backward_fake, lib=_library)


def _dense_setup(ctx, inputs, output):
    q, k, v, t_valid, ctx.num_heads, ctx.scale = inputs
    out, lse = output
    ctx.has_tv = t_valid is not None
    ctx.save_for_backward(*[t for t in (q, k, v, out, lse, t_valid) if t is not None])


def _dense_autograd(ctx, dout, _dlse):
    saved = list(ctx.saved_tensors)
    q, k, v, out, lse = saved[:5]
    t_valid = saved[5] if ctx.has_tv else None
    dq, dk, dv = getattr(torch.ops, NAMESPACE).global_attention_backward(dout, q, k, v, out, lse, t_valid,
                                                                         ctx.num_heads, ctx.scale)
    return dq, dk, dv, None, None, None


torch.library.register_autograd(NAMESPACE + "::global_attention_forward", _dense_autograd, setup_context=_dense_setup,
                                lib=_library)


def global_attention_op(q: Tensor, k: Tensor, v: Tensor, num_heads: int = 1, t_valid: Optional[Tensor] = None,
                        scale: float = 1.0) -> Tensor:
    """:func:`na1d_amd.dense.global_attention` through the registered op (traceable by ``torch.compile``)."""
    return getattr(torch.ops, NAMESPACE).global_attention_forward(q, k, v, t_valid, num_heads, float(scale))[0]
