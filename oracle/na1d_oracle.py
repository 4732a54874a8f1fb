"""CPU oracle for 1-D neighbourhood attention (NA1D).  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only the test-suite, the smoke
entry point and the ``cpu_baseline`` leg of the benchmark may import it.  The
shipped operator lives in the HIP library and must fail loudly without it.

It restates, in plain PyTorch CPU arithmetic (fp32 or fp64, chosen by the
dtype of the tensors passed in), the math of the reference's CPU branch and of
the autograd wiring around its kernels:

* window split ``win_size -> (W, left)``      models/PCF_NATransformer.py:46-54
* additive -100 mask                           models/PCF_NATransformer.py:87-99
* band QK^T (P1), zero filled outside [0,T)    models/PCF_NATransformer.py:161,
                                               na1d_tensorcore/bf16_ana1d_kernel.cu:100-111
* bias + mask + softmax                        models/PCF_NATransformer.py:143-148,163-165
* band . V (P2)                                models/PCF_NATransformer.py:172
* inverse-neighbourhood gather (P3)            na1d_tensorcore/bf16_ana1d_kernel.cu:457-459,
                                               na1d_tensorcore/nattn.py:46-54,69-78
* dilation > 1 (CPU only in the reference)     models/PCF_NATransformer.py:101-116,158-159,169-170
* dense attention of the global layers         models/PCF_NATransformer.py:215-221, mask :406-414

What pins each function (see tests/test_oracle_pins.py): brute-force index
loops on tiny shapes, W=1 row dots, the dense ``q @ k^T`` embedding for
``L=T-1, W=2T-1``, ``k=1`` zero-fill, one-hot / uniform probabilities for P2,
the exact adjoint identities between P1/P2/P3, closed-form masks, library
softmax on the valid slots, and ``torch.autograd.gradcheck`` in fp64; the dense
attention by index loops, ``F.scaled_dot_product_attention`` with the same mask,
the closed-form mask, the full-window NA1D it must agree with, and gradcheck; the
dropout hash by a C program compiled from an independent transcription of the rule
in include/na1d.h, bijectivity of the finaliser, and keep-rate / independence statistics.
No function here is "parity unpinned".

Layout everywhere: ``q, k, v : [B, T, C]`` with ``B = N * H`` (batch major,
head minor), scores / probabilities ``[B, T, W]``; slot ``j`` of query ``t``
addresses key ``t - left + j`` (``t + (j - left) * dilation`` when dilated).
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

MASK_VALUE = -100.0   # models/PCF_NATransformer.py:98


# --------------------------------------------------------------------------
# window geometry
# --------------------------------------------------------------------------
def split_window(win_size):
    """``int`` or ``[W, left]`` -> ``(W, left)``; models/PCF_NATransformer.py:46-54."""
    if isinstance(win_size, int):
        if win_size <= 0:
            raise ValueError("win_size must be positive")
        W, left = win_size, win_size - 1 - win_size // 2
    else:
        if len(win_size) != 2:
            raise ValueError("win_size list must be [W, left]")
        W, left = int(win_size[0]), int(win_size[1])
    if W > 80:
        raise ValueError("win_size must be <= 80")
    if not (0 <= left < W):
        raise ValueError("need 0 <= left < win_size")
    return W, left


def _windows(x, W, left, dilation=1):
    """[B,T,C] -> [B,T,W,C]; row ``t`` slot ``j`` is ``x[t+(j-left)*dilation]`` or 0.

    The undilated case is the reference's ``F.pad(...).unfold(...)``
    (models/PCF_NATransformer.py:161,172).
    """
    B, T, C = x.shape
    right = W - 1 - left
    xp = F.pad(x, (0, 0, left * dilation, right * dilation))
    if dilation == 1:
        return xp.unfold(1, W, 1).permute(0, 1, 3, 2)            # [B,T,W,C]
    idx = (torch.arange(T).unsqueeze(1) + torch.arange(W).unsqueeze(0) * dilation)  # padded coords
    return xp[:, idx]                                             # [B,T,W,C]


# --------------------------------------------------------------------------
# the three primitives
# --------------------------------------------------------------------------
def qk_band(q, k, W, left, dilation=1):
    """P1: ``S[b,t,j] = sum_c q[b,t,c] * k~[b,t-left+j,c]`` (k~ = 0 outside [0,T))."""
    return torch.einsum("btc,btwc->btw", q, _windows(k, W, left, dilation))


def av_band(p, v, W, left, dilation=1):
    """P2: ``O[b,t,c] = sum_j p[b,t,j] * v~[b,t-left+j,c]``."""
    return torch.einsum("btw,btwc->btc", p, _windows(v, W, left, dilation))


def inverse_gather(s, x, W, left, dilation=1):
    """P3: ``O[b,u,c] = sum_j s[b,u+left-j,j] * x[b,u+left-j,c]`` over valid rows.

    Written as the scatter of every (t, j) pair onto key ``u = t-left+j`` so that
    it shares no indexing code with :func:`_windows`.
    """
    B, T, C = x.shape
    out = torch.zeros_like(x)
    for j in range(W):
        off = (j - left) * dilation            # key = t + off
        lo, hi = max(0, -off), min(T, T - off)  # queries whose key is in range
        if hi > lo:
            out[:, lo + off:hi + off] += s[:, lo:hi, j:j + 1] * x[:, lo:hi]
    return out


# --------------------------------------------------------------------------
# mask, softmax, fused forms
# --------------------------------------------------------------------------
def attn_mask(T, W, left, padding=None, dilation=1, dtype=torch.float32):
    """[N,T,W] additive mask: -100 where the query row is padded or the key is
    outside ``[0, T - pad_n)``, else 0.  A single fill, never -200.
    models/PCF_NATransformer.py:87-99 (dilated :101-116).
    """
    if padding is None:
        padding = torch.zeros(1, dtype=torch.int64)
    padding = torch.as_tensor(padding, dtype=torch.int64).reshape(-1)
    t_valid = (T - padding).view(-1, 1, 1)                      # [N,1,1]
    t = torch.arange(T).view(1, T, 1)
    key = t + (torch.arange(W).view(1, 1, W) - left) * dilation
    bad = (t >= t_valid) | (key < 0) | (key >= t_valid)
    return torch.zeros(bad.shape, dtype=dtype).masked_fill(bad, MASK_VALUE)


def logits(q, k, W, left, rpb=None, padding=None, num_heads=1, dilation=1):
    """``S + rpb[h] + mask[n]`` in the order the reference adds them (:143-146)."""
    B, T, _ = q.shape
    z = qk_band(q, k, W, left, dilation)
    N = B // num_heads
    z = z.view(N, num_heads, T, W)
    if rpb is not None:
        z = z + rpb.to(z.dtype).view(1, num_heads, 1, W)
    m = attn_mask(T, W, left, padding, dilation, dtype=z.dtype)  # [N or 1, T, W]
    z = z + m.unsqueeze(1)
    return z.view(B, T, W)


def _mix32(x):
    """The 32-bit finaliser of the dropout hash on a uint32 array (wrapping arithmetic)."""
    x = x ^ (x >> np.uint32(16))
    x = x * np.uint32(0x7FEB352D)
    x = x ^ (x >> np.uint32(15))
    x = x * np.uint32(0x846CA68B)
    return x ^ (x >> np.uint32(16))


def dropout_keep(B, T, W, p, seed):
    """bool ``[B, T, W]``: which probabilities the fused operator's attention dropout keeps - the rule stated
    in include/na1d.h for na1d_fused_forward_dropout, a hash of (seed, row = b*T + t, slot j) against
    ``floor(p * 2^32)``.  Stands where the reference has nn.Dropout (models/PCF_NATransformer.py:71,149);
    the random stream is this library's own, the distribution (independent, keep rate 1 - p) is the reference's.
    """
    return torch.from_numpy(dropout_keep_rows(np.arange(B * T, dtype=np.uint64), W, p, seed)).view(B, T, W)


def dropout_keep_rows(row, W, p, seed):
    """The same for explicit row numbers ``b*T + t`` (uint64 array) -> bool ``[len(row), W]``."""
    gold = np.uint32(0x9E3779B9)
    with np.errstate(over="ignore"):
        row = np.asarray(row, dtype=np.uint64)
        lo, hi = (row & np.uint64(0xFFFFFFFF)).astype(np.uint32), (row >> np.uint64(32)).astype(np.uint32)
        key = _mix32(_mix32(lo ^ np.uint32(seed & 0xFFFFFFFF)) + hi * gold + np.uint32((seed >> 32) & 0xFFFFFFFF))
        h = _mix32(key[:, None] ^ (np.arange(W, dtype=np.uint32) * gold)[None, :])
    threshold = min(int(p * 4294967296.0), 0xFFFFFFFF)
    return h >= np.uint32(threshold)


def na1d_forward(q, k, v, W, left, rpb=None, padding=None, num_heads=1, dilation=1, keep=None, p_drop=0.0):
    """Full NA1D: returns ``(O, P, LSE)``; ``q`` is expected pre-scaled (:141).  With ``keep`` (bool
    ``[B,T,W]``) the probabilities go through dropout before the second contraction (:149): ``O = (keep * P /
    (1 - p_drop)) . V``; the returned ``P`` and ``LSE`` are those of the softmax."""
    z = logits(q, k, W, left, rpb, padding, num_heads, dilation)
    p = torch.softmax(z, dim=-1)
    lse = torch.logsumexp(z, dim=-1)
    pd = p if keep is None else p * keep.to(p.dtype) / (1.0 - p_drop)
    return av_band(pd, v, W, left, dilation), p, lse


def na1d_backward(q, k, v, do, W, left, rpb=None, padding=None, num_heads=1, dilation=1, keep=None, p_drop=0.0):
    """Gradients by ``torch.autograd`` through :func:`na1d_forward`.

    Returns ``(dq, dk, dv, drpb)`` with ``drpb`` shaped ``[H, W]`` (``None`` without bias).
    """
    q = q.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    v = v.detach().clone().requires_grad_(True)
    leaves = [q, k, v]
    if rpb is not None:
        rpb = rpb.detach().clone().requires_grad_(True)
        leaves.append(rpb)
    o, _, _ = na1d_forward(q, k, v, W, left, rpb, padding, num_heads, dilation, keep, p_drop)
    grads = torch.autograd.grad(o, leaves, do)
    drpb = grads[3].reshape(num_heads, W) if rpb is not None else None
    return grads[0], grads[1], grads[2], drpb


def na1d_backward_formulas(q, k, v, do, W, left, rpb=None, padding=None, num_heads=1):
    """The same gradients from the explicit formulas the reference's autograd
    wiring evaluates (nattn.py:46-54,69-78 plus softmax backward):
    ``dP = P1(dO,v)``, ``dV = P3(P,dO)``, ``dS = P*(dP - sum_j P*dP)``,
    ``dQ = P2(dS,k)``, ``dK = P3(dS,q)``, ``drpb[h,j] = sum_{n,t} dS``.
    """
    B, T, _ = q.shape
    _, p, _ = na1d_forward(q, k, v, W, left, rpb, padding, num_heads)
    dp = qk_band(do, v, W, left)
    dv = inverse_gather(p, do, W, left)
    ds = p * (dp - (p * dp).sum(-1, keepdim=True))
    dq = av_band(ds, k, W, left)
    dk = inverse_gather(ds, q, W, left)
    drpb = ds.view(B // num_heads, num_heads, T, W).sum(dim=(0, 2))
    return dq, dk, dv, drpb


# --------------------------------------------------------------------------
# dense attention of the global layers
# --------------------------------------------------------------------------
def global_mask(T, padding=None, dtype=torch.float32):
    """[N,T,T] additive mask: -100 where the query row or the key column is padded, one fill (never -200).
    models/PCF_NATransformer.py:406-414.
    """
    if padding is None:
        padding = torch.zeros(1, dtype=torch.int64)
    padding = torch.as_tensor(padding, dtype=torch.int64).reshape(-1)
    t_valid = (T - padding).view(-1, 1, 1)
    t = torch.arange(T)
    bad = (t.view(1, T, 1) >= t_valid) | (t.view(1, 1, T) >= t_valid)
    return torch.zeros(bad.shape, dtype=dtype).masked_fill(bad, MASK_VALUE)


def global_forward(q, k, v, scale, padding=None, num_heads=1, keep=None, p_drop=0.0):
    """``softmax(q k^T * scale + mask) v`` per head: returns ``(O, P, LSE)``.
    models/PCF_NATransformer.py:215-221 (``q * scale`` is applied here to the product instead).  ``keep`` (bool
    ``[B,T,T]``, e.g. ``dropout_keep(B, T, T, p, seed)``): dropout on the probabilities (:218).
    """
    B, T, _ = q.shape
    z = torch.einsum("btc,buc->btu", q, k) * scale
    m = global_mask(T, padding, dtype=z.dtype)                    # [N or 1, T, T]
    z = (z.view(B // num_heads, num_heads, T, T) + m.unsqueeze(1)).view(B, T, T)
    p = torch.softmax(z, dim=-1)
    pd = p if keep is None else p * keep.to(p.dtype) / (1.0 - p_drop)
    return torch.einsum("btu,buc->btc", pd, v), p, torch.logsumexp(z, dim=-1)


def global_backward(q, k, v, do, scale, padding=None, num_heads=1, keep=None, p_drop=0.0):
    """``(dq, dk, dv)`` by ``torch.autograd`` through :func:`global_forward`."""
    leaves = [x.detach().clone().requires_grad_(True) for x in (q, k, v)]
    o, _, _ = global_forward(*leaves, scale, padding, num_heads, keep, p_drop)
    return torch.autograd.grad(o, leaves, do)


# --------------------------------------------------------------------------
# helpers shared by tests and the benchmark's CPU leg
# --------------------------------------------------------------------------
def rel_l2(a, b):
    """``||a-b|| / ||b||`` in fp64 (the tolerance metric of the parity tests)."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    den = b.norm().item()
    return (a - b).norm().item() / (den if den > 0 else 1.0)


def seeded_qkv(B, T, C, seed, dtype=torch.bfloat16, n=3, scale_q=None):
    """``n`` tensors ~ N(0,1) in fp32 from ``seed``, rounded to ``dtype``.

    With ``scale_q`` the first tensor is multiplied by it *in the 16-bit dtype*,
    as ``q * self.scale`` does under autocast (models/PCF_NATransformer.py:141).
    """
    g = torch.Generator().manual_seed(seed)
    out = [torch.randn(B, T, C, generator=g, dtype=torch.float32).to(dtype) for _ in range(n)]
    if scale_q is not None:
        out[0] = out[0] * scale_q
    return out
