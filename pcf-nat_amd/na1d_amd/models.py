"""The callers of the NA1D operator: PCF-NAT and MFA-NAT speaker-embedding models.

A compact restatement of the reference's model definitions
(models/PCF_NATransformer.py, models/MFA_NATransformer.py, models/Modules.py,
models/Pooling.py, models/SoftMaxLoss.py:99-138) in plain torch.nn, built so that

* module and parameter names match the reference's ``state_dict`` (a reference
  checkpoint loads with ``load_state_dict``);
* the neighbourhood attention runs through this package's operator:
  ``na="fused"`` (one HIP kernel each way, no mask or score tensor),
  ``na="fused_qkv"`` (the same kernels reading q, k, v in place from a token-major qkv projection and
  writing the merged heads directly: no head split / merge copies, no ``q * scale`` pass),
  ``na="unfused"`` (the reference's own chain QK -> +rpb -> +mask -> softmax -> AV
  through the drop-in Functions), ``na="fused_op"`` (the fused and the dense operator through their
  ``torch.library`` registrations, which ``torch.compile`` traces: the reference trains compiled,
  configs/pcf_nat4x4.yaml:28), or any callable with the signature of
  :func:`na1d_amd.na1d_fused` (tests pass a CPU function here to build a twin).

One class covers both families: PCF-NAT keeps activations channels-first
``[N, C, T]`` with grouped 1x1 convolutions and one patch embedding per block
whose output is added to the previous block's (PCF_NATransformer.py:443-448);
MFA-NAT keeps them tokens-first ``[N, T, C]`` with linear layers
(MFA_NATransformer.py:446-456).
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .dense import global_attention
from .fused import na1d_fused, na1d_fused_qkv
from .nattn import getNA1dFunction

MASK_VALUE = -100.0   # PCF_NATransformer.py:98


# --------------------------------------------------------------------------- small pieces
def sinusoid_table(dim, max_len, channels_first):
    """Modules.py:38-56: even channels sin(pos * 10000^(c/dim)), odd channels cos (note: *, not /)."""
    pos = torch.arange(max_len, dtype=torch.float32)
    c = torch.arange(dim, dtype=torch.float32)
    rate = torch.pow(torch.tensor(10000.0), c / dim)
    table = pos.unsqueeze(1) * rate.unsqueeze(0)                          # [max_len, dim]
    table = torch.where((torch.arange(dim) % 2 == 0).unsqueeze(0), torch.sin(table), torch.cos(table))
    return table.t().unsqueeze(0) if channels_first else table.unsqueeze(0)


class BatchNorm1d(nn.BatchNorm1d):
    """nn.BatchNorm1d through torch's own kernels: the vendor library's inference kernel is an order of magnitude
    off the memory roofline at these shapes ([256, 256, 100] bf16 measured 98 us there, 21 us here)."""

    def forward(self, x):
        was = torch.backends.cudnn.enabled
        torch.backends.cudnn.enabled = False
        try:
            return super().forward(x)
        finally:
            torch.backends.cudnn.enabled = was


class Conv1x1(nn.Conv1d):
    """A (grouped) per-token projection on [N, C, T] as ONE batched matrix product, the group blocks sitting on
    the diagonal of a dense weight.  Same parameters, names and arithmetic as nn.Conv1d(cin, cout, 1, groups=g);
    the library's grouped convolution spends more time transposing to and from its own layout than computing."""

    def __init__(self, cin, cout, bias=True, groups=1):
        super().__init__(cin, cout, 1, bias=bias, groups=groups)

    def forward(self, x):
        w, b = _prepared(self, "dense", x, lambda: (_dense_weight(self), self.bias))
        y = torch.bmm(w.unsqueeze(0).expand(x.shape[0], -1, -1), x)
        return y if b is None else y.add_(b.view(1, -1, 1))


class PatchConv(nn.Conv1d):
    """nn.Conv1d(cin, cout, kernel_size=p, stride=p, groups=g): non-overlapping patches, so again one batched
    matrix product, on the input regrouped to [N, cin*p, T/p]."""

    def __init__(self, cin, cout, patch, groups=1):
        super().__init__(cin, cout, kernel_size=patch, stride=patch, groups=groups)

    def forward(self, x):
        n, cin, t = x.shape
        p, g = self.kernel_size[0], self.groups
        tp = (t - p) // p + 1
        xr = x[:, :, :tp * p].reshape(n, cin, tp, p).transpose(2, 3).reshape(n, cin * p, tp)
        def build():
            w = self.weight.reshape(self.out_channels, -1)                   # [cout, (cin/g) * p]
            return (torch.block_diag(*w.view(g, self.out_channels // g, -1)) if g > 1 else w), self.bias
        w, b = _prepared(self, "dense", x, build)
        return torch.bmm(w.unsqueeze(0).expand(n, -1, -1), xr).add_(b.view(1, -1, 1))


class TokenBatchNorm(nn.Module):
    """BatchNorm1d over the last dim of [N, T, C] (Modules.py:26-35)."""

    def __init__(self, dim):
        super().__init__()
        self.norm = BatchNorm1d(dim)

    def forward(self, x):
        return self.norm(x.transpose(-2, -1)).transpose(-2, -1) if x.dim() >= 3 else self.norm(x)


class DropPath(nn.Module):
    def __init__(self, p):
        super().__init__()
        self.drop_prob = p

    def forward(self, x):
        if self.drop_prob == 0.0 or not self.training:
            return x
        keep = 1 - self.drop_prob
        mask = (keep + torch.rand((x.shape[0],) + (1,) * (x.dim() - 1), dtype=x.dtype, device=x.device)).floor_()
        return x.div(keep) * mask


class TDNNBlock(nn.Module):
    """conv -> ReLU -> BatchNorm (Modules.py:15-23)."""

    def __init__(self, cin, cout, kernel_size=1):
        super().__init__()
        self.conv = Conv1x1(cin, cout) if kernel_size == 1 else nn.Conv1d(cin, cout, kernel_size, padding="same")
        self.activation = nn.ReLU(inplace=True)
        self.norm = BatchNorm1d(cout)

    def forward(self, x):
        return self.norm(self.activation(self.conv(x)))

    def forward_tokens(self, x, pre_norm=None):
        """Inference on ``[N, T, C]`` (kernel size 1): one matrix product over all tokens, a batch norm in front
        (`pre_norm`) folded into it, the one behind applied as its per-channel affine map."""
        w, b, a, c = _prepared(
            self, "tokens", x,
            lambda: (_fold_norm(pre_norm, self.conv) if pre_norm is not None else (_dense_weight(self.conv), self.conv.bias))
            + _bn_affine(self.norm),
            deps=[self.conv.weight, self.conv.bias] + _bn_tensors(self.norm) + (_bn_tensors(pre_norm) if pre_norm else []))
        return torch.addcmul(c, F.relu(F.linear(x, w, b)), a)


def _length_mask(shape, lens):
    n, _, t = shape
    count = torch.round(lens * t).view(n, 1, 1)
    return torch.arange(t, device=lens.device).expand(n, 1, t) < count, count


class AttentiveStatisticsPooling(nn.Module):
    """Pooling.py:16-59 (global context on)."""

    def __init__(self, channels, attention_channels=128):
        super().__init__()
        self.eps = 1e-12
        self.tdnn = TDNNBlock(channels * 3, attention_channels, 1)
        self.tanh = nn.Tanh()
        self.conv = Conv1x1(attention_channels, channels)

    def forward(self, x, lens=None):
        if lens is None:
            mask = None
            mean = x.mean(-1, keepdim=True)
            std = torch.sqrt(x.var(-1, keepdim=True).clamp(self.eps))
        else:
            mask, count = _length_mask(x.shape, lens)
            mean = (x * mask).sum(-1, keepdim=True) / count
            std = torch.sqrt((((x - mean).pow(2) * mask).sum(-1, keepdim=True) / count).clamp(self.eps))
        ctx = torch.cat([x, mean.expand_as(x), std.expand_as(x)], dim=1)
        w = self.conv(self.tanh(self.tdnn(ctx)))
        if mask is not None:
            w = w.masked_fill(mask == 0, -torch.inf)
        w = F.softmax(w, dim=-1)
        mean = (w * x).sum(-1, keepdim=True)
        std = torch.sqrt((w * (x - mean).pow(2)).sum(-1, keepdim=True).clamp(self.eps))
        return torch.cat((mean, std), dim=1).squeeze(-1)

    def forward_tokens(self, x, lens=None):
        """The same pooling in inference on ``[N, T, C]``: reductions over T run down the columns, and the context
        ``[x, mean, std]`` is never concatenated - the first convolution is split into its three column blocks and
        the mean / std blocks, constant along T, are applied once per utterance."""
        n, t, c = x.shape
        if lens is None:
            mask = None
            mean = x.mean(1, keepdim=True)
            std = torch.sqrt(x.var(1, keepdim=True).clamp(self.eps))
        else:
            count = torch.round(lens * t).view(n, 1, 1)
            mask = torch.arange(t, device=x.device).view(1, t, 1) < count
            mean = (x * mask).sum(1, keepdim=True) / count
            std = torch.sqrt((((x - mean).pow(2) * mask).sum(1, keepdim=True) / count).clamp(self.eps))
        tdnn = self.tdnn
        w, b, a, d, w2, b2 = _prepared(
            self, "tokens", x,
            lambda: (_dense_weight(tdnn.conv), tdnn.conv.bias) + _bn_affine(tdnn.norm) + (_dense_weight(self.conv), self.conv.bias),
            deps=[tdnn.conv.weight, tdnn.conv.bias, self.conv.weight, self.conv.bias] + _bn_tensors(tdnn.norm))
        dt = w.dtype
        const = F.linear(mean.to(dt), w[:, c:2 * c]) + F.linear(std.to(dt), w[:, 2 * c:], b)        # [N, 1, A]
        h = torch.addcmul(d, F.relu(F.linear(x.to(dt), w[:, :c]) + const), a)
        logits = F.linear(torch.tanh(h), w2, b2).float()
        if mask is not None:
            logits = logits.masked_fill(~mask, -torch.inf)
        p = F.softmax(logits, dim=1)
        mean = (p * x).sum(1, keepdim=True)
        std = torch.sqrt((p * (x - mean).pow(2)).sum(1, keepdim=True).clamp(self.eps))
        return torch.cat((mean, std), dim=2).squeeze(1)


class StatisticsPooling(nn.Module):
    def __init__(self):
        super().__init__()
        self.eps = 1e-12

    def forward(self, x, lens=None):
        if lens is None:
            mean = x.mean(-1, keepdim=True)
            std = torch.sqrt(x.var(-1, keepdim=True).clamp(self.eps))
        else:
            mask, count = _length_mask(x.shape, lens)
            mean = (x * mask).sum(-1, keepdim=True) / count
            std = torch.sqrt((((x - mean).pow(2) * mask).sum(-1, keepdim=True) / count).clamp(self.eps))
        return torch.cat([mean, std], dim=1).squeeze(-1)

    def forward_tokens(self, x, lens=None):
        return self.forward(x.transpose(1, 2), lens)


# --------------------------------------------------------------------------- attention
class _TokenLinearFn(torch.autograd.Function):
    """``x @ w^T + b`` over all tokens with the weight gradient summed in chunks: ``dy^T @ x`` contracts over
    N*T tokens into a small [out, in] matrix, which the library's matrix product runs on a few dozen workgroups
    (73 us for 12800 tokens, 256 -> 768 channels); as a batched product over 8 chunks of the tokens plus a sum it
    takes 27 us."""

    @staticmethod
    def forward(ctx, x, w, b):
        dt = _compute_dtype(x)
        x16, w16 = x.to(dt), w.to(dt)
        ctx.save_for_backward(x16, w16)
        ctx.has_bias = b is not None
        with torch.autocast(x.device.type, enabled=False):
            return F.linear(x16, w16, None if b is None else b.to(dt))

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        with torch.autocast(dy.device.type, enabled=False):
            dy = dy.to(x.dtype)
            x2, dy2 = x.reshape(-1, x.shape[-1]), dy.reshape(-1, dy.shape[-1])
            m = x2.shape[0]
            chunks = next((c for c in (8, 4, 2) if m % c == 0 and m // c >= 512), 1)
            if chunks > 1:
                dw = torch.bmm(dy2.view(chunks, m // chunks, -1).transpose(1, 2), x2.view(chunks, m // chunks, -1)).sum(0, dtype=torch.float32)
            else:
                dw = (dy2.t() @ x2).float()
            dx = (dy2 @ w).view(x.shape) if ctx.needs_input_grad[0] else None
            db = dy2.sum(0, dtype=torch.float32) if ctx.has_bias else None
        return dx, dw, db


class TokenLinear(nn.Linear):
    """nn.Linear on [N, T, C] (same parameters and names); on the GPU in training the backward sums the weight
    gradient in chunks of tokens."""

    def forward(self, x):
        if x.is_cuda and torch.is_grad_enabled() and self.weight.requires_grad:
            return _TokenLinearFn.apply(x, self.weight, self.bias)
        return super().forward(x)


class _Projection(nn.Module):
    """Per-token affine map on either layout: grouped 1x1 conv on [N,C,T] or Linear on [N,T,C]."""

    @staticmethod
    def make(cin, cout, bias, groups, channels_first):
        return Conv1x1(cin, cout, bias=bias, groups=groups) if channels_first else TokenLinear(cin, cout, bias=bias)


def _split_heads(x, num_heads, groups, channels_first):
    """qkv projection output -> contiguous [3, N*H, T, hd] (PCF :126-139, MFA :127-137)."""
    if channels_first:
        n, c3, t = x.shape
        c = c3 // 3
        x = x.view(n, c // groups, groups, 3, t).transpose(1, 2).contiguous().view(n, num_heads, c // num_heads, 3, t)
        x = x.permute(3, 0, 1, 4, 2)
    else:
        n, t, c3 = x.shape
        c = c3 // 3
        x = x.view(n, t, 3, num_heads, c // num_heads).permute(2, 0, 3, 1, 4)
    return x.contiguous().view(3, n * num_heads, t, c // num_heads)


def _merge_heads(x, n, num_heads, channels_first):
    """[N*H, T, hd] -> [N, C, T] or [N, T, C] (PCF :151-152, MFA :150-151)."""
    _, t, hd = x.shape
    x = x.view(n, num_heads, t, hd)
    if channels_first:
        return x.transpose(2, 3).contiguous().view(n, num_heads * hd, t)
    return x.transpose(1, 2).contiguous().view(n, t, num_heads * hd)


def _prepared(module, tag, like, build, deps=None):
    """`build()` -> tuple of tensors derived from `module`'s parameters (dense / reordered weights, biases), cast
    to the dtype the product on `like` runs in.  While autograd is recording they are rebuilt every call (the
    gradient has to reach the parameters); otherwise they are kept until a parameter changes.  `deps`: the
    tensors `build` reads, when they are not just the module's own parameters."""
    dt = _compute_dtype(like)
    deps = list(module.parameters(recurse=False)) if deps is None else [d for d in deps if d is not None]
    if torch.is_grad_enabled() and any(p.requires_grad for p in deps):
        return tuple(None if t is None else t.to(dt) for t in build())
    key = (tag, dt) + tuple((p.data_ptr(), p._version) for p in deps)
    cache = module.__dict__.setdefault("_prepared_cache", {})
    if cache.get("key") != key:
        cache["key"], cache["val"] = key, tuple(None if t is None else t.detach().to(dt) for t in build())
    return cache["val"]


def _bn_affine(bn):
    """Inference-mode batch norm as ``y = x * a + b`` per channel, in fp32."""
    a = bn.weight.float() * torch.rsqrt(bn.running_var.float() + bn.eps)
    return a, bn.bias.float() - bn.running_mean.float() * a


def _bn_tensors(bn):
    return [bn.weight, bn.bias, bn.running_mean, bn.running_var]


def _fold_norm(bn, proj, order=None):
    """Weight and bias (fp32) of ``proj(bn(x))`` as one affine map on tokens: ``W diag(a)`` and ``W b + bias``;
    `order` permutes the output channels."""
    a, b = _bn_affine(bn)
    w = _dense_weight(proj).float()
    bias = proj.bias.float() if proj.bias is not None else torch.zeros(w.shape[0], device=w.device)
    if order is not None:
        w, bias = w.index_select(0, order), bias.index_select(0, order)
    return w * a, bias + w @ b


def _compute_dtype(x):
    """The dtype a matrix product on `x` runs in (autocast's, when it is on)."""
    return torch.get_autocast_dtype(x.device.type) if torch.is_autocast_enabled(x.device.type) else x.dtype


def _dense_weight(proj):
    """[out, in] matrix of a per-token projection: a Linear's weight, or a grouped 1x1 convolution's blocks on
    the diagonal.  (Cast it before expanding it over the batch: casting afterwards materialises one copy per
    sample.)"""
    if isinstance(proj, nn.Linear):
        return proj.weight
    w = proj.weight[:, :, 0]
    return w if proj.groups == 1 else torch.block_diag(*w.view(proj.groups, w.shape[0] // proj.groups, w.shape[1]))


def _qkv_channel_order(dim, groups, device):
    """Output channel of the channels-first qkv convolution that holds (which, head-major channel f): the inverse
    of the view/transpose chain of :func:`_split_heads` (PCF_NATransformer.py:126-129), as a row index."""
    f = torch.arange(dim, device=device)
    per = dim // groups
    oc = ((f % per) * groups + f // per) * 3                      # which = 0
    return torch.cat([oc, oc + 1, oc + 2])


def _window_mask(T, W, left, padding, dtype, device):
    """[N, T, W] additive mask of PCF_NATransformer.py:87-99."""
    if padding is None:
        padding = torch.zeros(1, dtype=torch.int64, device=device)
    tv = (T - padding.to(device=device, dtype=torch.int64)).view(-1, 1, 1)
    t = torch.arange(T, device=device).view(1, T, 1)
    key = t - left + torch.arange(W, device=device).view(1, 1, W)
    bad = (t >= tv) | (key < 0) | (key >= tv)
    return torch.zeros(bad.shape, dtype=dtype, device=device).masked_fill(bad, MASK_VALUE)


class NAttention(nn.Module):
    """Neighbourhood attention layer (PCF_NATransformer.py:44-178 / MFA_NATransformer.py:43-177)."""

    def __init__(self, frames, dim, num_heads, win_size, groups=1, channels_first=True, dtype=torch.bfloat16,
                 na="fused", dilation=1, attn_drop=0.0, proj_drop=0.0):
        super().__init__()
        self.attn_drop, self.proj_drop = attn_drop, nn.Dropout(proj_drop)      # PCF :71-73
        if isinstance(win_size, int):
            assert win_size > 0
            left = win_size - 1 - win_size // 2
        else:
            win_size, left = win_size
        assert win_size <= 80 and 0 <= left < win_size
        head_dim = dim // num_heads
        assert dim % num_heads == 0 and head_dim % 8 == 0
        self.win_size, self.left, self.dim, self.num_heads, self.groups = win_size, left, dim, num_heads, groups
        self.channels_first, self.na, self.dilation = channels_first, na, dilation
        self.scale = head_dim ** -0.5
        self.qkv = _Projection.make(dim, dim * 3, True, groups, channels_first)
        self.relative_position_bias = nn.Parameter(torch.zeros(1, num_heads, 1, win_size))
        nn.init.normal_(self.relative_position_bias, mean=0.0, std=0.02)
        self.proj = _Projection.make(dim, dim, True, groups, channels_first)
        self.register_buffer("attn_mask", _window_mask(frames, win_size, left, None, torch.float32, "cpu").unsqueeze(1))
        if na == "unfused":     # like the reference's CUDA path, the two-call chain has no dilated kernels
            self.NA1d_QK_Function, self.NA1d_AV_Function = getNA1dFunction(C=head_dim, dilation=dilation, dtype=dtype)

    def forward(self, x, padding=None):
        n = x.shape[0]
        t = x.shape[-1] if self.channels_first else x.shape[1]
        h, w, left = self.num_heads, self.win_size, self.left
        if self.training:       # the reference trains with its constructor-time mask: fixed length, nothing padded (PCF :131-132)
            # that mask has `frames` rows, so any other length fails there (a shape error in the addition); it fails here too
            assert t == self.attn_mask.shape[-2], \
                "training uses the fixed-length mask built for %d tokens, got %d" % (self.attn_mask.shape[-2], t)
            padding = None
        t_valid = None if padding is None else (t - padding).to(torch.int32)
        dropping = self.attn_drop > 0.0 and self.training
        if self.na == "fused_qkv":                           # dropout (PCF :149) happens inside the kernels
            return self.proj_drop(self._forward_token_major(x, n, t, t_valid, self.attn_drop if dropping else 0.0))
        q, k, v = _split_heads(self.qkv(x), h, self.groups, self.channels_first)
        q = q * self.scale                                   # in the activation dtype, as the reference does (:141)
        extra = {} if self.dilation == 1 else {"dilation": self.dilation}
        if callable(self.na):
            out = self.na(q, k, v, w, left, rpb=self.relative_position_bias, t_valid=t_valid, num_heads=h, **extra)
        elif self.na == "fused_op":
            from . import ops
            assert self.dilation == 1 and not dropping, "the registered op covers dilation 1 without dropout"
            out = ops.na1d_fused_op(q, k, v, w, left, rpb=self.relative_position_bias.view(h, w), t_valid=t_valid,
                                    num_heads=h, scale=1.0)
        elif self.na in ("fused", "fused_qkv"):              # dropout (PCF :149) happens inside the kernels
            if dropping:
                extra["dropout_p"] = self.attn_drop
            out = na1d_fused(q, k, v, w, left, rpb=self.relative_position_bias, t_valid=t_valid, num_heads=h, **extra)
        else:                                                # the reference's un-fused chain (:141-150)
            attn = self.NA1d_QK_Function.apply(q, k, w, left, 1).view(n, h, t, w)
            attn = attn + self.relative_position_bias
            attn = attn + _window_mask(t, w, left, padding, x.dtype, x.device).unsqueeze(1)
            attn = torch.softmax(attn.view(n * h, t, w), dim=-1)
            attn = F.dropout(attn, self.attn_drop, self.training)
            out = self.NA1d_AV_Function.apply(attn, v, w, left, 1)
        return self.proj_drop(self.proj(_merge_heads(out, n, h, self.channels_first)))

    def _forward_token_major(self, x, n, t, t_valid, dropout_p=0.0):
        """The same layer with the operator reading the qkv projection in place.  Tokens-first models have the
        layout already; channels-first ones get it by running the two 1x1 convolutions as matrix products whose
        output rows are ordered (which, head, channel) - the same parameters, the same arithmetic, no copies."""
        h = self.num_heads
        if self.channels_first:
            order = _qkv_channel_order(self.dim, self.groups, x.device)
            wq, bq = _prepared(self.qkv, "token-major", x, lambda: (
                _dense_weight(self.qkv).index_select(0, order).t(), self.qkv.bias.index_select(0, order)))
            qkv = torch.bmm(x.transpose(1, 2), wq.unsqueeze(0).expand(n, -1, -1)).add_(bq)                   # [N, T, 3*dim]
        else:
            qkv = self.qkv(x)
        out = na1d_fused_qkv(qkv.view(n, t, 3, h, self.dim // h), self.win_size, self.left,
                             rpb=self.relative_position_bias, t_valid=t_valid, scale=self.scale,
                             dilation=self.dilation, dropout_p=dropout_p)                             # [N, T, dim]
        if self.channels_first:
            wp, bp = _prepared(self.proj, "dense", out, lambda: (_dense_weight(self.proj), self.proj.bias))
            return torch.bmm(wp.unsqueeze(0).expand(n, -1, -1), out.transpose(1, 2)).add_(bp.view(1, -1, 1))  # [N, dim, T]
        return self.proj(out)


class GlobalAttention(nn.Module):
    """Dense attention with an additive sinusoid input (PCF :181-225 / MFA :180-221)."""

    def __init__(self, dim, num_heads, groups=1, channels_first=True, dense="native", attn_drop=0.0, proj_drop=0.0):
        super().__init__()
        assert dense in ("native", "op", "sdpa")
        self.num_heads, self.groups, self.channels_first, self.dense = num_heads, groups, channels_first, dense
        self.attn_drop, self.proj_drop = attn_drop, nn.Dropout(proj_drop)      # PCF :193-195
        self.scale = (dim // num_heads) ** -0.5
        self.linear_pos = _Projection.make(dim, dim, False, groups, channels_first)
        self.qkv = _Projection.make(dim, dim * 3, True, groups, channels_first)
        self.proj = _Projection.make(dim, dim, True, groups, channels_first)

    def forward(self, x, pos_emb, attn_mask=None, padding=None):
        """``padding`` [N] (patches) says the same as ``attn_mask`` (-100 on padded rows and columns); the HIP
        kernels build the mask from it, the other paths add the tensor."""
        n = x.shape[0]
        x = x + self.linear_pos(pos_emb.to(x.dtype))
        q, k, v = _split_heads(self.qkv(x), self.num_heads, self.groups, self.channels_first)
        t, hd = q.shape[1], q.shape[2]
        drop_p = self.attn_drop if self.training else 0.0
        native = (self.dense in ("native", "op") and x.device.type == "cuda" and hd <= 128 and hd % 8 == 0
                  and q.dtype in (torch.bfloat16, torch.float16) and (attn_mask is None or padding is not None))
        if native:                       # the HIP kernels: no mask or score tensor
            t_valid = None if attn_mask is None else (t - padding).clamp(0, t).to(torch.int32)
            if self.dense == "op":       # the registered op, for torch.compile
                from . import ops
                assert drop_p == 0.0
                out = ops.global_attention_op(q.contiguous(), k.contiguous(), v.contiguous(), self.num_heads, t_valid,
                                              self.scale)
            else:
                out = global_attention(q.contiguous(), k.contiguous(), v.contiguous(), self.num_heads, t_valid,
                                       self.scale, dropout_p=drop_p)
            return self.proj_drop(self.proj(_merge_heads(out, n, self.num_heads, self.channels_first)))
        q, k, v = (z.view(n, self.num_heads, t, hd) for z in (q, k, v))
        if x.device.type == "cuda":      # one library kernel instead of matmul -> mask -> softmax -> matmul
            out = F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=drop_p, scale=self.scale)
        else:
            attn = (q * self.scale) @ k.transpose(-2, -1)
            if attn_mask is not None:
                attn = attn + attn_mask
            out = F.dropout(torch.softmax(attn, dim=-1), drop_p) @ v
        out = _merge_heads(out.reshape(n * self.num_heads, t, hd), n, self.num_heads, self.channels_first)
        return self.proj_drop(self.proj(out))


class Mlp(nn.Module):
    def __init__(self, dim, hidden, groups, channels_first, drop=0.0):
        super().__init__()
        self.fc1 = _Projection.make(dim, hidden, True, groups, channels_first)
        self.act = nn.GELU()
        self.fc2 = _Projection.make(hidden, dim, True, groups, channels_first)
        self.drop = nn.Dropout(drop)                            # PCF :33-40

    def forward(self, x):
        return self.drop(self.fc2(self.drop(self.act(self.fc1(x)))))


class NATFLayer(nn.Module):
    """norm -> attention -> residual; norm -> MLP -> residual (PCF :228-265)."""

    def __init__(self, frames, dim, num_heads, win_size, groups, drop_path, channels_first, dtype, na, mlp_ratio=4,
                 dilation=1, attn_drop=0.0, drop=0.0):
        super().__init__()
        self.local = isinstance(win_size, list) or win_size > 0
        if self.local:
            self.attn = NAttention(frames, dim, num_heads, win_size, groups, channels_first, dtype, na, dilation,
                                   attn_drop, drop)
        else:
            assert dilation == 1
            self.attn = GlobalAttention(dim, num_heads, groups, channels_first, attn_drop=attn_drop, proj_drop=drop,
                                        dense="op" if na == "fused_op" else "native")
        norm = BatchNorm1d if channels_first else TokenBatchNorm
        self.norm1 = norm(dim)
        self.drop_path = DropPath(drop_path) if drop_path > 0.0 else nn.Identity()
        self.mlp = Mlp(dim, int(dim * mlp_ratio), groups, channels_first, drop)
        self.norm2 = norm(dim)

    def forward(self, x, padding=None, pos_emb=None, attn_mask_global=None):
        y = self.norm1(x)
        if self.local:
            y = self.attn(y, padding=padding)
        else:
            y = self.attn(y, pos_emb=pos_emb, attn_mask=attn_mask_global,
                          padding=padding if attn_mask_global is not None else None)
        x = x + self.drop_path(y)
        return x + self.drop_path(self.mlp(self.norm2(x)))

    def tokens_ok(self):
        """Whether :meth:`forward_tokens` serves this layer."""
        return self.attn.na == "fused_qkv" if self.local else self.attn.dense == "native"    # not under torch.compile

    def forward_tokens(self, x, padding=None, pos_emb=None, masked=False):
        """The layer in inference on token-major ``x [N, T, C]`` (``pos_emb [1, T, C]``), whatever the layout of
        the model: the same parameters, with each batch norm folded into the projection that follows it (running
        statistics make it a per-channel affine map), every projection one matrix product over all N*T tokens
        with its bias in the epilogue, and the attention operators reading and writing the token-major tensors
        in place.  ``masked``: the global layers mask the padded rows and columns."""
        n, t, dim = x.shape
        attn, h = self.attn, self.attn.num_heads
        bn1 = self.norm1.norm if isinstance(self.norm1, TokenBatchNorm) else self.norm1
        bn2 = self.norm2.norm if isinstance(self.norm2, TokenBatchNorm) else self.norm2
        order = lambda: _qkv_channel_order(dim, attn.groups, x.device) if attn.channels_first else None
        if self.local:
            wq, bq, wp, bp = _prepared(
                attn, "tokens", x, lambda: _fold_norm(bn1, attn.qkv, order()) + (_dense_weight(attn.proj), attn.proj.bias),
                deps=_bn_tensors(bn1) + [attn.qkv.weight, attn.qkv.bias, attn.proj.weight, attn.proj.bias])
            qkv = F.linear(x, wq, bq)
            t_valid = None if padding is None else (t - padding).to(torch.int32)
            out = na1d_fused_qkv(qkv.view(n, t, 3, h, dim // h), attn.win_size, attn.left,
                                 rpb=attn.relative_position_bias, t_valid=t_valid, scale=attn.scale,
                                 dilation=attn.dilation)
        else:
            def build():
                wq, bq = _dense_weight(attn.qkv), attn.qkv.bias
                if attn.channels_first:
                    wq, bq = wq.index_select(0, order()), bq.index_select(0, order())
                return (wq, bq, _dense_weight(attn.linear_pos), _dense_weight(attn.proj), attn.proj.bias)
            wq, bq, wl, wp, bp = _prepared(attn, "tokens", x, build, deps=[
                attn.qkv.weight, attn.qkv.bias, attn.linear_pos.weight, attn.proj.weight, attn.proj.bias])
            a, b = _bn_affine(bn1)
            y = torch.addcmul(b + F.linear(pos_emb.to(wl.dtype), wl).float(), x.float(), a).to(wq.dtype)
            qkv = F.linear(y, wq, bq).view(n, t, 3, h, dim // h).permute(2, 0, 3, 1, 4).contiguous()
            q, k, v = qkv.view(3, n * h, t, dim // h).unbind(0)
            t_valid = (t - padding).clamp(0, t).to(torch.int32) if masked else None
            out = global_attention(q, k, v, h, t_valid, attn.scale)
            out = out.view(n, h, t, dim // h).transpose(1, 2).reshape(n, t, dim)
        x = x + F.linear(out, wp, bp)
        w1, b1, w2, b2 = _prepared(
            self.mlp, "tokens", x, lambda: _fold_norm(bn2, self.mlp.fc1) + (_dense_weight(self.mlp.fc2), self.mlp.fc2.bias),
            deps=_bn_tensors(bn2) + [self.mlp.fc1.weight, self.mlp.fc1.bias, self.mlp.fc2.weight, self.mlp.fc2.bias])
        return x + F.linear(F.gelu(F.linear(x, w1, b1)), w2, b2)


class NATFBlock(nn.Module):
    def __init__(self, frames, depth, dim, num_heads, win_size, groups, drop_path, channels_first, dtype, na,
                 use_checkpoint=False, dilation=1, attn_drop=0.0, drop=0.0):
        super().__init__()
        pick = lambda v, i: v[i] if isinstance(v, list) else v
        self.use_checkpoint = use_checkpoint if isinstance(use_checkpoint, list) else [use_checkpoint] * depth
        self.blocks = nn.ModuleList([
            NATFLayer(frames, dim, pick(num_heads, i), pick(win_size, i), pick(groups, i), pick(drop_path, i),
                      channels_first, dtype, na, dilation=pick(dilation, i), attn_drop=attn_drop, drop=drop)
            for i in range(depth)])

    def forward(self, x, padding=None, pos_emb=None, attn_mask_global=None):
        if (not self.training and not torch.is_grad_enabled() and x.is_cuda
                and _compute_dtype(x) in (torch.bfloat16, torch.float16) and all(l.tokens_ok() for l in self.blocks)):
            cf = self.blocks[0].attn.channels_first            # inference: the token-major pipeline
            pos = pos_emb.transpose(1, 2) if cf and pos_emb is not None else pos_emb
            y = self.forward_tokens(x.transpose(1, 2).contiguous() if cf else x, padding, pos, attn_mask_global is not None)
            return y.transpose(1, 2).contiguous() if cf else y
        for layer, ckpt in zip(self.blocks, self.use_checkpoint):
            if ckpt and self.training:      # activation checkpointing re-enters the operator's forward in backward
                x = torch.utils.checkpoint.checkpoint(layer, x, padding, pos_emb, attn_mask_global, use_reentrant=False)
            else:
                x = layer(x, padding=padding, pos_emb=pos_emb, attn_mask_global=attn_mask_global)
        return x


    def forward_tokens(self, x, padding=None, pos_emb=None, masked=False):
        x = x.to(_compute_dtype(x))
        for layer in self.blocks:
            x = layer.forward_tokens(x, padding, pos_emb, masked)
        return x


class PatchEmbed(nn.Module):
    def __init__(self, in_chans, embed_dim, patch_size, groups, channels_first):
        super().__init__()
        self.channels_first = channels_first
        self.proj = PatchConv(in_chans, embed_dim, patch_size, groups)
        self.norm = BatchNorm1d(embed_dim)

    def forward(self, x):
        x = self.norm(self.proj(x))
        return x if self.channels_first else x.transpose(1, 2)

    def forward_tokens(self, x):
        """Inference: ``[N, in_chans, frames]`` -> ``[N, T, embed_dim]`` as one matrix product over the patches,
        with the batch norm folded into it."""
        conv, bn = self.proj, self.norm
        n, cin, t = x.shape
        p, g = conv.kernel_size[0], conv.groups
        tp = (t - p) // p + 1
        def build():
            w = conv.weight.reshape(conv.out_channels, -1).float()           # [cout, (cin/g) * p]
            w = torch.block_diag(*w.view(g, conv.out_channels // g, -1)) if g > 1 else w
            a, b = _bn_affine(bn)
            return w * a.unsqueeze(1), conv.bias.float() * a + b
        w, b = _prepared(self, "tokens", x, build, deps=[conv.weight, conv.bias] + _bn_tensors(bn))
        patches = x[:, :, :tp * p].reshape(n, cin, tp, p).permute(0, 2, 1, 3).reshape(n, tp, cin * p)
        return F.linear(patches.to(w.dtype), w, b)


# --------------------------------------------------------------------------- the two model families
class _NATransformer(nn.Module):
    def __init__(self, channels_first, frames=300, patch_size=2, in_chans=80, output_emb_size=192, embed_dim=256,
                 depths=(4, 4, 4, 4), num_heads=None, win_size=None, groups=(8, 4, 2, 1), drop_path_rate=0.0,
                 proj_channel=1536, asp=True, poolnorm=True, use_checkpoint=False, dtype=torch.bfloat16, na="fused",
                 dilation=1, attn_drop=0.0, drop=0.0):
        super().__init__()
        depths = list(depths)
        nb = len(depths)
        self.channels_first, self.frames, self.patch_size, self.embed_dim, self.num_blocks = \
            channels_first, frames, patch_size, embed_dim, nb
        emb_frames = frames // patch_size
        pick = lambda v, i: v[i] if isinstance(v, (list, tuple)) else v
        if channels_first:
            self.patch_embeds = nn.ModuleList(
                [PatchEmbed(in_chans, embed_dim, patch_size, pick(groups, i), True) for i in range(nb)])
        else:
            self.patch_embed = PatchEmbed(in_chans, embed_dim, patch_size, 1, False)
        flat = [w for blk in win_size for w in (blk if isinstance(blk, list) else [blk])]
        self.attn_global = any(isinstance(w, int) and w < 1 for w in flat)
        if self.attn_global:
            self.register_buffer("pos_emb", sinusoid_table(embed_dim, emb_frames, channels_first))
            self.pos_emb_eval = None
        dpr = torch.linspace(0, drop_path_rate, sum(depths)).tolist()
        self.blocks = nn.ModuleList([
            NATFBlock(emb_frames, depths[i], embed_dim, pick(num_heads, i), pick(win_size, i),
                      pick(groups, i) if channels_first else 1, dpr[sum(depths[:i]):sum(depths[:i + 1])],
                      channels_first, dtype, na, pick(use_checkpoint, i), pick(dilation, i), attn_drop, drop)
            for i in range(nb)])
        self.norm = BatchNorm1d(embed_dim * nb)
        self.proj = TDNNBlock(embed_dim * nb, proj_channel, 1)
        self.pool = AttentiveStatisticsPooling(proj_channel) if asp else StatisticsPooling()
        self.pool_norm = BatchNorm1d(proj_channel * 2) if poolnorm else nn.Identity()
        self.fc = nn.Linear(proj_channel * 2, output_emb_size)
        for m in self.modules():                                   # PCF :392-400
            if isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, mean=0.0, std=0.02)
                if m.bias is not None:
                    nn.init.constant_(m.bias, 0)

    def forward(self, x, lens=None):
        """x: [N, in_chans, frames]; lens: relative lengths in (0, 1] or None.  Returns [N, output_emb_size]."""
        tin = x.shape[-1]
        assert self.frames == tin or not self.training
        padding = None
        if lens is not None:
            padding = ((tin - torch.round(lens * tin)) // self.patch_size).to(torch.int64)
        t = (tin - self.patch_size) // self.patch_size + 1
        pos_emb = mask_global = None
        if self.attn_global:
            if self.training:
                pos_emb = self.pos_emb
            else:
                if self.pos_emb_eval is None or self.pos_emb_eval.device != x.device:
                    self.pos_emb_eval = sinusoid_table(self.embed_dim, 40000, self.channels_first).to(x.device)
                pos_emb = self.pos_emb_eval[:, :, :t] if self.channels_first else self.pos_emb_eval[:, :t, :]
                if padding is not None:
                    pad = torch.arange(t, device=x.device).unsqueeze(0) >= (t - padding.to(x.device)).unsqueeze(1)
                    both = pad.unsqueeze(-1) | pad.unsqueeze(-2)
                    mask_global = torch.zeros(both.shape, dtype=x.dtype, device=x.device).masked_fill(both, MASK_VALUE)
                    mask_global = mask_global.unsqueeze(1)
        if padding is not None:
            padding = padding.to(x.device)
        if self._tokens_path(x):
            return self._forward_tokens(x, lens, padding, pos_emb, mask_global is not None)
        outs = []
        if self.channels_first:
            y = None
            for embed, block in zip(self.patch_embeds, self.blocks):
                e = embed(x)
                y = block(e if y is None else e + y, padding=padding, pos_emb=pos_emb, attn_mask_global=mask_global)
                outs.append(y)
            x = torch.cat(outs, dim=1)
        else:
            y = self.patch_embed(x)
            for block in self.blocks:
                y = block(y, padding=padding, pos_emb=pos_emb, attn_mask_global=mask_global)
                outs.append(y)
            x = torch.cat(outs, dim=-1).transpose(1, 2)
        x = self.proj(self.norm(x))
        return self.fc(self.pool_norm(self.pool(x, lens=lens)))


    def _tokens_path(self, x):
        return (not self.training and not torch.is_grad_enabled() and x.is_cuda
                and _compute_dtype(x) in (torch.bfloat16, torch.float16)
                and all(l.tokens_ok() for b in self.blocks for l in b.blocks))

    def _forward_tokens(self, x, lens, padding, pos_emb, masked):
        """Inference with every activation token-major ``[N, T, C]`` from the patch embedding to the pooling: the
        same parameters and arithmetic as :meth:`forward`, batch norms folded into the projections behind them,
        no layout changes between the blocks."""
        if pos_emb is not None and self.channels_first:
            pos_emb = pos_emb.transpose(1, 2)
        outs, y = [], None
        if self.channels_first:
            for embed, block in zip(self.patch_embeds, self.blocks):
                e = embed.forward_tokens(x)
                y = block.forward_tokens(e if y is None else e + y, padding, pos_emb, masked)
                outs.append(y)
        else:
            y = self.patch_embed.forward_tokens(x)
            for block in self.blocks:
                y = block.forward_tokens(y, padding, pos_emb, masked)
                outs.append(y)
        h = self.proj.forward_tokens(torch.cat(outs, dim=-1), pre_norm=self.norm)
        return self.fc(self.pool_norm(self.pool.forward_tokens(h, lens=lens)))


class PCF_NATransformer(_NATransformer):
    """models/PCF_NATransformer.py:319-462; defaults of configs/pcf_nat4x4.yaml:45-63."""

    def __init__(self, depths=(4, 4, 4, 4), num_heads=None, win_size=None, **kw):
        n = len(depths)
        num_heads = num_heads or [[16] * (depths[i] - 1) + [4 if i % 2 == 0 else 16] for i in range(n)]
        win_size = win_size or [[27] * (depths[i] - 1) + [0 if i % 2 == 0 else 27] for i in range(n)]
        super().__init__(True, depths=depths, num_heads=num_heads, win_size=win_size, **kw)


class MFA_NATransformer(_NATransformer):
    """models/MFA_NATransformer.py:325-466; defaults of configs/mfa_nat4x4.yaml:45-62."""

    def __init__(self, depths=(4, 4, 4, 4), num_heads=None, win_size=None, **kw):
        n = len(depths)
        num_heads = num_heads or [[16] * (depths[i] - 1) + [4 if i % 2 == 1 else 16] for i in range(n)]
        win_size = win_size or [[27] * (depths[i] - 1) + [0 if i % 2 == 1 else 27] for i in range(n)]
        kw.pop("groups", None)
        super().__init__(False, depths=depths, num_heads=num_heads, win_size=win_size, groups=1, **kw)


def pcf_nat_6x4(**kw):
    """configs/pcf_nat6x4.yaml:45-63 (activation checkpointing on the first four layers of block 0)."""
    kw.setdefault("use_checkpoint", [[True] * 4 + [False] * 2, False, False, False])
    return PCF_NATransformer(depths=(6, 6, 6, 6), **kw)


class ArcMarginSubCenters(nn.Module):
    """AAM-softmax with sub-centres (models/SoftMaxLoss.py:99-138)."""

    def __init__(self, emb_size=192, n_classes=5994, m=0.2, s=32.0, subcenters=3):
        super().__init__()
        self.s, self.m = s, m
        self.W = nn.Parameter(torch.empty(n_classes, subcenters, emb_size))
        nn.init.xavier_uniform_(self.W)
        self.cos_m, self.sin_m = math.cos(m), math.sin(m)
        self.th, self.mm = math.cos(math.pi - m), math.sin(math.pi - m) * m

    def forward(self, x, labels):
        cosine = torch.einsum("ne,cse->ncs", F.normalize(x, dim=-1), F.normalize(self.W, dim=-1)).amax(-1)
        with torch.no_grad():
            acc1 = (cosine.argmax(1) == labels).sum()
        sine = torch.sqrt(1.0 - cosine.pow(2))
        shifted = cosine * self.cos_m - sine * self.sin_m
        shifted = torch.where(cosine > self.th, shifted, cosine - self.mm)
        one_hot = F.one_hot(labels.long(), cosine.shape[1]).to(cosine.dtype)
        logits = (one_hot * shifted + (1.0 - one_hot) * cosine) * self.s
        return F.cross_entropy(logits, labels.long()), acc1
