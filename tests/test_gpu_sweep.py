"""Seeded random sweep over the operator's whole argument space - head_dim, window, split of the window, length,
heads, per-sample padding, bias, scale, dropout, both dtypes - against the CPU oracle.  The hand-picked geometries of
test_gpu_parity.py cover the known edges; this covers the combinations nobody thought of.  Deterministic: the cases
come from a fixed seed."""
import os
import random

import pytest
import torch

from oracle import na1d_oracle as O
from na1d_amd import _lib, na1d_fused, na1d_fused_qkv
from na1d_amd.dense import global_attention
from _util import TOL, make_inputs, seeded_scores

pytestmark = pytest.mark.gpu
SCALE = int(os.environ.get("NA1D_SWEEP_SCALE", "1"))      # multiply the number of cases for a longer soak of passing code


def _cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        C = rng.choice([8, 16, 16, 24, 32, 32, 40, 64, 64, 96, 128])
        W = rng.choice([1, 2, 3, 5, 7, 8, 9, 13, 15, 16, 17, 18, 21, 27, 27, 31, 32, 33, 40, 48, 49, 64, 65, 79, 80])
        L = rng.choice([0, W - 1, W // 2, W - 1 - W // 2, rng.randrange(W)])
        T = rng.choice([1, 2, 7, 15, 16, 17, 31, 33, 48, 63, 64, 65, 100, 127, 129, 150, 200, 257, 300])
        H = rng.choice([1, 2, 3, 4])
        N = rng.choice([1, 2, 3])
        out.append((i, N, H, T, C, W, L, rng.choice([torch.bfloat16, torch.float16]), rng.random() < 0.3,
                    rng.random() < 0.7, rng.random() < 0.7, rng.choice([1.0, None])))
    return out


def _err(got, ref, terms=1):
    """rel-L2 with a floor on the denominator: where the exact gradient is 0 (a one-slot window, a one-token
    sequence, fully padded samples) what is left is fp32 rounding of O(1) terms, measured against an rms of 0.05
    per element (times sqrt(terms) for a sum of that many independent terms, as the bias gradient is)."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return (got - ref).norm().item() / max(ref.norm().item(), 0.05 * (ref.numel() * terms) ** 0.5, 1e-1)


@pytest.mark.parametrize("case", _cases(160 * SCALE, 20240607), ids=lambda c: "%d-N%dH%dT%dC%dW%dL%d" % c[:7])
def test_fused_operator_random_geometry(case):
    i, N, H, T, C, W, L, dtype, drop, with_rpb, with_pad, scale = case
    B = N * H
    scale = C ** -0.5 if scale is None else scale
    q, k, v, do = make_inputs(B, T, C, W, 1000 + i, dtype, n=4, scale=None if scale != 1.0 else C ** -0.5)
    g = torch.Generator().manual_seed(i)
    rpb = torch.randn(H, W, generator=g) * 0.5 if with_rpb else None
    pad = torch.randint(0, T + 1, (N,), generator=g) if with_pad else None
    t_valid = None if pad is None else (T - pad).to(torch.int32).cuda()
    p, seed = (0.25, 7_000_000_007 * (i + 1)) if drop else (0.0, None)
    print("sweep", case, flush=True)

    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = None if rpb is None else rpb.cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=t_valid, num_heads=H, scale=scale, dropout_p=p, seed=seed)
    out.backward(do.cuda())

    keep = O.dropout_keep(B, T, W, p, seed) if drop else None
    qs = q.float() * scale                                      # the kernels scale the fp32 scores
    want_o, _, _ = O.na1d_forward(qs, k.float(), v.float(), W, L, rpb, pad, H, keep=keep, p_drop=p)
    wq, wk, wv, wr = O.na1d_backward(qs, k.float(), v.float(), do.float(), W, L, rpb, pad, H, keep=keep, p_drop=p)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert _err(qd.grad.float(), wq * scale) < tol, "dQ"
    assert _err(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"
    if rd is not None:
        assert _err(rd.grad, wr, terms=N * T) < tol, "drpb"

    if not drop:                                                # the in-place projection layout: same bits
        qkv = torch.stack([q.view(N, H, T, C), k.view(N, H, T, C), v.view(N, H, T, C)], 0).permute(1, 3, 0, 2, 4)
        xd = qkv.contiguous().cuda().requires_grad_(True)      # [N, T, 3, H, C]
        o2 = na1d_fused_qkv(xd, W, L, rpb=None if rpb is None else rpb.cuda(), t_valid=t_valid, scale=scale)
        assert torch.equal(o2.view(N, T, H, C).permute(0, 2, 1, 3).reshape(B, T, C), out)
        o2.backward(do.view(N, H, T, C).permute(0, 2, 1, 3).reshape(N, T, H * C).cuda())
        for j, z in enumerate((qd, kd, vd)):
            assert torch.equal(xd.grad[:, :, j].permute(0, 2, 1, 3).reshape(B, T, C), z.grad)


@pytest.mark.parametrize("case", _cases(40 * SCALE, 77), ids=lambda c: "%d-N%dH%dT%dC%d" % c[:5])
def test_dense_attention_random_geometry(case):
    i, N, H, T, C, _, _, dtype, _, _, with_pad, _ = case
    B = N * H
    q, k, v, do = make_inputs(B, T, C, 0, 2000 + i, dtype, n=4)
    pad = torch.randint(0, T + 1, (N,), generator=torch.Generator().manual_seed(i)) if with_pad else None
    t_valid = None if pad is None else (T - pad).to(torch.int32).cuda()
    print("dense sweep", case[:5], dtype, flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = global_attention(qd, kd, vd, H, t_valid=t_valid, scale=C ** -0.5)
    out.backward(do.cuda())
    want_o, _, _ = O.global_forward(q.float(), k.float(), v.float(), C ** -0.5, pad, H)
    wq, wk, wv = O.global_backward(q.float(), k.float(), v.float(), do.float(), C ** -0.5, pad, H)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert _err(qd.grad.float(), wq) < tol, "dQ"
    assert _err(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"


@pytest.mark.parametrize("case", _cases(64 * SCALE, 4242), ids=lambda c: "%d-N%dH%dT%dC%dW%dL%d" % c[:7])
def test_unfused_primitives_random_geometry(case):
    """The three drop-in primitives (band QK^T, band . V, inverse-band gather) behind the reference's six calls."""
    i, N, H, T, C, W, L, dtype = case[:8]
    B = N * H
    q, k, v = make_inputs(B, T, C, W, 3000 + i, dtype)
    s = seeded_scores(B, T, W, seed=i)
    print("unfused sweep", case[:8], flush=True)
    qd, kd, vd, sd = q.cuda(), k.cuda(), v.cuda(), s.cuda()
    attn = torch.empty(B, T, W, device="cuda")
    _lib.call_unfused("na1d_qk_forward", attn, qd, kd, B, T, C, W, L, dtype)
    want = O.qk_band(q.float(), k.float(), W, L)
    assert O.rel_l2(attn, want) < 1e-5, "P1"
    assert (attn.cpu()[want == 0] == 0).all()                 # zero fill is exact
    out = torch.empty_like(vd)
    _lib.call_unfused("na1d_av_forward", out, sd, vd, B, T, C, W, L, dtype)
    assert O.rel_l2(out.float(), O.av_band(s, v.float(), W, L)) < TOL[dtype], "P2"
    dk = torch.empty_like(qd)
    _lib.call_unfused("na1d_k_backward", dk, sd, qd, B, T, C, W, L, dtype)
    assert O.rel_l2(dk.float(), O.inverse_gather(s, q.float(), W, L)) < TOL[dtype], "P3"
