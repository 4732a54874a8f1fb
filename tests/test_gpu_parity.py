"""GPU parity: the HIP path (called through the C ABI) against the CPU oracle on
the same seeded inputs.  Tolerances are the contract's: relative L2 error
<= 1e-2 for bf16 and <= 2e-3 for fp16 on outputs and gradients; integer-like
facts (zero fill, shifts, aliasing) are checked bit for bit."""
import os

import pytest
import torch

from oracle import na1d_oracle as O
from na1d_amd import _lib, nattn, na1d_fused, na1d_fused_qkv
from na1d_amd.fused import na1d_fused_forward_lse
from _util import TOL, dev, make_inputs, seeded_scores

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16]

# (B, T, C, W, left): edge geometry the reference's CPU branch defines -
# T < W, even W, left = 0, left = W-1, W = 1, W = 80, T = 1, odd head_dim multiples
SHAPES = [
    (2, 9, 8, 5, 2), (2, 9, 16, 4, 1), (3, 7, 8, 1, 0), (2, 3, 16, 7, 3), (2, 2, 8, 5, 0),
    (2, 5, 8, 5, 4), (1, 1, 8, 3, 1), (2, 40, 24, 11, 5), (2, 33, 40, 8, 3), (1, 100, 16, 27, 13),
    (2, 100, 128, 80, 39), (2, 17, 16, 80, 0), (2, 130, 64, 7, 3), (4, 300, 32, 15, 7), (3, 65, 16, 27, 26),
    (2, 47, 48, 33, 16), (2, 64, 16, 27, 13), (1, 16, 32, 15, 7), (2, 15, 64, 7, 3), (2, 250, 16, 9, 8),
    (2, 70, 56, 27, 13), (1, 90, 72, 15, 7), (2, 50, 96, 40, 20), (1, 33, 120, 7, 3), (2, 40, 136, 9, 4),
    # the QK kernel's two forms side by side: key rows straight into registers (head_dim 16 with any window, head_dim
    # 32 up to three key blocks) and through LDS (head_dim 32 from four key blocks on), ragged and whole last tile pairs
    (3, 128, 16, 80, 40), (2, 113, 16, 49, 48), (2, 100, 32, 27, 13), (2, 129, 32, 33, 0), (3, 97, 24, 40, 20),
    (2, 144, 8, 17, 16),
]


def _err(got, ref):
    """rel-L2 for d rpb, with an absolute floor on the denominator: for a one-slot
    window or a one-token sequence the exact gradient is 0 (up to e^-100) and what
    is left is fp32 rounding of sums of O(1) terms."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return (got - ref).norm().item() / max(ref.norm().item(), 1e-1)


def _unfused(name, out, a, b, W, left):
    B, T, C = (a if a.dtype != torch.float32 else b).shape
    _lib.call_unfused(name, out, a, b, B, T, C, W, left, (a if a.dtype != torch.float32 else b).dtype)
    return out


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_unfused_primitives(shape, dtype):
    B, T, C, W, L = shape
    q, k, v = make_inputs(B, T, C, W, seed=sum(shape), dtype=dtype)
    s = seeded_scores(B, T, W, seed=7)
    qd, kd, vd, sd = dev(q, k, v, s)
    tol = TOL[dtype]

    attn = _unfused("na1d_qk_forward", torch.empty(B, T, W, device="cuda"), qd, kd, W, L)
    want = O.qk_band(q.float(), k.float(), W, L)
    assert O.rel_l2(attn, want) < 1e-5, "P1"
    # zero fill is exact
    assert (attn.cpu()[want == 0] == 0).all()

    out = _unfused("na1d_av_forward", torch.empty_like(vd), sd, vd, W, L)
    assert O.rel_l2(out.float(), O.av_band(s, v.float(), W, L)) < tol, "P2"

    dk = _unfused("na1d_k_backward", torch.empty_like(qd), sd, qd, W, L)
    assert O.rel_l2(dk.float(), O.inverse_gather(s, q.float(), W, L)) < tol, "P3"


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_aliasing_identities_bit_for_bit(dtype):
    """bf16_ana1d.cpp:57-104: av_forward == q_backward, a_backward == qk_forward on
    (dO, v), v_backward == k_backward on (P, dO)."""
    B, T, C, W, L = 4, 77, 32, 15, 7
    x, y, _ = make_inputs(B, T, C, W, 5, dtype)
    s = seeded_scores(B, T, W, 5)
    xd, yd, sd = dev(x, y, s)
    e16 = lambda: torch.empty_like(xd)
    e32 = lambda: torch.empty(B, T, W, device="cuda")
    assert torch.equal(_unfused("na1d_av_forward", e16(), sd, yd, W, L), _unfused("na1d_q_backward", e16(), sd, yd, W, L))
    assert torch.equal(_unfused("na1d_a_backward", e32(), xd, yd, W, L), _unfused("na1d_qk_forward", e32(), xd, yd, W, L))
    assert torch.equal(_unfused("na1d_v_backward", e16(), sd, xd, W, L), _unfused("na1d_k_backward", e16(), sd, xd, W, L))


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_one_hot_probabilities_shift_values_exactly(dtype):
    B, T, C, W, L = 2, 50, 16, 7, 3
    _, _, v = make_inputs(B, T, C, W, 11, dtype)
    vd = dev(v)
    for j0 in (0, 3, 6):
        p = torch.zeros(B, T, W)
        p[:, :, j0] = 1
        out = _unfused("na1d_av_forward", torch.empty_like(vd), p.cuda(), vd, W, L).cpu()
        want = torch.zeros_like(v)
        lo, hi = max(0, L - j0), min(T, T + L - j0)
        want[:, lo:hi] = v[:, lo - L + j0:hi - L + j0]
        assert torch.equal(out, want)


def _reference_style_chain(QK, AV, q, k, v, rpb, mask, H, W, L):
    """The CUDA branch of models/PCF_NATransformer.py:141-150 with our Functions."""
    B, T, _ = q.shape
    attn = QK.apply(q, k, W, L, 1)
    attn = attn.view(B // H, H, T, W) + rpb.view(1, H, 1, W)
    attn = attn + mask.unsqueeze(1)
    attn = torch.softmax(attn.view(B, T, W), dim=-1)
    return AV.apply(attn, v, W, L, 1)


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", [(2, 4, 60, 16, 27, 13), (3, 2, 33, 32, 15, 7), (2, 2, 9, 64, 7, 3), (2, 3, 21, 24, 8, 3)],
                         ids=lambda g: "x".join(map(str, g)))
def test_dropin_autograd_chain_matches_oracle(geom, dtype):
    N, H, T, C, W, L = geom
    B = N * H
    q, k, v, do = make_inputs(B, T, C, W, 21, dtype, n=4, scale=C ** -0.5)
    g = torch.Generator().manual_seed(3)
    rpb = torch.randn(H, W, generator=g) * 0.5
    pad = torch.tensor([0] + [T // 3] * (N - 1))
    QK, AV = nattn.getNA1dFunction(C, 1, dtype)

    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = rpb.cuda().requires_grad_(True)
    mask = O.attn_mask(T, W, L, pad).cuda()
    out = _reference_style_chain(QK, AV, qd, kd, vd, rd, mask, H, W, L)
    out.backward(do.cuda())

    want_o, _, _ = O.na1d_forward(q.float(), k.float(), v.float(), W, L, rpb, pad, H)
    wq, wk, wv, wr = O.na1d_backward(q.float(), k.float(), v.float(), do.float(), W, L, rpb, pad, H)
    tol = TOL[dtype]
    assert out.dtype == dtype and qd.grad.dtype == dtype
    assert O.rel_l2(out.float(), want_o) < tol
    assert O.rel_l2(qd.grad.float(), wq) < tol
    assert O.rel_l2(kd.grad.float(), wk) < tol
    assert O.rel_l2(vd.grad.float(), wv) < tol
    assert _err(rd.grad, wr) < tol


FUSED_GEOMS = [  # (N, H, T, C, W, left)
    (2, 4, 60, 16, 27, 13), (3, 2, 33, 32, 15, 7), (2, 2, 9, 64, 7, 3), (2, 3, 21, 24, 8, 3), (1, 1, 1, 8, 3, 1),
    (2, 2, 5, 16, 27, 13), (1, 2, 100, 16, 27, 0), (1, 2, 100, 16, 27, 26), (2, 1, 70, 40, 80, 40), (2, 16, 100, 16, 27, 13),
    (3, 4, 150, 16, 27, 13), (2, 8, 300, 32, 15, 7), (4, 4, 200, 64, 7, 3), (1, 2, 129, 128, 5, 2), (2, 2, 48, 16, 1, 0),
    (1, 4, 257, 32, 40, 7), (1, 2, 31, 64, 33, 20), (2, 2, 90, 56, 27, 13), (1, 2, 75, 72, 15, 7), (2, 1, 60, 96, 50, 25),
    (1, 2, 40, 120, 7, 3), (2, 2, 100, 8, 27, 13), (1, 2, 50, 136, 9, 4),
    # either side of the backward's single-strip form (a strip of at most eight tiles that is the whole sequence)
    (2, 2, 128, 16, 27, 13), (1, 3, 128, 32, 15, 7), (2, 2, 127, 32, 9, 4), (1, 2, 113, 16, 17, 16), (1, 2, 129, 16, 27, 13),
    (2, 1, 64, 64, 7, 3), (1, 2, 65, 64, 15, 7), (1, 1, 32, 128, 5, 2), (1, 2, 16, 16, 27, 13),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", FUSED_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_fused_forward_backward_matches_oracle(geom, dtype):
    N, H, T, C, W, L = geom
    B = N * H
    q, k, v, do = make_inputs(B, T, C, W, 31, dtype, n=4, scale=C ** -0.5)
    g = torch.Generator().manual_seed(4)
    rpb = torch.randn(H, W, generator=g) * 0.5
    pad = torch.tensor([0, T // 2, T][:N] + [1] * max(0, N - 3))
    t_valid = (T - pad).to(torch.int32)

    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = rpb.cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=t_valid.cuda(), num_heads=H)
    out.backward(do.cuda())

    qf, kf, vf = q.float(), k.float(), v.float()
    want_o, _, want_lse = O.na1d_forward(qf, kf, vf, W, L, rpb, pad, H)
    wq, wk, wv, wr = O.na1d_backward(qf, kf, vf, do.float(), W, L, rpb, pad, H)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert O.rel_l2(qd.grad.float(), wq) < tol, "dQ"
    assert O.rel_l2(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"
    assert _err(rd.grad, wr) < tol, "drpb"
    _, lse = na1d_fused_forward_lse(qd.detach(), kd.detach(), vd.detach(), W, L, rd.detach(), t_valid.cuda(), H)
    assert torch.allclose(lse.cpu(), want_lse, atol=2e-3, rtol=1e-4), "LSE"


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", [g for g in FUSED_GEOMS if g[2] > 1], ids=lambda g: "x".join(map(str, g)))
def test_fused_on_projection_layout_matches_oracle_and_packed_operator(geom, dtype):
    """q, k, v read in place from a [N, T, 3, H, C] projection output, out written as [N, T, H*C]: against
    the oracle on the packed copies, and bit for bit against the packed operator where the same kernels serve
    both (shapes they do not cover go through the packing fallback)."""
    N, H, T, C, W, L = geom
    g = torch.Generator().manual_seed(12)
    qkv = (torch.randn(N, T, 3, H, C, generator=g) * (C ** -0.25)).to(dtype)
    do = torch.randn(N, T, H * C, generator=g).to(dtype)
    rpb = torch.randn(H, W, generator=g) * 0.5
    pad = torch.tensor([0, T // 2, T][:N] + [1] * max(0, N - 3))
    t_valid = (T - pad).to(torch.int32).cuda()

    xd = qkv.cuda().requires_grad_(True)
    rd = rpb.cuda().requires_grad_(True)
    out = na1d_fused_qkv(xd, W, L, rpb=rd, t_valid=t_valid)
    assert out.shape == (N, T, H * C) and out.is_contiguous()
    out.backward(do.cuda())

    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3).contiguous().view(N * H, T, C) for i in range(3))   # the reference's packing
    dop = do.view(N, T, H, C).permute(0, 2, 1, 3).contiguous().view(N * H, T, C)
    unpack = lambda z: z.reshape(N, H, T, C).permute(0, 2, 1, 3)
    want_o, _, _ = O.na1d_forward(q.float(), k.float(), v.float(), W, L, rpb, pad, H)
    wq, wk, wv, wr = O.na1d_backward(q.float(), k.float(), v.float(), dop.float(), W, L, rpb, pad, H)
    tol = TOL[dtype]
    assert O.rel_l2(out.float().view(N, T, H, C), unpack(want_o)) < tol, "O"
    for i, (name, want) in enumerate((("dQ", wq), ("dK", wk), ("dV", wv))):
        assert O.rel_l2(xd.grad[:, :, i].float(), unpack(want)) < tol, name
    assert _err(rd.grad, wr) < tol, "drpb"

    qd, kd, vd = (z.cuda().requires_grad_(True) for z in (q, k, v))
    packed = na1d_fused(qd, kd, vd, W, L, rpb=rpb.cuda(), t_valid=t_valid, num_heads=H)
    packed.backward(dop.cuda())
    assert torch.equal(out.view(N, T, H, C), unpack(packed))
    for i, z in enumerate((qd, kd, vd)):
        assert torch.equal(xd.grad[:, :, i], unpack(z.grad))


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", [(2, 4, 61, 16, 27, 13, 2), (3, 2, 50, 32, 15, 7, 3), (2, 2, 40, 64, 7, 3, 4),
                                  (2, 3, 33, 24, 8, 3, 2), (1, 2, 5, 16, 5, 2, 7), (2, 2, 100, 16, 9, 0, 5)],
                         ids=lambda g: "x".join(map(str, g)))
def test_dilated_windows_match_oracle(geom, dtype):
    """dilation > 1 (CPU-only in the reference, models/PCF_NATransformer.py:101-116,158-170): slot j of row t is
    row t + (j - left) * d; packed and projection-layout operators, with rpb and per-sample valid lengths."""
    N, H, T, C, W, L, D = geom
    g = torch.Generator().manual_seed(21)
    qkv = (torch.randn(N, T, 3, H, C, generator=g) * (C ** -0.25)).to(dtype)
    do = torch.randn(N, T, H * C, generator=g).to(dtype)
    rpb = torch.randn(H, W, generator=g) * 0.5
    pad = torch.tensor([0, T // 3, T - 1][:N] + [1] * max(0, N - 3))
    t_valid = (T - pad).to(torch.int32).cuda()
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3).contiguous().view(N * H, T, C) for i in range(3))
    dop = do.view(N, T, H, C).permute(0, 2, 1, 3).contiguous().view(N * H, T, C)
    want_o, _, _ = O.na1d_forward(q.float(), k.float(), v.float(), W, L, rpb, pad, H, dilation=D)
    wq, wk, wv, wr = O.na1d_backward(q.float(), k.float(), v.float(), dop.float(), W, L, rpb, pad, H, dilation=D)
    tol = TOL[dtype]

    qd, kd, vd = (z.cuda().requires_grad_(True) for z in (q, k, v))
    rd = rpb.cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=t_valid, num_heads=H, dilation=D)
    out.backward(dop.cuda())
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    for name, got, want in (("dQ", qd.grad, wq), ("dK", kd.grad, wk), ("dV", vd.grad, wv)):
        assert O.rel_l2(got.float(), want) < tol, name
    assert _err(rd.grad, wr) < tol, "drpb"

    xd = qkv.cuda().requires_grad_(True)
    out2 = na1d_fused_qkv(xd, W, L, rpb=rpb.cuda(), t_valid=t_valid, dilation=D)
    out2.backward(do.cuda())
    unpack = lambda z: z.reshape(N, H, T, C).permute(0, 2, 1, 3)
    assert torch.equal(out2.view(N, T, H, C), unpack(out))
    for i, z in enumerate((qd, kd, vd)):
        assert torch.equal(xd.grad[:, :, i], unpack(z.grad))


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_strided_entry_points_leave_the_gaps_alone(dtype):
    """Rows 3*H*C apart with the k and v slots (and a pad column) between them: nothing but the addressed
    rows may be written."""
    N, H, T, C, W, L = 2, 3, 50, 16, 27, 13
    g = torch.Generator().manual_seed(5)
    buf = torch.randn(N, T, 3, H, C + 8, generator=g).to(dtype).cuda()        # 8 pad channels per head row
    views = [buf[:, :, i, :, :C].permute(0, 2, 1, 3) for i in range(3)]       # [N, H, T, C], row stride 3*H*(C+8)
    obuf = torch.full((N, T, H, C + 8), 7.0, dtype=dtype, device="cuda")
    out = obuf[..., :C].permute(0, 2, 1, 3)
    lse = torch.empty(N * H, T, device="cuda")
    assert _lib.call_fused_forward_strided(out, lse, *views, None, None, W, L, 1.0) == 0
    assert torch.all(obuf[..., C:] == 7.0)
    packed = [z.contiguous().view(N * H, T, C) for z in views]
    want, _ = na1d_fused_forward_lse(*packed, W, L)
    assert torch.equal(out.contiguous().view(N * H, T, C), want)

    gbuf = torch.full_like(buf, float("nan"))
    gviews = [gbuf[:, :, i, :, :C].permute(0, 2, 1, 3) for i in range(3)]
    do = torch.randn(N, H, T, C, generator=g).to(dtype).cuda()
    assert _lib.call_fused_backward_strided(*gviews, None, *views, do, lse, None, None, W, L, 1.0) == 0
    assert torch.isnan(gbuf[..., C:]).all()
    assert not torch.isnan(gbuf[..., :C]).any()


@pytest.mark.parametrize("geom", [(2, 16, 100, 16, 27, 13, 24), (3, 8, 75, 32, 15, 7, 40), (2, 4, 37, 16, 27, 13, 8),
                                  (1, 2, 21, 32, 17, 8, 0)], ids=lambda g: "x".join(map(str, g)))
@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_grouped_heads_keep_to_their_rows(geom, dtype):
    """Projection layout with head groups (four heads of 16 channels or two of 32 staged together, output rows written
    back as whole lines out of LDS): T is not a multiple of the tile or the strip, rows are wider than H*C by `gap`
    sentinel columns, and everything sits between sentinel bands.  Outputs and gradients must be bit-identical to the
    packed operator and no sentinel may change."""
    N, H, T, C, W, L, gap = geom
    g = torch.Generator().manual_seed(11)
    row = 3 * H * C + gap                                               # elements from one token to the next
    buf, qkv, pad = _guarded((N, T, row), dtype, 5.0)
    qkv.copy_(torch.randn(N, T, row, generator=g).to(dtype))
    qkv[..., 3 * H * C:] = 5.0                                          # the gap columns
    views = [qkv[..., i * H * C:(i + 1) * H * C].view(N, T, H, C).permute(0, 2, 1, 3) for i in range(3)]
    orow = H * C + gap
    obuf, o3, opad = _guarded((N, T, orow), dtype, 5.0)
    out = o3[..., :H * C].view(N, T, H, C).permute(0, 2, 1, 3)
    rpb = (torch.randn(H, W, generator=g) * 0.3).cuda()
    tv = torch.tensor(([T, T // 2, 1] * N)[:N], dtype=torch.int32, device="cuda")
    lse = torch.empty(N * H, T, device="cuda")
    assert _lib.call_fused_forward_strided(out, lse, *views, rpb, tv, W, L, 0.5) == 0
    torch.cuda.synchronize()
    assert (obuf[:opad] == 5.0).all() and (obuf[opad + o3.numel():] == 5.0).all() and (o3[..., H * C:] == 5.0).all()
    packed = [z.contiguous().view(N * H, T, C) for z in views]
    want, want_lse = na1d_fused_forward_lse(*packed, W, L, rpb=rpb, t_valid=tv, num_heads=H, scale=0.5)
    assert torch.equal(out.contiguous().view(N * H, T, C), want) and torch.equal(lse, want_lse)

    gbuf, gqkv, gpad = _guarded((N, T, row), dtype, 5.0)
    gviews = [gqkv[..., i * H * C:(i + 1) * H * C].view(N, T, H, C).permute(0, 2, 1, 3) for i in range(3)]
    dbuf, d3, dpad = _guarded((N, T, orow), dtype, 5.0)
    d3[..., :H * C] = torch.randn(N, T, H * C, generator=g).to(dtype).cuda()
    do = d3[..., :H * C].view(N, T, H, C).permute(0, 2, 1, 3)
    drpb = torch.zeros(H, W, device="cuda")
    assert _lib.call_fused_backward_strided(*gviews, drpb, *views, do, lse, rpb, tv, W, L, 0.5) == 0
    torch.cuda.synchronize()
    assert (gbuf[:gpad] == 5.0).all() and (gbuf[gpad + gqkv.numel():] == 5.0).all() and (gqkv[..., 3 * H * C:] == 5.0).all()
    wq, wk, wv = (torch.empty_like(want) for _ in range(3))
    wr = torch.zeros(H, W, device="cuda")
    _lib.call_fused_backward(wq, wk, wv, wr, *packed, want, do.contiguous().view(N * H, T, C), want_lse, rpb, tv, N * H, H, T, C,
                             W, L, 0.5)
    for name, a, b in zip(("dq", "dk", "dv"), gviews, (wq, wk, wv)):
        assert torch.equal(a.contiguous().view(N * H, T, C), b), name
    assert torch.allclose(drpb, wr, rtol=1e-4, atol=1e-4)


WIDE_GEOMS = [  # (N, H, T, C, W, left): windows the two/three-block kernels do not cover
    (2, 2, 100, 16, 33, 16), (2, 2, 130, 32, 40, 7), (1, 2, 90, 64, 48, 47), (2, 1, 200, 16, 64, 0), (1, 2, 70, 128, 65, 32),
    (2, 2, 300, 32, 80, 39), (1, 3, 45, 16, 80, 79), (2, 2, 17, 32, 80, 0), (1, 1, 500, 64, 27, 20), (2, 2, 64, 16, 31, 30),
    (1, 2, 1, 16, 80, 40), (2, 4, 257, 32, 49, 24),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", WIDE_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_wide_windows_match_oracle(geom, dtype):
    """W up to 80 and lopsided windows (more than 16 keys on one side) on the matrix-core path."""
    N, H, T, C, W, L = geom
    B = N * H
    q, k, v, do = make_inputs(B, T, C, W, 77, dtype, n=4, scale=C ** -0.5)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(9)) * 0.5
    pad = torch.tensor([0, T // 2, T][:N] + [1] * max(0, N - 3))
    t_valid = (T - pad).to(torch.int32).cuda()
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = rpb.cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=t_valid, num_heads=H)
    out.backward(do.cuda())
    want_o, _, want_lse = O.na1d_forward(q.float(), k.float(), v.float(), W, L, rpb, pad, H)
    wq, wk, wv, wr = O.na1d_backward(q.float(), k.float(), v.float(), do.float(), W, L, rpb, pad, H)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    _, lse = na1d_fused_forward_lse(qd.detach(), kd.detach(), vd.detach(), W, L, rd.detach(), t_valid, H)
    assert torch.allclose(lse.cpu(), want_lse, atol=2e-3, rtol=1e-4), "LSE"
    for name, got, want in (("dQ", qd.grad, wq), ("dK", kd.grad, wk), ("dV", vd.grad, wv)):
        assert O.rel_l2(got.float(), want) < tol, name
    assert _err(rd.grad, wr) < tol, "drpb"
    _lib.load().na1d_force_generic(1)               # the generic kernels are the second opinion
    try:
        ref, _ = na1d_fused_forward_lse(qd.detach(), kd.detach(), vd.detach(), W, L, rd.detach(), t_valid, H)
    finally:
        _lib.load().na1d_force_generic(0)
    assert O.rel_l2(out.float(), ref.float()) < tol


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_fused_scale_argument_and_optional_inputs(dtype):
    """scale multiplies the fp32 scores; rpb / t_valid / lse are optional."""
    N, H, T, C, W, L = 2, 2, 40, 32, 15, 7
    B = N * H
    q, k, v, do = make_inputs(B, T, C, W, 41, dtype, n=4)
    scale = C ** -0.5
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = na1d_fused(qd, kd, vd, W, L, scale=scale)
    out.backward(do.cuda())
    qs = (q.float() * scale).requires_grad_(True)
    want_o, _, _ = O.na1d_forward(qs, k.float(), v.float(), W, L)
    wq, wk, wv, _ = O.na1d_backward(q.float() * scale, k.float(), v.float(), do.float(), W, L)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol
    assert O.rel_l2(qd.grad.float(), wq * scale) < tol      # chain rule through q*scale
    assert O.rel_l2(kd.grad.float(), wk) < tol
    assert O.rel_l2(vd.grad.float(), wv) < tol
    # lse = NULL is allowed for inference
    o2 = torch.empty_like(qd)
    _lib.call_fused_forward(o2, None, qd.detach(), kd.detach(), vd.detach(), None, None, B, 1, T, C, W, L, scale)
    assert torch.equal(o2, out.detach())


def test_config1_forward_bf16():
    """Single NA1D forward, bf16: batch 32, heads 4, T 200, head_dim 64, window 7."""
    N, H, T, C, W = 32, 4, 200, 64, 7
    _, L = O.split_window(W)
    q, k, v = make_inputs(N * H, T, C, W, 1, torch.bfloat16, scale=C ** -0.5)
    out = na1d_fused(*dev(q, k, v), W, L, num_heads=H)
    want, _, _ = O.na1d_forward(q.float(), k.float(), v.float(), W, L)
    assert O.rel_l2(out.float(), want) < 1e-2
    QK, AV = nattn.getNA1dFunction(C, 1, torch.bfloat16)
    qd, kd, vd = dev(q, k, v)
    out2 = AV.apply(torch.softmax(QK.apply(qd, kd, W, L, 1) + O.attn_mask(T, W, L).cuda(), -1), vd, W, L, 1)
    assert O.rel_l2(out2.float(), want) < 1e-2


def test_config2_forward_backward_fp16():
    """NA1D fwd+bwd, fp16: batch 128, heads 8, T 300, head_dim 32, window 15; dQ/dK/dV vs fp32."""
    N, H, T, C, W = 128, 8, 300, 32, 15
    _, L = O.split_window(W)
    q, k, v, do = make_inputs(N * H, T, C, W, 2, torch.float16, n=4, scale=C ** -0.5)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = na1d_fused(qd, kd, vd, W, L, num_heads=H)
    out.backward(do.cuda())
    torch.set_num_threads(max(1, min(16, os.cpu_count() or 1)))
    qf, kf, vf = q.float(), k.float(), v.float()
    want, _, _ = O.na1d_forward(qf, kf, vf, W, L)
    wq, wk, wv, _ = O.na1d_backward_formulas(qf, kf, vf, do.float(), W, L)
    for name, got, ref in (("O", out, want), ("dQ", qd.grad, wq), ("dK", kd.grad, wk), ("dV", vd.grad, wv)):
        assert O.rel_l2(got.float(), ref) < 2e-3, name


FULL_LAUNCHES = [  # (N, H, T, C, W, L, dtype): the configurations' shapes and a wide window, forward and backward
    (128, 16, 100, 16, 27, 13, torch.float16), (128, 8, 300, 32, 15, 7, torch.float16),
    (64, 16, 1000, 16, 27, 13, torch.bfloat16), (128, 8, 300, 32, 65, 32, torch.float16),
]


@pytest.mark.parametrize("case", FULL_LAUNCHES, ids=lambda c: "x".join(map(str, c[:6])))
def test_full_launches_are_deterministic_and_batch_invariant(case):
    """Under a launch that fills the card (every CU holds several workgroups, copies and matrix instructions of
    different workgroups interleave) the kernels give the same bits twice, and a slice of the batch run alone gives
    the bits it has inside the batch: outputs and the gradients of q, k, v (d rpb, summed with float atomics by
    default, is left out).  The slice is checked against the oracle."""
    N, H, T, C, W, L, dtype = case
    B = N * H
    q, k, v, do = make_inputs(B, T, C, W, 7, dtype, n=4, scale=C ** -0.5)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(3)) * 0.5
    t_valid = torch.full((N,), T, dtype=torch.int32)
    t_valid[N // 2:] = T - T // 4
    sl, ns = slice(B // 2 - 2 * H, B // 2 + 2 * H), slice(N // 2 - 2, N // 2 + 2)
    print("full launch", case, flush=True)

    def run(qq, kk, vv, dd, tv):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (qq, kk, vv))
        out = na1d_fused(qd, kd, vd, W, L, rpb=rpb.cuda(), t_valid=tv.cuda(), num_heads=H)
        out.backward(dd.cuda())
        return out.detach(), qd.grad, kd.grad, vd.grad

    full = run(q, k, v, do, t_valid)
    again = run(q, k, v, do, t_valid)
    alone = run(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), do[sl].contiguous(), t_valid[ns])
    for name, a, b, c in zip(("O", "dQ", "dK", "dV"), full, again, alone):
        assert torch.equal(a, b), name + ": two runs differ"
        assert torch.equal(a[sl], c), name + ": a slice alone differs from the slice inside the batch"
    pad = T - t_valid[ns]
    qf, kf, vf = q[sl].float(), k[sl].float(), v[sl].float()
    want, _, _ = O.na1d_forward(qf, kf, vf, W, L, rpb=rpb, padding=pad, num_heads=H)
    assert O.rel_l2(alone[0].float().cpu(), want) < TOL[dtype]


@pytest.mark.parametrize("case", [(256, 16, 100, 16, 27, 13, torch.bfloat16), (128, 8, 300, 32, 15, 7, torch.float16)],
                         ids=lambda c: "x".join(map(str, c[:6])))
def test_full_launches_in_the_projection_layout_and_through_the_two_call_api(case):
    """The same two properties for the operator on the qkv projection's output (head-group forward, strided backward)
    and for the un-fused functions of the reference's API, at full size."""
    N, H, T, C, W, L, dtype = case
    g = torch.Generator().manual_seed(11)
    qkv = (torch.randn(N, T, 3, H, C, generator=g) * 0.5).to(dtype)
    do = torch.randn(N, T, H * C, generator=g).to(dtype)
    rpb = torch.randn(H, W, generator=g) * 0.5
    ns = slice(N // 2 - 2, N // 2 + 2)
    print("full launch, projection layout", case, flush=True)

    def run(x, dd):
        xd = x.cuda().requires_grad_(True)
        out = na1d_fused_qkv(xd, W, L, rpb=rpb.cuda(), scale=C ** -0.5)
        out.backward(dd.cuda())
        return out.detach(), xd.grad

    full, again, alone = run(qkv, do), run(qkv, do), run(qkv[ns].contiguous(), do[ns].contiguous())
    for name, a, b, c in zip(("O", "dqkv"), full, again, alone):
        assert torch.equal(a, b), name + ": two runs differ"
        assert torch.equal(a[ns], c), name + ": a slice alone differs from the slice inside the batch"

    QK, AV = nattn.getNA1dFunction(C, 1, dtype)
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3).reshape(N * H, T, C).contiguous() for i in range(3))
    sl = slice(ns.start * H, ns.stop * H)

    def chain(qq, kk, vv):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (qq, kk, vv))
        attn = QK.apply(qd, kd, W, L, 1)
        out = AV.apply(torch.softmax(attn, -1), vd, W, L, 1)
        out.float().square().sum().backward()
        return attn.detach(), out.detach(), qd.grad, kd.grad, vd.grad

    full, again, alone = chain(q, k, v), chain(q, k, v), chain(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous())
    for name, a, b, c in zip(("S", "O", "dQ", "dK", "dV"), full, again, alone):
        assert torch.equal(a, b), name + ": two runs differ"
        assert torch.equal(a[sl], c), name + ": a slice alone differs from the slice inside the batch"


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_model_shape_properties_at_full_size(dtype):
    """cfg3's NA shape (B 4096, T 100, C 16, W 27): size-independent properties
    instead of a full CPU oracle pass - batch invariance, agreement of the fused
    kernel with the un-fused chain, rows of P summing to one via v = 1."""
    N, H, T, C, W, L = 256, 16, 100, 16, 27, 13
    B = N * H
    q, k, v = make_inputs(B, T, C, W, 51, dtype, scale=0.25)
    qd, kd, vd = dev(q, k, v)
    out = na1d_fused(qd, kd, vd, W, L, num_heads=H)
    # a slice alone gives the same bits as inside the batch
    sl = slice(1000, 1016)
    out_sl = na1d_fused(qd[sl].contiguous(), kd[sl].contiguous(), vd[sl].contiguous(), W, L, num_heads=H)
    assert torch.equal(out[sl], out_sl)
    # the slice against the oracle
    want, _, _ = O.na1d_forward(q[sl].float(), k[sl].float(), v[sl].float(), W, L)
    assert O.rel_l2(out_sl.float(), want) < TOL[dtype]
    # fused == un-fused chain (two independent kernel families)
    QK, AV = nattn.getNA1dFunction(C, 1, dtype)
    chain = AV.apply(torch.softmax(QK.apply(qd, kd, W, L, 1) + O.attn_mask(T, W, L).cuda(), -1), vd, W, L, 1)
    assert O.rel_l2(out.float(), chain.float()) < TOL[dtype]
    # v = 1 -> every output element is sum_j P = 1 (up to e^-100 on masked slots)
    ones = na1d_fused(qd, kd, torch.ones_like(vd), W, L, num_heads=H)
    assert (ones.float() - 1).abs().max().item() < (2e-2 if dtype == torch.bfloat16 else 4e-3)


def test_tensors_beyond_4_gib_are_addressed_with_64_bit_offsets():
    """B*T*C*2 bytes > 2^32 per tensor: the first and the last sequences of the big call must equal the same
    sequences run alone, bit for bit (the reference indexes with 32-bit ints and cannot run this size)."""
    B, T, C, W, L = 2200, 8000, 128, 15, 7
    assert B * T * C * 2 > 2 ** 32
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v, do = (torch.randn(B, T, C, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(4))
    q.mul_(C ** -0.5)
    out, lse = na1d_fused_forward_lse(q, k, v, W, L)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    _lib.call_fused_backward(dq, dk, dv, None, q, k, v, out, do, lse, None, None, B, 1, T, C, W, L, 1.0)
    for b in (0, B - 1):
        sl = slice(b, b + 1)
        o1, l1 = na1d_fused_forward_lse(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), W, L)
        assert torch.equal(o1, out[sl]) and torch.equal(l1, lse[sl])
        g1 = [torch.empty_like(o1) for _ in range(3)]
        _lib.call_fused_backward(*g1, None, q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), o1,
                                 do[sl].contiguous(), l1, None, None, 1, 1, T, C, W, L, 1.0)
        for got, big in zip(g1, (dq, dk, dv)):
            assert torch.equal(got, big[sl])
    attn = torch.empty(B, T, W, device="cuda")
    _unfused("na1d_qk_forward", attn, q, k, W, L)
    a1 = _unfused("na1d_qk_forward", torch.empty(1, T, W, device="cuda"), q[B - 1:].contiguous(), k[B - 1:].contiguous(), W, L)
    assert torch.equal(a1, attn[B - 1:])


@pytest.mark.parametrize("C,W,L", [(16, 27, 13), (48, 15, 7), (24, 9, 2)], ids=["hd16", "hd48", "hd24"])
def test_deterministic_rpb_gradient_is_bit_reproducible(C, W, L):
    """With deterministic=True d rpb is folded in a fixed order: two runs give the same bits, and the
    atomics path agrees with it to fp32 rounding - also for head dims that run at the next kernel width."""
    N, H, T = 16, 16, 100
    q, k, v, do = make_inputs(N * H, T, C, W, 71, torch.float16, n=4, scale=0.25)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(5)) * 0.3
    grads = []
    for det in (True, True, False):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        rd = rpb.cuda().requires_grad_(True)
        na1d_fused(qd, kd, vd, W, L, rpb=rd, num_heads=H, deterministic=det).backward(do.cuda())
        grads.append((rd.grad.clone(), qd.grad.clone(), kd.grad.clone(), vd.grad.clone()))
    assert all(torch.equal(a, b) for a, b in zip(grads[0], grads[1]))
    assert all(torch.equal(a, b) for a, b in zip(grads[0][1:], grads[2][1:]))       # dq, dk, dv: no atomics at all
    assert torch.allclose(grads[0][0], grads[2][0], rtol=1e-4, atol=1e-4)


def test_deterministic_rpb_gradient_with_dilated_windows():
    """Dilation 2 on 257 rows: residue classes of 129 and 128 rows, and the 128-row class needs the larger workspace.
    One workspace sized over both keeps the fixed order for every class: two runs give the same bits."""
    N, H, T, C, W, L, d = 16, 4, 257, 16, 27, 13, 2
    q, k, v, do = make_inputs(N * H, T, C, W, 73, torch.float16, n=4, scale=0.25)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(6)) * 0.3
    assert _lib.fused_backward_workspace_bytes(N * H, H, 129, C, W, L, torch.float16) < \
        _lib.fused_backward_workspace_bytes(N * H, H, 128, C, W, L, torch.float16)
    grads = []
    for det in (True, True, False):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        rd = rpb.cuda().requires_grad_(True)
        na1d_fused(qd, kd, vd, W, L, rpb=rd, num_heads=H, deterministic=det, dilation=d).backward(do.cuda())
        grads.append((rd.grad.clone(), qd.grad.clone(), kd.grad.clone(), vd.grad.clone()))
    assert all(torch.equal(a, b) for a, b in zip(grads[0], grads[1]))
    assert torch.allclose(grads[0][0], grads[2][0], rtol=1e-4, atol=1e-4)
    # and the library refuses a workspace that is too small instead of falling back to atomics
    B = N * H
    qd, kd, vd, dd = dev(q[:, :128].contiguous(), k[:, :128].contiguous(), v[:, :128].contiguous(), do[:, :128].contiguous())
    out, lse = torch.empty_like(qd), torch.empty(B, 128, device="cuda")
    _lib.call_fused_forward(out, lse, qd, kd, vd, rpb.cuda(), None, B, H, 128, C, W, L, 1.0)
    small = torch.empty(_lib.fused_backward_workspace_bytes(B, H, 129, C, W, L, torch.float16), dtype=torch.uint8, device="cuda")
    with pytest.raises(_lib.NA1DError, match="workspace"):
        _lib.call_fused_backward(torch.empty_like(qd), torch.empty_like(qd), torch.empty_like(qd), torch.zeros(H, W, device="cuda"),
                                 qd, kd, vd, out, dd, lse, rpb.cuda(), None, B, H, 128, C, W, L, 1.0, workspace=small)


def test_deterministic_mode_is_refused_where_it_cannot_be_honoured():
    """Heads wider than 128 channels run the generic kernels, which have no fixed-order reduction of d rpb: asking
    for one raises instead of falling back to atomics without a word."""
    N, H, T, C, W, L = 2, 2, 40, 136, 9, 4
    q, k, v, do = make_inputs(N * H, T, C, W, 72, torch.float16, n=4, scale=0.25)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = (torch.randn(H, W) * 0.3).cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, num_heads=H, deterministic=True)
    with pytest.raises(_lib.NA1DError, match="deterministic"):
        out.backward(do.cuda())
    na1d_fused(qd, kd, vd, W, L, rpb=rd, num_heads=H).backward(do.cuda())          # the default still works
    assert torch.isfinite(rd.grad).all()


@pytest.mark.parametrize("geom", [(8, 4, 150, 32, 33, 16), (4, 2, 200, 16, 65, 32), (3, 2, 90, 64, 80, 0)],
                         ids=lambda g: "x".join(map(str, g)))
def test_deterministic_rpb_gradient_with_wide_windows(geom):
    """The wide-window backward folds d rpb in a fixed order too, given a workspace: two runs give the same bits and
    the atomics path agrees to fp32 rounding."""
    N, H, T, C, W, L = geom
    q, k, v, do = make_inputs(N * H, T, C, W, 74, torch.bfloat16, n=4, scale=C ** -0.5)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(7)) * 0.3
    grads = []
    for det in (True, True, False):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        rd = rpb.cuda().requires_grad_(True)
        na1d_fused(qd, kd, vd, W, L, rpb=rd, num_heads=H, deterministic=det).backward(do.cuda())
        grads.append((rd.grad.clone(), qd.grad.clone(), kd.grad.clone(), vd.grad.clone()))
    assert all(torch.equal(a, b) for a, b in zip(grads[0], grads[1]))
    assert all(torch.equal(a, b) for a, b in zip(grads[0][1:], grads[2][1:]))
    assert torch.allclose(grads[0][0], grads[2][0], rtol=1e-4, atol=1e-4)
    want = O.na1d_backward(q.float(), k.float(), v.float(), do.float(), W, L, rpb, None, H)[3]
    assert _err(grads[0][0].cpu(), want) < TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_two_kernel_families_agree(dtype):
    """The matrix-core kernels and the generic kernels are independent implementations; na1d_force_generic(1)
    routes the same C-ABI calls to the generic ones."""
    N, H, T, C, W, L = 3, 4, 150, 32, 15, 7
    B = N * H
    q, k, v, do = dev(*make_inputs(B, T, C, W, 81, dtype, n=4, scale=C ** -0.5))
    s = seeded_scores(B, T, W, 9).cuda()
    rpb = (torch.randn(H, W, generator=torch.Generator().manual_seed(6)) * 0.3).cuda()
    tv = torch.tensor([T, T - 17, 40], dtype=torch.int32).cuda()

    def run_all():
        attn = _unfused("na1d_qk_forward", torch.empty(B, T, W, device="cuda"), q, k, W, L)
        av = _unfused("na1d_av_forward", torch.empty_like(v), s, v, W, L)
        ga = _unfused("na1d_k_backward", torch.empty_like(q), s, q, W, L)
        qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
        rd = rpb.clone().requires_grad_(True)
        o = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=tv, num_heads=H)
        o.backward(do)
        return [attn, av.float(), ga.float(), o.detach().float(), qd.grad.float(), kd.grad.float(), vd.grad.float(), rd.grad]

    fast = run_all()
    assert _lib.load().na1d_force_generic(1) == 0
    try:
        slow = run_all()
    finally:
        assert _lib.load().na1d_force_generic(0) == 1
    assert O.rel_l2(fast[0], slow[0]) < 1e-5
    for a, b in zip(fast[1:], slow[1:]):
        assert O.rel_l2(a, b) < TOL[dtype]
    assert not torch.equal(fast[1], slow[1]) or not torch.equal(fast[3], slow[3])     # they really are different code


def test_forward_and_backward_replay_from_a_hip_graph():
    """The C ABI allocates nothing and launches only on the stream it is given, so a step can be captured once and
    replayed: three replays on changing inputs, eager work in between, each checked against the eager result."""
    N, H, T, C, W, L = 4, 4, 150, 16, 27, 13
    B = N * H
    gen = torch.Generator(device="cuda").manual_seed(3)
    new = lambda *shape: torch.randn(*shape, device="cuda", generator=gen)
    q, k, v, do = (new(B, T, C).to(torch.bfloat16) for _ in range(4))
    rpb = new(H, W) * 0.3
    tv = torch.tensor([T, T - 9, 70, 1], dtype=torch.int32, device="cuda")
    out, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    lse = torch.empty(B, T, device="cuda")
    drpb = torch.zeros(H, W, device="cuda")
    nbytes = _lib.fused_backward_workspace_bytes(B, H, T, C, W, L, q.dtype)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")

    def step():
        drpb.zero_()                                   # a fill kernel, not a memset node
        _lib.call_fused_forward(out, lse, q, k, v, rpb, tv, B, H, T, C, W, L, 1.0)
        _lib.call_fused_backward(dq, dk, dv, drpb, q, k, v, out, do, lse, rpb, tv, B, H, T, C, W, L, 1.0, workspace=ws)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                         # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for t in (q, k, v, do):
            t.copy_(new(B, T, C).to(torch.bfloat16))   # eager work between the replays
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, lse, dq, dk, dv, drpb)]
        step()
        torch.cuda.synchronize()
        for a, b in zip(got, (out, lse, dq, dk, dv, drpb)):
            assert torch.equal(a, b), rep              # the workspace path makes d rpb reproducible too


def test_profile_events_bracket_the_kernel():
    """na1d_profile_events: the pair is recorded around the kernel by the launch itself; switched off again, launches
    are ordinary ones."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    lib = _lib.load()
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipEventCreate(ctypes.byref(a)) == 0 and hip.hipEventCreate(ctypes.byref(b)) == 0
    q, k, v = dev(*make_inputs(512, 300, 32, 15, 2, torch.float16, n=3))
    want, _ = na1d_fused_forward_lse(q, k, v, 15, 7)
    assert lib.na1d_profile_events(a, b) == 0
    try:
        got, _ = na1d_fused_forward_lse(q, k, v, 15, 7)
    finally:
        assert lib.na1d_profile_events(None, None) == 0
    torch.cuda.synchronize()
    ms = ctypes.c_float()
    assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
    assert 1e-3 < ms.value < 1.0                      # a few microseconds of kernel, not a stream's worth of gaps
    assert torch.equal(got, want)
    again, _ = na1d_fused_forward_lse(q, k, v, 15, 7)
    assert torch.equal(again, want)
    hip.hipEventDestroy(a)
    hip.hipEventDestroy(b)


def test_profile_events_are_refused_under_capture_and_record_nothing():
    """With a pair of events set, a launch on a capturing stream comes back as NA1D_ERR_LAUNCH and the graph stays
    empty - the reduction kernel that follows the backward's main launch included."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    lib = _lib.load()
    N, H, T, C, W, L = 4, 4, 100, 16, 27, 13
    B = N * H
    q, k, v, do = dev(*make_inputs(B, T, C, W, 4, torch.bfloat16, n=4))
    rpb = torch.zeros(H, W, device="cuda")
    out, lse = torch.empty_like(q), torch.empty(B, T, device="cuda")
    _lib.call_fused_forward(out, lse, q, k, v, rpb, None, B, H, T, C, W, L, 1.0)
    dq, dk, dv, drpb = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.zeros(H, W, device="cuda")
    ws = torch.empty(_lib.fused_backward_workspace_bytes(B, H, T, C, W, L, q.dtype), dtype=torch.uint8, device="cuda")
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipEventCreate(ctypes.byref(a)) == 0 and hip.hipEventCreate(ctypes.byref(b)) == 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    stream = ctypes.c_void_p(side.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    graph = ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 2) == 0          # relaxed mode: other threads of the process are left alone
    try:
        assert lib.na1d_profile_events(a, b) == 0
        st = lib.na1d_fused_backward(P(dq), P(dk), P(dv), P(drpb), P(q), P(k), P(v), P(out), P(do), P(lse), P(rpb), None,
                                     B, H, T, C, W, L, 1.0, _lib.dtype_tag(q.dtype), P(ws), ws.numel(), stream)
    finally:
        lib.na1d_profile_events(None, None)
        assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
    assert st == -7
    count = ctypes.c_size_t(99)
    assert hip.hipGraphGetNodes(graph, None, ctypes.byref(count)) == 0
    assert count.value == 0
    hip.hipGraphDestroy(graph)
    hip.hipEventDestroy(a)
    hip.hipEventDestroy(b)
    # the stream is usable again and an ordinary launch on it works
    with torch.cuda.stream(side):
        _lib.call_fused_backward(dq, dk, dv, drpb, q, k, v, out, do, lse, rpb, None, B, H, T, C, W, L, 1.0, workspace=ws)
    side.synchronize()
    assert torch.isfinite(dq.float()).all()


def test_runs_on_the_current_stream():
    """Launches go to torch's current stream (the reference uses the legacy default
    stream; its data prefetcher runs a side stream, public/Utils.py:89-100)."""
    B, T, C, W, L = 8, 120, 16, 27, 13
    q, k, v = dev(*make_inputs(B, T, C, W, 61, torch.bfloat16))
    base = na1d_fused(q, k, v, W, L)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = na1d_fused(q, k, v, W, L)
    side.synchronize()
    assert torch.equal(base, other)


def test_errors_become_python_exceptions():
    q = torch.zeros(2, 8, 16, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.NA1DError):
        _lib.call_unfused("na1d_qk_forward", torch.empty(2, 8, 81, device="cuda"), q, q, 2, 8, 16, 81, 3, q.dtype)
    with pytest.raises(_lib.NA1DError):
        _lib.call_unfused("na1d_qk_forward", torch.empty(2, 8, 5, device="cuda"), q, q, 2, 8, 12, 5, 2, q.dtype)


# --------------------------------------------------------------------------- attention dropout inside the kernels
DROP_GEOMS = [  # (N, H, T, C, W, L): two-block, merged three-block, wide and lopsided windows, padded head dims, ragged tiles
    (2, 2, 61, 32, 15, 7), (2, 4, 100, 16, 27, 13), (1, 2, 150, 64, 33, 16), (2, 1, 90, 32, 65, 32),
    (2, 2, 47, 24, 9, 0), (1, 3, 130, 128, 17, 16), (2, 2, 5, 16, 27, 13), (1, 2, 300, 48, 80, 50),
    (2, 2, 40, 136, 9, 4), (1, 2, 70, 160, 27, 13),      # heads wider than 128 channels: the generic kernels
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", DROP_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_fused_dropout_matches_oracle_with_the_same_mask(geom, dtype):
    N, H, T, C, W, L = geom
    B, p, seed = N * H, 0.3, 0x1234_5678_9ABC_DEF0
    q, k, v, do = make_inputs(B, T, C, W, 51, dtype, n=4, scale=C ** -0.5)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(6)) * 0.5
    pad = torch.tensor([0, T // 3][:N])
    t_valid = (T - pad).to(torch.int32).cuda()
    print("fused dropout", geom, dtype, flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = rpb.cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=t_valid, num_heads=H, dropout_p=p, seed=seed)
    out.backward(do.cuda())

    keep = O.dropout_keep(B, T, W, p, seed)
    qf, kf, vf = q.float(), k.float(), v.float()
    want_o, _, _ = O.na1d_forward(qf, kf, vf, W, L, rpb, pad, H, keep=keep, p_drop=p)
    wq, wk, wv, wr = O.na1d_backward(qf, kf, vf, do.float(), W, L, rpb, pad, H, keep=keep, p_drop=p)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert O.rel_l2(qd.grad.float(), wq) < tol, "dQ"
    assert O.rel_l2(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"
    assert _err(rd.grad, wr) < tol, "drpb"
    # the dropped operator is not the plain one, and the same seed gives the same bits
    plain = na1d_fused(qd.detach(), kd.detach(), vd.detach(), W, L, rpb=rpb.cuda(), t_valid=t_valid, num_heads=H)
    again = na1d_fused(qd.detach(), kd.detach(), vd.detach(), W, L, rpb=rpb.cuda(), t_valid=t_valid, num_heads=H,
                       dropout_p=p, seed=seed)
    assert torch.equal(again, out) and not torch.equal(plain, out)


@pytest.mark.parametrize("W,L", [(15, 7), (27, 13), (65, 32), (31, 3)])
def test_dropout_mask_is_bit_exact(W, L):
    """One-hot values turn the output into the dropped probability matrix itself: with zero queries every
    in-range slot has a positive probability, so out[t, u] != 0 exactly where slot u - t + L of row t is kept."""
    B, T, C, p, seed = 3, 100, 128, 0.5, 99
    q = torch.zeros(B, T, C, dtype=torch.float16, device="cuda")
    v = torch.zeros(B, T, C, dtype=torch.float16)
    v[:, torch.arange(T), torch.arange(T)] = 1.0
    out = na1d_fused(q, q, v.cuda(), W, L, dropout_p=p, seed=seed).cpu()
    keep = O.dropout_keep(B, T, W, p, seed)
    want = torch.zeros(B, T, C, dtype=torch.bool)
    for j in range(W):
        lo, hi = max(0, L - j), min(T, T + L - j)
        rows = torch.arange(lo, hi)
        want[:, rows, rows - L + j] = keep[:, lo:hi, j]
    assert torch.equal(out != 0, want)
    kept = out[out != 0].float()
    assert ((kept * (1 - p) * W).round() >= 1).all()                 # survivors carry 1 / (1 - p)


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom,dilation", [((2, 2, 61, 32, 15, 7), 2), ((2, 4, 100, 16, 27, 13), 3), ((1, 2, 150, 64, 33, 16), 2),
                                           ((2, 2, 47, 24, 9, 0), 4), ((2, 1, 90, 32, 65, 32), 2), ((2, 2, 5, 16, 27, 13), 7)],
                         ids=lambda g: "x".join(map(str, g)) if isinstance(g, tuple) else "d%d" % g)
def test_fused_dropout_with_dilated_windows_matches_oracle(geom, dilation, dtype):
    """The launches on the residue classes drop by (sequence, row, slot) of the whole operator: same oracle mask as
    for dilation 1, applied to the dilated window (models/PCF_NATransformer.py:149 with :158-170)."""
    N, H, T, C, W, L = geom
    B, p, seed = N * H, 0.3, 0x0FED_CBA9_8765_4321
    q, k, v, do = make_inputs(B, T, C, W, 52, dtype, n=4, scale=C ** -0.5)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(7)) * 0.5
    pad = torch.tensor([0, T // 3][:N])
    t_valid = (T - pad).to(torch.int32).cuda()
    print("fused dropout dilated", geom, dilation, dtype, flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rd = rpb.cuda().requires_grad_(True)
    out = na1d_fused(qd, kd, vd, W, L, rpb=rd, t_valid=t_valid, num_heads=H, dilation=dilation, dropout_p=p, seed=seed)
    out.backward(do.cuda())
    keep = O.dropout_keep(B, T, W, p, seed)
    qf, kf, vf = q.float(), k.float(), v.float()
    want_o, _, _ = O.na1d_forward(qf, kf, vf, W, L, rpb, pad, H, dilation, keep=keep, p_drop=p)
    wq, wk, wv, wr = O.na1d_backward(qf, kf, vf, do.float(), W, L, rpb, pad, H, dilation, keep=keep, p_drop=p)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert O.rel_l2(qd.grad.float(), wq) < tol, "dQ"
    assert O.rel_l2(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"
    assert _err(rd.grad, wr) < tol, "drpb"


@pytest.mark.parametrize("W,L,dilation", [(15, 7, 2), (27, 13, 3), (65, 32, 2), (9, 0, 5)])
def test_dilated_dropout_mask_is_bit_exact(W, L, dilation):
    """As test_dropout_mask_is_bit_exact, with slot j of row t at column t + (j - L) * dilation."""
    B, T, C, p, seed = 3, 100, 128, 0.5, 77
    q = torch.zeros(B, T, C, dtype=torch.float16, device="cuda")
    v = torch.zeros(B, T, C, dtype=torch.float16)
    v[:, torch.arange(T), torch.arange(T)] = 1.0
    out = na1d_fused(q, q, v.cuda(), W, L, dilation=dilation, dropout_p=p, seed=seed).cpu()
    keep = O.dropout_keep(B, T, W, p, seed)
    want = torch.zeros(B, T, C, dtype=torch.bool)
    for j in range(W):
        off = (j - L) * dilation
        rows = torch.arange(max(0, -off), min(T, T - off))
        if rows.numel():
            want[:, rows, rows + off] = keep[:, rows, j]
    assert torch.equal(out != 0, want)


def test_strided_dropout_rejects_rows_outside_the_sequence():
    q = torch.zeros(2, 2, 20, 32, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(4, 20, device="cuda")
    ok = _lib.call_fused_forward_strided(torch.empty_like(q), lse, q, q, q, None, None, 5, 2, 1.0, dropout=(0.5, 1, 2, 1, 40))
    assert ok == 0
    for bad in [(0.5, 1, 2, 2, 40), (0.5, 1, 2, 1, 39), (0.5, 1, 0, 0, 40), (1.0, 1, 1, 0, 20)]:
        with pytest.raises(_lib.NA1DError):
            _lib.call_fused_forward_strided(torch.empty_like(q), lse, q, q, q, None, None, 5, 2, 1.0, dropout=bad)


@pytest.mark.parametrize("dilation", [1, 2])
def test_in_place_qkv_operator_drops_like_the_split_one(dilation):
    """na1d_fused_qkv(..., dropout_p, seed) on [N, T, 3, H, C] draws the mask na1d_fused draws on the split tensors
    (sequence n * H + h), forward and backward."""
    N, H, T, C, W, L, p, seed = 2, 4, 90, 16, 27, 13, 0.25, 1234567
    g = torch.Generator().manual_seed(8)
    qkv = (torch.randn(N, T, 3, H, C, generator=g) * 0.5).to(torch.float16).cuda().requires_grad_(True)
    rpb = (torch.randn(H, W, generator=g) * 0.3).cuda().requires_grad_(True)
    t_valid = torch.tensor([T, T - 17], dtype=torch.int32).cuda()
    do = torch.randn(N, T, H * C, generator=g).to(torch.float16).cuda()
    out = na1d_fused_qkv(qkv, W, L, rpb=rpb, t_valid=t_valid, scale=1.0, dilation=dilation, dropout_p=p, seed=seed)
    out.backward(do)
    q, k, v = (qkv.detach()[:, :, i].permute(0, 2, 1, 3).reshape(N * H, T, C).contiguous().requires_grad_(True) for i in range(3))
    rpb2 = rpb.detach().clone().requires_grad_(True)
    ref = na1d_fused(q, k, v, W, L, rpb=rpb2, t_valid=t_valid, num_heads=H, dilation=dilation, dropout_p=p, seed=seed)
    ref.backward(do.view(N, T, H, C).permute(0, 2, 1, 3).reshape(N * H, T, C))
    assert torch.equal(out.view(N, T, H, C).permute(0, 2, 1, 3).reshape(N * H, T, C), ref)
    for i, z in enumerate((q, k, v)):
        assert torch.equal(qkv.grad[:, :, i].permute(0, 2, 1, 3).reshape(N * H, T, C), z.grad)
    assert torch.allclose(rpb.grad, rpb2.grad, rtol=1e-4, atol=1e-5)
    plain = na1d_fused_qkv(qkv.detach(), W, L, rpb=rpb.detach(), t_valid=t_valid, dilation=dilation)
    assert not torch.equal(plain, out.detach())


def test_dropout_rate_zero_is_the_plain_operator_and_bad_rates_are_rejected():
    q, k, v = dev(*make_inputs(4, 50, 32, 15, 3, torch.bfloat16))
    assert torch.equal(na1d_fused(q, k, v, 15, 7, dropout_p=0.0), na1d_fused(q, k, v, 15, 7))
    out = torch.empty_like(q)
    with pytest.raises(_lib.NA1DError):
        _lib.call_fused_forward(out, None, q, k, v, None, None, 4, 1, 50, 32, 15, 7, 1.0, dropout=(1.0, 1))
    wide = torch.randn(2, 9, 3, 1, 136, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).cuda()
    with pytest.raises(_lib.NA1DError, match="dilated"):              # head_dim > 128: dropout, but not on dilated windows
        na1d_fused_qkv(wide.requires_grad_(True), 5, 2, dilation=2, dropout_p=0.5, seed=1)


def test_inference_path_of_the_projection_layout_equals_the_autograd_path():
    """Without gradients na1d_fused_qkv makes one library call on raw pointers; same bits as the autograd path."""
    N, H, T, C, W, L = 3, 4, 77, 16, 27, 13
    g = torch.Generator().manual_seed(2)
    qkv = (torch.randn(N, T, 3, H, C, generator=g) * 0.5).to(torch.bfloat16).cuda()
    rpb = (torch.randn(1, H, 1, W, generator=g) * 0.3).cuda()
    tv = torch.tensor([T, 40, 0], dtype=torch.int32).cuda()
    with torch.no_grad():
        lean = na1d_fused_qkv(qkv, W, L, rpb=rpb, t_valid=tv, scale=0.25)
    full = na1d_fused_qkv(qkv.clone().requires_grad_(True), W, L, rpb=rpb, t_valid=tv, scale=0.25)
    assert lean.shape == (N, T, H * C) and torch.equal(lean, full.detach())
    with torch.no_grad():                                   # head_dim > 128: falls through to the general path
        wide = torch.randn(1, 9, 3, 1, 136, generator=g).to(torch.bfloat16).cuda()
        assert na1d_fused_qkv(wide, 5, 2).shape == (1, 9, 136)


def _guarded(shape, dtype, fill):
    """A tensor in the middle of a larger allocation whose surroundings hold a sentinel."""
    n = 1
    for s in shape:
        n *= s
    pad = 4096                                               # elements on each side; keeps 16-byte alignment
    buf = torch.full((n + 2 * pad,), fill, dtype=dtype, device="cuda")
    return buf, buf[pad:pad + n].view(shape), pad


@pytest.mark.parametrize("geom", [(3, 2, 37, 32, 15, 7), (2, 4, 100, 16, 27, 13), (2, 1, 45, 64, 65, 32), (1, 2, 5, 24, 9, 4),
                                  (2, 2, 129, 128, 17, 0)], ids=lambda g: "x".join(map(str, g)))
def test_no_entry_point_writes_outside_its_outputs(geom):
    """Ragged last tiles, padded head dims and halo rows: every output sits between sentinel bands that must come
    back untouched (an out-of-bounds store inside the allocation would not fault, it would land there)."""
    N, H, T, C, W, L = geom
    B, dtype = N * H, torch.bfloat16
    q, k, v, do = dev(*make_inputs(B, T, C, W, 61, dtype, n=4))
    rpb = torch.zeros(H, W, device="cuda")
    outs = {name: _guarded((B, T, C), dtype, 3.0) for name in ("out", "dq", "dk", "dv", "gout", "gdq", "gdk", "gdv", "av", "kb")}
    f32 = {name: _guarded(shape, torch.float32, 3.0) for name, shape in
           (("lse", (B, T)), ("glse", (B, T)), ("attn", (B, T, W)), ("drpb", (H, W)), ("ws", (B, T)))}
    f32["drpb"][1].zero_()
    _lib.call_fused_forward(outs["out"][1], f32["lse"][1], q, k, v, rpb, None, B, H, T, C, W, L, 0.3)
    _lib.call_fused_backward(outs["dq"][1], outs["dk"][1], outs["dv"][1], f32["drpb"][1], q, k, v, outs["out"][1], do,
                             f32["lse"][1], rpb, None, B, H, T, C, W, L, 0.3)
    _lib.call_global_forward(outs["gout"][1], f32["glse"][1], q, k, v, None, B, H, T, C, 0.3)
    _lib.call_global_backward(outs["gdq"][1], outs["gdk"][1], outs["gdv"][1], q, k, v, outs["gout"][1], do, f32["glse"][1],
                              None, B, H, T, C, 0.3, f32["ws"][1])
    _lib.call_unfused("na1d_qk_forward", f32["attn"][1], q, k, B, T, C, W, L, dtype)
    _lib.call_unfused("na1d_av_forward", outs["av"][1], f32["attn"][1], v, B, T, C, W, L, dtype)
    _lib.call_unfused("na1d_k_backward", outs["kb"][1], f32["attn"][1], q, B, T, C, W, L, dtype)
    torch.cuda.synchronize()
    for name, (buf, view, pad) in {**outs, **f32}.items():
        assert (buf[:pad] == 3.0).all() and (buf[pad + view.numel():] == 3.0).all(), name
        assert torch.isfinite(view.float()).all(), name
