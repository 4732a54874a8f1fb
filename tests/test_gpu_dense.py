"""GPU parity of the dense ("global") attention kernels against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import na1d_oracle as O
from na1d_amd import _lib
from na1d_amd.dense import global_attention
from _util import TOL, make_inputs

pytestmark = pytest.mark.gpu


DTYPES = [torch.bfloat16, torch.float16]
GEOMS = [  # (N, H, T, C): one tile, ragged tiles, several strips and chunks, every kernel width, padded widths
    (1, 1, 1, 16), (2, 2, 16, 16), (3, 2, 37, 32), (2, 4, 64, 16), (3, 1, 65, 64), (2, 2, 130, 32), (1, 2, 300, 16),
    (2, 1, 129, 128), (2, 2, 100, 24), (1, 3, 77, 48), (2, 1, 90, 104), (1, 1, 1000, 32),
    # sequences of up to 128 rows take the whole-sequence kernels: at most 4 tiles, 5 to 8 tiles, 8 tiles exactly, and
    # launches of many sequences
    (2, 3, 49, 64), (2, 2, 128, 64), (1, 2, 113, 64), (1, 2, 128, 128), (1, 1, 17, 128), (3, 256, 100, 16),
    (2, 400, 128, 32), (3, 256, 81, 64),
    # long sequences in a launch large enough for two tiles to a wave (strips in pairs), padded and not
    (2, 256, 200, 16), (1, 512, 250, 32),
    # long sequences with a sample that is padding from its first row on
    (3, 2, 150, 32), (3, 1, 200, 64),
    # long sequences of heads narrower than the kernel's width
    (2, 2, 140, 24), (1, 2, 260, 104),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_global_attention_matches_oracle(geom, dtype):
    N, H, T, C = geom
    B = N * H
    q, k, v, do = make_inputs(B, T, C, 0, 77, dtype, n=4)
    scale = C ** -0.5
    pad = torch.tensor([0, T // 2, T][:N])
    t_valid = (T - pad).to(torch.int32)
    print("global attention", geom, dtype, flush=True)

    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = global_attention(qd, kd, vd, H, t_valid=t_valid.cuda(), scale=scale)
    out.backward(do.cuda())
    torch.cuda.synchronize()

    qf, kf, vf = q.float(), k.float(), v.float()
    want_o, _, want_lse = O.global_forward(qf, kf, vf, scale, pad, H)
    wq, wk, wv = O.global_backward(qf, kf, vf, do.float(), scale, pad, H)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert O.rel_l2(qd.grad.float(), wq) < tol, "dQ"
    assert O.rel_l2(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"
    lse = torch.empty(B, T, dtype=torch.float32, device="cuda")
    o2 = torch.empty_like(qd)
    assert _lib.call_global_forward(o2, lse, qd.detach(), kd.detach(), vd.detach(), t_valid.cuda(), B, H, T, C, scale) == 0
    assert torch.allclose(lse.cpu(), want_lse, atol=2e-3, rtol=1e-4), "LSE"
    assert torch.equal(o2, out)


def test_global_attention_without_padding_and_without_lse():
    N, H, T, C, dtype = 2, 2, 150, 32, torch.bfloat16
    B = N * H
    q, k, v = make_inputs(B, T, C, 0, 5, dtype)
    qd, kd, vd = (t.cuda() for t in (q, k, v))
    out = torch.empty_like(qd)
    assert _lib.call_global_forward(out, None, qd, kd, vd, None, B, H, T, C, 0.2) == 0
    want, _, _ = O.global_forward(q.float(), k.float(), v.float(), 0.2, None, H)
    assert O.rel_l2(out.float(), want) < TOL[dtype]


def test_global_attention_is_deterministic_and_leaves_neighbours_alone():
    """Every output is written once by one wave: two runs agree bit for bit, and rows of neighbouring
    sequences (T not a multiple of the tile) are not touched by the ragged last tile."""
    N, H, T, C, dtype = 2, 3, 41, 32, torch.float16
    B = N * H
    q, k, v, do = make_inputs(B, T, C, 0, 9, dtype, n=4)
    grads = []
    for _ in range(2):
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        global_attention(qd, kd, vd, H).backward(do.cuda())
        grads.append((qd.grad, kd.grad, vd.grad))
    for a, b in zip(*grads):
        assert torch.equal(a, b)
    # sequence b alone equals sequence b inside the batch
    qd, kd, vd = (t[2:3].contiguous().cuda() for t in (q, k, v))
    alone = global_attention(qd, kd, vd, 1)
    full = global_attention(q.cuda(), k.cuda(), v.cuda(), H)
    assert torch.equal(alone[0], full[2])


def test_global_attention_rejects_wide_heads():
    q = torch.zeros(1, 4, 136, dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(q)
    assert _lib.call_global_forward(out, None, q, q, q, None, 1, 1, 4, 136, 1.0) == _lib.UNSUPPORTED


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("geom", [(2, 2, 37, 32), (1, 3, 130, 64), (2, 1, 100, 24), (1, 2, 300, 16), (2, 384, 100, 16),
                                  (2, 2, 128, 64), (2, 256, 200, 16)],
                         ids=lambda g: "x".join(map(str, g)))
def test_global_attention_dropout_matches_oracle_with_the_same_mask(geom, dtype):
    N, H, T, C = geom
    B, p, seed = N * H, 0.3, 0xFEDC_BA98_7654_3210
    q, k, v, do = make_inputs(B, T, C, 0, 88, dtype, n=4)
    scale = C ** -0.5
    pad = torch.tensor([0, T // 3][:N])
    t_valid = (T - pad).to(torch.int32).cuda()
    print("global attention dropout", geom, dtype, flush=True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = global_attention(qd, kd, vd, H, t_valid=t_valid, scale=scale, dropout_p=p, seed=seed)
    out.backward(do.cuda())
    keep = O.dropout_keep(B, T, T, p, seed)
    want_o, _, _ = O.global_forward(q.float(), k.float(), v.float(), scale, pad, H, keep, p)
    wq, wk, wv = O.global_backward(q.float(), k.float(), v.float(), do.float(), scale, pad, H, keep, p)
    tol = TOL[dtype]
    assert O.rel_l2(out.float(), want_o) < tol, "O"
    assert O.rel_l2(qd.grad.float(), wq) < tol, "dQ"
    assert O.rel_l2(kd.grad.float(), wk) < tol, "dK"
    assert O.rel_l2(vd.grad.float(), wv) < tol, "dV"
    again = global_attention(qd.detach(), kd.detach(), vd.detach(), H, t_valid=t_valid, scale=scale, dropout_p=p, seed=seed)
    assert torch.equal(again, out)


def test_global_attention_dropout_mask_is_bit_exact():
    """One-hot values turn the output into the dropped probability matrix: out[t, u] != 0 exactly where kept."""
    B, T, C, p, seed = 2, 100, 128, 0.5, 31
    q = torch.zeros(B, T, C, dtype=torch.float16, device="cuda")
    v = torch.zeros(B, T, C, dtype=torch.float16)
    v[:, torch.arange(T), torch.arange(T)] = 1.0
    out = global_attention(q, q, v.cuda(), 1, scale=1.0, dropout_p=p, seed=seed).cpu()
    keep = O.dropout_keep(B, T, T, p, seed)
    assert torch.equal(out[:, :, :T] != 0, keep) and (out[:, :, T:] == 0).all()


FULL_SIZE = [  # (N, H, T, C, dtype, backward): the models' dense layers at their benchmark sizes, and a long backward
    (256, 4, 100, 64, torch.bfloat16, False), (64, 4, 1000, 64, torch.bfloat16, False),
    (128, 4, 100, 64, torch.float16, True), (64, 4, 520, 64, torch.bfloat16, True),
]


@pytest.mark.parametrize("case", FULL_SIZE, ids=lambda c: "x".join(map(str, c[:4])) + ("-bwd" if c[5] else ""))
def test_global_attention_properties_at_full_size(case):
    """Size-independent properties under a full launch, where every CU holds several workgroups: a slice of the batch
    run alone gives the same bits as inside the batch (forward and gradients), two runs agree bit for bit, rows of P
    sum to one (v = 1 gives 1), and the slice agrees with the oracle."""
    N, H, T, C, dtype, bwd = case
    B = N * H
    q, k, v, do = make_inputs(B, T, C, 0, 123, dtype, n=4)
    scale = C ** -0.5
    t_valid = torch.full((N,), T, dtype=torch.int32)
    t_valid[N // 2:] = T - T // 3                     # half the samples padded
    sl = slice(B // 2 - 2 * H, B // 2 + 2 * H)        # two unpadded and two padded samples
    ns = slice(N // 2 - 2, N // 2 + 2)
    print("global attention at full size", case, flush=True)

    def run(qq, kk, vv, dd, tv):
        qd, kd, vd = (t.cuda().requires_grad_(bwd) for t in (qq, kk, vv))
        out = global_attention(qd, kd, vd, H, t_valid=tv.cuda(), scale=scale)
        if bwd:
            out.backward(dd.cuda())
            return out.detach(), qd.grad, kd.grad, vd.grad
        return (out.detach(),)

    full = run(q, k, v, do, t_valid)
    again = run(q, k, v, do, t_valid)
    alone = run(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), do[sl].contiguous(), t_valid[ns])
    for name, a, b, c in zip(("O", "dQ", "dK", "dV"), full, again, alone):
        assert torch.equal(a, b), name + ": two runs differ"
        assert torch.equal(a[sl], c), name + ": a slice alone differs from the slice inside the batch"
    pad = T - t_valid[ns]
    qf, kf, vf = q[sl].float(), k[sl].float(), v[sl].float()
    want_o, _, _ = O.global_forward(qf, kf, vf, scale, pad, H)
    assert O.rel_l2(alone[0].float().cpu(), want_o) < TOL[dtype], "O"
    if bwd:
        wq, wk, wv = O.global_backward(qf, kf, vf, do[sl].float(), scale, pad, H)
        for name, got, ref in (("dQ", alone[1], wq), ("dK", alone[2], wk), ("dV", alone[3], wv)):
            assert O.rel_l2(got.float().cpu(), ref) < TOL[dtype], name
    ones = run(q, k, torch.ones_like(v), do, t_valid)[0]
    assert (ones.float() - 1).abs().max() < 2e-2
