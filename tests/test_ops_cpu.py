"""The torch.library statement of the boundary: names and schemas of the reference's twelve ops
(extension_na/na_cuda/csrc_tc240_or_bigger/main.cpp:27-41 inside pcf_nat_pytorch2.7.zip) and shape propagation
through their fake kernels - no GPU needed."""
import pytest
import torch

from na1d_amd import ops

NAMES = ["%s_ana_%s" % (p, s) for p in ("bf16", "fp16")
         for s in ("qk_forward", "q_backward", "k_backward", "av_forward", "attn_backward", "v_backward")]


@pytest.mark.parametrize("name", NAMES)
def test_schema_matches_the_reference(name):
    op = getattr(torch.ops.na_cuda, name).default
    args = op._schema.arguments
    assert [a.name for a in args[2:]] == ["N", "T", "C", "win_size", "left"]
    assert [str(a.type) for a in args] == ["Tensor", "Tensor", "int", "int", "int", "int", "int"]
    assert [str(r.type) for r in op._schema.returns] == ["Tensor"]


@pytest.mark.parametrize("prefix,dtype", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_fake_kernels_propagate_shapes(prefix, dtype):
    N, T, C, W, L = 3, 20, 16, 7, 3
    ns = torch.ops.na_cuda
    x = torch.empty(N, T, C, dtype=dtype, device="meta")
    s = torch.empty(N, T, W, dtype=torch.float32, device="meta")
    for name in ("qk_forward", "attn_backward"):
        out = getattr(ns, "%s_ana_%s" % (prefix, name))(x, x, N, T, C, W, L)
        assert out.shape == (N, T, W) and out.dtype == torch.float32
    for name, a, b in (("q_backward", s, x), ("k_backward", s, x), ("av_forward", s, x), ("v_backward", s, x)):
        out = getattr(ns, "%s_ana_%s" % (prefix, name))(a, b, N, T, C, W, L)
        assert out.shape == (N, T, C) and out.dtype == dtype
    with pytest.raises(Exception):
        getattr(ns, prefix + "_ana_qk_forward")(x.float(), x.float(), N, T, C, W, L)     # wrong dtype
    with pytest.raises(Exception):
        getattr(ns, prefix + "_ana_av_forward")(s, x, N, T, C, W + 1, L)                 # score tensor of another window
    o, lse = ns.na1d_fused_forward(x, x, x, None, None, 1, W, L, 1.0)
    assert o.shape == (N, T, C) and lse.shape == (N, T) and lse.dtype == torch.float32
    o, lse = ns.global_attention_forward(x, x, x, None, 1, 1.0)
    assert o.shape == (N, T, C) and o.dtype == dtype and lse.shape == (N, T) and lse.dtype == torch.float32
    assert all(g.shape == (N, T, C) for g in ns.global_attention_backward(x, x, x, x, x, lse, None, 1, 1.0))


def test_wrappers_pick_the_op_by_dtype():
    x = torch.empty(2, 8, 16, dtype=torch.float16, device="meta")
    assert ops.ana_qk(x, x, 5, 2).shape == (2, 8, 5)
    assert ops.ana_av(torch.empty(2, 8, 5, device="meta"), x, 5, 2).dtype == torch.float16
    with pytest.raises(AssertionError):
        ops.ana_qk(x.float(), x.float(), 5, 2)
