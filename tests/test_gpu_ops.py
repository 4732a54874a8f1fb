"""The torch.library ops on the GPU: equal to the drop-in Functions, differentiable, and traceable by
torch.compile (aot_eager backend: dynamo + AOT autograd over fake tensors, no code generation)."""
import pytest
import torch

from oracle import na1d_oracle as O
from na1d_amd import nattn, na1d_fused, ops
from _util import TOL, dev, make_inputs

pytestmark = pytest.mark.gpu
DTYPES = [torch.bfloat16, torch.float16]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_ops_equal_the_dropin_functions_and_differentiate(dtype):
    B, T, C, W, L = 6, 70, 16, 27, 13
    q, k, v, do = dev(*make_inputs(B, T, C, W, 3, dtype, n=4, scale=C ** -0.5))
    QK, AV = nattn.getNA1dFunction(C=C, dilation=1, dtype=dtype)

    def chain(qk, av, q, k, v):
        return av(torch.softmax(qk(q, k), dim=-1), v)

    a = [t.clone().requires_grad_(True) for t in (q, k, v)]
    b = [t.clone().requires_grad_(True) for t in (q, k, v)]
    out_a = chain(lambda x, y: QK.apply(x, y, W, L, 1), lambda s, x: AV.apply(s, x, W, L, 1), *a)
    out_b = chain(lambda x, y: ops.ana_qk(x, y, W, L), lambda s, x: ops.ana_av(s, x, W, L), *b)
    out_a.backward(do)
    out_b.backward(do)
    assert torch.equal(out_a, out_b)
    for x, y in zip(a, b):
        assert torch.equal(x.grad, y.grad)


def test_opcheck_on_one_op_of_each_kind():
    x = torch.randn(2, 20, 16, device="cuda").to(torch.bfloat16)
    s = torch.randn(2, 20, 7, device="cuda")
    tests = ("test_schema", "test_faketensor")
    torch.library.opcheck(torch.ops.na_cuda.bf16_ana_qk_forward.default, (x, x, 2, 20, 16, 7, 3), test_utils=tests)
    torch.library.opcheck(torch.ops.na_cuda.bf16_ana_v_backward.default, (s, x, 2, 20, 16, 7, 3), test_utils=tests)
    torch.library.opcheck(torch.ops.na_cuda.na1d_fused_forward.default, (x, x, x, None, None, 1, 7, 3, 1.0),
                          test_utils=tests)


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_compiled_function_through_the_ops_matches_eager_and_the_oracle(dtype):
    N, H, T, C, W, L = 2, 4, 60, 16, 27, 13
    q, k, v, do = make_inputs(N * H, T, C, W, 8, dtype, n=4, scale=C ** -0.5)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(2)) * 0.3
    pad = torch.tensor([0, 9])
    tv = (T - pad).to(torch.int32).cuda()

    def layer(q, k, v, rpb):
        unfused = ops.ana_av(torch.softmax(ops.ana_qk(q, k, W, L), dim=-1), v, W, L)
        fused = ops.na1d_fused_op(q, k, v, W, L, rpb=rpb, t_valid=tv, num_heads=H)
        return unfused, fused

    compiled = torch.compile(layer, backend="aot_eager", fullgraph=True)
    ins_e = [t.cuda().requires_grad_(True) for t in (q, k, v, rpb)]
    ins_c = [t.cuda().requires_grad_(True) for t in (q, k, v, rpb)]
    ue, fe = layer(*ins_e)
    uc, fc = compiled(*ins_c)
    (ue.float().sum() + (fe * do.cuda()).float().sum()).backward()
    (uc.float().sum() + (fc * do.cuda()).float().sum()).backward()
    assert torch.equal(ue, uc) and torch.equal(fe, fc)
    for x, y in zip(ins_e[:3], ins_c[:3]):
        assert torch.equal(x.grad, y.grad)
    assert torch.allclose(ins_e[3].grad, ins_c[3].grad, rtol=1e-4, atol=1e-5)      # float atomics: order varies

    want, _, _ = O.na1d_forward(q.float(), k.float(), v.float(), W, L, rpb, pad, H)
    assert O.rel_l2(fc.float(), want) < TOL[dtype]
    ref = na1d_fused(ins_e[0].detach(), ins_e[1].detach(), ins_e[2].detach(), W, L, rpb=rpb.cuda(), t_valid=tv, num_heads=H)
    assert torch.equal(fc, ref)


def test_dense_attention_op_compiles_and_equals_the_eager_operator():
    from na1d_amd.dense import global_attention
    N, H, T, C, dtype = 2, 2, 70, 32, torch.bfloat16
    q, k, v, do = make_inputs(N * H, T, C, 0, 21, dtype, n=4)
    pad = torch.tensor([0, 30])
    tv = (T - pad).to(torch.int32).cuda()
    fn = lambda q, k, v: ops.global_attention_op(q, k, v, H, tv, C ** -0.5)
    compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
    ins_c = [t.cuda().requires_grad_(True) for t in (q, k, v)]
    ins_e = [t.cuda().requires_grad_(True) for t in (q, k, v)]
    oc = compiled(*ins_c)
    oc.backward(do.cuda())
    oe = global_attention(*ins_e, H, tv, C ** -0.5)
    oe.backward(do.cuda())
    assert torch.equal(oc, oe)
    for x, y in zip(ins_c, ins_e):
        assert torch.equal(x.grad, y.grad)
    want, _, _ = O.global_forward(q.float(), k.float(), v.float(), C ** -0.5, pad, H)
    assert O.rel_l2(oc.float(), want) < TOL[dtype]
    x = q.cuda()
    torch.library.opcheck(torch.ops.na_cuda.global_attention_forward.default, (x, x, x, tv, H, 0.2),
                          test_utils=["test_schema", "test_faketensor"])


def test_ops_compile_with_the_inductor_backend():
    """The reference trains under torch.compile (configs/pcf_nat4x4.yaml:28, train_main.py:168-170): the default
    backend lowers the surrounding torch ops itself and may hand the ops tensors with other strides than eager did,
    which they pack.  Compiled and eager results agree to rounding, gradients included."""
    N, H, T, C, W, L, dtype = 2, 4, 60, 16, 27, 13, torch.bfloat16
    q, k, v, do = make_inputs(N * H, T, C, W, 17, dtype, n=4)
    rpb = torch.randn(H, W, generator=torch.Generator().manual_seed(3)) * 0.3

    def layer(q, k, v, rpb):
        attn = torch.softmax(ops.ana_qk(q * 0.25, k, W, L) + rpb.repeat(N, 1).unsqueeze(1), dim=-1)
        return (ops.ana_av(attn, v, W, L) + ops.na1d_fused_op(q, k, v, W, L, rpb=rpb, num_heads=H, scale=0.25)
                + ops.global_attention_op(q, k, v, H, None, 0.25))

    compiled = torch.compile(layer, backend="inductor", fullgraph=True)
    ins_e = [t.cuda().requires_grad_(True) for t in (q, k, v, rpb)]
    ins_c = [t.cuda().requires_grad_(True) for t in (q, k, v, rpb)]
    oe, oc = layer(*ins_e), compiled(*ins_c)
    (oe * do.cuda()).float().sum().backward()
    (oc * do.cuda()).float().sum().backward()
    assert O.rel_l2(oc.float(), oe.float()) < TOL[dtype]
    for x, y in zip(ins_c, ins_e):
        assert O.rel_l2(x.grad.float(), y.grad.float()) < 2 * TOL[dtype]
    # a transposed view straight into an op: packed inside, same result
    qt = ins_e[0].detach().transpose(0, 1).contiguous().transpose(0, 1)
    assert not qt.is_contiguous()
    assert torch.equal(ops.ana_qk(qt.contiguous(), ins_e[1].detach(), W, L),
                       torch.ops.na_cuda.bf16_ana_qk_forward(qt, ins_e[1].detach(), N * H, T, C, W, L))
