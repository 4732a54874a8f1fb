"""The entry point that allocates nothing: na1d_fused_backward_noalloc keeps the d rpb partial sums in the
library's static per-GPU scratch array instead of a caller's workspace.  It must give the bits of
na1d_fused_backward with a workspace, also on a second call with a smaller input (the array keeps the first
call's contents)."""
import ctypes

import pytest
import torch

from na1d_amd import _lib
from _util import make_inputs

pytestmark = pytest.mark.gpu

P = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())


def _free_bytes():
    """Free device memory as the HIP runtime reports it: a hipMalloc inside the library would show here, which
    torch's allocator statistics cannot see."""
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _backward_both_ways(N, H, T, C, W, L, dtype, seed, pad=None, first_on_device=False):
    lib = _lib.load()
    B = N * H
    q, k, v, do = (t.cuda() for t in make_inputs(B, T, C, W, seed, dtype, n=4, scale=C ** -0.5))
    rpb = (torch.randn(H, W, generator=torch.Generator().manual_seed(seed)) * 0.3).cuda()
    tv = None if pad is None else (T - torch.tensor(pad, dtype=torch.int32)).cuda()
    out, lse = torch.empty_like(q), torch.empty(B, T, device="cuda")
    _lib.call_fused_forward(out, lse, q, k, v, rpb, tv, B, H, T, C, W, L, 1.0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tag = _lib.dtype_tag(dtype)
    nbytes = _lib.fused_backward_workspace_bytes(B, H, T, C, W, L, dtype)
    assert 0 < nbytes <= 4 * 1024 * 1024
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    want = [torch.empty_like(q) for _ in range(3)] + [torch.zeros(H, W, device="cuda")]
    got = [torch.full_like(q, float("nan")) for _ in range(3)] + [torch.zeros(H, W, device="cuda")]
    st = lib.na1d_fused_backward(P(want[0]), P(want[1]), P(want[2]), P(want[3]), P(q), P(k), P(v), P(out), P(do), P(lse),
                                 P(rpb), P(tv), B, H, T, C, W, L, 1.0, tag, P(ws), nbytes, stream)
    _lib.check(st, "na1d_fused_backward")
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.memory_allocated()
    free_before = _free_bytes()
    st = lib.na1d_fused_backward_noalloc(P(got[0]), P(got[1]), P(got[2]), P(got[3]), P(q), P(k), P(v), P(out), P(do),
                                         P(lse), P(rpb), P(tv), B, H, T, C, W, L, 1.0, tag, stream)
    _lib.check(st, "na1d_fused_backward_noalloc")
    torch.cuda.synchronize()
    assert before == (torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.memory_allocated())
    if not first_on_device:       # the very first call may make the runtime load the code object's data
        assert _free_bytes() == free_before
    for name, a, b in zip(("dq", "dk", "dv", "drpb"), got, want):
        assert torch.equal(a, b), name
    assert want[3].abs().max() > 0


def test_no_alloc_backward_matches_the_workspace_backward_twice():
    """Two calls in a row on the same GPU, the second with a smaller input: the scratch array still holds the
    first call's partial sums and the second call must not read them."""
    _backward_both_ways(64, 8, 300, 32, 15, 7, torch.float16, seed=1, first_on_device=True)
    _backward_both_ways(3, 4, 90, 16, 27, 13, torch.bfloat16, seed=2, pad=[0, 30, 90])
    _backward_both_ways(5, 2, 40, 48, 9, 4, torch.float16, seed=3)          # head_dim run at the next kernel width
    _backward_both_ways(6, 4, 150, 32, 65, 32, torch.bfloat16, seed=4, pad=[0, 0, 20, 150, 3, 77])   # wide window


def test_no_alloc_backward_replays_from_a_captured_graph():
    """The use the entry point is for: after one call outside the capture (which looks the scratch array's address
    up), the call is captured and replayed on changing inputs; every replay gives the bits of the workspace path."""
    lib = _lib.load()
    N, H, T, C, W, L, dtype = 8, 4, 100, 16, 27, 13, torch.bfloat16
    B = N * H
    gen = torch.Generator(device="cuda").manual_seed(9)
    new = lambda *shape: torch.randn(*shape, device="cuda", generator=gen)
    q, k, v, do = (new(B, T, C).to(dtype) for _ in range(4))
    rpb = new(H, W) * 0.3
    out, lse = torch.empty_like(q), torch.empty(B, T, device="cuda")
    got = [torch.empty_like(q) for _ in range(3)] + [torch.zeros(H, W, device="cuda")]
    want = [torch.empty_like(q) for _ in range(3)] + [torch.zeros(H, W, device="cuda")]
    tag = _lib.dtype_tag(dtype)
    nbytes = _lib.fused_backward_workspace_bytes(B, H, T, C, W, L, dtype)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")

    def call_noalloc():
        got[3].zero_()                                 # a fill kernel, not a memset node
        _lib.call_fused_forward(out, lse, q, k, v, rpb, None, B, H, T, C, W, L, 1.0)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        st = lib.na1d_fused_backward_noalloc(P(got[0]), P(got[1]), P(got[2]), P(got[3]), P(q), P(k), P(v), P(out), P(do),
                                             P(lse), P(rpb), None, B, H, T, C, W, L, 1.0, tag, stream)
        _lib.check(st, "na1d_fused_backward_noalloc")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call_noalloc()                                 # outside the capture: resolves the scratch array's address
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call_noalloc()
    for rep in range(3):
        for t in (q, k, v, do):
            t.copy_(new(B, T, C).to(dtype))            # eager work between the replays
        graph.replay()
        torch.cuda.synchronize()
        want[3].zero_()
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        st = lib.na1d_fused_backward(P(want[0]), P(want[1]), P(want[2]), P(want[3]), P(q), P(k), P(v), P(out), P(do),
                                     P(lse), P(rpb), None, B, H, T, C, W, L, 1.0, tag, P(ws), nbytes, stream)
        _lib.check(st, "na1d_fused_backward")
        torch.cuda.synchronize()
        for name, a, b in zip(("dq", "dk", "dv", "drpb"), got, want):
            assert torch.equal(a, b), (rep, name)


def test_no_alloc_backward_limits():
    lib = _lib.load()
    ok = ctypes.c_void_p(0x1000)
    f = lib.na1d_fused_backward_noalloc
    # more workgroups than the scratch array has rows for: refused before anything is launched
    assert f(ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, None, 1 << 16, 1, 16, 16, 27, 13, 1.0, 0, None) == -9
    assert b"scratch" in lib.na1d_status_string(-9)
    # a head_dim the workspace path does not cover
    assert f(ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, None, 4, 1, 64, 136, 27, 13, 1.0, 0, None) == -8
    assert f(ok, ok, ok, ok, ok, ok, ok, ok, ok, None, ok, None, 4, 1, 64, 16, 27, 13, 1.0, 0, None) == -1
