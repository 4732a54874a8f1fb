"""CPU-side checks of the C-ABI library: it loads, exports every symbol the
header declares, and validates arguments before touching the GPU."""
import ctypes
import os
import re

import pytest
import torch

from na1d_amd import _lib, nattn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "na1d.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(na1d_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), name
    assert set(_lib.SYMBOLS) <= set(names)
    assert lib.na1d_version() >= 100


def test_status_strings():
    lib = _lib.load()
    assert lib.na1d_status_string(0) == b"ok"
    for code in range(-11, 0):
        assert len(lib.na1d_status_string(code)) > 3 and lib.na1d_status_string(code) != b"unknown status"
    assert lib.na1d_status_string(-99) == b"unknown status"


def _call(lib, name, o, a, b, B, T, C, W, left, dtype):
    P = ctypes.c_void_p
    return getattr(lib, name)(P(o), P(a), P(b), B, T, C, W, left, dtype, None)


@pytest.mark.parametrize("name", ["na1d_qk_forward", "na1d_av_forward", "na1d_q_backward",
                                  "na1d_k_backward", "na1d_a_backward", "na1d_v_backward"])
def test_argument_validation_happens_before_any_launch(name):
    """Bad arguments come back as status codes (the reference has no checks at
    all: bad shapes are silent out-of-bounds there).  0x1000 is a fake aligned
    address: validation must reject before it is ever dereferenced."""
    lib = _lib.load()
    ok = 0x1000
    assert _call(lib, name, ok, ok, ok, 2, 8, 12, 5, 2, 0) == -3      # C % 8
    assert _call(lib, name, ok, ok, ok, 2, 8, 0, 5, 2, 0) == -3
    assert _call(lib, name, ok, ok, ok, 2, 8, 16, 81, 2, 0) == -4     # W > 80
    assert _call(lib, name, ok, ok, ok, 2, 8, 16, 0, 0, 0) == -4
    assert _call(lib, name, ok, ok, ok, 2, 8, 16, 5, 5, 0) == -4      # left >= W
    assert _call(lib, name, ok, ok, ok, 2, 8, 16, 5, -1, 0) == -4
    assert _call(lib, name, ok, ok, ok, 2, 8, 16, 5, 2, 7) == -2      # dtype
    assert _call(lib, name, ok, ok, ok, -1, 8, 16, 5, 2, 0) == -5
    assert _call(lib, name, ok, ok, ok, 1 << 40, 1 << 40, 16, 5, 2, 0) == -5   # overflow
    assert _call(lib, name, None, ok, ok, 2, 8, 16, 5, 2, 0) == -1
    assert _call(lib, name, ok, None, ok, 2, 8, 16, 5, 2, 0) == -1
    assert _call(lib, name, ok, ok, ok + 2, 2, 8, 16, 5, 2, 0) == -6   # alignment
    # empty problems are a no-op, even with null pointers
    assert _call(lib, name, None, None, None, 0, 8, 16, 5, 2, 0) == 0
    assert _call(lib, name, None, None, None, 2, 0, 16, 5, 2, 1) == 0


def test_fused_entry_points_validate():
    lib = _lib.load()
    P = ctypes.c_void_p
    ok = P(0x1000)
    f = lib.na1d_fused_forward
    assert f(ok, None, ok, ok, ok, None, None, 4, 3, 8, 16, 5, 2, 1.0, 0, None) == -5   # B % H
    assert f(ok, None, ok, ok, None, None, None, 4, 2, 8, 16, 5, 2, 1.0, 0, None) == -1  # v missing
    assert f(ok, None, ok, ok, ok, None, None, 4, 2, 8, 20, 5, 2, 1.0, 0, None) == -3
    assert f(None, None, None, None, None, None, None, 0, 1, 8, 16, 5, 2, 1.0, 0, None) == 0
    b = lib.na1d_fused_backward
    assert b(ok, ok, ok, None, ok, ok, ok, ok, ok, None, None, None, 4, 2, 8, 16, 5, 2, 1.0, 0, None, 0, None) == -1  # lse
    assert b(ok, ok, ok, None, ok, ok, ok, ok, ok, ok, None, None, 4, 2, 8, 16, 90, 2, 1.0, 0, None, 0, None) == -4
    assert b(ok, ok, ok, None, ok, ok, ok, ok, ok, ok, None, None, 4, 2, 8, 16, 5, 2, 1.0, 0, P(0x1008), 64, None) == -6
    # scale has to be a finite number above zero (the reference's is head_dim ** -0.5)
    for bad in (0.0, -0.25, float("nan"), float("inf")):
        assert f(ok, None, ok, ok, ok, None, None, 4, 2, 8, 16, 5, 2, bad, 0, None) == -11
        assert b(ok, ok, ok, None, ok, ok, ok, ok, ok, ok, None, None, 4, 2, 8, 16, 5, 2, bad, 0, None, 0, None) == -11
    # a workspace that is passed but too small is refused before anything is launched (d rpb asked for)
    assert b(ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, None, None, 4, 2, 8, 16, 5, 2, 1.0, 0, ok, 64, None) == -10
    w = lib.na1d_fused_backward_workspace_bytes
    assert w(4096, 16, 100, 16, 27, 13, 0) == 4096 * 32 * 4      # one 32-float row per work item
    assert w(1024, 8, 300, 32, 15, 7, 1) > 0
    assert w(4, 2, 8, 136, 5, 2, 0) == 0                         # generic kernel: no workspace
    assert w(64, 2, 300, 32, 65, 32, 0) > 0 and w(64, 2, 300, 32, 65, 32, 0) % (80 * 4) == 0   # wide windows: rows of 80 floats
    assert w(4, 3, 8, 16, 5, 2, 0) == -5 and w(4, 2, 8, 16, 99, 2, 0) == -4


def test_noalloc_entry_point_validates_and_respects_the_kernel_family_switch():
    """na1d_fused_backward_noalloc checks its arguments like na1d_fused_backward and, while the generic kernels are
    forced, reports that it has no kernel (they have no fixed-order reduction)."""
    lib = _lib.load()
    ok = ctypes.c_void_p(0x1000)
    f = lib.na1d_fused_backward_noalloc
    args = lambda **kw: [ok, ok, ok, None, ok, ok, ok, ok, ok, kw.get("lse", ok), None, None, kw.get("B", 4), 2, 8,
                         kw.get("C", 16), kw.get("W", 5), 2, kw.get("scale", 1.0), 0, None]
    assert f(*args(lse=None)) == -1 and f(*args(C=20)) == -3 and f(*args(W=99)) == -4 and f(*args(scale=0.0)) == -11
    assert f(*args(B=0)) == 0                        # nothing to do
    assert f(*args(C=136)) == -8                     # head_dim above 128: the generic kernels have no fixed-order reduction
    assert f(*args(B=1 << 20)) == -9                 # more workgroups than the static scratch holds rows for
    was = lib.na1d_force_generic(1)
    try:
        assert f(*args()) == -8
    finally:
        lib.na1d_force_generic(was)


def test_deterministic_workspace_covers_every_residue_class():
    """With dilation d the backward runs once per residue class t mod d, on ceil(T/d) or floor(T/d) rows, all with one
    workspace.  The split into workgroups is not monotonic in the length (64 sequences: 129 rows need 24576 bytes,
    128 rows 32768), so the workspace has to be sized over every class, not for the longest."""
    from na1d_amd import fused
    w = lambda B, T: _lib.fused_backward_workspace_bytes(B, 4, T, 16, 27, 13, torch.bfloat16)
    assert w(64, 129) < w(64, 128)                   # the case in point
    assert fused._deterministic_workspace_bytes(64, 4, 257, 16, 27, 13, 2, torch.bfloat16) == w(64, 128)
    for B in (4, 64, 256, 4096):
        for T in (1, 2, 3, 31, 100, 129, 257, 300, 1000):
            for d in (1, 2, 3, 4, 7):
                need = max(w(B, -(-(T - r) // d)) for r in range(min(d, T)))
                assert fused._deterministic_workspace_bytes(B, 4, T, 16, 27, 13, d, torch.bfloat16) == need, (B, T, d)


def test_strided_entry_points_validate():
    lib = _lib.load()
    P, ok = ctypes.c_void_p, ctypes.c_void_p(0x1000)
    S = lambda *v: (ctypes.c_int64 * 3)(*v)
    qkv, out = S(8 * 3 * 2 * 16, 16, 3 * 2 * 16), S(8 * 2 * 16, 16, 2 * 16)     # [N, T, 3, H, C] / [N, T, H*C], T=8, H=2, C=16
    f = lib.na1d_fused_forward_strided
    args = lambda **kw: [kw.get("o", ok), None, ok, ok, kw.get("v", ok), None, None, kw.get("N", 2), 2, 8, kw.get("C", 16),
                         kw.get("W", 5), 2, 1.0, 0, kw.get("qs", qkv), kw.get("os", out), None]
    assert f(*args(qs=None)) == -1 and f(*args(os=None)) == -1 and f(*args(v=None)) == -1
    assert f(*args(qs=S(768, 16, 8))) == -5          # rows closer than C
    assert f(*args(qs=S(768, 12, 96))) == -6         # head stride not a multiple of 8 elements
    assert f(*args(os=S(-256, 16, 32))) == -5
    assert f(*args(C=20)) == -3 and f(*args(W=99)) == -4 and f(*args(N=-1)) == -5
    assert f(*args(N=0)) == 0                        # nothing to do
    assert f(*args(C=136, qs=S(8 * 3 * 2 * 136, 136, 3 * 2 * 136), os=S(8 * 2 * 136, 136, 272))) == -8   # no strided kernel above 128
    b = lib.na1d_fused_backward_strided
    bargs = lambda **kw: [ok, ok, ok, None, ok, ok, ok, kw.get("g", ok), kw.get("lse", ok), None, None, 2, 2, 8, 16, 5, 2,
                          1.0, 0, kw.get("qs", qkv), out, kw.get("ws", None), 64, None]
    assert b(*bargs(lse=None)) == -1 and b(*bargs(g=None)) == -1 and b(*bargs(qs=None)) == -1
    assert b(*bargs(ws=P(0x1008))) == -6


def test_dropout_entry_points_validate():
    lib = _lib.load()
    ok = ctypes.c_void_p(0x1000)
    f = lib.na1d_fused_forward_dropout
    args = lambda **kw: [ok, None, ok, ok, kw.get("v", ok), None, None, kw.get("B", 4), 2, 8, kw.get("C", 16), 5, 2, 1.0, 0,
                         kw.get("p", 0.5), 7, None]
    assert f(*args(v=None)) == -1 and f(*args(C=20)) == -3 and f(*args(B=0)) == 0
    assert f(*args(p=1.0)) == -5 and f(*args(p=-0.1)) == -5 and f(*args(p=float("nan"))) == -5
    b = lib.na1d_fused_backward_dropout
    bargs = lambda **kw: [ok, ok, ok, None, ok, ok, ok, ok, ok, kw.get("lse", ok), None, None, 4, 2, 8, 16, 5, 2, 1.0, 0,
                          kw.get("p", 0.5), 7, None, 0, None]
    assert b(*bargs(lse=None)) == -1 and b(*bargs(p=1.5)) == -5


def test_strided_dropout_entry_points_validate():
    lib = _lib.load()
    ok = ctypes.c_void_p(0x1000)
    S = lambda *v: (ctypes.c_int64 * 3)(*v)
    qkv, out = S(8 * 3 * 2 * 16, 16, 3 * 2 * 16), S(8 * 2 * 16, 16, 2 * 16)     # [N, T, 3, H, C] / [N, T, H*C], T=8, H=2, C=16
    f = lib.na1d_fused_forward_strided_dropout
    args = lambda **kw: [ok, None, ok, ok, kw.get("v", ok), None, None, kw.get("N", 2), 2, 8, kw.get("C", 16), 5, 2, 1.0, 0,
                         kw.get("qs", qkv), out, kw.get("p", 0.5), 7, kw.get("stride", 2), kw.get("offset", 1),
                         kw.get("rows", 16), None]
    assert f(*args(v=None)) == -1 and f(*args(qs=None)) == -1 and f(*args(C=20)) == -3
    assert f(*args(p=1.0)) == -5 and f(*args(p=float("nan"))) == -5
    assert f(*args(stride=0)) == -5 and f(*args(offset=2)) == -5 and f(*args(offset=-1)) == -5
    assert f(*args(rows=15)) == -5                   # row 1 + 2 * 7 = 15 needs 16 rows
    assert f(*args(rows=1 << 31)) == -5
    assert f(*args(N=0)) == 0                        # nothing to do
    assert f(*args(C=136, qs=S(8 * 3 * 2 * 136, 136, 3 * 2 * 136))) in (-5, -8)
    b = lib.na1d_fused_backward_strided_dropout
    bargs = lambda **kw: [ok, ok, ok, None, ok, ok, ok, kw.get("g", ok), kw.get("lse", ok), None, None, 2, 2, 8, 16, 5, 2,
                          1.0, 0, qkv, out, kw.get("p", 0.5), 7, kw.get("stride", 2), 1, kw.get("rows", 16),
                          kw.get("ws", None), 64, None]
    assert b(*bargs(lse=None)) == -1 and b(*bargs(g=None)) == -1 and b(*bargs(p=1.5)) == -5
    assert b(*bargs(stride=0)) == -5 and b(*bargs(rows=15)) == -5
    assert b(*bargs(ws=ctypes.c_void_p(0x1008))) == -6


def test_dense_attention_entry_points_validate():
    lib = _lib.load()
    P, ok = ctypes.c_void_p, ctypes.c_void_p(0x1000)
    f = lib.na1d_global_forward
    args = lambda **kw: [kw.get("o", ok), None, ok, ok, kw.get("v", ok), None, kw.get("B", 4), kw.get("H", 2), 8,
                         kw.get("C", 16), 1.0, kw.get("dtype", 0), kw.get("p", 0.0), 3, None]
    assert f(*args(o=None)) == -1 and f(*args(v=None)) == -1 and f(*args(p=1.0)) == -5
    assert f(*args(v=P(0x1004))) == -6
    assert f(*args(C=20)) == -3 and f(*args(dtype=7)) == -2 and f(*args(B=3)) == -5
    assert f(*args(B=0)) == 0                        # nothing to do
    assert f(*args(C=136)) == -8                     # no dense kernel above 128
    b = lib.na1d_global_backward
    bargs = lambda **kw: [ok, ok, ok, ok, ok, ok, kw.get("out", ok), ok, kw.get("lse", ok), None, 4, 2, 8, 16, 1.0, 0,
                          0.25, 3, kw.get("ws", ok), kw.get("wsb", 4 * 8 * 4), None]
    assert b(*bargs(out=None)) == -1 and b(*bargs(lse=None)) == -1 and b(*bargs(ws=None)) == -1
    assert b(*bargs(ws=P(0x1008))) == -6
    assert b(*bargs(wsb=4 * 8 * 4 - 1)) == -5        # one fp32 per row is required
    assert lib.na1d_global_backward_workspace_bytes(4, 2, 8, 16, 0) == 4 * 8 * 4
    assert lib.na1d_global_backward_workspace_bytes(4, 2, 8, 12, 0) == -3


def test_python_layer_mirrors_reference_entry_points():
    """Names, dispatch and asserts of na1d_tensorcore/nattn.py:128-137."""
    qk, av = nattn.getNA1dFunction(C=16, dilation=1, dtype=torch.bfloat16)
    assert (qk.__name__, av.__name__) == ("bf16_ANA1d_QK_Function", "bf16_ANA1d_AV_Function")
    qk, av = nattn.getNA1dFunction(C=32, dilation=1, dtype=torch.float16)
    assert (qk.__name__, av.__name__) == ("fp16_ANA1d_QK_Function", "fp16_ANA1d_AV_Function")
    assert issubclass(qk, torch.autograd.Function) and issubclass(av, torch.autograd.Function)
    with pytest.raises(AssertionError):
        nattn.getNA1dFunction(C=12, dilation=1, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        nattn.getNA1dFunction(C=16, dilation=2, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        nattn.getNA1dFunction(C=16, dilation=1, dtype=torch.float32)
    import na1d_tensorcore.nattn as shim      # the import path the reference models use
    assert shim.getNA1dFunction is nattn.getNA1dFunction


def test_no_cpu_fallback():
    """CPU tensors are refused loudly; nothing routes through the oracle."""
    qk, _ = nattn.getNA1dFunction(C=8, dilation=1, dtype=torch.bfloat16)
    q = torch.zeros(1, 4, 8, dtype=torch.bfloat16)
    with pytest.raises(Exception):
        qk.apply(q, q, 3, 1, 1)
    src = open(os.path.join(ROOT, "pcf-nat_amd", "na1d_amd", "_lib.py")).read()
    for mod in ("nattn.py", "fused.py", "_lib.py", "__init__.py"):
        text = open(os.path.join(ROOT, "pcf-nat_amd", "na1d_amd", mod)).read()
        assert "oracle" not in text.replace("no CPU path", "")
    assert "CDLL" in src
