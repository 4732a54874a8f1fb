"""Pins for the CPU oracle: every check here is chosen so that a plausible
mistake in oracle/na1d_oracle.py (dropped term, wrong sign, shifted or clamped
window, transposed operand) fails it.  None of them re-types the oracle's
formula; they use brute-force index loops, library routines on special cases,
closed forms and algebraic identities."""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import na1d_oracle as O

torch.manual_seed(0)
F64 = torch.float64

GEOMS = [  # (T, W, left)
    (9, 5, 2), (9, 4, 1), (9, 4, 2), (7, 1, 0), (3, 7, 3), (2, 5, 0), (5, 5, 4), (1, 3, 1), (6, 11, 5),
]


def _rand(*shape):
    return torch.randn(*shape, dtype=F64)


# ---------------------------------------------------------------- brute force
def _brute_p1(q, k, W, L, d=1):
    B, T, C = q.shape
    s = torch.zeros(B, T, W, dtype=q.dtype)
    for b, t, j in itertools.product(range(B), range(T), range(W)):
        u = t + (j - L) * d
        if 0 <= u < T:
            s[b, t, j] = sum(q[b, t, c] * k[b, u, c] for c in range(C))
    return s


def _brute_p2(p, v, W, L, d=1):
    B, T, C = v.shape
    o = torch.zeros(B, T, C, dtype=v.dtype)
    for b, t, j in itertools.product(range(B), range(T), range(W)):
        u = t + (j - L) * d
        if 0 <= u < T:
            o[b, t] += p[b, t, j] * v[b, u]
    return o


def _brute_p3(s, x, W, L, d=1):
    """Gather form, as the reference kernel indexes it (.cu:457-459)."""
    B, T, C = x.shape
    o = torch.zeros(B, T, C, dtype=x.dtype)
    for b, u, j in itertools.product(range(B), range(T), range(W)):
        t = u - (j - L) * d
        if 0 <= t < T:
            o[b, u] += s[b, t, j] * x[b, t]
    return o


@pytest.mark.parametrize("T,W,L", GEOMS)
def test_primitives_match_brute_force(T, W, L):
    q, k, v = _rand(2, T, 8), _rand(2, T, 8), _rand(2, T, 8)
    s = _rand(2, T, W)
    assert torch.allclose(O.qk_band(q, k, W, L), _brute_p1(q, k, W, L), atol=1e-12)
    assert torch.allclose(O.av_band(s, v, W, L), _brute_p2(s, v, W, L), atol=1e-12)
    assert torch.allclose(O.inverse_gather(s, q, W, L), _brute_p3(s, q, W, L), atol=1e-12)


@pytest.mark.parametrize("d", [2, 3])
def test_dilated_primitives_match_brute_force(d):
    T, W, L = 11, 5, 2
    q, k, v, s = _rand(1, T, 8), _rand(1, T, 8), _rand(1, T, 8), _rand(1, T, W)
    assert torch.allclose(O.qk_band(q, k, W, L, d), _brute_p1(q, k, W, L, d), atol=1e-12)
    assert torch.allclose(O.av_band(s, v, W, L, d), _brute_p2(s, v, W, L, d), atol=1e-12)
    assert torch.allclose(O.inverse_gather(s, q, W, L, d), _brute_p3(s, q, W, L, d), atol=1e-12)


# ---------------------------------------------------------------- special cases → library routines
def test_p1_w1_is_rowwise_dot():
    q, k = _rand(3, 10, 16), _rand(3, 10, 16)
    assert torch.allclose(O.qk_band(q, k, 1, 0)[..., 0], (q * k).sum(-1), atol=1e-12)


def test_p1_full_window_contains_dense_matmul():
    """L=T-1, W=2T-1: S[t, u-t+L] = (q @ k^T)[t,u] for every (t,u); the rest is 0."""
    T = 6
    q, k = _rand(2, T, 8), _rand(2, T, 8)
    L, W = T - 1, 2 * T - 1
    s = O.qk_band(q, k, W, L)
    dense = q @ k.transpose(1, 2)
    seen = torch.zeros_like(s, dtype=torch.bool)
    for t in range(T):
        for u in range(T):
            assert torch.allclose(s[:, t, u - t + L], dense[:, t, u], atol=1e-12)
            seen[:, t, u - t + L] = True
    assert (s[~seen] == 0).all()


def test_p1_k_ones_counts_zero_fill_not_clamping():
    """k = 1: S[t,j] = sum_c q[t,c] where the key exists and exactly 0 elsewhere;
    a clamped or shifted (NATTEN-style) window would give non-zero edge slots."""
    T, W, L = 8, 5, 2
    q = _rand(1, T, 8)
    s = O.qk_band(q, torch.ones(1, T, 8, dtype=F64), W, L)
    for t in range(T):
        for j in range(W):
            inside = 0 <= t - L + j < T
            want = q[0, t].sum() if inside else torch.tensor(0.0, dtype=F64)
            assert torch.allclose(s[0, t, j], want, atol=1e-12)
    assert (s[0, 0, :L] == 0).all() and (s[0, T - 1, L + 1:] == 0).all()


def test_p2_one_hot_is_exact_shift():
    T, W, L, C = 9, 5, 2, 8
    v = _rand(2, T, C)
    for j0 in range(W):
        p = torch.zeros(2, T, W, dtype=F64)
        p[:, :, j0] = 1
        o = O.av_band(p, v, W, L)
        for t in range(T):
            u = t - L + j0
            want = v[:, u] if 0 <= u < T else torch.zeros(2, C, dtype=F64)
            assert torch.equal(o[:, t], want)


def test_p2_uniform_probabilities_do_not_renormalise():
    T, W, L, C = 10, 7, 3, 8
    o = O.av_band(torch.full((1, T, W), 1.0 / W, dtype=F64), torch.full((1, T, C), 2.5, dtype=F64), W, L)
    for t in range(T):
        n_valid = sum(0 <= t - L + j < T for j in range(W))
        assert torch.allclose(o[0, t], torch.full((C,), 2.5 * n_valid / W, dtype=F64), atol=1e-12)


# ---------------------------------------------------------------- adjoint identities
@pytest.mark.parametrize("T,W,L", GEOMS)
def test_adjoint_identities(T, W, L):
    q, k, v = _rand(2, T, 8), _rand(2, T, 8), _rand(2, T, 8)
    G, P, GO = _rand(2, T, W), _rand(2, T, W), _rand(2, T, 8)
    a = (O.qk_band(q, k, W, L) * G).sum()
    assert torch.allclose(a, (q * O.av_band(G, k, W, L)).sum(), atol=1e-10)
    assert torch.allclose(a, (k * O.inverse_gather(G, q, W, L)).sum(), atol=1e-10)
    b = (O.av_band(P, v, W, L) * GO).sum()
    assert torch.allclose(b, (P * O.qk_band(GO, v, W, L)).sum(), atol=1e-10)
    assert torch.allclose(b, (v * O.inverse_gather(P, GO, W, L)).sum(), atol=1e-10)


# ---------------------------------------------------------------- window split
def test_split_window():
    assert O.split_window(27) == (27, 13)
    assert O.split_window(15) == (15, 7)
    assert O.split_window(7) == (7, 3)
    assert O.split_window(8) == (8, 3)          # even: left = W-1-W//2
    assert O.split_window(1) == (1, 0)
    assert O.split_window([9, 0]) == (9, 0)
    assert O.split_window([9, 8]) == (9, 8)
    for bad in (0, 81, [5, 5], [5, -1]):
        with pytest.raises(ValueError):
            O.split_window(bad)


# ---------------------------------------------------------------- mask + softmax
@pytest.mark.parametrize("T,W,L", GEOMS)
def test_mask_closed_form(T, W, L):
    pads = [0, 1, T // 2, T]
    m = O.attn_mask(T, W, L, torch.tensor(pads))
    assert m.shape == (len(pads), T, W)
    for n, pad in enumerate(pads):
        tv = T - pad
        for t in range(T):
            for j in range(W):
                u = t - L + j
                want = -100.0 if (t >= tv or u < 0 or u >= tv) else 0.0
                assert m[n, t, j].item() == want
    assert set(m.unique().tolist()) <= {0.0, -100.0}


def test_zero_query_gives_softmax_of_bias_over_valid_slots():
    N, H, T, W, L, C = 2, 3, 8, 5, 2, 8
    rpb = _rand(H, W)
    pad = torch.tensor([0, 3])
    q = torch.zeros(N * H, T, C, dtype=F64)
    k, v = _rand(N * H, T, C), _rand(N * H, T, C)
    _, p, lse = O.na1d_forward(q, k, v, W, L, rpb, pad, H)
    p = p.view(N, H, T, W)
    for n in range(N):
        tv = T - int(pad[n])
        for h in range(H):
            for t in range(T):
                valid = [j for j in range(W) if 0 <= t - L + j < tv] if t < tv else []
                if valid:
                    want = torch.softmax(rpb[h, valid], 0)
                    assert torch.allclose(p[n, h, t, valid], want, atol=1e-12)
                    rest = [j for j in range(W) if j not in valid]
                    assert (p[n, h, t, rest] < 1e-40).all()
                else:  # fully padded row: uniform -100 shift cancels
                    assert torch.allclose(p[n, h, t], torch.softmax(rpb[h], 0), atol=1e-12)
    assert torch.allclose(p.sum(-1), torch.ones(N, H, T, dtype=F64), atol=1e-12)
    z = O.logits(q, k, W, L, rpb, pad, H)
    assert torch.allclose(lse, torch.log(torch.exp(z).sum(-1)), atol=1e-12)


def test_interior_rows_equal_dense_local_softmax():
    T, W, L, C = 12, 5, 2, 8
    q, k, v = _rand(1, T, C), _rand(1, T, C), _rand(1, T, C)
    o, _, _ = O.na1d_forward(q, k, v, W, L)
    dense = (q @ k.transpose(1, 2))[0]
    for t in range(T):
        lo, hi = max(0, t - L), min(T, t + (W - 1 - L) + 1)
        w = torch.softmax(dense[t, lo:hi], 0)
        assert torch.allclose(o[0, t], w @ v[0, lo:hi], atol=1e-12)


def test_padded_keys_do_not_reach_valid_rows():
    N, H, T, W, L, C = 2, 2, 10, 5, 2, 8
    pad = torch.tensor([4, 0])
    q, k, v = _rand(N * H, T, C), _rand(N * H, T, C), _rand(N * H, T, C)
    o1, _, _ = O.na1d_forward(q, k, v, W, L, None, pad, H)
    k2, v2 = k.clone(), v.clone()
    k2[:H, T - 4:] = 7.0
    v2[:H, T - 4:] = -3.0
    o2, _, _ = O.na1d_forward(q, k2, v2, W, L, None, pad, H)
    assert torch.allclose(o1[:H, :T - 4], o2[:H, :T - 4], atol=1e-30)
    assert torch.equal(o1[H:], o2[H:])


# ---------------------------------------------------------------- gradients
def test_gradcheck_fp64():
    N, H, T, W, L, C = 1, 2, 6, 4, 1, 8
    q, k, v = (_rand(N * H, T, C).requires_grad_(True) for _ in range(3))
    rpb = _rand(H, W).requires_grad_(True)
    pad = torch.tensor([1])
    f = lambda q, k, v, r: O.na1d_forward(q, k, v, W, L, r, pad, H)[0]
    assert torch.autograd.gradcheck(f, (q, k, v, rpb), eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("T,W,L", [(9, 5, 2), (3, 7, 3), (9, 4, 1), (12, 8, 3)])
def test_formula_backward_equals_autograd(T, W, L):
    N, H, C = 2, 2, 8
    q, k, v, do = _rand(N * H, T, C), _rand(N * H, T, C), _rand(N * H, T, C), _rand(N * H, T, C)
    rpb = _rand(H, W)
    pad = torch.tensor([0, min(2, T)])
    a = O.na1d_backward(q, k, v, do, W, L, rpb, pad, H)
    b = O.na1d_backward_formulas(q, k, v, do, W, L, rpb, pad, H)
    for x, y in zip(a, b):
        assert torch.allclose(x, y, atol=1e-10)


def test_batch_invariance():
    """The reference's own (commented-out) smoke check: sample 0 alone equals
    sample 0 inside a batch (pcf_nat_pytorch2.7.zip!/extension_na/test.py:24-51)."""
    T, W, L, C = 20, 7, 3, 16
    q, k, v = _rand(8, T, C), _rand(8, T, C), _rand(8, T, C)
    o_all, _, _ = O.na1d_forward(q, k, v, W, L)
    o_one, _, _ = O.na1d_forward(q[:1], k[:1], v[:1], W, L)
    assert torch.allclose(o_all[:1], o_one, atol=1e-14)


def test_seeded_inputs_are_reproducible_and_rounded():
    a = O.seeded_qkv(2, 5, 8, seed=3, dtype=torch.bfloat16, scale_q=0.125)
    b = O.seeded_qkv(2, 5, 8, seed=3, dtype=torch.bfloat16, scale_q=0.125)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    assert a[0].dtype == torch.bfloat16
    assert math.isclose(O.rel_l2(a[1].float(), a[1].float()), 0.0)


# --------------------------------------------------------------------------
# dense attention of the global layers
# --------------------------------------------------------------------------
def test_global_mask_closed_form():
    T, pads = 7, [0, 3, 7]
    m = O.global_mask(T, pads)
    assert m.shape == (3, T, T)
    for n, pad in enumerate(pads):
        for t in range(T):
            for u in range(T):
                want = O.MASK_VALUE if (t >= T - pad or u >= T - pad) else 0.0
                assert m[n, t, u].item() == want
    assert O.global_mask(T).abs().sum() == 0


def test_global_forward_matches_index_loops():
    import math
    N, H, T, C, scale, pads = 2, 2, 5, 3, 0.37, [0, 2]
    q, k, v = _rand(N * H, T, C), _rand(N * H, T, C), _rand(N * H, T, C)
    o, p, lse = O.global_forward(q, k, v, scale, pads, H)
    for b in range(N * H):
        tv = T - pads[b // H]
        for t in range(T):
            z = [sum(q[b, t, c].item() * k[b, u, c].item() for c in range(C)) * scale
                 + (O.MASK_VALUE if (t >= tv or u >= tv) else 0.0) for u in range(T)]
            den = sum(math.exp(x) for x in z)
            assert abs(lse[b, t].item() - math.log(den)) < 1e-9
            for c in range(C):
                want = sum(math.exp(z[u]) / den * v[b, u, c].item() for u in range(T))
                assert abs(o[b, t, c].item() - want) < 1e-9


def test_global_forward_matches_library_attention():
    N, H, T, C, scale, pads = 2, 3, 11, 8, 0.2, [4, 0]
    q, k, v = _rand(N * H, T, C), _rand(N * H, T, C), _rand(N * H, T, C)
    o, _, _ = O.global_forward(q, k, v, scale, pads, H)
    m = O.global_mask(T, pads, dtype=q.dtype).unsqueeze(1)
    want = F.scaled_dot_product_attention(q.view(N, H, T, C), k.view(N, H, T, C), v.view(N, H, T, C), attn_mask=m,
                                          scale=scale)
    assert torch.allclose(o.view(N, H, T, C), want, atol=1e-10)


def test_global_forward_equals_full_window_na1d():
    # a window that reaches every key from every row, no bias, no padding: the out-of-range slots carry -100 and
    # zero keys, i.e. weights of e^-100 relative to the in-range ones
    B, T, C = 2, 6, 4
    q, k, v = _rand(B, T, C), _rand(B, T, C), _rand(B, T, C)
    o_dense, _, lse_dense = O.global_forward(q, k, v, 1.0)
    o_band, _, lse_band = O.na1d_forward(q, k, v, 2 * T - 1, T - 1)
    assert torch.allclose(o_dense, o_band, atol=1e-12)
    assert torch.allclose(lse_dense, lse_band, atol=1e-12)


def test_global_gradcheck_fp64():
    N, H, T, C = 2, 2, 5, 3
    q, k, v = (_rand(N * H, T, C).requires_grad_(True) for _ in range(3))
    assert torch.autograd.gradcheck(lambda a, b, c: O.global_forward(a, b, c, 0.4, [1, 0], H)[0], (q, k, v), atol=1e-7)
    do = _rand(N * H, T, C)
    dq, dk, dv = O.global_backward(q, k, v, do, 0.4, [1, 0], H)
    # the textbook softmax-attention gradients
    o, p, _ = O.global_forward(q.detach(), k.detach(), v.detach(), 0.4, [1, 0], H)
    dp = torch.einsum("btc,buc->btu", do, v.detach())
    ds = p * (dp - (do * o).sum(-1, keepdim=True))
    assert torch.allclose(dv, torch.einsum("btu,btc->buc", p, do), atol=1e-12)
    assert torch.allclose(dq, 0.4 * torch.einsum("btu,buc->btc", ds, k.detach()), atol=1e-12)
    assert torch.allclose(dk, 0.4 * torch.einsum("btu,btc->buc", ds, q.detach()), atol=1e-12)


# --------------------------------------------------------------------------
# attention dropout of the fused operator
# --------------------------------------------------------------------------
_DROPOUT_C = r"""
/* keep rule of na1d_fused_forward_dropout, transcribed from its statement in the public header */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
static uint32_t mix(uint32_t x) { x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }
int main(int argc, char **argv) {
    uint64_t seed = strtoull(argv[1], 0, 10);
    uint32_t threshold = (uint32_t)strtoull(argv[2], 0, 10);
    int W = atoi(argv[3]);
    for (int a = 4; a < argc; ++a) {
        uint64_t row = strtoull(argv[a], 0, 10);
        uint32_t key = mix(mix((uint32_t)row ^ (uint32_t)seed) + (uint32_t)(row >> 32) * 0x9E3779B9U + (uint32_t)(seed >> 32));
        for (int j = 0; j < W; ++j) putchar(mix(key ^ ((uint32_t)j * 0x9E3779B9U)) >= threshold ? '1' : '0');
        putchar('\n');
    }
    return 0;
}
"""


def test_dropout_hash_matches_a_c_transcription(tmp_path):
    import subprocess
    import numpy as np
    src = tmp_path / "keep.c"
    src.write_text(_DROPOUT_C)
    exe = tmp_path / "keep"
    subprocess.run(["gcc", "-O1", "-o", str(exe), str(src)], check=True)
    rows = [0, 1, 2, 299, 300, 2 ** 31, 2 ** 32 - 1, 2 ** 32, 2 ** 32 + 1, 2 ** 40 + 5, 2 ** 63 + 12345]
    for seed, p in ((0, 0.5), (12345678901234567, 0.1), (2 ** 64 - 1, 0.9), (77, 1e-9)):
        thr = min(int(p * 4294967296.0), 0xFFFFFFFF)
        out = subprocess.run([str(exe), str(seed), str(thr), "80"] + [str(r) for r in rows], check=True,
                             capture_output=True, text=True).stdout.split()
        want = np.array([[c == "1" for c in line] for line in out])
        got = O.dropout_keep_rows(np.array(rows, dtype=np.uint64), 80, p, seed)
        assert (got == want).all()
    assert O.dropout_keep(3, 5, 7, 0.0, 9).all()                      # threshold 0 keeps everything
    full = O.dropout_keep(3, 5, 7, 0.25, 9)
    assert (full.view(15, 7).numpy() == O.dropout_keep_rows(np.arange(15), 7, 0.25, 9)).all()   # row = b*T + t


def test_dropout_finaliser_is_a_bijection():
    import numpy as np
    def unshift(y, s):                       # inverse of x ^= x >> s
        x = y.copy()
        for _ in range(32 // s + 1):
            x = y ^ (x >> np.uint32(s))
        return x
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2 ** 32, 1 << 16, dtype=np.uint32)
    with np.errstate(over="ignore"):
        y = O._mix32(x)
        z = unshift(y, 16) * np.uint32(pow(0x846CA68B, -1, 2 ** 32))
        z = unshift(z, 15) * np.uint32(pow(0x7FEB352D, -1, 2 ** 32))
        z = unshift(z, 16)
    assert (z == x).all()
    assert O._mix32(np.zeros(1, dtype=np.uint32))[0] == 0            # the one fixed point the construction implies


def test_dropout_mask_statistics():
    B, T, W = 16, 300, 27
    n = B * T * W
    for p in (0.1, 0.5, 0.8):
        keep = O.dropout_keep(B, T, W, p, 2024).double()
        sigma = (p * (1 - p) / n) ** 0.5
        assert abs(keep.mean().item() - (1 - p)) < 5 * sigma
        c = keep - keep.mean()
        var = (c * c).mean()
        for a, b in ((c[:, :, 1:], c[:, :, :-1]), (c[:, 1:], c[:, :-1]), (c[1:], c[:-1])):   # slots, rows, sequences
            assert abs(((a * b).mean() / var).item()) < 5 / n ** 0.5 * 2
        other = O.dropout_keep(B, T, W, p, 2025).double()
        assert abs(((other - other.mean()) * c).mean().item() / var.item()) < 10 / n ** 0.5      # seeds are unrelated


def test_forward_with_dropout_matches_index_loops_and_differentiates():
    B, T, C, W, L, p = 2, 7, 3, 5, 2, 0.4
    q, k, v = _rand(B, T, C), _rand(B, T, C), _rand(B, T, C)
    keep = O.dropout_keep(B, T, W, p, 3)
    assert 0 < keep.sum() < keep.numel()
    o, prob, _ = O.na1d_forward(q, k, v, W, L, keep=keep, p_drop=p)
    o_plain, prob_plain, _ = O.na1d_forward(q, k, v, W, L)
    assert torch.equal(prob, prob_plain)                              # the softmax is not renormalised
    for b in range(B):
        for t in range(T):
            want = torch.zeros(C, dtype=F64)
            for j in range(W):
                u = t - L + j
                if 0 <= u < T and keep[b, t, j]:
                    want += prob[b, t, j] / (1 - p) * v[b, u]
            assert torch.allclose(o[b, t], want, atol=1e-12)
    q, k, v = (x.requires_grad_(True) for x in (q, k, v))
    assert torch.autograd.gradcheck(lambda a, b_, c: O.na1d_forward(a, b_, c, W, L, keep=keep, p_drop=p)[0], (q, k, v),
                                    atol=1e-7)
