"""Pins the CPU oracle without the reference: explicit loops, closed forms,
autograd/finite differences.  Each check is chosen so that a plausible slip (a
flipped tap axis, padding on the wrong side, the two causal masks swapped, L
taken as a log-sum-exp, dW not summed over the batch) fails at least one."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute_force as bf
from oracle import conv_attn_oracle as orc

torch.manual_seed(0)


def _rand(B, H, Nq, Nk, d, c_q, c_k, seed=0, dtype=torch.float64, wstd=0.3):
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, Nq, d, generator=g, dtype=dtype)
    K = torch.randn(B, H, Nk, d, generator=g, dtype=dtype)
    V = torch.randn(B, H, Nk, d, generator=g, dtype=dtype)
    W = wstd * torch.randn(H, c_q, c_k, generator=g, dtype=dtype)
    dO = torch.randn(B, H, Nq, d, generator=g, dtype=dtype)
    return Q, K, V, W, dO


@pytest.mark.parametrize("c_q,c_k", [(1, 1), (1, 3), (2, 1), (3, 5), (6, 11), (4, 3), (5, 5)])
@pytest.mark.parametrize("causal", [True, False])
def test_forward_matches_explicit_loops(c_q, c_k, causal):
    Q, K, V, W, _ = _rand(2, 2, 11, 11, 4, c_q, c_k, seed=c_q * 31 + c_k)
    O, M, L = orc.forward(Q, K, V, W, causal=causal)
    Ob, Mb, Lb = bf.forward(Q.numpy(), K.numpy(), V.numpy(), W.numpy(), causal=causal)
    np.testing.assert_allclose(O.numpy(), Ob, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(M.numpy(), Mb, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(L.numpy(), Lb, rtol=1e-10, atol=1e-12)


def test_forward_noncausal_rectangular_matches_loops():
    # Nq != Nk is the decode shape.
    Q, K, V, W, _ = _rand(1, 2, 6, 19, 4, 6, 11, seed=5)
    O, M, L = orc.forward(Q, K, V, W, causal=False)
    Ob, Mb, Lb = bf.forward(Q.numpy(), K.numpy(), V.numpy(), W.numpy(), causal=False)
    np.testing.assert_allclose(O.numpy(), Ob, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(L.numpy(), Lb, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("c_q,c_k", [(3, 5), (6, 11), (1, 1)])
def test_identity_tap_is_plain_causal_attention(c_q, c_k):
    Q, K, V, _, _ = _rand(2, 3, 17, 17, 8, c_q, c_k, seed=3)
    W = torch.zeros(3, c_q, c_k, dtype=Q.dtype)
    W[:, c_q - 1, c_k // 2] = 1.0
    O, M, L = orc.forward(Q, K, V, W, causal=True)
    ref = F.scaled_dot_product_attention(Q, K, V, is_causal=True)
    torch.testing.assert_close(O, ref, rtol=1e-10, atol=1e-12)
    S = (Q @ K.transpose(-1, -2)) / math.sqrt(8)
    S = S.masked_fill(torch.triu(torch.ones(17, 17, dtype=torch.bool), 1), float("-inf"))
    torch.testing.assert_close(M, S.max(-1).values)
    torch.testing.assert_close(L, torch.exp(S - S.max(-1, keepdim=True).values).sum(-1))


@pytest.mark.parametrize("a0,b0", [(0, 0), (1, 4), (2, 1), (0, 2), (2, 3)])
def test_single_tap_is_a_shifted_copy_of_masked_scores(a0, b0):
    # W = w at one tap: C[i,j] = w * S_m[i+a0-pq, j+b0-pk]; pins both tap
    # orientations, the pad sides and that the pre-mask zeroes (not -inf).
    c_q, c_k, N = 3, 5, 9
    pq, pk = 2, 2
    Q, K, V, _, _ = _rand(1, 1, N, N, 4, c_q, c_k, seed=7)
    W = torch.zeros(1, c_q, c_k, dtype=Q.dtype)
    W[0, a0, b0] = 0.7
    S_m = orc.masked_scores(Q, K, 0.5, True)
    C = orc.conv_scores(S_m, W)
    expect = torch.zeros(N, N, dtype=Q.dtype)
    for i in range(N):
        for j in range(N):
            r, c = i + a0 - pq, j + b0 - pk
            if 0 <= r < N and 0 <= c < N and c <= r:
                expect[i, j] = 0.7 * 0.5 * float(Q[0, 0, r] @ K[0, 0, c])
    torch.testing.assert_close(C[0, 0], expect, rtol=1e-12, atol=1e-12)


def test_one_by_one_kernel_rescales_attention():
    Q, K, V, _, _ = _rand(1, 2, 13, 13, 8, 1, 1, seed=9)
    W = torch.tensor([[[1.7]], [[-0.4]]], dtype=Q.dtype)
    O, _, _ = orc.forward(Q, K, V, W, causal=True, scale=0.3)
    for h, w in enumerate([1.7, -0.4]):
        ref = F.scaled_dot_product_attention(Q[:, h], K[:, h], V[:, h], is_causal=True, scale=0.3 * w)
        torch.testing.assert_close(O[:, h], ref, rtol=1e-10, atol=1e-12)


def test_invariants():
    Q, K, V, W, _ = _rand(2, 2, 15, 15, 8, 6, 11, seed=11)
    O, M, L = orc.forward(Q, K, V, W)
    assert (L >= 1.0 - 1e-12).all()                         # the max itself contributes exp(0)
    torch.testing.assert_close(O[:, :, 0], V[:, :, 0])      # row 0 sees only key 0
    # future keys/values cannot leak into earlier rows
    K2, V2 = K.clone(), V.clone()
    K2[:, :, 10:] += 5.0
    V2[:, :, 10:] -= 3.0
    O2, _, _ = orc.forward(Q, K2, V2, W)
    torch.testing.assert_close(O2[:, :, :10], O[:, :, :10])
    # conv scores are linear in W
    S = orc.masked_scores(Q, K, 0.25, True)
    W2 = torch.randn_like(W)
    torch.testing.assert_close(orc.conv_scores(S, W + 2 * W2),
                               orc.conv_scores(S, W) + 2 * orc.conv_scores(S, W2))


def test_chunked_forward_equals_forward():
    Q, K, V, W, _ = _rand(1, 2, 70, 70, 8, 6, 11, seed=13, dtype=torch.float32)
    a = orc.forward(Q, K, V, W)
    b = orc.forward_chunked(Q, K, V, W, rows=16)
    for x, y in zip(a, b):
        torch.testing.assert_close(x, y, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("c_q,c_k", [(3, 5), (6, 11), (2, 3)])
@pytest.mark.parametrize("causal", [True, False])
def test_manual_backward_equals_autograd_and_loops(c_q, c_k, causal):
    Q, K, V, W, dO = _rand(2, 2, 10, 10, 4, c_q, c_k, seed=17 + c_q)
    man = orc.backward_manual(Q, K, V, W, dO, causal=causal)
    aut = orc.backward_autograd(Q, K, V, W, dO, causal=causal)
    loops = bf.backward(Q.numpy(), K.numpy(), V.numpy(), W.numpy(), dO.numpy(), causal=causal)
    for m, a, l in zip(man, aut, loops):
        torch.testing.assert_close(m, a, rtol=1e-9, atol=1e-11)
        np.testing.assert_allclose(m.numpy(), l, rtol=1e-9, atol=1e-11)


def test_autograd_gradcheck_fp64():
    Q, K, V, W, _ = _rand(1, 2, 6, 6, 3, 3, 5, seed=23)
    Q, K, V, W = (t.requires_grad_(True) for t in (Q, K, V, W))
    assert torch.autograd.gradcheck(lambda q, k, v, w: orc.forward(q, k, v, w)[0], (Q, K, V, W),
                                    eps=1e-6, atol=1e-6)


def test_dw_single_tap_finite_difference():
    Q, K, V, W, dO = _rand(2, 1, 8, 8, 4, 3, 5, seed=29)
    _, _, _, dW = orc.backward_manual(Q, K, V, W, dO)
    eps = 1e-6
    for a, b in [(0, 0), (2, 2), (1, 4)]:
        Wp, Wm = W.clone(), W.clone()
        Wp[0, a, b] += eps
        Wm[0, a, b] -= eps
        f = lambda w: float((orc.forward(Q, K, V, w)[0] * dO).sum())
        fd = (f(Wp) - f(Wm)) / (2 * eps)
        assert abs(fd - float(dW[0, a, b])) < 1e-6 * max(1.0, abs(fd))


def test_identity_tap_backward_equals_sdpa_autograd():
    Q, K, V, _, dO = _rand(1, 2, 12, 12, 8, 6, 11, seed=31)
    W = torch.zeros(2, 6, 11, dtype=Q.dtype)
    W[:, 5, 5] = 1.0
    dQ, dK, dV, _ = orc.backward_manual(Q, K, V, W, dO)
    q, k, v = (t.clone().requires_grad_(True) for t in (Q, K, V))
    F.scaled_dot_product_attention(q, k, v, is_causal=True).backward(dO)
    torch.testing.assert_close(dQ, q.grad, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(dK, k.grad, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(dV, v.grad, rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("r", [1, 3, 6, 16])
def test_decode_matches_loops_and_front_zero_padding(r):
    c_q, c_k = 6, 11
    Q, K, V, W, _ = _rand(2, 2, r, 37, 4, c_q, c_k, seed=37 + r)
    O, M, L = orc.decode(Q, K, V, W)
    Ob, Mb, Lb = bf.decode(Q.numpy(), K.numpy(), V.numpy(), W.numpy())
    np.testing.assert_allclose(O.numpy(), Ob, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(M.numpy(), Mb, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(L.numpy(), Lb, rtol=1e-10, atol=1e-12)
    # zero rows in front of the resident rows change nothing
    Qp = torch.cat([torch.zeros(2, 2, 16 - r, 4, dtype=Q.dtype), Q], dim=2) if r < 16 else Q
    O2, M2, L2 = orc.decode(Qp, K, V, W)
    torch.testing.assert_close(O2, O)
    torch.testing.assert_close(L2, L)


def test_decode_equals_training_row_when_only_current_row_taps():
    # With W[a < pq, :] = 0 neither causal mask can bite on the last row.
    c_q, c_k, N = 6, 11, 33
    Q, K, V, W, _ = _rand(1, 2, N, N, 4, c_q, c_k, seed=41)
    W[:, :c_q - 1, :] = 0.0
    O, M, L = orc.forward(Q, K, V, W, causal=True)
    Od, Md, Ld = orc.decode(Q[:, :, -c_q:], K, V, W)
    torch.testing.assert_close(Od[:, :, 0], O[:, :, -1])
    torch.testing.assert_close(Md[:, :, 0], M[:, :, -1])
    torch.testing.assert_close(Ld[:, :, 0], L[:, :, -1])


def test_causal_decode_equals_training_last_row():
    c_q, c_k, N = 6, 11, 29
    Q, K, V, W, _ = _rand(1, 2, N, N, 4, c_q, c_k, seed=43)
    O, M, L = orc.forward(Q, K, V, W, causal=True)
    Od, Md, Ld = orc.decode(Q[:, :, -c_q:], K, V, W, causal=True)
    torch.testing.assert_close(Od[:, :, 0], O[:, :, -1])
    torch.testing.assert_close(Ld[:, :, 0], L[:, :, -1])


def test_combine_splits_is_split_invariant():
    g = torch.Generator().manual_seed(47)
    c = torch.randn(3, 40, generator=g, dtype=torch.float64) * 4
    V = torch.randn(3, 40, 5, generator=g, dtype=torch.float64)
    full = torch.softmax(c, -1).unsqueeze(-2) @ V
    for cuts in ([0, 40], [0, 7, 40], [0, 1, 13, 14, 40]):
        Os, Ms, Ls = [], [], []
        for s, e in zip(cuts[:-1], cuts[1:]):
            m = c[:, s:e].max(-1).values
            p = torch.exp(c[:, s:e] - m[:, None])
            Os.append((p.unsqueeze(-2) @ V[:, s:e]).squeeze(-2))
            Ms.append(m)
            Ls.append(p.sum(-1))
        O, M, L = orc.combine_splits(torch.stack(Os, 1), torch.stack(Ms, 1), torch.stack(Ls, 1))
        torch.testing.assert_close(O, full.squeeze(-2))
        torch.testing.assert_close(M, c.max(-1).values)
        torch.testing.assert_close(L, torch.exp(c - c.max(-1, keepdim=True).values).sum(-1))
