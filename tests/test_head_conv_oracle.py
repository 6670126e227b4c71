"""Pins of the head-mixing oracle (CPU): explicit loops, closed forms, the reference's own
formulation of the head map, fp64 gradients."""
import math

import torch
import torch.nn.functional as F

from oracle import head_conv_oracle as hc


def _case(B=2, H=4, N=9, d=8, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn(B, H, N, d, generator=g, dtype=dtype) for _ in range(4))
    W = torch.randn(H, H, generator=g, dtype=dtype) / math.sqrt(H)
    return Q, K, V, dO, W


def test_forward_matches_explicit_loops():
    for causal in (False, True):
        Q, K, V, _, W = _case(B=1, H=3, N=6, d=4, seed=1)
        O, L, M = hc.forward(Q, K, V, W, causal, scale=0.7)
        Ob, Lb, Mb = hc.brute_force_forward(Q, K, V, W, causal, scale=0.7)
        assert torch.allclose(O, Ob, atol=1e-12) and torch.allclose(L, Lb, atol=1e-12) and torch.allclose(M, Mb, atol=1e-12)


def test_identity_map_is_textbook_attention():
    Q, K, V, _, _ = _case(seed=2)
    for causal in (False, True):
        O, L, M = hc.forward(Q, K, V, torch.eye(Q.shape[1], dtype=Q.dtype), causal)
        ref = F.scaled_dot_product_attention(Q, K, V, is_causal=causal)
        assert torch.allclose(O, ref, atol=1e-12)
        S = torch.matmul(Q, K.transpose(-1, -2)) / math.sqrt(Q.shape[-1])
        if causal:
            S = S.masked_fill(torch.triu(torch.ones(S.shape[-2:], dtype=torch.bool), 1), float("-inf"))
        assert torch.allclose(M + torch.log(L), torch.logsumexp(S, dim=-1), atol=1e-12)


def test_permutation_map_permutes_the_score_heads():
    Q, K, V, _, _ = _case(seed=3)
    H = Q.shape[1]
    perm = torch.tensor([2, 0, 3, 1])
    Wp = torch.zeros(H, H, dtype=Q.dtype)
    Wp[torch.arange(H), perm] = 1.0          # output head h takes the scores of head perm[h]
    O, _, _ = hc.forward(Q, K, V, Wp, causal=True)
    ref = F.scaled_dot_product_attention(Q[:, perm], K[:, perm], V, is_causal=True)
    assert torch.allclose(O, ref, atol=1e-12)


def test_head_map_as_the_reference_writes_it():
    # head_conv_fn_pytorch.py:17-26: F.linear over the score tensor with heads moved to the last axis
    Q, K, V, _, W = _case(seed=4)
    sc = 0.3
    scores = torch.matmul(Q, K.transpose(2, 3)) * sc
    z_ref = F.linear(scores.transpose(1, -1), W).transpose(1, -1)
    _, Z = hc.mixed_scores(Q, K, W, sc, causal=False)
    assert torch.allclose(Z, z_ref, atol=1e-12)
    O, L, M = hc.forward(Q, K, V, W, causal=False, scale=sc)
    assert torch.allclose(O, torch.matmul(torch.softmax(z_ref, -1), V), atol=1e-12)
    assert torch.allclose(M, z_ref.max(-1).values) and torch.allclose(L, torch.exp(z_ref - M[..., None]).sum(-1))


def test_gradients():
    for causal in (False, True):
        Q, K, V, dO, W = _case(B=1, H=3, N=5, d=4, seed=5)
        f = lambda q, k, v, w: hc.forward(q, k, v, w, causal, 0.5)[0]
        assert torch.autograd.gradcheck(f, tuple(t.clone().requires_grad_(True) for t in (Q, K, V, W)), atol=1e-6)
        man = hc.backward_manual(Q, K, V, W, dO, causal, 0.5)
        aut = hc.backward_autograd(Q, K, V, W, dO, causal, 0.5)
        for a, b in zip(man, aut):
            assert torch.allclose(a, b, atol=1e-10)


def test_finite_difference_of_the_map():
    Q, K, V, dO, W = _case(B=1, H=3, N=5, d=4, seed=6)
    dW = hc.backward_manual(Q, K, V, W, dO, True)[3]
    eps = 1e-6
    for (a, b) in ((0, 0), (1, 2), (2, 1)):
        Wp, Wm = W.clone(), W.clone()
        Wp[a, b] += eps
        Wm[a, b] -= eps
        fd = ((hc.forward(Q, K, V, Wp, True)[0] - hc.forward(Q, K, V, Wm, True)[0]) * dO).sum() / (2 * eps)
        assert abs(float(fd) - float(dW[a, b])) < 1e-6
