"""CPU oracle for head-mixing attention (the reference's ``head_conv_attn``).  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` do, and only as the checker.

What is restated here (reference = Gusanidas/flash-multi-token-attention):

* ``forward``  follows ``flash_multi_token_attention/head_conv_attn/head_conv_fn_pytorch.py:7-54``
  (scores = Q K^T * scale -> linear map over the head axis -> -inf above the diagonal ->
  M = row max, L = sum exp(scores - M) -> softmax -> P V) and returns (O, L, M) as it does.
  The same definition as a module: ``head_conv_attn/head_conv_pytorch.py:19-39``.
* ``backward_manual``  the closed-form gradients that the reference's Triton kernels implement
  (``head_conv_attn/bwd_dq_dw.py:130-371``, ``bwd_dk_dv.py:130-400``): dP = dO V^T,
  D = rowsum(dO * O), dZ = P (dP - D), dS = scale W^T dZ, dW = sum dZ S^T, dQ = dS K, dK = dS^T Q,
  dV = P^T dO.  ``backward_autograd`` differentiates ``forward`` with torch autograd.

Pinning (the reference holds no golden vectors for this path, and it was not imported): in
``tests/test_head_conv_oracle.py`` against explicit loops over (batch, head, row, key) on small
inputs, the closed form w = identity == textbook softmax attention
(``F.scaled_dot_product_attention``), w = a head permutation == attention with permuted Q / K
heads, the reference's own formulation of the head map (``F.linear`` over a transposed score
tensor), fp64 gradcheck of ``forward`` and agreement of ``backward_manual`` with it.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


def _scale(d: int, scale: Optional[float]) -> float:
    return 1.0 / math.sqrt(d) if scale is None else float(scale)


def mixed_scores(Q, K, W, scale, causal):
    """Z[b,h,i,j] = sum_h' W[h,h'] scale <Q[b,h',i], K[b,h',j]>, -inf above the diagonal if causal."""
    S = torch.matmul(Q, K.transpose(-1, -2)) * scale
    Z = torch.einsum("gh,bhij->bgij", W.to(S.dtype), S)
    if causal:
        N, Nk = Z.shape[-2], Z.shape[-1]
        future = torch.triu(torch.ones(N, Nk, dtype=torch.bool), diagonal=1)
        Z = Z.masked_fill(future, float("-inf"))
    return S, Z


def forward(Q, K, V, W, causal: bool = False, scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    sc = _scale(Q.shape[-1], scale)
    _, Z = mixed_scores(Q, K, W, sc, causal)
    M = Z.max(dim=-1).values
    E = torch.exp(Z - M[..., None])
    L = E.sum(dim=-1)
    O = torch.matmul(E / L[..., None], V)
    return O, L, M


def backward_manual(Q, K, V, W, dO, causal: bool = False, scale: Optional[float] = None):
    sc = _scale(Q.shape[-1], scale)
    S, Z = mixed_scores(Q, K, W, sc, causal)
    P = torch.softmax(Z, dim=-1)
    O = torch.matmul(P, V)
    dP = torch.matmul(dO, V.transpose(-1, -2))
    D = (dO * O).sum(dim=-1, keepdim=True)
    dZ = P * (dP - D)
    dW = torch.einsum("bgij,bhij->gh", dZ, S)
    dS = torch.einsum("gh,bgij->bhij", W.to(dZ.dtype), dZ) * sc
    dQ = torch.matmul(dS, K)
    dK = torch.matmul(dS.transpose(-1, -2), Q)
    dV = torch.matmul(P.transpose(-1, -2), dO)
    return dQ, dK, dV, dW


def backward_autograd(Q, K, V, W, dO, causal: bool = False, scale: Optional[float] = None):
    q, k, v, w = (t.detach().clone().requires_grad_(True) for t in (Q, K, V, W))
    O, _, _ = forward(q, k, v, w, causal, scale)
    O.backward(dO)
    return q.grad, k.grad, v.grad, w.grad


def brute_force_forward(Q, K, V, W, causal: bool = False, scale: Optional[float] = None):
    """Explicit loops, float64 python arithmetic; for tiny inputs only."""
    B, H, N, d = Q.shape
    sc = _scale(d, scale)
    Qd, Kd, Vd, Wd = (t.double() for t in (Q, K, V, W))
    O = torch.zeros(B, H, N, d, dtype=torch.float64)
    L = torch.zeros(B, H, N, dtype=torch.float64)
    M = torch.zeros(B, H, N, dtype=torch.float64)
    for b in range(B):
        for i in range(N):
            jmax = i + 1 if causal else N
            raw = [[sc * float((Qd[b, hp, i] * Kd[b, hp, j]).sum()) for j in range(jmax)] for hp in range(H)]
            for h in range(H):
                z = [sum(float(Wd[h, hp]) * raw[hp][j] for hp in range(H)) for j in range(jmax)]
                m = max(z)
                e = [math.exp(x - m) for x in z]
                l = sum(e)
                M[b, h, i], L[b, h, i] = m, l
                for j in range(jmax):
                    O[b, h, i] += (e[j] / l) * Vd[b, h, j]
    return O, L, M
