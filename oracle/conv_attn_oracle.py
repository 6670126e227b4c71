"""CPU oracle for the fused conv-attention path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
only as the checker.  The product path is the HIP library and fails loudly
when that library is missing.

What is restated here (reference = Gusanidas/flash-multi-token-attention):

* ``forward``          follows ``flash_multi_token_attention/conv_attn/
  conv_attention_pytorch.py:117-185`` (QK^T -> zero the future -> scale ->
  zero-pad (pad_k, pad_k, pad_q, 0) -> grouped cross-correlation -> -inf the
  future -> M, L, softmax -> PV).
* ``lse`` / ``delta``  follow ``conv_attn/conv_attention_cuda.py:130,144``
  (LSE = M + log L, D = rowsum(dO * O)) but stay in fp32.
* ``backward_manual``  the closed-form gradients the reference kernels
  implement (``kernels/dq_bwd.cu:237-494``, ``kernels/dkdv_kernel.cu:273-411``,
  ``common/conv_utils.cuh:145-231``); ``backward_autograd`` differentiates
  ``forward`` with torch autograd, which is what the reference's own test
  compares against (``scripts/test_conv_attn.py:122-126``).
* ``decode``           follows ``conv_attn/flash_conv_attention_inference.py:
  57-67`` and ``scripts/test_fwd_inference_conv_attn.py:77-84``: the
  non-causal forward over the resident query rows, last row kept.
* ``combine_splits``   follows ``kernels/fwd_inference.cu:332-362``.

Pinning (no golden vectors exist in the reference, and the reference module
was not imported): every function above is checked in ``tests/test_oracle.py``
against an independent explicit-loop implementation (``oracle/brute_force.py``),
closed forms (identity tap == textbook softmax attention, single-tap == shifted
scores, 1x1 kernel == rescaled attention), fp64 gradcheck / finite differences,
and the split-invariance of the decode merge.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def pads(c_q: int, c_k: int) -> Tuple[int, int]:
    """(pad_q, pad_k) as the reference derives them (conv_attention_cuda.py:80-81)."""
    return c_q - 1, (c_k - 1) // 2


def _future(n_q: int, n_k: int, device) -> torch.Tensor:
    """Boolean [n_q, n_k] mask of key j strictly after query i (j > i)."""
    i = torch.arange(n_q, device=device).unsqueeze(1)
    j = torch.arange(n_k, device=device).unsqueeze(0)
    return j > i


def masked_scores(Q, K, scale: float, causal: bool) -> torch.Tensor:
    """S_m = scale * Q K^T with the strictly-future entries set to zero."""
    S = torch.matmul(Q, K.transpose(-2, -1))
    if causal:
        S = S.masked_fill(_future(Q.shape[-2], K.shape[-2], Q.device), 0.0)
    return S * scale


def conv_scores(S_m: torch.Tensor, W: torch.Tensor) -> torch.Tensor:
    """Per-head cross-correlation of the score plane with W[h] (zero padded:
    pad_q rows on top, pad_k columns either side)."""
    H, c_q, c_k = W.shape
    pq, pk = pads(c_q, c_k)
    x = F.pad(S_m, (pk, pk, pq, 0), value=0.0)
    return F.conv2d(x, W.unsqueeze(1).to(S_m.dtype), padding=0, groups=H)


def forward(Q, K, V, W, causal: bool = True, scale: Optional[float] = None):
    """Returns (O, M, L) with M the row max of the masked conv scores and L the
    plain sum of exp(C - M) (not a log-sum-exp)."""
    if scale is None:
        scale = 1.0 / math.sqrt(Q.shape[-1])
    S_m = masked_scores(Q, K, scale, causal)
    C = conv_scores(S_m, W)
    if causal:
        C = C.masked_fill(_future(Q.shape[-2], K.shape[-2], Q.device), float("-inf"))
    M = C.max(dim=-1).values
    E = torch.exp(C - M.unsqueeze(-1))
    L = E.sum(dim=-1)
    P = E / L.unsqueeze(-1)
    O = torch.matmul(P, V)
    return O, M, L


def lse(M: torch.Tensor, L: torch.Tensor) -> torch.Tensor:
    return M + torch.log(L)


def delta(O: torch.Tensor, dO: torch.Tensor) -> torch.Tensor:
    return (O * dO).sum(dim=-1)


def backward_autograd(Q, K, V, W, dO, causal: bool = True, scale: Optional[float] = None):
    """(dQ, dK, dV, dW) by differentiating ``forward`` with autograd."""
    Q, K, V, W = (t.detach().clone().requires_grad_(True) for t in (Q, K, V, W))
    O, _, _ = forward(Q, K, V, W, causal, scale)
    O.backward(dO)
    return Q.grad, K.grad, V.grad, W.grad


def backward_manual(Q, K, V, W, dO, causal: bool = True, scale: Optional[float] = None):
    """(dQ, dK, dV, dW) from the closed-form expressions the kernels use.

    dC = P * (dP - D); dW[a,b] = sum dC[i,j] * S_m[i+a-pq, j+b-pk];
    dS_m = transposed correlation of dC with W, re-zeroed on the future;
    dQ = scale * dS_m K; dK = scale * dS_m^T Q; dV = P^T dO.
    """
    if scale is None:
        scale = 1.0 / math.sqrt(Q.shape[-1])
    B, H, Nq, d = Q.shape
    Nk = K.shape[-2]
    c_q, c_k = W.shape[1:]
    pq, pk = pads(c_q, c_k)
    S_m = masked_scores(Q, K, scale, causal)
    C = conv_scores(S_m, W)
    fut = _future(Nq, Nk, Q.device)
    if causal:
        C = C.masked_fill(fut, float("-inf"))
    O, M, L = forward(Q, K, V, W, causal, scale)
    P = torch.exp(C - lse(M, L).unsqueeze(-1))
    dP = torch.matmul(dO, V.transpose(-2, -1))
    dC = P * (dP - delta(O, dO).unsqueeze(-1))
    dV = torch.matmul(P.transpose(-2, -1), dO)
    # dW: correlate dC with the zero-padded masked scores, summed over batch.
    Sp = F.pad(S_m, (pk, pk, pq, 0))
    dW = torch.zeros_like(W, dtype=Q.dtype)
    for a in range(c_q):
        for b in range(c_k):
            dW[:, a, b] = (dC * Sp[..., a:a + Nq, b:b + Nk]).sum(dim=(0, 2, 3))
    # dS_m[r,c] = sum_ab W[a,b] dC[r-a+pq, c-b+pk]: rows below, columns around.
    dCp = F.pad(dC, (pk, pk, 0, pq))
    dS = torch.zeros_like(S_m)
    for a in range(c_q):
        for b in range(c_k):
            w = W[:, a, b].to(Q.dtype).view(1, H, 1, 1)
            dS = dS + w * dCp[..., pq - a:pq - a + Nq, 2 * pk - b:2 * pk - b + Nk]
    if causal:
        dS = dS.masked_fill(fut, 0.0)
    dQ = scale * torch.matmul(dS, K)
    dK = scale * torch.matmul(dS.transpose(-2, -1), Q)
    return dQ, dK, dV, dW


def decode(Q_res, K, V, W, scale: Optional[float] = None, causal: bool = False):
    """Decode step: Q_res holds the last r resident query rows (r >= 1; fewer
    than c_q rows behave as zero rows in front).  Returns O [B,H,1,d], M, L
    [B,H,1] of the last row of the non-causal forward over (Q_res, K, V).

    ``causal=True`` is the training-consistent variant: the resident rows are
    taken to sit at positions Nk-r .. Nk-1 and the training masks are applied.
    """
    if scale is None:
        scale = 1.0 / math.sqrt(Q_res.shape[-1])
    if not causal:
        O, M, L = forward(Q_res, K, V, W, causal=False, scale=scale)
        return O[..., -1:, :], M[..., -1:], L[..., -1:]
    r, Nk = Q_res.shape[-2], K.shape[-2]
    S = torch.matmul(Q_res, K.transpose(-2, -1))
    pos = torch.arange(Nk - r, Nk, device=Q_res.device).unsqueeze(1)
    j = torch.arange(Nk, device=Q_res.device).unsqueeze(0)
    S = S.masked_fill(j > pos, 0.0) * scale
    C = conv_scores(S, W)[..., -1:, :]
    M = C.max(dim=-1).values
    E = torch.exp(C - M.unsqueeze(-1))
    L = E.sum(dim=-1)
    return torch.matmul(E / L.unsqueeze(-1), V), M, L


def gather_paged(pool: torch.Tensor, block_table: torch.Tensor, seq_len: int, b: int) -> torch.Tensor:
    """Dense [H_kv, seq_len, d] rows of batch entry ``b`` from a pool [n_pages, H_kv, page_size, d]:
    keys [i*page_size, (i+1)*page_size) are page ``block_table[b, i]`` (the layout vLLM-style serving
    caches use; the reference has no paged cache, so this only restates the indexing)."""
    ps = pool.shape[2]
    n = (seq_len + ps - 1) // ps
    pages = pool[block_table[b, :n].long()]                     # [n, H_kv, ps, d]
    return pages.permute(1, 0, 2, 3).reshape(pool.shape[1], n * ps, pool.shape[3])[:, :seq_len]


def decode_kv(Q_res, K_of, V_of, W, seq_lens, scale: Optional[float] = None, causal: bool = False):
    """Decode step over shared KV heads and per-sequence lengths, one batch entry at a time:
    ``K_of(b)`` / ``V_of(b)`` return the dense [H_kv, seq_lens[b], d] rows of entry b; query head h
    reads KV head h // (H // H_kv).  Returns O [B,H,1,d], M, L [B,H,1] (``decode`` per entry)."""
    B, H = Q_res.shape[0], Q_res.shape[1]
    outs = []
    for b in range(B):
        Kb, Vb = K_of(b), V_of(b)
        rep = H // Kb.shape[0]
        Kb = Kb.repeat_interleave(rep, dim=0).unsqueeze(0)
        Vb = Vb.repeat_interleave(rep, dim=0).unsqueeze(0)
        outs.append(decode(Q_res[b:b + 1], Kb[:, :, :seq_lens[b]], Vb[:, :, :seq_lens[b]], W, scale, causal))
    return tuple(torch.cat([o[i] for o in outs], dim=0) for i in range(3))


def combine_splits(O_part, M_part, L_part):
    """Merge per-split un-normalised partials: O_part [..., S, d], M_part,
    L_part [..., S] -> normalised O [..., d], M, L [...]."""
    M = M_part.max(dim=-1).values
    w = torch.exp(M_part - M.unsqueeze(-1))
    L = (L_part * w).sum(dim=-1)
    O = (O_part * w.unsqueeze(-1)).sum(dim=-2) / L.unsqueeze(-1)
    return O, M, L


def forward_chunked(Q, K, V, W, causal: bool = True, scale: Optional[float] = None,
                    rows: int = 1024):
    """Same result as ``forward`` but one (batch, head) and ``rows`` query rows
    at a time, so the [N, N] temporaries stay small at long N."""
    B, H, N, d = Q.shape
    pq, _ = pads(*W.shape[1:])
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    O = torch.empty_like(Q)
    M = torch.empty(B, H, N, dtype=Q.dtype)
    L = torch.empty(B, H, N, dtype=Q.dtype)
    Nk = K.shape[-2]
    j = torch.arange(Nk).unsqueeze(0)
    for b in range(B):
        for h in range(H):
            for r0 in range(0, N, rows):
                r1 = min(N, r0 + rows)
                lo = max(0, r0 - pq)
                i = torch.arange(lo, r1).unsqueeze(1)
                S = Q[b, h, lo:r1] @ K[b, h].T
                if causal:
                    S = S.masked_fill(j > i, 0.0)
                S = S * scale
                # conv_scores zero-pads pq rows above row ``lo``; rows >= r0 only
                # ever reach back to r0 - pq >= lo (or to the true top edge).
                C = conv_scores(S[None, None], W[h:h + 1])[0, 0][r0 - lo:]
                if causal:
                    C = C.masked_fill(j > torch.arange(r0, r1).unsqueeze(1), float("-inf"))
                m = C.max(dim=-1).values
                E = torch.exp(C - m.unsqueeze(-1))
                l = E.sum(dim=-1)
                O[b, h, r0:r1] = (E / l.unsqueeze(-1)) @ V[b, h]
                M[b, h, r0:r1] = m
                L[b, h, r0:r1] = l
    return O, M, L
