"""Explicit-loop conv-attention in float64 numpy.  TEST INFRASTRUCTURE ONLY.

Written from the index formula alone (reference README.md:11-24 and the mask
predicates of common/conv_utils.cuh:62-116), with no tensor-library
convolution, so that a transposed tap, a wrong pad side or a swapped mask in
``conv_attn_oracle`` cannot also be wrong here in the same way:

    S_m[i,j] = scale*<q_i,k_j>  if (not causal or j <= i) else 0
    C[i,j]   = sum_{a<c_q} sum_{b<c_k} W[a,b] * S_m[i+a-(c_q-1), j+b-(c_k-1)//2]
               (terms whose indices leave [0,Nq)x[0,Nk) are dropped)
    C[i,j]   = -inf if causal and j > i
    M = rowmax C, L = rowsum exp(C-M), O = softmax(C) V

Only for small shapes: the loops are O(Nq*Nk*c_q*c_k) in Python.
"""
import math

import numpy as np


def forward_one(q, k, v, w, causal=True, scale=None):
    """q [Nq,d], k,v [Nk,d], w [c_q,c_k] -> O [Nq,d], M [Nq], L [Nq], C, S_m."""
    q, k, v, w = (np.asarray(t, dtype=np.float64) for t in (q, k, v, w))
    Nq, d = q.shape
    Nk = k.shape[0]
    c_q, c_k = w.shape
    pq, pk = c_q - 1, (c_k - 1) // 2
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    S = np.zeros((Nq, Nk))
    for i in range(Nq):
        for j in range(Nk):
            if causal and j > i:
                continue
            S[i, j] = scale * float(np.dot(q[i], k[j]))
    C = np.zeros((Nq, Nk))
    for i in range(Nq):
        for j in range(Nk):
            if causal and j > i:
                C[i, j] = -np.inf
                continue
            acc = 0.0
            for a in range(c_q):
                r = i + a - pq
                if r < 0 or r >= Nq:
                    continue
                for b in range(c_k):
                    c = j + b - pk
                    if c < 0 or c >= Nk:
                        continue
                    acc += w[a, b] * S[r, c]
            C[i, j] = acc
    M = C.max(axis=1)
    E = np.exp(C - M[:, None])
    L = E.sum(axis=1)
    O = (E / L[:, None]) @ v
    return O, M, L, C, S


def forward(Q, K, V, W, causal=True, scale=None):
    """Q [B,H,Nq,d] ... W [H,c_q,c_k] -> (O, M, L) float64 arrays."""
    Q, K, V, W = (np.asarray(t, dtype=np.float64) for t in (Q, K, V, W))
    B, H, Nq, d = Q.shape
    O = np.zeros((B, H, Nq, d))
    M = np.zeros((B, H, Nq))
    L = np.zeros((B, H, Nq))
    for b in range(B):
        for h in range(H):
            O[b, h], M[b, h], L[b, h], _, _ = forward_one(Q[b, h], K[b, h], V[b, h], W[h], causal, scale)
    return O, M, L


def backward(Q, K, V, W, dO, causal=True, scale=None):
    """(dQ, dK, dV, dW) by explicit accumulation of the chain rule, element by
    element (no matrix identities): for every (i,j) with dC = P*(dP-D), push
    W[a,b]*dC into dS_m[i+a-pq, j+b-pk] and S_m*dC into dW[a,b]."""
    Q, K, V, W, dO = (np.asarray(t, dtype=np.float64) for t in (Q, K, V, W, dO))
    B, H, Nq, d = Q.shape
    Nk = K.shape[2]
    c_q, c_k = W.shape[1:]
    pq, pk = c_q - 1, (c_k - 1) // 2
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    dQ, dK, dV, dW = np.zeros_like(Q), np.zeros_like(K), np.zeros_like(V), np.zeros_like(W)
    for b in range(B):
        for h in range(H):
            O, M, L, C, S = forward_one(Q[b, h], K[b, h], V[b, h], W[h], causal, scale)
            P = np.exp(C - M[:, None]) / L[:, None]
            dS = np.zeros((Nq, Nk))
            for i in range(Nq):
                Di = float(np.dot(O[i], dO[b, h, i]))
                for j in range(Nk):
                    if P[i, j] == 0.0:
                        continue
                    dV[b, h, j] += P[i, j] * dO[b, h, i]
                    dC = P[i, j] * (float(np.dot(dO[b, h, i], V[b, h, j])) - Di)
                    for a in range(c_q):
                        r = i + a - pq
                        if r < 0 or r >= Nq:
                            continue
                        for bb in range(c_k):
                            c = j + bb - pk
                            if c < 0 or c >= Nk:
                                continue
                            dW[h, a, bb] += dC * S[r, c]
                            if not (causal and c > r):
                                dS[r, c] += W[h, a, bb] * dC
            dQ[b, h] = scale * dS @ K[b, h]
            dK[b, h] = scale * dS.T @ Q[b, h]
    return dQ, dK, dV, dW


def decode(Q_res, K, V, W, scale=None):
    """Last row of the non-causal forward over the resident query rows."""
    O, M, L = forward(Q_res, K, V, W, causal=False, scale=scale)
    return O[:, :, -1:, :], M[:, :, -1:], L[:, :, -1:]
