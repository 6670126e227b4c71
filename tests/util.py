"""Helpers shared by the parity tests."""
import math

import torch

from oracle import conv_attn_oracle as orc

# Tolerances of the headline metric's definition.
TOL_BF16 = 2e-2      # max-abs, O / dQ / dK / dV from bf16 inputs
TOL_DW_REL = 5e-2    # max-abs error of dW relative to max |dW|
TOL_FP32 = 1e-4      # max-abs, fp32 mode


def rand_case(B, H, Nq, Nk, d, c_q, c_k, dtype, seed=0, sigma=0.05, w_mode="delta"):
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, Nq, d, generator=g)
    K = torch.randn(B, H, Nk, d, generator=g)
    V = torch.randn(B, H, Nk, d, generator=g)
    dO = torch.randn(B, H, Nq, d, generator=g)
    E = torch.randn(H, c_q, c_k, generator=g)
    if w_mode == "delta":
        W = sigma * E
        W[:, c_q - 1, (c_k - 1) // 2] += 1.0
    else:
        W = 0.2 * E
    if dtype == torch.bfloat16:
        Q, K, V, dO = (t.to(torch.bfloat16) for t in (Q, K, V, dO))
    return Q, K, V, dO, W


def oracle_fwd(Q, K, V, W, causal, scale=None):
    return orc.forward(Q.float().cpu(), K.float().cpu(), V.float().cpu(), W.float().cpu(), causal, scale)


def oracle_bwd(Q, K, V, W, dO, causal, scale=None):
    return orc.backward_autograd(Q.float().cpu(), K.float().cpu(), V.float().cpu(), W.float().cpu(),
                                 dO.float().cpu(), causal, scale)


def max_abs(a, b):
    return float((a.float().cpu() - b.float().cpu()).abs().max())


def rel_max(a, b):
    """Largest absolute difference relative to the largest reference entry.  The floor of
    1e-3 on the denominator covers references that are zero throughout (one query row and one
    key: dW is exactly 0, while a kernel that sums D in another order leaves ~1e-7)."""
    b = b.float().cpu()
    return float((a.float().cpu() - b).abs().max() / b.abs().max().clamp_min(1e-3))


def scale_of(d):
    return 1.0 / math.sqrt(d)
