"""CPU emulation of the quantisation step of the backward's dC tiles: dC = P (dP - D) is stored as
fp16 times a power of two s per (batch, head).  Without s, dC underflows fp16 for small upstream
gradients; with s taken from amax|D| (csrc/mfma_common.hpp: dc_scale_log2_from_d) or from
amax|dO| amax|V| (csrc/bwd_chain_mfma.hip: dc_scale_finish_kernel) the relative error of the
quantised dC does not depend on the magnitude of dO."""
import math

import pytest
import torch

from oracle import conv_attn_oracle as orc


def _scale_from_d(D: torch.Tensor) -> float:
    mx = float(D.abs().max())
    return 2.0 ** min(max(math.floor(8.0 - math.log2(mx)), -100), 100) if 0 < mx < 3e38 else 1.0


def _scale_from_inputs(dO: torch.Tensor, V: torch.Tensor, d: int) -> float:
    m = math.sqrt(d) * float(dO.abs().max()) * float(V.abs().max())
    return 2.0 ** min(max(math.floor(12.0 - math.log2(m)), -120), 120) if m > 0 else 1.0


def _dc(Q, K, V, W, dO, scale):
    """P, dP, D and dC of the oracle's manual backward for one (batch, head) (float64)."""
    S = orc.masked_scores(Q, K, scale, True)
    C = orc.conv_scores(S, W)
    N = Q.shape[-2]
    fut = torch.triu(torch.ones(N, N, dtype=torch.bool), diagonal=1)
    P = torch.softmax(C.masked_fill(fut, float("-inf")), dim=-1)
    dP = dO @ V.transpose(-2, -1)
    D = (P * dP).sum(-1, keepdim=True)
    return P, dP, D, P * (dP - D)


@pytest.mark.parametrize("mag", [1.0, 1e-3, 1e-6, 1e-8, 1e3])
def test_scaled_fp16_dc_is_scale_invariant(mag):
    g = torch.Generator().manual_seed(3)
    N, d = 256, 64
    Q, K, V, dO = (torch.randn(1, 1, N, d, generator=g, dtype=torch.float64) for _ in range(4))
    W = torch.zeros(1, 6, 11, dtype=torch.float64)
    W[0, 5, 5] = 1.0   # identity tap
    dO = dO * mag
    P, dP, D, dC = _dc(Q, K, V, W, dO, 1.0 / math.sqrt(d))
    big = dC.abs() > 1e-4 * float(dC.abs().max())   # entries that matter for the gradients
    for s in (_scale_from_d(D), _scale_from_inputs(dO, V, d)):
        q = (dC * s).to(torch.float16).to(torch.float64) / s
        assert torch.isfinite(q).all()
        rel = ((q - dC).abs() / dC.abs())[big].max()
        assert rel <= 2.0 ** -10, (mag, s, float(rel))   # fp16 rounding (2^-11) plus subnormal slack
    if mag <= 1e-6:
        # what the unscaled fp16 tile did: most of these entries are flushed or lose their bits
        q0 = dC.to(torch.float16).to(torch.float64)
        rel0 = ((q0 - dC).abs() / dC.abs())[big]
        assert float((rel0 > 2.0 ** -6).float().mean()) > 0.5
