"""Head-mixing attention on the GPU against its CPU oracle (through the C ABI).

Tolerances: bf16 inputs, fp32 arithmetic: O within 2e-2 (bf16 output rounding), L relative 1e-3,
M 1e-3 absolute, gradients (fp32 outputs) within 2e-3 of the oracle's scale."""
import math

import pytest
import torch

from oracle import head_conv_oracle as hc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(B, H, N, d, seed, w_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn(B, H, N, d, generator=g).to(torch.bfloat16) for _ in range(4))
    W = w_scale * torch.randn(H, H, generator=g) / math.sqrt(H) + torch.eye(H)
    return Q, K, V, dO, W


def _ops():
    from flash_multi_token_attention_amd.head_conv_attn import ops
    return ops


SHAPES = [
    (2, 16, 201, 32),    # the reference's own check: fwd_kernel.py:383-390
    (1, 16, 64, 64),
    (1, 32, 48, 32),
    (1, 32, 130, 128),
    (2, 16, 16, 128),
    (1, 16, 1, 32),
    (1, 32, 257, 64),
]


@pytest.mark.parametrize("B,H,N,d", SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_forward(B, H, N, d, causal):
    Q, K, V, _, W = _case(B, H, N, d, seed=N + d)
    sc = 1.0 / math.sqrt(d)
    O, L, M = _ops().forward(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), scale=sc, causal=causal)
    Or, Lr, Mr = hc.forward(Q.float(), K.float(), V.float(), W, causal, sc)
    assert O.dtype == torch.bfloat16 and L.dtype == torch.float32
    assert float((O.float().cpu() - Or).abs().max()) <= 2e-2
    assert float((M.cpu() - Mr).abs().max()) <= 1e-3
    assert float(((L.cpu() - Lr).abs() / Lr).max()) <= 1e-3


@pytest.mark.parametrize("B,H,N,d", SHAPES)
@pytest.mark.parametrize("causal", [False, True])
def test_backward(B, H, N, d, causal):
    Q, K, V, dO, W = _case(B, H, N, d, seed=3 * N + d)
    sc = 1.0 / math.sqrt(d)
    ops = _ops()
    g = [t.to(DEV) for t in (Q, K, V, W, dO)]
    O, L, M = ops.forward(g[0], g[1], g[2], g[3], scale=sc, causal=causal)
    dQ, dW = ops.bwd_dq_dw(g[0], g[1], g[2], g[3], O, g[4], L, M, causal=causal, scale=sc)
    dK, dV = ops.bwd_dkdv(g[0], g[1], g[2], g[3], O, g[4], L, M, causal=causal, scale=sc)
    ref = hc.backward_autograd(Q.float(), K.float(), V.float(), W, dO.float(), causal, sc)
    for name, got, want in zip(("dQ", "dK", "dV", "dW"), (dQ, dK, dV, dW), ref):
        assert got.dtype == torch.float32
        # observed 2e-3 .. 5e-3 of the gradient's scale (D = rowsum(dO o O) is taken from the bf16 O, the tile x
        # input products round the tile to bf16): the bound leaves a factor of two, not ten
        tol = 1e-2 * max(1.0, float(want.abs().max()))
        err = float((got.cpu() - want).abs().max())
        assert err <= tol, (name, err, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_other_input_dtypes_are_used_as_bf16(dtype):
    # float32 and float16 tensors are converted to bfloat16 (the kernels' operand type): the results are those of
    # the converted inputs, bit for bit; O comes back in the dtype of q
    Q, K, V, dO, W = _case(2, 16, 90, 64, seed=5)
    ops = _ops()
    lo = [t.to(DEV) for t in (Q, K, V, W, dO)]
    hi = [t.to(dtype) if t.dtype == torch.bfloat16 else t for t in lo]
    O, L, M = ops.forward(*lo[:4], scale=0.125, causal=True)
    O2, L2, M2 = ops.forward(*hi[:4], scale=0.125, causal=True)
    # (O is rounded once, to the dtype of q: within a bf16 rounding of the bf16 result; the statistics are the same)
    assert O2.dtype == dtype and torch.equal(L2, L) and torch.equal(M2, M)
    assert float((O2.float() - O.float()).abs().max()) <= 2.0 ** -8 * max(1.0, float(O.float().abs().max()))
    for fn in (ops.bwd_dq_dw, ops.bwd_dkdv):
        a = fn(*lo[:4], O, lo[4], L, M, causal=True, scale=0.125)
        b = fn(*hi[:4], O, hi[4], L, M, causal=True, scale=0.125)
        assert all(torch.equal(x, y) for x, y in zip(a, b))


def test_identity_map_is_plain_attention():
    Q, K, V, _, _ = _case(1, 16, 100, 64, seed=9)
    O, _, _ = _ops().forward(Q.to(DEV), K.to(DEV), V.to(DEV), torch.eye(16, device=DEV), scale=0.125, causal=True)
    ref = torch.nn.functional.scaled_dot_product_attention(Q.float(), K.float(), V.float(), is_causal=True)
    assert float((O.float().cpu() - ref).abs().max()) <= 2e-2


def test_module_autograd():
    from flash_multi_token_attention.head_conv_attn.head_conv_attn import HeadConvAttention, head_conv_attention
    torch.manual_seed(0)
    mod = HeadConvAttention(16, dtype=torch.bfloat16).to(DEV)
    assert tuple(mod.head_conv_weights.shape) == (16, 16)
    Q, K, V, dO, _ = _case(1, 16, 40, 32, seed=11)
    q, k, v = (t.to(DEV).requires_grad_(True) for t in (Q, K, V))
    out = mod(q, k, v, causal=True)
    out.backward(dO.to(DEV))
    W = mod.head_conv_weights.detach().float().cpu()
    ref = hc.backward_autograd(Q.float(), K.float(), V.float(), W, dO.float(), True, None)
    for got, want in zip((q.grad, k.grad, v.grad, mod.head_conv_weights.grad), ref):
        # (bf16 module: the gradients themselves are rounded to bf16, 4e-3 of their scale)
        assert float((got.float().cpu() - want).abs().max()) <= 1.5e-2 * max(1.0, float(want.abs().max()))
    out2 = head_conv_attention(q.detach(), k.detach(), v.detach(), mod.head_conv_weights.detach(), True, None)
    assert torch.equal(out2, out.detach())


def test_rejections():
    ops = _ops()
    Q = torch.zeros(1, 8, 16, 32, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError, match="n_heads must be 16 or 32"):
        ops.forward(Q, Q, Q, torch.eye(8, device=DEV))
    Q = torch.zeros(1, 16, 16, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError, match="d_model must be <= 128"):
        ops.forward(Q, Q, Q, torch.eye(16, device=DEV))
