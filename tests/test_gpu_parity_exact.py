"""GPU parity of the fp32-arithmetic kernels (fp32 mode, and bf16 inputs with
CONVATTN_FLAG_EXACT) against the CPU oracle, through the C ABI."""
import pytest
import torch

from flash_multi_token_attention_amd import synthetic
from flash_multi_token_attention_amd.conv_attn import ops, fwd_conv_attn_inference
from oracle import conv_attn_oracle as orc
from tests.util import (TOL_BF16, TOL_DW_REL, TOL_FP32, max_abs, oracle_bwd, oracle_fwd, rand_case,
                        rel_max, scale_of)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = [
    # B, H, N, d, c_q, c_k
    (1, 2, 37, 32, 3, 5),
    (2, 2, 100, 64, 6, 11),
    (1, 3, 129, 128, 6, 11),
    (1, 1, 16, 64, 3, 3),
    (1, 2, 65, 64, 1, 1),
    (1, 2, 80, 40, 11, 11),
    (1, 1, 50, 64, 16, 33),
    (1, 2, 7, 8, 2, 7),
]


def test_c1_fp32_forward_matches_oracle():
    wl = synthetic.WORKLOADS["c1_cpu_fp32"]
    t = synthetic.make_inputs(wl, seed=0)
    O_ref, M_ref, L_ref = orc.forward(t["Q"], t["K"], t["V"], t["W"], True, wl.scale)
    g = {k: v.to(DEV) for k, v in t.items()}
    O, M, L = ops.forward(g["Q"], g["K"], g["V"], g["W"], wl.scale, wl.pad_q, wl.pad_k, True)
    assert ops.kernel_path(g["Q"], g["K"], g["W"]) == "fp32"
    assert max_abs(O, O_ref) <= TOL_FP32
    assert max_abs(M, M_ref) <= TOL_FP32
    assert rel_max(L, L_ref) <= TOL_FP32


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("causal", [True, False])
def test_forward_fp32(shape, causal):
    B, H, N, d, c_q, c_k = shape
    Q, K, V, _, W = rand_case(B, H, N, N, d, c_q, c_k, torch.float32, seed=N + c_k, w_mode="rand")
    O_ref, M_ref, L_ref = oracle_fwd(Q, K, V, W, causal)
    O, M, L = ops.forward(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), scale_of(d), c_q - 1,
                          (c_k - 1) // 2, causal)
    assert max_abs(O, O_ref) <= TOL_FP32
    assert max_abs(M, M_ref) <= TOL_FP32
    assert rel_max(L, L_ref) <= TOL_FP32


def test_forward_noncausal_rectangular():
    Q, K, V, _, W = rand_case(1, 2, 40, 93, 64, 6, 11, torch.float32, seed=3)
    O_ref, M_ref, L_ref = oracle_fwd(Q, K, V, W, False)
    O, M, L = ops.forward(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), scale_of(64), 5, 5, False)
    assert max_abs(O, O_ref) <= TOL_FP32 and max_abs(M, M_ref) <= TOL_FP32


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("causal", [True, False])
def test_backward_fp32(shape, causal):
    B, H, N, d, c_q, c_k = shape
    Q, K, V, dO, W = rand_case(B, H, N, N, d, c_q, c_k, torch.float32, seed=2 * N + c_q, w_mode="rand")
    dQ_ref, dK_ref, dV_ref, dW_ref = oracle_bwd(Q, K, V, W, dO, causal)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    sc, pq, pk = scale_of(d), c_q - 1, (c_k - 1) // 2
    O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, pq, pk, causal)
    D, LSE = ops.bwd_preprocess(O, g[3], M, L)
    dQ, dW = ops.dq_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal)
    dK, dV = ops.dkdv_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal)
    assert max_abs(dQ, dQ_ref) <= TOL_FP32 * max(1.0, float(dQ_ref.abs().max()))
    assert max_abs(dK, dK_ref) <= TOL_FP32 * max(1.0, float(dK_ref.abs().max()))
    assert max_abs(dV, dV_ref) <= TOL_FP32 * max(1.0, float(dV_ref.abs().max()))
    assert rel_max(dW, dW_ref) <= 1e-3
    # fixed-order reduction: bitwise repeatable
    dQ2, dW2 = ops.dq_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal)
    assert torch.equal(dW, dW2) and torch.equal(dQ, dQ2)
    # the whole-backward entry point runs the same fp32 kernels for these shapes
    dQ3, dK3, dV3, dW3 = ops.backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal)
    assert torch.equal(dQ3, dQ) and torch.equal(dK3, dK) and torch.equal(dV3, dV) and torch.equal(dW3, dW)


def test_bf16_inputs_exact_kernels_fwd_bwd():
    B, H, N, d, c_q, c_k = 2, 2, 150, 64, 6, 11
    Q, K, V, dO, W = rand_case(B, H, N, N, d, c_q, c_k, torch.bfloat16, seed=5)
    O_ref, M_ref, L_ref = oracle_fwd(Q, K, V, W, True)
    dQ_ref, dK_ref, dV_ref, dW_ref = oracle_bwd(Q, K, V, W, dO, True)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    sc = scale_of(d)
    O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, 5, 5, True, out_dtype=torch.bfloat16, exact=True)
    assert O.dtype == torch.bfloat16
    assert max_abs(O, O_ref) <= TOL_BF16 and max_abs(M, M_ref) <= 1e-3
    D, LSE = ops.bwd_preprocess(O, g[3], M, L)
    dQ, dW = ops.dq_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True,
                             out_dtype=torch.bfloat16, exact=True)
    dK, dV = ops.dkdv_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True,
                               out_dtype=torch.bfloat16, exact=True)
    assert max_abs(dQ, dQ_ref) <= TOL_BF16
    assert max_abs(dK, dK_ref) <= TOL_BF16
    assert max_abs(dV, dV_ref) <= TOL_BF16
    assert rel_max(dW, dW_ref) <= TOL_DW_REL


@pytest.mark.parametrize("r,Nk,d,c_q,c_k,splits", [
    (16, 240, 32, 5, 5, 4),      # the reference's own decode test shape
    (6, 500, 128, 6, 11, 3),
    (1, 77, 64, 6, 11, 1),
    (3, 300, 64, 3, 5, 7),
    (6, 64, 64, 6, 11, 64),
])
@pytest.mark.parametrize("causal", [False, True])
def test_decode_fp32(r, Nk, d, c_q, c_k, splits, causal):
    Q, K, V, _, W = rand_case(2, 2, r, Nk, d, c_q, c_k, torch.float32, seed=Nk + r, w_mode="rand")
    O_ref, M_ref, L_ref = orc.decode(Q, K, V, W, scale_of(d), causal=causal)
    O, M, L = fwd_conv_attn_inference(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), splits, scale_of(d),
                                      c_q - 1, (c_k - 1) // 2, causal)
    assert O.shape == (2, 2, 1, d) and M.shape == (2, 2, 1) and L.shape == (2, 2, 1)
    assert max_abs(O, O_ref) <= TOL_FP32
    assert max_abs(M, M_ref) <= TOL_FP32
    assert rel_max(L, L_ref) <= TOL_FP32


def test_decode_split_invariance_and_reference_shaped_op():
    Q, K, V, _, W = rand_case(1, 2, 6, 1000, 64, 6, 11, torch.float32, seed=9)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    outs = [fwd_conv_attn_inference(g[0], g[1], g[2], g[3], s, 0.125, 5, 5, False) for s in (1, 2, 5, 16)]
    for O, M, L in outs[1:]:
        assert max_abs(O, outs[0][0]) <= 1e-5 and max_abs(M, outs[0][1]) <= 1e-6
    Os, Ms, Ls = ops.forward_inference(g[0], g[1], g[2], g[3], 5, 0.125, 5, 5, False, 0)
    assert Os.shape == (1, 2, 5, 64) and Ms.shape == (1, 2, 5)
    assert max_abs(Os[:, :, 0:1], outs[0][0]) <= 1e-5
