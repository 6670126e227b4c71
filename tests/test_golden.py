"""The torch oracle (CPU) and the fp32-arithmetic GPU kernels against the committed
golden fixtures (explicit-loop float64 values, see tests/golden/make_golden.py)."""
import os

import numpy as np
import pytest
import torch

from flash_multi_token_attention_amd import synthetic
from oracle import conv_attn_oracle as orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _t(a):
    return torch.from_numpy(np.asarray(a))


def test_oracle_c1_forward_matches_golden():
    wl = synthetic.WORKLOADS["c1_cpu_fp32"]
    t = synthetic.make_inputs(wl, seed=0)
    gold = np.load(os.path.join(GOLD, "c1_forward.npz"))
    torch.testing.assert_close(t["W"], _t(gold["W"]))          # the generator is part of the contract
    O, M, L = orc.forward(t["Q"].double(), t["K"].double(), t["V"].double(), t["W"].double(), True, wl.scale)
    np.testing.assert_allclose(O.numpy(), gold["O"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(M.numpy(), gold["M"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(L.numpy(), gold["L"], rtol=2e-5, atol=2e-6)
    # and in fp32, the precision the CPU baseline runs at: within the fp32-mode tolerance
    O32, M32, L32 = orc.forward(t["Q"], t["K"], t["V"], t["W"], True, wl.scale)
    assert float((O32 - _t(gold["O"])).abs().max()) <= 1e-4


@pytest.mark.parametrize("tag", ["a", "b"])
def test_oracle_small_fwd_bwd_matches_golden(tag):
    g = np.load(os.path.join(GOLD, "small_fwd_bwd.npz"))
    Q, K, V, dO, W = (_t(g[f"{tag}_{k}"]).double() for k in ("Q", "K", "V", "dO", "W"))
    O, M, L = orc.forward(Q, K, V, W, True)
    np.testing.assert_allclose(O.numpy(), g[f"{tag}_O"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(L.numpy(), g[f"{tag}_L"], rtol=2e-5, atol=2e-6)
    for fn in (orc.backward_manual, orc.backward_autograd):
        for got, name in zip(fn(Q, K, V, W, dO, True), ("dQ", "dK", "dV", "dW")):
            np.testing.assert_allclose(got.numpy(), g[f"{tag}_{name}"], rtol=2e-4, atol=2e-5)


def test_oracle_decode_matches_golden():
    g = np.load(os.path.join(GOLD, "decode_small.npz"))
    O, M, L = orc.decode(*(_t(g[k]).double() for k in ("Q", "K", "V", "W")))
    np.testing.assert_allclose(O.numpy(), g["O"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(M.numpy(), g["M"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(L.numpy(), g["L"], rtol=2e-5, atol=2e-6)


@pytest.mark.gpu
def test_gpu_fp32_kernels_match_golden():
    from flash_multi_token_attention_amd.conv_attn import ops, fwd_conv_attn_inference
    dev = "cuda:0"
    wl = synthetic.WORKLOADS["c1_cpu_fp32"]
    t = {k: v.to(dev) for k, v in synthetic.make_inputs(wl, seed=0).items()}
    gold = np.load(os.path.join(GOLD, "c1_forward.npz"))
    O, M, L = ops.forward(t["Q"], t["K"], t["V"], t["W"], wl.scale, wl.pad_q, wl.pad_k, True)
    assert float((O.cpu() - _t(gold["O"])).abs().max()) <= 1e-4
    assert float((M.cpu() - _t(gold["M"])).abs().max()) <= 1e-4
    assert float(((L.cpu() - _t(gold["L"])) / _t(gold["L"])).abs().max()) <= 1e-4
    g = np.load(os.path.join(GOLD, "small_fwd_bwd.npz"))
    for tag, (c_q, c_k) in {"a": (3, 5), "b": (6, 11)}.items():
        Q, K, V, dO, W = (_t(g[f"{tag}_{k}"]).to(dev) for k in ("Q", "K", "V", "dO", "W"))
        sc, pq, pk = 8 ** -0.5, c_q - 1, (c_k - 1) // 2
        O, M, L = ops.forward(Q, K, V, W, sc, pq, pk, True)
        D, LSE = ops.bwd_preprocess(O, dO, M, L)
        dQ, dW = ops.dq_backward(Q, K, V, dO, D, LSE, W, sc, pq, pk, True)
        dK, dV = ops.dkdv_backward(Q, K, V, dO, D, LSE, W, sc, pq, pk, True)
        for got, name in zip((O, dQ, dK, dV, dW), ("O", "dQ", "dK", "dV", "dW")):
            assert float((got.cpu() - _t(g[f"{tag}_{name}"])).abs().max()) <= 1e-4, (tag, name)
    g = np.load(os.path.join(GOLD, "decode_small.npz"))
    Q, K, V, W = (_t(g[k]).to(dev) for k in ("Q", "K", "V", "W"))
    O, M, L = fwd_conv_attn_inference(Q, K, V, W, 3, 16 ** -0.5, 5, 5, False)
    assert float((O.cpu() - _t(g["O"])).abs().max()) <= 1e-4
    assert float((M.cpu() - _t(g["M"])).abs().max()) <= 1e-4
