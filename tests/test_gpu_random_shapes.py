"""Seeded random shapes through the C ABI against the CPU oracle: the MFMA training kernels
(forward, one-pass and two-pass backward), the decode stream with every kind of split count and
the head-mixing kernels.
The fixed lists of the other test files sit on the tile edges; these draws cover the combinations
between them.  Each case prints its shape before it runs."""
import random

import pytest
import torch

from tests.util import TOL_BF16, TOL_DW_REL, max_abs, oracle_bwd, oracle_fwd, rand_case, rel_max, scale_of

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def test_random_training_shapes_match_oracle():
    from flash_multi_token_attention_amd.conv_attn import ops
    rnd = random.Random(2024)
    for case in range(80):
        d = rnd.choice([32, 64, 128])
        c_q = rnd.choice([1, 2, 3, 5, 6, 7, 8, 9, 10, 11])
        c_k = rnd.choice([1, 3, 5, 7, 9, 11, 13, 15])
        causal = rnd.random() < 0.6
        N = rnd.choice([1, 7, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 200, 255, 256, 257, 300, 333, 384, 500])
        Nk = N if causal else rnd.choice([N, max(1, N - 17), N + 45])
        B, H = rnd.choice([(1, 1), (1, 2), (2, 2), (1, 3)])
        one_pass = rnd.random() < 0.6
        w_mode = rnd.choice(["delta", "rand"])
        print(f"case {case}: B{B} H{H} Nq{N} Nk{Nk} d{d} {c_q}x{c_k} causal={causal} one_pass={one_pass} W={w_mode}", flush=True)
        Q, K, V, dO, W = rand_case(B, H, N, Nk, d, c_q, c_k, torch.bfloat16, seed=case * 7 + 1, w_mode=w_mode)
        ref_o = oracle_fwd(Q, K, V, W, causal)
        ref = oracle_bwd(Q, K, V, W, dO, causal)
        g = [t.to(DEV) for t in (Q, K, V, dO, W)]
        assert ops.kernel_path(g[0], g[1], g[4], causal, op="bwd") == "mfma"
        sc, pq, pk = scale_of(d), c_q - 1, (c_k - 1) // 2
        O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, pq, pk, causal, out_dtype=torch.float32)
        D, LSE = ops.bwd_preprocess(O, g[3], M, L)
        if one_pass:
            dQ, dK, dV, dW = ops.backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal, out_dtype=torch.float32)
        else:
            dQ, dW = ops.dq_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal, out_dtype=torch.float32)
            dK, dV = ops.dkdv_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, pq, pk, causal, out_dtype=torch.float32)
        assert max_abs(O, ref_o[0]) <= TOL_BF16, case
        assert max_abs(M, ref_o[1]) <= 2e-2 and rel_max(L, ref_o[2]) <= 2e-2, case
        assert max_abs(dQ, ref[0]) <= TOL_BF16 and max_abs(dK, ref[1]) <= TOL_BF16 and max_abs(dV, ref[2]) <= TOL_BF16, case
        assert rel_max(dW, ref[3]) <= TOL_DW_REL, case


def test_random_decode_shapes_match_oracle():
    from flash_multi_token_attention_amd.conv_attn import ops
    from oracle import conv_attn_oracle as orc
    rnd = random.Random(4242)
    for case in range(100):
        d = rnd.choice([32, 64, 128])
        c_q = rnd.choice([1, 2, 3, 5, 6, 7, 8, 11, 16])
        c_k = rnd.choice([1, 3, 5, 7, 11, 17])
        r = rnd.choice([1, c_q, min(16, c_q + 2), 16])
        causal = rnd.random() < 0.5
        Nk = rnd.choice([1, 5, 31, 64, 77, 128, 255, 256, 257, 500, 1000, 2049, 5000, 9000])
        B, H = rnd.choice([(1, 1), (2, 3), (1, 8), (3, 2)])
        splits = rnd.choice([0, 1, 2, 3, 7, 8, 9, 16, 33, 100, 257, 600, 1024])   # 0: the library's choice
        if splits > Nk:
            splits = max(1, Nk // 3)
        out_dtype = rnd.choice([torch.float32, torch.bfloat16])
        print(f"case {case}: B{B} H{H} r{r} Nk{Nk} d{d} {c_q}x{c_k} causal={causal} splits={splits} out={out_dtype}", flush=True)
        Q, K, V, _, W = rand_case(B, H, r, Nk, d, c_q, c_k, torch.bfloat16, seed=case * 13 + 5, w_mode=rnd.choice(["delta", "rand"]))
        O_ref, M_ref, L_ref = orc.decode(Q.float(), K.float(), V.float(), W, scale_of(d), causal=causal)
        g = [t.to(DEV) for t in (Q, K, V, W)]
        O, M, L, _ = ops.decode(g[0], g[1], g[2], g[3], splits, scale_of(d), causal, out_dtype=out_dtype)
        assert max_abs(O, O_ref) <= TOL_BF16, case
        assert max_abs(M, M_ref) <= 1e-3 and rel_max(L, L_ref) <= 1e-3, case


def test_random_head_mixing_shapes_match_oracle():
    import math
    from flash_multi_token_attention_amd.head_conv_attn import ops
    from oracle import head_conv_oracle as hc
    rnd = random.Random(777)
    for case in range(40):
        H = rnd.choice([16, 32])
        d = rnd.choice([32, 64, 128])
        N = rnd.choice([1, 15, 16, 17, 31, 33, 64, 100, 127, 129, 200, 257, 300])
        B = rnd.choice([1, 2, 3])
        causal = rnd.random() < 0.6
        w_scale = rnd.choice([0.3, 1.0])
        print(f"case {case}: B{B} H{H} N{N} d{d} causal={causal} w_scale={w_scale}", flush=True)
        g = torch.Generator().manual_seed(1000 + case)
        Q, K, V, dO = (torch.randn(B, H, N, d, generator=g).to(torch.bfloat16) for _ in range(4))
        W = w_scale * torch.randn(H, H, generator=g) / math.sqrt(H) + torch.eye(H)
        sc = 1.0 / math.sqrt(d)
        t = [x.to(DEV) for x in (Q, K, V, W, dO)]
        O, L, M = ops.forward(t[0], t[1], t[2], t[3], scale=sc, causal=causal)
        Or, Lr, Mr = hc.forward(Q.float(), K.float(), V.float(), W, causal, sc)
        assert float((O.float().cpu() - Or).abs().max()) <= TOL_BF16, case
        assert float((M.cpu() - Mr).abs().max()) <= 1e-3 and float(((L.cpu() - Lr).abs() / Lr).max()) <= 1e-3, case
        dQ, dW = ops.bwd_dq_dw(t[0], t[1], t[2], t[3], O, t[4], L, M, causal=causal, scale=sc)
        dK, dV = ops.bwd_dkdv(t[0], t[1], t[2], t[3], O, t[4], L, M, causal=causal, scale=sc)
        ref = hc.backward_autograd(Q.float(), K.float(), V.float(), W, dO.float(), causal, sc)
        for name, got, want in zip(("dQ", "dK", "dV", "dW"), (dQ, dK, dV, dW), ref):
            tol = 1e-2 * max(1.0, float(want.abs().max()))
            err = float((got.cpu() - want).abs().max())
            assert err <= tol, (case, name, err, tol)
