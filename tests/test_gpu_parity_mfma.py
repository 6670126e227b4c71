"""GPU parity of the bf16 MFMA kernels against the CPU oracle (small shapes) and
against the fp32-arithmetic GPU kernels (full benchmark shapes), through the C ABI.
Tolerances: max-abs 2e-2 for O / dQ / dK / dV, 5e-2 relative for dW."""
import pytest
import torch

from flash_multi_token_attention_amd import synthetic
from flash_multi_token_attention_amd.conv_attn import ops
from tests.util import TOL_BF16, TOL_DW_REL, max_abs, oracle_bwd, oracle_fwd, rand_case, rel_max, scale_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

FWD_SHAPES = [
    # B, H, N, d, c_q, c_k
    (1, 2, 128, 128, 6, 11),
    (2, 2, 300, 128, 6, 11),
    (1, 2, 257, 64, 6, 11),
    (1, 2, 100, 64, 3, 5),
    (1, 1, 64, 128, 1, 1),
    (1, 2, 200, 64, 11, 11),
    (1, 2, 257, 128, 8, 9),
    (1, 1, 200, 64, 7, 7),
    (1, 1, 130, 128, 6, 17),
    (1, 2, 31, 64, 2, 3),
    (1, 1, 1, 64, 6, 11),
    # head dimension 32 (the reference dispatches 32, 64 and 128: kernels/fwd_wrapper.cu:69-95)
    (2, 2, 300, 32, 6, 11),
    (1, 2, 161, 32, 3, 3),
    (1, 1, 200, 32, 11, 11),
]


@pytest.mark.parametrize("shape", FWD_SHAPES)
@pytest.mark.parametrize("causal", [True, False])
def test_forward_bf16_mfma(shape, causal):
    B, H, N, d, c_q, c_k = shape
    Q, K, V, _, W = rand_case(B, H, N, N, d, c_q, c_k, torch.bfloat16, seed=N + c_q)
    O_ref, M_ref, L_ref = oracle_fwd(Q, K, V, W, causal)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    assert ops.kernel_path(g[0], g[1], g[3], causal) == "mfma"
    for odt in (torch.bfloat16, torch.float32):
        O, M, L = ops.forward(g[0], g[1], g[2], g[3], scale_of(d), c_q - 1, (c_k - 1) // 2, causal,
                              out_dtype=odt)
        assert O.dtype == odt
        assert max_abs(O, O_ref) <= TOL_BF16
        assert max_abs(M, M_ref) <= TOL_BF16
        assert rel_max(L, L_ref) <= TOL_BF16


def test_forward_random_window_weights():
    # all taps of comparable size (the reference module's init_random=True)
    Q, K, V, _, W = rand_case(1, 2, 260, 260, 128, 6, 11, torch.bfloat16, seed=4, w_mode="rand")
    O_ref, M_ref, _ = oracle_fwd(Q, K, V, W, True)
    O, M, _ = ops.forward(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), scale_of(128), 5, 5, True)
    assert max_abs(O, O_ref) <= TOL_BF16 and max_abs(M, M_ref) <= TOL_BF16


def test_forward_noncausal_rectangular_mfma():
    Q, K, V, _, W = rand_case(1, 2, 70, 333, 128, 6, 11, torch.bfloat16, seed=6)
    O_ref, M_ref, _ = oracle_fwd(Q, K, V, W, False)
    O, M, _ = ops.forward(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), scale_of(128), 5, 5, False)
    assert max_abs(O, O_ref) <= TOL_BF16 and max_abs(M, M_ref) <= TOL_BF16


def test_c2_full_size_forward_against_fp32_kernels():
    wl = synthetic.WORKLOADS["c2_fwd"]
    t = {k: v.to(DEV) for k, v in synthetic.make_inputs(wl, seed=0).items()}
    args = (t["Q"], t["K"], t["V"], t["W"], wl.scale, wl.pad_q, wl.pad_k, True)
    O, M, L = ops.forward(*args, out_dtype=torch.bfloat16)
    O_x, M_x, L_x = ops.forward(*args, out_dtype=torch.float32, exact=True)
    assert ops.kernel_path(t["Q"], t["K"], t["W"]) == "mfma"
    assert max_abs(O, O_x) <= TOL_BF16
    assert max_abs(M, M_x) <= TOL_BF16
    assert rel_max(L, L_x) <= TOL_BF16
    # rows of P sum to one: with V = 1 the output is 1 wherever the row sees a key
    ones = torch.ones_like(t["V"])
    O1, _, _ = ops.forward(t["Q"], t["K"], ones, t["W"], wl.scale, wl.pad_q, wl.pad_k, True,
                           out_dtype=torch.float32)
    assert float((O1 - 1).abs().max()) <= 1e-2


BWD_SHAPES = [
    # B, H, N, d, c_q, c_k
    (1, 2, 128, 128, 6, 11),
    (2, 2, 300, 128, 6, 11),
    (1, 2, 257, 64, 6, 11),
    (1, 2, 100, 64, 3, 5),
    (1, 1, 64, 128, 1, 1),
    (1, 2, 200, 64, 11, 11),
    (1, 1, 130, 128, 6, 15),
    (1, 2, 31, 64, 2, 3),
    (1, 1, 1, 64, 6, 11),
    # windows of 9 to 11 query taps: the 12-slot instance of the key-stationary kernel
    (1, 2, 330, 128, 11, 11),
    (1, 1, 257, 128, 9, 7),
    (2, 2, 150, 64, 10, 15),
    # head dimension 32
    (2, 2, 300, 32, 6, 11),
    (1, 2, 161, 32, 3, 3),
    (1, 1, 200, 32, 8, 9),
    (1, 2, 200, 32, 11, 11),
]


def _run_bwd(Q, K, V, dO, W, causal, odt, one_pass=False):
    """Backward through the two independent passes the reference exposes (dq_backward,
    dkdv_backward) or, with ``one_pass``, through the single-pass backward."""
    d = Q.shape[-1]
    c_q, c_k = W.shape[1:]
    sc, pq, pk = scale_of(d), c_q - 1, (c_k - 1) // 2
    O, M, L = ops.forward(Q, K, V, W, sc, pq, pk, causal, out_dtype=odt)
    D, LSE = ops.bwd_preprocess(O, dO, M, L)
    if one_pass:
        dQ, dK, dV, dW = ops.backward(Q, K, V, dO, D, LSE, W, sc, pq, pk, causal, out_dtype=odt)
        return dQ, dK, dV, dW
    dQ, dW = ops.dq_backward(Q, K, V, dO, D, LSE, W, sc, pq, pk, causal, out_dtype=odt)
    dK, dV = ops.dkdv_backward(Q, K, V, dO, D, LSE, W, sc, pq, pk, causal, out_dtype=odt)
    return dQ, dK, dV, dW


@pytest.mark.parametrize("shape", BWD_SHAPES)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("one_pass", [False, True])
def test_backward_bf16_mfma(shape, causal, one_pass):
    B, H, N, d, c_q, c_k = shape
    Q, K, V, dO, W = rand_case(B, H, N, N, d, c_q, c_k, torch.bfloat16, seed=3 * N + c_q)
    ref = oracle_bwd(Q, K, V, W, dO, causal)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    assert ops.kernel_path(g[0], g[1], g[4], causal, op="bwd") == "mfma"
    for odt in (torch.bfloat16, torch.float32):
        dQ, dK, dV, dW = _run_bwd(*g, causal, odt, one_pass)
        assert dQ.dtype == odt and dW.dtype == torch.float32
        assert max_abs(dQ, ref[0]) <= TOL_BF16
        assert max_abs(dK, ref[1]) <= TOL_BF16
        assert max_abs(dV, ref[2]) <= TOL_BF16
        assert rel_max(dW, ref[3]) <= TOL_DW_REL


@pytest.mark.parametrize("one_pass", [False, True])
def test_backward_random_window_weights_and_determinism(one_pass):
    Q, K, V, dO, W = rand_case(2, 2, 260, 260, 128, 6, 11, torch.bfloat16, seed=8, w_mode="rand")
    ref = oracle_bwd(Q, K, V, W, dO, True)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    out = _run_bwd(*g, True, torch.bfloat16, one_pass)
    for got, want in zip(out[:3], ref[:3]):
        assert max_abs(got, want) <= TOL_BF16
    assert rel_max(out[3], ref[3]) <= TOL_DW_REL
    again = _run_bwd(*g, True, torch.bfloat16, one_pass)
    for a, b in zip(out, again):
        assert torch.equal(a, b)       # no atomics anywhere: bitwise repeatable


@pytest.mark.parametrize("one_pass", [False, True])
@pytest.mark.parametrize("Nq,Nk", [(70, 333), (333, 70), (200, 129)])
def test_backward_noncausal_rectangular_mfma(Nq, Nk, one_pass):
    Q, K, V, dO, W = rand_case(1, 2, Nq, Nk, 128, 6, 11, torch.bfloat16, seed=10)
    ref = oracle_bwd(Q, K, V, W, dO, False)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    out = _run_bwd(*g, False, torch.bfloat16, one_pass)
    for got, want in zip(out[:3], ref[:3]):
        assert max_abs(got, want) <= TOL_BF16
    assert rel_max(out[3], ref[3]) <= TOL_DW_REL


def test_one_pass_backward_workspace_garbage_and_tile_edges():
    # The dS workspace is never initialised by the caller: poison the allocator's pool with
    # NaNs first, then check sequence lengths around the 32-key / 64-row / 128-row tile edges.
    poison = torch.full((64 << 20,), float("nan"), device=DEV)
    del poison
    for N in (63, 64, 65, 127, 129, 191, 193, 257, 449):
        Q, K, V, dO, W = rand_case(1, 1, N, N, 64, 6, 11, torch.bfloat16, seed=N)
        ref = oracle_bwd(Q, K, V, W, dO, True)
        g = [t.to(DEV) for t in (Q, K, V, dO, W)]
        out = _run_bwd(*g, True, torch.float32, one_pass=True)
        for got, want in zip(out[:3], ref[:3]):
            assert torch.isfinite(got).all() and max_abs(got, want) <= TOL_BF16, N
        assert rel_max(out[3], ref[3]) <= TOL_DW_REL, N


@pytest.mark.parametrize("one_pass", [False, True])
def test_backward_more_than_65535_batch_head_pairs(one_pass):
    # B * H beyond a grid dimension's 65535 (every kernel of the backward puts heads and batch entries on
    # separate grid dimensions).  Every (batch, head) pair is computed on its own: the last heads of the big
    # run must equal, bit for bit, a run of those heads alone, and a sample of pairs the CPU oracle.
    B, H, N, d, c_q, c_k = 2, 33000, 2, 32, 3, 3
    Q, K, V, dO, W = rand_case(B, H, N, N, d, c_q, c_k, torch.bfloat16, seed=11)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    assert ops.kernel_path(g[0], g[1], g[4], True, op="bwd") == "mfma"
    big = _run_bwd(*g, True, torch.float32, one_pass)
    sl = slice(H - 40, H)
    part = _run_bwd(*(t[:, sl].contiguous() for t in g[:4]), g[4][sl].contiguous(), True, torch.float32, one_pass)
    for got, want in zip(big[:3], part[:3]):
        assert torch.equal(got[:, sl], want)
    assert torch.equal(big[3][sl], part[3])
    ref = oracle_bwd(Q[:, sl], K[:, sl], V[:, sl], W[sl], dO[:, sl], True)
    for got, want in zip(part[:3], ref[:3]):
        assert max_abs(got, want) <= TOL_BF16
    assert rel_max(part[3], ref[3]) <= TOL_DW_REL


def test_module_autograd_matches_oracle_autograd():
    from flash_multi_token_attention_amd.conv_attn import ConvAttentionCUDA
    B, H, N, d, c_q, c_k = 2, 4, 192, 128, 6, 11
    Q, K, V, dO, W = rand_case(B, H, N, N, d, c_q, c_k, torch.bfloat16, seed=12)
    mod = ConvAttentionCUDA(H, c_q, c_k, init_random=False).to(DEV)
    with torch.no_grad():
        mod.conv_weight.copy_(W)
    q, k, v = (t.to(DEV).requires_grad_(True) for t in (Q, K, V))
    O = mod(q, k, v, causal=True)
    assert O.dtype == torch.bfloat16
    O.backward(dO.to(DEV))
    O_ref, _, _ = oracle_fwd(Q, K, V, W, True)
    ref = oracle_bwd(Q, K, V, W, dO, True)
    assert max_abs(O.detach(), O_ref) <= TOL_BF16
    assert max_abs(q.grad, ref[0]) <= TOL_BF16 and max_abs(k.grad, ref[1]) <= TOL_BF16
    assert max_abs(v.grad, ref[2]) <= TOL_BF16
    assert rel_max(mod.conv_weight.grad, ref[3]) <= TOL_DW_REL
    # identity window == plain causal attention
    ident = ConvAttentionCUDA(H, c_q, c_k, init_random=False).to(DEV)
    O_id = ident(q.detach(), k.detach(), v.detach())
    sdpa = torch.nn.functional.scaled_dot_product_attention(Q.float(), K.float(), V.float(), is_causal=True)
    assert max_abs(O_id, sdpa) <= TOL_BF16


@pytest.mark.parametrize("r,Nk,d,c_q,c_k,splits", [
    (6, 500, 128, 6, 11, 3),
    (6, 8192, 128, 6, 11, 1),
    (16, 240, 64, 5, 5, 4),
    (1, 77, 64, 6, 11, 1),
    (3, 1000, 128, 3, 5, 7),
    (6, 64, 64, 6, 11, 64),
    (6, 130, 128, 16, 17, 2),
    (16, 240, 32, 5, 5, 4),      # the reference's own decode test (scripts/test_fwd_inference_conv_attn.py:31-56)
    (6, 1000, 32, 6, 11, 2),
    (11, 40000, 64, 11, 11, 700),  # more splits than the merge kernel has threads (a long cache as in scripts/benchmark_fwd_inference_conv_attn.py)
])
@pytest.mark.parametrize("causal", [False, True])
def test_decode_bf16_stream(r, Nk, d, c_q, c_k, splits, causal):
    from flash_multi_token_attention_amd.conv_attn import fwd_conv_attn_inference
    from oracle import conv_attn_oracle as orc
    Q, K, V, _, W = rand_case(2, 3, r, Nk, d, c_q, c_k, torch.bfloat16, seed=Nk + r)
    O_ref, M_ref, L_ref = orc.decode(Q.float(), K.float(), V.float(), W, scale_of(d), causal=causal)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    assert ops.kernel_path(g[0], g[1], g[3], causal, op="decode") == "mfma"
    O, M, L = fwd_conv_attn_inference(g[0], g[1], g[2], g[3], splits, scale_of(d), c_q - 1,
                                      (c_k - 1) // 2, causal)
    assert O.shape == (2, 3, 1, d)
    assert max_abs(O, O_ref) <= TOL_BF16
    assert max_abs(M, M_ref) <= 1e-3
    assert rel_max(L, L_ref) <= 1e-3


@pytest.mark.parametrize("dtype,d,n_max", [(torch.bfloat16, 128, 700), (torch.bfloat16, 64, 512), (torch.float32, 64, 333)])
def test_decode_reads_views_of_a_longer_cache_in_place(dtype, d, n_max):
    """K / V as cache[:, :, :Nk] of a [B,H,N_max,d] cache: same bits as a dense copy, both kernel
    families; the rows after Nk are poisoned and must not be read into the result."""
    from flash_multi_token_attention_amd.conv_attn import fwd_conv_attn_inference
    B, H, r, Nk, c_q, c_k = 2, 3, 6, 300, 6, 11
    Q, K, V, _, W = rand_case(B, H, r, Nk, d, c_q, c_k, dtype, seed=n_max)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    Kc = torch.full((B, H, n_max, d), float("nan"), dtype=dtype, device=DEV)
    Vc = torch.full((B, H, n_max, d), float("nan"), dtype=dtype, device=DEV)
    Kc[:, :, :Nk] = g[1]
    Vc[:, :, :Nk] = g[2]
    Kv, Vv = Kc[:, :, :Nk], Vc[:, :, :Nk]
    assert not Kv.is_contiguous()
    for causal in (False, True):
        for splits in (1, 3):
            dense = fwd_conv_attn_inference(g[0], g[1], g[2], g[3], splits, scale_of(d), c_q - 1, (c_k - 1) // 2, causal)
            view = fwd_conv_attn_inference(g[0], Kv, Vv, g[3], splits, scale_of(d), c_q - 1, (c_k - 1) // 2, causal)
            for a, b in zip(dense, view):
                assert torch.equal(a, b)
    # a sequence-major cache ([B,N,H,d] permuted) has no dense rows per head: rejected, as a
    # non-contiguous tensor is by the reference
    Ks = g[1].permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    with pytest.raises(RuntimeError, match="contiguous"):
        fwd_conv_attn_inference(g[0], Ks, Ks, g[3], 1, scale_of(d), c_q - 1, (c_k - 1) // 2, False)
    with pytest.raises(RuntimeError, match="same strides"):
        fwd_conv_attn_inference(g[0], Kv, g[2], g[3], 1, scale_of(d), c_q - 1, (c_k - 1) // 2, False)


def test_decode_full_size_properties():
    # c4-sized cache per (batch, head) (fewer pairs): split invariance, agreement with
    # the fp32-arithmetic kernel, and sum of probabilities == 1 (V = 1 -> O = 1).
    from flash_multi_token_attention_amd.conv_attn.ops import decode
    wl = synthetic.WORKLOADS["c4_decode"]
    g = torch.Generator(device=DEV).manual_seed(1)
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV).to(torch.bfloat16)
    Q, K, V = mk(4, 8, wl.Nq, wl.d), mk(4, 8, wl.Nk, wl.d), mk(4, 8, wl.Nk, wl.d)
    W = synthetic.conv_weight(synthetic.Workload("x", 4, 8, 6, 8192, 128, 6, 11),
                              torch.randn(8, 6, 11, generator=torch.Generator().manual_seed(2))).to(DEV)
    base = decode(Q, K, V, W, 1, wl.scale)
    exact = decode(Q, K, V, W, 4, wl.scale, exact=True)
    assert max_abs(base[0], exact[0]) <= 2e-3 and max_abs(base[1], exact[1]) <= 1e-3
    for s in (2, 5, 32):
        o = decode(Q, K, V, W, s, wl.scale)
        assert max_abs(o[0], base[0]) <= 1e-4 and rel_max(o[2], base[2]) <= 1e-4
    ones = decode(Q, K, torch.ones_like(V), W, 3, wl.scale)
    assert float((ones[0] - 1).abs().max()) <= 1e-4


def test_c3_full_size_fwd_bwd_against_fp32_kernels():
    # The headline workload at full size: MFMA kernels vs the fp32-arithmetic kernels on the GPU
    # (the CPU oracle would need minutes), plus properties that do not depend on the size.
    wl = synthetic.WORKLOADS["c3_fwd_bwd"]
    t = {k: v.to(DEV) for k, v in synthetic.make_inputs(wl, seed=0).items()}
    Q, K, V, dO, W = t["Q"], t["K"], t["V"], t["dO"], t["W"]
    args = (wl.scale, wl.pad_q, wl.pad_k, True)
    O, M, L = ops.forward(Q, K, V, W, *args, out_dtype=torch.bfloat16)
    O_x, M_x, L_x = ops.forward(Q, K, V, W, *args, out_dtype=torch.float32, exact=True)
    assert max_abs(O, O_x) <= TOL_BF16 and max_abs(M, M_x) <= TOL_BF16 and rel_max(L, L_x) <= TOL_BF16
    D, LSE = ops.bwd_preprocess(O, dO, M, L)
    D_x, LSE_x = ops.bwd_preprocess(O_x, dO, M_x, L_x)
    dQ, dW = ops.dq_backward(Q, K, V, dO, D, LSE, W, *args, out_dtype=torch.bfloat16)
    dK, dV = ops.dkdv_backward(Q, K, V, dO, D, LSE, W, *args, out_dtype=torch.bfloat16)
    dQ_x, dW_x = ops.dq_backward(Q, K, V, dO, D_x, LSE_x, W, *args, exact=True)
    dK_x, dV_x = ops.dkdv_backward(Q, K, V, dO, D_x, LSE_x, W, *args, exact=True)
    assert max_abs(dQ, dQ_x) <= TOL_BF16
    assert max_abs(dK, dK_x) <= TOL_BF16
    assert max_abs(dV, dV_x) <= TOL_BF16
    assert rel_max(dW, dW_x) <= TOL_DW_REL
    # the one-pass backward: another kernel (the score chain stays in registers)
    dQ1, dK1, dV1, dW1 = ops.backward(Q, K, V, dO, D, LSE, W, *args, out_dtype=torch.bfloat16)
    assert max_abs(dK1, dK_x) <= TOL_BF16 and max_abs(dV1, dV_x) <= TOL_BF16
    assert max_abs(dQ1, dQ_x) <= TOL_BF16 and rel_max(dW1, dW_x) <= TOL_DW_REL
    # dV is linear in dO, dQ/dK/dW are too: doubling dO doubles them (D doubles with it)
    dQ2, dW2 = ops.dq_backward(Q, K, V, (2 * dO.float()).to(torch.bfloat16), 2 * D, LSE, W, *args,
                               out_dtype=torch.float32)
    assert rel_max(dW2, 2 * dW) <= 1e-3
    # row 0 attends to key 0 only: O[0] = V[0]
    assert max_abs(O[:, :, 0], V[:, :, 0]) <= 1e-6


def test_c5_long_context_one_head_forward_and_backward():
    # N = 16384 (the long-context workload) for one (batch, head) pair with the decaying window
    # of that workload: forward and backward against the fp32-arithmetic kernels.
    wl = synthetic.Workload("c5_one_head", 1, 1, 16384, 16384, 128, 6, 11, sigma=0.1, key_decay=3.0,
                            backward=True)
    t = {k: v.to(DEV) for k, v in synthetic.make_inputs(wl, seed=0).items()}
    Q, K, V, dO, W = t["Q"], t["K"], t["V"], t["dO"], t["W"]
    args = (wl.scale, wl.pad_q, wl.pad_k, True)
    O, M, L = ops.forward(Q, K, V, W, *args, out_dtype=torch.bfloat16)
    O_x, M_x, L_x = ops.forward(Q, K, V, W, *args, out_dtype=torch.float32, exact=True)
    assert max_abs(O, O_x) <= TOL_BF16 and max_abs(M, M_x) <= TOL_BF16
    D, LSE = ops.bwd_preprocess(O, dO, M, L)
    dQ, dW = ops.dq_backward(Q, K, V, dO, D, LSE, W, *args, out_dtype=torch.bfloat16)
    dK, dV = ops.dkdv_backward(Q, K, V, dO, D, LSE, W, *args, out_dtype=torch.bfloat16)
    D_x, LSE_x = ops.bwd_preprocess(O_x, dO, M_x, L_x)
    dQ_x, dW_x = ops.dq_backward(Q, K, V, dO, D_x, LSE_x, W, *args, exact=True)
    dK_x, dV_x = ops.dkdv_backward(Q, K, V, dO, D_x, LSE_x, W, *args, exact=True)
    assert max_abs(dQ, dQ_x) <= TOL_BF16 and max_abs(dK, dK_x) <= TOL_BF16 and max_abs(dV, dV_x) <= TOL_BF16
    assert rel_max(dW, dW_x) <= TOL_DW_REL
    dQ1, dK1, dV1, dW1 = ops.backward(Q, K, V, dO, D, LSE, W, *args, out_dtype=torch.bfloat16)
    assert max_abs(dQ1, dQ_x) <= TOL_BF16 and max_abs(dK1, dK_x) <= TOL_BF16 and max_abs(dV1, dV_x) <= TOL_BF16
    assert rel_max(dW1, dW_x) <= TOL_DW_REL


def test_one_pass_backward_steps_through_the_c_abi():
    # The three steps of convattn_bwd_fused called one by one on raw pointers (what bench.py
    # times) give exactly what the single call gives, and what the Python op returns.
    import ctypes as C

    from flash_multi_token_attention_amd import _lib
    lib = _lib.load()
    B, H, N, d, c_q, c_k = 2, 2, 300, 128, 6, 11
    Q, K, V, dO, W = (t.to(DEV) for t in rand_case(B, H, N, N, d, c_q, c_k, torch.bfloat16, seed=21))
    sc = scale_of(d)
    O, M, L = ops.forward(Q, K, V, W, sc, c_q - 1, (c_k - 1) // 2, True, out_dtype=torch.bfloat16)
    D, LSE = ops.bwd_preprocess(O, dO, M, L)
    ref = ops.backward(Q, K, V, dO, D, LSE, W, sc, c_q - 1, (c_k - 1) // 2, True, out_dtype=torch.bfloat16)
    desc = _lib.Desc(B, H, N, N, d, c_q, c_k, sc, 1, _lib.BF16, _lib.BF16, 1, 0)
    ws = torch.empty(lib.convattn_bwd_fused_workspace_bytes(C.byref(desc)), dtype=torch.uint8, device=DEV)
    p = lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ins = (p(Q), p(K), p(V), p(dO), p(D), p(LSE), p(W))
    for whole in (True, False):
        dQ, dK, dV = (torch.empty_like(Q) for _ in range(3))
        dW = torch.empty_like(W)
        ws.fill_(0xFF)   # NaN patterns: nothing may depend on the workspace's previous contents
        if whole:
            assert lib.convattn_bwd_fused(C.byref(desc), *ins, p(dQ), p(dK), p(dV), p(dW), p(ws), st) == 0
        else:
            assert lib.convattn_bwd_fused_dkdv(C.byref(desc), *ins, p(dK), p(dV), p(ws), st) == 0
            assert lib.convattn_bwd_fused_dq(C.byref(desc), *ins, p(dQ), p(ws), st) == 0
            assert lib.convattn_bwd_fused_dw(C.byref(desc), p(ws), p(dW), st) == 0
        torch.cuda.synchronize()
        for got, want in zip((dQ, dK, dV, dW), ref):
            assert torch.equal(got, want)


def test_seeded_random_shapes_forward_and_both_backward_paths():
    # Lengths on and around the 32/64/128-row tile borders, both head dims, every tap-slot
    # class of the kernels (<=3, <=6, <=11 query taps), odd key windows up to 15 taps.
    import random
    rng = random.Random(7)
    lengths = [1, 2, 17, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 160, 191, 192, 255, 257, 300,
               383, 385, 450]
    for t in range(24):
        d = rng.choice([64, 128])
        c_q, c_k = rng.randint(1, 11), rng.choice([1, 3, 5, 7, 9, 11, 13, 15])
        causal = rng.random() < 0.6
        Nq = rng.choice(lengths)
        Nk = Nq if causal else rng.choice([Nq, max(1, Nq // 2), Nq + 37, 129])
        B, H = rng.choice([(1, 1), (1, 2), (2, 1)])
        Q, K, V, dO, W = rand_case(B, H, Nq, Nk, d, c_q, c_k, torch.bfloat16, seed=100 + t,
                                   w_mode=rng.choice(["rand", "delta"]))
        O_ref, _, _ = oracle_fwd(Q, K, V, W, causal)
        ref = oracle_bwd(Q, K, V, W, dO, causal)
        g = [x.to(DEV) for x in (Q, K, V, dO, W)]
        case = f"B{B} H{H} Nq{Nq} Nk{Nk} d{d} {c_q}x{c_k} causal={causal}"
        O, _, _ = ops.forward(g[0], g[1], g[2], g[4], scale_of(d), c_q - 1, (c_k - 1) // 2, causal)
        assert max_abs(O, O_ref) <= TOL_BF16, case
        for one_pass in (False, True):
            dQ, dK, dV, dW = _run_bwd(*g, causal, torch.bfloat16, one_pass)
            assert max_abs(dQ, ref[0]) <= TOL_BF16, case
            assert max_abs(dK, ref[1]) <= TOL_BF16, case
            assert max_abs(dV, ref[2]) <= TOL_BF16, case
            assert rel_max(dW, ref[3]) <= TOL_DW_REL, case


@pytest.mark.parametrize("causal", [True, False])
def test_forward_rising_row_maxima_and_wide_score_range(causal):
    # Scores that grow along the keys (the softmax base of every row has to be raised again and
    # again) on top of a wide random range (exponents tens of binary orders apart).
    B, H, N, d, c_q, c_k = 1, 2, 300, 128, 6, 11
    Q, K, V, _, W = rand_case(B, H, N, N, d, c_q, c_k, torch.float32, seed=33)
    u = torch.nn.functional.normalize(torch.randn(d, generator=torch.Generator().manual_seed(1)), dim=0)
    ramp = torch.linspace(0.0, 1.0, N)[None, None, :, None]
    K = (K + 24.0 * ramp * u).to(torch.bfloat16)
    Q = (Q + 5.0 * u).to(torch.bfloat16)
    V = V.to(torch.bfloat16)
    O_ref, M_ref, L_ref = oracle_fwd(Q, K, V, W, causal)
    assert float(M_ref.max() - M_ref.min()) > 8.0   # the case is what it claims to be
    O, M, L = ops.forward(Q.to(DEV), K.to(DEV), V.to(DEV), W.to(DEV), scale_of(d), c_q - 1, (c_k - 1) // 2, causal,
                          out_dtype=torch.bfloat16)
    assert max_abs(O, O_ref) <= TOL_BF16
    assert max_abs(M, M_ref) <= TOL_BF16
    assert rel_max(L, L_ref) <= TOL_BF16
