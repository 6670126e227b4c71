"""The benchmark configurations at their real shapes, and the corners the small parity cases do not
reach: offsets beyond 2^31 bytes (C4's K / V, C5's dS workspace), two (batch, head) pairs of C3
against the CPU oracle itself, the autograd function's partial-gradient branches, gradients that
stay linear in dO over many orders of magnitude, scores at the fp16 limit of the score tile."""
import pytest
import torch

from flash_multi_token_attention_amd import synthetic
from flash_multi_token_attention_amd.conv_attn import ConvAttentionCUDA, FlashConvAttentionCUDAFunction, ops
from flash_multi_token_attention_amd.conv_attn.inference import fwd_conv_attn_inference
from oracle import conv_attn_oracle as orc
from tests.util import TOL_BF16, TOL_DW_REL, max_abs, oracle_bwd, oracle_fwd, rand_case, rel_max, scale_of

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _fwd_bwd(Q, K, V, dO, W, scale, pq, pk, causal=True):
    O, M, L = ops.forward(Q, K, V, W, scale, pq, pk, causal, out_dtype=torch.bfloat16)
    D, LSE = ops.bwd_preprocess(O, dO, M, L)
    dQ, dK, dV, dW = ops.backward(Q, K, V, dO, D, LSE, W, scale, pq, pk, causal, out_dtype=torch.bfloat16)
    return O, M, L, dQ, dK, dV, dW


def test_c3_two_pairs_against_the_cpu_oracle():
    # two (batch, head) pairs of the headline workload, forward and autograd backward of the oracle on
    # the CPU (N = 4096: 67 MB per N x N temporary), against the same pairs of the full GPU run
    wl = synthetic.WORKLOADS["c3_fwd_bwd"]
    t = synthetic.make_inputs(wl, seed=0)
    g = {k: v.to(DEV) for k, v in t.items()}
    O, M, L, dQ, dK, dV, dW = _fwd_bwd(g["Q"], g["K"], g["V"], g["dO"], g["W"], wl.scale, wl.pad_q, wl.pad_k)
    for b, h in ((0, 0), (3, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        Qc, Kc, Vc, dOc = (t[k][sl].float() for k in ("Q", "K", "V", "dO"))
        Wc = t["W"][h:h + 1]
        O_ref, M_ref, L_ref = orc.forward(Qc, Kc, Vc, Wc, True, wl.scale)
        assert max_abs(O[sl], O_ref) <= TOL_BF16
        assert max_abs(M[sl], M_ref) <= TOL_BF16 and rel_max(L[sl], L_ref) <= TOL_BF16
        ref = orc.backward_autograd(Qc, Kc, Vc, Wc, dOc, True, wl.scale)
        errs = [max_abs(dQ[sl], ref[0]), max_abs(dK[sl], ref[1]), max_abs(dV[sl], ref[2])]
        print(f"C3 pair ({b},{h}) max-abs errors vs oracle: O {max_abs(O[sl], O_ref):.4f} dQ {errs[0]:.4f} "
              f"dK {errs[1]:.4f} dV {errs[2]:.4f}")
        assert max(errs) <= TOL_BF16
    # dW sums over the batch: the oracle's dW of head 0 over all four batches
    ref_w = sum(orc.backward_autograd(*(t[k][b:b + 1, 0:1].float() for k in ("Q", "K", "V")), t["W"][0:1],
                                      t["dO"][b:b + 1, 0:1].float(), True, wl.scale)[3] for b in range(wl.B))
    assert rel_max(dW[0:1], ref_w) <= TOL_DW_REL


def test_c5_real_shape_heads_match_one_head_runs():
    # B=1, H=32, N=16384: the dS workspace of the one-pass backward is 8.6 GB (the causal triangle), its block offsets pass
    # 2^32 elements.  Heads 15 and 31 of the full run must equal a run of that head alone (every
    # (batch, head) is computed independently, in the same order of operations).
    wl = synthetic.WORKLOADS["c5_long"]
    t = {k: v.to(DEV) for k, v in synthetic.make_inputs(wl, seed=0).items()}
    full = _fwd_bwd(t["Q"], t["K"], t["V"], t["dO"], t["W"], wl.scale, wl.pad_q, wl.pad_k)
    O = full[0]
    assert max_abs(O[:, :, 0], t["V"][:, :, 0]) <= 1e-6      # row 0 attends to key 0 only
    assert all(bool(torch.isfinite(x.float()).all()) for x in full)
    for h in (15, 31):
        one = _fwd_bwd(*(t[k][:, h:h + 1].contiguous() for k in ("Q", "K", "V", "dO")), t["W"][h:h + 1].contiguous(),
                       wl.scale, wl.pad_q, wl.pad_k)
        for name, a, b in zip(("O", "M", "L", "dQ", "dK", "dV"), full[:6], one[:6]):
            assert torch.equal(a[:, h:h + 1], b), f"{name} of head {h}"
        assert torch.equal(full[6][h:h + 1], one[6])         # dW: B = 1, one partial order
    del full, one
    torch.cuda.empty_cache()


def test_c5_one_head_against_the_cpu_oracle():
    # one head of the long-context workload (N = 16384) against the oracle's forward and autograd backward
    # on the CPU (1 GB per N x N temporary), the GPU side run on that head alone (bit-equal to the head
    # inside the full run: test above)
    wl = synthetic.WORKLOADS["c5_long"]
    t = synthetic.make_inputs(wl, seed=0)
    h = 31
    Qc, Kc, Vc, dOc = (t[k][:, h:h + 1].contiguous() for k in ("Q", "K", "V", "dO"))
    Wc = t["W"][h:h + 1].contiguous()
    O, M, L, dQ, dK, dV, dW = _fwd_bwd(*(x.to(DEV) for x in (Qc, Kc, Vc, dOc, Wc)), wl.scale, wl.pad_q, wl.pad_k)
    O_ref, M_ref, L_ref = orc.forward_chunked(Qc.float(), Kc.float(), Vc.float(), Wc, True, wl.scale, rows=2048)
    assert max_abs(O, O_ref) <= TOL_BF16
    assert max_abs(M, M_ref) <= TOL_BF16 and rel_max(L, L_ref) <= TOL_BF16
    ref = orc.backward_autograd(Qc.float(), Kc.float(), Vc.float(), Wc, dOc.float(), True, wl.scale)
    errs = [max_abs(dQ, ref[0]), max_abs(dK, ref[1]), max_abs(dV, ref[2])]
    print(f"C5 head {h} max-abs errors vs oracle: O {max_abs(O, O_ref):.4f} dQ {errs[0]:.4f} dK {errs[1]:.4f} "
          f"dV {errs[2]:.4f} dW rel {rel_max(dW, ref[3]):.4f}")
    assert max(errs) <= TOL_BF16
    assert rel_max(dW, ref[3]) <= TOL_DW_REL


def test_c2_one_pair_against_the_cpu_oracle():
    # one (batch, head) pair of the forward-only workload (N = 2048, d = 64) inside the full run
    wl = synthetic.WORKLOADS["c2_fwd"]
    t = synthetic.make_inputs(wl, seed=0)
    g = {k: v.to(DEV) for k, v in t.items()}
    O, M, L = ops.forward(g["Q"], g["K"], g["V"], g["W"], wl.scale, wl.pad_q, wl.pad_k, True, out_dtype=torch.bfloat16)
    for b, h in ((0, 0), (3, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        O_ref, M_ref, L_ref = orc.forward(*(t[k][sl].float() for k in ("Q", "K", "V")), t["W"][h:h + 1], True, wl.scale)
        assert max_abs(O[sl], O_ref) <= TOL_BF16
        assert max_abs(M[sl], M_ref) <= TOL_BF16 and rel_max(L[sl], L_ref) <= TOL_BF16


def test_c4_real_shape_decode():
    # B=32, H=32, Nk=8192: K and V are 2 GiB each (offsets beyond 2^31 bytes)
    wl = synthetic.WORKLOADS["c4_decode"]
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    Q, K, V = mk(wl.B, wl.H, wl.Nq, wl.d), mk(wl.B, wl.H, wl.Nk, wl.d), mk(wl.B, wl.H, wl.Nk, wl.d)
    W = synthetic.conv_weight(wl, torch.randn(wl.H, wl.c_q, wl.c_k, generator=torch.Generator().manual_seed(0))).to(DEV)
    O, M, L = fwd_conv_attn_inference(Q, K, V, W, None, wl.scale, wl.pad_q, wl.pad_k, False)
    for b, h in ((0, 0), (15, 31), (31, 31)):
        O_ref, M_ref, L_ref = orc.decode(Q[b:b + 1, h:h + 1].float().cpu(), K[b:b + 1, h:h + 1].float().cpu(),
                                         V[b:b + 1, h:h + 1].float().cpu(), W[h:h + 1].cpu(), wl.scale)
        assert max_abs(O[b:b + 1, h:h + 1], O_ref) <= TOL_BF16
        assert max_abs(M[b:b + 1, h:h + 1], M_ref) <= TOL_BF16 and rel_max(L[b:b + 1, h:h + 1], L_ref) <= TOL_BF16
    # V = 1 everywhere: every output is 1 (sum of the probabilities), for all 1024 pairs
    O1, _, _ = fwd_conv_attn_inference(Q, K, torch.ones_like(V), W, None, wl.scale, wl.pad_q, wl.pad_k, False)
    assert max_abs(O1, torch.ones_like(O1)) <= 2e-3


@pytest.mark.parametrize("need", ["qw", "kv", "q", "v"])
def test_autograd_function_partial_gradients(need):
    # only some inputs require a gradient: the function runs the dQ + dW pass, the dK / dV pass or
    # the one-pass backward accordingly; every gradient it returns matches the oracle's
    Q, K, V, dO, W = rand_case(2, 2, 200, 200, 128, 6, 11, torch.bfloat16, seed=21)
    ref = oracle_bwd(Q, K, V, W, dO, True)
    q, k, v, w = (t.to(DEV).clone() for t in (Q, K, V, W))
    q.requires_grad_(need in ("qw", "q"))
    w.requires_grad_(need == "qw")
    k.requires_grad_(need == "kv")
    v.requires_grad_(need in ("kv", "v"))
    O = FlashConvAttentionCUDAFunction.apply(q, k, v, w, scale_of(128), 5, 5, True)
    O.backward(dO.to(DEV))
    for name, t, r, wanted in (("dQ", q, ref[0], need in ("qw", "q")), ("dK", k, ref[1], need == "kv"),
                               ("dV", v, ref[2], need in ("kv", "v")), ("dW", w, ref[3], need == "qw")):
        if not wanted:
            assert t.grad is None, name
        elif name == "dW":
            assert rel_max(t.grad, r) <= TOL_DW_REL
        else:
            assert max_abs(t.grad, r) <= TOL_BF16, name


@pytest.mark.parametrize("factor", [2.0 ** -20, 2.0 ** -10, 2.0 ** 10])
@pytest.mark.parametrize("mode", ["one_pass", "two_pass", "low_memory"])
@pytest.mark.parametrize("c_q", [6, 11])
def test_backward_is_linear_in_dO_over_many_orders_of_magnitude(factor, mode, c_q):
    # dC is carried as fp16 times a power of two chosen from the magnitude of the upstream gradient:
    # gradients of dO * factor are factor times the gradients of dO, to the same tolerance as at
    # factor 1 (a mean loss over many tokens in bf16 training gives dO of 1e-6 and less).  Windows of
    # up to 6 query taps run the key-stationary kernel, wider ones and the low-memory dQ pass the
    # kernels with the score tiles in LDS.
    Q, K, V, dO, W = rand_case(2, 2, 300, 300, 128, c_q, 11, torch.bfloat16, seed=5)
    ref = oracle_bwd(Q, K, V, W, dO, True)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    sc, pq, pk = scale_of(128), c_q - 1, 5
    O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, pq, pk, True, out_dtype=torch.bfloat16)
    dOs = (g[3].float() * factor).to(torch.bfloat16)     # a power of two: exact in bf16
    D, LSE = ops.bwd_preprocess(O, dOs, M, L)
    if mode == "one_pass":
        dQ, dK, dV, dW = ops.backward(g[0], g[1], g[2], dOs, D, LSE, g[4], sc, pq, pk, True, out_dtype=torch.float32)
    else:
        dQ, dW = ops.dq_backward(g[0], g[1], g[2], dOs, D, LSE, g[4], sc, pq, pk, True, out_dtype=torch.float32,
                                 low_memory=(mode == "low_memory"))
        dK, dV = ops.dkdv_backward(g[0], g[1], g[2], dOs, D, LSE, g[4], sc, pq, pk, True, out_dtype=torch.float32)
    assert max_abs(dQ / factor, ref[0]) <= TOL_BF16
    assert max_abs(dK / factor, ref[1]) <= TOL_BF16
    assert max_abs(dV / factor, ref[2]) <= TOL_BF16
    assert rel_max(dW / factor, ref[3]) <= TOL_DW_REL


def test_scores_at_the_fp16_limit_of_the_score_tile_stay_finite():
    # raw q.k beyond +-65504 is clamped in the fp16 score tile (the reference keeps fp32 scores): the
    # outputs and gradients stay finite, and rows whose scores are far from the limit are unaffected
    Q, K, V, dO, W = rand_case(1, 2, 128, 128, 128, 6, 11, torch.bfloat16, seed=9)
    Qb = Q.clone()
    Qb[:, :, 100] = 60.0     # q.k up to ~ 60 * 128 * |k| for the rows that see row 100
    Kb = K.clone()
    Kb[:, :, 90] = 30.0      # 60 * 30 * 128 = 230400 > 65504
    g = [t.to(DEV) for t in (Qb, Kb, V, dO, W)]
    out = _fwd_bwd(*g, scale_of(128), 5, 5)
    assert all(bool(torch.isfinite(x.float()).all()) for x in out)
    # rows before key 90 enters any window (row < 90) never see the large score
    O_ref, _, _ = oracle_fwd(Qb, Kb, V, W, True)
    assert max_abs(out[0][:, :, :90], O_ref[:, :, :90]) <= TOL_BF16


def test_backward_falls_back_to_the_two_passes_when_the_workspace_is_capped(monkeypatch):
    # the one-pass backward's workspace is O(N^2); beyond the cap the two passes with O(N) scratch run
    Q, K, V, dO, W = rand_case(1, 2, 260, 260, 128, 6, 11, torch.bfloat16, seed=4)
    ref = oracle_bwd(Q, K, V, W, dO, True)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    sc = scale_of(128)
    O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, 5, 5, True, out_dtype=torch.bfloat16)
    D, LSE = ops.bwd_preprocess(O, g[3], M, L)
    monkeypatch.setenv("CONVATTN_MAX_WORKSPACE_BYTES", "1024")
    dQ, dK, dV, dW = ops.backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True, out_dtype=torch.float32)
    assert max_abs(dQ, ref[0]) <= TOL_BF16 and max_abs(dK, ref[1]) <= TOL_BF16 and max_abs(dV, ref[2]) <= TOL_BF16
    assert rel_max(dW, ref[3]) <= TOL_DW_REL
    # the low-memory dQ + dW pass asks for O(N) scratch only
    import ctypes as C
    from flash_multi_token_attention_amd import _lib
    d_fast = ops._desc(g[0], g[1], g[4], sc, True, torch.float32)
    d_low = ops._desc(g[0], g[1], g[4], sc, True, torch.float32, low_memory=True)
    lib = _lib.load()
    assert lib.convattn_dw_partial_bytes(C.byref(d_low)) < lib.convattn_dw_partial_bytes(C.byref(d_fast)) // 8


def test_dq_backward_falls_back_to_linear_scratch_when_the_workspace_is_capped(monkeypatch):
    # the dQ + dW op alone (what the autograd function calls when only Q or the window needs a gradient):
    # its fast path needs the O(N^2) dS scratch; above the cap it must run with O(N) scratch instead
    Q, K, V, dO, W = rand_case(1, 2, 260, 260, 128, 6, 11, torch.bfloat16, seed=6)
    ref = oracle_bwd(Q, K, V, W, dO, True)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    sc = scale_of(128)
    O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, 5, 5, True, out_dtype=torch.bfloat16)
    D, LSE = ops.bwd_preprocess(O, g[3], M, L)
    fast = ops.dq_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True, out_dtype=torch.float32)
    monkeypatch.setenv("CONVATTN_MAX_WORKSPACE_BYTES", "1024")
    asked = []
    real_empty = torch.empty
    monkeypatch.setattr(torch, "empty", lambda *a, **k: (asked.append(a[0]) or real_empty(*a, **k)))
    dQ, dW = ops.dq_backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True, out_dtype=torch.float32)
    monkeypatch.undo()
    flat = [a for a in asked if isinstance(a, int)]
    assert flat and max(flat) * 4 < 2 * 260 * 260 * 2      # no allocation the size of the dS matrix
    assert max_abs(dQ, ref[0]) <= TOL_BF16 and rel_max(dW, ref[3]) <= TOL_DW_REL
    assert max_abs(dQ, fast[0]) <= TOL_BF16 and rel_max(dW, fast[1]) <= TOL_DW_REL


@pytest.mark.gpu
def test_backward_runs_by_groups_of_heads_when_the_workspace_is_capped(monkeypatch):
    # a cap that one (batch, head) pair fits but the whole problem does not: the one-pass backward
    # runs per group of heads; dQ, dK, dV are those of the single call, dW is summed over the batch
    Q, K, V, dO, W = rand_case(2, 3, 300, 300, 128, 6, 11, torch.bfloat16, seed=5)
    g = [t.to(DEV) for t in (Q, K, V, dO, W)]
    sc = scale_of(128)
    O, M, L = ops.forward(g[0], g[1], g[2], g[4], sc, 5, 5, True, out_dtype=torch.bfloat16)
    D, LSE = ops.bwd_preprocess(O, g[3], M, L)
    whole = ops.backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True, out_dtype=torch.float32)
    import ctypes as C
    from flash_multi_token_attention_amd import _lib
    desc = ops._desc(g[0], g[1], g[4], sc, True, torch.float32)
    nbytes = _lib.load().convattn_bwd_fused_workspace_bytes(C.byref(desc))
    monkeypatch.setenv("CONVATTN_MAX_WORKSPACE_BYTES", str(nbytes // 6 * 2 + 4096))   # two heads of one batch entry
    parts = ops.backward(g[0], g[1], g[2], g[3], D, LSE, g[4], sc, 5, 5, True, out_dtype=torch.float32)
    for a, b in zip(whole[:3], parts[:3]):
        assert torch.equal(a, b)
    assert rel_max(parts[3], whole[3]) <= 1e-5
