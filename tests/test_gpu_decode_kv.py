"""Decode over shared KV heads, a paged cache and ragged sequence lengths (convattn_decode_kv)
against the CPU oracle on the gathered dense rows."""
import pytest
import torch

from flash_multi_token_attention_amd.conv_attn import ops
from oracle import conv_attn_oracle as orc
from tests.util import TOL_BF16, max_abs, scale_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(B, H, H_kv, Nk, d, c_q, c_k, seed):
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, c_q, d, generator=g).to(torch.bfloat16)
    K = torch.randn(B, H_kv, Nk, d, generator=g).to(torch.bfloat16)
    V = torch.randn(B, H_kv, Nk, d, generator=g).to(torch.bfloat16)
    W = 0.3 * torch.randn(H, c_q, c_k, generator=g)
    return Q, K, V, W


def _check(out, ref):
    O, M, L = out[:3]
    assert max_abs(O, ref[0]) <= TOL_BF16
    # M + log L is the log-sum-exp of the row: independent of how the keys were split
    assert max_abs(M + torch.log(L), ref[1] + torch.log(ref[2])) <= 2e-2


@pytest.mark.parametrize("H,H_kv,c_q", [(8, 8, 6), (8, 2, 6), (6, 1, 6), (8, 1, 8), (4, 2, 3), (8, 2, 11), (16, 2, 1)])
@pytest.mark.parametrize("causal", [False, True])
def test_gqa_dense_and_cache_view(H, H_kv, c_q, causal):
    # (groups of 4 and 2 query heads share one K / V stream when the window has at most 8 query taps;
    # 11 taps and odd groups run one head per workgroup)
    B, Nk, d, c_k = 2, 700, 128, 11
    Q, K, V, W = _case(B, H, H_kv, Nk, d, c_q, c_k, seed=H * 10 + H_kv + c_q)
    sc = scale_of(d)
    ref = orc.decode_kv(Q.float(), lambda b: K[b].float(), lambda b: V[b].float(), W, [Nk] * B, sc, causal)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    _check(ops.decode_gqa(g[0], g[1], g[2], g[3], 3, sc, causal), ref)
    # the same rows as a view of a longer cache
    cache_k = torch.zeros(B, H_kv, Nk + 100, d, dtype=torch.bfloat16, device=DEV)
    cache_v = torch.zeros_like(cache_k)
    cache_k[:, :, :Nk], cache_v[:, :, :Nk] = g[1], g[2]
    out = ops.decode_gqa(g[0], cache_k[:, :, :Nk], cache_v[:, :, :Nk], g[3], 2, sc, causal)
    _check(out, ref)
    if H == H_kv:
        # one KV head per query head is the plain decode entry, bit for bit
        plain = ops.decode(g[0], g[1], g[2], g[3], 3, sc, causal)
        same = ops.decode_gqa(g[0], g[1], g[2], g[3], 3, sc, causal)
        assert torch.equal(plain[0], same[0]) and torch.equal(plain[1], same[1]) and torch.equal(plain[2], same[2])


@pytest.mark.parametrize("d,page,H,H_kv", [(128, 16, 4, 4), (128, 64, 8, 2), (64, 128, 4, 1), (32, 32, 8, 2)])
@pytest.mark.parametrize("causal", [False, True])
def test_paged_cache_with_ragged_lengths(d, page, H, H_kv, causal):
    B, c_q, c_k = 3, 6, 11
    lens = [1000, 37, 513]
    max_len = max(lens)
    n_seq_pages = (max_len + page - 1) // page
    n_pages = B * n_seq_pages + 5
    g = torch.Generator().manual_seed(d + page + H)
    Q = torch.randn(B, H, c_q, d, generator=g).to(torch.bfloat16)
    k_pool = torch.randn(n_pages, H_kv, page, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(n_pages, H_kv, page, d, generator=g).to(torch.bfloat16)
    W = 0.3 * torch.randn(H, c_q, c_k, generator=g)
    # every sequence gets its own shuffled pages; entries past a sequence's last page are never read
    perm = torch.randperm(n_pages, generator=g)[: B * n_seq_pages].reshape(B, n_seq_pages).to(torch.int32)
    sc = scale_of(d)
    ref = orc.decode_kv(Q.float(), lambda b: orc.gather_paged(k_pool.float(), perm, lens[b], b),
                        lambda b: orc.gather_paged(v_pool.float(), perm, lens[b], b), W, lens, sc, causal)
    out = ops.decode_paged(Q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), perm.to(DEV),
                           torch.tensor(lens, dtype=torch.int32, device=DEV), max_len, W.to(DEV), 2, sc, causal)
    _check(out, ref)
    # without seq_lens every entry has max_len keys (pages of the short sequences exist: the table is full)
    ref_full = orc.decode_kv(Q.float(), lambda b: orc.gather_paged(k_pool.float(), perm, max_len, b),
                             lambda b: orc.gather_paged(v_pool.float(), perm, max_len, b), W, [max_len] * B, sc, causal)
    out_full = ops.decode_paged(Q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), perm.to(DEV), None, max_len, W.to(DEV),
                                4, sc, causal)
    _check(out_full, ref_full)


def test_paged_equals_contiguous_bitwise():
    # pages in order = the dense cache: the paged instance of the kernel returns the dense instance's bits
    B, H, Nk, d, page = 2, 4, 2048, 128, 64
    Q, K, V, W = _case(B, H, H, Nk, d, 6, 11, seed=7)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    sc = scale_of(d)
    n = Nk // page
    k_pool = g[1].reshape(B, H, n, page, d).permute(0, 2, 1, 3, 4).reshape(B * n, H, page, d).contiguous()
    v_pool = g[2].reshape(B, H, n, page, d).permute(0, 2, 1, 3, 4).reshape(B * n, H, page, d).contiguous()
    table = torch.arange(B * n, dtype=torch.int32, device=DEV).reshape(B, n)
    dense = ops.decode(g[0], g[1], g[2], g[3], 4, sc, False)
    paged = ops.decode_paged(g[0], k_pool, v_pool, table, None, Nk, g[3], 4, sc, False)
    for a, b in zip(dense[:3], paged[:3]):
        assert torch.equal(a, b)


def test_kv_layout_rejections():
    B, H, Nk, d = 1, 4, 256, 128
    Q, K, V, W = _case(B, H, H, Nk, d, 6, 11, seed=1)
    g = [t.to(DEV) for t in (Q, K, V, W)]
    sc = scale_of(d)
    with pytest.raises(RuntimeError):   # 3 KV heads do not divide 4 query heads
        ops.decode_gqa(g[0], g[1][:, :3].contiguous(), g[2][:, :3].contiguous(), g[3], 1, sc)
    pool = torch.zeros(8, H, 48, d, dtype=torch.bfloat16, device=DEV)   # page size not a power of two
    table = torch.zeros(B, 8, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError):
        ops.decode_paged(g[0], pool, pool, table, None, 256, g[3], 1, sc)
    pool = torch.zeros(8, H, 64, d, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):   # table too short for max_seq_len
        ops.decode_paged(g[0], pool, pool, table[:, :2].contiguous(), None, 256, g[3], 1, sc)
    with pytest.raises(RuntimeError):   # fp32 runs the fp32-arithmetic decode kernel, which has no KV layouts
        ops.decode_gqa(g[0].float(), g[1].float(), g[2].float(), g[3], 1, sc)
