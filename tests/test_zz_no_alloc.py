"""convattn_decode_noalloc (the decode step with the split partials in the library's own buffer)
against convattn_decode + convattn_decode_combine with caller-allocated partials, through the C ABI."""
import ctypes as C

import pytest
import torch

from flash_multi_token_attention_amd import _lib

pytestmark = pytest.mark.gpu


def _p(t):
    return C.c_void_p(t.data_ptr())


def _case(B, H, r, Nk, d, c_q, c_k, splits, seed):
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn(B, H, r, d, generator=g).to(torch.bfloat16).cuda()
    K = torch.randn(B, H, Nk, d, generator=g).to(torch.bfloat16).cuda()
    V = torch.randn(B, H, Nk, d, generator=g).to(torch.bfloat16).cuda()
    W = 0.05 * torch.randn(H, c_q, c_k, generator=g)
    W[:, c_q - 1, (c_k - 1) // 2] += 1.0
    desc = _lib.Desc(B, H, r, Nk, d, c_q, c_k, d ** -0.5, 0, _lib.BF16, _lib.F32, splits, 0)
    return desc, Q, K, V, W.cuda()


def _both(lib, desc, Q, K, V, W):
    B, H, d, ns, Nk = desc.B, desc.H, desc.d, desc.n_splits, desc.Nk
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    f32 = dict(dtype=torch.float32, device="cuda")
    Op, Mp, Lp = torch.empty(B, H, ns, d, **f32), torch.empty(B, H, ns, **f32), torch.empty(B, H, ns, **f32)
    out = [[torch.empty(B, H, 1, d, **f32), torch.empty(B, H, 1, **f32), torch.empty(B, H, 1, **f32)] for _ in range(2)]
    rc = lib.convattn_decode(C.byref(desc), _p(Q), _p(K), _p(V), _p(W), _p(Op), _p(Mp), _p(Lp), st)
    assert rc == 0, _lib.strerror(rc)
    rc = lib.convattn_decode_combine(C.byref(desc), _p(Op), _p(Mp), _p(Lp), *(_p(t) for t in out[0]), st)
    assert rc == 0, _lib.strerror(rc)
    rc = lib.convattn_decode_noalloc(C.byref(desc), _p(Q), _p(K), _p(V), _p(W), C.c_longlong(H * Nk * d),
                                     C.c_longlong(Nk * d), *(_p(t) for t in out[1]), st)
    assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    return out


def test_decode_noalloc_matches_decode_two_calls_second_smaller():
    lib = _lib.load()
    # two calls in a row on the same buffer, the second with a smaller input: nothing of the first
    # call's partials may leak into the second
    for shape in ((3, 4, 6, 1500, 128, 6, 11, 5, 1), (2, 3, 4, 300, 64, 3, 5, 2, 2)):
        desc, Q, K, V, W = _case(*shape)
        assert 0 < lib.convattn_decode_noalloc_bytes(C.byref(desc)) <= 8 << 20
        ref, got = _both(lib, desc, Q, K, V, W)
        for a, b in zip(ref, got):
            assert torch.equal(a, b)   # same kernels, same order of operations


def test_decode_noalloc_rejects_what_does_not_fit():
    lib = _lib.load()
    # 32 x 32 x 64 splits x 130 floats = 34 MB of partials: more than the built-in 8 MiB
    desc = _lib.Desc(32, 32, 6, 8192, 128, 6, 11, 0.1, 0, _lib.BF16, _lib.F32, 64, 0)
    assert lib.convattn_decode_noalloc_bytes(C.byref(desc)) > 8 << 20
    ok = C.c_void_p(4096)
    rc = lib.convattn_decode_noalloc(C.byref(desc), ok, ok, ok, ok, C.c_longlong(32 * 8192 * 128),
                                     C.c_longlong(8192 * 128), ok, ok, ok, None)
    assert rc == -13 and b"scratch" in lib.convattn_strerror(rc)
