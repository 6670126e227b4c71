"""Host-only checks of the C ABI: the library loads without a GPU, exports every
symbol include/convattn.h declares, and rejects bad descriptors with the
documented status codes before touching the device."""
import ctypes as C
import os
import re

import pytest
import torch

from flash_multi_token_attention_amd import _lib
from flash_multi_token_attention_amd.conv_attn import ops, fwd_conv_attn_inference, ConvAttentionCUDA

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from flash_multi_token_attention_amd import build
        build.build(verbose=False)
    return _lib.load()


def desc(**kw):
    base = dict(B=2, H=4, Nq=128, Nk=128, d=64, c_q=6, c_k=11, scale=0.125, causal=1,
                in_dtype=_lib.BF16, out_dtype=_lib.BF16, n_splits=1, flags=0)
    base.update(kw)
    return _lib.Desc(**base)


def test_header_symbols_are_exported(lib):
    text = open(os.path.join(ROOT, "include", "convattn.h")).read()
    declared = set(re.findall(r"^(?:int|size_t|const char \*)\s*(convattn_[a-z_]+)\s*\(", text, re.M))
    assert declared, "no declarations parsed"
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.convattn_version() == 300


def test_desc_layout_matches_header():
    # 7 int32, float, 4 int32, uint32 -> 13 * 4 bytes, no padding
    assert C.sizeof(_lib.Desc) == 52


@pytest.mark.parametrize("kw,op,code", [
    (dict(), _lib.OP_FWD, 0),
    (dict(), _lib.OP_BWD, 0),
    (dict(B=0), _lib.OP_FWD, -2),
    (dict(Nk=-1), _lib.OP_FWD, -2),
    (dict(d=60), _lib.OP_FWD, -3),
    (dict(d=256), _lib.OP_FWD, -3),
    (dict(c_k=10), _lib.OP_FWD, -4),
    (dict(c_q=17), _lib.OP_FWD, -4),
    (dict(c_k=35), _lib.OP_BWD, -4),
    (dict(in_dtype=7), _lib.OP_FWD, -5),
    (dict(out_dtype=-1), _lib.OP_BWD, -5),
    (dict(scale=float("nan")), _lib.OP_FWD, -9),
    (dict(Nq=64), _lib.OP_FWD, -10),
    (dict(Nq=64, causal=0), _lib.OP_FWD, 0),
    (dict(Nq=6, Nk=8192, causal=0, n_splits=4), _lib.OP_DECODE, 0),
    (dict(Nq=17, Nk=8192, causal=0), _lib.OP_DECODE, -8),
    (dict(Nq=6, Nk=8192, causal=0, n_splits=0), _lib.OP_DECODE, -7),
    (dict(Nq=6, Nk=100, causal=0, n_splits=101), _lib.OP_DECODE, -7),
    (dict(Nq=6, Nk=8192, causal=0, n_splits=2000), _lib.OP_DECODE, -7),
    (dict(B=70000), _lib.OP_FWD, -12),
])
def test_validate_codes(lib, kw, op, code):
    assert lib.convattn_validate(C.byref(desc(**kw)), op) == code


def test_null_and_misaligned_pointers_rejected_before_launch(lib):
    d = desc()
    null = C.c_void_p(0)
    ok = C.c_void_p(4096)
    odd = C.c_void_p(4100)
    assert lib.convattn_fwd(C.byref(d), null, ok, ok, ok, ok, ok, ok, null) == -1
    assert lib.convattn_fwd(C.byref(d), ok, ok, odd, ok, ok, ok, ok, null) == -6
    assert lib.convattn_bwd_dkdv(C.byref(d), ok, ok, ok, ok, ok, ok, ok, ok, null, null) == -1
    assert lib.convattn_validate(None, 0) == -1
    # strided decode: heads closer together than Nk*d, or strides that break the 16-byte alignment
    dd = desc(Nq=6, causal=0, n_splits=2)
    LL = C.c_longlong
    dense_h = dd.Nk * dd.d
    assert lib.convattn_decode_strided(C.byref(dd), ok, ok, ok, ok, LL(dense_h * dd.H), LL(dense_h - 8), ok, ok, ok, null) == -2
    assert lib.convattn_decode_strided(C.byref(dd), ok, ok, ok, ok, LL(dense_h * dd.H), LL(dense_h + 4), ok, ok, ok, null) == -2
    assert lib.convattn_decode_strided(C.byref(dd), null, ok, ok, ok, LL(dense_h * dd.H), LL(dense_h), ok, ok, ok, null) == -1
    assert lib.convattn_dw_partial_bytes(C.byref(desc(d=3))) == 0
    assert lib.convattn_decode_partial_bytes(C.byref(desc(Nq=6, causal=0, n_splits=8))) == 2 * 4 * 8 * 64 * 4


def test_strerror_texts(lib):
    assert "kernel size" in _lib.strerror(-4)
    assert "head dimension" in _lib.strerror(-3)
    assert "between 1 and 16" in _lib.strerror(-8)
    assert _lib.strerror(0) == "ok"
    assert _lib.strerror(-999) == "unknown convattn status"


def test_dw_partial_size_matches_tiling(lib):
    n = lib.convattn_dw_partial_bytes(C.byref(desc(in_dtype=_lib.F32)))
    assert n > 0 and n % (2 * 4 * 66 * 4) == 0


def test_fused_backward_workspace_size(lib):
    # bf16, N = 128, d = 64, 6 query taps: dS blocks of 32 rows x 32 keys bf16, ceil((128 + 8) / 128) * 4 = 8 key tiles x
    # ceil(128 / 32) = 4 row tiles per (batch, head) without a mask; under the causal mask key tile kt keeps the row
    # tiles from kt - 1 on: 4 + 4 + 3 + 2 + 1 = 14 blocks.  Then one dW partial per 128-key workgroup, then
    # {scale, log2 scale} of dC and 32 x 2 partial maxima per (batch, head); each part 256-aligned
    tail = (2 * 4 * 2 * 66 * 4 + 255) // 256 * 256 + (2 * 4 * 66 * 4 + 255) // 256 * 256
    assert lib.convattn_bwd_fused_workspace_bytes(C.byref(desc(causal=0))) == 2 * 4 * 8 * 4 * 32 * 32 * 2 + tail
    assert lib.convattn_bwd_fused_workspace_bytes(C.byref(desc())) == 2 * 4 * 14 * 32 * 32 * 2 + tail
    # (N = 4096: 128 + sum(128 .. 1) = 8384 of 132 x 128 = 16896 blocks)
    big = desc(B=1, H=1, Nq=4096, Nk=4096)
    tail_big = (33 * 66 * 4 + 255) // 256 * 256 + (66 * 4 + 255) // 256 * 256   # 33 workgroups of 128 keys
    assert lib.convattn_bwd_fused_workspace_bytes(C.byref(big)) == 8384 * 32 * 32 * 2 + tail_big
    # 8 query taps: the same layout (88 taps per dW partial), also for 9 to 11 query taps
    n = lib.convattn_bwd_fused_workspace_bytes(C.byref(desc(c_q=8)))
    assert n == 2 * 4 * 14 * 32 * 32 * 2 + (2 * 4 * 2 * 88 * 4 + 255) // 256 * 256 + (2 * 4 * 66 * 4 + 255) // 256 * 256
    n = lib.convattn_bwd_fused_workspace_bytes(C.byref(desc(c_q=9)))
    assert n == 2 * 4 * 14 * 32 * 32 * 2 + (2 * 4 * 2 * 99 * 4 + 255) // 256 * 256 + (2 * 4 * 66 * 4 + 255) // 256 * 256
    # fp32 inputs run the two fp32 passes: the workspace is only the dW partial buffer
    f32 = desc(in_dtype=_lib.F32, out_dtype=_lib.F32)
    assert lib.convattn_bwd_fused_workspace_bytes(C.byref(f32)) == lib.convattn_dw_partial_bytes(C.byref(f32))
    assert lib.convattn_bwd_fused_workspace_bytes(C.byref(desc(d=3))) == 0
    ok = C.c_void_p(4096)
    assert lib.convattn_bwd_fused(C.byref(desc()), ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, None, None) == -1


def test_python_shim_errors_without_gpu():
    Q = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16)
    W = torch.zeros(2, 3, 3)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ops.forward(Q, Q, Q, W, 0.125, 2, 1, True)
    with pytest.raises(ValueError, match="<= 16"):
        fwd_conv_attn_inference(torch.zeros(1, 2, 17, 64), Q, Q, W, 1, 0.125, 2, 1, False)
    with pytest.raises(RuntimeError, match="k_splits must be positive"):
        ops.forward_inference(Q, Q, Q, W, 0, 0.125, 2, 1, False, 1)


def test_module_state_dict_and_init_modes():
    m = ConvAttentionCUDA(4, 6, 11, init_random=False)
    assert list(m.state_dict()) == ["conv_weight"]
    assert m.conv_weight.shape == (4, 6, 11)
    w = m.conv_weight.detach()
    assert w.sum() == 4 and (w[:, 5, 5] == 1).all()
    f = ConvAttentionCUDA(2, 3, 5, init_random=False, init_first=True).conv_weight.detach()
    assert f.sum() == 2 and (f[:, 0, 0] == 1).all()
    torch.manual_seed(0)
    r = ConvAttentionCUDA(8, 7, 7).conv_weight.detach()
    assert 0.1 < float(r.std()) < 0.3
    m2 = ConvAttentionCUDA(4, 6, 11)
    m2.load_state_dict(m.state_dict())
    assert torch.equal(m2.conv_weight, m.conv_weight)


def test_drop_in_import_path():
    import flash_multi_token_attention as ref_name
    import flash_multi_token_attention.conv_attn as ca
    assert ref_name.FlashConvAttention is ConvAttentionCUDA
    for name in ("FlashConvAttention", "FlashConvAttentionFunction", "forward", "dq_backward",
                 "dkdv_backward", "fwd_conv_attn", "dq_bwd_conv_attn", "dkdv_bwd_conv_attn"):
        assert hasattr(ca, name)


def test_kernel_path_selection(lib):
    # 1 = bf16 MFMA kernels, 0 = fp32-arithmetic kernels
    assert lib.convattn_kernel_path(C.byref(desc()), _lib.OP_FWD) == 1
    assert lib.convattn_kernel_path(C.byref(desc()), _lib.OP_BWD) == 1
    assert lib.convattn_kernel_path(C.byref(desc(in_dtype=_lib.F32, out_dtype=_lib.F32)), _lib.OP_FWD) == 0
    assert lib.convattn_kernel_path(C.byref(desc(flags=_lib.FLAG_EXACT)), _lib.OP_FWD) == 0
    assert lib.convattn_kernel_path(C.byref(desc(c_k=17)), _lib.OP_FWD) == 1
    assert lib.convattn_kernel_path(C.byref(desc(c_k=17)), _lib.OP_BWD) == 0   # backward: c_k <= 15
    assert lib.convattn_kernel_path(C.byref(desc(c_k=19)), _lib.OP_FWD) == 0
    # the forward addresses K / V of one (batch, head) with 32-bit byte offsets
    big = 1 << 24
    assert lib.convattn_kernel_path(C.byref(desc(Nq=big, Nk=big, d=64)), _lib.OP_FWD) == 0
    assert lib.convattn_kernel_path(C.byref(desc(Nq=big - 64, Nk=big - 64, d=64)), _lib.OP_FWD) == 0
    # ... and puts its row tiles (88 rows at the least) on the grid's z dimension: at most 65535 of them
    assert lib.convattn_kernel_path(C.byref(desc(Nq=65535 * 88, Nk=65535 * 88, d=64)), _lib.OP_FWD) == 1
    assert lib.convattn_kernel_path(C.byref(desc(Nq=65535 * 88 + 1, Nk=65535 * 88 + 1, d=64)), _lib.OP_FWD) == 0
    # the backward kernels' tiles are 128 rows or keys
    assert lib.convattn_kernel_path(C.byref(desc(Nq=65535 * 128 - 16, Nk=65535 * 128 - 16, d=64)), _lib.OP_BWD) == 1
    assert lib.convattn_kernel_path(C.byref(desc(Nq=65535 * 128, Nk=65535 * 128, d=64)), _lib.OP_BWD) == 0


def test_benchmark_tables_parse_and_plot(tmp_path):
    # the sweep tables committed under profiles/ are what `benchmarks plot` draws the reference's figures from
    import os
    from flash_multi_token_attention_amd import benchmarks
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    train, decode = os.path.join(root, "profiles", "sweep_train.md"), os.path.join(root, "profiles", "sweep_decode.md")
    rows = benchmarks.parse_table(train)
    assert len(rows) == len(benchmarks.TRAIN_SWEEP) and {"N", "window", "conv fwd", "sdpa fwd+bwd"} <= set(rows[0])
    assert all(float(r["conv fwd"]) > 0 for r in rows)
    files = benchmarks.plot(train, decode, str(tmp_path))
    # speed-up against plain attention, speed-up against the materialising module (the reference's own
    # figure; its columns come from tests/bench_materialising.py), forward times, backward times, decode
    assert len(files) == 5 and all(os.path.getsize(f) > 10000 for f in files)
    assert any(f.endswith("speedup_vs_materialising.png") for f in files)
    assert float(rows[4]["materialising fwd+bwd"]) > float(rows[4]["conv fwd+bwd"])


def test_kv_layout_rejected_before_launch(lib):
    # convattn_decode_kv checks the layout on the host: nothing below reaches a kernel launch
    dd = desc(Nq=6, causal=0, n_splits=2, H=8, Nk=4096, d=128)
    null, ok = C.c_void_p(0), C.c_void_p(4096)
    row = dd.d

    def call(layout, q=ok):
        return lib.convattn_decode_kv(C.byref(dd), q, ok, ok, C.byref(layout), ok, ok, ok, ok, null)

    dense = dict(H_kv=2, page_size=0, batch_stride=2 * dd.Nk * row, head_stride=dd.Nk * row, page_stride=0,
                 block_table=None, table_stride=0, reserved=0, seq_lens=None)
    assert call(_lib.KvLayout(**dense), q=null) == -1                                  # the layout is fine, q is NULL
    assert call(_lib.KvLayout(**{**dense, "H_kv": 3})) == -14                          # 8 % 3 != 0
    assert call(_lib.KvLayout(**{**dense, "head_stride": dd.Nk * row - 8})) == -14     # KV heads overlap
    assert call(_lib.KvLayout(**{**dense, "reserved": 1})) == -14
    paged = dict(H_kv=2, page_size=64, batch_stride=0, head_stride=64 * row, page_stride=2 * 64 * row,
                 block_table=4096, table_stride=64, reserved=0, seq_lens=None)
    assert call(_lib.KvLayout(**paged), q=null) == -1
    assert call(_lib.KvLayout(**{**paged, "page_size": 48})) == -14                    # not a power of two
    assert call(_lib.KvLayout(**{**paged, "page_size": 8, "head_stride": 8 * row, "page_stride": 16 * row})) == -14
    assert call(_lib.KvLayout(**{**paged, "table_stride": 63})) == -14                 # 63 pages < 4096 keys
    assert call(_lib.KvLayout(**{**paged, "block_table": None})) == -14
    assert call(_lib.KvLayout(**{**paged, "page_stride": 64 * row - 8})) == -14
    # fp32 inputs run the fp32-arithmetic decode kernel, which reads dense K / V only
    dd32 = desc(Nq=6, causal=0, n_splits=2, H=8, Nk=4096, d=128, in_dtype=_lib.F32)
    assert lib.convattn_decode_kv(C.byref(dd32), ok, ok, ok, C.byref(_lib.KvLayout(**dense)), ok, ok, ok, ok, null) == -14
    assert b"KV layout" in lib.convattn_strerror(-14)


def test_headmix_descriptor_checks_and_import_paths(lib):
    # host-only checks of the head-mixing entry points (nothing below reaches a launch)
    def hd(**kw):
        base = dict(B=2, H=16, N=201, d=32, scale=0.17, causal=1, in_dtype=_lib.BF16, out_dtype=_lib.BF16)
        base.update(kw)
        return _lib.HeadmixDesc(**base)

    assert lib.convattn_headmix_validate(C.byref(hd())) == 0
    assert lib.convattn_headmix_validate(C.byref(hd(H=8))) == -15
    assert lib.convattn_headmix_validate(C.byref(hd(d=48))) == -15
    assert lib.convattn_headmix_validate(C.byref(hd(in_dtype=_lib.F32))) == -15
    assert lib.convattn_headmix_validate(C.byref(hd(N=0))) == -2
    assert lib.convattn_headmix_validate(C.byref(hd(scale=float("nan")))) == -9
    assert b"16 or 32" in lib.convattn_strerror(-15)
    # D and LSE of every row, one [H][H] partial per 16-row tile and batch entry
    want = 2 * ((2 * 16 * 201 * 4 + 255) // 256 * 256) + (2 * 13 * 16 * 16 * 4 + 255) // 256 * 256
    assert lib.convattn_headmix_bwd_workspace_bytes(C.byref(hd())) == want
    assert lib.convattn_headmix_bwd_workspace_bytes(C.byref(hd(H=7))) == 0
    null, ok = C.c_void_p(0), C.c_void_p(4096)
    assert lib.convattn_headmix_fwd(C.byref(hd()), ok, ok, null, ok, ok, ok, ok, null) == -1
    assert lib.convattn_headmix_fwd(C.byref(hd()), ok, ok, C.c_void_p(4100), ok, ok, ok, ok, null) == -6
    # the import statements of the reference's head_conv_attn/head_conv_attn.py:6-8 and of its users
    from flash_multi_token_attention.head_conv_attn.fwd_kernel import head_conv_attention_forward  # noqa: F401
    from flash_multi_token_attention.head_conv_attn.bwd_dq_dw import head_conv_attention_bwd_dq_dw  # noqa: F401
    from flash_multi_token_attention.head_conv_attn.bwd_dk_dv import head_conv_attention_bwd_dkdv  # noqa: F401
    from flash_multi_token_attention.head_conv_attn.head_conv_attn import (  # noqa: F401
        HeadConvAttention, HeadConvAttentionFunction, head_conv_attention)
    mod = HeadConvAttention(16, dtype=torch.bfloat16)
    assert tuple(mod.head_conv_weights.shape) == (16, 16) and mod.head_conv_weights.dtype == torch.bfloat16
    assert list(mod.state_dict()) == ["head_conv_weights"]
