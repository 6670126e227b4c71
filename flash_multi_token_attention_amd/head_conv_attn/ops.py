"""Op layer of head-mixing attention: the three functions the reference's Triton wrappers expose
(``head_conv_attention_forward``, head_conv_attn/fwd_kernel.py:270-365;
``head_conv_attention_bwd_dq_dw``, bwd_dq_dw.py:373-470; ``head_conv_attention_bwd_dkdv``,
bwd_dk_dv.py:407-500), same arguments and results, calling the C ABI of libconvattn_hip.so.

Python owns every allocation; launches go on torch's current stream.  Inputs are bfloat16 (float16
and float32 inputs are converted to bfloat16 first: the kernels widen bf16 to fp32 operands); the
mixing matrix is used at fp32 precision whatever dtype it arrives in; O comes back in the dtype of
q, L and M and all gradients in float32, as in the reference.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional, Tuple

import torch

from .. import _lib


def _ptr(t: torch.Tensor):
    return C.c_void_p(t.data_ptr())


def _stream(t: torch.Tensor):
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(t.get_device()))


def _bf16(t: torch.Tensor, name: str) -> torch.Tensor:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if t.dim() != 4:
        raise RuntimeError(f"{name} must be [batch, heads, seq_len, d_model]")
    return t.to(torch.bfloat16).contiguous()


def _desc(q: torch.Tensor, w: torch.Tensor, scale: float, causal: bool, out_dtype: torch.dtype):
    B, H, N, d = q.shape
    if tuple(w.shape) != (H, H):
        raise RuntimeError(f"w must be [heads_out, heads_in] = [{H}, {H}], got {tuple(w.shape)}")
    desc = _lib.HeadmixDesc(B, H, N, d, float(scale), int(bool(causal)), _lib.BF16,
                            _lib.BF16 if out_dtype == torch.bfloat16 else _lib.F32)
    rc = _lib.load().convattn_headmix_validate(C.byref(desc))
    if rc:
        if H not in (16, 32):
            raise AssertionError(f"n_heads must be 16 or 32, got {H}")          # fwd_kernel.py:289
        if d > 128:
            raise AssertionError("d_model must be <= 128")                       # fwd_kernel.py:302
        _lib.check(rc, "head_conv_attention")
    return desc


def forward(q, k, v, w, scale: float = 1.0, causal: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(O, L, M): O [B,H,N,d] in q's dtype, L = sum_j exp(Z - M) and M = max_j Z, float32 [B,H,N]."""
    out_dtype = torch.bfloat16 if q.dtype == torch.bfloat16 else torch.float32
    qb, kb, vb = _bf16(q, "q"), _bf16(k, "k"), _bf16(v, "v")
    if kb.shape != qb.shape or vb.shape != qb.shape:
        raise RuntimeError("q, k and v must have the same shape")
    wf = w.detach().to(torch.float32).contiguous()
    desc = _desc(qb, wf, scale, causal, out_dtype)
    B, H, N, d = qb.shape
    o = torch.empty(B, H, N, d, dtype=out_dtype, device=q.device)
    l = torch.empty(B, H, N, dtype=torch.float32, device=q.device)
    m = torch.empty_like(l)
    rc = _lib.load().convattn_headmix_fwd(C.byref(desc), _ptr(qb), _ptr(kb), _ptr(vb), _ptr(wf), _ptr(o), _ptr(l),
                                          _ptr(m), _stream(q))
    _lib.check(rc, "head_conv_attention_forward")
    return (o if out_dtype == q.dtype else o.to(q.dtype)), l, m


def _backward(entry: str, q, k, v, w, o, do, l, m, causal: bool, scale: Optional[float]):
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    qb, kb, vb, gb = _bf16(q, "q"), _bf16(k, "k"), _bf16(v, "v"), _bf16(do, "do")
    out_dtype = torch.bfloat16 if o.dtype == torch.bfloat16 else torch.float32
    ob = o.to(out_dtype).contiguous()
    wf = w.detach().to(torch.float32).contiguous()
    desc = _desc(qb, wf, scale, causal, out_dtype)
    lf, mf = l.to(torch.float32).contiguous(), m.to(torch.float32).contiguous()
    lib = _lib.load()
    ws = torch.empty(lib.convattn_headmix_bwd_workspace_bytes(C.byref(desc)), dtype=torch.uint8, device=q.device)
    B, H, N, d = qb.shape
    if entry == "dq_dw":
        g0 = torch.empty(B, H, N, d, dtype=torch.float32, device=q.device)
        g1 = torch.empty(H, H, dtype=torch.float32, device=q.device)
        fn = lib.convattn_headmix_bwd_dq_dw
    else:
        g0 = torch.empty(B, H, N, d, dtype=torch.float32, device=q.device)
        g1 = torch.empty_like(g0)
        fn = lib.convattn_headmix_bwd_dkdv
    rc = fn(C.byref(desc), _ptr(qb), _ptr(kb), _ptr(vb), _ptr(wf), _ptr(ob), _ptr(gb), _ptr(lf), _ptr(mf), _ptr(ws),
            _ptr(g0), _ptr(g1), _stream(q))
    _lib.check(rc, "head_conv_attention_bwd_" + entry)
    return g0, g1


def bwd_dq_dw(q, k, v, w, o, do, l, m, causal: bool = False, scale: Optional[float] = None):
    """(dQ [B,H,N,d], dW [H,H]), float32."""
    return _backward("dq_dw", q, k, v, w, o, do, l, m, causal, scale)


def bwd_dkdv(q, k, v, w, o, do, l, m, causal: bool = False, scale: Optional[float] = None):
    """(dK, dV) [B,H,N,d], float32."""
    return _backward("dkdv", q, k, v, w, o, do, l, m, causal, scale)
