"""Op layer of conv-attention: the functions the reference binds with pybind11
(``forward``, ``dq_backward``, ``dkdv_backward`` in conv_attn/bindings.cpp:46-56,
``forward_inference`` in conv_attn/fwd_inference_bindings.cpp:20-23), same
argument order, calling the C ABI of libconvattn_hip.so through ctypes.

Python owns every allocation; launches go on torch's current stream.

Differences from the reference ops, all deliberate:
  * rectangular windows (c_q != c_k) work; the reference dispatches square ones only
  * Q, K, V, dO may be bfloat16 or float32 (float32 runs the fp32-arithmetic kernels)
  * ``conv_kernel`` is used at fp32 precision whatever dtype it arrives in
  * statistics (M, L, D, LSE) are fp32; ``D`` / ``L`` arguments in other dtypes are upcast
  * ``out_dtype`` picks the dtype of O / dQ / dK / dV (default float32, as the reference returns)
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Tuple

import torch

from .. import _lib

_DT = {torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


def _ptr(t: Optional[torch.Tensor]):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream(t: torch.Tensor):
    # (the raw handle of torch's current stream on the tensor's device; torch.cuda.current_stream()
    # builds a Stream object per call, which costs more than the launch it is asked for)
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(t.get_device()))


def _check_input(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _is_cache_view(t: torch.Tensor) -> bool:
    """[B,H,N,d] view of a longer cache: rows of a head dense, heads and batches strided."""
    if t.dim() != 4:
        return False
    B, H, N, d = t.shape
    sb, sh, sn, sd = t.stride()
    return (sd == 1 and sn == d and sh >= N * d and sh % 8 == 0 and sb % 8 == 0
            and (B == 1 or sb >= N * d))


def _check_qkv(Q, K, V, names=("Q", "K", "V"), kv_views=False):
    for t, n in zip((Q, K, V), names):
        if kv_views and t is not Q and t.is_cuda and _is_cache_view(t):
            pass  # decode reads K / V views of a preallocated cache in place
        else:
            _check_input(t, n)
        if t.dim() != 4:
            raise RuntimeError(f"{n} must be [batch, heads, seq_len, d_head]")
    if Q.dtype not in _DT:
        raise RuntimeError("Q must be bfloat16 or float32")
    if K.dtype != Q.dtype or V.dtype != Q.dtype:
        raise RuntimeError("K and V must have the dtype of Q")
    B, H, Nq, d = Q.shape
    if K.shape[0] != B or V.shape[0] != B:
        raise RuntimeError("K batch size must match Q" if K.shape[0] != B else "V batch size must match Q")
    if K.shape[1] != H or V.shape[1] != H:
        raise RuntimeError("K num_heads must match Q" if K.shape[1] != H else "V num_heads must match Q")
    if K.shape[3] != d or V.shape[3] != d:
        raise RuntimeError("K d_head must match Q" if K.shape[3] != d else "V d_head must match Q")
    if V.shape[2] != K.shape[2]:
        raise RuntimeError("V seq_len must match K")
    if Q.device != K.device or Q.device != V.device:
        raise RuntimeError("Q, K and V must be on the same device")


def _weights(conv_kernel: torch.Tensor, H: int, pad_q: int, pad_k: int, device) -> torch.Tensor:
    if conv_kernel.dim() != 3 or conv_kernel.shape[0] != H:
        raise RuntimeError("conv_kernel must be [heads, kernel_size_q, kernel_size_k]")
    c_q, c_k = conv_kernel.shape[1], conv_kernel.shape[2]
    if c_k % 2 == 0:
        raise RuntimeError(f"Unsupported kernel size: {c_q}x{c_k} (kernel_size_k must be odd)")
    if pad_q != c_q - 1 or pad_k != (c_k - 1) // 2:
        raise RuntimeError(
            f"pad_q/pad_k must be kernel_size_q-1 and (kernel_size_k-1)//2 "
            f"(got {pad_q}, {pad_k} for a {c_q}x{c_k} kernel)")
    if not conv_kernel.is_cuda:
        raise RuntimeError("conv_kernel must be a CUDA tensor")
    W = conv_kernel.detach().to(device=device, dtype=torch.float32).contiguous()
    # a slice of a larger parameter (heads h..h') can start off a 16-byte boundary
    return W if W.data_ptr() % 16 == 0 else W.clone()


def _desc(Q, K, W, scale, causal, out_dtype, n_splits=1, exact=False, low_memory=False) -> _lib.Desc:
    if out_dtype not in _DT:
        raise RuntimeError("out_dtype must be bfloat16 or float32")
    B, H, Nq, d = Q.shape
    return _lib.Desc(B, H, Nq, K.shape[2], d, W.shape[1], W.shape[2], float(scale), int(bool(causal)),
                     _DT[Q.dtype], _DT[out_dtype], int(n_splits),
                     (_lib.FLAG_EXACT if exact else 0) | (_lib.FLAG_LOW_MEMORY if low_memory else 0))


def _stat(t: torch.Tensor, name: str, like: torch.Tensor) -> torch.Tensor:
    _check_input(t, name)
    if tuple(t.shape) != tuple(like.shape[:3]):
        raise RuntimeError(f"{name} must be [batch, heads, seq_len]")
    return t if t.dtype == torch.float32 else t.float()


def kernel_path(Q, K, conv_kernel, causal=True, op="fwd", exact=False) -> str:
    """'mfma' or 'fp32': which kernel family a call with these tensors runs."""
    W = conv_kernel
    desc = _desc(Q, K, W, 1.0, causal, Q.dtype if Q.dtype in _DT else torch.float32, exact=exact)
    code = _lib.load().convattn_kernel_path(C.byref(desc), {"fwd": 0, "bwd": 1, "decode": 2}[op])
    _lib.check(min(code, 0), "convattn_kernel_path")
    return "mfma" if code == 1 else "fp32"


def forward(Q, K, V, conv_kernel, scale, pad_q, pad_k, causal, out_dtype=torch.float32,
            exact=False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Training forward -> (O [B,H,N,d], M [B,H,N], L [B,H,N]); M is the row max of
    the convolved scores and L the sum of exp(C - M)."""
    _check_qkv(Q, K, V)
    W = _weights(conv_kernel, Q.shape[1], pad_q, pad_k, Q.device)
    desc = _desc(Q, K, W, scale, causal, out_dtype, exact=exact)
    B, H, Nq, d = Q.shape
    O = torch.empty((B, H, Nq, d), dtype=out_dtype, device=Q.device)
    M = torch.empty((B, H, Nq), dtype=torch.float32, device=Q.device)
    L = torch.empty((B, H, Nq), dtype=torch.float32, device=Q.device)
    rc = _lib.load().convattn_fwd(C.byref(desc), _ptr(Q), _ptr(K), _ptr(V), _ptr(W), _ptr(O), _ptr(M),
                                  _ptr(L), _stream(Q))
    _lib.check(rc, "conv_attn.forward")
    return O, M, L


def bwd_preprocess(O, dO, M, L) -> Tuple[torch.Tensor, torch.Tensor]:
    """(D, LSE) = (rowsum(dO * O), M + log L) in fp32, fused in one kernel."""
    _check_input(O, "O")
    _check_input(dO, "dO")
    B, H, Nq, d = O.shape
    if dO.shape != O.shape:
        raise RuntimeError("dO must have the shape of O")
    if dO.dtype not in _DT or O.dtype not in _DT:
        raise RuntimeError("O and dO must be bfloat16 or float32")
    M = _stat(M, "M", O)
    L = _stat(L, "L", O)
    desc = _lib.Desc(B, H, Nq, Nq, d, 1, 1, 1.0, 0, _DT[dO.dtype], _DT[O.dtype], 1, 0)
    D = torch.empty((B, H, Nq), dtype=torch.float32, device=O.device)
    LSE = torch.empty((B, H, Nq), dtype=torch.float32, device=O.device)
    rc = _lib.load().convattn_bwd_preprocess(C.byref(desc), _ptr(O), _ptr(dO), _ptr(M), _ptr(L),
                                             _ptr(D), _ptr(LSE), _stream(O))
    _lib.check(rc, "conv_attn.bwd_preprocess")
    return D, LSE


def _bwd_common(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal, out_dtype, exact, low_memory=False):
    _check_qkv(Q, K, V)
    _check_input(dO, "dO")
    if dO.shape != Q.shape or dO.dtype != Q.dtype:
        raise RuntimeError("dO must have the shape and dtype of Q")
    W = _weights(conv_kernel, Q.shape[1], pad_q, pad_k, Q.device)
    D = _stat(D, "D", Q)
    L = _stat(L, "L", Q)
    return W, D, L, _desc(Q, K, W, scale, causal, out_dtype, exact=exact, low_memory=low_memory)


def dq_backward(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal,
                out_dtype=torch.float32, exact=False, low_memory=False) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (dQ [B,H,N,d], dconv_kernel [H,c_q,c_k] fp32).  ``L`` is the log-sum-exp
    M + log L and ``D`` is rowsum(dO * O), as the reference passes them.  On the MFMA path the
    scratch of this op holds the bf16 dS matrix (B*H*Nq*Nk*2 bytes, causal: half of that); ``low_memory`` runs the
    slower query-stationary kernel whose scratch is O(N)."""
    W, D, L, desc = _bwd_common(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal,
                                out_dtype, exact, low_memory)
    lib = _lib.load()
    dQ = torch.empty(Q.shape, dtype=out_dtype, device=Q.device)
    nbytes = lib.convattn_dw_partial_bytes(C.byref(desc))
    if nbytes == 0:
        _lib.check(lib.convattn_validate(C.byref(desc), _lib.OP_BWD), "conv_attn.dq_backward")
    # The dS scratch is O(Nq*Nk): above the workspace cap, or when the allocation fails, the
    # query-stationary kernel with O(N) scratch runs instead (same results within the tolerances).
    part = None
    if nbytes <= max_workspace_bytes() or low_memory:
        try:
            part = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=Q.device)
        except torch.OutOfMemoryError:
            if low_memory:
                raise
    if part is None:
        return dq_backward(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal, out_dtype, exact,
                           low_memory=True)
    dW = torch.empty(W.shape, dtype=torch.float32, device=Q.device)
    st = _stream(Q)
    rc = lib.convattn_bwd_dq_dw(C.byref(desc), _ptr(Q), _ptr(K), _ptr(V), _ptr(dO), _ptr(D), _ptr(L),
                                _ptr(W), _ptr(dQ), _ptr(part), st)
    _lib.check(rc, "conv_attn.dq_backward")
    rc = lib.convattn_dw_reduce(C.byref(desc), _ptr(part), _ptr(dW), st)
    _lib.check(rc, "conv_attn.dq_backward (dW reduce)")
    return dQ, dW


def dkdv_backward(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal,
                  out_dtype=torch.float32, exact=False) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (dK, dV) [B,H,N,d]; same arguments as ``dq_backward``."""
    W, D, L, desc = _bwd_common(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal,
                                out_dtype, exact)
    dK = torch.empty(K.shape, dtype=out_dtype, device=Q.device)
    dV = torch.empty(V.shape, dtype=out_dtype, device=Q.device)
    rc = _lib.load().convattn_bwd_dkdv(C.byref(desc), _ptr(Q), _ptr(K), _ptr(V), _ptr(dO), _ptr(D),
                                       _ptr(L), _ptr(W), _ptr(dK), _ptr(dV), _stream(Q))
    _lib.check(rc, "conv_attn.dkdv_backward")
    return dK, dV


def max_workspace_bytes() -> int:
    """Largest workspace ``backward`` allocates in one piece (``CONVATTN_MAX_WORKSPACE_BYTES``,
    default 16 GiB).  Beyond it the one-pass backward runs over groups of heads that fit, and if
    not even one (batch, head) fits, the two separate passes with O(N) scratch run instead."""
    return int(os.environ.get("CONVATTN_MAX_WORKSPACE_BYTES", 16 << 30))


def backward(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal,
             out_dtype=torch.float32, exact=False):
    """-> (dQ, dK, dV, dconv_kernel) from one pass over the score tiles: the results of
    ``dq_backward`` + ``dkdv_backward`` (same arguments) without computing the scores, the
    convolution and dC twice.  Needs a workspace the size of the bf16 dS matrix
    (B*H*Nq*Nk*2 bytes, causal: half of that: 1.1 GB at B4 H16 N4096, 8.6 GB at B1 H32 N16384).  A workspace above
    ``max_workspace_bytes()`` is avoided by running the pass once per group of heads of one batch
    entry (every (batch, head) pair is independent; dconv_kernel is summed over the batch in index
    order); when a single pair does not fit or the allocation fails, the two passes with O(N)
    scratch run instead."""
    W, D, L, desc = _bwd_common(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal,
                                out_dtype, exact)
    lib = _lib.load()
    nbytes = lib.convattn_bwd_fused_workspace_bytes(C.byref(desc))
    if nbytes == 0:
        _lib.check(lib.convattn_validate(C.byref(desc), _lib.OP_BWD), "conv_attn.backward")
    B, H = Q.shape[0], Q.shape[1]
    cap = max_workspace_bytes()
    if nbytes > cap:
        per_pair = -(-nbytes // (B * H))
        group = min(H, int(0.95 * cap) // per_pair)
        if group >= 1:
            group = -(-H // -(-H // group))   # equal groups: H heads in ceil(H / group) launches
            dQ = torch.empty(Q.shape, dtype=out_dtype, device=Q.device)
            dK = torch.empty(K.shape, dtype=out_dtype, device=Q.device)
            dV = torch.empty(V.shape, dtype=out_dtype, device=Q.device)
            dW = torch.zeros(W.shape, dtype=torch.float32, device=Q.device)
            for b in range(B):
                for h0 in range(0, H, group):
                    sl = (slice(b, b + 1), slice(h0, min(H, h0 + group)))
                    gq, gk, gv, gw = backward(Q[sl], K[sl], V[sl], dO[sl], D[sl], L[sl], conv_kernel[sl[1]], scale,
                                              pad_q, pad_k, causal, out_dtype, exact)
                    dQ[sl], dK[sl], dV[sl] = gq, gk, gv
                    dW[sl[1]] += gw
            return dQ, dK, dV, dW
    ws = None
    if nbytes <= cap:
        try:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=Q.device)
        except torch.OutOfMemoryError:
            ws = None
    if ws is None:
        dQ, dW = dq_backward(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal, out_dtype, exact,
                             low_memory=True)
        dK, dV = dkdv_backward(Q, K, V, dO, D, L, conv_kernel, scale, pad_q, pad_k, causal, out_dtype, exact)
        return dQ, dK, dV, dW
    dQ = torch.empty(Q.shape, dtype=out_dtype, device=Q.device)
    dK = torch.empty(K.shape, dtype=out_dtype, device=Q.device)
    dV = torch.empty(V.shape, dtype=out_dtype, device=Q.device)
    dW = torch.empty(W.shape, dtype=torch.float32, device=Q.device)
    rc = lib.convattn_bwd_fused(C.byref(desc), _ptr(Q), _ptr(K), _ptr(V), _ptr(dO), _ptr(D), _ptr(L),
                                _ptr(W), _ptr(dQ), _ptr(dK), _ptr(dV), _ptr(dW), _ptr(ws), _stream(Q))
    _lib.check(rc, "conv_attn.backward")
    return dQ, dK, dV, dW


def default_k_splits(B: int, H: int, Nk: int) -> int:
    """Enough (batch, head, split) workgroups to fill 256 CUs eight times over: where the read
    stream of this machine peaks (a pure non-temporal read stream: 6.6 TB/s with 1024 workgroups
    of 256 threads, 7.2 with 2048, 6.4 with 4096)."""
    want = max(1, (8 * 256 + B * H - 1) // (B * H))
    return max(1, min(want, Nk // 256 if Nk >= 256 else 1, 1024))


def decode(Q, K, V, conv_kernel, k_splits, scale, causal=False, out_dtype=torch.float32,
           exact=False, workspace=None):
    """Decode step -> (O [B,H,1,d], M, L [B,H,1], partials).  Q holds the resident
    last rows (1..16).  ``k_splits`` None/0 picks a split count from the shape.
    K and V may be views ``cache[:, :, :Nk]`` of a cache allocated as [B,H,N_max,d] (same
    strides for both): they are read in place, where the reference's CHECK_CONTIGUOUS
    (conv_attn/kernels/fwd_inference_wrapper.cu:8,26-27) forces a copy per step."""
    _check_qkv(Q, K, V, kv_views=True)
    if K.stride() != V.stride():
        raise RuntimeError("K and V must have the same strides")
    B, H, r, d = Q.shape
    c_q, c_k = conv_kernel.shape[1], conv_kernel.shape[2]
    W = _weights(conv_kernel, H, c_q - 1, (c_k - 1) // 2, Q.device)
    if not k_splits:
        k_splits = default_k_splits(B, H, K.shape[2])
    desc = _desc(Q, K, W, scale, causal, out_dtype, n_splits=k_splits, exact=exact)
    lib = _lib.load()
    if r > 16:
        raise ValueError(f"Q sequence length must be <= 16 for inference, got {r}")
    if not 1 <= k_splits <= 1024:
        # (every other argument is checked by the launch itself; a split count out of range would size the
        # partial buffers first)
        _lib.check(lib.convattn_validate(C.byref(desc), _lib.OP_DECODE), "conv_attn.forward_inference")
    if workspace is None:
        O_part = torch.empty((B, H, k_splits, d), dtype=torch.float32, device=Q.device)
        M_part = torch.empty((B, H, k_splits), dtype=torch.float32, device=Q.device)
        L_part = torch.empty((B, H, k_splits), dtype=torch.float32, device=Q.device)
    else:
        O_part, M_part, L_part = workspace
    O = torch.empty((B, H, 1, d), dtype=out_dtype, device=Q.device)
    M = torch.empty((B, H, 1), dtype=torch.float32, device=Q.device)
    L = torch.empty((B, H, 1), dtype=torch.float32, device=Q.device)
    st = _stream(Q)
    Nk = K.shape[2]
    kv_bs, kv_hs = (H * Nk * d, Nk * d) if K.is_contiguous() else (K.stride(0), K.stride(1))
    rc = lib.convattn_decode_strided(C.byref(desc), _ptr(Q), _ptr(K), _ptr(V), _ptr(W),
                                     C.c_longlong(kv_bs), C.c_longlong(kv_hs),
                                     _ptr(O_part), _ptr(M_part), _ptr(L_part), st)
    _lib.check(rc, "conv_attn.forward_inference")
    rc = lib.convattn_decode_combine(C.byref(desc), _ptr(O_part), _ptr(M_part), _ptr(L_part), _ptr(O),
                                     _ptr(M), _ptr(L), st)
    _lib.check(rc, "conv_attn.forward_inference (combine)")
    return O, M, L, (O_part, M_part, L_part)


def _decode_kv(Q, K, V, layout: "_lib.KvLayout", Nk: int, conv_kernel, k_splits, scale, causal, out_dtype, what: str):
    B, H, r, d = Q.shape
    c_q, c_k = conv_kernel.shape[1], conv_kernel.shape[2]
    W = _weights(conv_kernel, H, c_q - 1, (c_k - 1) // 2, Q.device)
    if not k_splits:
        # a workgroup takes 4 or 2 query heads of one KV head when the window has at most 8 query taps
        group = H // max(1, layout.H_kv or H)
        heads_per_wg = 1 if c_q > 8 else 4 if group % 4 == 0 else 2 if group % 2 == 0 else 1
        k_splits = default_k_splits(B, H // heads_per_wg, Nk)
    if out_dtype not in _DT:
        raise RuntimeError("out_dtype must be bfloat16 or float32")
    desc = _lib.Desc(B, H, r, Nk, d, c_q, c_k, float(scale), int(bool(causal)), _DT[Q.dtype], _DT[out_dtype],
                     int(k_splits), 0)
    lib = _lib.load()
    rc = lib.convattn_validate(C.byref(desc), _lib.OP_DECODE)
    if rc == _lib.ERR_QROWS:
        raise ValueError(f"Q sequence length must be <= 16 for inference, got {r}")
    _lib.check(rc, what)
    O_part = torch.empty((B, H, k_splits, d), dtype=torch.float32, device=Q.device)
    M_part = torch.empty((B, H, k_splits), dtype=torch.float32, device=Q.device)
    L_part = torch.empty((B, H, k_splits), dtype=torch.float32, device=Q.device)
    O = torch.empty((B, H, 1, d), dtype=out_dtype, device=Q.device)
    M = torch.empty((B, H, 1), dtype=torch.float32, device=Q.device)
    L = torch.empty((B, H, 1), dtype=torch.float32, device=Q.device)
    st = _stream(Q)
    _lib.check(lib.convattn_decode_kv(C.byref(desc), _ptr(Q), _ptr(K), _ptr(V), C.byref(layout), _ptr(W),
                                      _ptr(O_part), _ptr(M_part), _ptr(L_part), st), what)
    _lib.check(lib.convattn_decode_combine(C.byref(desc), _ptr(O_part), _ptr(M_part), _ptr(L_part), _ptr(O),
                                           _ptr(M), _ptr(L), st), what + " (combine)")
    return O, M, L, (O_part, M_part, L_part)


def _seq_lens(seq_lens, B: int, device):
    if seq_lens is None:
        return None
    if seq_lens.dtype != torch.int32 or seq_lens.shape != (B,) or not seq_lens.is_cuda or not seq_lens.is_contiguous():
        raise RuntimeError("seq_lens must be a contiguous int32 CUDA tensor [batch]")
    return seq_lens


def decode_gqa(Q, K, V, conv_kernel, k_splits, scale, causal=False, out_dtype=torch.float32, seq_lens=None):
    """Decode step with shared KV heads: Q [B,H,r,d], K and V [B,H_kv,Nk,d] (or views
    ``cache[:, :, :Nk]`` of a longer cache), H a multiple of H_kv; query head h reads KV head
    h // (H // H_kv), the window weights stay per query head.  ``seq_lens`` (int32 [B] on the device,
    each 1..Nk) gives every batch entry its own number of keys.  -> (O [B,H,1,d], M, L, partials).
    bf16 only (the streaming decode kernel)."""
    for t, n in ((Q, "Q"), (K, "K"), (V, "V")):
        if t.dim() != 4:
            raise RuntimeError(f"{n} must be [batch, heads, seq_len, d_head]")
        if not t.is_cuda:
            raise RuntimeError(f"{n} must be a CUDA tensor")
    if not Q.is_contiguous():
        raise RuntimeError("Q must be contiguous")
    if not (K.is_contiguous() or _is_cache_view(K)) or K.stride() != V.stride() or K.shape != V.shape:
        raise RuntimeError("K and V must be [batch, kv_heads, seq_len, d_head] tensors (or views of a longer cache) "
                           "with the same shape and strides")
    B, H, r, d = Q.shape
    H_kv, Nk = K.shape[1], K.shape[2]
    if K.shape[0] != B or K.shape[3] != d or H % H_kv != 0 or K.dtype != Q.dtype:
        raise RuntimeError("K / V must match Q in batch, head dim and dtype, and their head count must divide Q's")
    bs, hs = (H_kv * Nk * d, Nk * d) if K.is_contiguous() else (K.stride(0), K.stride(1))
    sl = _seq_lens(seq_lens, B, Q.device)
    layout = _lib.KvLayout(H_kv, 0, bs, hs, 0, None, 0, 0, _ptr(sl) if sl is not None else None)
    return _decode_kv(Q, K, V, layout, Nk, conv_kernel, k_splits, scale, causal, out_dtype, "conv_attn.decode_gqa")


def decode_paged(Q, k_pool, v_pool, block_table, seq_lens, max_seq_len, conv_kernel, k_splits, scale,
                 causal=False, out_dtype=torch.float32):
    """Decode step over a paged KV cache: pools [n_pages, H_kv, page_size, d] (page_size a power
    of two >= 16), ``block_table`` int32 [B, pages per sequence] on the device (keys
    [i*page_size, (i+1)*page_size) of entry b live in page block_table[b, i]), ``seq_lens`` int32
    [B] on the device or None (then every entry has ``max_seq_len`` keys); ``max_seq_len`` is a host
    integer (no device synchronisation).  H may be a multiple of H_kv.
    -> (O [B,H,1,d], M, L, partials).  bf16 only (the streaming decode kernel)."""
    if k_pool.dim() != 4 or k_pool.shape != v_pool.shape or not k_pool.is_contiguous() or not v_pool.is_contiguous():
        raise RuntimeError("k_pool and v_pool must be contiguous [n_pages, kv_heads, page_size, d_head] tensors of one shape")
    if Q.dim() != 4 or not Q.is_contiguous() or not Q.is_cuda or not k_pool.is_cuda:
        raise RuntimeError("Q must be a contiguous CUDA tensor [batch, heads, rows, d_head]")
    B, H, r, d = Q.shape
    _, H_kv, ps, dk = k_pool.shape
    if dk != d or H % H_kv != 0 or k_pool.dtype != Q.dtype:
        raise RuntimeError("the pools must match Q in head dim and dtype, and their head count must divide Q's")
    if (block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.shape[0] != B
            or not block_table.is_cuda or not block_table.is_contiguous()):
        raise RuntimeError("block_table must be a contiguous int32 CUDA tensor [batch, pages per sequence]")
    if block_table.shape[1] * ps < max_seq_len:
        raise RuntimeError("block_table has fewer pages than max_seq_len needs")
    sl = _seq_lens(seq_lens, B, Q.device)
    layout = _lib.KvLayout(H_kv, ps, 0, ps * d, H_kv * ps * d, _ptr(block_table), block_table.shape[1], 0,
                           _ptr(sl) if sl is not None else None)
    return _decode_kv(Q, k_pool, v_pool, layout, int(max_seq_len), conv_kernel, k_splits, scale, causal, out_dtype,
                      "conv_attn.decode_paged")


def forward_inference(Q, K, V, conv_kernel, k_splits, scale, pad_q, pad_k, causal,
                      num_k_blocks=None):
    """Reference-shaped decode op -> (O [B,H,k_splits,d], M, L [B,H,k_splits]) fp32
    whose slot 0 holds the merged, normalised result (the other slots keep the
    per-split partials).  ``num_k_blocks`` is accepted and ignored: tiling is
    chosen by the kernel."""
    if k_splits is None or k_splits <= 0:
        raise RuntimeError("k_splits must be positive")
    if Q.dim() == 4 and not (0 < Q.shape[2] <= 16):
        raise RuntimeError("Q sequence length must be between 1 and 16 for inference")
    _weights(conv_kernel, Q.shape[1], pad_q, pad_k, Q.device)  # checks pad_q / pad_k
    O, M, L, (O_part, M_part, L_part) = decode(Q, K, V, conv_kernel, k_splits, scale, causal)
    O_part[:, :, 0, :] = O[:, :, 0, :]
    M_part[:, :, 0] = M[:, :, 0]
    L_part[:, :, 0] = L[:, :, 0]
    return O_part, M_part, L_part
