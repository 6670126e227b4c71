"""Decode-time conv-attention: counterpart of the reference's
``fwd_conv_attn_inference`` (conv_attn/flash_conv_attention_inference.py:33-93)."""
from __future__ import annotations

from . import ops
from .ops import forward_inference  # noqa: F401  (re-exported, as the reference module does)


def fwd_conv_attn_inference(Q, K, V, conv_kernel, k_splits, scale, pad_q, pad_k, causal):
    """Last-query-row attention over a KV cache.

    Q [B,H,q_len<=16,d] holds the most recent query rows (the convolution looks
    kernel_size_q-1 rows back; missing rows count as zero rows, which is what
    the reference's front padding to 16 rows amounts to), K, V [B,H,Nk,d].
    Returns O [B,H,1,d], M [B,H,1], L [B,H,1] in fp32, always normalised.
    ``causal=False`` is the reference behaviour (its kernel ignores the flag);
    ``causal=True`` applies the training masks to the resident rows so that the
    result equals the last row of the causal training forward.
    """
    if Q.shape[2] > 16:
        raise ValueError(f"Q sequence length must be <= 16 for inference, got {Q.shape[2]}")
    if conv_kernel.dim() != 3 or pad_q != conv_kernel.shape[1] - 1 or pad_k != (conv_kernel.shape[2] - 1) // 2:
        ops._weights(conv_kernel, Q.shape[1], pad_q, pad_k, Q.device)  # raises, naming what is wrong
    O, M, L, _ = ops.decode(Q, K, V, conv_kernel, k_splits, scale, causal)
    return O, M, L
