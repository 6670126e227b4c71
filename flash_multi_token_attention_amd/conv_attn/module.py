"""nn.Module and autograd Function of conv-attention, with the constructor
arguments, parameter name and call signatures of the reference's
``ConvAttentionCUDA`` / ``FlashConvAttentionCUDAFunction``
(conv_attn/conv_attention_cuda.py:8-163)."""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from . import ops


class FlashConvAttentionCUDAFunction(torch.autograd.Function):
    """O = conv_attention(Q, K, V, conv_kernel).  bf16 or fp32 inputs (fp32 runs
    the fp32-arithmetic kernels); O and the gradients come back in the input
    dtype, dconv_kernel in the dtype of ``conv_kernel``.  M, L, LSE and D stay
    fp32 between forward and backward."""

    @staticmethod
    def forward(ctx, Q, K, V, conv_kernel, scale, pad_q, pad_k, causal):
        if Q.dtype not in (torch.bfloat16, torch.float32):
            Q = Q.to(torch.bfloat16)
        K = K.to(Q.dtype)
        V = V.to(Q.dtype)
        Q, K, V = Q.contiguous(), K.contiguous(), V.contiguous()
        O, M, L = ops.forward(Q, K, V, conv_kernel, scale, pad_q, pad_k, causal, out_dtype=Q.dtype)
        ctx.save_for_backward(Q, K, V, conv_kernel, M, L, O)
        ctx.scale, ctx.pad_q, ctx.pad_k, ctx.causal = scale, pad_q, pad_k, causal
        return O

    @staticmethod
    def backward(ctx, dO):
        Q, K, V, conv_kernel, M, L, O = ctx.saved_tensors
        dO = dO.to(Q.dtype).contiguous()
        D, LSE = ops.bwd_preprocess(O, dO, M, L)
        args = (Q, K, V, dO, D, LSE, conv_kernel, ctx.scale, ctx.pad_q, ctx.pad_k, ctx.causal)
        need_q, need_k, need_v, need_w = ctx.needs_input_grad[:4]
        dQ = dW = dK = dV = None
        if (need_q or need_w) and (need_k or need_v):
            dQ, dK, dV, dW = ops.backward(*args, out_dtype=Q.dtype)
            return dQ, dK, dV, dW.to(conv_kernel.dtype), None, None, None, None
        if need_q or need_w:
            dQ, dW = ops.dq_backward(*args, out_dtype=Q.dtype)
            dW = dW.to(conv_kernel.dtype)
        if need_k or need_v:
            dK, dV = ops.dkdv_backward(*args, out_dtype=Q.dtype)
        return dQ, dK, dV, dW, None, None, None, None


class ConvAttentionCUDA(nn.Module):
    """Attention with a per-head (kernel_size_q x kernel_size_k) convolution of the
    scaled scores before the softmax.  ``forward`` returns O [B,H,N,d].

    ``compute_dtype`` (not in the reference, which always computes in bf16):
    torch.bfloat16 runs the MFMA kernels, torch.float32 the fp32-arithmetic ones.
    """

    def __init__(self, n_heads: int, kernel_size_q: int = 3, kernel_size_k: int = 3,
                 init_random: bool = True, init_first: bool = False,
                 compute_dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.n_heads = n_heads
        self.kernel_size_q = kernel_size_q
        self.kernel_size_k = kernel_size_k
        self.init_random = init_random
        self.init_first = init_first
        self.compute_dtype = compute_dtype
        self.conv_weight = nn.Parameter(torch.empty(n_heads, kernel_size_q, kernel_size_k))
        self._init_parameters()

    def _init_parameters(self):
        """N(0, 0.2) taps, or a one at tap [0, 0], or a one at the identity tap
        [kernel_size_q - 1, kernel_size_k // 2] (plain attention)."""
        with torch.no_grad():
            if self.init_random:
                nn.init.normal_(self.conv_weight, mean=0.0, std=0.2)
                return
            self.conv_weight.zero_()
            if self.init_first:
                self.conv_weight[:, 0, 0] = 1.0
            else:
                self.conv_weight[:, self.kernel_size_q - 1, self.kernel_size_k // 2] = 1.0

    def forward(self, Q, K, V, causal=True, softmax_scale=None):
        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(Q.shape[-1])
        dt = self.compute_dtype
        return FlashConvAttentionCUDAFunction.apply(
            Q.to(dt), K.to(dt), V.to(dt), self.conv_weight, softmax_scale,
            self.kernel_size_q - 1, (self.kernel_size_k - 1) // 2, causal)

    def forward_with_stats(self, Q, K, V, causal=True, softmax_scale=None):
        """(O, M, L) without autograd, the tuple the reference's docstring promises."""
        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(Q.shape[-1])
        dt = self.compute_dtype
        with torch.no_grad():
            return ops.forward(Q.to(dt).contiguous(), K.to(dt).contiguous(), V.to(dt).contiguous(),
                               self.conv_weight, softmax_scale, self.kernel_size_q - 1,
                               (self.kernel_size_k - 1) // 2, causal, out_dtype=dt)


# Names the reference package exports (flash_multi_token_attention/__init__.py:7-10,
# conv_attn/__init__.py:34-36).
FlashConvAttention = ConvAttentionCUDA
FlashConvAttentionFunction = FlashConvAttentionCUDAFunction
