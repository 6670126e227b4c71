"""conv_attn: same public names as flash_multi_token_attention.conv_attn
(conv_attn/__init__.py:28-36 of the reference)."""
from .ops import forward, dq_backward, dkdv_backward, forward_inference, bwd_preprocess, kernel_path
from .module import (ConvAttentionCUDA, FlashConvAttention, FlashConvAttentionCUDAFunction,
                     FlashConvAttentionFunction)
from .inference import fwd_conv_attn_inference

# The reference exports these three from a module that is absent from its tree;
# they are the op-level entry points under their long names.
fwd_conv_attn = forward
dq_bwd_conv_attn = dq_backward
dkdv_bwd_conv_attn = dkdv_backward

__all__ = ["FlashConvAttention", "FlashConvAttentionFunction", "forward", "dq_backward",
           "dkdv_backward", "fwd_conv_attn", "dq_bwd_conv_attn", "dkdv_bwd_conv_attn",
           "ConvAttentionCUDA", "FlashConvAttentionCUDAFunction", "forward_inference",
           "fwd_conv_attn_inference", "bwd_preprocess", "kernel_path"]
