"""MI355X-native fused conv-attention (multi-token attention with a per-head
causal 2-D convolution over the score plane before the softmax).

Drop-in for ``flash_multi_token_attention`` of
Gusanidas/flash-multi-token-attention: same class and function names, backed by
a C-ABI HIP library for gfx950 instead of JIT-built CUDA extensions.
"""
from .conv_attn import (  # noqa: F401
    ConvAttentionCUDA,
    FlashConvAttention,
    FlashConvAttentionCUDAFunction,
    FlashConvAttentionFunction,
)

__version__ = "0.1.0"
__all__ = ["FlashConvAttention", "FlashConvAttentionFunction"]
