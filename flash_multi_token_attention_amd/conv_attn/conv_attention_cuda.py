"""Module path of the reference's ``conv_attn/conv_attention_cuda.py``: the nn.Module and the
autograd Function under the names its callers import
(``from flash_multi_token_attention.conv_attn.conv_attention_cuda import ConvAttentionCUDA``,
scripts/test_conv_attn.py:7, scripts/benchmark_conv_attention_cuda.py:18-19)."""
from .module import ConvAttentionCUDA, FlashConvAttentionCUDAFunction  # noqa: F401

__all__ = ["ConvAttentionCUDA", "FlashConvAttentionCUDAFunction"]
