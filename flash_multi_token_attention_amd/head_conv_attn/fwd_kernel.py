"""``head_conv_attention_forward`` under the reference's module path (head_conv_attn/fwd_kernel.py:270)."""
from .ops import forward as head_conv_attention_forward  # noqa: F401

__all__ = ["head_conv_attention_forward"]
