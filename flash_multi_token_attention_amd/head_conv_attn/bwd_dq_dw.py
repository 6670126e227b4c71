"""``head_conv_attention_bwd_dq_dw`` under the reference's module path (head_conv_attn/bwd_dq_dw.py:373)."""
from .ops import bwd_dq_dw as head_conv_attention_bwd_dq_dw  # noqa: F401

__all__ = ["head_conv_attention_bwd_dq_dw"]
