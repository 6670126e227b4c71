"""``head_conv_attention_bwd_dkdv`` under the reference's module path (head_conv_attn/bwd_dk_dv.py:407)."""
from .ops import bwd_dkdv as head_conv_attention_bwd_dkdv  # noqa: F401

__all__ = ["head_conv_attention_bwd_dkdv"]
