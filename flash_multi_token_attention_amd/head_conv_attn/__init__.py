"""Head-mixing attention (the reference's ``head_conv_attn`` package) on the HIP library."""
from .head_conv_attn import HeadConvAttention, HeadConvAttentionFunction, head_conv_attention  # noqa: F401
from .ops import bwd_dkdv as head_conv_attention_bwd_dkdv  # noqa: F401
from .ops import bwd_dq_dw as head_conv_attention_bwd_dq_dw  # noqa: F401
from .ops import forward as head_conv_attention_forward  # noqa: F401

__all__ = ["HeadConvAttention", "HeadConvAttentionFunction", "head_conv_attention", "head_conv_attention_forward",
           "head_conv_attention_bwd_dq_dw", "head_conv_attention_bwd_dkdv"]
