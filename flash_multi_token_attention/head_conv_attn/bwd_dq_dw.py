"""Alias of ``flash_multi_token_attention_amd.head_conv_attn.bwd_dq_dw`` under the reference's module path."""
from flash_multi_token_attention_amd.head_conv_attn.bwd_dq_dw import *  # noqa: F401,F403
from flash_multi_token_attention_amd.head_conv_attn.bwd_dq_dw import __all__  # noqa: F401
