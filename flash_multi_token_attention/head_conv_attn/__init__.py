"""Alias of ``flash_multi_token_attention_amd.head_conv_attn`` under the reference's package path."""
from flash_multi_token_attention_amd.head_conv_attn import *  # noqa: F401,F403
from flash_multi_token_attention_amd.head_conv_attn import __all__  # noqa: F401
