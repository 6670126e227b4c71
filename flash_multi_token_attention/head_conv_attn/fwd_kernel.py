"""Alias of ``flash_multi_token_attention_amd.head_conv_attn.fwd_kernel`` under the reference's module path."""
from flash_multi_token_attention_amd.head_conv_attn.fwd_kernel import *  # noqa: F401,F403
from flash_multi_token_attention_amd.head_conv_attn.fwd_kernel import __all__  # noqa: F401
