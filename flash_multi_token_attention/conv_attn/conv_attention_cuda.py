"""Alias of ``flash_multi_token_attention_amd.conv_attn.conv_attention_cuda`` under the reference's module path."""
from flash_multi_token_attention_amd.conv_attn.conv_attention_cuda import *  # noqa: F401,F403
from flash_multi_token_attention_amd.conv_attn.conv_attention_cuda import __all__  # noqa: F401
