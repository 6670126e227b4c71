"""Alias of ``flash_multi_token_attention_amd.conv_attn.flash_conv_attention_inference`` under the reference's module path."""
from flash_multi_token_attention_amd.conv_attn.flash_conv_attention_inference import *  # noqa: F401,F403
from flash_multi_token_attention_amd.conv_attn.flash_conv_attention_inference import __all__  # noqa: F401
