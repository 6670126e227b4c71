"""Module path of the reference's ``conv_attn/flash_conv_attention_inference.py``: the decode
shim and the raw decode op under the names its callers import
(scripts/test_fwd_inference_conv_attn.py:15-18, scripts/benchmark_fwd_inference_conv_attn.py:11)."""
from .inference import fwd_conv_attn_inference, forward_inference  # noqa: F401

__all__ = ["fwd_conv_attn_inference", "forward_inference"]
