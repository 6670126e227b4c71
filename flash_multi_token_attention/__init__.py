"""Import-path alias: ``import flash_multi_token_attention`` resolves to the
MI355X implementation in ``flash_multi_token_attention_amd``."""
from flash_multi_token_attention_amd import *  # noqa: F401,F403
from flash_multi_token_attention_amd import __all__, __version__  # noqa: F401
