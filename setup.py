"""Builds libconvattn_hip.so with hipcc (gfx950) and installs the Python packages."""
from setuptools import find_packages, setup
from setuptools.command.build_ext import build_ext as _build_ext
from setuptools.command.build_py import build_py as _build_py


def _hip_build():
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from flash_multi_token_attention_amd import build
    build.build()


class build_ext(_build_ext):
    def run(self):
        _hip_build()


class build_py(_build_py):
    def run(self):
        _hip_build()
        super().run()


setup(
    name="flash-multi-token-attention-amd",
    version="0.1.0",
    description="MI355X-native fused conv-attention (multi-token attention), drop-in for flash_multi_token_attention.conv_attn",
    packages=find_packages(include=["flash_multi_token_attention_amd*", "flash_multi_token_attention*"]),
    package_data={"flash_multi_token_attention_amd": ["libconvattn_hip.so", "csrc/*"]},
    python_requires=">=3.8",
    install_requires=["torch"],
    cmdclass={"build_ext": build_ext, "build_py": build_py},
)
