"""Ahead-of-time build of the conv-attention HIP library for gfx950.

``python -m flash_multi_token_attention_amd.build`` (or ``setup.py build_ext``)
compiles every source under ``csrc/`` with hipcc and links
``libconvattn_hip.so`` next to this file.  hipcc cross-compiles, so no GPU is
needed to build.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB_NAME = "libconvattn_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

# MFMA results in ordinary VGPRs (the 512-register dQ kernel otherwise copies every transient
# accumulator out of the accumulation file).  Not for the dK/dV kernel: with its two tile loops
# this compiler's MFMA rewrite pass crashes on it under this option.
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]

# (source, object name, extra flags).  The dK/dV kernel is compiled as two objects (narrow /
# 11-tap windows) so that they build in parallel.
UNITS = [
    ("api.hip", "api", []),
    ("generic_kernels.hip", "generic_kernels", []),
    ("reduce_kernels.hip", "reduce_kernels", []),
    ("fwd_reg_mfma.hip", "fwd_reg_mfma", []),
    ("bwd_dq_mfma.hip", "bwd_dq_mfma", VGPR_FORM),
    ("bwd_chain_mfma.hip", "bwd_chain_mfma_all", ["-DCONVATTN_CHAIN_UNIT=3"]),
    ("bwd_chain_mfma.hip", "bwd_chain_mfma_kv", ["-DCONVATTN_CHAIN_UNIT=1"]),
    ("bwd_chain_mfma.hip", "bwd_chain_mfma_qw", ["-DCONVATTN_CHAIN_UNIT=2"]),
    ("bwd_chain3_mfma.hip", "bwd_chain3_mfma_all", ["-DCONVATTN_CHAIN_UNIT=3"]),
    ("bwd_chain3_mfma.hip", "bwd_chain3_mfma_kv", ["-DCONVATTN_CHAIN_UNIT=1"]),
    ("bwd_chain3_mfma.hip", "bwd_chain3_mfma_qw", ["-DCONVATTN_CHAIN_UNIT=2"]),
    ("bwd_dq_rows.hip", "bwd_dq_rows", []),
    ("decode_stream.hip", "decode_stream", []),
    ("headmix_attn.hip", "headmix_attn", []),
]
SOURCES = sorted({u[0] for u in UNITS})

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall",
    "-Wno-unused-command-line-argument",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # machine scheduler tuned for instruction-level parallelism rather than occupancy: every kernel
    # here runs at a fixed one or two waves per SIMD (measured: forward, backward and decode 0.5-1 % faster)
    "-mllvm", "-amdgpu-sched-strategy=max-ilp",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def _compile(cc: str, src: str, obj: str, extra) -> None:
    cmd = [cc, *HIPCC_FLAGS, *extra, "-I", INCLUDE, "-I", CSRC, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = "is not a recognized feature for this target"
    err = "\n".join(ln for ln in r.stderr.splitlines() if noise not in ln).strip()
    if err:
        sys.stderr.write(err + "\n")


def build(verbose: bool = True, extra_flags=()) -> str:
    """Compile all sources (always, even if the library exists) and link."""
    cc = hipcc()
    obj_dir = os.path.join(ROOT, "build", "convattn_obj")
    os.makedirs(obj_dir, exist_ok=True)
    jobs = []
    for name, obj_name, unit_flags in UNITS:
        jobs.append((os.path.join(CSRC, name), os.path.join(obj_dir, obj_name + ".o"), unit_flags))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        list(ex.map(lambda so: _compile(cc, so[0], so[1], [*so[2], *extra_flags]), jobs))
    tmp = LIB_PATH + ".tmp"
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", *[j[1] for j in jobs], "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build()
