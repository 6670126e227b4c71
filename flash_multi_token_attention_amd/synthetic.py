"""Seeded synthetic workloads for the conv-attention path.

One CPU generator, one draw order (Q, K, V, dO, E), so the same seed gives the
same tensors on every machine: W = delta at the (current query, same key) tap
plus sigma * E.  bf16 workloads round Q, K, V, dO to bf16; W stays fp32.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    B: int
    H: int
    Nq: int
    Nk: int
    d: int
    c_q: int
    c_k: int
    dtype: str = "bf16"          # "bf16" | "fp32"
    causal: bool = True
    sigma: float = 0.05
    key_decay: float = 0.0        # >0: sigma * exp(-|b - pad_k| / key_decay) along keys
    decode: bool = False
    backward: bool = False

    @property
    def pad_q(self) -> int:
        return self.c_q - 1

    @property
    def pad_k(self) -> int:
        return (self.c_k - 1) // 2

    @property
    def scale(self) -> float:
        return 1.0 / math.sqrt(self.d)


# The five configurations the headline metric is quoted on.
WORKLOADS: Dict[str, Workload] = {
    "c1_cpu_fp32": Workload("c1_cpu_fp32", 1, 2, 256, 256, 64, 3, 5, dtype="fp32"),
    "c2_fwd": Workload("c2_fwd", 4, 16, 2048, 2048, 64, 6, 11),
    "c3_fwd_bwd": Workload("c3_fwd_bwd", 4, 16, 4096, 4096, 128, 6, 11, backward=True),
    "c4_decode": Workload("c4_decode", 32, 32, 6, 8192, 128, 6, 11, causal=False, decode=True),
    "c5_long": Workload("c5_long", 1, 32, 16384, 16384, 128, 6, 11, sigma=0.1, key_decay=3.0,
                        backward=True),
}


def conv_weight(wl: Workload, E: torch.Tensor) -> torch.Tensor:
    W = torch.zeros(wl.H, wl.c_q, wl.c_k, dtype=torch.float32)
    W[:, wl.c_q - 1, wl.pad_k] = 1.0
    if wl.key_decay > 0:
        b = torch.arange(wl.c_k, dtype=torch.float32)
        env = wl.sigma * torch.exp(-(b - wl.pad_k).abs() / wl.key_decay)
        return W + env.view(1, 1, -1) * E
    return W + wl.sigma * E


def make_inputs(wl: Workload, seed: int = 0, device: str = "cpu") -> Dict[str, torch.Tensor]:
    """Q [B,H,Nq,d], K,V [B,H,Nk,d], dO like Q (backward workloads), W [H,c_q,c_k] fp32."""
    g = torch.Generator("cpu").manual_seed(seed)
    Q = torch.randn(wl.B, wl.H, wl.Nq, wl.d, generator=g)
    K = torch.randn(wl.B, wl.H, wl.Nk, wl.d, generator=g)
    V = torch.randn(wl.B, wl.H, wl.Nk, wl.d, generator=g)
    out = {"Q": Q, "K": K, "V": V}
    if wl.backward:
        out["dO"] = torch.randn(wl.B, wl.H, wl.Nq, wl.d, generator=g)
    E = torch.randn(wl.H, wl.c_q, wl.c_k, generator=g)
    if wl.dtype == "bf16":
        out = {k: v.to(torch.bfloat16) for k, v in out.items()}
    out["W"] = conv_weight(wl, E)
    return {k: v.to(device) for k, v in out.items()}


def useful_flops(wl: Workload) -> Dict[str, float]:
    """Matmul FLOPs that count as useful: 4*d per causal pair forward, 10*d
    backward; the convolution's VALU/MFMA work is reported separately."""
    pairs = wl.Nq * (wl.Nq + 1) / 2 if wl.causal else wl.Nq * wl.Nk
    bh = wl.B * wl.H
    return {
        "fwd": 4.0 * wl.d * pairs * bh,
        "bwd": 10.0 * wl.d * pairs * bh,
        "conv_per_pass": 2.0 * wl.c_q * wl.c_k * pairs * bh,
    }


def decode_bytes(wl: Workload, elem: int = 2) -> int:
    """Algorithmic HBM bytes of one decode step: K + V once, Q, O and W."""
    kv = 2 * wl.B * wl.H * wl.Nk * wl.d * elem
    q = wl.B * wl.H * wl.Nq * wl.d * elem
    o = wl.B * wl.H * wl.d * elem
    w = wl.H * wl.c_q * wl.c_k * 4
    return kv + q + o + w
