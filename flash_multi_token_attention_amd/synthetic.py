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


def executed_mfma_flops(wl: Workload, two_pass: bool = False) -> Dict[str, object]:
    """FLOPs the bf16 MFMA kernels execute on the matrix cores for one step of a causal workload
    with d in {64, 128} and at most 6 query taps, counted from their tiles (every MFMA is
    16 x 16 x 32 = 16384 FLOP), next to the useful ones; the difference is halo, convolution, dW and
    recompute.  Per kernel:

    forward: a wave owns 33 - T output rows (T = 3 or 6 tap slots) of a 32-row score tile and walks
      the keys in 32-key steps up to its last row + 16: per step S^T 2 (row fragments) x 2 (key
      blocks) x d/32, convolution 4 T, P V 2 x d/16 MFMAs.
    key-stationary backward: a wave triple owns 32 keys and walks 32-row tiles from the first row that
      sees its keys: per tile S^T 6 d/32 (48 keys for 32 owned), convolution 4 T (32 keys), dP 4 d/32,
      transposed convolution 4 T, dV and dK 2 d/16 each, dW 4 T MFMAs; for the last of a workgroup's
      four triples a second score chain computes the 16 keys after its own (S^T 4 d/32 for the two
      16-key blocks around them, convolution 2 T, dP 2 d/32).
    dQ = dS K: 2 x d/16 per 32 rows x 32 keys below the diagonal (nothing wasted but the diagonal
      blocks' upper halves).
    """
    assert wl.causal and wl.Nq == wl.Nk
    N, d, T, bh = wl.Nq, wl.d, (3 if wl.c_q <= 3 else 6), wl.B * wl.H
    mf = 16.0 * 16 * 32 * 2
    rows = 33 - T
    fwd = 0
    for w0 in range(0, N, rows):                       # one wave per `rows` output rows
        wg_end = min(N, (w0 // (4 * rows) + 1) * 4 * rows)          # its workgroup's last row + 1
        steps = min((w0 + rows + 15) // 32 + 1, (wg_end + 16 + 31) // 32)
        fwd += steps * (4 * d // 32 + 4 * T + 2 * d // 16)
    consumer = 4 * T + 4 * d // 16 + 4 * T             # transposed convolution, dV and dK, dW
    light = 6 * d // 32 + 4 * T + 4 * d // 32
    extra = 4 * d // 32 + 2 * T + 2 * d // 32           # the score chain of the block after the workgroup's keys
    heavy = light + extra
    full = kv = qw = s_only = 0
    for c0 in range(0, (N + 8 + 127) // 128 * 128, 32):   # one wave pair per 32 keys
        k0 = c0 // 128 * 128
        last = c0 - k0 == 96                            # the last pair of its workgroup
        r_begin = max(0, k0 - 8) // 32 * 32
        n_t = max(0, (N - r_begin + 31) // 32)
        skipped = sum(1 for t in range(n_t) if r_begin + 32 * t + 31 < c0 - 8)   # scores only
        producer = heavy if last else light
        full += (n_t - skipped) * (producer + consumer)
        kv += (n_t - skipped) * (producer + consumer - 4 * T)          # dK / dV pass: no dW
        qw += (n_t - skipped) * (producer + consumer - 4 * d // 16)    # dQ + dW pass: no dV, dK
        s_only += (skipped + 1) * (10 if last else 6) * d // 32        # + the 32 rows above the first tile
    dq = sum((min(N, (r // 128 + 1) * 128) + 63) // 64 * 2 for r in range(0, N, 32)) * 2 * d // 16
    out = {"fwd": fwd * mf * bh}
    if wl.backward:
        if two_pass:
            out["bwd_dkdv"] = (kv + s_only) * mf * bh
            out["bwd_dq_dw"] = (qw + s_only + dq) * mf * bh
        else:
            out["bwd_fused_dkdv"] = (full + s_only) * mf * bh
            out["bwd_fused_dq"] = dq * mf * bh
    total = sum(out.values())
    fl = useful_flops(wl)
    useful = fl["fwd"] + (fl["bwd"] if wl.backward else 0.0)
    return {"executed_mfma_flop_per_step": total, "executed_mfma_flop_per_kernel": out,
            "halo_recompute_flop_per_step": total - useful}


def decode_bytes(wl: Workload, elem: int = 2) -> int:
    """Algorithmic HBM bytes of one decode step: K + V once, Q, O and W."""
    kv = 2 * wl.B * wl.H * wl.Nk * wl.d * elem
    q = wl.B * wl.H * wl.Nq * wl.d * elem
    o = wl.B * wl.H * wl.d * elem
    w = wl.H * wl.c_q * wl.c_k * 4
    return kv + q + o + w
