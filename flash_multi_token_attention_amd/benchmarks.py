"""Sequence-length sweeps of the conv-attention module and of the decode shim, the
counterpart of the reference's benchmark scripts
(scripts/benchmark_conv_attention_cuda.py:119-344: batch 1, 8 heads, head dim 64, N from 256
to 8192, square windows of 3, 7 and 11 taps, forward and forward+backward;
scripts/plot_benchmark_seq_len.py:83-165: HIP-event style timing after warm-up;
scripts/benchmark_fwd_inference_conv_attn.py:45-122: last-row decode over a KV cache).

Each line times this library beside torch's ``scaled_dot_product_attention`` on the same
tensors (the reference's "Flash Attention" comparison line) and prints a markdown table:

    python -m flash_multi_token_attention_amd.benchmarks train  [--quick]
    python -m flash_multi_token_attention_amd.benchmarks decode [--quick]

The reference's third line, its materialising PyTorch module, allocates [B,H,N,N] fp32
temporaries and is not part of this package; it is timed on the CPU by ``bench.py``.
"""
from __future__ import annotations

import argparse
import math
import statistics
from typing import Callable, List

import torch
import torch.nn.functional as F

from .conv_attn.inference import fwd_conv_attn_inference
from .conv_attn.module import ConvAttentionCUDA

# (seq_len, window) pairs of the reference's suite, then the sweep of its plots.
TRAIN_SUITE = [(256, 3), (512, 3), (1024, 3), (2048, 7), (2048, 11), (4096, 11), (8192, 11)]
TRAIN_SWEEP = [(n, k) for k in (3, 7, 11) for n in (256, 512, 1024, 2048, 4096, 8192)]
DECODE_SWEEP = [1024, 4096, 16384, 65536]


def time_ms(fn: Callable[[], None], iters: int = 20, warmup: int = 5) -> float:
    """Median over ``iters`` single-call timings with device events."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    out: List[float] = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        out.append(a.elapsed_time(b))
    return statistics.median(out)


def train_case(B: int, H: int, N: int, d: int, k: int, iters: int) -> dict:
    dev = "cuda:0"
    g = torch.Generator().manual_seed(42)
    Q, K, V, dO = (torch.randn(B, H, N, d, generator=g).to(torch.bfloat16).to(dev) for _ in range(4))
    for t in (Q, K, V):
        t.requires_grad_(True)
    mod = ConvAttentionCUDA(H, k, k, init_random=True).to(dev)
    scale = 1.0 / math.sqrt(d)

    def conv_fwd():
        with torch.no_grad():
            mod(Q, K, V, causal=True, softmax_scale=scale)

    def conv_fwd_bwd():
        O = mod(Q, K, V, causal=True, softmax_scale=scale)
        O.backward(dO)
        Q.grad = K.grad = V.grad = mod.conv_weight.grad = None

    def sdpa_fwd():
        with torch.no_grad():
            F.scaled_dot_product_attention(Q, K, V, is_causal=True, scale=scale)

    def sdpa_fwd_bwd():
        O = F.scaled_dot_product_attention(Q, K, V, is_causal=True, scale=scale)
        O.backward(dO)
        Q.grad = K.grad = V.grad = None

    pairs = B * H * N * (N + 1) / 2
    r = {"N": N, "k": k,
         "conv_fwd": time_ms(conv_fwd, iters), "conv_fwd_bwd": time_ms(conv_fwd_bwd, iters),
         "sdpa_fwd": time_ms(sdpa_fwd, iters), "sdpa_fwd_bwd": time_ms(sdpa_fwd_bwd, iters)}
    r["conv_tflops"] = 14 * d * pairs / (r["conv_fwd_bwd"] * 1e-3) / 1e12
    return r


def decode_case(B: int, H: int, Nk: int, d: int, c_q: int, c_k: int, iters: int) -> dict:
    dev = "cuda:0"
    g = torch.Generator().manual_seed(42)
    Q = torch.randn(B, H, c_q, d, generator=g).to(torch.bfloat16).to(dev)
    K, V = (torch.randn(B, H, Nk, d, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    W = (0.02 * torch.randn(H, c_q, c_k, generator=g)).to(dev)
    scale = 1.0 / math.sqrt(d)
    q_last = Q[:, :, -1:, :].contiguous()

    def conv():
        fwd_conv_attn_inference(Q, K, V, W, 0, scale, c_q - 1, (c_k - 1) // 2, False)

    def sdpa():
        F.scaled_dot_product_attention(q_last, K, V, scale=scale)

    r = {"Nk": Nk, "conv": time_ms(conv, iters), "sdpa": time_ms(sdpa, iters)}
    r["conv_gbs"] = 2 * B * H * Nk * d * 2 / (r["conv"] * 1e-3) / 1e9
    return r


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("which", choices=["train", "decode"])
    ap.add_argument("--quick", action="store_true", help="the reference's 7-line suite / fewer decode lengths")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--heads", type=int, default=None)
    ap.add_argument("--head-dim", type=int, default=None)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("benchmarks need a GPU")
    print(f"device: {torch.cuda.get_device_name(0)}")
    if a.which == "train":
        B, H, d = a.batch or 1, a.heads or 8, a.head_dim or 64
        print(f"B={B} H={H} d={d} bf16 causal; ms per call (median of {a.iters}); "
              "TFLOP/s = 14 d N(N+1)/2 B H / fwd+bwd time")
        print("| N | window | conv fwd | conv fwd+bwd | sdpa fwd | sdpa fwd+bwd | fwd+bwd vs sdpa | conv TFLOP/s |")
        print("|---|---|---|---|---|---|---|---|")
        for N, k in (TRAIN_SUITE if a.quick else TRAIN_SWEEP):
            r = train_case(B, H, N, d, k, a.iters)
            print(f"| {N} | {k}x{k} | {r['conv_fwd']:.3f} | {r['conv_fwd_bwd']:.3f} | {r['sdpa_fwd']:.3f} | "
                  f"{r['sdpa_fwd_bwd']:.3f} | {r['conv_fwd_bwd'] / r['sdpa_fwd_bwd']:.2f}x | {r['conv_tflops']:.1f} |",
                  flush=True)
    else:
        B, H, d = a.batch or 2, a.heads or 2, a.head_dim or 64
        print(f"B={B} H={H} d={d} bf16, 11x11 window, 11 resident query rows; ms per call (median of {a.iters}); "
              "GB/s = K and V bytes / time")
        print("| Nk | conv decode | sdpa last row | conv GB/s |")
        print("|---|---|---|---|")
        for Nk in (DECODE_SWEEP[:2] if a.quick else DECODE_SWEEP):
            r = decode_case(B, H, Nk, d, 11, 11, a.iters)
            print(f"| {Nk} | {r['conv']:.4f} | {r['sdpa']:.4f} | {r['conv_gbs']:.0f} |", flush=True)


if __name__ == "__main__":
    main()
