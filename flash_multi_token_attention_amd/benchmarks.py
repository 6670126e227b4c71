"""Sequence-length sweeps of the conv-attention module and of the decode shim, the
counterpart of the reference's benchmark scripts
(scripts/benchmark_conv_attention_cuda.py:119-344: batch 1, 8 heads, head dim 64, N from 256
to 8192, square windows of 3, 7 and 11 taps, forward and forward+backward;
scripts/plot_benchmark_seq_len.py:83-165: HIP-event style timing after warm-up;
scripts/benchmark_fwd_inference_conv_attn.py:45-122: last-row decode over a KV cache).

Each line times this library beside torch's ``scaled_dot_product_attention`` on the same
tensors (the reference's "Flash Attention" comparison line) and prints a markdown table:

    python -m flash_multi_token_attention_amd.benchmarks train  [--quick] [--md FILE]
    python -m flash_multi_token_attention_amd.benchmarks decode [--quick] [--md FILE]
    python -m flash_multi_token_attention_amd.benchmarks head_conv [--quick] [--md FILE]
    python -m flash_multi_token_attention_amd.benchmarks plot --train FILE [--decode FILE] [--out DIR]

``plot`` draws the figures of the reference's plot scripts from such tables
(scripts/plot_benchmark_seq_len.py:233-310: speed relative to the comparison line, forward
times and backward times against the sequence length, one line per window;
scripts/plot_fwd_inference_speedup.py: decode time against the cache length) and needs no GPU.

``head_conv`` times the three kernels of the head-mixing variant (the reference's
head_conv_attn package; it ships no benchmark for it, its own check runs B=2, 16 heads, N=201, d=32,
head_conv_attn/fwd_kernel.py:383-390).

The reference's third line, its materialising PyTorch module ([B,H,N,N] fp32 temporaries), is
not part of this package: ``tests/bench_materialising.py`` times a restatement of it on the GPU
and adds its two columns to a ``train`` table; ``plot`` then also draws the reference's own
speed-up figure (fused module against materialising module) from them.
"""
from __future__ import annotations

import argparse
import math
import statistics
from typing import Callable, List

import torch
import torch.nn.functional as F

import os
import sys

# (seq_len, window) pairs of the reference's suite, then the sweep of its plots.
TRAIN_SUITE = [(256, 3), (512, 3), (1024, 3), (2048, 7), (2048, 11), (4096, 11), (8192, 11)]
TRAIN_SWEEP = [(n, k) for k in (3, 7, 11) for n in (256, 512, 1024, 2048, 4096, 8192)]
DECODE_SWEEP = [1024, 4096, 16384, 65536]
# the configuration of the reference's decode figure (scripts/plot_fwd_inference_speedup.py:59-70):
# batch 2, 2 heads, 16 query rows, head dim 64, 7x7 window, 32 key splits, not causal
DECODE_REF_SWEEP = [512, 1024, 2048, 4096]


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
    from .conv_attn.module import ConvAttentionCUDA
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


def decode_case(B: int, H: int, Nk: int, d: int, c_q: int, c_k: int, iters: int, q_rows: int = 0,
                k_splits: int = 0) -> dict:
    from .conv_attn.inference import fwd_conv_attn_inference
    dev = "cuda:0"
    g = torch.Generator().manual_seed(42)
    Q = torch.randn(B, H, q_rows or c_q, d, generator=g).to(torch.bfloat16).to(dev)
    K, V = (torch.randn(B, H, Nk, d, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    W = (0.02 * torch.randn(H, c_q, c_k, generator=g)).to(dev)
    scale = 1.0 / math.sqrt(d)
    q_last = Q[:, :, -1:, :].contiguous()

    def conv():
        fwd_conv_attn_inference(Q, K, V, W, k_splits, scale, c_q - 1, (c_k - 1) // 2, False)

    def sdpa():
        F.scaled_dot_product_attention(q_last, K, V, scale=scale)

    r = {"Nk": Nk, "conv": time_ms(conv, iters), "sdpa": time_ms(sdpa, iters)}
    r["conv_gbs"] = 2 * B * H * Nk * d * 2 / (r["conv"] * 1e-3) / 1e9
    return r


HEAD_CONV_SWEEP = [(2, 16, 201, 32), (2, 16, 2048, 64), (2, 32, 2048, 64), (2, 32, 2048, 128), (4, 16, 4096, 128)]


def head_conv_case(B: int, H: int, N: int, d: int, iters: int) -> dict:
    from .head_conv_attn import ops
    dev = "cuda:0"
    g = torch.Generator().manual_seed(42)
    Q, K, V, dO = (torch.randn(B, H, N, d, generator=g).to(torch.bfloat16).to(dev) for _ in range(4))
    W = (torch.randn(H, H, generator=g) / math.sqrt(H)).to(dev)
    scale = 1.0 / math.sqrt(d)
    O, L, M = ops.forward(Q, K, V, W, scale=scale, causal=True)
    r = {"B": B, "H": H, "N": N, "d": d,
         "fwd": time_ms(lambda: ops.forward(Q, K, V, W, scale=scale, causal=True), iters),
         "dq_dw": time_ms(lambda: ops.bwd_dq_dw(Q, K, V, W, O, dO, L, M, causal=True, scale=scale), iters),
         "dkdv": time_ms(lambda: ops.bwd_dkdv(Q, K, V, W, O, dO, L, M, causal=True, scale=scale), iters),
         "sdpa_fwd": time_ms(lambda: F.scaled_dot_product_attention(Q, K, V, is_causal=True, scale=scale), iters)}
    pairs = B * H * N * (N + 1) / 2
    # per (row, key, head): 4 d (Q K^T, P V) + 2 H (head mix) forward; 10 d + 6 H backward (S, dP, dV, dQ, dK; mix, mix back, dW)
    r["tflops"] = (14 * d + 8 * H) * pairs / ((r["fwd"] + r["dq_dw"] + r["dkdv"]) * 1e-3) / 1e12
    return r


def parse_table(path: str) -> List[dict]:
    """Rows of the first markdown table of ``path`` as dicts keyed by the header cells."""
    head, rows = None, []
    for line in open(path):
        line = line.strip()
        if not line.startswith("|"):
            if head is not None:
                break   # the end of the first table
            continue
        cells = [c.strip() for c in line.strip("|").split("|")]
        if head is None:
            head = cells
        elif not all(set(c) <= set("-: ") for c in cells):
            rows.append(dict(zip(head, cells)))
    return rows


def plot(train_md: str, decode_md: str, out_dir: str) -> List[str]:
    """The reference's figures from the tables ``train`` / ``decode`` print; returns the files written."""
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    os.makedirs(out_dir, exist_ok=True)
    written = []

    def save(name):
        path = os.path.join(out_dir, name)
        plt.tight_layout()
        plt.savefig(path, dpi=150, bbox_inches="tight")
        plt.close()
        written.append(path)

    if train_md:
        rows = parse_table(train_md)
        windows = sorted({r["window"] for r in rows}, key=lambda w: int(w.split("x")[0]))
        per = {w: sorted((r for r in rows if r["window"] == w), key=lambda r: int(r["N"])) for w in windows}
        # 1: time of the comparison line over this library's time (the reference plots its CUDA
        # module against its PyTorch module; the line both suites share is plain attention)
        plt.figure(figsize=(10, 5))
        for w in windows:
            n = [int(r["N"]) for r in per[w]]
            plt.plot(n, [float(r["sdpa fwd"]) / float(r["conv fwd"]) for r in per[w]], "o-", label=f"forward, {w}")
            plt.plot(n, [float(r["sdpa fwd+bwd"]) / float(r["conv fwd+bwd"]) for r in per[w]], "s--", label=f"forward+backward, {w}")
        plt.axhline(1.0, color="gray", linewidth=0.8)
        plt.xscale("log", base=2); plt.xlabel("Sequence length"); plt.ylabel("SDPA time / conv-attention time")
        plt.title("Conv-attention against plain attention (MI355X)"); plt.grid(True, alpha=0.3); plt.legend(fontsize=7)
        save("benchmark_seq_len_speedup.png")
        # 1b: the reference's published figure: its fused module against its materialising PyTorch module
        # (columns added by tests/bench_materialising.py; rows without them are left out)
        mat = {w: [r for r in per[w] if r.get("materialising fwd", "-") not in ("-", "")] for w in windows}
        if any(mat.values()):
            plt.figure(figsize=(10, 5))
            for w in windows:
                if not mat[w]:
                    continue
                n = [int(r["N"]) for r in mat[w]]
                plt.plot(n, [float(r["materialising fwd"]) / float(r["conv fwd"]) for r in mat[w]], "o-", label=f"forward, {w}")
                plt.plot(n, [float(r["materialising fwd+bwd"]) / float(r["conv fwd+bwd"]) for r in mat[w]], "s--",
                         label=f"forward+backward, {w}")
            plt.axhline(1.0, color="gray", linewidth=0.8)
            plt.xscale("log", base=2); plt.yscale("log"); plt.xlabel("Sequence length")
            plt.ylabel("materialising PyTorch time / fused time")
            plt.title("Fused conv-attention against the materialising PyTorch module (MI355X)")
            plt.grid(True, alpha=0.3); plt.legend(fontsize=7)
            save("benchmark_seq_len_speedup_vs_materialising.png")
        # 2 and 3: absolute times
        for col, other, name, title in (("conv fwd", "sdpa fwd", "benchmark_seq_len_forward_times.png", "Forward"),
                                        ("conv fwd+bwd", "sdpa fwd+bwd", "benchmark_seq_len_backward_times.png", "Forward+backward")):
            plt.figure(figsize=(10, 5))
            for w in windows:
                n = [int(r["N"]) for r in per[w]]
                plt.plot(n, [float(r[col]) for r in per[w]], "o-", label=f"conv-attention {w}")
            w0 = windows[0]
            plt.plot([int(r["N"]) for r in per[w0]], [float(r[other]) for r in per[w0]], "g^-", label="SDPA (no convolution)")
            plt.xscale("log", base=2); plt.yscale("log"); plt.xlabel("Sequence length"); plt.ylabel("Time (ms)")
            plt.title(f"{title} time against sequence length (MI355X)"); plt.grid(True, alpha=0.3); plt.legend(fontsize=7)
            save(name)
    if decode_md:
        rows = sorted(parse_table(decode_md), key=lambda r: int(r["Nk"]))
        n = [int(r["Nk"]) for r in rows]
        plt.figure(figsize=(10, 5))
        plt.plot(n, [float(r["conv decode"]) for r in rows], "ro-", label="conv-attention decode step")
        plt.plot(n, [float(r["sdpa last row"]) for r in rows], "g^-", label="SDPA, last row")
        plt.xscale("log", base=2); plt.yscale("log"); plt.xlabel("Cache length"); plt.ylabel("Time (ms)")
        plt.title("Decode step against cache length (MI355X)"); plt.grid(True, alpha=0.3); plt.legend()
        save("fwd_inference_times.png")
    return written


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("which", choices=["train", "decode", "head_conv", "plot"])
    ap.add_argument("--quick", action="store_true", help="the reference's 7-line suite / fewer decode lengths")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--heads", type=int, default=None)
    ap.add_argument("--head-dim", type=int, default=None)
    ap.add_argument("--md", default=None, help="train / decode / head_conv: also write the table, with its command line, to this file")
    ap.add_argument("--train", default=None, help="plot: table written by `train`")
    ap.add_argument("--decode", default=None, help="plot: table written by `decode`")
    ap.add_argument("--out", default="plots", help="plot: directory for the figures")
    a = ap.parse_args(argv)
    if a.which == "plot":
        if not (a.train or a.decode):
            raise SystemExit("plot needs --train and / or --decode")
        for path in plot(a.train, a.decode, a.out):
            print(path)
        return
    if not torch.cuda.is_available():
        raise SystemExit("benchmarks need a GPU")
    lines: List[str] = []

    def emit(line: str) -> None:
        print(line, flush=True)
        lines.append(line)

    emit("Command: python -m flash_multi_token_attention_amd.benchmarks " + " ".join(argv if argv is not None else sys.argv[1:]))
    emit("")
    emit(f"device: {torch.cuda.get_device_name(0)}")
    if a.which == "train":
        B, H, d = a.batch or 1, a.heads or 8, a.head_dim or 64
        emit(f"B={B} H={H} d={d} bf16 causal; ms per call (median of {a.iters}); "
             "TFLOP/s = 14 d N(N+1)/2 B H / fwd+bwd time")
        emit("")
        emit("| N | window | conv fwd | conv fwd+bwd | sdpa fwd | sdpa fwd+bwd | fwd+bwd vs sdpa | conv TFLOP/s |")
        emit("|---|---|---|---|---|---|---|---|")
        for N, k in (TRAIN_SUITE if a.quick else TRAIN_SWEEP):
            r = train_case(B, H, N, d, k, a.iters)
            emit(f"| {N} | {k}x{k} | {r['conv_fwd']:.3f} | {r['conv_fwd_bwd']:.3f} | {r['sdpa_fwd']:.3f} | "
                 f"{r['sdpa_fwd_bwd']:.3f} | {r['conv_fwd_bwd'] / r['sdpa_fwd_bwd']:.2f}x | {r['conv_tflops']:.1f} |")
    elif a.which == "head_conv":
        emit(f"bf16 inputs, causal; ms per call (median of {a.iters}); TFLOP/s = (14 d + 8 H) N(N+1)/2 B H / "
             "(fwd + dq_dw + dkdv time): the three products of the forward and the seven of the backward, the "
             "recomputation of S and of the head mix in the second backward kernel not counted")
        emit("")
        emit("| B | H | N | d | fwd | bwd dq+dw | bwd dk+dv | sdpa fwd | fwd+bwd TFLOP/s |")
        emit("|---|---|---|---|---|---|---|---|---|")
        for B, H, N, d in (HEAD_CONV_SWEEP[:2] if a.quick else HEAD_CONV_SWEEP):
            r = head_conv_case(B, H, N, d, a.iters)
            emit(f"| {B} | {H} | {N} | {d} | {r['fwd']:.3f} | {r['dq_dw']:.3f} | {r['dkdv']:.3f} | {r['sdpa_fwd']:.3f} | "
                 f"{r['tflops']:.1f} |")
    else:
        B, H, d = a.batch or 2, a.heads or 2, a.head_dim or 64
        emit(f"B={B} H={H} d={d} bf16, 11x11 window, 11 resident query rows; ms per call (median of {a.iters}); "
             "GB/s = K and V bytes / time")
        emit("")
        emit("| Nk | conv decode | sdpa last row | conv GB/s |")
        emit("|---|---|---|---|")
        for Nk in (DECODE_SWEEP[:2] if a.quick else DECODE_SWEEP):
            r = decode_case(B, H, Nk, d, 11, 11, a.iters)
            emit(f"| {Nk} | {r['conv']:.4f} | {r['sdpa']:.4f} | {r['conv_gbs']:.0f} |")
        if not (a.batch or a.heads or a.head_dim):
            emit("")
            emit("The configuration of the reference's decode figure (B=2 H=2 d=64, 16 query rows, 7x7 window, "
                 "k_splits=32, not causal):")
            emit("")
            emit("| Nk | conv decode | sdpa last row |")
            emit("|---|---|---|")
            for Nk in (DECODE_REF_SWEEP[:2] if a.quick else DECODE_REF_SWEEP):
                r = decode_case(2, 2, Nk, 64, 7, 7, a.iters, q_rows=16, k_splits=32)
                emit(f"| {Nk} | {r['conv']:.4f} | {r['sdpa']:.4f} |")
    if a.md:
        with open(a.md, "w") as f:
            f.write("\n".join(lines) + "\n")


if __name__ == "__main__":
    main()
