#!/usr/bin/env python3
"""The reference's third benchmark line: its materialising PyTorch module, timed on the GPU.

The reference plots its fused CUDA module against its own pure-PyTorch ``ConvAttention``
(scripts/plot_benchmark_seq_len.py:168-230: the module's forward and forward + backward per
sequence length; :233-310: the speed-up figure) and publishes those ratios (README.md:31-41).
That module's op sequence is restated in ``oracle/conv_attn_oracle.py`` (``forward`` /
``backward_autograd``: [B,H,N,N] fp32 temporaries, ``F.conv2d`` over the score plane); this
script times it in fp32 on the GPU for the rows of a sweep table written by
``python -m flash_multi_token_attention_amd.benchmarks train --md FILE`` and rewrites the table
with two more columns, from which ``benchmarks plot`` draws the reference's speed-up figure.

    python tests/bench_materialising.py profiles/sweep_train.md [--max-n 4096] [--out FILE]

It lives under tests/ because the shipped package must not import the oracle; it is not collected
by pytest (no ``test_`` prefix).
"""
from __future__ import annotations

import argparse
import math
import os
import statistics
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from oracle import conv_attn_oracle as orc  # noqa: E402

MAT_FWD, MAT_BWD = "materialising fwd", "materialising fwd+bwd"


def time_ms(fn, iters=5, warmup=1):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        out.append(a.elapsed_time(b))
    return statistics.median(out)


def materialising_case(B, H, N, d, k, iters):
    dev = "cuda:0"
    g = torch.Generator().manual_seed(42)
    Q, K, V, dO = (torch.randn(B, H, N, d, generator=g).to(dev) for _ in range(4))
    W = (0.02 * torch.randn(H, k, k, generator=g)).to(dev)
    scale = 1.0 / math.sqrt(d)

    def fwd():
        with torch.no_grad():
            orc.forward(Q, K, V, W, True, scale)

    def fwd_bwd():
        orc.backward_autograd(Q, K, V, W, dO, True, scale)

    return time_ms(fwd, iters), time_ms(fwd_bwd, iters)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("table")
    ap.add_argument("--max-n", type=int, default=4096, help="longest sequence timed (the temporaries are [B,H,N,N] fp32)")
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--out", default=None, help="file to write (default: the table itself)")
    a = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_materialising.py needs a GPU")
    lines = open(a.table).read().splitlines()
    cfg = next(l for l in lines if l.startswith("B="))
    B, H, d = (int(tok.split("=")[1]) for tok in cfg.split()[:3])
    out, head = [], None
    for line in lines:
        s = line.strip()
        if not s.startswith("|"):
            out.append(line)
            continue
        cells = [c.strip() for c in s.strip("|").split("|")]
        if head is None:
            head = [c for c in cells if c not in (MAT_FWD, MAT_BWD)]
            out.append("| " + " | ".join(head + [MAT_FWD, MAT_BWD]) + " |")
        elif all(set(c) <= set("-: ") for c in cells):
            out.append("|" + "---|" * (len(head) + 2))
        else:
            row = dict(zip(head, cells))
            N, k = int(row["N"]), int(row["window"].split("x")[0])
            if N <= a.max_n:
                f, fb = materialising_case(B, H, N, d, k, a.iters)
                extra = [f"{f:.3f}", f"{fb:.3f}"]
            else:
                extra = ["-", "-"]
            out.append("| " + " | ".join([row[h] for h in head] + extra) + " |")
            print(out[-1], flush=True)
    note = (f"Columns `{MAT_FWD}` / `{MAT_BWD}`: the reference's materialising PyTorch module (op sequence of "
            "conv_attention_pytorch.py:117-185, fp32, [B,H,N,N] temporaries) on the same GPU, "
            f"`python tests/bench_materialising.py {a.table} --max-n {a.max_n}`; '-' = not timed.")
    out = [l for l in out if not l.startswith("Columns `" + MAT_FWD)]
    out.append("")
    out.append(note)
    with open(a.out or a.table, "w") as f:
        f.write("\n".join(out).rstrip("\n") + "\n")


if __name__ == "__main__":
    main()
