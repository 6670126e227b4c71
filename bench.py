#!/usr/bin/env python3
"""Headline benchmark: conv-attention forward + backward on one MI355X.

One step = training forward + backward (D/LSE preparation, dQ + dW partials,
one-pass dK/dV/dW/dS kernel, dQ = dS K, ordered dW reduction) of workload c3_fwd_bwd (B=4, H=16, N=4096, d=128,
6x11 window, bf16, causal) through the C ABI, inputs and outputs resident in
HBM.  ``value`` is useful TFLOP/s: (4 + 10) * d * N(N+1)/2 * B * H matmul FLOPs
per step; the convolution's work and every recomputed tile are not counted.

Prints one JSON line with the step metric, the roofline of the dominant kernel
(HIP-event time per launch), the decode step's HBM rate (workload c4_decode) and
a CPU baseline (the oracle on a bounded sample, host cores of this machine).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from flash_multi_token_attention_amd import _lib, synthetic  # noqa: E402

MFMA_BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBPS = 8000.0


def measured_traffic(kernel, workload):
    """HBM bytes per launch of `kernel` on `workload` as measured with rocprofv3
    FETCH_SIZE / WRITE_SIZE (calibrated on a plain copy), from profiles/traffic.json;
    None when that kernel has not been measured."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(f"{kernel}@{workload}", {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def _p(t):
    return C.c_void_p(t.data_ptr())


class TrainStep:
    """Pre-allocated forward + backward of one workload, straight on the C ABI."""

    def __init__(self, wl, dev, exact=False):
        self.wl, self.lib = wl, _lib.load()
        t = synthetic.make_inputs(wl, seed=0)
        self.Q, self.K, self.V, self.W = (t[k].to(dev) for k in ("Q", "K", "V", "W"))
        self.dO = t["dO"].to(dev) if "dO" in t else torch.zeros_like(self.Q)
        dt = _lib.BF16 if wl.dtype == "bf16" else _lib.F32
        tdt = torch.bfloat16 if wl.dtype == "bf16" else torch.float32
        self.desc = _lib.Desc(wl.B, wl.H, wl.Nq, wl.Nk, wl.d, wl.c_q, wl.c_k, wl.scale, int(wl.causal),
                              dt, dt, 1, _lib.FLAG_EXACT if exact else 0)
        shp = (wl.B, wl.H, wl.Nq, wl.d)
        stat = (wl.B, wl.H, wl.Nq)
        self.O = torch.empty(shp, dtype=tdt, device=dev)
        self.dQ, self.dK, self.dV = (torch.empty(shp, dtype=tdt, device=dev) for _ in range(3))
        self.M, self.L, self.D, self.LSE = (torch.empty(stat, dtype=torch.float32, device=dev) for _ in range(4))
        nb = self.lib.convattn_dw_partial_bytes(C.byref(self.desc))
        assert nb > 0, "descriptor rejected"
        self.part = torch.empty(nb // 4, dtype=torch.float32, device=dev)
        self.ws = torch.empty(self.lib.convattn_bwd_fused_workspace_bytes(C.byref(self.desc)), dtype=torch.uint8,
                              device=dev)
        self.dW = torch.empty_like(self.W)
        self.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        d, s = C.byref(self.desc), self.stream
        bwd_in = (_p(self.Q), _p(self.K), _p(self.V), _p(self.dO), _p(self.D), _p(self.LSE), _p(self.W))
        # the step: forward, D/LSE, then the one-pass backward (its three launches timed one by one)
        self.kernels = {
            "fwd": lambda: self.lib.convattn_fwd(d, _p(self.Q), _p(self.K), _p(self.V), _p(self.W),
                                                 _p(self.O), _p(self.M), _p(self.L), s),
            "bwd_preprocess": lambda: self.lib.convattn_bwd_preprocess(
                d, _p(self.O), _p(self.dO), _p(self.M), _p(self.L), _p(self.D), _p(self.LSE), s),
            "bwd_fused_dkdv": lambda: self.lib.convattn_bwd_fused_dkdv(d, *bwd_in, _p(self.dK), _p(self.dV),
                                                                        _p(self.ws), s),
            "bwd_fused_dq": lambda: self.lib.convattn_bwd_fused_dq(d, *bwd_in, _p(self.dQ), _p(self.ws), s),
            "bwd_fused_dw": lambda: self.lib.convattn_bwd_fused_dw(d, _p(self.ws), _p(self.dW), s),
        }
        # the two independent passes behind dq_backward / dkdv_backward (--two-pass, --only)
        self.two_pass = {
            "bwd_dq_dw": lambda: self.lib.convattn_bwd_dq_dw(
                d, _p(self.Q), _p(self.K), _p(self.V), _p(self.dO), _p(self.D), _p(self.LSE), _p(self.W),
                _p(self.dQ), _p(self.part), s),
            "dw_reduce": lambda: self.lib.convattn_dw_reduce(d, _p(self.part), _p(self.dW), s),
            "bwd_dkdv": lambda: self.lib.convattn_bwd_dkdv(
                d, _p(self.Q), _p(self.K), _p(self.V), _p(self.dO), _p(self.D), _p(self.LSE), _p(self.W),
                _p(self.dK), _p(self.dV), s),
        }

    def step(self, two_pass=False):
        todo = dict(self.kernels)
        if two_pass:
            todo = {k: v for k, v in todo.items() if not k.startswith("bwd_fused")}
            todo.update(self.two_pass)
        for name, fn in todo.items():
            rc = fn()
            if rc:
                raise RuntimeError(f"{name}: {_lib.strerror(rc)}")

    def path(self):
        f = self.lib.convattn_kernel_path(C.byref(self.desc), _lib.OP_FWD)
        b = self.lib.convattn_kernel_path(C.byref(self.desc), _lib.OP_BWD)
        return {"fwd": "mfma" if f == 1 else "fp32", "bwd": "mfma" if b == 1 else "fp32"}


class DecodeStep:
    def __init__(self, wl, dev):
        self.wl, self.lib = wl, _lib.load()
        g = torch.Generator(device=dev).manual_seed(0)
        mk = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        self.Q, self.K, self.V = mk(wl.B, wl.H, wl.Nq, wl.d), mk(wl.B, wl.H, wl.Nk, wl.d), mk(wl.B, wl.H, wl.Nk, wl.d)
        E = torch.randn(wl.H, wl.c_q, wl.c_k, generator=torch.Generator().manual_seed(0))
        self.W = synthetic.conv_weight(wl, E).to(dev)
        from flash_multi_token_attention_amd.conv_attn.ops import default_k_splits
        self.splits = default_k_splits(wl.B, wl.H, wl.Nk)
        self.desc = _lib.Desc(wl.B, wl.H, wl.Nq, wl.Nk, wl.d, wl.c_q, wl.c_k, wl.scale, 0,
                              _lib.BF16, _lib.BF16, self.splits, 0)
        f32 = dict(dtype=torch.float32, device=dev)
        self.Op = torch.empty(wl.B, wl.H, self.splits, wl.d, **f32)
        self.Mp = torch.empty(wl.B, wl.H, self.splits, **f32)
        self.Lp = torch.empty(wl.B, wl.H, self.splits, **f32)
        self.O = torch.empty(wl.B, wl.H, 1, wl.d, dtype=torch.bfloat16, device=dev)
        self.M = torch.empty(wl.B, wl.H, 1, **f32)
        self.L = torch.empty(wl.B, wl.H, 1, **f32)
        self.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(self):
        d, s = C.byref(self.desc), self.stream
        rc = self.lib.convattn_decode(d, _p(self.Q), _p(self.K), _p(self.V), _p(self.W), _p(self.Op),
                                      _p(self.Mp), _p(self.Lp), s)
        rc = rc or self.lib.convattn_decode_combine(d, _p(self.Op), _p(self.Mp), _p(self.Lp), _p(self.O),
                                                    _p(self.M), _p(self.L), s)
        if rc:
            raise RuntimeError(f"decode: {_lib.strerror(rc)}")


def time_events(fn, iters, warmup):
    """Average milliseconds per call of ``fn`` from HIP events on the current
    stream (the stream every launch of this program goes to)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def cpu_baseline(wl, budget_s=12.0):
    """The oracle (same torch op sequence as the reference's PyTorch module plus
    autograd), fp32, on (batch, head) pairs of the workload until ``budget_s``
    of CPU time is spent; useful FLOPs of the pairs done / time."""
    from oracle import conv_attn_oracle as orc
    t = synthetic.make_inputs(synthetic.Workload(**{**wl.__dict__, "B": 1, "H": 16}), seed=0)
    fl = synthetic.useful_flops(wl)
    per_pair = (fl["fwd"] + fl["bwd"]) / (wl.B * wl.H)
    done, t0 = 0, time.perf_counter()
    while done < 16:
        sl = slice(done, done + 1)
        Q, K, V, dO = (t[k][:, sl].float() for k in ("Q", "K", "V", "dO"))
        orc.backward_autograd(Q, K, V, t["W"][sl], dO, wl.causal, wl.scale)
        done += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    return {"value": per_pair * done / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{done} of {wl.B * wl.H} (batch, head) pairs of {wl.name}, fwd+autograd bwd, fp32, "
                      f"{dt:.1f} s on {os.cpu_count()} logical CPUs"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (a step takes 2 ms; the per-kernel timings run before the step is timed, see below)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3_fwd_bwd", choices=["c3_fwd_bwd", "c5_long", "c2_fwd"])
    ap.add_argument("--exact", action="store_true", help="force the fp32-arithmetic kernels")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode measurement")
    ap.add_argument("--only", default=None, help="run only this kernel of the step (for profiling)")
    ap.add_argument("--two-pass", action="store_true",
                    help="backward as the two independent passes (dQ+dW, dK/dV) instead of the one-pass backward")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; run with --gpus 1 "
                 "(the path shards by batch and head with no exchange between GPUs)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    wl = synthetic.WORKLOADS[args.workload]
    fl = synthetic.useful_flops(wl)

    if args.only == "copy":
        # plain device copy of known size: calibrates the HBM traffic counters
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        ms = time_events(lambda: dst.copy_(src), args.steps, args.warmup)
        print(json.dumps({"only": "copy", "bytes_read": 1 << 30, "bytes_written": 1 << 30, "ms": ms,
                          "GBps": 2 * (1 << 30) / ms / 1e6}))
        return
    ts = TrainStep(wl, dev, exact=args.exact)
    if args.only:
        if args.only == "decode":
            ds = DecodeStep(synthetic.WORKLOADS["c4_decode"], dev)
            ms = time_events(ds.step, args.steps, args.warmup)
        else:
            ts.step()
            ms = time_events({**ts.kernels, **ts.two_pass}[args.only], args.steps, args.warmup)
        print(json.dumps({"only": args.only, "ms": ms}))
        return

    step = (lambda: ts.step(args.two_pass)) if wl.backward else ts.kernels["fwd"]
    # per-kernel launch durations first (HIP events, same stream): they also bring the device to its
    # sustained clocks before the step is timed (a step takes 2 ms; timed from idle, the first tens of
    # milliseconds of any run read 5 to 8 % slower per step)
    for _ in range(10):
        step()
    allk = {**ts.kernels, **ts.two_pass}
    names = ["fwd"]
    if wl.backward:
        names = [n for n in ts.kernels if not (args.two_pass and n.startswith("bwd_fused"))]
        names += list(ts.two_pass) if args.two_pass else []
    k_ms = {n: time_events(allk[n], max(3, args.steps // 2), 1) for n in names}

    # the step: W untimed warm-up steps, then K steps back to back between two synchronisations
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    useful = fl["fwd"] + (fl["bwd"] if wl.backward else 0.0)
    # spread of single steps (HIP events around each of a second batch of steps; not the headline
    # number, which is the wall clock of the back-to-back run above)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in evs:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    per_step = sorted(a.elapsed_time(b) for a, b in evs)

    # useful FLOPs a launch of each kernel is credited with (recompute not counted): the backward
    # has five products of equal size (S, dP, dV, dK, dQ)
    credit = {"fwd": fl["fwd"], "bwd_dq_dw": 0.6 * fl["bwd"], "bwd_dkdv": 0.4 * fl["bwd"],
              "bwd_fused_dkdv": 0.8 * fl["bwd"], "bwd_fused_dq": 0.2 * fl["bwd"]}
    dom = max((n for n in names if n in credit), key=lambda n: k_ms[n])
    achieved = credit[dom] / (k_ms[dom] * 1e-3) / 1e12
    out = {
        "metric": "conv-attn fwd+bwd TFLOP/s (N=4k,d=128 bf16); decode HBM GB/s vs peak",
        "value": useful / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wl.dtype, "data": "synthetic",
        "config": {"workload": f"{wl.name}: B={wl.B} H={wl.H} N={wl.Nq} d={wl.d} window={wl.c_q}x{wl.c_k} "
                               f"causal={wl.causal} fwd+bwd", "kernel_path": ts.path(),
                   "useful_flop_per_step": useful, "conv_flop_per_pass": fl["conv_per_pass"],
                   **synthetic.executed_mfma_flops(wl, two_pass=args.two_pass)},
        "ms_per_step_min": per_step[0], "ms_per_step_median": per_step[len(per_step) // 2],
        "kernel_ms": k_ms,
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": measured_traffic(dom, wl.name)},
    }
    if not args.no_decode:
        dwl = synthetic.WORKLOADS["c4_decode"]
        del ts
        torch.cuda.empty_cache()
        ds = DecodeStep(dwl, dev)
        dms = time_events(ds.step, max(10, args.steps), 3)
        nbytes = synthetic.decode_bytes(dwl)
        gbps = nbytes / (dms * 1e-3) / 1e9
        out["decode"] = {"workload": f"{dwl.name}: B={dwl.B} H={dwl.H} Nk={dwl.Nk} d={dwl.d} "
                                     f"window={dwl.c_q}x{dwl.c_k} resident_rows={dwl.Nq} splits={ds.splits}",
                         "ms": dms, "bytes": nbytes,
                         "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                      "frac": gbps / HBM_PEAK_GBPS,
                                      "traffic": measured_traffic("decode", dwl.name)}}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
