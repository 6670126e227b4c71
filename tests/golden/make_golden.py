"""Writes the golden fixtures of this directory.

The reference repository holds no stored vectors for this path, and its PyTorch
module was not imported; the expected values here come from the explicit-loop
float64 implementation in oracle/brute_force.py (index formula only, no tensor
library convolution), which is independent of the torch restatement that the
tests compare against it.

    python tests/golden/make_golden.py

* c1_forward.npz     workload c1_cpu_fp32 (B=1, H=2, N=256, d=64, 3x5 window,
                     causal, seed 0 of the canonical generator): O, M, L.
                     Inputs are regenerated from the seed, only W is stored.
* small_fwd_bwd.npz  B=2, H=2, N=24, d=8, 3x5 and a 6x11 case: inputs, O, M, L,
                     dQ, dK, dV, dW for a stored dO.
* decode_small.npz   6 resident rows against 50 keys, 6x11: O, M, L.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from flash_multi_token_attention_amd import synthetic  # noqa: E402
from oracle import brute_force as bf  # noqa: E402


def main():
    wl = synthetic.WORKLOADS["c1_cpu_fp32"]
    t = synthetic.make_inputs(wl, seed=0)
    O, M, L = bf.forward(t["Q"].numpy(), t["K"].numpy(), t["V"].numpy(), t["W"].numpy(), True, wl.scale)
    np.savez_compressed(os.path.join(HERE, "c1_forward.npz"), W=t["W"].numpy(),
                        O=O.astype(np.float32), M=M.astype(np.float32), L=L.astype(np.float32))

    out = {}
    for tag, (c_q, c_k) in {"a": (3, 5), "b": (6, 11)}.items():
        g = torch.Generator().manual_seed(100 + c_q)
        Q, K, V, dO = (torch.randn(2, 2, 24, 8, generator=g).numpy() for _ in range(4))
        W = (0.3 * torch.randn(2, c_q, c_k, generator=g)).numpy()
        O, M, L = bf.forward(Q, K, V, W, True)
        dQ, dK, dV, dW = bf.backward(Q, K, V, W, dO, True)
        for k, v in dict(Q=Q, K=K, V=V, dO=dO, W=W, O=O, M=M, L=L, dQ=dQ, dK=dK, dV=dV, dW=dW).items():
            out[f"{tag}_{k}"] = np.asarray(v, dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "small_fwd_bwd.npz"), **out)

    g = torch.Generator().manual_seed(7)
    Q = torch.randn(2, 2, 6, 16, generator=g).numpy()
    K, V = (torch.randn(2, 2, 50, 16, generator=g).numpy() for _ in range(2))
    W = (0.3 * torch.randn(2, 6, 11, generator=g)).numpy()
    O, M, L = bf.decode(Q, K, V, W)
    np.savez_compressed(os.path.join(HERE, "decode_small.npz"), Q=Q, K=K, V=V, W=W,
                        O=O.astype(np.float32), M=M.astype(np.float32), L=L.astype(np.float32))


if __name__ == "__main__":
    main()
