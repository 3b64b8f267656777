"""Writes tests/golden/config1_samples.npz from the CPU oracle (oracle/dwo_oracle.c).

The reference ships no vectors for this path, so these fixtures freeze the pinned oracle's
answers on the CPU-runnable configuration (N=2, C=96, H=W=56, K=31, theta_c = (c mod 8)*pi/8,
torch.manual_seed(0), x ~ N(0,1), w ~ N(0,0.02), dy ~ N(0,1)) at 4096 sampled positions per
tensor, so that both the oracle and the HIP path can be checked against committed data.

    python tests/golden/make_golden.py
"""
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import dwo_oracle as oracle  # noqa: E402


def config1_inputs():
    torch.manual_seed(0)
    x = torch.randn(2, 96, 56, 56)
    w = torch.randn(96, 1, 1, 31) * 0.02
    dy = torch.randn(2, 96, 56, 56)
    theta = torch.tensor([(c % 8) * math.pi / 8 for c in range(96)], dtype=torch.float32)
    return x.numpy(), w.numpy(), dy.numpy(), theta.numpy()


def main():
    x, w, dy, theta = config1_inputs()
    y = oracle.fprop(x, w, theta)
    dx = oracle.dgrad(dy, w, theta)
    dw = oracle.wgrad(dy, x, theta, 31)
    rng = np.random.default_rng(0)
    idx = np.sort(rng.choice(y.size, 4096, replace=False))
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_samples.npz")
    np.savez_compressed(
        out,
        idx=idx.astype(np.int64),
        y=y.reshape(-1)[idx],
        dx=dx.reshape(-1)[idx],
        dw=dw.reshape(96, 31),
        x_sum=np.float64(x.astype(np.float64).sum()),
        w_sum=np.float64(w.astype(np.float64).sum()),
        dy_sum=np.float64(dy.astype(np.float64).sum()),
    )
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
