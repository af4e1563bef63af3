"""Writes tests/golden/config1.npz: expected outputs of benchmark configuration 1
(8 experts x 128 rows, 128 -> 128, NN; forward, input gradient, weight gradient) from this
repository's CPU oracle.  Inputs are not stored: they are regenerated from torch's CPU
generator with seed 0, which gives the same values on every machine.  Every 8th row of
each output is kept, as fp32.

Run from the repository root:  python tests/golden/make_config1.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import gmm_oracle  # noqa: E402


def inputs():
    torch.manual_seed(0)
    a = torch.randn(1024, 128).to(torch.bfloat16)
    b = torch.randn(8, 128, 128).to(torch.bfloat16)
    grad = torch.randn(1024, 128).to(torch.bfloat16)
    sizes = torch.tensor([128] * 8, dtype=torch.int64)
    return a, b, grad, sizes


def expected(a, b, grad, sizes):
    fwd = gmm_oracle.gmm_c(a, b, sizes)[0]
    agrad = gmm_oracle.gmm_c(grad, b, sizes, trans_b=True)[0]
    bgrad = gmm_oracle.gmm_c(a, grad, sizes, trans_a=True)[0]
    return fwd, agrad, bgrad


if __name__ == "__main__":
    fwd, agrad, bgrad = expected(*inputs())
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1.npz")
    np.savez_compressed(out, fwd=fwd[::8].numpy(), agrad=agrad[::8].numpy(), bgrad=bgrad[:, ::8].numpy())
    print("wrote", out, os.path.getsize(out), "bytes")
