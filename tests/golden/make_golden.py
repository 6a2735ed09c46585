"""Writes tests/golden/ns_small.npz from the CPU oracle (oracle/oracle.py).

The reference ships no golden vectors for this path and cannot run without a CUDA device, so the
fixture pins the oracle against drift; the oracle is pinned against mathematics in
tests/test_oracle.py.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle  # noqa: E402


def main():
    g = torch.Generator().manual_seed(20240)
    G = torch.randn(64, 96, generator=g).bfloat16()
    bits = G.view(torch.int16).numpy().astype(np.uint16)
    sig = torch.tensor([1.0, 0.5, 0.25, 0.125, 0.0625], dtype=torch.float64)   # exact in bf16
    s = sig / (sig.norm() + oracle.NS_EPS)
    a, b, c = oracle.NS_COEFFS
    for _ in range(5):
        s = a * s + b * s ** 3 + c * s ** 5
    np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "ns_small.npz"),
             G_bf16_bits=bits,
             xxt_fp32=oracle.xxt(G).numpy(),
             ns5_fp32=oracle.newtonschulz(G, 5).numpy(),
             diag_sigma=sig.numpy(), diag_ns5=s.numpy())


if __name__ == "__main__":
    main()
