"""Seeded synthetic inputs for the benchmark configurations, generated on the CPU so that the
device path and a CPU checker see identical bits.  (The reference draws unseeded inputs on the
device, benchmark.py:63.)
"""
import math

import torch


def _gen(seed):
    return torch.Generator(device="cpu").manual_seed(int(seed))


def gaussian_bf16(rows, cols, seed):
    """randn(rows, cols) in fp32, cast to bf16 -- the matmul_transpose inputs."""
    return torch.randn(rows, cols, generator=_gen(seed), dtype=torch.float32).bfloat16()


def gradient_like_bf16(rows, cols, rank, seed):
    """A gradient-shaped matrix: N(0, 1e-3^2) noise plus a rank-`rank` spike U diag(S) V^T with
    orthonormal U, V and S log-uniform in [1e-2, 1]; Frobenius-normalised, cast to bf16."""
    g = _gen(seed)
    G = 1e-3 * torch.randn(rows, cols, generator=g, dtype=torch.float32)
    U, _ = torch.linalg.qr(torch.randn(rows, rank, generator=g, dtype=torch.float32))
    V, _ = torch.linalg.qr(torch.randn(cols, rank, generator=g, dtype=torch.float32))
    S = torch.exp(torch.rand(rank, generator=g, dtype=torch.float32) * math.log(1e-2))
    G = G + (U * S) @ V.T
    G = G / (G.norm() + 1e-7)
    return G.bfloat16()


# shapes of one Llama-7B decoder layer, in the order q, k, v, o, gate, up, down
LLAMA7B_LAYER_SHAPES = [(4096, 4096)] * 4 + [(11008, 4096)] * 2 + [(4096, 11008)]


def llama7b_layer(layer, device="cpu"):
    """(params, grads) of one layer: p ~ 0.02 N(0,1), g ~ 1e-3 N(0,1), bf16, seed 1000*layer+index."""
    params, grads = [], []
    for idx, (r, c) in enumerate(LLAMA7B_LAYER_SHAPES):
        g = _gen(1000 * layer + idx)
        p = (0.02 * torch.randn(r, c, generator=g, dtype=torch.float32)).bfloat16()
        d = (1e-3 * torch.randn(r, c, generator=g, dtype=torch.float32)).bfloat16()
        params.append(p.to(device))
        grads.append(d.to(device))
    return params, grads


def syrk_useful_flop(M, K):
    """Multiply-adds of the upper triangle including the diagonal, as 2 flop each."""
    return K * M * (M + 1)


def ns_useful_flop(rows, cols, steps):
    M, K = min(rows, cols), max(rows, cols)
    return steps * (K * M * (M + 1) + M * M * (M + 1) + 2 * M * M * K)
