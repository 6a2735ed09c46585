"""Pins for the CPU oracle itself (no GPU): closed forms, brute force and invariants chosen so that
a dropped term, a wrong sign or a transposed operand fails at least one of them."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_xxt_integer_bruteforce():
    g = torch.Generator().manual_seed(1)
    X = torch.randint(-2, 3, (37, 53), generator=g).float()
    ref = torch.zeros(37, 37, dtype=torch.int64)
    Xi = X.long()
    for i in range(37):
        for j in range(37):
            ref[i, j] = int((Xi[i] * Xi[j]).sum())
    assert torch.equal(oracle.xxt_int64(X), ref)
    assert torch.equal(oracle.xxt(X).long(), ref)


def test_xxt_closed_forms():
    assert torch.equal(oracle.xxt(torch.eye(16)), torch.eye(16))
    assert torch.equal(oracle.xxt(torch.ones(5, 64)), torch.full((5, 5), 64.0))
    H = torch.tensor([[1.0]])
    for _ in range(5):
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    assert torch.equal(oracle.xxt(H), 32 * torch.eye(32))
    # a non-symmetric-looking mistake (X.T @ X) has the wrong shape for a rectangular input
    assert oracle.xxt(torch.ones(3, 7)).shape == (3, 3)


def _poly(s, steps):
    a, b, c = oracle.NS_COEFFS
    for _ in range(steps):
        s = a * s + b * s ** 3 + c * s ** 5
    return s


@pytest.mark.parametrize("shape", [(24, 40), (40, 24), (32, 32)])
def test_newtonschulz_matches_svd_closed_form(shape):
    # X = U diag(s) V^T  ->  NS(X) = U diag(p^5(s/|s|)) V^T ; inputs exactly representable in bf16
    # are not needed because the closed form starts from the bf16-cast matrix as the oracle does
    g = torch.Generator().manual_seed(7)
    G = torch.randn(*shape, generator=g)
    Gb = G.bfloat16().double()
    U, S, Vh = torch.linalg.svd(Gb, full_matrices=False)
    s = S / (S.norm() + oracle.NS_EPS)
    want = (U * _poly(s, 5)) @ Vh
    got = oracle.newtonschulz(G, 5, dtype=torch.float64)
    assert oracle.rel_fro(got, want) < 1e-9
    got32 = oracle.newtonschulz(G, 5, dtype=torch.float32)
    assert oracle.rel_fro(got32, want) < 2e-5


def test_newtonschulz_diagonal_scalar_recurrence():
    sig = torch.tensor([1.0, 0.5, 0.1, 0.01])
    G = torch.diag(sig)
    out = oracle.newtonschulz(G, 5, dtype=torch.float64)
    sb = sig.bfloat16().double()
    want = _poly(sb / (sb.norm() + oracle.NS_EPS), 5)
    assert torch.allclose(torch.diagonal(out), want, rtol=1e-10, atol=0)
    off = out - torch.diag(torch.diagonal(out))
    assert off.abs().max() == 0
    # the values quoted for this case: (0.6990, 1.1188, 0.7120, 0.6866) for exact sigma;
    # bf16-casting 0.1 and 0.01 moves them in the third decimal only
    assert torch.allclose(want, torch.tensor([0.6990, 1.1188, 0.7120, 0.6866]).double(), atol=5e-3)


def test_newtonschulz_invariants():
    g = torch.Generator().manual_seed(3)
    G = torch.randn(20, 48, generator=g).bfloat16()
    o1 = oracle.newtonschulz(G, 5, dtype=torch.float64)
    o2 = oracle.newtonschulz(G.mT.contiguous(), 5, dtype=torch.float64)
    assert torch.equal(o1, o2.mT)                       # NS(G^T) == NS(G)^T
    o3 = oracle.newtonschulz(G * 4, 5, dtype=torch.float64)   # power-of-two scale: same bf16 mantissas
    assert oracle.rel_fro(o3, o1) < 1e-6
    assert oracle.newtonschulz(G, 0).shape == G.shape
    # steps = 0 is just the normalisation
    n = oracle.newtonschulz(G, 0, dtype=torch.float64)
    assert abs(float(n.norm()) - 1.0) < 1e-6
    # singular values of the result sit in the band the quintic maps (0, 1] into
    sv = torch.linalg.svdvals(o1)
    assert sv.min() > 0.3 and sv.max() < 1.3
    # zero input: eps keeps it finite
    z = oracle.newtonschulz(torch.zeros(4, 6), 5)
    assert torch.equal(z, torch.zeros(4, 6))


def test_ns_step_trace_consistent():
    g = torch.Generator().manual_seed(5)
    G = torch.randn(16, 32, generator=g)
    out, st = oracle.newtonschulz(G, 3, trace=True)
    assert len(st) == 4
    assert torch.equal(oracle.ns_step(st[1]), st[2])
    assert torch.equal(out, st[3])


def test_rel_fro_known_values():
    """The parity metric itself: known non-zero answers, so that a metric that returned 0 (or the
    wrong ratio) could not pass the floating-point tests silently."""
    g = torch.Generator().manual_seed(2)
    R = torch.randn(37, 53, generator=g, dtype=torch.float64)
    assert oracle.rel_fro(R, R) == 0.0
    assert abs(oracle.rel_fro(1.01 * R, R) - 0.01) < 1e-12
    assert abs(oracle.rel_fro(torch.zeros_like(R), R) - 1.0) < 1e-15
    assert abs(oracle.rel_fro(-R, R) - 2.0) < 1e-15
    E = torch.zeros(4, 4, dtype=torch.float64)
    E[1, 2] = 0.5                                   # ||E||_F = 0.5, ||I_4||_F = 2
    assert abs(oracle.rel_fro(torch.eye(4, dtype=torch.float64) + E, torch.eye(4, dtype=torch.float64)) - 0.25) < 1e-15
    # it is relative to the SECOND argument: ||R - 3R|| / ||3R|| = 2/3, not 2
    assert abs(oracle.rel_fro(R, 3 * R) - 2.0 / 3.0) < 1e-12
    # bf16 inputs are compared by value (one rounding of N(0,1) data is about 2^-9 / sqrt(3) relative)
    assert 1.5e-3 < oracle.rel_fro(R.bfloat16(), R) < 3e-3


def test_newtonschulz_leading_dimensions_are_a_batch():
    """muon.py:13 admits ndim >= 2 and muon.py:23 normalises over the last two dimensions: every
    matrix of a batch goes through the iteration on its own, with its own norm."""
    g = torch.Generator().manual_seed(17)
    G = torch.randn(3, 2, 24, 40, generator=g, dtype=torch.float64)
    G[1] *= 1e3                                      # very different norms must not leak between matrices
    G[2, 1] *= 1e-4
    got = oracle.newtonschulz(G, 5, torch.float64)
    assert got.shape == G.shape
    for i in range(3):
        for j in range(2):
            U, S, Vh = torch.linalg.svd(G[i, j].bfloat16().double(), full_matrices=False)
            s = S / (S.norm() + oracle.NS_EPS)
            a, b, c = oracle.NS_COEFFS
            for _ in range(5):
                s = a * s + b * s ** 3 + c * s ** 5
            want = U @ torch.diag(s) @ Vh
            assert oracle.rel_fro(got[i, j], want) < 1e-9
    # tall matrices in a batch: transposed, iterated, transposed back
    T = G.mT.contiguous()
    assert oracle.rel_fro(oracle.newtonschulz(T, 5, torch.float64), got.mT) < 1e-12
    e = oracle.newtonschulz_eager_bf16(G, 5)
    assert e.shape == G.shape and e.dtype == torch.bfloat16


def _bf(x):
    """Round a python float / fp32 value to bf16 and back (one torch rounding)."""
    return float(torch.tensor(x, dtype=torch.float32).bfloat16().float())


def test_eager_bf16_scalar_recurrence_on_a_diagonal_input():
    """newtonschulz_eager_bf16 on diag(sigma) is a scalar recurrence per singular value in which
    every torch op of muon.py:23-29 rounds to bf16: written out here op by op (norm, divide, A, A^2,
    b*A, c*A^2, their sum, a*X, B@X, their sum), it has to reproduce the matrix code bit for bit.
    A transposed operand, a dropped term or a missing rounding in the matrix code breaks it."""
    a, b, c = oracle.NS_COEFFS
    sig = [1.0, 0.5, 0.11, 0.013]
    G = torch.diag(torch.tensor(sig, dtype=torch.float32))
    got = torch.diagonal(oracle.newtonschulz_eager_bf16(G, 5)).float().tolist()
    xs = [_bf(v) for v in sig]
    norm = _bf(math.sqrt(sum(v * v for v in xs)))           # X.norm() comes back as a bf16 scalar
    den = _bf(norm + oracle.NS_EPS)
    xs = [_bf(v / den) for v in xs]
    for _ in range(5):
        nxt = []
        for x in xs:
            A = _bf(x * x)
            A2 = _bf(A * A)
            B = _bf(_bf(b * A) + _bf(c * A2))
            nxt.append(_bf(_bf(a * x) + _bf(B * x)))
        xs = nxt
    assert got == xs
    off = oracle.newtonschulz_eager_bf16(G, 5).float() - torch.diag(torch.tensor(got))
    assert float(off.abs().max()) == 0.0


def test_eager_bf16_close_to_fp32():
    g = torch.Generator().manual_seed(11)
    G = torch.randn(64, 96, generator=g)
    e = oracle.newtonschulz_eager_bf16(G, 5)
    r = oracle.newtonschulz(G, 5)
    assert e.dtype == torch.bfloat16 and e.shape == G.shape
    assert oracle.rel_fro(e, r) < 5e-2


def test_momentum_and_weight_update_closed_forms():
    mu, lr, wd = 0.95, 0.02, 0.01
    g = torch.tensor([[1.0, -2.0], [0.5, 4.0]], dtype=torch.float64)
    used, nb, ng = oracle.momentum_nesterov(g, torch.zeros_like(g), mu, True)
    assert torch.allclose(nb, (1 - mu) * g, rtol=1e-14)
    assert torch.allclose(ng, (1 - mu * mu) * g, rtol=1e-14)   # g + mu((1-mu)g - g)
    assert used is ng
    used2, nb2, ng2 = oracle.momentum_nesterov(g, torch.zeros_like(g), mu, False)
    assert used2 is nb2 and ng2 is g
    # second step of the recurrence
    g2 = torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=torch.float64)
    _, nb3, ng3 = oracle.momentum_nesterov(g2, nb, mu, True)
    assert torch.allclose(nb3, mu * (1 - mu) * g + (1 - mu) * g2, rtol=1e-14)
    assert torch.allclose(ng3, (1 - mu) * g2 + mu * nb3, rtol=1e-14)
    # weight update: tall parameter gets sqrt(rows/cols), wide gets 1
    p = torch.ones(8, 2, dtype=torch.float64)
    u = torch.full((16,), 0.5, dtype=torch.float64)
    assert torch.allclose(oracle.weight_update(p, u, lr, wd), torch.full((8, 2), 1 - lr * wd - lr * 2.0 * 0.5, dtype=torch.float64))
    p = torch.ones(2, 8, dtype=torch.float64)
    assert torch.allclose(oracle.weight_update(p, u, lr, wd), torch.full((2, 8), 1 - lr * wd - lr * 0.5, dtype=torch.float64))


def test_muon_first_step_closed_form():
    g = torch.Generator().manual_seed(9)
    p = torch.randn(12, 20, generator=g).bfloat16()
    d = torch.randn(12, 20, generator=g).bfloat16()
    lr, wd, mu = 0.02, 0.01, 0.95
    (np_,), (ng,), (nb,), (u,) = oracle.muon_step([p], [d], [None], lr, wd, mu, True, 5, torch.float64)
    assert torch.allclose(nb, (1 - mu) * d.double(), rtol=1e-12)
    assert torch.allclose(ng, (1 - mu * mu) * d.double(), rtol=1e-12)
    want_u = oracle.newtonschulz(((1 - mu * mu) * d.double()).bfloat16(), 5, torch.float64)
    assert torch.allclose(u, want_u)
    assert torch.allclose(np_, p.double() * (1 - lr * wd) - lr * want_u, rtol=1e-12)
    # 4-D parameter behaves as its (len, -1) view
    p4, d4 = p.reshape(12, 5, 2, 2), d.reshape(12, 5, 2, 2)
    (np4,), _, _, _ = oracle.muon_step([p4], [d4], [None], lr, wd, mu, True, 5, torch.float64)
    scale4 = max(1, 2 / 2) ** 0.5
    assert torch.allclose(np4.reshape(12, 20), p.double() * (1 - lr * wd) - lr * scale4 * want_u, rtol=1e-12)


def test_golden_fixtures_match_oracle():
    """The committed vectors (written by tests/golden/make_golden.py from this oracle) still match."""
    z = np.load(os.path.join(GOLDEN, "ns_small.npz"))
    G = torch.from_numpy(z["G_bf16_bits"].astype(np.int32)).to(torch.int16).view(torch.bfloat16)
    out = oracle.newtonschulz(G, 5)
    assert oracle.rel_fro(out, torch.from_numpy(z["ns5_fp32"])) < 1e-5
    Y = oracle.xxt(G)
    assert oracle.rel_fro(Y, torch.from_numpy(z["xxt_fp32"])) < 1e-6
    sig = torch.from_numpy(z["diag_sigma"])
    want = torch.from_numpy(z["diag_ns5"])
    got = torch.diagonal(oracle.newtonschulz(torch.diag(sig), 5, dtype=torch.float64))
    assert torch.allclose(got, want, rtol=1e-9)
