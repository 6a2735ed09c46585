"""CPU oracle for the flash-muon hot path.  TEST INFRASTRUCTURE ONLY.

This module restates the reference's algorithm in plain torch on the CPU (fp32, optionally fp64).
It is imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py as
the checker or the timed CPU baseline; nothing in flash_muon_amd/ imports it and nothing here
is ever used to produce a result the library returns.

What each function follows in the reference (/root/reference):
    xxt                 benchmark.py:20-21 (`G @ G.T`), the value flash_muon/matmul_transpose_triton.py:20-75 computes
    ns_prepare          flash_muon/muon.py:15-17, 23   (bf16 cast, transpose-if-tall, Frobenius normalise)
    ns_step             flash_muon/muon.py:26-29        (A = XX^T, B = bA + cAA, X = aX + BX)
    newtonschulz        flash_muon/muon.py:6-33 and benchmark.py:23-47
    newtonschulz_eager_bf16  the same lines with a bf16 rounding after every torch op, as the
                        reference executes them
    momentum_nesterov   flash_muon/muon.py:99-100
    weight_update       flash_muon/muon.py:87-89
    muon_step           flash_muon/muon.py:76-110 at world_size == 1

How the oracle itself is pinned (tests/test_oracle.py; the reference ships no tests, golden
vectors or fixtures for this path, and its Triton/CUDA code cannot run without a GPU):
    xxt           against an int64 brute force on integer-valued inputs, and identity / all-ones /
                  Hadamard closed forms;
    newtonschulz  against the closed form U diag(p^steps(sigma/|sigma|)) V^T computed from an
                  fp64 SVD and a scalar recurrence, plus NS(G^T) == NS(G)^T and scale invariance;
    momentum_nesterov, weight_update, muon_step   against the first- and second-step closed
                  forms of the lerp recurrences written out by hand in fp64.
The low-order bits of the reference's own bf16 outputs depend on its autotuned tile shape
(matmul_transpose_triton.py:6-18) and are outside the contract; no function here claims them.
"""
import torch

NS_COEFFS = (3.4445, -4.7750, 2.0315)   # flash_muon/muon.py:14
NS_EPS = 1e-7                            # flash_muon/muon.py:23


def xxt(X, dtype=torch.float32):
    """X @ X.T of the values X holds, accumulated in `dtype` (benchmark.py:20-21)."""
    Xf = X.detach().cpu().to(dtype)
    return Xf @ Xf.T


def xxt_int64(X):
    """Brute-force X @ X.T for integer-valued X in int64 (exact)."""
    Xi = X.detach().cpu().to(torch.float64).round().to(torch.int64)
    return Xi @ Xi.T


def ns_prepare(G, dtype=torch.float32):
    """bf16-cast G, take the wide orientation and Frobenius-normalise (muon.py:15-17, 23).

    Returns (X, tall).  The norm is kept in `dtype`; the reference's is rounded to bf16, a uniform
    scale error of at most 2^-9 that Newton-Schulz is insensitive to.
    """
    X = G.detach().cpu().bfloat16().to(dtype)
    tall = G.size(-2) > G.size(-1)
    if tall:
        X = X.mT
    # the norm is taken over the last two dimensions (muon.py:23): leading ones are a batch
    X = X / (X.norm(dim=(-2, -1), keepdim=True) + NS_EPS)
    return X.contiguous(), tall


def ns_step(X, coeffs=NS_COEFFS):
    """One quintic iteration in X's dtype (muon.py:26-29)."""
    a, b, c = coeffs
    A = X @ X.mT
    B = b * A + c * (A @ A)
    return a * X + B @ X


def newtonschulz(G, steps=5, dtype=torch.float32, trace=False):
    """fast_newtonschulz computed without intermediate bf16 roundings (muon.py:6-33).

    Returns the result in `dtype` with G's shape; with trace=True also the list of iterates in the
    wide orientation (X_0 after normalisation, then one per step).  Leading dimensions of G are a
    batch of independent matrices, each normalised by its own norm (muon.py:13, 23).
    """
    X, tall = ns_prepare(G, dtype)
    states = [X]
    for _ in range(steps):
        X = ns_step(X)
        states.append(X)
    out = X.mT if tall else X
    return (out, states) if trace else out


def newtonschulz_eager_bf16(G, steps=5):
    """The reference's own op sequence on the CPU: every torch op rounds to bf16 (muon.py:15-32)."""
    a, b, c = NS_COEFFS
    X = G.detach().cpu().bfloat16()
    tall = G.size(-2) > G.size(-1)
    if tall:
        X = X.mT
    X = X / (X.norm(dim=(-2, -1), keepdim=True) + NS_EPS)
    for _ in range(steps):
        A = (X.float() @ X.float().mT).bfloat16()
        A2 = (A.float() @ A.float().mT).bfloat16()
        B = b * A + c * A2
        X = a * X + (B.float() @ X.float()).bfloat16()
    return X.mT if tall else X


def lerp(start, end, weight):
    """start + weight * (end - start) (the value torch.lerp computes)."""
    return start + weight * (end - start)


def momentum_nesterov(g, buf, momentum, nesterov=True):
    """Returns (g_used, new_buf, new_grad) for muon.py:99-100 in the inputs' dtype, no rounding."""
    new_buf = lerp(buf, g, 1 - momentum)
    if nesterov:
        new_g = lerp(g, new_buf, momentum)
        return new_g, new_buf, new_g
    return new_buf, new_buf, g


def weight_update(p, u, lr, weight_decay):
    """p * (1 - lr*wd) - lr * sqrt(max(1, rows/cols)) * u (muon.py:87-89)."""
    scale = max(1, p.size(-2) / p.size(-1)) ** 0.5
    return p * (1 - lr * weight_decay) - lr * scale * u.reshape(p.shape)


def muon_step(params, grads, bufs, lr=0.02, weight_decay=0.01, momentum=0.95, nesterov=True,
              ns_steps=5, dtype=torch.float32):
    """One optimizer step at world_size == 1 (muon.py:76-110) on CPU copies, in `dtype`.

    params, grads, bufs are lists of tensors (bufs entries may be None for a fresh state).
    Returns (new_params, new_grads, new_bufs, updates).
    """
    new_p, new_g, new_b, ups = [], [], [], []
    for p, g, buf in zip(params, grads, bufs):
        pf = p.detach().cpu().to(dtype)
        gf = g.detach().cpu().to(dtype)
        bf = torch.zeros_like(gf) if buf is None else buf.detach().cpu().to(dtype)
        used, nb, ng = momentum_nesterov(gf, bf, momentum, nesterov)
        m = used.reshape(len(used), -1) if used.ndim == 4 else used
        # the reference hands NS the tensor in the gradient's storage dtype
        u = newtonschulz(m.to(g.dtype), ns_steps, dtype)
        new_p.append(weight_update(pf, u, lr, weight_decay))
        new_g.append(ng)
        new_b.append(nb)
        ups.append(u)
    return new_p, new_g, new_b, ups


def rel_fro(Y, R):
    """||Y - R||_F / ||R||_F in fp64: the parity metric for every floating-point comparison."""
    Y = Y.detach().cpu().double()
    R = R.detach().cpu().double()
    return float((Y - R).norm() / R.norm().clamp_min(1e-300))
