"""GPU parity of fast_newtonschulz against the fp32 CPU oracle.

Tolerance: Frobenius-relative error <= 1e-2 per Newton-Schulz step, each step started from the
oracle's state cast to bf16, and <= 1e-2 for the free-running result after the default five
steps on gradient-like inputs."""
import pytest
import torch

from flash_muon_amd import fast_newtonschulz, synthetic
from oracle import oracle
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2
TOL_SMALL = 2e-2


def _tol(rows, cols):
    return TOL if min(rows, cols) >= 128 else TOL_SMALL


@pytest.mark.parametrize("rows,cols,rank,seed", [(256, 1024, 8, 3), (512, 512, 16, 4), (1024, 384, 8, 5), (200, 333, 4, 6)])
def test_per_step_resynchronised(lib, rows, cols, rank, seed):
    G = synthetic.gradient_like_bf16(rows, cols, rank, seed)
    _, states = oracle.newtonschulz(G, 5, trace=True)          # wide orientation, fp32
    for s in range(5):
        Xin = states[s].bfloat16()
        ref = oracle.ns_step(Xin.float())
        Xo, XoT, A, P = gpu_util.ns_step(lib, Xin.to(DEV), oracle.NS_COEFFS)
        err = oracle.rel_fro(Xo, ref)
        print("step %d: rel_fro %.3e" % (s + 1, err), flush=True)
        assert err < TOL
        assert torch.equal(A, A.T) and torch.equal(P, P.T)
        assert torch.equal(XoT, Xo.T.contiguous())


@pytest.mark.parametrize("rows,cols,rank,seed", [(256, 1024, 8, 3), (512, 512, 16, 4), (1024, 384, 8, 5),
                                                 (200, 333, 4, 6), (1, 7, 1, 7), (64, 64, 4, 8)])
def test_free_running_five_steps(rows, cols, rank, seed):
    G = synthetic.gradient_like_bf16(rows, cols, rank, seed)
    ref = oracle.newtonschulz(G, 5)
    got = fast_newtonschulz(G.to(DEV), 5)
    assert got.dtype == torch.bfloat16 and got.shape == G.shape
    err = oracle.rel_fro(got, ref)
    print("free-running 5 steps %dx%d: rel_fro %.3e" % (rows, cols, err), flush=True)
    assert err < _tol(rows, cols)
    # never worse than the reference's own rounding order on the same input
    assert err < 1.2 * oracle.rel_fro(oracle.newtonschulz_eager_bf16(G, 5), ref)


@pytest.mark.parametrize("steps", [0, 1, 2, 3])
def test_step_counts(steps):
    G = synthetic.gradient_like_bf16(128, 320, 4, 21)
    ref = oracle.newtonschulz(G, steps)
    got = fast_newtonschulz(G.to(DEV), steps)
    assert oracle.rel_fro(got, ref) < TOL
    if steps == 0:
        assert abs(float(got.float().norm()) - 1.0) < 5e-3


def test_transpose_invariance_bitwise():
    G = synthetic.gradient_like_bf16(192, 448, 4, 22).to(DEV)
    wide = fast_newtonschulz(G, 5)
    tall = fast_newtonschulz(G.T.contiguous(), 5)
    assert torch.equal(wide, tall.T)
    view = fast_newtonschulz(G.T, 5)                    # transposed view, no copy
    assert torch.equal(view, tall)


def test_diagonal_closed_form():
    sig = torch.tensor([1.0, 0.5, 0.25, 0.125, 0.0625])
    a, b, c = oracle.NS_COEFFS
    s = (sig / sig.norm()).double()
    for _ in range(5):
        s = a * s + b * s ** 3 + c * s ** 5
    got = fast_newtonschulz(torch.diag(sig).to(DEV), 5).cpu().double()
    # five isolated singular values: no averaging, and the quintic's slope reaches 1.5 on [0.7, 1.2]
    assert (torch.diagonal(got) - s).abs().max() < 6e-2
    assert (got - torch.diag(torch.diagonal(got))).abs().max() == 0


def test_input_dtypes_and_scale_invariance():
    G = synthetic.gradient_like_bf16(160, 288, 4, 23)
    base = fast_newtonschulz(G.to(DEV), 5)
    assert torch.equal(fast_newtonschulz(G.float().to(DEV), 5), base)       # same values after the bf16 cast
    assert torch.equal(fast_newtonschulz(G.double().to(DEV), 5), base)
    scaled = fast_newtonschulz((G * 8).to(DEV), 5)                           # power of two: same mantissas
    assert oracle.rel_fro(scaled, base.float()) < 1e-2
    h = fast_newtonschulz(G.half().to(DEV), 5)
    assert oracle.rel_fro(h, oracle.newtonschulz(G.half(), 5)) < TOL


def test_zero_and_padded_inputs():
    z = fast_newtonschulz(torch.zeros(32, 48, device=DEV), 5)
    assert torch.equal(z.cpu(), torch.zeros(32, 48, dtype=torch.bfloat16))
    G = synthetic.gradient_like_bf16(96, 200, 4, 24)
    pad = torch.zeros(96, 256, dtype=torch.bfloat16, device=DEV)
    pad[:, :200] = G.to(DEV)
    assert torch.equal(fast_newtonschulz(pad[:, :200], 5), fast_newtonschulz(G.to(DEV), 5))
    assert fast_newtonschulz(torch.zeros(0, 8, device=DEV)).shape == (0, 8)


def test_singular_values_land_in_band():
    G = synthetic.gradient_like_bf16(512, 2048, 8, 25)
    out = fast_newtonschulz(G.to(DEV), 5).float().cpu()
    sv = torch.linalg.svdvals(out)
    # the leading singular values (the spike and the bulk above ~1e-3 of the norm) end near 1
    assert sv[0] < 1.3 and sv[:8].min() > 0.5


@pytest.mark.parametrize("rows,cols", [(256, 768), (640, 256), (200, 333)])
def test_batched_matches_single_and_oracle(lib, rows, cols):
    """One launch per stage over several matrices of a shape (fm_newtonschulz_batched_bf16): every
    matrix meets the oracle at the same tolerance as alone, and a batch of one is the single call."""
    import ctypes
    from flash_muon_amd import _lib
    Gs = [synthetic.gradient_like_bf16(rows, cols, 4, 40 + i).to(DEV) for i in range(5)]
    outs = [torch.empty(rows, cols, dtype=torch.bfloat16, device=DEV) for _ in Gs]
    a, b, c = oracle.NS_COEFFS
    n = len(Gs)
    ws = torch.empty(lib.fm_newtonschulz_batched_workspace_bytes(n, rows, cols), dtype=torch.uint8, device=DEV)
    st = lib.fm_newtonschulz_batched_bf16((ctypes.c_void_p * n)(*[g.data_ptr() for g in Gs]), 0, n, rows, cols, cols,
                                          (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs]), cols, 5, a, b, c, 1e-7,
                                          ws.data_ptr(), ws.numel(), _lib.stream_ptr(Gs[0].device))
    assert st == 0
    for G, out in zip(Gs, outs):
        single = fast_newtonschulz(G, 5)
        ref = oracle.newtonschulz(G.cpu(), 5)
        assert oracle.rel_fro(out, ref) < TOL
        # the batch changes which tiles fall into the split last round, hence fp32 summation order
        assert oracle.rel_fro(out, single.float()) < TOL
    # too many matrices, a missing pointer and an output aliasing another input are refused
    assert lib.fm_newtonschulz_batched_bf16((ctypes.c_void_p * 33)(), 0, 33, rows, cols, cols, (ctypes.c_void_p * 33)(), cols,
                                            5, a, b, c, 1e-7, ws.data_ptr(), ws.numel(), None) == 2
    assert lib.fm_newtonschulz_batched_bf16((ctypes.c_void_p * 2)(Gs[0].data_ptr(), None), 0, 2, rows, cols, cols,
                                            (ctypes.c_void_p * 2)(outs[0].data_ptr(), outs[1].data_ptr()), cols,
                                            5, a, b, c, 1e-7, ws.data_ptr(), ws.numel(), None) == 1
    assert lib.fm_newtonschulz_batched_bf16((ctypes.c_void_p * 2)(Gs[0].data_ptr(), Gs[1].data_ptr()), 0, 2, rows, cols, cols,
                                            (ctypes.c_void_p * 2)(outs[0].data_ptr(), Gs[0].data_ptr()), cols,
                                            5, a, b, c, 1e-7, ws.data_ptr(), ws.numel(), None) == 5


def test_leading_dimensions_are_a_batch():
    """ndim > 2: every matrix of the leading dimensions is orthogonalised on its own (the norm of
    muon.py:23 is over the last two dimensions), here 35 of them in chunks of 18 and 17."""
    g = torch.Generator().manual_seed(31)
    G = (1e-3 * torch.randn(35, 96, 160, generator=g)).bfloat16().to(DEV)
    out = fast_newtonschulz(G, 5)
    assert out.shape == G.shape and out.dtype == torch.bfloat16
    # against the CPU oracle on the whole batch (per-matrix norms, muon.py:23), every member
    Gc = G.cpu().clone()
    Gc[3] *= 64.0                                     # norms that differ between members
    ref = oracle.newtonschulz(Gc, 5)
    got = fast_newtonschulz(Gc.to(DEV), 5)
    for i in range(G.size(0)):
        err = oracle.rel_fro(got[i], ref[i])
        assert err < _tol(96, 160), "member %d: %g" % (i, err)
    tall_ref = oracle.newtonschulz(Gc[:4].mT.contiguous(), 5)
    tall_got = fast_newtonschulz(Gc[:4].mT.contiguous().to(DEV), 5)
    assert tall_got.shape == (4, 160, 96)
    assert oracle.rel_fro(tall_got, tall_ref) < _tol(96, 160)
    for i in (0, 7, 31, 32, 34):
        assert torch.equal(out[i], fast_newtonschulz(G[i], 5))
    G4 = G[:6].reshape(2, 3, 96, 160)
    assert torch.equal(fast_newtonschulz(G4, 5), out[:6].reshape(2, 3, 96, 160))
    tall = G[:3].mT                                  # a batch of transposed views
    assert torch.equal(fast_newtonschulz(tall, 5), out[:3].mT)
