"""GPU parity of the fused Newton-Schulz kernels and the streaming kernels, each called through
the C ABI: b*A + c*A*A, a*X + P*X (with its transposed second output), sum of squares and the
normalising cast."""
import math

import pytest
import torch

from oracle import oracle
from flash_muon_amd import _lib
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _int_sym(M, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(lo, hi + 1, (M, M), generator=g)
    A = torch.triu(A) + torch.triu(A, 1).T
    return A.float().bfloat16()


@pytest.mark.parametrize("M", [1, 7, 64, 100, 129, 256, 300, 520])
@pytest.mark.parametrize("b,c", [(1.0, 1.0), (2.0, -1.0)])
def test_poly_integer_bit_exact(lib, M, b, c):
    A = _int_sym(M, 40 + M, -1, 1)
    Ai = A.double().round().long()
    want = (int(b) * Ai + int(c) * (Ai @ Ai)).float().bfloat16()
    got = gpu_util.syrk_poly(lib, A.to(DEV), b, c).cpu()
    assert torch.equal(got, want)
    assert torch.equal(got, got.T)


@pytest.mark.parametrize("M", [384, 1024])
def test_poly_gaussian(lib, M):
    g = torch.Generator().manual_seed(M)
    X = torch.randn(M, 2 * M, generator=g) / math.sqrt(2 * M) / 4
    A = (X @ X.T).bfloat16()
    A = torch.triu(A) + torch.triu(A, 1).T            # symmetric bit for bit
    a, b, c = oracle.NS_COEFFS
    Af = A.float()
    ref = b * Af + c * (Af @ Af)
    got = gpu_util.syrk_poly(lib, A.to(DEV), b, c).cpu()
    assert torch.equal(got, got.T)
    assert oracle.rel_fro(got, ref) < 3e-3


@pytest.mark.parametrize("M,K", [(1, 1), (5, 9), (64, 64), (100, 37), (130, 264), (256, 512), (300, 1000), (520, 2056)])
def test_axpby_integer_bit_exact(lib, M, K):
    g = torch.Generator().manual_seed(M * 31 + K)
    P = torch.randint(-1, 2, (M, M), generator=g).float().bfloat16()    # need not be symmetric here
    X = torch.randint(-2, 3, (M, K), generator=g).float().bfloat16()
    want = (2 * X.double() + P.double() @ X.double()).float().bfloat16()
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0)
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    only_x, none_t = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_xt=False)
    assert none_t is None and torch.equal(only_x.cpu(), want)
    none_x, only_t = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_x=False)
    assert none_x is None and torch.equal(only_t.cpu(), want.T)


def test_axpby_gaussian(lib):
    g = torch.Generator().manual_seed(77)
    M, K = 512, 1536
    P = (torch.randn(M, M, generator=g) / math.sqrt(M)).bfloat16()
    X = torch.randn(M, K, generator=g).bfloat16()
    a = oracle.NS_COEFFS[0]
    ref = a * X.float() + P.float() @ X.float()
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), a)
    assert torch.equal(Xo.T.contiguous(), XoT)
    assert oracle.rel_fro(Xo, ref) < 3e-3


def test_split_diagonal_roundtrip(lib):
    """The fp32 diagonal that fm_syrk_poly_bf16 hands out and fm_gemm_axpby_bf16 takes back."""
    M, K = 200, 328
    A = _int_sym(M, 91, -1, 1)
    Ai = A.double().round().long()
    full = (Ai + 2 * (Ai @ Ai))
    P, d = gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0, split_diag=True)
    assert torch.equal(d.cpu().long(), torch.diagonal(full))
    assert (torch.diagonal(P) == 0).all()
    off = full - torch.diag(torch.diagonal(full))
    assert torch.equal(P.cpu(), off.float().bfloat16())
    g = torch.Generator().manual_seed(92)
    X = torch.randint(-1, 2, (M, K), generator=g).float().bfloat16()
    want = (3 * X.double() + full.double() @ X.double()).float().bfloat16()
    Xo, XoT = gpu_util.gemm_axpby(lib, P, X.to(DEV), 3.0, row_alpha=d)
    assert torch.equal(Xo.cpu(), want) and torch.equal(XoT.cpu(), want.T)


def test_axpby_rejects_aliasing(lib):
    X = torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV)
    P = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    XT = torch.zeros(128, 64, dtype=torch.bfloat16, device=DEV)
    st = lib.fm_gemm_axpby_bf16(P.data_ptr(), 64, XT.data_ptr(), 64, X.data_ptr(), 128, X.data_ptr(), 128,
                                None, 0, 64, 128, 1.0, None, None, 0, None)
    assert st == 5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (64, 64), (100, 37), (257, 1000), (128, 384), (640, 128), (1024, 2048)])
def test_sumsq_and_scale_cast(lib, dtype, shape):
    g = torch.Generator().manual_seed(shape[0] + shape[1])
    G = torch.randn(*shape, generator=g).to(dtype)
    Gb = G.bfloat16().double()                          # the reference casts to bf16 first (muon.py:15)
    ss = gpu_util.sumsq(lib, G.to(DEV))
    assert abs(float(ss.cpu()) / float((Gb ** 2).sum()) - 1) < 1e-5
    D, T = gpu_util.scale_cast(lib, G.to(DEV), ss, 1e-7)
    denom = torch.tensor(float(ss.cpu()), dtype=torch.float32).sqrt() + 1e-7
    want = (Gb.float() / denom).bfloat16()
    assert torch.equal(D.cpu(), want)
    assert torch.equal(T.cpu(), want.T)
    D2, none = gpu_util.scale_cast(lib, G.to(DEV), ss, 1e-7, want_t=False)
    assert none is None and torch.equal(D2.cpu(), want)
    none, T2 = gpu_util.scale_cast(lib, G.to(DEV), ss, 1e-7, want_d=False)
    assert none is None and torch.equal(T2.cpu(), want.T)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_scale_cast_of_whole_tiles_with_row_pitches(lib, dtype):
    """Whole 128x128 tiles take a kernel of their own; input and both outputs with rows longer than the matrix."""
    rows, cols = 256, 384
    g = torch.Generator().manual_seed(11)
    big = torch.randn(rows, cols + 64, generator=g).to(dtype).to(DEV)
    G = big[:, :cols]
    ss = gpu_util.sumsq(lib, G)
    denom = torch.tensor(float(ss.cpu()), dtype=torch.float32).sqrt() + 1e-7
    want = (G.cpu().bfloat16().float() / denom).bfloat16()
    Dbig = torch.full((rows, cols + 8), 7.0, dtype=torch.bfloat16, device=DEV)
    Tbig = torch.full((cols, rows + 24), 7.0, dtype=torch.bfloat16, device=DEV)
    st = lib.fm_scale_cast_bf16(G.data_ptr(), _lib.dtype_code(G.dtype), rows, cols, G.stride(0), ss.data_ptr(), 1e-7,
                                Dbig.data_ptr(), Dbig.stride(0), Tbig.data_ptr(), Tbig.stride(0), None)
    assert st == 0
    torch.cuda.synchronize()
    assert torch.equal(Dbig[:, :cols].cpu(), want) and torch.equal(Tbig[:, :rows].cpu(), want.T)
    assert bool((Dbig[:, cols:] == 7.0).all()) and bool((Tbig[:, rows:] == 7.0).all())   # nothing beyond the matrices is touched


def test_sumsq_closed_forms_and_strides(lib):
    ones = torch.ones(96, 160, dtype=torch.bfloat16, device=DEV)
    assert float(gpu_util.sumsq(lib, ones).cpu()) == 96 * 160
    z = torch.zeros(8, 8, dtype=torch.bfloat16, device=DEV)
    ss = gpu_util.sumsq(lib, z)
    assert float(ss.cpu()) == 0.0
    D, T = gpu_util.scale_cast(lib, z, ss, 1e-7)
    assert torch.equal(D.cpu(), torch.zeros(8, 8, dtype=torch.bfloat16))     # eps keeps 0/0 away
    # row-padded input
    big = torch.full((50, 80), 3.0, dtype=torch.bfloat16, device=DEV)
    view = big[:, :33]
    assert float(gpu_util.sumsq(lib, view).cpu()) == 9.0 * 50 * 33
    # two runs give the same bits (fixed reduction tree)
    g = torch.Generator().manual_seed(1)
    G = torch.randn(999, 1001, generator=g).to(DEV)
    assert torch.equal(gpu_util.sumsq(lib, G), gpu_util.sumsq(lib, G))
