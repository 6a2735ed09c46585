"""GPU parity of the fp32 symmetric product (fm_syrk_f32 behind matmul_transpose on float32 tensors;
the reference's kernel takes its element type from the input, matmul_transpose_triton.py:63)
against the CPU oracle: bit-exact on integer-valued inputs and closed forms, bit-exact symmetry,
within fp32 accumulation error of the fp64 oracle on Gaussian inputs."""
import pytest
import torch

from flash_muon_amd import matmul_transpose, matmul_transpose_assign
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ints(M, K, seed, lo=-50, hi=50):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (M, K), generator=g).float()


# single element, below one MFMA tile, ragged M and K, K not a multiple of 4 (element-wise loads),
# K a multiple of 4 but not of 32 (zero-filled tail), several k stages, both tile configurations
@pytest.mark.parametrize("M,K", [(1, 1), (5, 3), (32, 16), (64, 32), (100, 37), (129, 72), (256, 200),
                                 (257, 513), (1000, 777), (640, 1024), (4100, 36)])
def test_integer_inputs_bit_exact(M, K):
    X = _ints(M, K, 500 + M + K)                       # |sums| <= 2500 K < 2^24: exact in fp32
    want = oracle.xxt_int64(X).float()
    got = matmul_transpose(X.to(DEV)).cpu()
    assert got.dtype == torch.float32 and got.shape == (M, M)
    assert torch.equal(got, want)
    assert torch.equal(got, got.T)


def test_closed_forms_and_precision():
    eye = torch.eye(192)
    assert torch.equal(matmul_transpose(eye.to(DEV)).cpu(), eye)
    # 1 + 2^-12 has no bf16 or fp16 neighbour; its square summed over K = 64 is exact in fp32
    # only if the products are formed from all 24 significant bits
    x = torch.full((64, 64), 1.0 + 2.0 ** -12)
    want = torch.full((64, 64), 64.0 * (1.0 + 2.0 ** -12) ** 2, dtype=torch.float64).float()
    assert torch.equal(matmul_transpose(x.to(DEV)).cpu(), want)
    assert matmul_transpose(torch.zeros(0, 8, device=DEV)).shape == (0, 0)
    z = matmul_transpose(torch.zeros(33, 0, device=DEV))
    assert torch.equal(z.cpu(), torch.zeros(33, 33))


@pytest.mark.parametrize("M,K,seed", [(1024, 1024, 0), (700, 333, 2), (2048, 2048, 2048)])
def test_gaussian_against_fp64_oracle(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(M, K, generator=g)
    ref = oracle.xxt(X, dtype=torch.float64)
    got = matmul_transpose(X.to(DEV)).cpu()
    assert torch.equal(got, got.T)
    assert (torch.diagonal(got) >= 0).all()
    # fp32 products and accumulation, no rounding of the result
    assert float(oracle.rel_fro(got, ref)) < 2e-6


def test_strided_output_and_views():
    X = _ints(300, 136, 9).to(DEV)
    big = torch.zeros(300, 700, device=DEV)
    out = big[:, 5:605:2]
    matmul_transpose_assign(X, out)
    assert torch.equal(out.cpu(), oracle.xxt_int64(X).float())
    Xt = _ints(136, 300, 10).to(DEV)                   # a transposed view is copied, as in the reference
    assert torch.equal(matmul_transpose(Xt.T).cpu(), oracle.xxt_int64(Xt.T).float())
