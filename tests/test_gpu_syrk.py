"""GPU parity of the symmetric product (fm_syrk_bf16 behind matmul_transpose) against the CPU
oracle: bit-exact on integer-valued inputs and closed forms, bit-exact symmetry everywhere, and
within one bf16 rounding of the fp32 oracle on Gaussian inputs."""
import pytest
import torch

from flash_muon_amd import matmul_transpose, matmul_transpose_assign, synthetic
from oracle import oracle
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _int_matrix(M, K, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (M, K), generator=g).float().bfloat16()


# shapes cover: single element, M or K below one MFMA tile, ragged M and K, K not a multiple of 8
# (scalar load path), K a multiple of 8 but not of 64 (zero-filled tail), several k stages,
# both tile configurations (128x128 and 256x256) and more than one tile per dimension
INT_SHAPES = [(1, 1), (1, 64), (5, 3), (32, 16), (64, 64), (100, 37), (130, 64), (129, 72),
              (256, 200), (300, 136), (257, 513), (1000, 777), (640, 1024), (4100, 72)]


@pytest.mark.parametrize("M,K", INT_SHAPES)
def test_integer_inputs_bit_exact(M, K):
    X = _int_matrix(M, K, 100 + M + K)
    want = oracle.xxt_int64(X).float().bfloat16()     # exact integer, then the one bf16 rounding
    got = matmul_transpose(X.to(DEV)).cpu()
    assert got.dtype == torch.bfloat16 and got.shape == (M, M)
    assert torch.equal(got, want)
    assert torch.equal(got, got.T)


def test_closed_forms():
    eye = torch.eye(192, dtype=torch.bfloat16)
    assert torch.equal(matmul_transpose(eye.to(DEV)).cpu(), eye)
    ones = torch.ones(70, 128, dtype=torch.bfloat16)
    assert torch.equal(matmul_transpose(ones.to(DEV)).cpu(), torch.full((70, 70), 128.0, dtype=torch.bfloat16))
    H = torch.tensor([[1.0]])
    for _ in range(9):
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    got = matmul_transpose(H.bfloat16().to(DEV)).cpu()
    assert torch.equal(got, (512 * torch.eye(512)).bfloat16())
    z = matmul_transpose(torch.zeros(33, 0, dtype=torch.bfloat16, device=DEV))
    assert torch.equal(z.cpu(), torch.zeros(33, 33, dtype=torch.bfloat16))
    assert matmul_transpose(torch.zeros(0, 8, dtype=torch.bfloat16, device=DEV)).shape == (0, 0)


@pytest.mark.parametrize("M,K,seed", [(1024, 1024, 0), (96, 4096, 1), (700, 333, 2), (2048, 2048, 2048)])
def test_gaussian_against_fp32_oracle(M, K, seed):
    # config 1 of the benchmark set is the first case (1024 x 1024, seed 0)
    X = synthetic.gaussian_bf16(M, K, seed)
    ref = oracle.xxt(X)
    got = matmul_transpose(X.to(DEV)).cpu()
    assert torch.equal(got, got.T)                      # bit-exact symmetry
    assert (torch.diagonal(got).float() >= 0).all()
    # one round-to-nearest bf16 of an fp32-accumulated sum: Frobenius-relative error about 2^-9/sqrt(3)
    assert oracle.rel_fro(got, ref) < 3e-3
    # elementwise: half an ulp of bf16 (2^-9 relative) plus fp32 accumulation slack
    err = (got.float() - ref).abs()
    bound = ref.abs() * 2.0 ** -8 + 1e-3 * K ** 0.5
    assert (err <= bound).all()


@pytest.mark.parametrize("dim", [4096, 8192])
def test_large_square_symmetry_and_sampled_rows(dim):
    X = synthetic.gaussian_bf16(dim, dim, dim)
    Y = matmul_transpose(X.to(DEV))
    assert torch.equal(Y, Y.T)
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 257, dim // 2 - 1, dim // 2, dim - 257, dim - 2, dim - 1])
    ref = X[rows].float() @ X.float().T
    got = Y[rows.to(DEV)].cpu()
    assert oracle.rel_fro(got, ref) < 3e-3
    # linearity check that needs no CPU product: (2X)(2X)^T == 4 XX^T exactly in bf16
    Y2 = matmul_transpose((X * 2).to(DEV))
    assert torch.equal(Y2, Y * 4)


def test_output_strides_and_input_views():
    X = _int_matrix(200, 96, 5)
    want = oracle.xxt_int64(X).float().bfloat16()
    Xd = X.to(DEV)
    # transposed output view
    Yt = torch.zeros(200, 200, dtype=torch.bfloat16, device=DEV)
    matmul_transpose_assign(Xd, Yt.T)
    assert torch.equal(Yt.cpu(), want)
    # padded rows
    big = torch.full((200, 260), 7.0, dtype=torch.bfloat16, device=DEV)
    matmul_transpose_assign(Xd, big[:, :200])
    assert torch.equal(big[:, :200].cpu(), want)
    assert (big[:, 200:] == 7).all()                    # nothing written past the view
    # both strides non-unit
    big = torch.full((400, 600), 7.0, dtype=torch.bfloat16, device=DEV)
    view = big[::2, ::3]
    matmul_transpose_assign(Xd, view)
    assert torch.equal(view.cpu(), want)
    assert (big[1::2] == 7).all() and (big[:, 1::3] == 7).all()
    # input: a transposed view (copied, as the reference's .contiguous() does) and a row-padded view
    XT = X.T.contiguous().to(DEV)
    assert torch.equal(matmul_transpose(XT.T).cpu(), want)
    pad = torch.zeros(200, 128, dtype=torch.bfloat16, device=DEV)
    pad[:, :96] = Xd
    assert torch.equal(matmul_transpose(pad[:, :96]).cpu(), want)
    # misaligned base pointer (odd element offset) goes through the scalar load path
    flat = torch.zeros(200 * 96 + 1, dtype=torch.bfloat16, device=DEV)
    flat[1:] = Xd.flatten()
    assert torch.equal(matmul_transpose(flat[1:].view(200, 96)).cpu(), want)


def test_argument_contract_on_device():
    x = torch.zeros(8, 8, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError, match="same data type"):
        matmul_transpose_assign(x, torch.zeros(8, 8, dtype=torch.float16, device=DEV))
    with pytest.raises(AssertionError, match="2D tensor"):
        matmul_transpose_assign(x.view(2, 4, 8), x)
    with pytest.raises(AssertionError, match="First dimension"):
        matmul_transpose_assign(x, torch.zeros(8, 9, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(AssertionError, match="must be a CUDA tensor"):
        matmul_transpose_assign(x, torch.zeros(8, 8, dtype=torch.bfloat16))
    with pytest.raises(TypeError):
        matmul_transpose(torch.zeros(8, 8, dtype=torch.float64, device=DEV))


def test_direct_c_abi_call(lib):
    X = _int_matrix(96, 64, 9).to(DEV)
    Y = gpu_util.syrk(lib, X)
    assert torch.equal(Y.cpu(), oracle.xxt_int64(X).float().bfloat16())
