"""GPU parity of the fp16 symmetric product (fm_syrk_f16 behind matmul_transpose on float16
tensors; the reference's kernel takes its element type from the input,
matmul_transpose_triton.py:63) against the CPU oracle: bit-exact on integer-valued inputs and
closed forms, bit-exact symmetry, within one fp16 rounding of the fp32 oracle on Gaussian inputs."""
import pytest
import torch

from flash_muon_amd import matmul_transpose, matmul_transpose_assign
from oracle import oracle
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ints(M, K, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (M, K), generator=g).half()


# general path (ragged, unaligned, small) and the 256x256 path (whole tiles, k a multiple of 64,
# several rounds, a split last round)
@pytest.mark.parametrize("M,K", [(1, 1), (5, 3), (64, 64), (100, 37), (129, 72), (257, 513), (1000, 777),
                                 (256, 64), (512, 320), (1280, 2048), (2048, 2048), (4096, 1024)])
def test_integer_inputs_bit_exact(M, K):
    X = _ints(M, K, 300 + M + K)
    want = oracle.xxt_int64(X).double().half()         # |values| <= 4K <= 8192: exact or one rounding
    got = matmul_transpose(X.to(DEV)).cpu()
    assert got.dtype == torch.float16 and got.shape == (M, M)
    assert torch.equal(got, want)
    assert torch.equal(got, got.T)


def test_closed_forms():
    eye = torch.eye(192, dtype=torch.float16)
    assert torch.equal(matmul_transpose(eye.to(DEV)).cpu(), eye)
    ones = torch.ones(70, 128, dtype=torch.float16)
    assert torch.equal(matmul_transpose(ones.to(DEV)).cpu(), torch.full((70, 70), 128.0, dtype=torch.float16))
    # 1/1024 is exact in fp16 but has no bf16 neighbour below 2^-10 resolution at 1: the product
    # (1 + 2^-10)^2 summed over K = 64 separates an fp16 datapath from a bf16 one
    x = torch.full((64, 64), 1.0 + 2.0 ** -10, dtype=torch.float16)
    want = (64.0 * (1.0 + 2.0 ** -10) ** 2 * torch.ones(64, 64, dtype=torch.float64)).half()
    assert torch.equal(matmul_transpose(x.to(DEV)).cpu(), want)
    assert matmul_transpose(torch.zeros(0, 8, dtype=torch.float16, device=DEV)).shape == (0, 0)


@pytest.mark.parametrize("M,K,seed", [(1024, 1024, 0), (700, 333, 2), (2048, 2048, 2048), (4096, 4096, 4096)])
def test_gaussian_against_fp32_oracle(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(M, K, generator=g).half()
    ref = oracle.xxt(X)
    got = matmul_transpose(X.to(DEV)).cpu()
    assert torch.equal(got, got.T)
    assert (torch.diagonal(got).float() >= 0).all()
    # one round-to-nearest fp16 (11 significant bits) of an fp32-accumulated sum
    assert float(oracle.rel_fro(got, ref)) < 4e-4
    # elementwise: half an fp16 ulp of the value plus the fp32 accumulation error of both sides
    err = (got.double() - ref.double()).abs()
    assert bool((err <= ref.double().abs() * 2.0 ** -11 + 2e-5 * K ** 0.5).all())


def test_strided_output_and_mixed_dtypes():
    X = _ints(300, 136, 9).to(DEV)
    big = torch.zeros(300, 700, dtype=torch.float16, device=DEV)
    out = big[:, 5:605:2]
    matmul_transpose_assign(X, out)
    assert torch.equal(out.cpu(), oracle.xxt_int64(X).double().half())
    with pytest.raises(AssertionError):
        matmul_transpose_assign(X, torch.empty(300, 300, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(TypeError):
        matmul_transpose(torch.zeros(8, 8, dtype=torch.int32, device=DEV))


def test_fast_and_general_paths_agree(lib):
    """The same fp16 input through the 256x256 path (with workspace) and the tiled path (without)."""
    g = torch.Generator().manual_seed(11)
    X = torch.randint(-2, 3, (1024, 4096), generator=g).half().to(DEV)
    want = oracle.xxt_int64(X).double().half()
    fast = torch.empty(1024, 1024, dtype=torch.float16, device=DEV)
    ws = gpu_util._ws(lib.fm_gemm_workspace_bytes(1024, 1024), X.device)
    assert lib.fm_syrk_f16(X.data_ptr(), X.stride(0), fast.data_ptr(), 1024, 1, 1024, 4096,
                           ws.data_ptr(), ws.numel(), gpu_util._stream(X)) == 0
    slow = torch.empty_like(fast)
    assert lib.fm_syrk_f16(X.data_ptr(), X.stride(0), slow.data_ptr(), 1024, 1, 1024, 4096, None, 0,
                           gpu_util._stream(X)) == 0
    assert torch.equal(fast.cpu(), want) and torch.equal(slow.cpu(), want)
