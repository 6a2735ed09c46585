"""The 128x128 copy-fed path of the GEMM-shaped kernels: whole 128-tiles, k a multiple of 64, too
little work for the 256x256 rounds (or an output that is not a whole number of 256-tiles).
Integer-valued inputs make every comparison bit-exact."""
import pytest
import torch

from flash_muon_amd import matmul_transpose
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ints(shape, seed, lo=-2, hi=2, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).float().to(dtype)


# 1 tile and 1 k stage; fewer stages than the ring is deep; odd tile counts; config 1 (1024^2);
# more tiles than CUs
SYRK_SHAPES = [(128, 64), (128, 128), (128, 192), (384, 320), (640, 1024), (1024, 1024), (1152, 2048),
               (2048, 2048), (3200, 256)]


@pytest.mark.parametrize("M,K", SYRK_SHAPES)
def test_syrk_integer_bit_exact(lib, M, K):
    X = _ints((M, K), 11 * M + K)
    want = (X.double() @ X.double().T).float().bfloat16()
    Y = torch.full((M, M), 7.0, dtype=torch.bfloat16, device=DEV)
    gpu_util.syrk(lib, X.to(DEV), Y)
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


@pytest.mark.parametrize("M,K", [(128, 64), (640, 1024), (2048, 2048)])
def test_syrk_f16_integer_bit_exact(M, K):
    X = _ints((M, K), 13 * M + K, dtype=torch.float16)
    want = (X.double() @ X.double().T).half()
    assert torch.equal(matmul_transpose(X.to(DEV)).cpu(), want)


@pytest.mark.parametrize("M", [128, 384, 1024, 1280])
def test_poly_integer_bit_exact(lib, M):
    g = torch.Generator().manual_seed(M)
    A = torch.randint(-1, 2, (M, M), generator=g)
    A = (torch.triu(A) + torch.triu(A, 1).T).float().bfloat16()
    Ad = A.double()
    full = Ad + 2 * (Ad @ Ad)
    assert torch.equal(gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0).cpu(), full.float().bfloat16())
    P, d = gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0, split_diag=True)
    assert torch.equal(d.cpu().double(), torch.diagonal(full))
    assert torch.equal(P.cpu(), (full - torch.diag(torch.diagonal(full))).float().bfloat16())
    assert torch.equal(P, P.T)


@pytest.mark.parametrize("M,K", [(128, 128), (384, 640), (1024, 1024), (640, 2048), (128, 4096)])
def test_axpby_integer_bit_exact(lib, M, K):
    P = _ints((M, M), 3 * M + K, -1, 1)
    X = _ints((M, K), 5 * M + K)
    d = torch.arange(M, dtype=torch.float32) % 3 - 1            # per-row addition to a
    want = ((2 + d.double())[:, None] * X.double() + P.double() @ X.double()).float().bfloat16()
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, row_alpha=d.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    only_t = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_x=False, row_alpha=d.to(DEV))[1]
    assert torch.equal(only_t.cpu(), want.T)
    only_x = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_xt=False)[0]
    assert torch.equal(only_x.cpu(), (2 * X.double() + P.double() @ X.double()).float().bfloat16())


def test_agrees_with_the_general_path_on_gaussian_input(lib, knobs):
    """Same bf16 input through this path and, with it switched off, through the general tiled
    path: both are one rounding of an fp32 sum, so they agree to within that rounding."""
    g = torch.Generator().manual_seed(5)
    X = torch.randn(1024, 2048, generator=g).bfloat16().to(DEV)
    mid = gpu_util.syrk(lib, X)
    knobs("FLASHMUON_NO_MID", 1)
    gen = gpu_util.syrk(lib, X)
    ref = X.float() @ X.float().T
    for Y in (mid, gen):
        assert torch.equal(Y, Y.T)
        assert float((Y.float() - ref).norm() / ref.norm()) < 3e-3
    assert float((mid.float() - gen.float()).norm() / ref.norm()) < 3e-3


@pytest.fixture
def no_256_path(knobs):
    knobs("FLASHMUON_FAST_MIN_UNITS", 10 ** 15)   # whatever the shape, not the 256x256 path


@pytest.mark.parametrize("ksplit", [2, 3, 5, 16, 64])
@pytest.mark.parametrize("M,K", [(128, 1024), (384, 640), (640, 2048), (256, 4096)])
def test_syrk_tiles_cut_along_k(lib, knobs, no_256_path, M, K, ksplit):
    """Every 128x128 tile cut into `ksplit` parts along k (the KSPLIT knob; more parts than k stages
    are capped), their fp32 sums added in k order by the second kernel."""
    knobs("FLASHMUON_KSPLIT", ksplit)
    X = _ints((M, K), 17 * M + K + ksplit)
    want = (X.double() @ X.double().T).float().bfloat16()
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=DEV)
    gpu_util.syrk(lib, X.to(DEV), Y)
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


@pytest.mark.parametrize("ksplit", [2, 7])
def test_poly_axpby_and_f16_tiles_cut_along_k(lib, knobs, no_256_path, ksplit):
    knobs("FLASHMUON_KSPLIT", ksplit)
    M, K = 512, 1280
    g = torch.Generator().manual_seed(M + ksplit)
    A = torch.randint(-1, 2, (M, M), generator=g)
    A = (torch.triu(A) + torch.triu(A, 1).T).float().bfloat16()
    Ad = A.double()
    full = Ad + 2 * (Ad @ Ad)
    P, d = gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0, split_diag=True)
    assert torch.equal(d.cpu().double(), torch.diagonal(full))
    assert torch.equal(P.cpu(), (full - torch.diag(torch.diagonal(full))).float().bfloat16())
    X = _ints((M, K), 5 * M + K + ksplit)
    ra = torch.arange(M, dtype=torch.float32) % 3 - 1
    want = ((2 + ra.double())[:, None] * X.double() + Ad @ X.double()).float().bfloat16()
    Xo, XoT = gpu_util.gemm_axpby(lib, A.to(DEV), X.to(DEV), 2.0, row_alpha=ra.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    Xh = _ints((M, K), 7 * M + K, dtype=torch.float16)
    assert torch.equal(matmul_transpose(Xh.to(DEV)).cpu(), (Xh.double() @ Xh.double().T).half())


@pytest.mark.parametrize("M,K", [(768, 3072), (1024, 8192)])
def test_few_tiles_long_k_chosen_by_shape(lib, knobs, M, K):
    """Left to the library these shapes are cut along k; against the same tiles whole (KSPLIT = 1),
    to within the rounding of the fp32 sums' different grouping, and against the fp32 product."""
    g = torch.Generator().manual_seed(M + K)
    X = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    auto = matmul_transpose(X)
    knobs("FLASHMUON_KSPLIT", 1)
    whole = matmul_transpose(X)
    ref = X.float() @ X.float().T
    assert torch.equal(auto, auto.T)
    for Y in (auto, whole):
        assert float((Y.float() - ref).norm() / ref.norm()) < 3e-3
    assert float((auto.float() - whole.float()).norm() / ref.norm()) < 3e-3


def test_batched_newtonschulz_with_tiles_cut_along_k(lib, knobs, no_256_path):
    """Three matrices per launch, every 128x128 tile of every product cut into 2 parts along k: the
    tile list and the parts' slots run over the whole batch (at most 90 x 2 parts, which the 256
    slots of the workspace hold; with more the tiles would stay whole).  Against one matrix at a time
    with the same cut (bitwise) and the tiles whole (to the rounding of the regrouped fp32 sums)."""
    from flash_muon_amd import fast_newtonschulz
    g = torch.Generator().manual_seed(21)
    G = torch.randn(3, 384, 1280, generator=g).bfloat16().to(DEV)
    knobs("FLASHMUON_KSPLIT", 2)
    cut = fast_newtonschulz(G, steps=5)
    for i in range(3):
        assert torch.equal(cut[i], fast_newtonschulz(G[i], steps=5))
    knobs("FLASHMUON_KSPLIT", 1)
    whole = fast_newtonschulz(G, steps=5)
    assert float((cut.float() - whole.float()).norm() / whole.float().norm()) < 2e-2
