"""The half-tile schedule of the 256x256 path: items of 128x256, a diagonal tile of a symmetric
product as one item whose waves take the lower triangles of its two diagonal squares and the
square between them.  It is chosen by shape when all items fit into one round; the HALF knob
forces it here (and FAST_MIN_UNITS = 0 lets small inputs take the 256x256 path at all), the GRID
knob makes several rounds and part-filled last rounds.  Integer-valued inputs make every
comparison with the fp64 product bit-exact."""
import pytest
import torch

from flash_muon_amd import _lib, matmul_transpose
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _half_tiles(knobs):
    knobs("FLASHMUON_FAST_MIN_UNITS", 0)
    knobs("FLASHMUON_HALF", 1)


def _ints(shape, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).float().bfloat16()


def _exact(x):   # exact integer matrix product in fp64, then the single rounding
    return x.float().bfloat16()


# (M, K): one diagonal item and one stage; odd stage counts around the 3-slot ring of the diagonal
# item and the 6-stage loop of the others; tile grids of 2..10 (the 8x8 blocks of the tile order end
# inside 9 and 10)
SYRK_SHAPES = [(256, 64), (256, 128), (256, 192), (256, 256), (256, 448), (512, 64), (512, 320), (768, 1024),
               (1024, 576), (2048, 2048), (2304, 192), (2560, 128), (1280, 8192)]


@pytest.mark.parametrize("M,K", SYRK_SHAPES)
def test_syrk_half_tiles_integer_bit_exact(lib, M, K):
    X = _ints((M, K), M + K)
    want = _exact(X.double() @ X.double().T)
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=DEV)
    gpu_util.syrk(lib, X.to(DEV), Y)
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


@pytest.mark.parametrize("grid", [1, 3, 7, 8, 20, 33])
@pytest.mark.parametrize("M,K", [(1280, 512), (2048, 448), (2304, 128)])
def test_syrk_half_tiles_small_grids(lib, knobs, M, K, grid):
    """Several rounds of items and last rounds of every fill."""
    knobs("FLASHMUON_GRID", grid)
    X = _ints((M, K), 3 * M + K + grid)
    want = _exact(X.double() @ X.double().T)
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=DEV)
    gpu_util.syrk(lib, X.to(DEV), Y)
    assert torch.equal(Y.cpu(), want)


def test_syrk_half_tiles_strided_output_and_input_view(lib):
    M, K = 768, 320
    big = _ints((M, K + 64), 5)
    X = big[:, 32:32 + K]                    # a view with a row stride of K + 64
    want = _exact(X.double() @ X.double().T)
    Ybig = torch.full((M, M + 128), float("nan"), dtype=torch.bfloat16, device=DEV)
    Y = Ybig[:, 64:64 + M]
    Xd = big.to(DEV)[:, 32:32 + K]
    gpu_util.syrk(lib, Xd, Y)
    assert torch.equal(Y.cpu(), want)
    assert torch.isnan(Ybig[:, :64]).all() and torch.isnan(Ybig[:, 64 + M:]).all()


@pytest.mark.parametrize("M", [256, 512, 1024, 1536, 2304])
def test_poly_half_tiles_integer_bit_exact(lib, M):
    g = torch.Generator().manual_seed(M)
    A = torch.randint(-1, 2, (M, M), generator=g)
    A = (torch.triu(A) + torch.triu(A, 1).T).float().bfloat16()
    Ad = A.double()
    full = Ad + 2 * (Ad @ Ad)
    assert torch.equal(gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0).cpu(), _exact(full))
    P, d = gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0, split_diag=True)
    assert torch.equal(d.cpu().double(), torch.diagonal(full))
    assert torch.equal(P.cpu(), _exact(full - torch.diag(torch.diagonal(full))))
    assert torch.equal(P, P.T)
    # any beta: c = 3 takes the other instance of the kernel than c = 1 would
    full3 = 2 * Ad + 3 * (Ad @ Ad)
    assert torch.equal(gpu_util.syrk_poly(lib, A.to(DEV), 2.0, 3.0).cpu(), _exact(full3))


@pytest.mark.parametrize("M,K", [(256, 256), (256, 1280), (512, 768), (1024, 2048), (768, 4096)])
def test_axpby_half_tiles_integer_bit_exact(lib, M, K):
    P = _ints((M, M), 3 * M + K, -1, 1)
    X = _ints((M, K), 5 * M + K)
    d = torch.arange(M, dtype=torch.float32) % 3 - 1
    want = _exact((2 + d.double())[:, None] * X.double() + P.double() @ X.double())
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, row_alpha=d.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    Xo, _ = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_xt=False, row_alpha=d.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    want0 = _exact(2 * X.double() + P.double() @ X.double())
    _, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_x=False)
    assert torch.equal(XoT.cpu(), want0.T)


@pytest.mark.parametrize("M,K", [(256, 64), (512, 320), (1280, 256)])
def test_syrk_f16_half_tiles_integer_bit_exact(lib, M, K):
    g = torch.Generator().manual_seed(M + K)
    X = torch.randint(-2, 3, (M, K), generator=g).to(torch.float16)
    want = (X.double() @ X.double().T).to(torch.float16)
    Xd = X.to(DEV)
    Y = torch.full((M, M), float("nan"), dtype=torch.float16, device=DEV)
    ws = torch.empty(max(int(lib.fm_gemm_workspace_bytes(M, M)), 256), dtype=torch.uint8, device=DEV)
    st = lib.fm_syrk_f16(Xd.data_ptr(), Xd.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), M, K,
                         ws.data_ptr(), ws.numel(), _lib.stream_ptr(Xd.device))
    _lib.check("fm_syrk_f16", st)
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


@pytest.mark.parametrize("M,K", [(3072, 3072), (4096, 1024), (4096, 4096)])
def test_chosen_by_shape_and_equal_to_whole_tiles_on_gaussian_input(lib, knobs, M, K):
    """Left to the library (HALF on automatic), these shapes take the half-tile schedule: every sum
    runs over k in the same order as in a whole tile, so the bits are those of the whole-tile
    schedule, which the other tests of this path pin to the oracle."""
    knobs("FLASHMUON_FAST_MIN_UNITS", -1)
    g = torch.Generator().manual_seed(M + K)
    X = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    knobs("FLASHMUON_HALF", 0)
    whole = matmul_transpose(X)
    knobs("FLASHMUON_HALF", 1)
    forced = matmul_transpose(X)
    knobs("FLASHMUON_HALF", -1)
    auto = matmul_transpose(X)
    assert torch.equal(forced, whole)
    assert torch.equal(auto, whole)
    assert torch.equal(auto, auto.T)
    A = (whole.float() / K).bfloat16()
    knobs("FLASHMUON_HALF", 0)
    Pw, dw = gpu_util.syrk_poly(lib, A, -4.775, 2.0315, split_diag=True)
    knobs("FLASHMUON_HALF", -1)
    Pa, da = gpu_util.syrk_poly(lib, A, -4.775, 2.0315, split_diag=True)
    assert torch.equal(Pa, Pw) and torch.equal(da, dw)


def test_batched_newtonschulz_takes_half_tiles(lib, knobs):
    """Two 1024 x 2048 matrices in one launch: 2 x 16 half items of the symmetric products, 2 x 64 of
    the last product of a step.  Against the same call on whole tiles (bitwise) and one matrix alone."""
    from flash_muon_amd import fast_newtonschulz
    g = torch.Generator().manual_seed(9)
    G = torch.randn(2, 1024, 2048, generator=g).bfloat16().to(DEV)
    knobs("FLASHMUON_HALF", 1)
    half = fast_newtonschulz(G, steps=5)
    knobs("FLASHMUON_HALF", 0)
    whole = fast_newtonschulz(G, steps=5)
    assert torch.equal(half, whole)
    one = fast_newtonschulz(G[1], steps=5)
    assert torch.equal(half[1], one)
