"""Products of few 256x256 tiles run whole on 64x64 sub-tiles over the whole k, 16 workgroups per tile
(the schedule the tiles left after the last full round of a large product use).  It is chosen by
estimate for at most 16 tiles with up to about 64-80 k stages; NO_SUB64 = 0 forces it here wherever
it fits (with FAST_MIN_UNITS = 0 so that small inputs take the 256x256 path at all), NO_SUB64 = 1
forbids it.  Integer-valued inputs make every comparison with the fp64 product bit-exact."""
import pytest
import torch

from flash_muon_amd import _lib, fast_newtonschulz, matmul_transpose, synthetic
from oracle import oracle
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


@pytest.fixture
def forced(knobs):
    knobs("FLASHMUON_FAST_MIN_UNITS", 0)
    knobs("FLASHMUON_NO_SUB64", 0)


def _ints(shape, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).float().bfloat16()


def _exact(x):   # exact integer matrix product in fp64, then the single rounding
    return x.float().bfloat16()


# one tile and one stage; stage counts around the 8-stage ring of a sub-tile; 3, 6, 10 and 15 tiles
SYRK_SHAPES = [(256, 64), (256, 128), (256, 448), (256, 512), (256, 576), (512, 64), (512, 1088), (768, 320),
               (1024, 1024), (1024, 4096), (1280, 192)]


@pytest.mark.parametrize("M,K", SYRK_SHAPES)
def test_syrk_integer_bit_exact_without_a_workspace(lib, forced, M, K):
    X = _ints((M, K), M + K)
    want = _exact(X.double() @ X.double().T)
    Xd = X.to(DEV)
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=DEV)
    st = lib.fm_syrk_bf16(Xd.data_ptr(), K, Y.data_ptr(), M, 1, M, K, None, 0, gpu_util._stream(Xd))
    assert st == 0
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


def test_syrk_strided_output_and_input_view(lib, forced):
    M, K = 768, 320
    big = _ints((M, K + 64), 5)
    X = big[:, 32:32 + K]
    want = _exact(X.double() @ X.double().T)
    Ybig = torch.full((M, M + 128), float("nan"), dtype=torch.bfloat16, device=DEV)
    Y = Ybig[:, 64:64 + M]
    gpu_util.syrk(lib, big.to(DEV)[:, 32:32 + K], Y)
    assert torch.equal(Y.cpu(), want)
    assert torch.isnan(Ybig[:, :64]).all() and torch.isnan(Ybig[:, 64 + M:]).all()


@pytest.mark.parametrize("M", [256, 512, 1024, 1280])
def test_poly_integer_bit_exact(lib, forced, M):
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
    full3 = 2 * Ad + 3 * (Ad @ Ad)
    assert torch.equal(gpu_util.syrk_poly(lib, A.to(DEV), 2.0, 3.0).cpu(), _exact(full3))


@pytest.mark.parametrize("M,K", [(256, 256), (256, 1024), (512, 768), (1024, 1024), (768, 1280)])
def test_axpby_integer_bit_exact(lib, forced, M, K):
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


@pytest.mark.parametrize("M,K", [(256, 64), (512, 320), (1024, 256)])
def test_syrk_f16_integer_bit_exact(lib, forced, M, K):
    g = torch.Generator().manual_seed(M + K)
    X = torch.randint(-2, 3, (M, K), generator=g).to(torch.float16)
    want = (X.double() @ X.double().T).to(torch.float16)
    Xd = X.to(DEV)
    Y = torch.full((M, M), float("nan"), dtype=torch.float16, device=DEV)
    st = lib.fm_syrk_f16(Xd.data_ptr(), Xd.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), M, K, None, 0,
                         _lib.stream_ptr(Xd.device))
    _lib.check("fm_syrk_f16", st)
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


@pytest.mark.parametrize("M,K", [(512, 512), (1024, 1024), (1024, 2048), (768, 3072), (512, 2048)])
def test_chosen_by_shape_and_equal_to_whole_tiles_on_gaussian_input(lib, knobs, M, K):
    """Left to the library these shapes take the sub-tiles; every sum runs over k in the same order as
    in a whole 256x256 tile, so the bits are those of the whole-tile schedule, which the tests of
    that path pin to the oracle."""
    X = synthetic.gaussian_bf16(M, K, M + K).to(DEV)
    auto = matmul_transpose(X)
    knobs("FLASHMUON_FAST_MIN_UNITS", 0)
    knobs("FLASHMUON_NO_SUB64", 0)
    sub = matmul_transpose(X)
    knobs("FLASHMUON_NO_SUB64", 1)
    knobs("FLASHMUON_KSPLIT", 1)
    knobs("FLASHMUON_HALF", 0)
    whole = matmul_transpose(X)
    assert torch.equal(sub, whole)
    assert torch.equal(auto, whole)
    assert torch.equal(auto, auto.T)
    ref = oracle.xxt(X.cpu())
    assert oracle.rel_fro(auto, ref) < 3e-3


@pytest.mark.parametrize("rows,cols", [(512, 512), (1024, 768), (256, 1536), (1000, 1000)])
def test_newtonschulz_against_the_oracle(rows, cols):
    G = synthetic.gradient_like_bf16(rows, cols, 8, rows + cols)
    ref = oracle.newtonschulz(G, 5)
    got = fast_newtonschulz(G.to(DEV), 5)
    err = oracle.rel_fro(got, ref)
    print("five steps %dx%d: rel_fro %.3e" % (rows, cols, err), flush=True)
    assert err < TOL
    assert err < 1.2 * oracle.rel_fro(oracle.newtonschulz_eager_bf16(G, 5), ref)
    assert torch.equal(fast_newtonschulz(G.T.contiguous().to(DEV), 5).T, got) or rows == cols


def test_batched_newtonschulz_forced_and_forbidden_agree(lib, knobs):
    """Three 512 x 768 matrices in one launch: 3 x 3 tiles of the symmetric products, 3 x 6 of the last
    product of a step (more than 16: that one stays on whole tiles).  Same bits with the sub-tiles
    forbidden, every matrix within the oracle's tolerance."""
    Gs = torch.stack([synthetic.gradient_like_bf16(512, 768, 4, 70 + i) for i in range(3)])
    knobs("FLASHMUON_FAST_MIN_UNITS", 0)
    knobs("FLASHMUON_KSPLIT", 1)
    knobs("FLASHMUON_HALF", 0)
    knobs("FLASHMUON_NO_SUB64", 0)
    sub = fast_newtonschulz(Gs.to(DEV), 5)
    knobs("FLASHMUON_NO_SUB64", 1)
    whole = fast_newtonschulz(Gs.to(DEV), 5)
    assert torch.equal(sub, whole)
    for i in range(3):
        assert oracle.rel_fro(sub[i], oracle.newtonschulz(Gs[i], 5)) < TOL
