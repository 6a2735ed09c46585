"""The 256x256 path of the GEMM-shaped kernels (rounds of whole tiles, tiles cut along k where the
chip would otherwise idle).  It is chosen by shape (whole 256-tiles, k a multiple of 64, enough k
stages to share out); the FAST_MIN_UNITS knob is set to 0 for every test here (fm_set_knob), so that small inputs take it too and the partial-tile hand-over is exercised with few,
many and uneven parts per tile.  Integer-valued inputs make every comparison bit-exact."""
import pytest
import torch

from flash_muon_amd import matmul_transpose
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _small_inputs_take_the_256_path(knobs):
    knobs("FLASHMUON_FAST_MIN_UNITS", 0)
    knobs("FLASHMUON_HALF", 0)   # whole tiles: the half-tile schedule has tests of its own


def _ints(shape, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).float().bfloat16()


def _exact(x):   # exact integer matrix product in fp64, then the single bf16 rounding
    return x.float().bfloat16()


# (M, K): 1 tile and 1 stage; odd stage counts; many tiles; one tile split over many workgroups
SYRK_SHAPES = [(256, 64), (256, 192), (256, 4096), (512, 320), (768, 1024), (1024, 576), (2048, 2048), (1280, 8192)]


@pytest.mark.parametrize("M,K", SYRK_SHAPES)
def test_syrk_fast_integer_bit_exact(lib, M, K):
    X = _ints((M, K), M + K)
    want = _exact(X.double() @ X.double().T)
    Y = gpu_util.syrk(lib, X.to(DEV))
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)
    # a second run into a poisoned output gives the same bits (no dependence on arrival order)
    Y2 = torch.full_like(Y, 7.0)
    gpu_util.syrk(lib, X.to(DEV), Y2)
    assert torch.equal(Y2, Y)


@pytest.mark.parametrize("ksplit", [1, 2, 3, 4, 7, 16])
@pytest.mark.parametrize("M,K", [(256, 448), (768, 1024), (1280, 8192), (4096, 1024)])
def test_syrk_fast_forced_base_split(lib, knobs, M, K, ksplit):
    """Every tile cut into `ksplit` base parts along k (fm_set_knob):
    full rounds of partial tiles, a cut last round, and the second kernel over every tile."""
    knobs("FLASHMUON_KSPLIT", ksplit)
    X = _ints((M, K), 7 * M + K + ksplit)
    want = _exact(X.double() @ X.double().T)
    Y = torch.full((M, M), 7.0, dtype=torch.bfloat16, device=DEV)
    gpu_util.syrk(lib, X.to(DEV), Y)
    assert torch.equal(Y.cpu(), want)


def test_syrk_fast_few_tiles_long_k(lib):
    """10 tiles and 1024 k stages: every tile is cut into 16 base parts so that 160 workgroups run."""
    X = _ints((1024, 65536), 77)
    want = _exact(X.double() @ X.double().T)
    Y = gpu_util.syrk(lib, X.to(DEV))
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)


@pytest.mark.parametrize("grid", [3, 8, 20, 24, 40, 57])
@pytest.mark.parametrize("M,K,ksplit", [(1280, 512, 1), (2048, 1024, 1), (2048, 448, 2), (1792, 1344, 3)])
def test_syrk_fast_small_grids(lib, knobs, M, K, ksplit, grid):
    """Few workgroups per round (the GRID knob): several full
    rounds, last rounds of every fill, cut and uncut, on top of base parts."""
    knobs("FLASHMUON_GRID", grid)
    knobs("FLASHMUON_KSPLIT", ksplit)
    X = _ints((M, K), 3 * M + K + grid)
    want = _exact(X.double() @ X.double().T)
    Y = torch.full((M, M), 7.0, dtype=torch.bfloat16, device=DEV)
    gpu_util.syrk(lib, X.to(DEV), Y)
    assert torch.equal(Y.cpu(), want)


@pytest.mark.parametrize("grid", [8, 24, 40])
def test_axpby_and_poly_fast_small_grids(lib, knobs, grid):
    knobs("FLASHMUON_GRID", grid)
    M, K = 1024, 2304
    P = _ints((M, M), 41 + grid, -1, 1)
    X = _ints((M, K), 43 + grid)
    d = torch.arange(M, dtype=torch.float32) % 3 - 1
    want = _exact((2 + d.double())[:, None] * X.double() + P.double() @ X.double())
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, row_alpha=d.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    A = torch.triu(P.float()) + torch.triu(P.float(), 1).T
    full = A.double() + 2 * (A.double() @ A.double())
    Pp, dg = gpu_util.syrk_poly(lib, A.bfloat16().to(DEV), 1.0, 2.0, split_diag=True)
    assert torch.equal(dg.cpu().double(), torch.diagonal(full))
    assert torch.equal(Pp.cpu(), _exact(full - torch.diag(torch.diagonal(full))))


@pytest.mark.parametrize("ksplit", [2, 3])
def test_axpby_fast_forced_base_split(lib, knobs, ksplit):
    knobs("FLASHMUON_KSPLIT", ksplit)
    M, K = 768, 1536
    P = _ints((M, M), 31 + ksplit, -1, 1)
    X = _ints((M, K), 37 + ksplit)
    d = torch.arange(M, dtype=torch.float32) % 3 - 1
    want = _exact((2 + d.double())[:, None] * X.double() + P.double() @ X.double())
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, row_alpha=d.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)


@pytest.mark.parametrize("M", [256, 512, 1024, 1536])
def test_poly_fast_integer_bit_exact(lib, M):
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


@pytest.mark.parametrize("M,K", [(256, 256), (256, 1280), (512, 768), (1024, 2048), (768, 4096)])
def test_axpby_fast_integer_bit_exact(lib, M, K):
    P = _ints((M, M), 3 * M + K, -1, 1)
    X = _ints((M, K), 5 * M + K)
    d = torch.arange(M, dtype=torch.float32) % 3 - 1            # per-row addition to a
    want = _exact((2 + d.double())[:, None] * X.double() + P.double() @ X.double())
    Xo, XoT = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, row_alpha=d.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    only_t = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_x=False, row_alpha=d.to(DEV))[1]
    assert torch.equal(only_t.cpu(), want.T)
    only_x = gpu_util.gemm_axpby(lib, P.to(DEV), X.to(DEV), 2.0, want_xt=False, row_alpha=d.to(DEV))[0]
    assert torch.equal(only_x.cpu(), want)


def test_fast_and_general_paths_agree_on_gaussian_input(lib):
    """Same input through the 256x256 path (with workspace) and the tiled path (without): both are
    one bf16 rounding of an fp32 sum, so they agree to within that rounding."""
    g = torch.Generator().manual_seed(5)
    X = torch.randn(1024, 2048, generator=g).bfloat16().to(DEV)
    fast = gpu_util.syrk(lib, X)
    slow = torch.empty_like(fast)
    st = lib.fm_syrk_bf16(X.data_ptr(), X.stride(0), slow.data_ptr(), slow.stride(0), 1, 1024, 2048, None, 0,
                          gpu_util._stream(X))
    assert st == 0
    assert torch.equal(fast, fast.T) and torch.equal(slow, slow.T)
    ref = X.float() @ X.float().T
    for Y in (fast, slow):
        assert float((Y.float() - ref).norm() / ref.norm()) < 3e-3
    assert torch.equal(matmul_transpose(X), fast)


@pytest.mark.parametrize("no_sub64", [0, 1])
@pytest.mark.parametrize("M,K,grid", [(2048, 1024, 34), (2048, 320, 35), (1536, 2048, 20), (2304, 512, 43), (2048, 64, 34)])
def test_syrk_fast_last_round_in_space_or_along_k(lib, knobs, M, K, grid, no_sub64):
    """One or two whole tiles left after the last full round (the GRID knob makes small inputs end
    that way; at 8192^2 on 256 CUs it is 16 of 528): by default they are computed as 64x64
    sub-tiles over the whole k, 16 workgroups each, with NO_SUB64 they are cut along k into fp32
    parts and added up by the second kernel.  The left-over tiles include a diagonal one (written
    once) and an off-diagonal one (written twice)."""
    knobs("FLASHMUON_GRID", grid)
    knobs("FLASHMUON_NO_SUB64", no_sub64)
    X = _ints((M, K), M + 3 * K + grid)
    want = _exact(X.double() @ X.double().T)
    Y = torch.full((M, M), 7.0, dtype=torch.bfloat16, device=DEV)
    if no_sub64:
        gpu_util.syrk(lib, X.to(DEV), Y)
    else:                                              # the cut in space needs no workspace at all
        Xd = X.to(DEV)
        st = lib.fm_syrk_bf16(Xd.data_ptr(), K, Y.data_ptr(), M, 1, M, K, None, 0, gpu_util._stream(Xd))
        assert st == 0
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)
    # Gaussian input: both ways of cutting sum every element in the same k order as a whole tile
    g = torch.Generator().manual_seed(grid)
    G = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    got = gpu_util.syrk(lib, G)
    assert torch.equal(got, got.T)
    knobs("FLASHMUON_GRID", -1)
    knobs("FLASHMUON_NO_SUB64", -1)
    whole = gpu_util.syrk(lib, G)                      # every tile whole (no left-over at this size on 256 CUs)
    if not no_sub64:
        assert torch.equal(got, whole)
    else:
        assert float((got.float() - whole.float()).norm() / whole.float().norm()) < 1e-3


@pytest.mark.parametrize("M,K,grid", [(8192, 128, -1), (2560, 256, 53), (4352, 64, 144), (3072, 192, 75), (3072, 64, 74)])
def test_left_over_tiles_of_a_symmetric_product_are_diagonal_ones(lib, knobs, M, K, grid):
    """The tiles left after the last full round of a symmetric product are taken from the end of the
    diagonal (one operand panel each, 10 distinct sub-tiles of 16), the others close ranks in the blocked
    order: 16 of 528 at 8192^2 (two whole 8x8 blocks of the order lose their diagonal), 2 of 55, 9 of 153,
    3 and 4 of 78 (a block that loses part of its diagonal, or all of it).  Every tile must still be computed exactly
    once: integer input against the exact product, and the same bits as the plain order (the DIAG_LAST
    knob) on Gaussian input."""
    knobs("FLASHMUON_GRID", grid)
    X = _ints((M, K), M + K + 1)
    want = _exact(X.double() @ X.double().T)
    Xd = X.to(DEV)
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=DEV)
    st = lib.fm_syrk_bf16(Xd.data_ptr(), K, Y.data_ptr(), M, 1, M, K, None, 0, gpu_util._stream(Xd))
    assert st == 0
    assert torch.equal(Y.cpu(), want)
    assert torch.equal(Y, Y.T)
    g = torch.Generator().manual_seed(M + grid)
    G = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    got = gpu_util.syrk(lib, G)
    knobs("FLASHMUON_DIAG_LAST", 0)
    plain = gpu_util.syrk(lib, G)
    assert torch.equal(got, plain)
    assert torch.equal(got, got.T)


@pytest.mark.parametrize("no_sub64", [0, 1])
def test_poly_and_axpby_fast_last_round_in_space(lib, knobs, no_sub64):
    """The epilogue operand, the fp32 diagonal and the per-row addition on the 64x64 sub-tiles."""
    knobs("FLASHMUON_NO_SUB64", no_sub64)
    knobs("FLASHMUON_GRID", 34)
    M = 2048
    g = torch.Generator().manual_seed(9)
    A = torch.randint(-1, 2, (M, M), generator=g)
    A = (torch.triu(A) + torch.triu(A, 1).T).float().bfloat16()
    Ad = A.double()
    full = Ad + 2 * (Ad @ Ad)
    assert torch.equal(gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0).cpu(), _exact(full))
    P, d = gpu_util.syrk_poly(lib, A.to(DEV), 1.0, 2.0, split_diag=True)
    assert torch.equal(d.cpu().double(), torch.diagonal(full))
    assert torch.equal(P.cpu(), _exact(full - torch.diag(torch.diagonal(full))))
    assert torch.equal(P, P.T)
    knobs("FLASHMUON_GRID", 17)                        # 3 x 6 = 18 tiles: one left over
    M, K = 768, 1536
    Pm = _ints((M, M), 31, -1, 1)
    X = _ints((M, K), 37)
    dd = torch.arange(M, dtype=torch.float32) % 3 - 1
    want = _exact((2 + dd.double())[:, None] * X.double() + Pm.double() @ X.double())
    Xo, XoT = gpu_util.gemm_axpby(lib, Pm.to(DEV), X.to(DEV), 2.0, row_alpha=dd.to(DEV))
    assert torch.equal(Xo.cpu(), want)
    assert torch.equal(XoT.cpu(), want.T)
    only_t = gpu_util.gemm_axpby(lib, Pm.to(DEV), X.to(DEV), 2.0, want_x=False, row_alpha=dd.to(DEV))[1]
    assert torch.equal(only_t.cpu(), want.T)


def test_syrk_f16_fast_last_round_in_space(lib, knobs):
    knobs("FLASHMUON_GRID", 34)
    X = _ints((2048, 512), 5).half()
    want = (X.double() @ X.double().T).half()
    Xd = X.to(DEV)
    Y = torch.full((2048, 2048), 7.0, dtype=torch.float16, device=DEV)
    st = lib.fm_syrk_f16(Xd.data_ptr(), 512, Y.data_ptr(), 2048, 1, 2048, 512, None, 0, gpu_util._stream(Xd))
    assert st == 0
    assert torch.equal(Y.cpu(), want)


def _across_4gib(big, nbytes, dtype, shape):
    """A view of `shape` into the byte buffer `big` whose middle lies on a multiple of 4 GiB."""
    base = big.data_ptr()
    boundary = (base + 2**32 - 1) // 2**32 * 2**32
    start = boundary - nbytes // 2
    assert start >= base and start + nbytes <= base + big.numel() and start % 256 == 0
    v = big[start - base: start - base + nbytes].view(dtype).view(shape)
    assert v.data_ptr() < boundary < v.data_ptr() + nbytes
    return v


def test_operands_and_outputs_across_a_4gib_boundary(lib, knobs):
    """Every operand panel and every output in turn lies across a multiple of 4 GiB, where the low
    half of its 64-bit addresses wraps: the results are the bits of the same call on tensors that
    lie elsewhere.  (The copies into LDS take a scalar base and a 32-bit lane offset; a carry lost
    between the halves of that base reads 4 GiB too low.)"""
    big = torch.empty(5 * 2**30, dtype=torch.uint8, device=DEV)
    M, K = 2048, 1024
    X = _ints((M, K), 77).to(DEV)
    want = gpu_util.syrk(lib, X)
    assert torch.equal(want.cpu(), _exact(X.cpu().double() @ X.cpu().double().T))
    for grid in (-1, 34):                                # whole rounds; sub-tiles in the last round
        knobs("FLASHMUON_GRID", grid)
        Xb = _across_4gib(big, M * K * 2, torch.bfloat16, (M, K))
        Xb.copy_(X)
        assert torch.equal(gpu_util.syrk(lib, Xb), want)
        Yb = _across_4gib(big, M * M * 2, torch.bfloat16, (M, M))
        Yb.fill_(7.0)
        assert torch.equal(gpu_util.syrk(lib, X, Yb), want)
    knobs("FLASHMUON_GRID", -1)
    # the epilogue operand and both outputs of a X + P X
    M, K = 768, 1536
    Pm = _ints((M, M), 31, -1, 1).to(DEV)
    Xs = _ints((M, K), 37).to(DEV)
    XT = Xs.T.contiguous()
    Xo, XoT = gpu_util.gemm_axpby(lib, Pm, Xs, 2.0)
    XTb = _across_4gib(big, M * K * 2, torch.bfloat16, (K, M))
    XTb.copy_(XT)
    got = gpu_util.gemm_axpby(lib, Pm, Xs, 2.0, XT=XTb)
    assert torch.equal(got[0], Xo) and torch.equal(got[1], XoT)
    Pb = _across_4gib(big, M * M * 2, torch.bfloat16, (M, M))
    Pb.copy_(Pm)
    got = gpu_util.gemm_axpby(lib, Pb, Xs, 2.0)
    assert torch.equal(got[0], Xo) and torch.equal(got[1], XoT)


def _ticket_word(ws):
    """The 64-bit word the sub-tile tickets are counted in: the first of the workspace's last 256 bytes."""
    nb = ws.numel() // 256 * 256
    return ws[nb - 256: nb - 248].view(torch.int64)


@pytest.mark.parametrize("M,K,grid", [(2048, 1024, 34), (2304, 512, 43), (4352, 128, 144)])
def test_sub_tiles_by_ticket_whatever_the_workspace_holds(lib, knobs, M, K, grid):
    """With a workspace the sub-tiles of the last round are handed out by ticket (fewer workgroups than
    sub-tiles here, so workgroups come back for more).  The ticket word may hold anything when the call
    starts: zero, an earlier launch's count, a value smaller or larger than any launch number (the last
    means no tickets: sub-tile w to workgroup w), or what a call that cut its tiles along k wrote there.
    Every sub-tile is computed exactly once each time, and the word is left at zero, or alone."""
    knobs("FLASHMUON_GRID", grid)
    X = _ints((M, K), M + K + grid)
    want = _exact(X.double() @ X.double().T)
    Xd = X.to(DEV)
    ws = torch.zeros(lib.fm_gemm_workspace_bytes(M, M), dtype=torch.uint8, device=DEV)
    word = _ticket_word(ws)

    def run():
        Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=DEV)
        st = lib.fm_syrk_bf16(Xd.data_ptr(), K, Y.data_ptr(), M, 1, M, K, ws.data_ptr(), ws.numel(), gpu_util._stream(Xd))
        assert st == 0
        torch.cuda.synchronize()
        assert torch.equal(Y.cpu(), want)

    for start in (0, 5, 1 << 20, (1 << 62) + 12345, -1, -(1 << 40)):
        word.fill_(start)
        run()
        left = int(word.item())
        if 0 <= start < (1 << 46):
            assert left == 0, (start, left)          # below every launch number: tickets, and the last one clears the word
        else:
            assert left == (start if start >= 0 else start), (start, left)   # beyond them: no tickets, the word is left alone
        run()                                        # and again over what that call left
    # a call of the same shape that cuts its left-over tiles along k fills the slots in front of the word
    word.fill_(0)
    knobs("FLASHMUON_NO_SUB64", 1)
    run()
    knobs("FLASHMUON_NO_SUB64", -1)
    run()
    assert int(word.item()) == 0
    # no tickets at all by knob: same result
    knobs("FLASHMUON_NO_TICKETS", 1)
    word.fill_(77)
    run()
    assert int(word.item()) == 77


def test_sub_tiles_by_ticket_in_a_graph(lib, knobs):
    """A captured call carries its launch number with it: every replay finds the word at zero (the last
    ticket of the replay before cleared it) and counts from there."""
    knobs("FLASHMUON_GRID", 34)
    M, K = 2048, 512
    X = torch.randn(M, K, generator=torch.Generator().manual_seed(3)).bfloat16().to(DEV)
    ws = torch.zeros(lib.fm_gemm_workspace_bytes(M, M), dtype=torch.uint8, device=DEV)
    Y = torch.empty(M, M, dtype=torch.bfloat16, device=DEV)
    want = gpu_util.syrk(lib, X)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = lib.fm_syrk_bf16(X.data_ptr(), K, Y.data_ptr(), M, 1, M, K, ws.data_ptr(), ws.numel(),
                              torch.cuda.current_stream().cuda_stream)
        assert st == 0
    for i in range(4):
        Y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Y, want), "replay %d" % i
        assert int(_ticket_word(ws).item()) == 0
        assert torch.equal(gpu_util.syrk(lib, X), want)   # eager calls in between, with a workspace of their own
