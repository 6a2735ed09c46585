"""GPU parity of the symmetric product on matrices whose sides are not whole 128-tiles, which run
through zero-padded copies in the workspace when it has fm_syrk_workspace_bytes(M, K): bit-exact
against the integer CPU oracle, bit-exact symmetry, the same bits as the general schedule on integer
inputs, nothing written outside the M x M result, and within one bf16 rounding of the fp32 oracle on
Gaussian inputs."""
import pytest
import torch

from flash_muon_amd import _lib, matmul_transpose, matmul_transpose_assign, synthetic
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = [(257, 513), (300, 1100), (1000, 777), (1000, 1000), (129, 4097), (2000, 136), (1111, 2047), (3100, 200)]


def _int_matrix(M, K, seed, lo=-2, hi=2):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (M, K), generator=g).float().bfloat16()


def _call(lib, entry, X, Y, ws_bytes):
    M, K = X.shape
    ws = torch.empty(max(int(ws_bytes), 256), dtype=torch.uint8, device=X.device)
    st = getattr(lib, entry)(X.data_ptr(), X.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), M, K,
                             ws.data_ptr(), int(ws_bytes), _lib.stream_ptr(X.device))
    _lib.check(entry, st)
    torch.cuda.synchronize()
    return Y


def test_workspace_sizes(lib):
    # whole tiles and small matrices need what the product itself needs; ragged ones room for the copies
    assert lib.fm_syrk_workspace_bytes(1024, 2048) == lib.fm_gemm_workspace_bytes(1024, 1024)
    assert lib.fm_syrk_workspace_bytes(100, 37) == lib.fm_gemm_workspace_bytes(100, 100)
    assert lib.fm_syrk_workspace_bytes(1000, 1000) >= 2 * 1024 * 1024 * 2
    assert lib.fm_syrk_workspace_bytes(4000, 4000) >= 2 * 4096 * 4096 * 2
    assert lib.fm_syrk_workspace_bytes(0, 5) == 0


@pytest.mark.parametrize("M,K", SHAPES)
def test_integer_inputs_bit_exact_on_both_schedules(lib, M, K):
    X = _int_matrix(M, K, 300 + M + K)
    want = oracle.xxt_int64(X).float().bfloat16()
    Xd = X.to(DEV)
    padded = _call(lib, "fm_syrk_bf16", Xd, torch.empty(M, M, dtype=torch.bfloat16, device=DEV),
                   lib.fm_syrk_workspace_bytes(M, K))
    general = _call(lib, "fm_syrk_bf16", Xd, torch.empty(M, M, dtype=torch.bfloat16, device=DEV),
                    lib.fm_gemm_workspace_bytes(M, M))
    assert torch.equal(padded.cpu(), want)
    assert torch.equal(general.cpu(), want)
    assert torch.equal(padded, padded.T)
    assert torch.equal(matmul_transpose(Xd).cpu(), want)


def test_fp16_elements(lib):
    M, K = 700, 333
    X = _int_matrix(M, K, 7).half()
    want = oracle.xxt_int64(X).float().half()
    got = _call(lib, "fm_syrk_f16", X.to(DEV), torch.empty(M, M, dtype=torch.float16, device=DEV),
                lib.fm_syrk_workspace_bytes(M, K))
    assert torch.equal(got.cpu(), want)
    assert torch.equal(matmul_transpose(X.to(DEV)).cpu(), want)


@pytest.mark.parametrize("M,K,seed", [(1000, 1000, 0), (700, 333, 2), (2000, 3000, 3)])
def test_gaussian_against_fp32_oracle(M, K, seed):
    X = synthetic.gaussian_bf16(M, K, seed)
    ref = oracle.xxt(X)
    got = matmul_transpose(X.to(DEV)).cpu()
    assert torch.equal(got, got.T)
    assert oracle.rel_fro(got, ref) < 3e-3
    # one bf16 rounding of an fp32-accumulated sum: half an ulp (2^-9 relative) plus accumulation slack
    err = (got.float() - ref).abs()
    bound = ref.abs() * 2.0 ** -8 + 1e-3 * K ** 0.5
    assert (err <= bound).all()


def test_strided_inputs_and_outputs_leave_the_rest_alone(lib):
    M, K = 515, 1030
    X = _int_matrix(M, K, 11)
    want = oracle.xxt_int64(X).float().bfloat16()
    xbuf = torch.full((M, K + 6), 3.0, dtype=torch.bfloat16, device=DEV)       # row pitch not a multiple of 8
    xbuf[:, :K] = X.to(DEV)
    ybuf = torch.full((M, M + 13), 7.0, dtype=torch.bfloat16, device=DEV)
    _call(lib, "fm_syrk_bf16", xbuf[:, :K], ybuf[:, :M], lib.fm_syrk_workspace_bytes(M, K))
    assert torch.equal(ybuf[:, :M].cpu(), want)
    assert bool((ybuf[:, M:] == 7.0).all())
    # column-major output (a transposed view): the unit stride is along the columns
    ycol = torch.full((M + 3, M), 7.0, dtype=torch.bfloat16, device=DEV)
    matmul_transpose_assign(X.to(DEV), ycol[:M].T)                            # strides (1, M)
    assert torch.equal(ycol[:M].cpu(), want)
    assert bool((ycol[M:] == 7.0).all())
    yt = torch.full((M, M + 5), 7.0, dtype=torch.bfloat16, device=DEV)
    view = yt[:, :M].T                                                        # strides (1, M + 5)
    assert view.stride() == (1, M + 5)
    matmul_transpose_assign(X.to(DEV), view)
    assert torch.equal(yt[:, :M].cpu(), want)
    assert bool((yt[:, M:] == 7.0).all())
    # a unit-stride slice of the input at an odd element offset (not 16-byte aligned)
    xoff = torch.zeros(M * (K + 1) + 1, dtype=torch.bfloat16, device=DEV)
    xv = xoff[1:].view(M, K + 1)[:, :K]
    xv.copy_(X.to(DEV))
    assert torch.equal(matmul_transpose(xv).cpu(), want)


def test_too_little_workspace_takes_the_general_schedule(lib):
    M, K = 900, 1300
    X = _int_matrix(M, K, 13).to(DEV)
    want = oracle.xxt_int64(X.cpu()).float().bfloat16()
    for ws_bytes in (0, 4096, lib.fm_syrk_workspace_bytes(M, K) - 256):
        got = _call(lib, "fm_syrk_bf16", X, torch.empty(M, M, dtype=torch.bfloat16, device=DEV), ws_bytes)
        assert torch.equal(got.cpu(), want)


def test_repeated_calls_of_changing_shapes_share_the_workspace():
    # the shared workspace keeps the last call's contents: the padding has to be rewritten every time
    a = _int_matrix(1000, 900, 17).to(DEV)
    b = _int_matrix(600, 1500, 18).to(DEV)
    wa = oracle.xxt_int64(a.cpu()).float().bfloat16()
    wb = oracle.xxt_int64(b.cpu()).float().bfloat16()
    for _ in range(2):
        assert torch.equal(matmul_transpose(a).cpu(), wa)
        assert torch.equal(matmul_transpose(torch.full((1024, 2048), 5.0, dtype=torch.bfloat16, device=DEV))[0, 0].cpu(),
                           torch.tensor(25.0 * 2048).bfloat16())
        assert torch.equal(matmul_transpose(b).cpu(), wb)
