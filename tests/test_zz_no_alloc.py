"""fm_syrk_bf16_static, the entry point that allocates nothing (its partial tiles go to an array the
library holds in device memory), against fm_syrk_bf16 with a caller-owned workspace: same bits, on
two calls in a row of which the second is smaller and lays the shared array out differently."""
import pytest
import torch

from flash_muon_amd import _lib, synthetic
from oracle import oracle
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _static(lib, X):
    M, K = X.shape
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=X.device)
    st = lib.fm_syrk_bf16_static(X.data_ptr(), X.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), M, K,
                                 _lib.stream_ptr(X.device))
    _lib.check("fm_syrk_bf16_static", st)
    return Y


def test_static_scratch_entry_point_matches_the_workspace_one(lib):
    # 8192^2: 528 tiles, the 16 of the last round are cut into 16 parts each (256 slots of the array);
    # then 1280 x 8192: 15 tiles, every one cut in two along k and the remainder again (other slots,
    # other sizes), over what the first call left in the array
    for (M, K, seed) in ((8192, 8192, 8192), (1280, 8192, 5), (8192, 8192, 8192)):
        X = synthetic.gaussian_bf16(M, K, seed).to(DEV)
        got = _static(lib, X)
        want = gpu_util.syrk(lib, X)
        torch.cuda.synchronize()
        assert torch.equal(got, want), "%d x %d differs from fm_syrk_bf16" % (M, K)
        assert torch.equal(got, got.T)
        if M <= 2048:
            assert oracle.rel_fro(got, oracle.xxt(X)) < 3e-3
    # integer-valued input: bit-exact against the brute force, strided output
    g = torch.Generator().manual_seed(3)
    X = torch.randint(-2, 3, (768, 1024), generator=g).float().bfloat16().to(DEV)
    buf = torch.zeros(768, 1024, dtype=torch.bfloat16, device=DEV)
    Y = buf[:, 128:896]
    st = lib.fm_syrk_bf16_static(X.data_ptr(), X.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), 768, 1024,
                                 _lib.stream_ptr(X.device))
    assert st == 0
    assert torch.equal(Y.cpu(), oracle.xxt_int64(X).double().bfloat16())   # exact sums, one rounding
    assert float(buf[:, :128].abs().max()) == 0 and float(buf[:, 896:].abs().max()) == 0
    # beyond the stated maximum: refused before anything is launched
    assert lib.fm_syrk_bf16_static(X.data_ptr(), 1024, Y.data_ptr(), 1024, 1, 65536 + 256, 64, None) == 2
    assert lib.fm_syrk_bf16_static(X.data_ptr(), 1 << 21, Y.data_ptr(), 1024, 1, 256, (1 << 20) + 64, None) == 2
    # the usual argument checks still apply
    assert lib.fm_syrk_bf16_static(None, 1024, Y.data_ptr(), 1024, 1, 768, 1024, None) == 1
