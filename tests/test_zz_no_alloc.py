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


def _syrk_ws(lib, X, ws):
    M, K = X.shape
    Y = torch.full((M, M), float("nan"), dtype=torch.bfloat16, device=X.device)
    st = lib.fm_syrk_bf16(X.data_ptr(), X.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), M, K,
                          ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
                          _lib.stream_ptr(X.device))
    _lib.check("fm_syrk_bf16", st)
    return Y


def test_static_scratch_entry_point_matches_the_workspace_one(lib, knobs):
    """Two calls in a row whose partial tiles go through the array, the second smaller:
    8192^2 with the NO_SUB64 knob (528 tiles of 256x256; the 16 left after the two full rounds are cut
    into 16 parts each along k: all 256 slots of 256 KiB), then 1280 x 8192 (55 tiles of 128x128, every
    one cut in four along k: 220 parts of 64 KiB over what the first call left there), then the first
    again.  Each against fm_syrk_bf16 with a caller-owned workspace of the array's 64 MiB: same bits.
    That the parts really went through the array shows in the bits as well: without any scratch the
    same calls run their last tiles whole, which sums over k in another order and rounds a few
    hundred elements differently."""
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    for (M, K, seed, no_sub64) in ((8192, 8192, 8192, 1), (1280, 8192, 5, -1), (8192, 8192, 8192, 1)):
        knobs("FLASHMUON_NO_SUB64", no_sub64)
        X = synthetic.gaussian_bf16(M, K, seed).to(DEV)
        got = _static(lib, X)
        want = _syrk_ws(lib, X, ws)
        bare = _syrk_ws(lib, X, None)
        torch.cuda.synchronize()
        assert torch.equal(got, want), "%d x %d differs from fm_syrk_bf16" % (M, K)
        assert torch.equal(got, got.T)
        assert not torch.equal(got, bare), "%d x %d: the parts did not go through the array" % (M, K)
        assert oracle.rel_fro(got.float(), bare.float()) < 1e-4
        if M <= 2048:
            assert oracle.rel_fro(got, oracle.xxt(X)) < 3e-3
    knobs("FLASHMUON_NO_SUB64", -1)
    # left to itself the large product ends in sub-tiles and needs no scratch at all: same bits as whole tiles
    X = synthetic.gaussian_bf16(8192, 8192, 8192).to(DEV)
    assert torch.equal(_static(lib, X), _syrk_ws(lib, X, None))
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
