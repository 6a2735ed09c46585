"""The momentum / Nesterov and weight-update entry points called directly through the C ABI, one
tensor at a time and batched, against the CPU oracle (flash_muon/muon.py:99-100, 87-89): bit-exact,
since each line is one fp32 expression rounded once to the storage type."""
import ctypes

import pytest
import torch

from flash_muon_amd import _lib
from oracle import oracle
from tests import gpu_util

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MU, LR, WD = 0.95, 0.02, 0.01


def _ptrs(ts):
    return (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])


EPS = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -23}


def _within_one_rounding(out, ref, dtype, scale):
    """out (storage type) against the fp32 oracle value: one rounding of the storage type, plus an
    fp32 ulp or two of the intermediate differences (the device may contract a*b+c)."""
    err = (out.float().cpu().double() - ref.double()).abs()
    sub = 2.0 ** -24 if dtype == torch.float16 else 0.0     # spacing of fp16 subnormals
    return bool((err <= ref.double().abs() * EPS[dtype] + scale * 2.0 ** -21 + sub).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
@pytest.mark.parametrize("nesterov", [True, False])
def test_momentum_single_and_batched(lib, dtype, n, nesterov):
    gen = torch.Generator().manual_seed(n)
    gs = [(1e-3 * torch.randn(n, generator=gen)).to(dtype) for _ in range(3)]
    bs = [(1e-3 * torch.randn(n, generator=gen)).to(dtype) for _ in range(3)]
    code = _lib.dtype_code(dtype)
    # one at a time
    g0, b0 = gs[0].to(DEV), bs[0].to(DEV)
    st = lib.fm_momentum_nesterov(g0.data_ptr(), b0.data_ptr(), code, n, 1 - MU, MU, int(nesterov), gpu_util._stream(g0))
    _lib.check("fm_momentum_nesterov", st)
    # all three in one launch: tensor 0 gets the same bits
    gd, bd = [g.to(DEV) for g in gs], [b.to(DEV) for b in bs]
    st = lib.fm_momentum_nesterov_batched(_ptrs(gd), _ptrs(bd), 3, code, n, 1 - MU, MU, int(nesterov), gpu_util._stream(g0))
    _lib.check("fm_momentum_nesterov_batched", st)
    assert torch.equal(g0, gd[0]) and torch.equal(b0, bd[0])
    for g_in, b_in, g_out, b_out in zip(gs, bs, gd, bd):
        _, nb, _ = oracle.momentum_nesterov(g_in.float(), b_in.float(), MU, nesterov)
        assert _within_one_rounding(b_out, nb, dtype, 1e-3)
        if nesterov:
            # the second line reads the ROUNDED buffer, as two successive lerp_ calls do
            ng = oracle.lerp(g_in.float(), b_out.float().cpu(), MU)
            assert _within_one_rounding(g_out, ng, dtype, 1e-3)
        else:
            assert torch.equal(g_out.cpu(), g_in)          # the gradient is left alone


@pytest.mark.parametrize("p_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n", [1, 9, 8192, 100003])
def test_weight_update_single_and_batched(lib, p_dtype, n):
    gen = torch.Generator().manual_seed(n + 1)
    ps = [(0.02 * torch.randn(n, generator=gen)).to(p_dtype) for _ in range(4)]
    us = [torch.randn(n, generator=gen).bfloat16() for _ in range(4)]
    alpha = -LR * 1.64
    code = _lib.dtype_code(p_dtype)
    pd, ud = [p.to(DEV) for p in ps], [u.to(DEV) for u in us]
    p0 = ps[0].to(DEV)
    st = lib.fm_weight_update(p0.data_ptr(), code, ud[0].data_ptr(), n, 1 - LR * WD, alpha, gpu_util._stream(p0))
    _lib.check("fm_weight_update", st)
    st = lib.fm_weight_update_batched(_ptrs(pd), code, _ptrs(ud), 4, n, 1 - LR * WD, alpha, gpu_util._stream(p0))
    _lib.check("fm_weight_update_batched", st)
    assert torch.equal(p0, pd[0])
    for p_in, u, p_out in zip(ps, us, pd):
        # mul_ then add_(alpha=): the decayed value is rounded to the storage type before the update is added
        decayed = (p_in.float() * torch.tensor(1 - LR * WD, dtype=torch.float32)).to(p_dtype).float()
        ref = decayed + torch.tensor(alpha, dtype=torch.float32) * u.float()
        assert _within_one_rounding(p_out, ref, p_dtype, 0.1)


def test_batched_argument_errors(lib):
    a = torch.zeros(64, dtype=torch.bfloat16, device=DEV)
    b = torch.zeros(64, dtype=torch.bfloat16, device=DEV)
    s = gpu_util._stream(a)
    assert lib.fm_momentum_nesterov_batched(_ptrs([a, a]), _ptrs([b, b]), 2, 0, 64, 0.05, 0.95, 1, s) == 5   # same g twice
    assert lib.fm_momentum_nesterov_batched(_ptrs([a]), _ptrs([b]), 33, 0, 64, 0.05, 0.95, 1, s) == 2       # batch > 32
    assert lib.fm_weight_update_batched(_ptrs([a, b]), 0, _ptrs([b, a]), 2, 64, 1.0, 1.0, s) == 5            # p aliases u
    assert lib.fm_weight_update_batched(_ptrs([a]), 7, _ptrs([b]), 1, 64, 1.0, 1.0, s) == 4
