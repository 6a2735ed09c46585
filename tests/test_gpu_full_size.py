"""The benchmark configurations at their full sizes: Newton-Schulz on 4096 x 16384 and 8192 x 8192
and one Llama-7B layer of Muon.step, against the fp32 CPU oracle (a few TFLOP each on the host, so
these are the slowest tests), plus properties that need no CPU product."""
import ctypes

import pytest
import torch

from flash_muon_amd import Muon, _lib, fast_newtonschulz, synthetic
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_rectangular_newtonschulz_4096x16384():
    G = synthetic.gradient_like_bf16(4096, 16384, 8, 3)
    got = fast_newtonschulz(G.to(DEV), 5)
    ref = oracle.newtonschulz(G, 5)
    err = oracle.rel_fro(got, ref)
    print("NS5 4096x16384 free-running rel_fro %.3e" % err, flush=True)
    assert err < 1e-2
    # the tall orientation is the same computation transposed, bit for bit
    tall = fast_newtonschulz(G.to(DEV).T.contiguous(), 5)
    assert torch.equal(tall.T, got)


def test_square_newtonschulz_8192():
    G = synthetic.gradient_like_bf16(8192, 8192, 16, 4)
    got = fast_newtonschulz(G.to(DEV), 5)
    ref, states = oracle.newtonschulz(G, 5, trace=True)
    err = oracle.rel_fro(got, ref)
    print("NS5 8192x8192 free-running rel_fro %.3e" % err, flush=True)
    assert err < 1e-2
    # per-step figure for the last, most sensitive step: start from the oracle's state
    Xin = states[4].bfloat16()
    one = fast_newtonschulz(Xin.to(DEV), 1)
    # fast_newtonschulz normalises first; the oracle's state has norm ~ sqrt(rank), so compare with
    # the oracle applied to the same bf16 input
    err1 = oracle.rel_fro(one, oracle.newtonschulz(Xin, 1))
    print("NS 8192x8192 single step from the oracle's step-4 state rel_fro %.3e" % err1, flush=True)
    assert err1 < 1e-2


def _applied_update(p_before, p_after, lr, wd):
    """The update Muon.step applied, recovered from an fp32 parameter:
    p' = p (1 - lr wd) - lr sqrt(max(1, rows/cols)) u   (muon.py:87-89)."""
    scale = max(1, p_before.size(0) / p_before.size(1)) ** 0.5
    return (p_before.double() * (1 - lr * wd) - p_after.double()) / (lr * scale)


def test_muon_step_one_llama7b_layer():
    """One layer of the Llama-7B configuration (4 x 4096^2, 2 x 11008x4096, 1 x 4096x11008), bf16
    parameters and gradients, against the oracle: state, gradient, parameter, and the update itself
    as step() applied it.  The update is read back from a second optimizer over fp32 copies of the
    same parameters (same gradients, same batches of 4 + 2 + 1 matrices through the same kernels):
    an fp32 parameter keeps the update to 1e-5 of its size, a bf16 parameter rounds it away."""
    lr, wd = 0.02, 0.01
    ps, gs = synthetic.llama7b_layer(0)
    params, params32 = [], []
    for p, g in zip(ps, gs):
        q = torch.nn.Parameter(p.clone().to(DEV))
        q.grad = g.clone().to(DEV)
        params.append(q)
        q32 = torch.nn.Parameter(p.float().to(DEV))
        if hasattr(q32, "grad_dtype"):
            q32.grad_dtype = None        # an fp32 parameter with a bf16 gradient
        q32.grad = g.clone().to(DEV)
        params32.append(q32)
    opt = Muon(params, lr=lr, momentum=0.95, nesterov=True, rank=0, world_size=1)
    opt32 = Muon(params32, lr=lr, momentum=0.95, nesterov=True, rank=0, world_size=1)
    opt.step()
    opt32.step()
    ref_p, ref_g, ref_b, ref_u = oracle.muon_step(ps, gs, [None] * len(ps), lr, wd, 0.95, True, 5)
    for q, q32, p0, rp, rg, rb, ru in zip(params, params32, ps, ref_p, ref_g, ref_b, ref_u):
        assert oracle.rel_fro(opt.state[q]["momentum_buffer"], rb) < 4e-3
        assert oracle.rel_fro(q.grad, rg) < 4e-3
        assert oracle.rel_fro(q.data, rp) < 3e-3
        assert torch.equal(q32.grad, q.grad)
        upd = _applied_update(p0.float(), q32.data.cpu(), lr, wd)
        assert bool(torch.isfinite(upd).all())
        err = oracle.rel_fro(upd, ru)
        print("applied update %s rel_fro %.3e" % (tuple(p0.shape), err), flush=True)
        assert err < 1e-2
        # the bf16 parameter moved by the same update, up to its own rounding (2^-9 of |p| ~ 0.02)
        moved = (p0.double() * (1 - lr * wd) - q.data.cpu().double())
        scale = max(1, p0.size(0) / p0.size(1)) ** 0.5
        assert oracle.rel_fro(moved, lr * scale * ru.double()) < 0.35
    # the group buffers end up holding the last update of their group (muon.py:108)
    for group in opt32.param_groups:
        last = group["params"][-1]
        idx = [i for i, q in enumerate(params32) if q is last][0]
        got = group["update_buffer"][0].view(ref_u[idx].shape)
        assert oracle.rel_fro(got, ref_u[idx]) < 1e-2


def _batched_ns(lib, Gs, steps=5):
    rows, cols = Gs[0].shape
    n = len(Gs)
    outs = [torch.empty(rows, cols, dtype=torch.bfloat16, device=DEV) for _ in Gs]
    a, b, c = oracle.NS_COEFFS
    ws = torch.empty(lib.fm_newtonschulz_batched_workspace_bytes(n, rows, cols), dtype=torch.uint8, device=DEV)
    st = lib.fm_newtonschulz_batched_bf16((ctypes.c_void_p * n)(*[g.data_ptr() for g in Gs]), 0, n, rows, cols, cols,
                                          (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs]), cols, steps, a, b, c,
                                          oracle.NS_EPS, ws.data_ptr(), ws.numel(), _lib.stream_ptr(Gs[0].device))
    _lib.check("fm_newtonschulz_batched_bf16", st)
    torch.cuda.synchronize()
    return outs


@pytest.mark.parametrize("n,rows,cols,checked", [
    (32, 4096, 4096, (0, 17, 31)), (32, 4096, 11008, (9, 31)), (32, 11008, 4096, (20,)),
    (16, 4096, 4096, (0, 11)), (16, 4096, 11008, (5, 15)), (16, 11008, 4096, (2,))])
def test_many_per_launch_schedules(lib, n, rows, cols, checked):
    """fm_newtonschulz_batched_bf16 with n Llama-7B-sized matrices per launch.  Thirty-two is what
    Muon.step and bench.py run on the Llama-7B set (flash_muon/muon.py:90-103 walks the same
    parameters one by one): 32 x 136 and 32 x 688 tiles of 256x256 are whole rounds of 256
    workgroups.  Sixteen end in a last round of tiles cut along k (2176 = 8 x 256 + 128 tiles), another
    code path.  The members in `checked` against the fp32 CPU oracle, every member for finite values
    and against the single-matrix call (which differs only in which tiles are summed from parts or run
    on half tiles, i.e. in fp32 summation order)."""
    Gs = [synthetic.gradient_like_bf16(rows, cols, 8, 700 + i) for i in range(n)]
    dGs = [G.to(DEV) for G in Gs]
    outs = _batched_ns(lib, dGs)
    for i in checked:
        err = oracle.rel_fro(outs[i], oracle.newtonschulz(Gs[i], 5))
        print("batch of %d, %dx%d, member %d: rel_fro %.3e" % (n, rows, cols, i, err), flush=True)
        assert err < 1e-2
    for i in range(n):
        assert bool(torch.isfinite(outs[i]).all())
        single = fast_newtonschulz(dGs[i], 5)
        assert oracle.rel_fro(outs[i], single.float()) < 6e-3
