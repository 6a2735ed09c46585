"""GPU parity of Muon.step (world_size == 1) against the fp32 CPU oracle and the closed forms of
the first and second step (flash_muon/muon.py:76-110)."""
import copy

import pytest
import torch

from flash_muon_amd import Muon, fast_newtonschulz
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LR, WD, MU = 0.02, 0.01, 0.95


def _make(shapes, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    ps, gs = [], []
    for s in shapes:
        ps.append((0.02 * torch.randn(*s, generator=g)).to(dtype))
        gs.append((1e-3 * torch.randn(*s, generator=g)).to(dtype))
    return ps, gs


def _device_params(ps, gs):
    out = []
    for p, g in zip(ps, gs):
        q = torch.nn.Parameter(p.clone().to(DEV))
        if g.dtype != p.dtype and hasattr(q, "grad_dtype"):
            q.grad_dtype = None          # an fp32 parameter with a bf16 gradient
        q.grad = g.clone().to(DEV)
        out.append(q)
    return out


def test_first_and_second_step_against_oracle():
    shapes = [(128, 128), (344, 128), (128, 344), (64, 256), (128, 128)]
    ps, gs = _make(shapes, 1)
    params = _device_params(ps, gs)
    opt = Muon(params, lr=LR, momentum=MU, rank=0, world_size=1)
    assert opt.step() is None
    ref_p, ref_g, ref_b, ref_u = oracle.muon_step(ps, gs, [None] * len(ps), LR, WD, MU, True, 5)
    for i, (q, g0, rp, rg, rb) in enumerate(zip(params, gs, ref_p, ref_g, ref_b)):
        st = opt.state[q]
        assert set(st.keys()) == {"momentum_buffer"}
        # closed form of the first step: buf = (1-mu) g, grad <- (1-mu^2) g, each rounded once
        assert oracle.rel_fro(st["momentum_buffer"], rb) < 4e-3
        assert oracle.rel_fro(q.grad, rg) < 4e-3
        assert torch.equal(st["momentum_buffer"].cpu(), ((1 - MU) * g0.float()).bfloat16()) or \
            oracle.rel_fro(st["momentum_buffer"], (1 - MU) * g0.float()) < 3e-3
        assert oracle.rel_fro(q.data, rp) < 3e-3
        # the move itself: lr * (update of O(1/sqrt(cols)) entries), seen through p's bf16 rounding
        delta_ref = rp - (1 - LR * WD) * ps[i].float()
        delta_got = q.data.cpu().float() - (1 - LR * WD) * ps[i].float()
        assert oracle.rel_fro(delta_got, delta_ref) < 0.15
    # second step: new gradients, momentum carried over
    _, gs2 = _make(shapes, 2)
    for q, g in zip(params, gs2):
        q.grad = g.clone().to(DEV)
    cur_p = [q.data.cpu().clone() for q in params]
    cur_b = [opt.state[q]["momentum_buffer"].cpu().clone() for q in params]
    opt.step()
    ref_p, ref_g, ref_b, _ = oracle.muon_step(cur_p, gs2, cur_b, LR, WD, MU, True, 5)
    for q, rp, rg, rb in zip(params, ref_p, ref_g, ref_b):
        assert oracle.rel_fro(opt.state[q]["momentum_buffer"], rb) < 4e-3
        assert oracle.rel_fro(q.grad, rg) < 4e-3
        assert oracle.rel_fro(q.data, rp) < 3e-3


def test_update_equals_orthogonalised_momentum():
    """p' = p (1 - lr wd) - lr sqrt(max(1, r/c)) NS(g'), with NS taken from the library itself, so
    the elementwise kernels are pinned to within their own bf16 roundings."""
    ps, gs = _make([(344, 128)], 3)
    (q,) = _device_params(ps, gs)
    opt = Muon([q], lr=LR, momentum=MU, rank=0, world_size=1)
    opt.step()
    u = fast_newtonschulz(q.grad, 5).float().cpu()          # q.grad now holds the Nesterov gradient
    scale = (344 / 128) ** 0.5
    decayed = (ps[0].float() * torch.tensor(1 - LR * WD, dtype=torch.float32)).bfloat16().float()
    want = (decayed + torch.tensor(-LR * scale, dtype=torch.float32) * u).bfloat16()
    got = q.data.cpu()
    # fused-multiply-add contraction on the device may move a result by one bf16 ulp
    diff = (got.float() - want.float()).abs()
    assert (diff <= want.float().abs() * 2.0 ** -7).all()
    assert (diff == 0).float().mean() > 0.98
    assert torch.equal(opt.param_groups[0]["update_buffer"][0].view(344, 128).cpu().float(), u)


def test_no_nesterov_uses_buffer_and_leaves_grad():
    ps, gs = _make([(96, 160)], 4)
    (q,) = _device_params(ps, gs)
    opt = Muon([q], lr=LR, momentum=MU, nesterov=False, rank=0, world_size=1)
    opt.step()
    assert torch.equal(q.grad.cpu(), gs[0])
    ref_p, _, ref_b, _ = oracle.muon_step(ps, gs, [None], LR, WD, MU, False, 5)
    assert oracle.rel_fro(opt.state[q]["momentum_buffer"], ref_b[0]) < 4e-3
    assert oracle.rel_fro(q.data, ref_p[0]) < 3e-3


def test_conv_filter_param_and_fp32_param():
    ps, gs = _make([(64, 8, 3, 3)], 5)
    (q,) = _device_params(ps, gs)
    opt = Muon([q], lr=LR, momentum=MU, rank=0, world_size=1)
    opt.step()
    ref_p, _, _, _ = oracle.muon_step(ps, gs, [None], LR, WD, MU, True, 5)
    assert oracle.rel_fro(q.data, ref_p[0]) < 3e-3
    ps, gs = _make([(80, 200)], 6, torch.float32)
    (q,) = _device_params(ps, gs)
    opt = Muon([q], lr=LR, momentum=MU, rank=0, world_size=1)
    opt.step()
    ref_p, ref_g, ref_b, _ = oracle.muon_step(ps, gs, [None], LR, WD, MU, True, 5)
    assert q.dtype == torch.float32 and opt.state[q]["momentum_buffer"].dtype == torch.float32
    assert oracle.rel_fro(opt.state[q]["momentum_buffer"], ref_b[0]) < 1e-6
    assert oracle.rel_fro(q.grad, ref_g[0]) < 1e-6
    delta_got = q.data.cpu() - (1 - LR * WD) * ps[0]
    delta_ref = ref_p[0] - (1 - LR * WD) * ps[0]
    assert oracle.rel_fro(delta_got, delta_ref) < 2e-2       # the update itself, at NS tolerance (80 rows)


def test_groups_state_dict_and_missing_grad():
    ps, gs = _make([(64, 64), (32, 128), (128, 32), (64, 32)], 7)
    params = _device_params(ps, gs)
    opt = Muon(params, lr=LR, momentum=MU, rank=0, world_size=1)
    groups = opt.param_groups
    # one group per numel, in the iteration order of the reference's set expression (muon.py:68)
    assert [g["params"][0].numel() for g in groups] == list({p.numel() for p in params}) == [4096, 2048]
    assert len(groups[0]["params"]) == 3 and len(groups[1]["params"]) == 1
    for g in groups:
        assert set(g.keys()) >= {"params", "update_buffer", "update_buffer_views", "lr", "weight_decay",
                                 "momentum", "nesterov", "ns_steps"}
        assert g["update_buffer"].shape == (1, g["params"][0].numel())
        assert g["update_buffer"].dtype == torch.bfloat16
        assert g["weight_decay"] == 0.01 and g["ns_steps"] == 5
    opt.step()
    sd = opt.state_dict()
    assert all("momentum_buffer" in s for s in sd["state"].values())
    params[0].grad = None
    with pytest.raises(AssertionError):
        opt.step()


def test_state_dict_round_trip_continues_identically():
    """A second optimizer that loads the first one's state after step 1 takes the same step 2."""
    shapes = [(128, 128), (256, 128), (128, 128)]
    ps, gs = _make(shapes, 21)
    a = _device_params(ps, gs)
    opt_a = Muon(a, lr=LR, momentum=MU, rank=0, world_size=1)
    opt_a.step()
    b = [torch.nn.Parameter(q.detach().clone()) for q in a]
    opt_b = Muon(b, lr=LR, momentum=MU, rank=0, world_size=1)
    # through a deep copy, as through torch.save / torch.load: load_state_dict itself keeps the
    # tensors it is given, and the two optimizers must not share momentum buffers
    opt_b.load_state_dict(copy.deepcopy(opt_a.state_dict()))
    for q, r in zip(a, b):
        assert torch.equal(opt_a.state[q]["momentum_buffer"], opt_b.state[r]["momentum_buffer"])
    _, gs2 = _make(shapes, 22)
    for q, r, g in zip(a, b, gs2):
        q.grad = g.clone().to(DEV)
        r.grad = g.clone().to(DEV)
    opt_a.step()
    opt_b.step()
    for q, r in zip(a, b):
        assert torch.equal(q, r)
        assert torch.equal(opt_a.state[q]["momentum_buffer"], opt_b.state[r]["momentum_buffer"])


def test_batched_step_matches_unbatched():
    """Same-shape parameters are orthogonalised several per launch; the step must not depend on it
    beyond the fp32 summation order of split tiles, and two steps must land on the oracle's
    parameters whatever the batch size (fp32 parameters, so that the two updates are not rounded
    away)."""
    shapes = [(256, 512)] * 5 + [(512, 256)] * 3 + [(128, 1024)] * 2   # one numel, three shapes
    ps, gs = _make(shapes, 11)
    ps = [p.float() for p in ps]
    # the second step reuses the first step's Nesterov-updated gradient, as it stays in p.grad
    ref_p, ref_g, ref_b, _ = oracle.muon_step(ps, gs, [None] * len(ps), LR, WD, MU, True, 5)
    ref_p2, _, _, _ = oracle.muon_step(ref_p, [g.bfloat16() for g in ref_g], ref_b, LR, WD, MU, True, 5)
    res = {}
    for batch in (1, 4, 32):
        params = _device_params(ps, gs)
        opt = Muon(params, lr=LR, momentum=MU, rank=0, world_size=1, batch=batch)
        opt.step()
        opt.step()
        res[batch] = [q.data.cpu().float() for q in params]
        for q, p0, r2 in zip(res[batch], ps, ref_p2):
            # what two steps moved, against what the oracle moved
            assert oracle.rel_fro(q.double() - p0.double(), r2.double() - p0.double()) < 1e-2
    for batch in (4, 32):
        for x, y, p0 in zip(res[1], res[batch], ps):
            assert oracle.rel_fro(x.double() - p0.double(), y.double() - p0.double()) < 4e-3


def test_buckets_larger_than_a_launch_go_in_equal_chunks():
    """A bucket of more same-shape parameters than one launch takes is handed over in chunks of equal
    size (48 as 24 + 24, 70 as 24 + 24 + 22) at the default batch of 32: every parameter must move as
    it does one matrix per launch (flash_muon/muon.py:90-103 walks them one by one), and no chunk may
    be skipped or taken twice."""
    shapes = [(384, 256)] * 48 + [(128, 512)] * 70
    ps, gs = _make(shapes, 23)
    ps = [p.float() for p in ps]
    res = {}
    for batch in (1, None):
        params = _device_params(ps, gs)
        opt = Muon(params, lr=LR, momentum=MU, rank=0, world_size=1, batch=batch)
        opt.step()
        torch.cuda.synchronize()
        res[batch] = [q.data.cpu() for q in params]
    for i, (x, y, p0) in enumerate(zip(res[1], res[None], ps)):
        assert bool(torch.isfinite(y).all())
        moved = y.double() - p0.double() * (1 - LR * WD)
        assert float(moved.abs().max()) > 0, "parameter %d was not updated" % i
        assert oracle.rel_fro(moved, x.double() - p0.double() * (1 - LR * WD)) < 6e-3, i
    # two members against the oracle
    for i in (30, 100):
        ref_p, _, _, _ = oracle.muon_step([ps[i]], [gs[i]], [None], LR, WD, MU, True, 5)
        assert oracle.rel_fro(res[None][i].double() - ps[i].double() * (1 - LR * WD),
                              ref_p[0].double() - ps[i].double() * (1 - LR * WD)) < 1e-2
