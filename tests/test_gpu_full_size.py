"""The benchmark configurations at their full sizes: Newton-Schulz on 4096 x 16384 and 8192 x 8192
and one Llama-7B layer of Muon.step, against the fp32 CPU oracle (a few TFLOP each on the host, so
these are the slowest tests), plus properties that need no CPU product."""
import pytest
import torch

from flash_muon_amd import Muon, fast_newtonschulz, synthetic
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


def test_muon_step_one_llama7b_layer():
    ps, gs = synthetic.llama7b_layer(0)
    params = []
    for p, g in zip(ps, gs):
        q = torch.nn.Parameter(p.clone().to(DEV))
        q.grad = g.clone().to(DEV)
        params.append(q)
    opt = Muon(params, lr=0.02, momentum=0.95, nesterov=True, rank=0, world_size=1)
    opt.step()
    ref_p, ref_g, ref_b, ref_u = oracle.muon_step(ps, gs, [None] * len(ps), 0.02, 0.01, 0.95, True, 5)
    for q, p0, rp, rg, rb, ru in zip(params, ps, ref_p, ref_g, ref_b, ref_u):
        assert oracle.rel_fro(opt.state[q]["momentum_buffer"], rb) < 4e-3
        assert oracle.rel_fro(q.grad, rg) < 4e-3
        assert oracle.rel_fro(q.data, rp) < 3e-3
        # the update itself, recovered from the parameter change in fp32 terms
        scale = max(1, p0.size(0) / p0.size(1)) ** 0.5
        upd = fast_newtonschulz(q.grad, 5).float().cpu()
        err = oracle.rel_fro(upd, ru)
        print("update %s rel_fro %.3e" % (tuple(p0.shape), err), flush=True)
        assert err < 1e-2
