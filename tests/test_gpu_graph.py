"""The entry points allocate nothing, synchronise nothing and launch only kernels, so a HIP graph
can hold them: a captured fast_newtonschulz and matmul_transpose replayed several times, with eager
work and synchronisations in between, give the eager result every time."""
import pytest
import torch

from flash_muon_amd import fast_newtonschulz, matmul_transpose_assign, synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# whole tiles, and sides that are not (zero-padded copies in the workspace)
@pytest.mark.parametrize("gshape,xshape", [((512, 1536), (768, 1024)), ((500, 1500), (700, 1000))])
def test_graph_replays_match_eager(gshape, xshape):
    G = synthetic.gradient_like_bf16(gshape[0], gshape[1], 8, 41).to(DEV)
    X = synthetic.gaussian_bf16(xshape[0], xshape[1], 42).to(DEV)
    Y = torch.empty(xshape[0], xshape[0], dtype=torch.bfloat16, device=DEV)
    want_ns = fast_newtonschulz(G, 5)
    want_y = torch.empty_like(Y)
    matmul_transpose_assign(X, want_y)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, as torch asks
        fast_newtonschulz(G, 5)
        matmul_transpose_assign(X, Y)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fast_newtonschulz(G, 5)
        matmul_transpose_assign(X, Y)
    for i in range(4):
        out.zero_()
        Y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_ns), "replay %d" % i
        assert torch.equal(Y, want_y), "replay %d" % i
        # eager work of the same kind between replays
        assert torch.equal(fast_newtonschulz(G, 5), want_ns)
        torch.cuda.synchronize()
    # new input values in place: the graph reads the same buffers
    G2 = synthetic.gradient_like_bf16(gshape[0], gshape[1], 8, 43).to(DEV)
    G.copy_(G2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, fast_newtonschulz(G2, 5))


def test_muon_step_in_a_graph_matches_eager():
    """Muon.step captured after its first (state-creating) eager step: replays with fresh gradients
    copied into the same .grad tensors follow an eager twin bit for bit."""
    from flash_muon_amd import Muon
    shapes = [(256, 256)] * 3 + [(512, 256)] * 2 + [(256, 512)]
    gen = torch.Generator().manual_seed(51)
    ps = [(0.02 * torch.randn(*s, generator=gen)).bfloat16() for s in shapes]

    def grads(seed):
        g = torch.Generator().manual_seed(seed)
        return [(1e-3 * torch.randn(*s, generator=g)).bfloat16().to(DEV) for s in shapes]

    a = [torch.nn.Parameter(p.clone().to(DEV)) for p in ps]
    b = [torch.nn.Parameter(p.clone().to(DEV)) for p in ps]
    for q, r, g in zip(a, b, grads(60)):
        q.grad = g.clone()
        r.grad = g.clone()
    opt_a = Muon(a, lr=0.02, momentum=0.95, rank=0, world_size=1)
    opt_b = Muon(b, lr=0.02, momentum=0.95, rank=0, world_size=1)
    opt_a.step()                       # creates the momentum buffers and the scratch
    opt_b.step()
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    for q, g in zip(a, grads(61)):
        q.grad.copy_(g)
    with torch.cuda.graph(graph, stream=side):
        opt_a.step()
    torch.cuda.synchronize()
    # capture does not run anything: replay once for the step with the gradients of seed 61
    for step_seed in (61, 62, 63):
        for q, r, g in zip(a, b, grads(step_seed)):
            q.grad.copy_(g)
            r.grad.copy_(g)
        graph.replay()
        opt_b.step()
        torch.cuda.synchronize()
        for q, r in zip(a, b):
            assert torch.equal(q, r), "step with seed %d" % step_seed
            assert torch.equal(opt_a.state[q]["momentum_buffer"], opt_b.state[r]["momentum_buffer"])
