"""The entry points allocate nothing, synchronise nothing and launch only kernels, so a HIP graph
can hold them: a captured fast_newtonschulz and matmul_transpose replayed several times, with eager
work and synchronisations in between, give the eager result every time."""
import pytest
import torch

from flash_muon_amd import fast_newtonschulz, matmul_transpose_assign, synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_graph_replays_match_eager():
    G = synthetic.gradient_like_bf16(512, 1536, 8, 41).to(DEV)
    X = synthetic.gaussian_bf16(768, 1024, 42).to(DEV)
    Y = torch.empty(768, 768, dtype=torch.bfloat16, device=DEV)
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
    G2 = synthetic.gradient_like_bf16(512, 1536, 8, 43).to(DEV)
    G.copy_(G2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, fast_newtonschulz(G2, 5))
