"""The torch.library operators on the GPU: same results as the plain functions, and a graph
captured by torch.compile (without a code-generating backend) holds them as single nodes."""
import pytest
import torch

import flash_muon_amd.ops  # noqa: F401  (registers the operators)
from flash_muon_amd import fast_newtonschulz, matmul_transpose, synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_operators_match_the_functions():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(200, 136, generator=g).bfloat16().to(DEV)
    assert torch.equal(torch.ops.flash_muon.matmul_transpose(x), matmul_transpose(x))
    G = torch.randn(96, 160, generator=g).to(DEV)
    assert torch.equal(torch.ops.flash_muon.newtonschulz(G, 5), fast_newtonschulz(G, 5))


def test_captured_graph_holds_the_operators():
    def f(x, G):
        return torch.ops.flash_muon.matmul_transpose(x) * 2, torch.ops.flash_muon.newtonschulz(G, 3) + 1

    g = torch.Generator().manual_seed(4)
    x = torch.randn(128, 64, generator=g).bfloat16().to(DEV)
    G = torch.randn(64, 128, generator=g).to(DEV)
    want = f(x, G)
    got = torch.compile(f, backend="aot_eager", fullgraph=True)(x, G)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_newtonschulz_operator_strides_match_its_fake_kernel():
    """A transposed view in: the plain function answers with a transposed view, the operator with a
    contiguous tensor, which is what its fake kernel promises to torch.compile."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    G = synthetic.gradient_like_bf16(96, 160, 4, 61).to(DEV)
    real = torch.ops.flash_muon.newtonschulz(G.mT, 5)
    assert real.shape == (160, 96) and real.is_contiguous()
    assert torch.equal(real, fast_newtonschulz(G.mT, 5))
    with FakeTensorMode():
        fake = torch.ops.flash_muon.newtonschulz(torch.empty(96, 160, dtype=torch.bfloat16).mT, 5)
    assert fake.shape == real.shape and fake.stride() == real.stride()
