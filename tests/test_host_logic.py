"""Host-side behaviour of the Python layer that needs no GPU: argument contract and errors, which
mirror flash_muon/matmul_transpose_triton.py:79-86 and flash_muon/muon.py:61-62."""
import pytest
import torch

import flash_muon_amd
from flash_muon_amd import Muon, fast_newtonschulz, matmul_transpose, matmul_transpose_assign
from flash_muon_amd import synthetic


def test_public_names():
    assert flash_muon_amd.__all__ == ["matmul_transpose", "matmul_transpose_assign", "fast_newtonschulz", "Muon"]


def test_cpu_tensors_are_rejected():
    x = torch.zeros(4, 4, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="must be a CUDA tensor"):
        matmul_transpose_assign(x, x.clone())
    with pytest.raises(AssertionError, match="must be a CUDA tensor"):
        matmul_transpose(x)
    with pytest.raises(AssertionError):
        fast_newtonschulz(x)
    with pytest.raises(AssertionError):
        fast_newtonschulz(torch.zeros(4))
    with pytest.raises(ValueError):
        matmul_transpose(torch.zeros(4))      # `M, _ = d_in.shape` on a 1-D tensor


def test_muon_requires_rank_and_world_size():
    p = torch.nn.Parameter(torch.zeros(4, 4))
    with pytest.raises(Exception, match="world_size and rank params required"):
        Muon([p])
    with pytest.raises(Exception, match="world_size and rank params required"):
        Muon([p], rank=0)
    with pytest.raises(NotImplementedError):
        Muon([p], rank=0, world_size=2)
    with pytest.raises(NotImplementedError):
        Muon([p], rank=1, world_size=1)


def test_synthetic_inputs_are_seeded():
    a = synthetic.gaussian_bf16(8, 8, 3)
    b = synthetic.gaussian_bf16(8, 8, 3)
    assert torch.equal(a, b) and a.dtype == torch.bfloat16
    g = synthetic.gradient_like_bf16(32, 64, 4, 5)
    assert g.shape == (32, 64) and abs(float(g.float().norm()) - 1.0) < 1e-2
    sv = torch.linalg.svdvals(g.float())
    assert sv[0] > 5 * sv[8]                   # the spike stands out of the noise floor
    assert synthetic.syrk_useful_flop(8192, 8192) == 8192 * 8192 * 8193
    assert synthetic.ns_useful_flop(4096, 16384, 5) == synthetic.ns_useful_flop(16384, 4096, 5)
    assert abs(synthetic.ns_useful_flop(8192, 8192, 5) / 1.100e13 - 1) < 1e-3
    assert abs(synthetic.ns_useful_flop(4096, 16384, 5) / 4.467e12 - 1) < 1e-3


def test_custom_operators_propagate_shapes_without_a_device():
    """The torch.library registrations: fake tensors go through without touching the library."""
    import flash_muon_amd.ops  # noqa: F401  (registers the operators)
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        x = torch.empty(48, 80, dtype=torch.bfloat16)
        y = torch.ops.flash_muon.matmul_transpose(x)
        assert y.shape == (48, 48) and y.dtype == torch.bfloat16
        u = torch.ops.flash_muon.newtonschulz(torch.empty(96, 32, dtype=torch.float32), 5)
        assert u.shape == (96, 32) and u.dtype == torch.bfloat16
