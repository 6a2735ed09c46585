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


def _reference_layout_state_dict(params, group_order, world_size=1, hyper=None):
    """A state_dict as the reference's Muon would produce it, written out by hand from
    flash_muon/muon.py:65-72 and :96-97: one group per numel in `group_order`, each carrying its
    hyper-parameters, `update_buffer` ([world_size, numel] bf16), `update_buffer_views` and the
    positions of its parameters; per-parameter state {"momentum_buffer": zeros_like(grad) + ...}."""
    hyper = hyper or dict(lr=0.02, weight_decay=0.01, momentum=0.95, nesterov=True, ns_steps=5)
    groups, state, nxt = [], {}, 0
    for numel in group_order:
        members = [p for p in params if p.numel() == numel]
        b = torch.full((world_size, numel), float(numel % 7), dtype=torch.bfloat16)
        ids = list(range(nxt, nxt + len(members)))
        nxt += len(members)
        # torch.optim.Optimizer.state_dict() fills in the per-group defaults it knows of
        groups.append(dict(hyper, update_buffer=b, update_buffer_views=[b[i] for i in range(world_size)],
                           params=ids, foreach=None, maximize=False, capturable=False,
                           differentiable=False, fused=None))
        for pid, p in zip(ids, members):
            state[pid] = {"momentum_buffer": torch.full(p.shape, float(pid + 1), dtype=p.dtype)}
    return {"state": state, "param_groups": groups}


def test_groups_follow_the_reference_set_order_and_reference_checkpoints_load():
    """flash_muon/muon.py:68 iterates a set of numels; CPython's order for {4096, 2048} is
    [4096, 2048], not sorted.  The optimizer builds its groups with the same expression, and a
    checkpoint in the reference's layout loads whatever order its groups are in."""
    shapes = [(64, 64), (32, 64), (64, 32), (64, 64), (16, 128)]          # numels 4096, 2048, 2048, 4096, 2048
    params = [torch.nn.Parameter(torch.zeros(*s)) for s in shapes]
    opt = Muon(params, rank=0, world_size=1)
    want_order = list({p.numel() for p in params})                        # the reference's own expression
    assert [g["update_buffer"].size(1) for g in opt.param_groups] == want_order
    assert want_order == [4096, 2048]                                     # the case sorting would get wrong
    for g in opt.param_groups:
        assert g["update_buffer"].shape == (1, g["params"][0].numel()) and g["update_buffer"].dtype == torch.bfloat16
        assert set(g.keys()) >= {"params", "update_buffer", "update_buffer_views", "lr", "weight_decay",
                                 "momentum", "nesterov", "ns_steps"}
    for order in ([4096, 2048], [2048, 4096]):                            # the reference's order, and a swapped one
        for ws in (1, 8):                                                 # a checkpoint written by an 8-rank job
            sd = _reference_layout_state_dict(params, order, world_size=ws,
                                              hyper=dict(lr=0.05, weight_decay=0.0, momentum=0.9, nesterov=False, ns_steps=3))
            fresh = Muon(params, rank=0, world_size=1)
            fresh.load_state_dict(sd)
            assert [g["update_buffer"].size(1) for g in fresh.param_groups] == want_order
            for g in fresh.param_groups:
                n = g["params"][0].numel()
                assert (g["lr"], g["weight_decay"], g["momentum"], g["nesterov"], g["ns_steps"]) == (0.05, 0.0, 0.9, False, 3)
                assert g["update_buffer"].shape == (1, n) and g["update_buffer_views"][0].data_ptr() == g["update_buffer"].data_ptr()
                assert float(g["update_buffer"][0, 0]) == float(n % 7)    # row 0 of the saved buffer is kept
                for p in g["params"]:
                    assert p.numel() == n
            # every parameter got the momentum buffer that was saved for it: ids count through the
            # saved groups in their order, members in constructor order inside a group
            pid = 0
            for numel in order:
                for p in [q for q in params if q.numel() == numel]:
                    buf = fresh.state[p]["momentum_buffer"]
                    assert buf.shape == p.shape and float(buf.flatten()[0]) == float(pid + 1)
                    pid += 1
    # our own state_dict round-trips too
    again = Muon(params, rank=0, world_size=1)
    again.load_state_dict(opt.state_dict())
    assert [g["update_buffer"].size(1) for g in again.param_groups] == want_order


def test_newtonschulz_fake_kernel_matches_the_real_strides():
    """The operator returns a contiguous tensor for any input layout, and its fake says the same
    (a transposed view goes through the row-major side internally)."""
    import flash_muon_amd.ops  # noqa: F401
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        g = torch.empty(32, 96, dtype=torch.bfloat16).mT
        u = torch.ops.flash_muon.newtonschulz(g, 5)
        assert u.shape == (96, 32) and u.stride() == (32, 1)
