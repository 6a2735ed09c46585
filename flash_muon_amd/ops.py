"""The two functional entry points as torch custom operators, so that a graph captured by
torch.compile / torch.export can hold them as single opaque nodes:

    import flash_muon_amd.ops                       # registers the operators
    y = torch.ops.flash_muon.matmul_transpose(x)
    u = torch.ops.flash_muon.newtonschulz(g, 5)

Not part of the reference's API (flash_muon/__init__.py:1-4 exports plain functions); the plain
functions of this package stay what they are and do not go through the dispatcher.
"""
import torch

from .matmul_transpose import matmul_transpose as _matmul_transpose
from .muon import fast_newtonschulz as _fast_newtonschulz


@torch.library.custom_op("flash_muon::matmul_transpose", mutates_args=())
def matmul_transpose(x: torch.Tensor) -> torch.Tensor:
    return _matmul_transpose(x)


@matmul_transpose.register_fake
def _(x):
    torch._check(x.dim() == 2, lambda: "Input `d_in` must be a 2D tensor")
    return x.new_empty((x.shape[0], x.shape[0]))


@torch.library.custom_op("flash_muon::newtonschulz", mutates_args=())
def newtonschulz(G: torch.Tensor, steps: int = 5) -> torch.Tensor:
    # fast_newtonschulz answers a transposed view with a transposed view; an operator's output
    # strides have to be what its fake kernel says, so the operator always returns contiguous
    return _fast_newtonschulz(G, steps).contiguous()


@newtonschulz.register_fake
def _(G, steps=5):
    torch._check(G.dim() >= 2, lambda: "Newton-Schulz needs at least two dimensions")
    return G.new_empty(G.shape, dtype=torch.bfloat16)
