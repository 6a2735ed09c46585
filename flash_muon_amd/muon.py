"""fast_newtonschulz and the single-GPU Muon optimizer on libflashmuon_hip.so.

Signatures, defaults, state keys and error behaviour follow flash_muon/muon.py:6-110.  The
Newton-Schulz loop (muon.py:25-29) runs as three fused kernels per step inside
fm_newtonschulz_bf16; the momentum and weight updates (muon.py:99-100, 87-89) are one kernel
each.  The all-gather of muon.py:108 has no counterpart: only world_size == 1 is implemented,
and no process group is needed.
"""
import torch
from torch import Tensor

from . import _lib

# quintic coefficients of flash_muon/muon.py:14
NS_COEFFS = (3.4445, -4.7750, 2.0315)
NS_EPS = 1e-7   # flash_muon/muon.py:23


def _rows_unit_stride(G):
    """A view or copy of 2-D G whose rows are unit-stride with pitch >= cols."""
    if G.size(1) <= 1 or G.stride(1) == 1:
        if G.size(0) <= 1 or G.stride(0) >= G.size(1):
            return G
    return G.contiguous()


def _newtonschulz_into(G, out, steps):
    """Orthogonalise 2-D G (bf16/fp16/fp32, rows unit-stride) into `out` (bf16, same shape)."""
    rows, cols = G.shape
    lib = _lib.load()
    a, b, c = NS_COEFFS
    ldg = G.stride(0) if rows > 1 else cols
    ldo = out.stride(0) if rows > 1 else cols
    with torch.cuda.device(G.device):
        ws, ws_bytes = _lib.workspace(lib.fm_newtonschulz_workspace_bytes(rows, cols), G.device)
        st = lib.fm_newtonschulz_bf16(G.data_ptr(), _lib.dtype_code(G.dtype), rows, cols, ldg,
                                      out.data_ptr(), ldo, steps, a, b, c, NS_EPS,
                                      ws.data_ptr(), ws_bytes, _lib.stream_ptr(G.device))
    _lib.check("fm_newtonschulz_bf16", st)


def fast_newtonschulz(G: Tensor, steps: int = 5) -> Tensor:
    """Quintic Newton-Schulz orthogonalisation of G; returns bf16 with G's shape.

    Arguments (as flash_muon/muon.py:6-12):
        G: The gradient or momentum matrix to be orthogonalized.
        steps: Number of Newton-Schulz iterations.

    The reference asserts ndim >= 2 (muon.py:13) but its buffers and its symmetric kernel only
    admit 2-D input (muon.py:19-20, matmul_transpose_triton.py:83); the same holds here.
    """
    assert G.ndim >= 2
    assert G.ndim == 2, "Input `d_in` must be a 2D tensor"
    assert G.is_cuda, "Input `d_in` must be a CUDA tensor"
    if G.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        G = G.bfloat16()
    if G.numel() == 0:
        return torch.empty(G.shape, dtype=torch.bfloat16, device=G.device)
    if G.size(1) > 1 and G.stride(1) != 1 and G.stride(0) == 1 and G.stride(1) >= G.size(0):
        # a transposed view: NS(G^T) == NS(G)^T, so work on the row-major side
        return fast_newtonschulz(G.mT, steps).mT
    G = _rows_unit_stride(G)
    out = torch.empty(G.shape, dtype=torch.bfloat16, device=G.device)
    _newtonschulz_into(G, out, int(steps))
    return out


class Muon(torch.optim.Optimizer):
    """Muon - MomentUm Orthogonalized by Newton-schulz, single GPU.

    Same constructor and state layout as flash_muon/muon.py:36-110:

    Arguments:
        lr: The learning rate used by the internal SGD.
        weight_decay: decoupled weight decay, applied as p *= 1 - lr * weight_decay.
        momentum: The momentum used by the internal SGD.
        nesterov: Whether to use Nesterov-style momentum in the internal SGD. (recommended)
        ns_steps: The number of Newton-Schulz iteration steps to use.
        rank, world_size: required, as in the reference; only (0, 1) is implemented.

    Not for embeddings, the final fully connected layer or 0/1-D parameters; 4-D convolution
    filters are flattened over their last three dimensions.
    """

    def __init__(self, params, lr=0.02, weight_decay=0.01, momentum=0.95, nesterov=True, ns_steps=5,
                 rank=None, world_size=None):
        if (rank is None) or (world_size is None):
            raise Exception("world_size and rank params required, if you want to use this optimizer on a single GPU, pass rank=0 and world_size=1.")
        if world_size != 1 or rank != 0:
            raise NotImplementedError("this build implements the single-GPU step only: pass rank=0 and world_size=1")
        self.rank = rank
        self.world_size = world_size
        defaults = dict(lr=lr, weight_decay=weight_decay, momentum=momentum, nesterov=nesterov, ns_steps=ns_steps)
        params = [*params]
        param_groups = []
        # one group per distinct numel, each with a [world_size, numel] bf16 update buffer
        # (flash_muon/muon.py:68-72); sorted so that the group order does not depend on hashing
        for size in sorted({p.numel() for p in params}):
            members = [p for p in params if p.numel() == size]
            b = torch.empty(world_size, size, dtype=torch.bfloat16, device=members[0].device if members[0].is_cuda else "cuda")
            group = dict(params=members, update_buffer=b,
                         update_buffer_views=[b[i] for i in range(world_size)])
            param_groups.append(group)
        super().__init__(param_groups, defaults)

    @torch.no_grad()
    def step(self):
        lib = _lib.load()
        for group in self.param_groups:
            update: Tensor = group["update_buffer_views"][self.rank]
            lr, wd, mu = group["lr"], group["weight_decay"], group["momentum"]
            for p in group["params"]:
                g = p.grad
                assert g is not None
                assert p.is_cuda and g.is_cuda, "Muon parameters and gradients must be CUDA tensors"
                state = self.state[p]
                if "momentum_buffer" not in state:
                    state["momentum_buffer"] = torch.zeros_like(g, memory_format=torch.contiguous_format)
                buf: Tensor = state["momentum_buffer"]
                if not buf.is_contiguous():   # e.g. a state loaded from elsewhere
                    buf = state["momentum_buffer"] = buf.contiguous()

                # buf.lerp_(g, 1 - mu); g.lerp_(buf, mu) in place on p.grad (muon.py:99-100)
                gc = g if g.is_contiguous() else g.contiguous()
                code = _lib.dtype_code(gc.dtype)
                stream = _lib.stream_ptr(gc.device)
                with torch.cuda.device(gc.device):
                    st = lib.fm_momentum_nesterov(gc.data_ptr(), buf.data_ptr(), code, gc.numel(),
                                                  1 - mu, mu, 1 if group["nesterov"] else 0, stream)
                _lib.check("fm_momentum_nesterov", st)
                if gc is not g and group["nesterov"]:
                    g.copy_(gc)
                src = gc if group["nesterov"] else buf
                if src.ndim == 4:   # conv filters (muon.py:101-102)
                    src = src.view(len(src), -1)
                assert src.ndim == 2, "Input `d_in` must be a 2D tensor"

                # orthogonalise straight into the group's update buffer (muon.py:103, 108)
                _newtonschulz_into(src, update.view(src.shape), group["ns_steps"])

                # p *= 1 - lr*wd ; p += -lr*sqrt(max(1, rows/cols)) * update (muon.py:87-89)
                pc = p if p.is_contiguous() else p.contiguous()
                alpha = -lr * max(1, p.size(-2) / p.size(-1)) ** 0.5
                with torch.cuda.device(pc.device):
                    st = lib.fm_weight_update(pc.data_ptr(), _lib.dtype_code(pc.dtype), update.data_ptr(),
                                              pc.numel(), 1 - lr * wd, alpha, stream)
                _lib.check("fm_weight_update", st)
                if pc is not p:
                    p.copy_(pc)
