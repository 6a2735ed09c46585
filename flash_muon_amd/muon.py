"""fast_newtonschulz and the single-GPU Muon optimizer on libflashmuon_hip.so.

Signatures, defaults, state keys and error behaviour follow flash_muon/muon.py:6-110.  The
Newton-Schulz loop (muon.py:25-29) runs as three fused kernels per step inside
fm_newtonschulz_bf16; the momentum and weight updates (muon.py:99-100, 87-89) are one kernel
each.  The all-gather of muon.py:108 has no counterpart: only world_size == 1 is implemented,
and no process group is needed.
"""
import ctypes

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


MAX_BATCH = 32  # kMaxBatch of the library: matrices per batched launch


def _newtonschulz_into(Gs, outs, steps):
    """Orthogonalise the 2-D matrices Gs (one shape, dtype and row pitch; bf16/fp16/fp32, rows
    unit-stride) into `outs` (bf16, same shape, one row pitch), every stage one launch for all."""
    G0, n = Gs[0], len(Gs)
    rows, cols = G0.shape
    lib = _lib.load()
    a, b, c = NS_COEFFS
    ldg = G0.stride(0) if rows > 1 else cols
    ldo = outs[0].stride(0) if rows > 1 else cols
    g_ptrs = (ctypes.c_void_p * n)(*[g.data_ptr() for g in Gs])
    o_ptrs = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    with _lib.on_device(G0.device):
        ws, ws_bytes = _lib.workspace(lib.fm_newtonschulz_batched_workspace_bytes(n, rows, cols), G0.device)
        st = lib.fm_newtonschulz_batched_bf16(g_ptrs, _lib.dtype_code(G0.dtype), n, rows, cols, ldg,
                                              o_ptrs, ldo, steps, a, b, c, NS_EPS,
                                              ws.data_ptr(), ws_bytes, _lib.stream_ptr(G0.device))
    _lib.check("fm_newtonschulz_batched_bf16", st)


def fast_newtonschulz(G: Tensor, steps: int = 5) -> Tensor:
    """Quintic Newton-Schulz orthogonalisation of G; returns bf16 with G's shape.

    Arguments (as flash_muon/muon.py:6-12):
        G: The gradient or momentum matrix to be orthogonalized.
        steps: Number of Newton-Schulz iterations.

    The reference asserts ndim >= 2 (muon.py:13) and normalises over the last two dimensions
    (muon.py:23), but its buffers and its symmetric kernel only admit 2-D input (muon.py:19-20,
    matmul_transpose_triton.py:83).  Here leading dimensions are a batch of independent matrices,
    orthogonalised up to 32 per launch.
    """
    assert G.ndim >= 2
    assert G.is_cuda, "Input `d_in` must be a CUDA tensor"
    if G.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        G = G.bfloat16()
    if G.numel() == 0:
        return torch.empty(G.shape, dtype=torch.bfloat16, device=G.device)
    if G.ndim > 2:
        flat = G.reshape(-1, G.size(-2), G.size(-1)).contiguous()
        out = torch.empty(flat.shape, dtype=torch.bfloat16, device=G.device)
        count = flat.size(0)
        per = -(-count // -(-count // MAX_BATCH))   # chunks of equal size, as in Muon.step
        for i0 in range(0, count, per):
            n = min(per, count - i0)
            _newtonschulz_into([flat[i0 + i] for i in range(n)], [out[i0 + i] for i in range(n)], int(steps))
        return out.view(G.shape)
    if G.size(1) > 1 and G.stride(1) != 1 and G.stride(0) == 1 and G.stride(1) >= G.size(0):
        # a transposed view: NS(G^T) == NS(G)^T, so work on the row-major side
        return fast_newtonschulz(G.mT, steps).mT
    G = _rows_unit_stride(G)
    out = torch.empty(G.shape, dtype=torch.bfloat16, device=G.device)
    _newtonschulz_into([G], [out], int(steps))
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
        batch: (not in the reference) how many same-shape matrices are orthogonalised per launch,
            1..32; default 32.  Memory: the Newton-Schulz scratch of a launch (four padded copies of
            the iterate, two squares) is about 6.3 times the bytes of its bf16 matrices, 0.44 GB per
            4096 x 11008 matrix and 14 GB for 32 of them (the reference holds about 0.3 GB, one
            matrix at a time), taken from torch's caching allocator per call; a [batch, numel] bf16
            staging buffer per group stays with the optimizer (2.9 GB at the default for that
            shape).  A smaller batch shrinks both in proportion.

    Not for embeddings, the final fully connected layer or 0/1-D parameters; 4-D convolution
    filters are flattened over their last three dimensions.
    """

    def __init__(self, params, lr=0.02, weight_decay=0.01, momentum=0.95, nesterov=True, ns_steps=5,
                 rank=None, world_size=None, batch=None):
        if (rank is None) or (world_size is None):
            raise Exception("world_size and rank params required, if you want to use this optimizer on a single GPU, pass rank=0 and world_size=1.")
        if world_size != 1 or rank != 0:
            raise NotImplementedError("this build implements the single-GPU step only: pass rank=0 and world_size=1")
        self.rank = rank
        self.world_size = world_size
        self.batch = MAX_BATCH if batch is None else max(1, min(int(batch), MAX_BATCH))
        self._staging = {}
        defaults = dict(lr=lr, weight_decay=weight_decay, momentum=momentum, nesterov=nesterov, ns_steps=ns_steps)
        params = [*params]
        param_groups = []
        # One group per distinct numel, each with a [world_size, numel] bf16 update buffer, in the
        # iteration order of the same set expression as flash_muon/muon.py:68-72, so that groups
        # (and with them the entries of a state_dict) come out in the reference's order.  The
        # buffer lives where the parameters live (the reference writes "cuda", muon.py:69).
        for size in {p.numel() for p in params}:
            members = [p for p in params if p.numel() == size]
            b = torch.empty(world_size, size, dtype=torch.bfloat16, device=members[0].device)
            group = dict(params=members, update_buffer=b,
                         update_buffer_views=[b[i] for i in range(world_size)])
            param_groups.append(group)
        super().__init__(param_groups, defaults)

    def load_state_dict(self, state_dict):
        """torch pairs saved and live groups by position; a checkpoint whose groups were built in
        another order (another interpreter's set order, or a sorted one) is first put into this
        optimizer's order by the numel of each group's update buffer, the key the groups are made
        from (flash_muon/muon.py:68-71).  The buffers themselves are scratch: whatever their saved
        world size or device, each group keeps a [1, numel] bf16 buffer next to its parameters."""
        saved = state_dict["param_groups"]
        own = [g["update_buffer"].size(-1) for g in self.param_groups]
        theirs = [g["update_buffer"].size(-1) if torch.is_tensor(g.get("update_buffer")) else None for g in saved]
        if theirs != own and None not in theirs and sorted(theirs) == sorted(own):
            order = [theirs.index(n) for n in own]
            # parameter ids are positions in the saved order: renumber them for the new order
            remap, nxt = {}, 0
            groups = []
            for i in order:
                g = dict(saved[i])
                ids = []
                for pid in g["params"]:
                    remap[pid] = nxt
                    ids.append(nxt)
                    nxt += 1
                g["params"] = ids
                groups.append(g)
            state_dict = {"state": {remap.get(k, k): v for k, v in state_dict["state"].items()},
                          "param_groups": groups}
        super().load_state_dict(state_dict)
        for group in self.param_groups:
            dev = group["params"][0].device
            n = group["params"][0].numel()
            b = group.get("update_buffer")
            if not (torch.is_tensor(b) and b.shape == (1, n) and b.dtype == torch.bfloat16 and b.device == dev):
                nb = torch.zeros(1, n, dtype=torch.bfloat16, device=dev)
                if torch.is_tensor(b) and b.ndim == 2 and b.size(1) == n:
                    nb[0].copy_(b[0])
                group["update_buffer"] = nb
            group["update_buffer_views"] = [group["update_buffer"][0]]

    @torch.no_grad()
    def step(self):
        lib = _lib.load()
        for group in self.param_groups:
            update: Tensor = group["update_buffer_views"][self.rank]
            lr, wd, mu = group["lr"], group["weight_decay"], group["momentum"]
            nesterov = bool(group["nesterov"])
            # The matrices of one shape and dtype are independent (flash_muon/muon.py:90-103 walks
            # them one by one): take them `batch` at a time so that each Newton-Schulz stage is one
            # launch over the whole batch.
            buckets = {}
            for p in group["params"]:
                g = p.grad
                assert g is not None
                assert p.is_cuda and g.is_cuda, "Muon parameters and gradients must be CUDA tensors"
                buckets.setdefault((tuple(g.shape), g.dtype, p.dtype, g.device), []).append(p)
            for (_, _, _, dev), plist in buckets.items():
                # chunks of equal size (48 matrices go as 24 + 24, not 32 + 16): the launches of a small
                # chunk leave most of the GPU idle, and those of a full one spill into a second round
                per = -(-len(plist) // -(-len(plist) // self.batch))
                staging = self._staging_rows(update.numel(), per, dev)
                for i0 in range(0, len(plist), per):
                    chunk = plist[i0:i0 + per]
                    n = len(chunk)
                    stream = _lib.stream_ptr(dev)
                    gcs, bufs = [], []
                    for p in chunk:
                        g = p.grad
                        state = self.state[p]
                        if "momentum_buffer" not in state:
                            state["momentum_buffer"] = torch.zeros_like(g, memory_format=torch.contiguous_format)
                        buf: Tensor = state["momentum_buffer"]
                        # the kernel reads both through one dtype code and one element count
                        assert buf.shape == g.shape and buf.device == g.device, \
                            "momentum_buffer must match the gradient in shape and device"
                        if buf.dtype != g.dtype:   # load_state_dict casts state to the parameter's dtype
                            buf = state["momentum_buffer"] = buf.to(g.dtype)
                        if not buf.is_contiguous():   # e.g. a state loaded from elsewhere
                            buf = state["momentum_buffer"] = buf.contiguous()
                        gcs.append(g if g.is_contiguous() else g.contiguous())
                        bufs.append(buf)
                    # buf.lerp_(g, 1 - mu); g.lerp_(buf, mu) in place on p.grad (muon.py:99-100),
                    # one launch for the chunk
                    with _lib.on_device(dev):
                        st = lib.fm_momentum_nesterov_batched(
                            (ctypes.c_void_p * n)(*[t.data_ptr() for t in gcs]),
                            (ctypes.c_void_p * n)(*[t.data_ptr() for t in bufs]),
                            n, _lib.dtype_code(gcs[0].dtype), gcs[0].numel(), 1 - mu, mu,
                            1 if nesterov else 0, stream)
                    _lib.check("fm_momentum_nesterov_batched", st)
                    srcs = []
                    for p, gc, buf in zip(chunk, gcs, bufs):
                        if gc is not p.grad and nesterov:
                            p.grad.copy_(gc)
                        src = gc if nesterov else buf
                        if src.ndim == 4:   # conv filters (muon.py:101-102)
                            src = src.view(len(src), -1)
                        assert src.ndim == 2, "Input `d_in` must be a 2D tensor"
                        srcs.append(src)
                    # orthogonalise (muon.py:103) into rows of the staging buffer
                    outs = [staging[i].view(srcs[i].shape) for i in range(n)]
                    _newtonschulz_into(srcs, outs, group["ns_steps"])
                    # p *= 1 - lr*wd ; p += -lr*sqrt(max(1, rows/cols)) * update (muon.py:87-89),
                    # one launch for the chunk (same shape, so the same scale)
                    pcs = [p if p.is_contiguous() else p.contiguous() for p in chunk]
                    alpha = -lr * max(1, chunk[0].size(-2) / chunk[0].size(-1)) ** 0.5
                    with _lib.on_device(dev):
                        st = lib.fm_weight_update_batched(
                            (ctypes.c_void_p * n)(*[t.data_ptr() for t in pcs]), _lib.dtype_code(pcs[0].dtype),
                            (ctypes.c_void_p * n)(*[staging[i].data_ptr() for i in range(n)]),
                            n, pcs[0].numel(), 1 - lr * wd, alpha, stream)
                    _lib.check("fm_weight_update_batched", st)
                    for p, pc in zip(chunk, pcs):
                        if pc is not p:
                            p.copy_(pc)
                    if chunk[-1] is group["params"][-1]:
                        # the group's update buffer ends up holding the update of its last
                        # parameter, as after the last gather of muon.py:108
                        update.copy_(staging[len(chunk) - 1])

    def _staging_rows(self, numel, rows, device):
        """[rows, numel] bf16 scratch the batched orthogonalisation writes its updates to."""
        key = (numel, str(device))
        t = self._staging.get(key)
        if t is None or t.size(0) < rows:
            t = self._staging[key] = torch.empty(rows, numel, dtype=torch.bfloat16, device=device)
        return t
