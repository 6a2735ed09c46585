"""matmul_transpose / matmul_transpose_assign: y = x @ x.T on the upper-triangular tiles only.

Same signatures, argument checks and messages as the reference wrappers
(flash_muon/matmul_transpose_triton.py:78-107); the Triton launch at :90-101 is replaced by
fm_syrk_bf16 (fm_syrk_f16 / fm_syrk_f32 for float16 / float32 tensors) from libflashmuon_hip.so.
"""
import torch

from . import _lib

# the element type comes from the input, as in the reference's kernel (matmul_transpose_triton.py:63)
_ENTRY = {torch.bfloat16: "fm_syrk_bf16", torch.float16: "fm_syrk_f16", torch.float32: "fm_syrk_f32"}


def matmul_transpose_assign(d_in, d_out):
    """Write d_in @ d_in.T into d_out (any strides).  Returns None.

    Follows flash_muon/matmul_transpose_triton.py:78-101.  The reference's shape assert never
    looks at d_out.size(1) (:85); here both output dimensions are checked.
    """
    assert d_in.is_cuda, "Input `d_in` must be a CUDA tensor"
    assert d_out.is_cuda, "Input `d_out` must be a CUDA tensor"
    assert d_in.device == d_out.device, "Inputs `d_in` and `d_out` must be on the same CUDA device"
    assert d_in.dtype == d_out.dtype, "Inputs must have the same data type"
    assert d_in.ndim == 2, "Input `d_in` must be a 2D tensor"
    assert d_out.ndim == 2, "Input `d_out` must be a 2D tensor"
    assert d_in.size(0) == d_out.size(0) == d_out.size(1), \
        "First dimension of `d_in` must match first and second dimension of `d_out`"
    if d_in.dtype not in _ENTRY:
        raise TypeError("matmul_transpose: bfloat16, float16 and float32 are implemented on this device path, got %s"
                        % d_in.dtype)
    entry = _ENTRY[d_in.dtype]

    M, K = d_in.shape
    if M == 0:
        return
    # rows must be unit-stride in k; any row pitch is taken as it is
    if K > 0 and (d_in.stride(1) != 1 or d_in.stride(0) < K):
        d_in = d_in.contiguous()
    ldx = d_in.stride(0) if K > 0 and M > 1 else max(K, 1)
    lib = _lib.load()
    # an output whose strides fold two elements onto one address, or interleave rows and columns,
    # is written through a dense temporary, as the reference's masked stores would fill it
    rs, cs = (abs(d_out.stride(0)), abs(d_out.stride(1))) if M > 1 else (M, 1)
    dst = d_out
    if M > 1 and (min(rs, cs) == 0 or max(rs, cs) < M * min(rs, cs)):
        dst = torch.empty((M, M), device=d_in.device, dtype=d_in.dtype)
    with _lib.on_device(d_in.device):
        stream = _lib.stream_ptr(d_in.device)
        need = 0 if d_in.dtype == torch.float32 else lib.fm_syrk_workspace_bytes(M, K)
        ws, ws_bytes = _lib.gemm_workspace(need, d_in.device, stream)
        st = getattr(lib, entry)(d_in.data_ptr(), ldx, dst.data_ptr(),
                                 dst.stride(0) if M > 1 else M, dst.stride(1) if M > 1 else 1,
                                 M, K, ws.data_ptr() if ws is not None else None, ws_bytes, stream)
    _lib.check(entry, st)
    if dst is not d_out:
        d_out.copy_(dst)


def matmul_transpose(d_in):
    """Return d_in @ d_in.T as a new (M, M) tensor (flash_muon/matmul_transpose_triton.py:103-107)."""
    M, _ = d_in.shape
    d_out = torch.empty((M, M), device=d_in.device, dtype=d_in.dtype)
    matmul_transpose_assign(d_in, d_out)
    return d_out
