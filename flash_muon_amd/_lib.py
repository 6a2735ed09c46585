"""ctypes binding of libflashmuon_hip.so (the declarations mirror include/flashmuon.h).

There is no fallback: if the library has not been built, or a call returns a non-zero status,
an exception is raised.
"""
import ctypes
import os

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libflashmuon_hip.so")

# fm_status values (include/flashmuon.h)
FM_OK = 0
FM_ERR_STRIDE = 3
FM_ERR_ALIAS = 5
# fm_knob values
FM_KNOB_GRID, FM_KNOB_KSPLIT, FM_KNOB_FAST_MIN_UNITS, FM_KNOB_NO_MID, FM_KNOB_NO_SUB64, FM_KNOB_HALF, FM_KNOB_DIAG_LAST, FM_KNOB_NO_TICKETS = 0, 1, 2, 3, 4, 5, 6, 7
FM_BF16, FM_F16, FM_F32 = 0, 1, 2

_DTYPE_CODE = {torch.bfloat16: FM_BF16, torch.float16: FM_F16, torch.float32: FM_F32}

_vp, _i64, _i32, _f32, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                              ctypes.c_size_t)

# name -> (restype, argtypes); one entry per FM_API declaration in include/flashmuon.h
SIGNATURES = {
    "fm_status_string": (ctypes.c_char_p, [_i32]),
    "fm_version": (ctypes.c_char_p, []),
    "fm_set_knob": (_i32, [_i32, ctypes.c_longlong]),
    "fm_gemm_workspace_bytes": (_sz, [_i32, _i32]),
    "fm_syrk_workspace_bytes": (_sz, [_i32, _i32]),
    "fm_syrk_bf16": (_i32, [_vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp, _sz, _vp]),
    "fm_syrk_bf16_static": (_i32, [_vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp]),
    "fm_syrk_f16": (_i32, [_vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp, _sz, _vp]),
    "fm_syrk_f32": (_i32, [_vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp, _sz, _vp]),
    "fm_syrk_poly_bf16": (_i32, [_vp, _i64, _vp, _i64, _i32, _f32, _f32, _vp, _vp, _sz, _vp]),
    "fm_gemm_axpby_bf16": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i32, _i32,
                                  _f32, _vp, _vp, _sz, _vp]),
    "fm_sumsq_workspace_bytes": (_sz, []),
    "fm_sumsq": (_i32, [_vp, _i32, _i32, _i32, _i64, _vp, _vp, _sz, _vp]),
    "fm_scale_cast_bf16": (_i32, [_vp, _i32, _i32, _i32, _i64, _vp, _f32, _vp, _i64, _vp, _i64, _vp]),
    "fm_newtonschulz_workspace_bytes": (_sz, [_i32, _i32]),
    "fm_newtonschulz_bf16": (_i32, [_vp, _i32, _i32, _i32, _i64, _vp, _i64, _i32, _f32, _f32, _f32,
                                    _f32, _vp, _sz, _vp]),
    "fm_newtonschulz_batched_workspace_bytes": (_sz, [_i32, _i32, _i32]),
    "fm_newtonschulz_batched_bf16": (_i32, [_vp, _i32, _i32, _i32, _i32, _i64, _vp, _i64, _i32, _f32, _f32,
                                            _f32, _f32, _vp, _sz, _vp]),
    "fm_momentum_nesterov": (_i32, [_vp, _vp, _i32, _i64, _f32, _f32, _i32, _vp]),
    "fm_weight_update": (_i32, [_vp, _i32, _vp, _i64, _f32, _f32, _vp]),
    "fm_momentum_nesterov_batched": (_i32, [_vp, _vp, _i32, _i32, _i64, _f32, _f32, _i32, _vp]),
    "fm_weight_update_batched": (_i32, [_vp, _i32, _vp, _i32, _i64, _f32, _f32, _vp]),
}

_lib = None


def load():
    """Load the shared library once and attach the C signatures."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m flash_muon_amd.build` "
                "(there is no fallback path)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class FlashMuonError(RuntimeError):
    def __init__(self, fn, status):
        self.status = status
        msg = load().fm_status_string(status).decode()
        super().__init__("%s failed with status %d: %s" % (fn, status, msg))


def check(fn, status):
    if status != FM_OK:
        raise FlashMuonError(fn, status)


def dtype_code(dtype):
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (bfloat16, float16, float32 are supported)" % dtype)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device):
    """The hipStream_t of torch's current stream on `device`, as an integer."""
    if _raw_stream is not None:      # the same value without building a Stream object (a few us per call)
        idx = torch.device(device).index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def on_device(device):
    """Context that makes `device` the current one for the kernel launches of a call; nothing to
    enter or leave when it is current already."""
    idx = torch.device(device).index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(idx)


def workspace(nbytes, device):
    """Scratch for one call, taken from torch's caching allocator on the current stream."""
    if nbytes == 0:
        return None, 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return ws, nbytes


_gemm_ws = {}


def gemm_workspace(nbytes, device, stream=None):
    """The scratch of the single GEMM-shaped calls (partial tiles, at most 192 MiB; for a product
    whose sides are not whole tiles also its zero-padded operand and result), kept per device
    and stream: calls on one stream are ordered, so they can share it, and nothing is allocated
    per call."""
    if nbytes == 0:
        return None, 0
    key = (torch.device(device).index, stream_ptr(device) if stream is None else stream)
    ws = _gemm_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        # zeroed once: its last 256 bytes hold the word the library counts sub-tile tickets in, which
        # the library keeps in order from then on (garbage there costs speed, never correctness)
        ws = _gemm_ws[key] = torch.zeros(nbytes, dtype=torch.uint8, device=device)
    return ws, ws.numel()


def release_workspaces():
    """Give the cached scratch of the single GEMM-shaped calls back to torch's allocator.  One
    tensor per (device, stream) is kept and only ever grows (up to about 256 MiB each); call this after
    the last matmul_transpose on streams that will not be used again, or to drop a block that a call
    under graph capture took from the graph's private pool.  Not while such calls are in flight."""
    _gemm_ws.clear()
