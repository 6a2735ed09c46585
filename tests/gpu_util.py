"""Helpers for the GPU parity tests: direct calls into the C ABI on torch-owned device memory."""
import torch

from flash_muon_amd import _lib


def _stream(t):
    return _lib.stream_ptr(t.device)


def _ws(nbytes, dev):
    ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=dev)
    return ws


def syrk(lib, X, Y=None):
    M, K = X.shape
    if Y is None:
        Y = torch.empty(M, M, dtype=torch.bfloat16, device=X.device)
    ws = _ws(lib.fm_gemm_workspace_bytes(M, M), X.device)
    st = lib.fm_syrk_bf16(X.data_ptr(), X.stride(0), Y.data_ptr(), Y.stride(0), Y.stride(1), M, K,
                          ws.data_ptr(), ws.numel(), _stream(X))
    _lib.check("fm_syrk_bf16", st)
    return Y


def syrk_poly(lib, A, b, c, split_diag=False):
    """P = b*A + c*A*A; with split_diag returns (P with a zero diagonal, fp32 diagonal)."""
    M = A.size(0)
    P = torch.empty(M, M, dtype=torch.bfloat16, device=A.device)
    d = torch.empty(M, dtype=torch.float32, device=A.device) if split_diag else None
    ws = _ws(lib.fm_gemm_workspace_bytes(M, M), A.device)
    st = lib.fm_syrk_poly_bf16(A.data_ptr(), A.stride(0), P.data_ptr(), P.stride(0), M, b, c,
                               d.data_ptr() if split_diag else None,
                               ws.data_ptr(), ws.numel(), _stream(A))
    _lib.check("fm_syrk_poly_bf16", st)
    return (P, d) if split_diag else P


def gemm_axpby(lib, P, X, a, want_x=True, want_xt=True, XT=None, row_alpha=None):
    M, K = X.shape
    if XT is None:
        XT = X.T.contiguous()
    Xo = torch.empty(M, K, dtype=torch.bfloat16, device=X.device) if want_x else None
    XoT = torch.empty(K, M, dtype=torch.bfloat16, device=X.device) if want_xt else None
    ws = _ws(lib.fm_gemm_workspace_bytes(M, K), X.device)
    st = lib.fm_gemm_axpby_bf16(P.data_ptr(), P.stride(0), XT.data_ptr(), XT.stride(0),
                                X.data_ptr(), X.stride(0),
                                Xo.data_ptr() if want_x else None, Xo.stride(0) if want_x else 0,
                                XoT.data_ptr() if want_xt else None, XoT.stride(0) if want_xt else 0,
                                M, K, a, row_alpha.data_ptr() if row_alpha is not None else None,
                                ws.data_ptr(), ws.numel(), _stream(X))
    _lib.check("fm_gemm_axpby_bf16", st)
    return Xo, XoT


def sumsq(lib, G):
    rows, cols = G.shape
    out = torch.empty(1, dtype=torch.float32, device=G.device)
    ws = _ws(lib.fm_sumsq_workspace_bytes(), G.device)
    st = lib.fm_sumsq(G.data_ptr(), _lib.dtype_code(G.dtype), rows, cols, G.stride(0), out.data_ptr(),
                      ws.data_ptr(), ws.numel(), _stream(G))
    _lib.check("fm_sumsq", st)
    return out


def scale_cast(lib, G, ss, eps, want_d=True, want_t=True):
    rows, cols = G.shape
    D = torch.empty(rows, cols, dtype=torch.bfloat16, device=G.device) if want_d else None
    T = torch.empty(cols, rows, dtype=torch.bfloat16, device=G.device) if want_t else None
    st = lib.fm_scale_cast_bf16(G.data_ptr(), _lib.dtype_code(G.dtype), rows, cols, G.stride(0),
                                ss.data_ptr(), eps, D.data_ptr() if want_d else None, cols,
                                T.data_ptr() if want_t else None, rows, _stream(G))
    _lib.check("fm_scale_cast_bf16", st)
    return D, T


def ns_step(lib, X, coeffs):
    """One Newton-Schulz step on a bf16 device matrix X (M x K, M <= K) through the three kernels."""
    a, b, c = coeffs
    A = syrk(lib, X)
    P, d = syrk_poly(lib, A, b, c, split_diag=True)
    Xo, XoT = gemm_axpby(lib, P, X, a, row_alpha=d)
    return Xo, XoT, A, P
