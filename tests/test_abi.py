"""The C-ABI library loads, exports every symbol include/flashmuon.h declares, and rejects bad
arguments before launching anything (so these run without a GPU)."""
import ctypes
import os
import re

import pytest
import torch

from flash_muon_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flashmuon.h")


def _declared():
    text = open(HEADER).read()
    return re.findall(r"^FM_API\s+[\w\s\*]+?\b(fm_\w+)\s*\(", text, flags=re.M)


def test_header_declares_entry_points():
    names = _declared()
    assert len(names) == len(set(names)) >= 13
    for must in ["fm_syrk_bf16", "fm_syrk_poly_bf16", "fm_gemm_axpby_bf16", "fm_sumsq",
                 "fm_scale_cast_bf16", "fm_newtonschulz_bf16", "fm_momentum_nesterov",
                 "fm_weight_update", "fm_status_string"]:
        assert must in names


def test_every_declared_symbol_is_exported_and_bound(lib):
    for name in _declared():
        assert hasattr(lib, name), name
        assert name in _lib.SIGNATURES, "no ctypes signature for %s" % name
    assert set(_lib.SIGNATURES) == set(_declared())


def test_ctypes_signatures_have_the_declared_arity():
    text = open(HEADER).read()
    for name, params in re.findall(r"^FM_API\s+[\w\s\*]+?\b(fm_\w+)\s*\(([^;]*?)\);", text, flags=re.M | re.S):
        params = params.strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert len(_lib.SIGNATURES[name][1]) == n, name


def test_version_and_status_strings(lib):
    assert re.match(rb"\d+\.\d+\.\d+$", lib.fm_version())
    assert lib.fm_status_string(0) == b"ok"
    seen = {lib.fm_status_string(i) for i in range(0, 9)}
    assert len(seen) == 9
    assert lib.fm_status_string(1234) == b"unknown status"


def test_argument_errors_are_reported_before_any_launch(lib):
    X = ctypes.c_void_p(0x1000)   # never dereferenced on the host, never reaches a launch
    Y = ctypes.c_void_p(0x200000)
    assert lib.fm_syrk_bf16(None, 8, Y, 8, 1, 8, 8, None, 0, None) == 1            # NULL
    assert lib.fm_syrk_bf16(X, 8, None, 8, 1, 8, 8, None, 0, None) == 1
    assert lib.fm_syrk_bf16(X, 4, Y, 8, 1, 8, 8, None, 0, None) == 3               # ldx < K
    assert lib.fm_syrk_bf16(X, 8, Y, 8, 1, -1, 8, None, 0, None) == 2              # shape
    assert lib.fm_syrk_bf16(ctypes.c_void_p(0x1001), 8, Y, 8, 1, 8, 8, None, 0, None) == 8   # alignment
    assert lib.fm_syrk_bf16(X, 8, Y, 8, 1, 0, 8, None, 0, None) == 0               # empty: nothing to do
    assert lib.fm_syrk_bf16(X, 8, ctypes.c_void_p(0x1040), 8, 1, 8, 8, None, 0, None) == 5   # Y inside X
    assert lib.fm_syrk_f32(X, 8, ctypes.c_void_p(0x1080), 1, 8, 8, 8, None, 0, None) == 5
    assert lib.fm_syrk_poly_bf16(X, 8, X, 8, 8, 1.0, 1.0, None, None, 0, None) == 5      # P aliases A
    # Xout overlapping X is rejected: every output tile reads a whole column block of X
    assert lib.fm_gemm_axpby_bf16(X, 8, Y, 8, ctypes.c_void_p(0x400000), 16, ctypes.c_void_p(0x400000), 16,
                                  None, 0, 8, 16, 1.0, None, None, 0, None) == 5
    assert lib.fm_gemm_axpby_bf16(X, 8, Y, 8, ctypes.c_void_p(0x400000), 16, None, 0, None, 0,
                                  8, 16, 1.0, None, None, 0, None) == 1            # no output at all
    assert lib.fm_sumsq(X, 7, 4, 4, 4, Y, Y, 4096, None) == 4                      # dtype
    assert lib.fm_sumsq(X, 0, 4, 4, 4, Y, None, 0, None) == 6                      # workspace
    assert lib.fm_newtonschulz_bf16(X, 0, 8, 8, 8, Y, 8, 5, 1.0, 1.0, 1.0, 1e-7, None, 0, None) == 6
    assert lib.fm_newtonschulz_bf16(X, 0, 8, 8, 8, X, 8, 5, 1.0, 1.0, 1.0, 1e-7, Y, 1 << 30, None) == 5
    assert lib.fm_momentum_nesterov(X, X, 0, 16, 0.05, 0.95, 1, None) == 5
    assert lib.fm_weight_update(X, 0, None, 16, 1.0, 1.0, None) == 1


def test_workspace_sizes(lib):
    assert lib.fm_sumsq_workspace_bytes() >= 4096
    small = lib.fm_newtonschulz_workspace_bytes(64, 96)
    big = lib.fm_newtonschulz_workspace_bytes(4096, 16384)
    assert 0 < small < big
    # four M x K bf16 iterates and two M x M bf16 squares dominate
    assert big >= 4 * 4096 * 16384 * 2 + 2 * 4096 * 4096 * 2
    assert big == lib.fm_newtonschulz_workspace_bytes(16384, 4096)
    assert lib.fm_newtonschulz_workspace_bytes(0, 5) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()
