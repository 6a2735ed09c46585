"""MI355X (gfx950) implementation of flash-muon's hot path behind the reference's Python API.

The four public names and their signatures are those of the reference package
(flash_muon/__init__.py:1-4); the device code is libflashmuon_hip.so, reached through ctypes.
"""
from .matmul_transpose import matmul_transpose, matmul_transpose_assign
from .muon import fast_newtonschulz, Muon
from ._lib import release_workspaces   # not in the reference: drops the cached GEMM scratch

__all__ = ["matmul_transpose", "matmul_transpose_assign", "fast_newtonschulz", "Muon"]
