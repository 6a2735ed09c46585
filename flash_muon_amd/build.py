"""Build libflashmuon_hip.so for gfx950 with hipcc, in-tree, next to this file.

    python -m flash_muon_amd.build          # compile every source and link

The library has no dependency on torch or Python headers: it is plain HIP behind a C ABI.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJDIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libflashmuon_hip.so")
SOURCES = ["fm_gemm.hip", "fm_gemm_fast.hip", "fm_elementwise.hip", "fm_api.hip"]
# a measurement aid (MFMA-only loop) that only `bench.py --mfma-probe` loads; a library of its own
PROBE_LIB_PATH = os.path.join(HERE, "libflashmuon_probe.so")
PROBE_SOURCES = [os.path.join("probe", "fm_probe.hip")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(os.path.basename(src))[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass prints that it ignores the packed-fp32 target feature; drop that line
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def _link(objs, path):
    tmp = path + ".tmp"
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr)
    os.replace(tmp, path)


def build(verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=5) as ex:
        objs = list(ex.map(_compile, SOURCES + PROBE_SOURCES))
    _link(objs[:len(SOURCES)], LIB_PATH)
    _link(objs[len(SOURCES):], PROBE_LIB_PATH)
    if verbose:
        print("built", LIB_PATH, "and", PROBE_LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
