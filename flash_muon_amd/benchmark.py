"""Side-by-side timings of this library and plain torch on one GPU, in the shape of the table the
reference prints (benchmark.py:49-85): square bf16 inputs of 1024 .. 8192, 25 warm-up calls, 100
timed calls between device events.

    python -m flash_muon_amd.benchmark [--dims 1024 2048 4096 8192] [--warmup 25] [--rep 100] [--no-compile]

Two tables: `matmul_transpose` against `G @ G.T`, and `fast_newtonschulz` (5 steps) against the same
iteration written with torch operators (benchmark.py:20-47), each with the reference's three
columns: this library, the torch baseline, and `torch.compile(baseline)` (benchmark.py:52-53).
torch's GEMMs go to the vendor BLAS; the compiled column reads n/a where torch.compile cannot
build the function on this machine (the reason is printed once).
"""
import argparse

import torch

from .matmul_transpose import matmul_transpose
from .muon import fast_newtonschulz


def torch_matmul_transpose(G):
    return G @ G.T


def torch_newtonschulz5(G, steps=5):
    """Quintic Newton-Schulz with torch operators: bf16 iterate, wide orientation, Frobenius
    normalisation with eps 1e-7, coefficients (3.4445, -4.7750, 2.0315)."""
    a, b, c = 3.4445, -4.7750, 2.0315
    X = G.bfloat16()
    tall = G.size(0) > G.size(1)
    if tall:
        X = X.T
    X = X / (X.norm() + 1e-7)
    for _ in range(steps):
        A = X @ X.T
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    return X.T if tall else X


def _time(fn, x, warmup, rep):
    for _ in range(warmup):
        fn(x)
    torch.cuda.empty_cache()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(rep):
        fn(x)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / rep


def run(name, impl, baseline, dims, warmup, rep, with_compiled=True):
    device = torch.cuda.get_device_name(torch.cuda.current_device())
    compiled = torch.compile(baseline) if with_compiled else None
    rows = []
    for dim in dims:
        x = torch.randn(dim, dim, device="cuda").bfloat16()
        t_impl, t_base, t_comp = _time(impl, x, warmup, rep), _time(baseline, x, warmup, rep), None
        if compiled is not None:
            try:
                t_comp = _time(compiled, x, warmup, rep)
            except Exception as e:   # no working code generator on this machine: say so, once
                print("torch.compile(%s) is not available here: %s: %s" % (baseline.__name__, type(e).__name__,
                                                                            str(e).splitlines()[0][:200]))
                compiled = None
        rows.append((device, dim, t_impl, t_base, t_comp))
    print("\nbenchmark %s:" % name)
    print("%-28s %6s %12s %12s %13s %9s" % ("device", "dim", "flash(ms)", "torch(ms)", "compiled(ms)", "speedup"))
    for device, dim, t_impl, t_base, t_comp in rows:
        comp = "%13.6f" % t_comp if t_comp is not None else "%13s" % "n/a"
        print("%-28s %6d %12.6f %12.6f %s %8.2fx" % (device[:28], dim, t_impl, t_base, comp, t_base / t_impl))
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--dims", type=int, nargs="+", default=[1024, 2048, 4096, 8192])
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--rep", type=int, default=100)
    ap.add_argument("--no-compile", action="store_true", help="leave the torch.compile column out")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("flash_muon_amd.benchmark needs a GPU")
    run("matmul transpose", matmul_transpose, torch_matmul_transpose, args.dims, args.warmup, args.rep, not args.no_compile)
    run("zeropower", fast_newtonschulz, torch_newtonschulz5, args.dims, args.warmup, args.rep, not args.no_compile)


if __name__ == "__main__":
    main()
