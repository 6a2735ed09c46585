#!/usr/bin/env python3
"""Benchmark of the flash-muon hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] [--cpu-full]
    python bench.py --vendor-gemm {rocblas,hipblaslt} [--steps K] [--warmup W]   # torch.matmul(X, X.T) alone, for profiles
    python bench.py --mfma-probe                                                 # MFMA-only loops (libflashmuon_probe.so)

A step is one matmul_transpose call on the 8192 x 8192 bf16 input of the square sweep (seed 8192),
inputs resident in HBM.  Protocol of the reference's benchmark.py:49-79: W warm-up calls, then K
calls bracketed by device events.  One JSON line is printed; `value` is useful TFLOP/s
(K*M*(M+1) flop per call), `roofline` prices the same kernel against the dense bf16 MFMA peak,
`cpu_baseline` is torch's fp32 X @ X.T on the host cores of the same machine.  `extras` holds the
other timings of the path: the smaller sizes of the square sweep, fast_newtonschulz(5) on 8192^2
and 4096 x 16384 beside torch's, Muon.step on Llama-7B shapes (with checks that the 32-per-launch
schedule gives the bits of one matrix per launch), sides that are not whole tiles, and the vendor
GEMM X @ X.T on the same GPU: blocks of calls of this library, of torch.matmul through rocBLAS and
through hipBLASLt alternate right behind the headline (`xxt_8192_same_phase_ms`, `torch_xxt_*`),
so that all three are timed in the same phase of the chip's power management.  Order of the
timings: W + K calls straight after the input generation (the transient after idle), the extras,
100 + 200 calls (`xxt_8192_steady_ms`), the W + K calls of the headline, six blocks of 5.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
DIM = 8192
# L2-miss traffic of one 8192^2 call (a single kernel) is not measured by this script: it comes from
# rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of it, each scaled by what the same counter reads
# for a 128 MiB device copy.  The commands, the raw readings and the line
# `traffic_bytes_per_call: N` that is read here are in this file:
TRAFFIC_FILE = os.path.join("profiles", "syrk_bf16_8192_traffic.md")


def _traffic_bytes():
    """(bytes per call, where the figure comes from), or (None, why not)."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            for ln in f:
                if ln.startswith("traffic_bytes_per_call:"):
                    return int(float(ln.split(":", 1)[1].split()[0])), "constant from %s (rocprofv3 counters, not this run)" % TRAFFIC_FILE
    except OSError:
        pass
    return None, "%s holds no traffic_bytes_per_call line" % TRAFFIC_FILE


def _time_gpu(fn, steps, warmup, torch):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps   # ms per call


def _median(v):
    v = sorted(v)
    return v[len(v) // 2] if len(v) % 2 else 0.5 * (v[len(v) // 2 - 1] + v[len(v) // 2])


def _interleaved(fns, calls, blocks, warm, torch):
    """Time the functions of `fns` (name -> callable) in the same phase of the chip's power management:
    `warm` calls of each, then `blocks` rounds in which every function in turn is timed over `calls`
    calls (the reference times its functions back to back per size, benchmark.py:66-80).  Returns
    name -> (median ms per call over the blocks, the blocks)."""
    for fn in fns.values():
        for _ in range(warm):
            fn()
    torch.cuda.synchronize()
    t = {k: [] for k in fns}
    for _ in range(blocks):
        for k, fn in fns.items():
            t[k].append(_time_gpu(fn, calls, 0, torch))
    return {k: (_median(v), v) for k, v in t.items()}


def _mfma_probe(torch):
    """Sustained rate and clock of MFMA-only work (fm_probe_mfma_peak), on zeros and on N(0,1) bf16
    operands, for the two MFMA shapes and with or without the GEMM's LDS fragment traffic: about
    150 ms of back-to-back launches each, the second half timed."""
    import ctypes
    from flash_muon_amd import _lib, build
    if not os.path.exists(build.PROBE_LIB_PATH):
        build.build()
    lib = ctypes.CDLL(build.PROBE_LIB_PATH)   # the probe is not part of the product library
    vp = ctypes.c_void_p
    lib.fm_probe_mfma_peak.restype = ctypes.c_int
    lib.fm_probe_mfma_peak.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp, ctypes.c_int, ctypes.c_int]
    blocks, iters, launches = 256, 256, 480
    sink = torch.empty(blocks * 256, dtype=torch.float32, device="cuda")
    clocks = torch.zeros(blocks * 2, dtype=torch.int64, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(1)
    out = {}
    data = (("zeros", torch.zeros(blocks * 256 * 64, dtype=torch.bfloat16, device="cuda")),
            ("gaussian", torch.randn(blocks * 256 * 64, generator=g, device="cuda").bfloat16()))
    for rep in range(2):   # every variant twice, in turn, so that drift of the box shows
        for name, ops in data:
            for shape, lds in ((0, 0), (1, 0), (0, 1), (1, 1)):
                key = "%s_%s%s" % (name, ("32x32x16", "16x16x32")[shape], "_lds" if lds else "")
                st = _lib.stream_ptr("cuda")
                args = (ops.data_ptr(), blocks, iters, launches // 2, sink.data_ptr(), clocks.data_ptr(), st, shape, lds)
                lib.fm_probe_mfma_peak(*args)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                lib.fm_probe_mfma_peak(*args)
                e0.record()
                rc = lib.fm_probe_mfma_peak(*args)
                e1.record()
                torch.cuda.synchronize()
                assert rc == 0
                ms = e0.elapsed_time(e1) / (launches // 2)
                c = clocks.view(blocks, 2).double().mean(0)
                flop = blocks * 4 * iters * 64 * 32768.0
                out.setdefault(key, []).append(
                    {"tflops": flop / ms / 1e9, "ms_per_launch": ms, "shader_cycles": float(c[0]),
                     "realtime_ticks_100mhz": float(c[1]), "clock_ghz": float(c[0] / c[1] / 10.0),
                     "mfma_issue_fraction": iters * 64 * 32 / float(c[0])})
    return out


def _cpu_baseline(X, torch, ns=True, full=False):
    """torch fp32 X @ X.T on the host (the reference's own baseline, benchmark.py:20-21)."""
    from oracle import oracle
    M, K = X.shape
    t0 = time.perf_counter()
    oracle.xxt(X)                       # warm-up, also tells us how long one call takes
    first = time.perf_counter() - t0
    reps = 3 if first < 8.0 else 1
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.xxt(X)
    dt = (time.perf_counter() - t0) / reps
    from flash_muon_amd import synthetic
    out = {"value": synthetic.syrk_useful_flop(M, K) / dt / 1e12, "unit": "TFLOP/s (useful)",
           "cores": torch.get_num_threads(), "kind": "port",
           "sample": "torch CPU fp32 X@X.T on the full %dx%d input, 1 warm-up + %d reps, %.2f s each; "
                     "os.cpu_count()=%d" % (M, K, reps, dt, os.cpu_count())}
    if ns:
        # the fp32 Newton-Schulz oracle on the rectangular case, once (6.2 TFLOP), and the distance of
        # the GPU result from it on the same input
        from flash_muon_amd import fast_newtonschulz
        rows, cols = 4096, 16384
        G = synthetic.gradient_like_bf16(rows, cols, 8, 3)
        t0 = time.perf_counter()
        ref = oracle.newtonschulz(G, 5)
        ns_s = time.perf_counter() - t0
        got = fast_newtonschulz(G.cuda(), 5).cpu()
        out["ns5_4096x16384_cpu_s"] = ns_s
        out["ns5_4096x16384_cpu_tflops"] = 5 * (4.0 * rows * rows * cols + 2.0 * rows ** 3) / ns_s / 1e12
        out["ns5_4096x16384_gpu_vs_cpu_rel_fro"] = float(oracle.rel_fro(got, ref))
    if full:
        # the square Newton-Schulz case (16.5 TFLOP) and one Llama-7B layer of Muon.step (7 matrices,
        # 21.4 TFLOP) on the CPU, once each; the step over all 32 layers is 32 times that layer
        from flash_muon_amd import fast_newtonschulz
        G = synthetic.gradient_like_bf16(8192, 8192, 16, 4)
        t0 = time.perf_counter()
        ref = oracle.newtonschulz(G, 5)
        out["ns5_8192x8192_cpu_s"] = time.perf_counter() - t0
        out["ns5_8192x8192_gpu_vs_cpu_rel_fro"] = float(oracle.rel_fro(fast_newtonschulz(G.cuda(), 5).cpu(), ref))
        ps, gs = synthetic.llama7b_layer(0)
        t0 = time.perf_counter()
        oracle.muon_step(ps, gs, [None] * len(ps))
        layer_s = time.perf_counter() - t0
        out["muon_step_one_layer_cpu_s"] = layer_s
        out["muon_step_llama7b_cpu_s_extrapolated_x32"] = 32 * layer_s
    return out


def _torch_ns(G, steps, torch):
    """The plain-torch Newton-Schulz the reference benchmarks against (benchmark.py:23-47), on the GPU:
    vendor GEMMs and eager elementwise ops, bf16."""
    a, b, c = 3.4445, -4.7750, 2.0315
    X = G.bfloat16()
    tall = G.size(0) > G.size(1)
    if tall:
        X = X.T
    X = X / (X.norm() + 1e-7)
    for _ in range(steps):
        A = X @ X.T
        B = b * A + c * A @ A
        X = a * X + B @ X
    return X.T if tall else X


def _extras(Xd, steps, warmup, torch):
    from flash_muon_amd import Muon, fast_newtonschulz, synthetic
    ex = {}
    # The smaller sizes of the square sweep (seed = dim; 1024 is the CPU-sized case, seed 0) and a wide
    # input with few output tiles and a long k.  Every speed-up is a ratio of medians of blocks that
    # alternate between the two functions after a warm-up of both (six blocks of 50 calls each), so
    # that both are timed in the same state of the chip; the reference's own protocol (W + K calls
    # of one function, then of the other, benchmark.py:66-80) is reported as times only.
    from flash_muon_amd import matmul_transpose
    for rows, cols, seed in ((1024, 1024, 0), (2048, 2048, 2048), (4096, 4096, 4096), (1024, 8192, 1024)):
        Xs = synthetic.gaussian_bf16(rows, cols, seed).cuda()
        tag = "%d" % rows if rows == cols else "%dx%d" % (rows, cols)
        if rows == cols:
            ex["xxt_%s_ms" % tag] = _time_gpu(lambda: matmul_transpose(Xs), steps, warmup, torch)
            ex["torch_xxt_%s_ms" % tag] = _time_gpu(lambda: torch.matmul(Xs, Xs.T), steps, warmup, torch)
        r = _interleaved({"ours": lambda: matmul_transpose(Xs), "torch": lambda: torch.matmul(Xs, Xs.T)},
                         50, 6, 100, torch)
        ex["xxt_%s_steady_ms" % tag] = r["ours"][0]
        ex["torch_xxt_%s_steady_ms" % tag] = r["torch"][0]
        ex["xxt_%s_steady_speedup_vs_torch" % tag] = r["torch"][0] / r["ours"][0]
        ex["xxt_%s_steady_useful_tflops" % tag] = synthetic.syrk_useful_flop(rows, cols) / r["ours"][0] / 1e9
        del Xs
    # fast_newtonschulz(5) on the gradient-like inputs of the rectangular and the square case
    # (noise of std 1e-3 plus a rank-r spike, Frobenius-normalised; generated on the CPU from the
    # seed so that the CPU oracle sees the same bits)
    for rows, cols, rank, seed in ((8192, 8192, 16, 4), (4096, 16384, 8, 3)):
        G = synthetic.gradient_like_bf16(rows, cols, rank, seed).cuda()
        r = _interleaved({"ours": lambda: fast_newtonschulz(G, 5), "torch": lambda: _torch_ns(G, 5, torch)},
                         5, 3, 3, torch)
        ms, ref_ms = r["ours"][0], r["torch"][0]
        fl = synthetic.ns_useful_flop(rows, cols, 5)
        ex["ns5_%dx%d_ms" % (rows, cols)] = ms
        ex["ns5_%dx%d_useful_tflops" % (rows, cols)] = fl / ms / 1e9
        ex["ns5_%dx%d_frac_of_peak" % (rows, cols)] = fl / ms / 1e9 / PEAK_BF16_TFLOPS
        ex["torch_ns5_%dx%d_ms" % (rows, cols)] = ref_ms
        ex["ns5_%dx%d_speedup_vs_torch" % (rows, cols)] = ref_ms / ms
        del G
    # Muon.step on Llama-7B shapes: 32 layers x (4 x 4096^2, 2 x 11008x4096, 1 x 4096x11008)
    g = torch.Generator(device="cuda").manual_seed(5)
    params = []
    for layer in range(32):
        for (r, c) in synthetic.LLAMA7B_LAYER_SHAPES:
            p = torch.nn.Parameter((0.02 * torch.randn(r, c, generator=g, device="cuda", dtype=torch.float32)).bfloat16())
            p.grad = (1e-3 * torch.randn(r, c, generator=g, device="cuda", dtype=torch.float32)).bfloat16()
            params.append(p)
    opt = Muon(params, lr=0.02, momentum=0.95, nesterov=True, rank=0, world_size=1)
    # Twins of two parameters, stepped one matrix per launch afterwards: the last 4096^2 matrix (whose
    # update the group's buffer still holds after a step) and an 11008 x 4096 one.
    last_sq = max(i for i, p in enumerate(params) if tuple(p.shape) == (4096, 4096))
    tall = next(i for i, p in enumerate(params) if tuple(p.shape) == (11008, 4096))
    twins = []
    for i in (last_sq, tall):
        q = torch.nn.Parameter(params[i].detach().clone())
        q.grad = params[i].grad.clone()
        twins.append(q)
    nsteps = 4   # one warm-up and three timed steps
    ms = _time_gpu(opt.step, nsteps - 1, 1, torch)
    fl = sum(synthetic.ns_useful_flop(r, c, 5) for (r, c) in synthetic.LLAMA7B_LAYER_SHAPES) * 32
    ex["muon_step_llama7b_ms"] = ms
    ex["muon_step_llama7b_useful_tflops"] = fl / ms / 1e9
    ex["muon_step_llama7b_frac_of_peak"] = fl / ms / 1e9 / PEAK_BF16_TFLOPS
    # what was timed is looked at: every parameter finite, and the two twins, stepped the same number
    # of times one matrix per launch, end where their originals did (bf16 parameters: the two runs
    # differ in fp32 summation order, which flips the rounding of a few elements of a step)
    for p in params:
        assert bool(torch.isfinite(p).all()), "Muon.step left a parameter that is not finite"
    for q, i, name in ((twins[0], last_sq, "4096x4096"), (twins[1], tall, "11008x4096")):
        q0 = q.detach().clone()
        topt = Muon([q], lr=0.02, momentum=0.95, nesterov=True, rank=0, world_size=1, batch=1)
        for _ in range(nsteps):
            topt.step()
        moved = (params[i].detach().float() - q0.float())
        diff = (params[i].detach().float() - q.detach().float())
        rel = float(diff.norm() / moved.norm())
        ex["muon_step_llama7b_%s_vs_one_per_launch_rel_fro" % name] = rel
        assert rel < 0.1, "Muon.step at 32 per launch and at 1 per launch moved a %s parameter differently: %g" % (name, rel)
        assert torch.equal(q.grad, params[i].grad), "momentum / Nesterov state differs"
        if i == last_sq:   # the orthogonalised update itself, as the last step left it in the group's buffer
            ub = [g["update_buffer"][0] for g in opt.param_groups if g["params"][-1] is params[i]]
            if ub:
                tu = topt.param_groups[0]["update_buffer"][0].float()
                rel_u = float((ub[0].float() - tu).norm() / tu.norm())
                ex["muon_step_llama7b_update_vs_one_per_launch_rel_fro"] = rel_u
                assert rel_u < 6e-3, "update of the last 4096^2 parameter differs from the one-per-launch one: %g" % rel_u
        del topt
    del opt, params, twins
    torch.cuda.empty_cache()
    # sides that are not whole tiles: both calls run on zero-padded copies in their workspace
    Xr = synthetic.gaussian_bf16(4000, 4000, 4000).cuda()
    r = _interleaved({"ours": lambda: matmul_transpose(Xr), "torch": lambda: torch.matmul(Xr, Xr.T)}, 50, 4, 50, torch)
    ours_r, ref_r = r["ours"][0], r["torch"][0]
    ex["xxt_4000_steady_ms"] = ours_r
    ex["torch_xxt_4000_steady_ms"] = ref_r
    ex["xxt_4000_steady_speedup_vs_torch"] = ref_r / ours_r
    r = _interleaved({"ours": lambda: fast_newtonschulz(Xr, 5), "torch": lambda: _torch_ns(Xr, 5, torch)}, 5, 3, 3, torch)
    ns_r, ref_ns_r = r["ours"][0], r["torch"][0]
    ex["ns5_4000x4000_ms"] = ns_r
    ex["torch_ns5_4000x4000_ms"] = ref_ns_r
    ex["ns5_4000x4000_speedup_vs_torch"] = ref_ns_r / ns_r
    del Xr
    # Muon.step on a GPT-2-small-like set: 12 layers x (4 x 768^2, 3072x768, 768x3072)
    params = []
    for layer in range(12):
        for (r, c) in ((768, 768),) * 4 + ((3072, 768), (768, 3072)):
            p = torch.nn.Parameter((0.02 * torch.randn(r, c, generator=g, device="cuda", dtype=torch.float32)).bfloat16())
            p.grad = (1e-3 * torch.randn(r, c, generator=g, device="cuda", dtype=torch.float32)).bfloat16()
            params.append(p)
    opt = Muon(params, lr=0.02, momentum=0.95, nesterov=True, rank=0, world_size=1)
    ex["muon_step_gpt2_small_like_ms"] = _time_gpu(opt.step, 20, 5, torch)
    return ex


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--no-extras", action="store_true", help="skip vendor GEMM, Newton-Schulz and Muon.step timings")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-full", action="store_true",
                    help="also time the CPU oracle on Newton-Schulz 8192^2 and on one Llama-7B layer of "
                         "Muon.step (about a minute of CPU work)")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="only run the MFMA-only loop on zeros and on N(0,1) operands and print its sustained "
                         "TFLOP/s and shader clock: the ceiling the power cap sets for matrix work")
    ap.add_argument("--vendor-gemm", choices=("rocblas", "hipblaslt"),
                    help="only run W + K calls of torch.matmul(X, X.T) on the 8192^2 input with that BLAS back "
                         "end and print their time: the vendor kernel by itself, for counter runs beside ours")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 128 MiB device-to-device copy, the known-size kernel that "
                         "FETCH_SIZE / WRITE_SIZE counter readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path is built and measured on a single MI355X "
                 "(Muon's cross-rank gather is out of scope); run with --gpus 1")

    import torch
    from flash_muon_amd import _lib, matmul_transpose_assign, synthetic
    if not os.path.exists(_lib.LIB_PATH):
        from flash_muon_amd import build
        build.build()
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    if args.mfma_probe:
        print(json.dumps({"mfma_probe": _mfma_probe(torch)}))
        return

    X = synthetic.gaussian_bf16(DIM, DIM, DIM)
    Xd = X.cuda()
    if args.vendor_gemm:
        torch.backends.cuda.preferred_blas_library({"rocblas": "cublas", "hipblaslt": "cublaslt"}[args.vendor_gemm])
        ms = _time_gpu(lambda: torch.matmul(Xd, Xd.T), args.steps, args.warmup, torch)
        print(json.dumps({"vendor_gemm": args.vendor_gemm, "ms_per_call": ms, "steps": args.steps,
                          "executed_tflops": 2.0 * DIM ** 3 / ms / 1e9}))
        return
    Y = torch.empty(DIM, DIM, dtype=torch.bfloat16, device="cuda")
    torch.cuda.empty_cache()
    # The same W + K calls straight after the idle time of the input generation: the power
    # management of the chip overshoots for the first ~40 calls after idle (the second call is the
    # fastest of all, calls 5-25 the slowest), so this figure is reported beside the headline,
    # which is taken after the other timings below have run.
    cold_ms = _time_gpu(lambda: matmul_transpose_assign(Xd, Y), args.steps, args.warmup, torch)
    ex = None
    vendor = {}
    if not args.no_extras:
        ex = _extras(Xd, args.steps, args.warmup, torch)
        # The vendor GEMM for the same product, with both BLAS back ends torch can select, in the same
        # phase as this library's call: after 100 calls of ours, six rounds of 20 calls of each of
        # the three in turn.  Every speed-up over the vendor below is a ratio of these medians.
        def blas(pref):
            def f():
                torch.backends.cuda.preferred_blas_library(pref)
                return torch.matmul(Xd, Xd.T)
            return f
        try:
            vendor = _interleaved({"ours": lambda: matmul_transpose_assign(Xd, Y), "rocblas": blas("cublas"),
                                   "hipblaslt": blas("cublaslt")}, 20, 6, 34, torch)
        except Exception as e:   # report, never hide
            vendor = {"error": "%s" % e}
        torch.backends.cuda.preferred_blas_library("default")
    # sustained: 200 calls after 100 (a quarter of a second of nothing but this kernel)
    steady_ms = _time_gpu(lambda: matmul_transpose_assign(Xd, Y), 200, 100, torch)
    # the headline, straight after that sustained run
    ms = _time_gpu(lambda: matmul_transpose_assign(Xd, Y), args.steps, args.warmup, torch)
    assert torch.equal(Y, Y.T), "output is not symmetric"
    # the spread of the timed region, in blocks of 5 calls
    blocks = [_time_gpu(lambda: matmul_transpose_assign(Xd, Y), 5, 0, torch) for _ in range(6)]
    if args.copy_calibration:
        Z = torch.empty_like(Xd)
        Z.copy_(Xd)
        torch.cuda.synchronize()

    useful = synthetic.syrk_useful_flop(DIM, DIM)
    tflops = useful / ms / 1e9
    traffic, traffic_source = _traffic_bytes()
    line = {
        "metric": "matmul_transpose useful TFLOP/s at 8192x8192 bf16",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "matmul_transpose square sweep, dim=8192, bf16 N(0,1), seed 8192",
                   "M": DIM, "K": DIM},
        "effective_tflops": 2.0 * DIM * DIM * DIM / ms / 1e9,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": traffic,
                     "traffic_source": traffic_source,
                     "flop_per_launch": useful, "kernel": "gemm_nt_rounds_kernel"},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = _cpu_baseline(X, torch, ns=not args.no_extras, full=args.cpu_full)
    if ex is None:
        ex = {}
    if "error" in vendor:
        ex["torch_xxt_vendor"] = "failed: " + vendor["error"]
    elif vendor:
        ex["xxt_8192_same_phase_ms"] = vendor["ours"][0]
        ex["xxt_8192_same_phase_blocks_ms"] = vendor["ours"][1]
        for name in ("rocblas", "hipblaslt"):
            ex["torch_xxt_%s_ms" % name] = vendor[name][0]
            ex["torch_xxt_%s_blocks_ms" % name] = vendor[name][1]
            ex["torch_xxt_%s_speedup" % name] = vendor[name][0] / vendor["ours"][0]
    ex["xxt_8192_steady_ms"] = steady_ms
    ex["xxt_8192_steady_frac_of_peak"] = useful / steady_ms / 1e9 / PEAK_BF16_TFLOPS
    ex["ms_per_step_first_calls_after_idle"] = cold_ms
    ex["ms_per_step_blocks_of_5_after"] = blocks
    ex["ms_per_step_best_block"] = min(blocks)
    line["extras"] = ex
    print(json.dumps(line))


if __name__ == "__main__":
    main()
