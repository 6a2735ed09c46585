#!/usr/bin/env python3
"""Benchmark of the flash-muon hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] [--cpu-full]

A step is one matmul_transpose call on the 8192 x 8192 bf16 input of the square sweep (seed 8192),
inputs resident in HBM.  Protocol of the reference's benchmark.py:49-79: W warm-up calls, then K
calls bracketed by device events.  One JSON line is printed; `value` is useful TFLOP/s
(K*M*(M+1) flop per call), `roofline` prices the same kernel against the dense bf16 MFMA peak,
`cpu_baseline` is torch's fp32 X @ X.T on the host cores of the same machine.  `extras` holds the
other timings of the path: vendor GEMM X @ X.T on the same GPU, the smaller sizes of the square
sweep, fast_newtonschulz(5) on 8192^2 and 4096 x 16384, and Muon.step on Llama-7B shapes.
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
# L2-miss traffic of one 8192^2 call (a single kernel), from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, each scaled by what the same counter reads for a 128 MiB device copy (FETCH_SIZE reads
# half of the copied bytes there, WRITE_SIZE all of them): 508.3e3 KiB * 2.0 fetched + 131.1e3 KiB
# written.  The commands and the raw readings are in profiles/syrk_bf16_8192_traffic.md.
TRAFFIC_BYTES = int(508.3e3 * 1024 * 2.0 + 131.1e3 * 1024 * 1.0)


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


def _mfma_probe(torch):
    """Sustained rate and clock of MFMA-only work (fm_probe_mfma_peak), on zeros and on N(0,1) bf16
    operands: about 150 ms of back-to-back launches each, the second half timed."""
    from flash_muon_amd import _lib
    lib = _lib.load()
    blocks, iters, launches = 256, 256, 480
    sink = torch.empty(blocks * 256, dtype=torch.float32, device="cuda")
    clocks = torch.zeros(blocks * 2, dtype=torch.int64, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(1)
    out = {}
    for name, ops in (("zeros", torch.zeros(blocks * 256 * 64, dtype=torch.bfloat16, device="cuda")),
                      ("gaussian", torch.randn(blocks * 256 * 64, generator=g, device="cuda").bfloat16())):
        st = _lib.stream_ptr("cuda")
        lib.fm_probe_mfma_peak(ops.data_ptr(), blocks, iters, launches // 2, sink.data_ptr(), clocks.data_ptr(), st)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        lib.fm_probe_mfma_peak(ops.data_ptr(), blocks, iters, launches // 2, sink.data_ptr(), clocks.data_ptr(), st)
        e0.record()
        rc = lib.fm_probe_mfma_peak(ops.data_ptr(), blocks, iters, launches // 2, sink.data_ptr(), clocks.data_ptr(), st)
        e1.record()
        torch.cuda.synchronize()
        assert rc == 0
        ms = e0.elapsed_time(e1) / (launches // 2)
        c = clocks.view(blocks, 2).double().mean(0)
        flop = blocks * 4 * iters * 64 * 32768.0
        out[name] = {"tflops": flop / ms / 1e9, "ms_per_launch": ms, "shader_cycles": float(c[0]),
                     "realtime_ticks_100mhz": float(c[1]), "clock_ghz": float(c[0] / c[1] / 10.0),
                     "mfma_issue_fraction": iters * 64 * 32 / float(c[0])}
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
    # vendor GEMM for the same product, both BLAS back ends torch can select
    for name, pref in (("rocblas", "cublas"), ("hipblaslt", "cublaslt")):
        try:
            torch.backends.cuda.preferred_blas_library(pref)
            ex["torch_xxt_%s_ms" % name] = _time_gpu(lambda: torch.matmul(Xd, Xd.T), steps, warmup, torch)
        except Exception as e:   # report, never hide
            ex["torch_xxt_%s_ms" % name] = "failed: %s" % e
    torch.backends.cuda.preferred_blas_library("default")
    # the smaller sizes of the square sweep (seed = dim; 1024 is the CPU-sized case, seed 0)
    from flash_muon_amd import matmul_transpose
    for dim, seed in ((1024, 0), (2048, 2048), (4096, 4096)):
        Xs = synthetic.gaussian_bf16(dim, dim, seed).cuda()
        ours = _time_gpu(lambda: matmul_transpose(Xs), steps, warmup, torch)
        ref = _time_gpu(lambda: torch.matmul(Xs, Xs.T), steps, warmup, torch)
        ex["xxt_%d_ms" % dim] = ours
        ex["xxt_%d_useful_tflops" % dim] = synthetic.syrk_useful_flop(dim, dim) / ours / 1e9
        ex["torch_xxt_%d_ms" % dim] = ref
        ex["xxt_%d_speedup_vs_torch" % dim] = ref / ours
        # W + K calls of these sizes last a few milliseconds and fall into the power-management
        # transient after idle; the same pair once more over 100 + 200 calls each
        ours_s = _time_gpu(lambda: matmul_transpose(Xs), 200, 100, torch)
        ref_s = _time_gpu(lambda: torch.matmul(Xs, Xs.T), 200, 100, torch)
        ex["xxt_%d_steady_ms" % dim] = ours_s
        ex["torch_xxt_%d_steady_ms" % dim] = ref_s
        ex["xxt_%d_steady_speedup_vs_torch" % dim] = ref_s / ours_s
        del Xs
    # a wide input with few output tiles and a long k (cut along k on the 128x128 path), steady state
    Xw = synthetic.gaussian_bf16(1024, 8192, 1024).cuda()
    ours_w = _time_gpu(lambda: matmul_transpose(Xw), 200, 100, torch)
    ref_w = _time_gpu(lambda: torch.matmul(Xw, Xw.T), 200, 100, torch)
    ex["xxt_1024x8192_steady_ms"] = ours_w
    ex["torch_xxt_1024x8192_steady_ms"] = ref_w
    ex["xxt_1024x8192_steady_speedup_vs_torch"] = ref_w / ours_w
    del Xw
    # fast_newtonschulz(5) on the gradient-like inputs of the rectangular and the square case
    # (noise of std 1e-3 plus a rank-r spike, Frobenius-normalised; generated on the CPU from the
    # seed so that the CPU oracle sees the same bits)
    for rows, cols, rank, seed in ((8192, 8192, 16, 4), (4096, 16384, 8, 3)):
        G = synthetic.gradient_like_bf16(rows, cols, rank, seed).cuda()
        ms = _time_gpu(lambda: fast_newtonschulz(G, 5), 10, 3, torch)
        fl = synthetic.ns_useful_flop(rows, cols, 5)
        ex["ns5_%dx%d_ms" % (rows, cols)] = ms
        ex["ns5_%dx%d_useful_tflops" % (rows, cols)] = fl / ms / 1e9
        ref_ms = _time_gpu(lambda: _torch_ns(G, 5, torch), 10, 3, torch)
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
    ms = _time_gpu(opt.step, 3, 1, torch)
    fl = sum(synthetic.ns_useful_flop(r, c, 5) for (r, c) in synthetic.LLAMA7B_LAYER_SHAPES) * 32
    ex["muon_step_llama7b_ms"] = ms
    ex["muon_step_llama7b_useful_tflops"] = fl / ms / 1e9
    ex["muon_step_llama7b_frac_of_peak"] = fl / ms / 1e9 / PEAK_BF16_TFLOPS
    del opt, params
    torch.cuda.empty_cache()
    # sides that are not whole tiles: both calls run on zero-padded copies in their workspace
    Xr = synthetic.gaussian_bf16(4000, 4000, 4000).cuda()
    ours_r = _time_gpu(lambda: matmul_transpose(Xr), 100, 30, torch)
    ref_r = _time_gpu(lambda: torch.matmul(Xr, Xr.T), 100, 30, torch)
    ex["xxt_4000_steady_ms"] = ours_r
    ex["torch_xxt_4000_steady_ms"] = ref_r
    ex["xxt_4000_steady_speedup_vs_torch"] = ref_r / ours_r
    ns_r = _time_gpu(lambda: fast_newtonschulz(Xr, 5), 10, 3, torch)
    ref_ns_r = _time_gpu(lambda: _torch_ns(Xr, 5, torch), 10, 3, torch)
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
    Y = torch.empty(DIM, DIM, dtype=torch.bfloat16, device="cuda")
    torch.cuda.empty_cache()
    # The same W + K calls straight after the idle time of the input generation: the power
    # management of the chip overshoots for the first ~40 calls after idle (the second call is the
    # fastest of all, calls 5-25 the slowest), so this figure is reported beside the headline,
    # which is taken after the other timings below have run.
    cold_ms = _time_gpu(lambda: matmul_transpose_assign(Xd, Y), args.steps, args.warmup, torch)
    ex = None
    if not args.no_extras:
        ex = _extras(Xd, args.steps, args.warmup, torch)
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
    line = {
        "metric": "matmul_transpose useful TFLOP/s at 8192x8192 bf16",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "matmul_transpose square sweep, dim=8192, bf16 N(0,1), seed 8192",
                   "M": DIM, "K": DIM},
        "effective_tflops": 2.0 * DIM * DIM * DIM / ms / 1e9,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_BYTES,
                     "flop_per_launch": useful, "kernel": "gemm_nt_rounds_kernel"},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = _cpu_baseline(X, torch, ns=not args.no_extras, full=args.cpu_full)
    if ex is None:
        ex = {}
    else:
        for k in ("torch_xxt_rocblas_ms", "torch_xxt_hipblaslt_ms"):
            if isinstance(ex.get(k), float):
                ex[k.replace("_ms", "_speedup")] = ex[k] / ms
    ex["ms_per_step_first_calls_after_idle"] = cold_ms
    ex["ms_per_step_blocks_of_5_after"] = blocks
    ex["ms_per_step_best_block"] = min(blocks)
    line["extras"] = ex
    print(json.dumps(line))


if __name__ == "__main__":
    main()
