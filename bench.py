#!/usr/bin/env python3
"""Benchmark of the N:M sparse x dense fp32 multiplication on one MI355X.

One "step" is one launch of the hot path (nmspmm_spmm through the C-ABI) on the square sweep of
the baseline: M = Ncols = K = 4096, fp32, operands resident in HBM, at 2:4 (the headline value),
3:8, 2:8 and 1:8 (reported under "sweep").  Prints ONE JSON line:

  value            useful TFLOP/s at 2:4 = 2*M*Ncols*W / t   (W = K*n/m)
  roofline         the dominant kernel (spmm_direct_kernel at 2:4) against the fp32 MFMA peak
  cpu_baseline     the reference project's own nmGEMM_on_cpu (oracle/_ref) on a row slice
  sweep            per pattern: ms, useful and dense-equivalent TFLOP/s, speedup over the dense
                   fp32 GEMM of the same shape (rocBLAS/hipBLASLt through torch.mm), and the GPU
                   preprocessing time (the reference's call sequence, and the one-kernel entry)

Timing uses HIP events on the stream the kernels are launched on (torch's current stream is the
one handed to the C-ABI).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
M = N = K = 4096
PATTERNS = [(2, 4), (3, 8), (2, 8), (1, 8)]  # first one is the headline
NS = 128


def geometry(n, m):
    window, kept = {(2, 4): (32, 16), (3, 8): (32, 12), (2, 8): (64, 16), (1, 8): (64, 8)}[(n, m)]
    times = {4: 3, 8: 2}[m] + (1 if window == 64 else 0)
    return window, kept, times


class Case:
    """Operands of one pattern, resident on the GPU, preprocessed by the GPU kernels."""

    def __init__(self, torch, pkg, datagen, n, m, seed):
        d = datagen.init_data(M, N, K, n, m, seed=seed)
        self.d, self.n, self.m = d, n, m
        self.W, self.Q = d["W"], d["Q"]
        self.window, self.kept, times = geometry(n, m)
        self.A = torch.from_numpy(d["A_km"]).cuda()
        self.B = torch.from_numpy(d["BT"]).cuda()
        self.C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        DT0 = torch.from_numpy(d["DT"].reshape(-1).copy()).cuda()
        self.cinfo = None
        if self.window == 64:
            self.cinfo = torch.empty(pkg.column_info_ints(self.W, self.kept, self.window, N, NS), dtype=torch.int32,
                                     device="cuda")
        self.D = torch.empty_like(DT0)
        DT = torch.empty_like(DT0)

        def preprocess():
            DT.copy_(DT0)
            pn, pm = n, m
            for _ in range(times):
                pn, pm = pkg.trans_index_device(DT, self.W, N, self.Q, pn, pm)
            if self.cinfo is None:
                pkg.preprocess_low_device(DT, self.D, self.W, self.Q, NS)
            else:
                pkg.preprocess_high_device(self.cinfo, pm, pn, DT, self.D, self.W, self.Q, N, NS)

        preprocess()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            preprocess()
        e1.record()
        torch.cuda.synchronize()
        self.preprocess_ms = e0.elapsed_time(e1) / 5
        # the same work by the one-kernel entry point (widening folded into the re-blocking pass)
        pkg.preprocess_device(DT0, n, m, self.W, self.Q, N, NS, self.D, self.cinfo)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(20):
            pkg.preprocess_device(DT0, n, m, self.W, self.Q, N, NS, self.D, self.cinfo)
        e1.record()
        torch.cuda.synchronize()
        self.preprocess_one_kernel_ms = e0.elapsed_time(e1) / 20

    def launch(self, pkg):
        pkg.spmm(self.A, self.B, self.D, self.cinfo, self.C, M, N, K, self.W, self.window, self.kept, 32, NS, 1, None)

    def useful_flops(self):
        return 2.0 * M * N * self.W


PREWARM_S = 1.0


def time_launches(torch, fn, steps, warmup, prewarm_s=None):
    """`warmup` untimed steps, then exactly `steps` timed ones.  Before both, the step is repeated
    for about prewarm_s seconds: an idle MI355X sits near 1 GHz and takes some hundred milliseconds of
    load to reach its sustained shader clock, far longer than a few sub-millisecond launches."""
    t_end = time.perf_counter() + (PREWARM_S if prewarm_s is None else prewarm_s)
    while time.perf_counter() < t_end:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return e0.elapsed_time(e1) / steps, wall_ms


def cpu_baseline(case, rows):
    """The reference's nmGEMM_on_cpu (compiled from the reference sources into oracle/_ref) on the
    first `rows` rows of the 2:4 workload; rows are independent, so rows/M of the job."""
    from oracle.nm_oracle import Oracle, Reference
    d = case.d
    if Reference.available():
        ref, kind = Reference(), "reference"
    else:
        ref, kind = None, "port"
    orc = Oracle()
    A_sub = np.ascontiguousarray(d["A_km"][:, :rows]).reshape(-1)
    B, D = d["B_cm"].reshape(-1), d["D_cm"].reshape(-1)
    # The reference prints its thread count with printf; keep stdout for the one JSON line.
    sys.stdout.flush()
    saved = os.dup(1)
    os.dup2(2, 1)
    try:
        t0 = time.perf_counter()
        if ref is not None:
            C = ref.gemm_cpu(A_sub, B, D, rows, N, K, case.W)
        else:
            C = orc.gemm_cpu(A_sub, B, D, rows, N, case.W)
        dt = time.perf_counter() - t0
        import ctypes
        ctypes.CDLL(None).fflush(None)
    finally:
        os.dup2(saved, 1)
        os.close(saved)
    return C.reshape(rows, N), {
        "value": 2.0 * rows * N * case.W / dt / 1e12, "unit": "TFLOP/s (useful)", "cores": orc.threads(), "kind": kind,
        "sample": "rows [0,%d) of the M=%d 2:4 workload (rows are independent), %.1f s wall" % (rows, M, dt),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-rows", type=int, default=4096, help="rows of the CPU baseline sample (0 = skip)")
    ap.add_argument("--headline-only", action="store_true", help="time only the 2:4 kernel (for profiling runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy 5 times (known traffic, to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library is a single-GPU kernel library; run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    pkg = importlib.import_module("nm-spmm_amd")
    datagen = importlib.import_module("nm-spmm_amd.datagen")
    if not os.path.exists(pkg.LIB_PATH):  # load what is built; build only when nothing is
        importlib.import_module("__graft_entry__").build()
    pkg.lib()  # fails loudly if the HIP library is still missing: there is no fallback
    torch.cuda.set_device(0)
    torch.backends.cuda.matmul.allow_tf32 = False

    sweep = {}
    head = None
    dense_ms = None
    for idx, (n, m) in enumerate(PATTERNS):
        if args.headline_only and idx > 0:
            break
        case = Case(torch, pkg, datagen, n, m, seed=2000 + 10 * n + m)
        ms, wall_ms = time_launches(torch, lambda: case.launch(pkg), args.steps, args.warmup)
        assert pkg.last_kernel() == "mfma"
        if idx == 0:
            head = (case, ms, wall_ms)
            if not args.headline_only:
                Amk = case.A.t().contiguous()
                Bd = torch.randn((K, N), dtype=torch.float32, device="cuda")
                Cd = torch.empty((M, N), dtype=torch.float32, device="cuda")
                dense_ms, _ = time_launches(torch, lambda: torch.mm(Amk, Bd, out=Cd), args.steps, args.warmup)
                del Amk, Bd, Cd
        useful = case.useful_flops() / (ms * 1e-3) / 1e12
        entry = {"ms": round(ms, 4), "useful_tflops": round(useful, 2),
                 "dense_equiv_tflops": round(2.0 * M * N * K / (ms * 1e-3) / 1e12, 2),
                 "frac_fp32_mfma_peak": round(useful / FP32_MFMA_PEAK_TFLOPS, 4),
                 "preprocess_ms": round(case.preprocess_ms, 4),
                 "preprocess_one_kernel_ms": round(case.preprocess_one_kernel_ms, 4)}
        if dense_ms is not None:
            entry["speedup_vs_dense"] = round(dense_ms / ms, 3)
            entry["speedup_over_ideal"] = round(dense_ms / ms / (m / n), 3)
        sweep["%d:%d" % (n, m)] = entry
        if idx > 0:
            del case

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    case, ms, wall_ms = head
    achieved = case.useful_flops() / (ms * 1e-3) / 1e12
    cpu = None
    if args.cpu_rows > 0:
        case.launch(pkg)
        torch.cuda.synchronize()
        got = case.C[:args.cpu_rows].cpu().numpy().astype(np.float64)
        want, cpu = cpu_baseline(case, args.cpu_rows)
        want = want.astype(np.float64)
        rms = np.sqrt(np.mean(want * want))
        cpu["gpu_vs_cpu_scaled_max_error"] = float(np.max(np.abs(got - want) / np.maximum(np.abs(want), rms)))

    out = {
        "metric": "useful fp32 TFLOP/s, M=Ncols=K=4096, 2:4 (vector length 32)",
        "value": round(achieved, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "clock_prewarm_s": PREWARM_S,
        "config": {"workload": "square sweep M=Ncols=K=4096 fp32, uniform(-1,1), seeded n:m patterns per 32-column "
                               "vector; value at 2:4, others under sweep", "tile": "Ns=128", "split_k": 1},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / FP32_MFMA_PEAK_TFLOPS, 4),
                     # bytes behind L2 per launch: rocprofv3 FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, the
                     # factors coming from a plain 256 MiB copy in the same runs
                     # (profiles/spmm_direct_kernel_4096cubed_2of4.md)
                     "traffic": 411.2e6, "traffic_unit": "bytes per launch", "algorithmic_bytes": 168.8e6,
                     "kernel": "spmm_direct_kernel<32,16,4,1,8,false>", "flops_per_launch": case.useful_flops(),
                     "launch_ms_events": round(ms, 5), "launch_ms_wall": round(wall_ms, 5)},
        "cpu_baseline": cpu,
        "dense_fp32_gemm": None if dense_ms is None else {
            "ms": round(dense_ms, 4), "tflops": round(2.0 * M * N * K / (dense_ms * 1e-3) / 1e12, 2),
            "library": "torch.mm fp32 (rocBLAS/hipBLASLt)"},
        "sweep": sweep,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
