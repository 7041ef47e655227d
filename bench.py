#!/usr/bin/env python3
"""Benchmark of the N:M sparse x dense fp32 multiplication on one MI355X.

One "step" is one launch of the hot path (nmspmm_spmm through the C-ABI) on the square sweep of
the baseline: M = Ncols = K = 4096, fp32, operands resident in HBM, at 2:4 (the headline value).
Prints ONE JSON line; its parts:

  value            useful TFLOP/s at 2:4 = 2*M*Ncols*W / t   (W = K*n/m)
  roofline         the dominant kernel (the tile kernel at 2:4) against the fp32 MFMA peak
  cpu_baseline     the reference project's own nmGEMM_on_cpu (oracle/_ref) on a row slice
  sweep            3:8, 2:8, 1:8 beside 2:4: ms, useful TFLOP/s, speedup over the dense fp32 GEMM
  configs          the baseline's other workloads, each timed in this run:
                     llm     nine prefill-sized LLM-layer shapes at 2:8 against the dense fp32 GEMM,
                             with B re-read from the caches and with B streamed from HBM
                     ragged  nine shapes whose tiles do not fill whole rounds of the compute
                             units, one per way the library cuts the leftovers
                     decode  M in {1, 8, 16, 32} x two weight shapes x {1:8, 2:8}: microseconds and
                             algorithmic GB/s against the 8 TB/s HBM bound, with B re-read from the
                             caches ("hot") and streamed from HBM ("cold"), row list on and off
                     decode_llm, decode_wide: decode sizes of the LLM-layer weight shapes with and
                             without cut reductions; 48 and 64 rows on the row list
                     fine    4:32, 8:32, 16:32 and 2:4 with 4-column vectors at 4096 cubed
                     launch_constant, compress, rowmajor: the part of a launch that does not scale
                             with K; dense <-> compressed conversion; row-major activations
                     sweep100  the 100 shapes x 4 sparsities of the reference's kernel-performance
                             sweep against the dense fp32 GEMM
  preprocess       index preprocessing: one-kernel device call, the reference's call sequence on
                   the device, the host-pointer drop-in calls (wall time, PCIe included), and the
                   CPU restatement / the reference's own host code
  dispatch         the library's split / kernel choice against the best of the splits 1, 2, 4, 8

The printed line holds the headline fields whole and one digest per other workload (it stays under
4 KB); every case of every part goes to the detail file (--detail, default bench_detail.json).

Timing uses HIP events on the stream the kernels are launched on (torch's current stream is the
one handed to the C-ABI); decode-sized launches are replayed from a HIP graph so that the host's
launch rate does not enter.  --only selects parts (for profiling runs); the default runs all.
"""
import argparse
import importlib
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
M = N = K = 4096
PATTERNS = [(2, 4), (3, 8), (2, 8), (1, 8)]  # first one is the headline
NS = 128
GEOMETRY = {(1, 1): (32, 32), (1, 2): (32, 16), (3, 8): (32, 12), (1, 4): (64, 16), (1, 8): (64, 8)}
PARTS = ("sweep", "llm", "ragged", "decode", "decode_llm", "decode_wide", "fine", "ksweep", "compress", "rowmajor", "preprocess", "dispatch", "cpu", "sweep100")
OPT_IN_PARTS = ()   # parts that only run when named


def geometry(n, m):
    """(window, kept, transIndex doublings) the kernels run an n:m pattern at."""
    from math import gcd
    g = gcd(n, m)
    window, kept = GEOMETRY[(n // g, m // g)]
    times, mm = 0, m
    while mm < window:
        mm, times = mm * 2, times + 1
    return window, kept, times


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


def time_graph(torch, calls, replays=6, prewarm_s=0.15):
    """Milliseconds per call of a HIP graph that holds the calls back to back, best of `replays`
    (each replay is one event pair around the whole graph)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls[0]()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for c in calls:
            c()
    t_end = time.perf_counter() + prewarm_s
    while time.perf_counter() < t_end:
        graph.replay()
        torch.cuda.synchronize()
    best = 1e9
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / len(calls))
    del graph
    return best


class Case:
    """Operands of one square-sweep pattern from the seeded host generator (the CPU baseline needs
    the host arrays), resident on the GPU, preprocessed by the GPU kernels."""

    def __init__(self, torch, pkg, datagen, n, m, seed):
        d = datagen.init_data(M, N, K, n, m, seed=seed)
        self.d, self.n, self.m = d, n, m
        self.W, self.Q = d["W"], d["Q"]
        self.window, self.kept, _ = geometry(n, m)
        self.A = torch.from_numpy(d["A_km"]).cuda()
        self.B = torch.from_numpy(d["BT"]).cuda()
        self.C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        DT0 = torch.from_numpy(d["DT"].reshape(-1).copy()).cuda()
        self.cinfo = None
        if self.window == 64:
            self.cinfo = torch.empty(pkg.column_info_ints(self.W, self.kept, self.window, N, NS), dtype=torch.int32,
                                     device="cuda")
        self.D = torch.empty_like(DT0)
        pkg.preprocess_device(DT0, n, m, self.W, self.Q, N, NS, self.D, self.cinfo)
        torch.cuda.synchronize()

    def launch(self, pkg):
        pkg.spmm(self.A, self.B, self.D, self.cinfo, self.C, M, N, K, self.W, self.window, self.kept, 32, NS, 1, None)

    def useful_flops(self):
        return 2.0 * M * N * self.W


class GpuOperands:
    """Synthetic operands drawn on the GPU (values and per-vector patterns), preprocessed on the
    GPU: for the workloads whose results are checked by the test-suite, not here."""

    def __init__(self, torch, pkg, m_rows, n_cols, k, n, m, vec_len=32, normal=True, row_list=False):
        self.M, self.N, self.K, self.n, self.m, self.vl = m_rows, n_cols, k, n, m, vec_len
        self.W, self.Q = k // m * n, n_cols // vec_len
        scale = 0.02 if normal else 1.0
        if normal:
            self.A = torch.randn((k, m_rows), dtype=torch.float32, device="cuda")
            self.B = torch.randn((self.W, n_cols), dtype=torch.float32, device="cuda") * scale
        else:
            self.A = torch.rand((k, m_rows), dtype=torch.float32, device="cuda") * 2 - 1
            self.B = torch.rand((self.W, n_cols), dtype=torch.float32, device="cuda") * 2 - 1
        self.C = torch.zeros((m_rows, n_cols), dtype=torch.float32, device="cuda")
        pick = torch.rand((k // m, self.Q, m), device="cuda").argsort(dim=2)[:, :, :n].sort(dim=2).values
        self.DT = pick.permute(0, 2, 1).reshape(self.W, self.Q).to(torch.int32).contiguous()
        del pick
        self.D = torch.empty_like(self.DT)
        self.cinfo = None
        if vec_len == 32:
            self.window, self.kept, _ = geometry(n, m)
            if self.window == 64:
                self.cinfo = torch.empty(pkg.column_info_ints(self.W, self.kept, self.window, n_cols, NS),
                                         dtype=torch.int32, device="cuda")
            pkg.preprocess_device(self.DT, n, m, self.W, self.Q, n_cols, NS, self.D, self.cinfo)
        else:
            self.window, self.kept = m, n
            pkg.preprocess_low_device(self.DT, self.D, self.W, self.Q, NS, vec_len)
        self.R = None
        if row_list:
            self.R = torch.empty(pkg.row_index_ints(self.W, n_cols), dtype=torch.int32, device="cuda")
            pkg.row_index_device(self.D, self.cinfo, self.W, n_cols, self.window, self.kept, NS, self.R)
        torch.cuda.synchronize()

    def flops(self):
        return 2.0 * self.M * self.N * self.W

    def algorithmic_bytes(self):
        b = 4.0 * (self.M * self.K + self.W * self.N + self.W * self.N / self.vl + self.M * self.N)
        if self.cinfo is not None:
            b += 4.0 * self.cinfo.numel()
        return b


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
    with stdout_to_stderr():  # the reference prints its thread count with printf
        t0 = time.perf_counter()
        if ref is not None:
            C = ref.gemm_cpu(A_sub, B, D, rows, N, K, case.W)
        else:
            C = orc.gemm_cpu(A_sub, B, D, rows, N, case.W)
        dt = time.perf_counter() - t0
    return C.reshape(rows, N), {
        "value": 2.0 * rows * N * case.W / dt / 1e12, "unit": "TFLOP/s (useful)", "cores": orc.threads(), "kind": kind,
        "sample": "rows [0,%d) of the M=%d 2:4 workload (rows are independent), %.1f s wall" % (rows, M, dt),
    }


class stdout_to_stderr:
    """Keeps stdout for the one JSON line while C code that prints runs."""

    def __enter__(self):
        sys.stdout.flush()
        self.saved = os.dup(1)
        os.dup2(2, 1)

    def __exit__(self, *exc):
        import ctypes
        ctypes.CDLL(None).fflush(None)
        os.dup2(self.saved, 1)
        os.close(self.saved)


def tile_kernel_name(pkg, case):
    rows = pkg.tile_wave_rows(M, N, case.W, case.kept, NS, 1)
    if rows == 0:
        return "spmm_direct_inner_kernel (waves along K, %d rows)" % pkg.waves_along_k_rows(M, N, case.W, case.kept)
    qs = NS // 32
    high = "true" if case.cinfo is not None else "false"
    if pkg.tile_wave_sets(M, N, case.W, case.kept, NS, 1) == 2:
        return "spmm_direct_halves_kernel<%d,%d,%d,%d,%s>" % (case.window, case.kept, qs, 4 // qs, high)
    return "spmm_direct_kernel<%d,%d,%d,%d,%d,%s>" % (case.window, case.kept, qs, 4 // qs, rows // 32, high)


def profiled_traffic():
    """HBM-side bytes per launch of the headline kernel, from the tracked rocprofv3 counter summary
    (FETCH_SIZE and WRITE_SIZE scaled by a plain copy); None when the file does not hold it."""
    path = os.path.join(ROOT, "profiles", "spmm_direct_kernel_4096cubed_2of4.md")
    try:
        m = re.search(r"traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read())
    except OSError:
        return None, None
    return (float(m.group(1)), os.path.relpath(path, ROOT)) if m else (None, None)


def time_b_from_hbm(torch, B, call):
    """Milliseconds per call(b) with every launch on another copy of B, more than 640 MB in all:
    every byte of B then comes from HBM, as in a model whose layers do not fit the caches."""
    copies = [B] + [B.clone() for _ in range(int(640e6 // (B.numel() * 4)))]
    turn = [0]

    def step():
        turn[0] = (turn[0] + 1) % len(copies)
        call(copies[turn[0]])

    ms, _ = time_launches(torch, step, 3 * len(copies), len(copies), 0.1)
    return ms


def rate_entry(us, nbytes, from_hbm, digits):
    """Microseconds and algorithmic GB/s of one launch.  Only a launch whose operands come from HBM
    is set against the HBM peak; one that re-reads what the previous launch left in the 256 MB
    Infinity Cache is labelled so and carries no fraction."""
    gbs = nbytes / us / 1e3
    e = {"us": round(us, digits), "gbs": round(gbs, 0)}
    if from_hbm:
        e["frac_hbm"] = round(gbs / HBM_PEAK_GBS, 3)
    else:
        e["served_by"] = "infinity cache"
    return e


def run_llm(torch, pkg):
    """Config 3: nine prefill-sized layer shapes at 2:8, the library's own split, against torch.mm fp32."""
    rows = []
    for (k, n_cols) in ((4096, 4096), (4096, 11008), (11008, 4096)):
        for m_rows in (512, 2048, 8192):
            op = GpuOperands(torch, pkg, m_rows, n_cols, k, 2, 8)
            split = pkg.suggest_split_k(m_rows, n_cols, op.W, op.kept)
            ms, _ = time_launches(torch, lambda: pkg.gemm_auto(op.A, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k,
                                                               op.W, 0.75), 30, 5, 0.2)
            fam = pkg.last_kernel()
            cold_ms = time_b_from_hbm(torch, op.B, lambda b: pkg.gemm_auto(op.A, b, op.D, op.cinfo, op.C, m_rows, n_cols, k,
                                                                           op.W, 0.75))
            a = op.A.t().contiguous()
            b = torch.randn((k, n_cols), dtype=torch.float32, device="cuda")
            dms, _ = time_launches(torch, lambda: torch.mm(a, b, out=op.C), 20, 3, 0.2)
            useful = op.flops() / ms / 1e9
            rows.append({"M": m_rows, "K": k, "Ncols": n_cols, "pattern": "2:8", "kernel": fam, "split_k": split,
                         "waves_along_k_rows": pkg.waves_along_k_rows(m_rows, n_cols, op.W, op.kept),
                         "ms": round(ms, 4), "ms_b_from_hbm": round(cold_ms, 4), "useful_tflops": round(useful, 1),
                         "frac_fp32_mfma_peak": round(useful / FP32_MFMA_PEAK_TFLOPS, 3),
                         "dense_ms": round(dms, 4), "speedup_vs_dense": round(dms / ms, 2),
                         "speedup_over_ideal": round(dms / ms / 4.0, 3)})
            del op, a, b
    return rows


# Shapes whose tile counts do not fill whole rounds of the 256 compute units, one per way the tile
# kernel cuts the leftovers: (M, Ncols, K, n, m, what the launch is)
RAGGED_SHAPES = (
    (768, 4096, 14336, 2, 8, "192 tiles of 128 x 128: waves along K, three layers of 128-row workgroups on eight waves"),
    (640, 4096, 8192, 2, 4, "160 tiles: waves along K, five layers of 64-row workgroups on eight waves"),
    (2048, 4096, 8192, 2, 4, "256 tiles of 256 x 128, one per compute unit: two sets of waves per workgroup"),
    (1024, 4352, 4096, 2, 8, "272 tiles of 128 rows: the last 16 as eight workgroups each in the same launch"),
    (1024, 8704, 4096, 1, 8, "544 tiles of 128 rows, two whole layers: the last 32 as eight workgroups each"),
    (4096, 4224, 4096, 2, 8, "528 tiles of 256 rows: the 16 beyond one round as sixteen workgroups each, in a launch of their own"),
    (1152, 14848, 4096, 3, 8, "1044 tiles of 128 rows: the 20 beyond one round as eight workgroups each at the end of the launch"),
    (2048, 11008, 4096, 2, 4, "688 tiles of 256 rows: the 176 beyond one round as 64-row pieces in a launch of their own"),
    (160, 4096, 11008, 3, 8, "160 rows: 128 on the tile kernel (waves along K), the last 32 on the kernel with one workgroup per vector"),
)


def run_ragged(torch, pkg):
    """Unsplit multiplications of shapes with leftover tiles; `of_even` compares the useful rate with
    the headline shape's (4096 cubed at the same pattern is not timed here: the fraction of the fp32
    MFMA peak is the common scale)."""
    rows = []
    for (m_rows, n_cols, k, n, m, what) in RAGGED_SHAPES:
        op = GpuOperands(torch, pkg, m_rows, n_cols, k, n, m)
        call = lambda: pkg.spmm(op.A, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W, op.window, op.kept, 32, NS, 1, None)
        ms, _ = time_launches(torch, call, 30, 5, 0.2)
        cold_ms = time_b_from_hbm(torch, op.B, lambda b: pkg.spmm(op.A, b, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W,
                                                                  op.window, op.kept, 32, NS, 1, None))
        useful = op.flops() / ms / 1e9
        rows.append({"M": m_rows, "K": k, "Ncols": n_cols, "pattern": "%d:%d" % (n, m), "kernel": pkg.last_kernel(),
                     "launch": what, "rows_apart": pkg.rows_apart(m_rows, n_cols, op.W, op.kept),
                     "tile_wave_rows": pkg.tile_wave_rows(m_rows, n_cols, op.W, op.kept, NS, 1),
                     "tile_wave_sets": pkg.tile_wave_sets(m_rows, n_cols, op.W, op.kept, NS, 1),
                     "waves_along_k": [pkg.waves_along_k_rows(m_rows, n_cols, op.W, op.kept),
                                       pkg.waves_along_k_count(m_rows, n_cols, op.W, op.kept)],
                     "ms": round(ms, 4), "ms_b_from_hbm": round(cold_ms, 4), "useful_tflops": round(useful, 1),
                     "frac_fp32_mfma_peak": round(useful / FP32_MFMA_PEAK_TFLOPS, 3)})
        del op
    return rows


DECODE_MODES = (("hot", 0, True, False), ("cold", 0, True, True), ("cold_stream_hint", 2, True, True),
                ("hot_reference_layout", 0, False, False), ("cold_reference_layout", 0, False, True),
                ("hot_split", 4, True, False), ("cold_split", 4, True, True))
DECODE_DEFAULT_MODES = tuple(m[0] for m in DECODE_MODES[:5])
# the decode sizes of the LLM-layer shapes (config 3's K x Ncols): fewer column vectors than compute
# units, where NMSPMM_DECODE_SPLIT lets the kernel cut the reductions across workgroups
DECODE_LLM_SHAPES = ((4096, 4096), (11008, 4096), (4096, 11008))
DECODE_LLM_MODES = ("hot", "cold", "hot_split", "cold_split")


def run_decode(torch, pkg, rows_list=(1, 8, 16, 32), shapes=((8192, 8192), (4096, 14336)), patterns=((1, 8), (2, 8)),
               modes=DECODE_DEFAULT_MODES):
    """Config 4.  Per case: the decode kernel on the row list and the kernel on the reference-layout
    indices, with one B re-read by every launch (it then sits in the 256 MB Infinity Cache: "hot")
    and with launches that walk through copies of B adding up to more than 600 MB ("cold": every
    byte of B comes from HBM, as in a model whose layers do not fit the cache), the latter also
    with the non-temporal hint."""
    out = []
    for (k, n_cols) in shapes:
        for (n, m) in patterns:
            op = GpuOperands(torch, pkg, max(rows_list), n_cols, k, n, m, row_list=True)
            b_bytes = op.B.numel() * 4
            copies = [op.B] + [op.B.clone() for _ in range(int(640e6 // b_bytes))]
            for m_rows in rows_list:
                a = op.A[:, :m_rows].contiguous()
                c = torch.empty((m_rows, n_cols), dtype=torch.float32, device="cuda")
                op.M = m_rows

                def call(b, flags, rl):
                    return lambda: pkg.spmm_ex(a, b, op.D, op.cinfo, c, m_rows, n_cols, k, op.W, op.window, op.kept, 32,
                                               NS, 1, None, flags, op.R if rl else None)

                alg = op.algorithmic_bytes()
                # the launch can be no shorter than its bytes at the HBM rate or its flops at the
                # fp32 matrix-core peak, whichever is longer (the latter from about 48 rows on)
                floor_us = max(alg / (HBM_PEAK_GBS * 1e3), 2.0 * m_rows * n_cols * op.W / (FP32_MFMA_PEAK_TFLOPS * 1e6))
                entry = {"M": m_rows, "K": k, "Ncols": n_cols, "pattern": "%d:%d" % (n, m),
                         "algorithmic_bytes": int(alg), "roofline_us": round(floor_us, 2)}
                for label, flags, rl, cold in DECODE_MODES:
                    if label not in modes:
                        continue
                    calls = [call(b, flags, rl) for b in (copies if cold else [op.B] * 20)]
                    ms = time_graph(torch, calls)
                    if label == "hot":
                        entry["kernel"] = pkg.last_kernel()
                    elif label == "hot_reference_layout":
                        entry["kernel_reference_layout"] = pkg.last_kernel()
                    entry[label] = rate_entry(ms * 1e3, alg, cold, 2)
                out.append(entry)
                del a, c
            del op, copies
    return out


def run_fine(torch, pkg, cases):
    """Config 5: the n:32 patterns and 2:4 with 4-column vectors at 4096 cubed, with the device
    preprocessing time of each (one launch for 32-column vectors, the re-blocking launch for
    shorter ones); beyond the baseline's list, 2:8 and 1:8 with 4-column vectors, 1:8 with
    8-column ones, and the dense pattern 32:32 (the reference's geometry for a sparsity of 0)."""
    out = []
    for (n, m, vl) in cases:
        op = GpuOperands(torch, pkg, M, N, K, n, m, vec_len=vl, normal=False)
        ms, _ = time_launches(torch, lambda: pkg.spmm(op.A, op.B, op.D, op.cinfo, op.C, M, N, K, op.W, op.window,
                                                      op.kept, vl, NS, 1, None), 20, 3, 0.3)
        fam = pkg.last_kernel()
        if vl == 32:
            pre = lambda: pkg.preprocess_device(op.DT, n, m, op.W, op.Q, N, NS, op.D, op.cinfo)
        else:
            pre = lambda: pkg.preprocess_low_device(op.DT, op.D, op.W, op.Q, NS, vl)
        pre_ms, _ = time_launches(torch, pre, 20, 3, 0.05)
        useful = op.flops() / ms / 1e9
        out.append({"pattern": "%d:%d" % (n, m), "vec_len": vl, "kernel": fam, "ms": round(ms, 4),
                    "useful_tflops": round(useful, 1), "frac_fp32_mfma_peak": round(useful / FP32_MFMA_PEAK_TFLOPS, 3),
                    "preprocess_device_ms": round(pre_ms, 4), "index_bytes": int(op.D.numel() * 4)})
        del op
    return out


def run_ksweep(torch, pkg, ks=(64, 1024, 4096), patterns=((2, 4), (1, 8), (4, 32))):
    """M = Ncols = 4096 at three reduction lengths: separates the part of a launch that does not
    scale with K (the gap between launches, the first loads, the 64 MiB store of C) from the rate."""
    out = []
    for (n, m) in patterns:
        pts = []
        for k in ks:
            op = GpuOperands(torch, pkg, M, N, k, n, m, normal=False)
            ms, _ = time_launches(torch, lambda: pkg.spmm(op.A, op.B, op.D, op.cinfo, op.C, M, N, k, op.W, op.window,
                                                          op.kept, 32, NS, 1, None), 50, 5, 0.3)
            pts.append((k, ms, op.flops()))
            del op
        row = {"pattern": "%d:%d" % (n, m), "ms_at_K": {str(k): round(ms, 4) for (k, ms, _) in pts}}
        if len(pts) >= 2:
            (k1, t1, f1), (k2, t2, f2) = pts[-2], pts[-1]
            rate = (f2 - f1) / ((t2 - t1) * 1e-3) / 1e12        # TFLOP/s between the two longest reductions
            row["rate_tflops"] = round(rate, 1)
            row["constant_us"] = round((t2 * 1e-3 - f2 / (rate * 1e12)) * 1e6, 1)  # what is left at K -> 0
        out.append(row)
    return out


def run_compress(torch, pkg):
    """Dense B -> (values, indices) and back (nmspmm_compress_device / nmspmm_decompress_device):
    microseconds and algorithmic GB/s, 4*(K*Ncols + W*Ncols + W*Ncols/32) bytes either way."""
    out = []
    for (k, n_cols) in ((4096, 4096), (11008, 4096), (8192, 8192)):
        dense = torch.randn((k, n_cols), dtype=torch.float32, device="cuda")
        # the yardstick: a plain device-to-device copy of the dense operand (reads and writes it
        # once), cold in the same way; what fraction of 8 TB/s a kernel that only moves bytes gets
        pairs = [(dense, torch.empty_like(dense))]
        while len(pairs) * 2 * dense.numel() * 4 < 640e6 + 2 * dense.numel() * 4:
            pairs.append((dense.clone(), torch.empty_like(dense)))
        turn = [0]

        def copy_step():
            turn[0] = (turn[0] + 1) % len(pairs)
            pairs[turn[0]][1].copy_(pairs[turn[0]][0])

        cms, _ = time_launches(torch, copy_step, 3 * len(pairs), len(pairs), 0.05)
        copy = rate_entry(cms * 1e3, 2.0 * dense.numel() * 4, True, 1)
        del pairs
        for (n, m) in ((2, 4), (2, 8), (1, 8), (8, 32)):
            w, q = k // m * n, n_cols // 32
            bt = torch.empty((w, n_cols), dtype=torch.float32, device="cuda")
            dt = torch.empty((w, q), dtype=torch.int32, device="cuda")
            back = torch.empty_like(dense)
            nbytes = 4.0 * (k * n_cols + w * n_cols + w * q)
            row = {"K": k, "Ncols": n_cols, "pattern": "%d:%d" % (n, m), "plain_copy_of_the_dense_operand": copy}
            for name, fn in (("compress", lambda: pkg.compress_device(dense, k, n_cols, n, m, bt, dt)),
                             ("decompress", lambda: pkg.decompress_device(bt, dt, k, n_cols, n, m, back))):
                ms, _ = time_launches(torch, fn, 30, 5, 0.05)
                row[name + "_hot"] = rate_entry(ms * 1e3, nbytes, False, 1)
            # cold: every launch on another set of buffers, more than 640 MB touched between two
            # uses of the same one, so that neither the input nor the output sits in a cache
            sets = [(dense, bt, dt, back)]
            for _ in range(int(640e6 // nbytes) + 1):
                sets.append(tuple(t.clone() for t in sets[0]))
            turn = [0]

            def step(which):
                turn[0] = (turn[0] + 1) % len(sets)
                de, b_, d_, ba = sets[turn[0]]
                if which == "compress":
                    pkg.compress_device(de, k, n_cols, n, m, b_, d_)
                else:
                    pkg.decompress_device(b_, d_, k, n_cols, n, m, ba)

            for name in ("compress", "decompress"):
                ms, _ = time_launches(torch, lambda: step(name), 3 * len(sets), len(sets), 0.05)
                row[name] = rate_entry(ms * 1e3, nbytes, True, 1)
            out.append(row)
            del bt, dt, back, sets
        del dense
    return out


def run_rowmajor(torch, pkg):
    """Row-major activations (nmspmm_spmm_rowmajor): the transpose into the workspace, the
    multiplication alone, and both, on the LLM-layer shapes at 2:8 and at decode sizes."""
    out = []
    for (m_rows, k, n_cols) in ((512, 4096, 4096), (2048, 4096, 11008), (8192, 11008, 4096), (8, 8192, 8192),
                                (32, 8192, 8192)):
        op = GpuOperands(torch, pkg, m_rows, n_cols, k, 2, 8)
        a_rm = op.A.t().contiguous()
        split = pkg.suggest_split_k(m_rows, n_cols, op.W, op.kept)
        ws = torch.empty(max(pkg.workspace_bytes_rowmajor(m_rows, n_cols, k, split) // 4, 4), dtype=torch.float32,
                         device="cuda")
        ws_cm = torch.empty(max(pkg.workspace_bytes(m_rows, n_cols, split) // 4, 4), dtype=torch.float32, device="cuda")
        t_mm = time_graph(torch, [lambda: pkg.spmm(op.A, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W, op.window,
                                                  op.kept, 32, NS, split, ws_cm if split > 1 else None)] * 10, 4, 0.1)
        t_both = time_graph(torch, [lambda: pkg.spmm_rowmajor(a_rm, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W,
                                                              op.window, op.kept, ws, 32, NS, split)] * 10, 4, 0.1)
        out.append({"M": m_rows, "K": k, "Ncols": n_cols, "pattern": "2:8", "split_k": split,
                    "column_major_ms": round(t_mm, 4), "row_major_ms": round(t_both, 4),
                    "overhead": round(t_both / t_mm - 1.0, 3)})
        del op, a_rm, ws, ws_cm
    return out


def run_preprocess(torch, pkg, datagen):
    """Index preprocessing of the 4096 cubed patterns four ways: (i) the one-kernel device entry,
    (ii) the reference's call sequence (transIndex x t, then PreProcessing_*) on device-resident
    indices, (iii) the same sequence through the host-pointer drop-in calls (wall time: each call
    stages the indices through the GPU, PCIe both ways), (iv) on the CPU: the restatement, and the
    reference's own host code where oracle/_ref is built."""
    from oracle.nm_oracle import Oracle, Reference
    orc = Oracle()
    ref = Reference() if Reference.available() else None
    out = []
    for (n, m, vl) in ((2, 4, 32), (1, 8, 32), (8, 32, 32), (2, 4, 4)):
        d = datagen.init_data(4, N, K, n, m, vec_len=vl, seed=77 + n + vl)
        W, Q = d["W"], d["Q"]
        if vl == 32:
            window, kept, times = geometry(n, m)
        else:
            window, kept, times = m, n, 0
        high = window == 64
        DT0 = torch.from_numpy(d["DT"].reshape(-1).copy()).cuda()
        DT, D = torch.empty_like(DT0), torch.empty_like(DT0)
        cinfo = torch.empty(max(pkg.column_info_ints(W, kept, window, N, NS), 1), dtype=torch.int32, device="cuda")
        entry = {"pattern": "%d:%d" % (n, m), "vec_len": vl, "index_bytes": int(DT0.numel() * 4)}

        def sequence_device():
            DT.copy_(DT0)
            pn, pm = n, m
            for _ in range(times):
                pn, pm = pkg.trans_index_device(DT, W, N, Q, pn, pm)
            if high:
                pkg.preprocess_high_device(cinfo, pm, pn, DT, D, W, Q, N, NS, vl)
            else:
                pkg.preprocess_low_device(DT, D, W, Q, NS, vl)

        ms, _ = time_launches(torch, lambda: pkg.preprocess_device(DT0, n, m, W, Q, N, NS, D, cinfo if high else None),
                              20, 3, 0.05)
        entry["device_one_kernel_ms"] = round(ms, 4)
        ms, _ = time_launches(torch, sequence_device, 10, 2, 0.05)
        entry["device_reference_sequence_ms"] = round(ms, 4)

        def sequence(tr, low, hi):
            host = d["DT"].reshape(-1).copy()
            ci = np.empty(max(pkg.column_info_ints(W, kept, window, N, NS), 1) + window, np.int32)
            t0 = time.perf_counter()
            pn, pm = n, m
            for _ in range(times):
                pn, pm = tr(host, pn, pm)
            if high:
                hi(ci, pm, pn, host)
            else:
                low(host)
            return (time.perf_counter() - t0) * 1e3

        host_ms = min(sequence(lambda h, pn, pm: pkg.trans_index_host(h, W, N, Q, pn, pm),
                               lambda h: pkg.preprocess_low_host(h, W, Q, NS, vl),
                               lambda ci, pm, pn, h: pkg.preprocess_high_host(ci, pm, pn, h, W, Q, N, NS, vl))
                      for _ in range(3))
        entry["host_pointer_dropin_wall_ms"] = round(host_ms, 3)
        cpu_ms = min(sequence(lambda h, pn, pm: orc.trans_index(h, W, Q, pn, pm),
                              lambda h: orc.preprocess_low(h, W, Q, NS, vl),
                              lambda ci, pm, pn, h: orc.preprocess_high(pm, pn, h, W, Q, NS, vl))
                     for _ in range(2))
        entry["cpu_restatement_wall_ms"] = round(cpu_ms, 3)
        if ref is not None and vl == 32:
            with stdout_to_stderr():
                ref_ms = min(sequence(lambda h, pn, pm: ref.trans_index(h, W, N, Q, pn, pm),
                                      lambda h: ref.preprocess_low(h, W, Q, NS),
                                      lambda ci, pm, pn, h: ref.preprocess_high(pm, pn, h, W, Q, N, NS))
                             for _ in range(2))
            entry["cpu_reference_wall_ms"] = round(ref_ms, 3)
        out.append(entry)
        del DT0, DT, D, cinfo
    return out


# The reference's kernel-performance sweep (benchmark/kernel_performance/run_test/nmspmm/run_nmspmm.sh:16-18):
# five row counts x twenty (Ncols, K) pairs, at the n:32 patterns of its four sparsities (:29)
SWEEP100_M = (256, 512, 1024, 2048, 4096)
SWEEP100_N = (2048, 6144, 2048, 5632, 4096, 12288, 4096, 11008, 5120, 15360, 5120, 13824, 6656, 19968, 6656, 17920, 8192,
              24576, 8192, 22016)
SWEEP100_K = (2048, 2048, 5632, 2048, 4096, 4096, 11008, 4096, 5120, 5120, 13824, 5120, 6656, 6656, 17920, 6656, 8192,
              8192, 22016, 8192)
# mean speed-up over cuBLAS fp32 on the A100 over the same 100 shapes, from the reference's
# benchmark/kernel_performance/result_data/{nmspmm_a100_*,cublas_a100}.txt
SWEEP100_A100_MEAN = {"0.5": 1.83, "0.625": 2.38, "0.75": 3.46, "0.875": 6.34}


def run_sweep100(torch, pkg):
    """The 100 shapes of the reference's sweep at 50, 62.5, 75 and 87.5 % (16:32, 12:32, 8:32, 4:32):
    the library's own choice of kernel and split (the reference takes the best of four tiles and
    four splits by brute force, run_nmspmm.sh:19-36) against torch.mm fp32 of the same shape.  Line
    20*mi + i of each list is M[mi] with (Ncols, K)[i], as in the reference's result files.  Both
    sides are replayed from a HIP graph of five launches: the smallest shapes last about ten
    microseconds, less than a launch from Python."""
    by = {}
    dense_ms = []
    for m_rows in SWEEP100_M:
        for n_cols, k in zip(SWEEP100_N, SWEEP100_K):
            a = torch.randn((m_rows, k), dtype=torch.float32, device="cuda")
            b = torch.randn((k, n_cols), dtype=torch.float32, device="cuda")
            c = torch.empty((m_rows, n_cols), dtype=torch.float32, device="cuda")
            dense_ms.append(time_graph(torch, [lambda: torch.mm(a, b, out=c)] * 5, 3, 0.05))
            del a, b, c
    for kept, label in ((16, "0.5"), (12, "0.625"), (8, "0.75"), (4, "0.875")):
        rows, idx = [], 0
        for m_rows in SWEEP100_M:
            for n_cols, k in zip(SWEEP100_N, SWEEP100_K):
                op = GpuOperands(torch, pkg, m_rows, n_cols, k, kept, 32, normal=False)
                ms = time_graph(torch, [lambda: pkg.gemm_auto(op.A, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W,
                                                              float(label))] * 5, 3, 0.05)
                rows.append({"M": m_rows, "Ncols": n_cols, "K": k, "ms": round(ms, 4), "dense_ms": round(dense_ms[idx], 4),
                             "dense_equiv_tflops": round(2.0 * m_rows * n_cols * k / ms / 1e9, 2),
                             "speedup_vs_dense": round(dense_ms[idx] / ms, 3)})
                idx += 1
                del op
        sp = [r["speedup_vs_dense"] for r in rows]
        by[label] = {"pattern": "%d:32" % kept, "shapes": len(rows), "mean_speedup_vs_dense": round(float(np.mean(sp)), 3),
                     "min_speedup_vs_dense": min(sp), "max_speedup_vs_dense": max(sp),
                     "a100_reference_mean_speedup": SWEEP100_A100_MEAN[label], "rows": rows}
    return {"dense": "torch.mm fp32 (rocBLAS/hipBLASLt)", "by_sparsity": by}


def run_dispatch(torch, pkg):
    """The library's own choice (nmspmm_gemm_auto: split from its run-time model, kernel from the
    shape) against the best of the splits 1, 2, 4, 8 of nmspmm_spmm, on shapes from the reference's
    search grid (benchmark/different_kernel/search_shape/search_shape.sh:16-43) and LLM layers.
    Both sides are replayed from a HIP graph of ten launches: several of these problems last about
    ten microseconds, less than a launch from Python."""
    shapes = [(128, 4096, 4096, 2, 4), (256, 2048, 2048, 2, 8), (256, 4096, 4096, 1, 8), (512, 4096, 4096, 2, 8),
              (512, 1024, 1024, 2, 4), (1024, 4096, 4096, 3, 8), (1024, 5120, 5120, 2, 4), (2048, 4096, 11008, 2, 8),
              (160, 4096, 11008, 3, 8), (768, 4096, 14336, 2, 8), (4096, 4096, 4096, 1, 8), (2048, 11008, 4096, 2, 8)]
    rows, ratios = [], []
    for (m_rows, n_cols, k, n, m) in shapes:
        op = GpuOperands(torch, pkg, m_rows, n_cols, k, n, m, normal=False)
        best = (1e9, 0)
        for split in (1, 2, 4, 8):
            if split > op.W // op.kept:
                continue
            ws = None if split == 1 else torch.empty(pkg.workspace_bytes(m_rows, n_cols, split) // 4,
                                                     dtype=torch.float32, device="cuda")
            ms = time_graph(torch, [lambda: pkg.spmm(op.A, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W,
                                                     op.window, op.kept, 32, NS, split, ws)] * 10, 4, 0.1)
            best = min(best, (ms, split))
            del ws
        sparsity = 1.0 - n / m
        ms = time_graph(torch, [lambda: pkg.gemm_auto(op.A, op.B, op.D, op.cinfo, op.C, m_rows, n_cols, k, op.W,
                                                      sparsity)] * 10, 4, 0.1)
        ratio = ms / best[0]
        ratios.append(ratio)
        rows.append({"M": m_rows, "Ncols": n_cols, "K": k, "pattern": "%d:%d" % (n, m),
                     "library_split": pkg.suggest_split_k(m_rows, n_cols, op.W, op.kept), "library_ms": round(ms, 4),
                     "best_split": best[1], "best_ms": round(best[0], 4), "ratio": round(ratio, 3)})
        del op
    return {"shapes": rows, "mean_ratio": round(float(np.mean(ratios)), 3), "worst_ratio": round(float(np.max(ratios)), 3)}


MAX_LINE_BYTES = 4096
DIGEST_COLUMNS = ["cases", "min", "median", "max", "worst case"]


def digest(rows, value, name, higher_is_better=True):
    """[cases, min, median, max, worst case] of value(row) over the rows (DIGEST_COLUMNS)."""
    vals = [(value(r), name(r)) for r in rows]
    nums = sorted(v for v, _ in vals)
    worst = (min if higher_is_better else max)(vals)
    return [len(rows), nums[0], round(float(np.median(nums)), 3), nums[-1], worst[1]]


def summarize(configs, preprocess, dispatch):
    """One short digest per workload for the printed line; every case is in the detail file."""
    shape = lambda r: "%dx%dx%d %s" % (r["M"], r["Ncols"], r["K"], r["pattern"])
    s = {"digest_columns": DIGEST_COLUMNS}
    for key in ("llm", "ragged"):
        if key in configs:
            s[key] = {"frac_fp32_mfma_peak": digest(configs[key], lambda r: r["frac_fp32_mfma_peak"], shape)}
    if "llm" in configs:
        s["llm"]["speedup_over_ideal_4x"] = digest(configs["llm"], lambda r: r["speedup_over_ideal"], shape)
    for key in ("decode", "decode_llm", "decode_wide"):
        if key not in configs:
            continue
        s[key] = {}
        for mode in ("hot", "cold", "cold_reference_layout", "hot_split", "cold_split"):
            rows = [r for r in configs[key] if mode in r]
            if not rows:
                continue
            if "frac_hbm" in rows[0][mode]:     # B streamed from HBM
                s[key][mode + "_frac_hbm"] = digest(rows, lambda r: r[mode]["frac_hbm"], shape)
            else:                               # B re-read from the Infinity Cache: a rate, no HBM fraction
                s[key][mode + "_gbs"] = digest(rows, lambda r: r[mode]["gbs"], shape)
    if "fine" in configs:
        s["fine_frac_fp32_mfma_peak"] = {"%sx%d" % (r["pattern"], r["vec_len"]): r["frac_fp32_mfma_peak"]
                                         for r in configs["fine"]}
    if "launch_constant" in configs:
        s["launch_constant_us"] = {r["pattern"]: r.get("constant_us") for r in configs["launch_constant"]}
    if "compress" in configs:
        name = lambda r: "%dx%d %s" % (r["K"], r["Ncols"], r["pattern"])
        s["compress_frac_hbm"] = digest(configs["compress"], lambda r: r["compress"]["frac_hbm"], name)
        s["decompress_frac_hbm"] = digest(configs["compress"], lambda r: r["decompress"]["frac_hbm"], name)
        s["plain_copy_frac_hbm"] = digest(configs["compress"], lambda r: r["plain_copy_of_the_dense_operand"]["frac_hbm"], name)[1:4]
    if "rowmajor" in configs:
        s["rowmajor_overhead"] = digest(configs["rowmajor"], lambda r: r["overhead"], shape, higher_is_better=False)
    if "sweep100" in configs:
        s["sweep100_speedup_vs_dense"] = {"columns": ["mean", "min", "reference_on_a100_mean"]}
        for k, v in configs["sweep100"]["by_sparsity"].items():
            s["sweep100_speedup_vs_dense"][k] = [v["mean_speedup_vs_dense"], v["min_speedup_vs_dense"],
                                                 v["a100_reference_mean_speedup"]]
    if preprocess:
        s["preprocess_device_ms"] = {"%sx%d" % (r["pattern"], r["vec_len"]): r["device_one_kernel_ms"] for r in preprocess}
        s["preprocess_cpu_ms"] = {"%sx%d" % (r["pattern"], r["vec_len"]): r.get("cpu_reference_wall_ms", r["cpu_restatement_wall_ms"])
                                  for r in preprocess}
    if dispatch:
        s["dispatch"] = {"cases": len(dispatch["shapes"]), "mean_ratio": dispatch["mean_ratio"], "worst_ratio": dispatch["worst_ratio"]}
    return s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-rows", type=int, default=4096, help="rows of the CPU baseline sample (0 = skip)")
    ap.add_argument("--only", default="", help="comma list of parts to run beside the headline kernel: " +
                    ", ".join(PARTS) + " (default: all; 'none' times the headline kernel alone)")
    ap.add_argument("--headline-only", action="store_true", help="same as --only none --cpu-rows 0")
    ap.add_argument("--decode-rows", default="1,8,16,32", help="row counts of the decode part")
    ap.add_argument("--decode-shapes", default="8192x8192,4096x14336", help="K x Ncols of the decode part")
    ap.add_argument("--decode-patterns", default="1:8,2:8", help="patterns of the decode part")
    ap.add_argument("--decode-modes", default=",".join(DECODE_DEFAULT_MODES),
                    help="which of " + ", ".join(m[0] for m in DECODE_MODES) + " to time")
    ap.add_argument("--fine-cases", default="4:32x32,8:32x32,16:32x32,2:4x4,2:8x4,1:8x4,1:8x8,32:32x32",
                    help="cases of the fine part, n:m x vector length")
    ap.add_argument("--ksweep-ks", default="64,1024,4096", help="reduction lengths of the ksweep part")
    ap.add_argument("--ksweep-patterns", default="2:4,1:8,4:32", help="patterns of the ksweep part")
    ap.add_argument("--detail", default=os.path.join(ROOT, "bench_detail.json"),
                    help="file that receives every case of every part (the printed line holds digests)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy 5 times (known traffic, to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library is a single-GPU kernel library; run with --gpus 1", file=sys.stderr)
        return 2
    parts = (set(PARTS) - set(OPT_IN_PARTS)) if not args.only else set(p for p in args.only.split(",") if p and p != "none")
    if args.headline_only:
        parts = set()
    if args.cpu_rows <= 0:
        parts.discard("cpu")
    unknown = parts - set(PARTS)
    if unknown:
        print("bench.py: unknown part(s) %s" % ", ".join(sorted(unknown)), file=sys.stderr)
        return 2

    import torch
    pkg = importlib.import_module("nm-spmm_amd")
    datagen = importlib.import_module("nm-spmm_amd.datagen")
    if not os.path.exists(pkg.LIB_PATH):  # load what is built; build only when nothing is
        importlib.import_module("__graft_entry__").build()
    pkg.lib()  # fails loudly if the HIP library is still missing: there is no fallback
    torch.cuda.set_device(0)
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.manual_seed(20240)

    # ---- headline: 2:4 at 4096 cubed -------------------------------------------------------------
    head = Case(torch, pkg, datagen, 2, 4, seed=2024)
    ms, wall_ms = time_launches(torch, lambda: head.launch(pkg), args.steps, args.warmup)
    assert pkg.last_kernel() == "mfma"
    achieved = head.useful_flops() / (ms * 1e-3) / 1e12
    kernel_name = tile_kernel_name(pkg, head)

    sweep, dense = {}, None
    if "sweep" in parts:
        a = head.A.t().contiguous()
        b = torch.randn((K, N), dtype=torch.float32, device="cuda")
        c = torch.empty((M, N), dtype=torch.float32, device="cuda")
        dense_ms, _ = time_launches(torch, lambda: torch.mm(a, b, out=c), args.steps, args.warmup)
        del a, b, c
        dense = {"ms": round(dense_ms, 4), "tflops": round(2.0 * M * N * K / (dense_ms * 1e-3) / 1e12, 2),
                 "library": "torch.mm fp32 (rocBLAS/hipBLASLt)"}
        for idx, (n, m) in enumerate(PATTERNS):
            case = head if idx == 0 else Case(torch, pkg, datagen, n, m, seed=2000 + 10 * n + m)
            cms = ms if idx == 0 else time_launches(torch, lambda: case.launch(pkg), args.steps, args.warmup, 0.5)[0]
            useful = case.useful_flops() / (cms * 1e-3) / 1e12
            sweep["%d:%d" % (n, m)] = {
                "ms": round(cms, 4), "useful_tflops": round(useful, 2),
                "dense_equiv_tflops": round(2.0 * M * N * K / (cms * 1e-3) / 1e12, 2),
                "frac_fp32_mfma_peak": round(useful / FP32_MFMA_PEAK_TFLOPS, 4), "kernel": tile_kernel_name(pkg, case),
                "speedup_vs_dense": round(dense_ms / cms, 3), "speedup_over_ideal": round(dense_ms / cms / (m / n), 3)}
            if idx > 0:
                del case

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    cpu = None
    if "cpu" in parts:
        head.launch(pkg)
        torch.cuda.synchronize()
        got = head.C[:args.cpu_rows].cpu().numpy().astype(np.float64)
        want, cpu = cpu_baseline(head, args.cpu_rows)
        want = want.astype(np.float64)
        rms = np.sqrt(np.mean(want * want))
        cpu["gpu_vs_cpu_scaled_max_error"] = float(np.max(np.abs(got - want) / np.maximum(np.abs(want), rms)))

    configs = {}
    if "llm" in parts:
        configs["llm"] = run_llm(torch, pkg)
    if "ragged" in parts:
        configs["ragged"] = run_ragged(torch, pkg)
    if "decode" in parts:
        configs["decode"] = run_decode(
            torch, pkg, tuple(int(x) for x in args.decode_rows.split(",")),
            tuple(tuple(int(v) for v in x.split("x")) for x in args.decode_shapes.split(",")),
            tuple(tuple(int(v) for v in x.split(":")) for x in args.decode_patterns.split(",")),
            tuple(args.decode_modes.split(",")))
    if "decode_llm" in parts:
        configs["decode_llm"] = run_decode(torch, pkg, (1, 16, 32), DECODE_LLM_SHAPES, ((2, 8),), DECODE_LLM_MODES)
    if "decode_wide" in parts:
        # beyond the baseline's row counts: 33 to 64 rows on the row list (serving batches)
        configs["decode_wide"] = run_decode(torch, pkg, (48, 64), ((8192, 8192), (4096, 4096)), ((1, 8), (2, 8)),
                                            ("hot", "cold", "hot_reference_layout", "cold_reference_layout"))
    if "fine" in parts:
        configs["fine"] = run_fine(torch, pkg, tuple(
            (int(x.split(":")[0]), int(x.split(":")[1].split("x")[0]), int(x.split("x")[1])) for x in args.fine_cases.split(",")))
    if "ksweep" in parts:
        configs["launch_constant"] = run_ksweep(
            torch, pkg, tuple(int(x) for x in args.ksweep_ks.split(",")),
            tuple(tuple(int(v) for v in x.split(":")) for x in args.ksweep_patterns.split(",")))
    if "compress" in parts:
        configs["compress"] = run_compress(torch, pkg)
    if "rowmajor" in parts:
        configs["rowmajor"] = run_rowmajor(torch, pkg)
    if "sweep100" in parts:
        configs["sweep100"] = run_sweep100(torch, pkg)
    preprocess = run_preprocess(torch, pkg, datagen) if "preprocess" in parts else None
    dispatch = run_dispatch(torch, pkg) if "dispatch" in parts else None

    alg_bytes = 4.0 * (M * K + head.W * N + head.W * N / 32 + M * N)
    traffic, traffic_source = profiled_traffic()
    out = {
        "metric": "useful fp32 TFLOP/s, M=Ncols=K=4096, 2:4 (vector length 32)",
        "value": round(achieved, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "clock_prewarm_s": PREWARM_S,
        "device": dict(zip(("compute_units", "dies", "clock_hz"), pkg.device_figures())),
        "config": {"workload": "square sweep M=Ncols=K=4096 fp32, uniform(-1,1), seeded n:m patterns per 32-column "
                               "vector; value at 2:4, others under sweep", "tile": "Ns=128", "split_k": 1},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / FP32_MFMA_PEAK_TFLOPS, 4),
                     # HBM-side bytes per launch are a counter measurement (rocprofv3 FETCH_SIZE and
                     # WRITE_SIZE, scaled by a plain copy), taken in its own runs and read from the
                     # tracked summary; everything else in this object is computed in this run
                     "traffic": traffic, "traffic_unit": "bytes per launch", "traffic_source": traffic_source,
                     "algorithmic_bytes": alg_bytes, "kernel": kernel_name, "flops_per_launch": head.useful_flops(),
                     "launch_ms_events": round(ms, 5), "launch_ms_wall": round(wall_ms, 5)},
        "cpu_baseline": cpu,
        "dense_fp32_gemm": dense,
        "sweep": sweep,
    }
    detail = dict(out, configs=configs, preprocess=preprocess, dispatch=dispatch)
    detail_path = args.detail
    try:
        f = open(detail_path, "w")
    except OSError:  # a read-only tree: the line is still printed, the cases go beside the system's temporary files
        import tempfile
        detail_path = os.path.join(tempfile.gettempdir(), "bench_detail.json")
        f = open(detail_path, "w")
    with f:
        json.dump(detail, f, indent=1)
        f.write("\n")
    # the line itself stays short (harnesses keep only the last few KB of a run's output): the
    # headline fields whole, one digest per other workload, every case in the detail file
    out["sweep"] = {k: {f: v[f] for f in ("ms", "useful_tflops", "frac_fp32_mfma_peak", "speedup_vs_dense")}
                    for k, v in sweep.items()}
    out["summary"] = summarize(configs, preprocess, dispatch)
    out["detail_file"] = os.path.relpath(detail_path, ROOT) if os.path.abspath(detail_path).startswith(ROOT) else detail_path
    line = json.dumps(out, separators=(",", ":"))
    while len(line) > MAX_LINE_BYTES and out["summary"]:   # never at today's part list; the headline fields stay whatever happens
        out["summary"].popitem()
        out["summary_truncated"] = True
        line = json.dumps(out, separators=(",", ":"))
    print(line)
    return 0


if __name__ == "__main__":
    sys.exit(main())
