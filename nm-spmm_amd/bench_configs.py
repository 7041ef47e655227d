#!/usr/bin/env python3
"""Measurement of the baseline's other workloads (bench.py at the repository root covers the
square sweep): LLM-layer shapes, decode-sized M, and the fine-grained / short-vector patterns.
Prints one markdown table row per case.

    python nm-spmm_amd/bench_configs.py [llm] [decode] [fine] [compress] [rowmajor] [sweep100]

useful TFLOP/s = 2*M*Ncols*W / t; GB/s = algorithmic bytes
4*(M*K + W*Ncols + W*Ncols/L + M*Ncols) (+ column_info) / t.
"""
import importlib
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

pkg = importlib.import_module("nm-spmm_amd")
datagen = importlib.import_module("nm-spmm_amd.datagen")

GEOMETRY = {(2, 4): (32, 16), (3, 8): (32, 12), (2, 8): (64, 16), (1, 8): (64, 8),
            (16, 32): (32, 16), (12, 32): (32, 12), (8, 32): (64, 16), (4, 32): (64, 8)}


def timed(fn, steps=50, warmup=10, prewarm_s=0.3):
    # an idle GPU sits near 1 GHz; give it load until the shader clock has ramped up
    t_end = time.perf_counter() + prewarm_s
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    best = 1e9
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / steps)
    return best


class Operands:
    def __init__(self, M, N, K, n, m, vec_len=32, Ns=128, dist="uniform", b_scale=1.0, seed=0):
        d = datagen.init_data(M, N, K, n, m, vec_len=vec_len, seed=seed, dist=dist, b_scale=b_scale)
        self.M, self.N, self.K, self.W, self.Q, self.vl, self.Ns = M, N, K, d["W"], d["Q"], vec_len, Ns
        self.A = torch.from_numpy(d["A_km"]).cuda()
        self.B = torch.from_numpy(d["BT"]).cuda()
        self.C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        DT0 = torch.from_numpy(d["DT"].reshape(-1).copy()).cuda()
        DT, self.D = torch.empty_like(DT0), torch.empty_like(DT0)
        if vec_len == 32:
            self.window, self.kept = GEOMETRY[(n, m)]
        else:
            self.window, self.kept = m, n
        self.cinfo = None
        if self.window == 64:
            self.cinfo = torch.empty(pkg.column_info_ints(self.W, self.kept, self.window, N, Ns), dtype=torch.int32,
                                     device="cuda")

        def preprocess():
            DT.copy_(DT0)
            pn, pm = n, m
            while pm < self.window:
                pn, pm = pkg.trans_index_device(DT, self.W, N, self.Q, pn, pm)
            if self.cinfo is None:
                pkg.preprocess_low_device(DT, self.D, self.W, self.Q, Ns, vec_len)
            else:
                pkg.preprocess_high_device(self.cinfo, pm, pn, DT, self.D, self.W, self.Q, N, Ns, vec_len)

        self.preprocess_ms = timed(preprocess, 5, 1, 0.0)

    def launch(self, split_k=1, ws=None):
        pkg.spmm(self.A, self.B, self.D, self.cinfo, self.C, self.M, self.N, self.K, self.W, self.window, self.kept,
                 self.vl, self.Ns, split_k, ws)

    def flops(self):
        return 2.0 * self.M * self.N * self.W

    def bytes(self):
        b = 4.0 * (self.M * self.K + self.W * self.N + self.W * self.N / self.vl + self.M * self.N)
        if self.cinfo is not None:
            b += 4.0 * self.cinfo.numel()
        return b


def dense_ms(M, N, K):
    a = torch.randn((M, K), dtype=torch.float32, device="cuda")
    b = torch.randn((K, N), dtype=torch.float32, device="cuda")
    c = torch.empty((M, N), dtype=torch.float32, device="cuda")
    return timed(lambda: torch.mm(a, b, out=c))


def llm():
    print("| M | K x Ncols | pattern | kernel | best split of 1/2/4/8 | ms | useful TFLOP/s | library's split | ms | dense fp32 GEMM ms | speedup | of ideal 4x | preprocess ms |")
    print("|---|---|---|---|---|---|---|---|---|---|---|---|---|")
    for (K, N) in ((4096, 4096), (4096, 11008), (11008, 4096)):
        for M in (512, 2048, 8192):
            op = Operands(M, N, K, 2, 8, dist="normal", b_scale=0.02, seed=M + K)
            best = (1e9, 1)
            for split in (1, 2, 4, 8):
                if split > 1 and (M // 128) * (N // 128) * split > 4096:
                    continue
                ws = None if split == 1 else torch.empty(pkg.workspace_bytes(M, N, split) // 4, dtype=torch.float32,
                                                         device="cuda")
                best = min(best, (timed(lambda: op.launch(split, ws)), split))
            ms, split = best
            auto_split = pkg.suggest_split_k(M, N, op.W, op.kept)
            auto_ms = timed(lambda: pkg.gemm_auto(op.A, op.B, op.D, op.cinfo, op.C, M, N, K, op.W, 0.75))
            dms = dense_ms(M, N, K)
            print("| %d | %dx%d | 2:8 | %s | %d | %.4f | %.1f | %d | %.4f | %.4f | %.2f | %.2f | %.3f |" % (
                M, K, N, pkg.last_kernel(), split, ms, op.flops() / ms / 1e9, auto_split, auto_ms, dms, dms / auto_ms,
                dms / auto_ms / 4, op.preprocess_ms), flush=True)
            del op


def decode():
    print("| M | K x Ncols | pattern | kernel | us | GB/s (algorithmic) | of 8 TB/s |")
    print("|---|---|---|---|---|---|---|")
    for (K, N) in ((8192, 8192), (4096, 14336)):
        for (n, m) in ((1, 8), (2, 8)):
            for M in (1, 8, 16, 32, 64, 128):
                op = Operands(M, N, K, n, m, dist="normal", b_scale=0.02, seed=M)
                ms = timed(lambda: pkg.gemm_auto(op.A, op.B, op.D, op.cinfo, op.C, M, N, K, op.W, 1.0 - n / m))
                print("| %d | %dx%d | %d:%d | %s | %.1f | %.0f | %.3f |" % (
                    M, K, N, n, m, pkg.last_kernel(), ms * 1e3, op.bytes() / ms / 1e6, op.bytes() / ms / 1e6 / 8000), flush=True)
                del op


def fine():
    print("| pattern | vector length | kernel | ms | useful TFLOP/s | of fp32 MFMA peak | preprocess ms | index bytes |")
    print("|---|---|---|---|---|---|---|---|")
    for (n, m, vl) in ((4, 32, 32), (8, 32, 32), (16, 32, 32), (2, 4, 4), (2, 4, 8), (2, 4, 16), (2, 8, 4), (1, 8, 4)):
        op = Operands(4096, 4096, 4096, n, m, vec_len=vl, seed=n)
        ms = timed(lambda: op.launch(), 20, 2)
        print("| %d:%d | %d | %s | %.4f | %.1f | %.3f | %.3f | %d |" % (
            n, m, vl, pkg.last_kernel(), ms, op.flops() / ms / 1e9, op.flops() / ms / 1e9 / 157.3, op.preprocess_ms,
            op.D.numel() * 4), flush=True)
        del op


def compress():
    print("| op | K x Ncols | pattern | us | GB/s (algorithmic) | of 8 TB/s |")
    print("|---|---|---|---|---|---|")
    for (K, N) in ((4096, 4096), (11008, 4096), (8192, 8192)):
        dense = torch.randn((K, N), dtype=torch.float32, device="cuda")
        for (n, m) in ((2, 4), (2, 8), (1, 8), (8, 32)):
            W, Q = K // m * n, N // 32
            BT = torch.empty((W, N), dtype=torch.float32, device="cuda")
            DT = torch.empty((W, Q), dtype=torch.int32, device="cuda")
            back = torch.empty_like(dense)
            nbytes = 4.0 * (K * N + W * N + W * Q)
            for name, fn in (("compress", lambda: pkg.compress_device(dense, K, N, n, m, BT, DT)),
                             ("decompress", lambda: pkg.decompress_device(BT, DT, K, N, n, m, back))):
                ms = timed(fn)
                print("| %s | %dx%d | %d:%d | %.1f | %.0f | %.3f |" % (name, K, N, n, m, ms * 1e3, nbytes / ms / 1e6,
                                                                    nbytes / ms / 1e6 / 8000), flush=True)


def sweep100():
    """The reference's 100-shape comparison against the dense GEMM
    (benchmark/kernel_performance/run_test/nmspmm/run_nmspmm.sh:16-36): 5 row counts x 20 LLM layer
    shapes, patterns n:32 at 50 / 62.5 / 75 / 87.5 %, here with the split the library picks instead
    of the best of four timed ones.  Patterns and values are drawn on the GPU."""
    Ms = (256, 512, 1024, 2048, 4096)
    Ns = (2048, 6144, 2048, 5632, 4096, 12288, 4096, 11008, 5120, 15360, 5120, 13824, 6656, 19968, 6656, 17920, 8192,
          24576, 8192, 22016)
    Ks = (2048, 2048, 5632, 2048, 4096, 4096, 11008, 4096, 5120, 5120, 13824, 5120, 6656, 6656, 17920, 6656, 8192, 8192,
          22016, 8192)
    kinds = ((0.5, 16, 32, 16), (0.625, 12, 32, 12), (0.75, 8, 64, 16), (0.875, 4, 64, 8))  # sparsity, n of 32, window, kept
    dense = {}
    speed = {k[0]: [] for k in kinds}
    print("| sparsity | M | Ncols | K | split | ms | useful TFLOP/s | dense ms | speedup |")
    print("|---|---|---|---|---|---|---|---|---|")
    for (N, K) in zip(Ns, Ks):
        Q = N // 32
        for (sparsity, n, window, kept) in kinds:
            W = K // 32 * n
            B = torch.randn((W, N), dtype=torch.float32, device="cuda") * 0.02
            pick = torch.rand((K // 32, Q, 32), device="cuda").argsort(dim=2)[:, :, :n].sort(dim=2).values
            DT = pick.permute(0, 2, 1).reshape(W, Q).to(torch.int32).contiguous()
            D = torch.empty_like(DT)
            cinfo = None
            if window == 64:
                pn, pm = pkg.trans_index_device(DT, W, N, Q, n, 32)
                cinfo = torch.empty(pkg.column_info_ints(W, pn, pm, N, 128), dtype=torch.int32, device="cuda")
                pkg.preprocess_high_device(cinfo, pm, pn, DT, D, W, Q, N, 128)
            else:
                pkg.preprocess_low_device(DT, D, W, Q, 128)
            for M in Ms:
                A = torch.randn((K, M), dtype=torch.float32, device="cuda")
                C = torch.empty((M, N), dtype=torch.float32, device="cuda")
                ms = timed(lambda: pkg.gemm_auto(A, B, D, cinfo, C, M, N, K, W, sparsity), 20, 3, 0.05)
                if (M, N, K) not in dense:
                    Bd = torch.randn((K, N), dtype=torch.float32, device="cuda")
                    Am = A.t().contiguous()
                    dense[(M, N, K)] = timed(lambda: torch.mm(Am, Bd, out=C), 20, 3, 0.05)
                    del Bd, Am
                dms = dense[(M, N, K)]
                speed[sparsity].append(dms / ms)
                print("| %.3f | %d | %d | %d | %d | %.4f | %.1f | %.4f | %.2f |" % (
                    sparsity, M, N, K, pkg.suggest_split_k(M, N, W, kept), ms, 2.0 * M * N * W / ms / 1e9, dms, dms / ms),
                    flush=True)
            del B, DT, D, cinfo
    print()
    print("| sparsity | shapes | mean speedup over the dense fp32 GEMM | min | max | ideal |")
    print("|---|---|---|---|---|---|")
    for (sparsity, n, window, kept) in kinds:
        v = speed[sparsity]
        print("| %.3f | %d | %.2f | %.2f | %.2f | %.2f |" % (sparsity, len(v), sum(v) / len(v), min(v), max(v), 32.0 / n))


def rowmajor():
    print("| M | K x Ncols | pattern | transpose us | GB/s of 2*M*K*4 | multiply ms | both ms | overhead |")
    print("|---|---|---|---|---|---|---|---|")
    for (K, N) in ((4096, 4096), (4096, 11008), (11008, 4096)):
        for M in (512, 2048, 8192):
            op = Operands(M, N, K, 2, 8, dist="normal", b_scale=0.02, seed=M + K)
            A_rm = op.A.t().contiguous()
            split = pkg.suggest_split_k(M, N, op.W, op.kept)
            ws = torch.empty(pkg.workspace_bytes_rowmajor(M, N, K, split) // 4, dtype=torch.float32, device="cuda")
            ws_cm = torch.empty(max(pkg.workspace_bytes(M, N, split) // 4, 1), dtype=torch.float32, device="cuda")
            t_tr = timed(lambda: pkg.transpose_device(A_rm, M, K, ws))
            t_mm = timed(lambda: op.launch(split, ws_cm if split > 1 else None))
            t_both = timed(lambda: pkg.spmm_rowmajor(A_rm, op.B, op.D, op.cinfo, op.C, M, N, K, op.W, op.window, op.kept, ws,
                                                     32, op.Ns, split))
            print("| %d | %dx%d | 2:8 | %.1f | %.0f | %.4f | %.4f | %.1f %% |" % (
                M, K, N, t_tr * 1e3, 8.0 * M * K / t_tr / 1e6, t_mm, t_both, 100.0 * (t_both / t_mm - 1.0)), flush=True)
            del op


if __name__ == "__main__":
    which = sys.argv[1:] or ["llm", "decode", "fine", "compress", "rowmajor"]
    pkg.lib()
    for name in which:
        print("\n### %s" % name)
        {"llm": llm, "decode": decode, "fine": fine, "compress": compress, "rowmajor": rowmajor, "sweep100": sweep100}[name]()
