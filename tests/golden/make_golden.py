"""Writes the golden fixtures of tests/golden/ by running the REFERENCE's own host code
(oracle/_ref/libnmref.so, compiled by oracle/Makefile from /root/reference) on small seeded
inputs.  Run in the build container only:  python tests/golden/make_golden.py

Each .npz holds inputs and the reference's outputs (data only):
  preprocess_<tag>.npz  DT_in, after transIndex, after PreProcessing_{low,high}_sparsity (+column_info)
  gemm_<tag>.npz        A, B, D (reference CPU layouts) and C from nmGEMM_on_cpu
"""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.nm_oracle import Reference  # noqa: E402

datagen = importlib.import_module("nm-spmm_amd.datagen")
OUT = os.path.dirname(os.path.abspath(__file__))


def preprocess_case(ref, tag, N, K, n, m, seed, low_ns, high_ns, trans_times):
    d = datagen.init_data(4, N, K, n, m, seed=seed)
    W, Q = d["W"], d["Q"]
    out = {"N": N, "K": K, "W": W, "Q": Q, "n": n, "m": m, "DT_in": d["DT"]}
    for Ns in low_ns:
        x = d["DT"].reshape(-1).copy()
        ref.preprocess_low(x, W, Q, Ns)
        out["low_Ns%d" % Ns] = x
    x = d["DT"].reshape(-1).copy()
    pn, pm = n, m
    for t in range(trans_times):
        pn, pm = ref.trans_index(x, W, N, Q, pn, pm)
        out["trans%d" % (t + 1)] = x.copy()
    out["pN_final"], out["pM_final"] = pn, pm
    for Ns in high_ns:
        y = x.copy()
        ci = ref.preprocess_high(pm, pn, y, W, Q, N, Ns, slack=True)
        assert np.all(ci[-pm:] == -12345), "reference wrote the slack window"
        out["high_Ns%d_DT" % Ns] = y
        out["high_Ns%d_cinfo" % Ns] = ci[:-pm]
    np.savez_compressed(os.path.join(OUT, "preprocess_%s.npz" % tag), **out)


def gemm_case(ref, tag, M, N, K, n, m, seed):
    d = datagen.init_data(M, N, K, n, m, seed=seed)
    C = ref.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, K, d["W"])
    np.savez_compressed(os.path.join(OUT, "gemm_%s.npz" % tag), M=M, N=N, K=K, W=d["W"], n=n, m=m,
                        A=d["A_km"], B=d["B_cm"], D=d["D_cm"], C=C.reshape(M, N))


def main():
    ref = Reference()
    # native reference patterns (pruning_M = 32), one transIndex for the high path
    preprocess_case(ref, "8of32", N=256, K=256, n=8, m=32, seed=101, low_ns=[32, 64, 128], high_ns=[32, 64, 128], trans_times=1)
    preprocess_case(ref, "4of32", N=256, K=128, n=4, m=32, seed=102, low_ns=[128], high_ns=[32, 64, 128], trans_times=1)
    preprocess_case(ref, "16of32", N=128, K=128, n=16, m=32, seed=103, low_ns=[32, 64, 128], high_ns=[], trans_times=0)
    # narrow patterns widened by repeated transIndex
    preprocess_case(ref, "2of4", N=128, K=128, n=2, m=4, seed=104, low_ns=[128], high_ns=[], trans_times=3)
    preprocess_case(ref, "1of8", N=256, K=256, n=1, m=8, seed=105, low_ns=[], high_ns=[64, 128], trans_times=3)
    preprocess_case(ref, "2of8", N=128, K=128, n=2, m=8, seed=106, low_ns=[], high_ns=[128], trans_times=3)
    gemm_case(ref, "2of4", M=24, N=64, K=64, n=2, m=4, seed=201)
    gemm_case(ref, "1of8", M=16, N=96, K=128, n=1, m=8, seed=202)
    gemm_case(ref, "12of32", M=8, N=32, K=64, n=12, m=32, seed=203)


if __name__ == "__main__":
    main()
