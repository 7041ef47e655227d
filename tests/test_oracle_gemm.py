"""Pins the CPU checker's multiplication (nm_oracle_gemm_cpu): golden C matrices written by the
reference's nmGEMM_on_cpu, bit-exact agreement with the live compiled reference, and the
textbook identity C = A . decompress(B, D) evaluated by numpy in fp64."""
import glob
import os

import numpy as np
import pytest

from conftest import GOLDEN_DIR, datagen


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN_DIR, "gemm_*.npz"))), ids=os.path.basename)
def test_gemm_matches_reference_golden_bit_exact(oracle, path):
    g = np.load(path)
    M, N, W = int(g["M"]), int(g["N"]), int(g["W"])
    C = oracle.gemm_cpu(g["A"].reshape(-1), g["B"].reshape(-1), g["D"].reshape(-1), M, N, W)
    assert np.array_equal(C.reshape(M, N), g["C"])


@pytest.mark.parametrize("M,N,K,n,m", [(40, 96, 128, 2, 4), (33, 64, 256, 1, 8), (64, 128, 64, 3, 8), (16, 32, 32, 1, 1)])
def test_gemm_matches_live_reference_bit_exact(oracle, reference, M, N, K, n, m):
    d = datagen.init_data(M, N, K, n, m, seed=M * 7 + n)
    A, B, D = d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1)
    got = oracle.gemm_cpu(A, B, D, M, N, d["W"])
    want = reference.gemm_cpu(A, B, D, M, N, K, d["W"])
    assert np.array_equal(got, want)
    # accumulate-into-C semantics and row slices
    C0 = np.full(M * N, 0.5, np.float32)
    got = oracle.gemm_cpu(A, B, D, M, N, d["W"], C=C0.copy())
    want = reference.gemm_cpu(A, B, D, M, N, K, d["W"], C=C0.copy())
    assert np.array_equal(got, want)
    part = oracle.gemm_cpu(A, B, D, M, N, d["W"], rows=(3, 11))
    full = reference.gemm_cpu(A, B, D, M, N, K, d["W"]).reshape(M, N)
    assert np.array_equal(part.reshape(M, N)[3:11], full[3:11])
    assert not part.reshape(M, N)[:3].any() and not part.reshape(M, N)[11:].any()


@pytest.mark.parametrize("M,N,K,n,m,vl", [(48, 128, 256, 2, 4, 32), (20, 64, 128, 1, 8, 32), (32, 64, 64, 2, 4, 4),
                                           (8, 96, 96, 3, 8, 8)])
def test_gemm_equals_dense_product_of_decompressed_operand(oracle, M, N, K, n, m, vl):
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=5)
    A, B, D = d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1)
    dense = oracle.decompress(B, D, K, N, d["W"], vl)
    # decompress itself: the kept entries are exactly B, everything else is 0
    assert np.count_nonzero(dense) <= d["W"] * N
    cols = np.arange(N)
    for k in range(0, d["W"], 7):
        rows = d["D_cm"][cols // vl, k]
        assert np.array_equal(dense[rows, cols], d["BT"][k])
    assert np.isclose(np.abs(dense).sum(dtype=np.float64), np.abs(d["BT"]).sum(dtype=np.float64))
    want = d["A_km"].T.astype(np.float64) @ dense.astype(np.float64)
    got = oracle.gemm_cpu(A, B, D, M, N, d["W"], vl).reshape(M, N)
    assert np.allclose(got, want, rtol=0, atol=1e-5 * np.sqrt(K))


def test_dense_pattern_reduces_to_plain_gemm(oracle):
    M, N, K = 24, 64, 32
    d = datagen.init_data(M, N, K, 32, 32, seed=9)
    assert np.array_equal(d["DT"], np.broadcast_to(np.arange(K, dtype=np.int32)[:, None], (K, N // 32)))
    got = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"])
    want = d["A_km"].T.astype(np.float64) @ d["BT"].astype(np.float64)
    assert np.allclose(got.reshape(M, N), want, atol=1e-5)
