"""Seeded synthetic operands for the N:M sparse x dense path.

Plays the role of the reference's init_data (include/utils.h:10-66), which is seeded from the
clock and therefore cannot be reproduced: same operand meanings and layouts, but deterministic
(numpy PCG64), signed values, and any n:m pattern and vector length.

Returned arrays (numpy, C-contiguous):
  A_km   float32 [K][M]   A in the reference's column-major order (element (i,k) at [k][i])
  BT     float32 [W][N]   compressed values, row-major (what the GPU consumes)
  B_cm   float32 [N][W]   the same values column-major (element (k,j) at [j][k]; CPU check path)
  DT     int32   [W][Q]   window-local indices, row-major (input of the preprocessing)
  D_cm   int32   [Q][W]   global K indices column-major (element (k,a) at [a][k]; CPU check path)
"""
import numpy as np


def init_data(M, N, K, n, m, vec_len=32, seed=0, dist="uniform", a_scale=1.0, b_scale=1.0):
    assert K % m == 0 and N % vec_len == 0 and 0 < n <= m
    rng = np.random.default_rng(seed)
    nwin = K // m
    W = nwin * n
    Q = N // vec_len

    def values(shape, scale):
        if dist == "unit":  # [0, 1): the reference's own kind of data (rand() / RAND_MAX, include/utils.h:36,42)
            return (rng.random(shape, dtype=np.float32) * np.float32(scale)).astype(np.float32)
        if dist == "uniform":
            return ((rng.random(shape, dtype=np.float32) * 2.0 - 1.0) * np.float32(scale)).astype(np.float32)
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)).astype(np.float32)

    A_km = values((K, M), a_scale)
    BT = values((W, N), b_scale)
    # n distinct positions out of m per (window, column vector), ascending
    keys = rng.random((nwin, Q, m))
    pick = np.sort(np.argsort(keys, axis=-1)[..., :n], axis=-1).astype(np.int32)  # [nwin][Q][n]
    DT = np.ascontiguousarray(pick.transpose(0, 2, 1).reshape(W, Q))
    base = (np.arange(W, dtype=np.int32) // n * m)[:, None]
    D_cm = np.ascontiguousarray((DT + base).T)
    B_cm = np.ascontiguousarray(BT.T)
    return {"A_km": A_km, "BT": BT, "B_cm": B_cm, "DT": DT, "D_cm": D_cm, "M": M, "N": N, "K": K, "W": W, "Q": Q,
            "n": n, "m": m, "vec_len": vec_len}
