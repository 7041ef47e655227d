"""Pins the CPU checker's compression (nm_oracle_compress).  The reference has no compression
routine (it synthesises compressed operands, include/utils.h:40-64), so the checker is pinned by
what fixes the result independently of its own code: it must recover the generator's (BT, DT) from
their dense expansion, kept rows must dominate dropped rows in a score recomputed in fp64, equal
scores must resolve to the lower row, and negating the input must change nothing but signs."""
import numpy as np
import pytest

from conftest import datagen


def dense_of(d):
    """Scatter the generator's compressed operand to K x N with numpy only."""
    K, N, W, vl, n, m = d["K"], d["N"], d["W"], d["vec_len"], d["n"], d["m"]
    dense = np.zeros((K, N), np.float32)
    rows = (np.arange(W) // n * m)[:, None] + d["DT"]          # [W][Q] dense row of each kept row
    cols = np.arange(N)
    dense[np.repeat(rows, vl, axis=1), np.broadcast_to(cols, (W, N))] = d["BT"]
    return dense


@pytest.mark.parametrize("K,N,n,m,vl", [(64, 128, 2, 4, 32), (128, 96, 1, 8, 32), (96, 64, 3, 8, 32), (64, 64, 8, 32, 32),
                                         (32, 32, 2, 4, 4), (64, 48, 5, 16, 8), (64, 64, 3, 4, 16)])
def test_compress_recovers_generated_operand(oracle, K, N, n, m, vl):
    d = datagen.init_data(8, N, K, n, m, vec_len=vl, seed=K + n)
    dense = dense_of(d)
    BT, DT = oracle.compress(dense, n, m, vl)
    assert np.array_equal(DT, d["DT"])
    assert np.array_equal(BT, d["BT"])


@pytest.mark.parametrize("K,N,n,m,vl", [(128, 128, 2, 4, 32), (64, 256, 2, 8, 32), (64, 64, 1, 8, 4), (96, 96, 12, 32, 32)])
def test_kept_rows_dominate_dropped_rows(oracle, K, N, n, m, vl):
    rng = np.random.default_rng(K * 3 + n)
    dense = rng.standard_normal((K, N), dtype=np.float32)
    BT, DT = oracle.compress(dense, n, m, vl)
    Q = N // vl
    score = np.abs(dense.astype(np.float64)).reshape(K // m, m, Q, vl).sum(axis=3)   # [win][row][vec], exact enough
    kept = DT.reshape(K // m, n, Q)
    assert np.all(np.diff(kept, axis=1) > 0) and kept.min() >= 0 and kept.max() < m
    mask = np.zeros((K // m, m, Q), bool)
    np.put_along_axis(mask, kept, True, axis=1)
    worst_kept = np.where(mask, score, np.inf).min(axis=1)
    best_dropped = np.where(mask, -np.inf, score).max(axis=1)
    # fp32 pairwise sums differ from fp64 by at most a few ulp of the score
    assert np.all(worst_kept >= best_dropped * (1 - 1e-5))
    # values are the kept rows, verbatim
    rows = (np.arange(K // m * n) // n * m)[:, None] + DT
    assert np.array_equal(BT, dense[np.repeat(rows, vl, axis=1), np.broadcast_to(np.arange(N), BT.shape)])


def test_ties_prefer_lower_rows_and_sign_is_irrelevant(oracle):
    K, N, n, m, vl = 16, 64, 3, 8, 32
    dense = np.ones((K, N), np.float32)
    dense[1::2] *= -1.0                      # all scores equal in magnitude
    BT, DT = oracle.compress(dense, n, m, vl)
    assert np.array_equal(DT, np.tile(np.arange(n, dtype=np.int32)[:, None], (K // m, N // vl)))
    dense[5] *= 3.0                          # one clear winner in window 0, ties elsewhere
    _, DT = oracle.compress(dense, n, m, vl)
    assert np.array_equal(DT[:n, 0], [0, 1, 5])
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 64), dtype=np.float32)
    BTp, DTp = oracle.compress(x, 2, 4, 32)
    BTn, DTn = oracle.compress(-x, 2, 4, 32)
    assert np.array_equal(DTp, DTn) and np.array_equal(BTp, -BTn)


def test_score_is_the_pairwise_sum_not_the_sequential_one(oracle):
    # 32 values whose pairwise and left-to-right fp32 sums differ decide a near tie
    big, tiny = np.float32(1.0), np.float32(2.0 ** -24)
    row_a = np.array([big] + [tiny] * 31, np.float32)      # sequential: stays 1.0; pairwise: the tinies add up first
    pair = np.float32(0)
    level = row_a.copy()
    while level.size > 1:
        level = (level[0::2] + level[1::2]).astype(np.float32)
    pair = level[0]
    seq = np.float32(0)
    for v in row_a:
        seq = np.float32(seq + v)
    assert pair > seq
    between = np.float32((np.float64(pair) + np.float64(seq)) / 2)
    row_b = np.zeros(32, np.float32)
    row_b[0] = np.nextafter(pair, np.float32(0))          # just below the pairwise sum, above the sequential one
    assert seq <= row_b[0] < pair and between is not None
    dense = np.zeros((4, 32), np.float32)
    dense[2], dense[1] = row_a, row_b
    _, DT = oracle.compress(dense, 1, 4, 32)
    assert DT[0, 0] == 2
