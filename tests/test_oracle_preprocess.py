"""Pins the CPU checker's index preprocessing (oracle/nm_oracle.cpp) three independent ways:
golden vectors written by the reference's own code, the live compiled reference where it is
present, and facts the mathematics fixes (library transpose, sorted(set()), decode round trips).
None of the checks re-types the oracle's formulas."""
import glob
import os

import numpy as np
import pytest

from conftest import GOLDEN_DIR, datagen


def golden(pattern):
    files = sorted(glob.glob(os.path.join(GOLDEN_DIR, pattern)))
    assert files
    return files


@pytest.mark.parametrize("path", golden("preprocess_*.npz"), ids=os.path.basename)
def test_oracle_matches_reference_golden(oracle, path):
    g = np.load(path)
    W, Q, n, m = int(g["W"]), int(g["Q"]), int(g["n"]), int(g["m"])
    for key in g.files:
        if key.startswith("low_Ns"):
            Ns = int(key[6:])
            x = g["DT_in"].reshape(-1).copy()
            oracle.preprocess_low(x, W, Q, Ns)
            assert np.array_equal(x, g[key]), key
    x = g["DT_in"].reshape(-1).copy()
    pn, pm, t = n, m, 0
    while "trans%d" % (t + 1) in g.files:
        pn, pm = oracle.trans_index(x, W, Q, pn, pm)
        t += 1
        assert np.array_equal(x, g["trans%d" % t]), "trans%d" % t
    assert (pn, pm) == (int(g["pN_final"]), int(g["pM_final"]))
    for key in g.files:
        if key.startswith("high_Ns") and key.endswith("_DT"):
            Ns = int(key[7:-3])
            y = x.copy()
            ci = oracle.preprocess_high(pm, pn, y, W, Q, Ns)
            assert np.array_equal(y, g[key]), key
            assert np.array_equal(ci, g["high_Ns%d_cinfo" % Ns]), key


CASES = [  # N, K, n, m, doublings
    (128, 128, 2, 4, 3), (256, 256, 3, 8, 2), (384, 256, 2, 8, 3), (128, 512, 1, 8, 3),
    (256, 128, 8, 32, 1), (128, 256, 4, 32, 1), (128, 64, 16, 32, 0), (640, 128, 12, 32, 0),
]


@pytest.mark.parametrize("N,K,n,m,times", CASES)
def test_oracle_matches_live_reference(oracle, reference, N, K, n, m, times):
    d = datagen.init_data(4, N, K, n, m, seed=N + K + n + m)
    W, Q = d["W"], d["Q"]
    a, b = d["DT"].reshape(-1).copy(), d["DT"].reshape(-1).copy()
    pa = pb = (n, m)
    for _ in range(times):
        pa = oracle.trans_index(a, W, Q, *pa)
        pb = reference.trans_index(b, W, N, Q, *pb)
        assert pa == pb and np.array_equal(a, b)
    for Ns in (32, 64, 128):
        if N % Ns:
            continue
        x, y = a.copy(), a.copy()
        oracle.preprocess_low(x, W, Q, Ns)
        reference.preprocess_low(y, W, Q, Ns)
        assert np.array_equal(x, y)
        x, y = a.copy(), a.copy()
        ci = oracle.preprocess_high(pa[1], pa[0], x, W, Q, Ns)
        cr = reference.preprocess_high(pa[1], pa[0], y, W, Q, N, Ns, slack=True)
        assert np.array_equal(x, y)
        assert np.array_equal(ci, cr[:ci.size])
        assert np.all(cr[ci.size:] == -12345)  # the reference never writes its slack window


@pytest.mark.parametrize("N,K,n,m,times", CASES)
def test_trans_index_decodes_to_the_same_global_rows(oracle, N, K, n, m, times):
    """Whatever widening does, (window number * window size + local index) must still name the
    dense K row the generator chose; the widened indices stay ascending inside a window."""
    d = datagen.init_data(4, N, K, n, m, seed=7)
    W, Q = d["W"], d["Q"]
    x = d["DT"].reshape(-1).copy()
    pn, pm = n, m
    for _ in range(times):
        pn, pm = oracle.trans_index(x, W, Q, pn, pm)
    assert (pn, pm) == (n << times, m << times)
    x = x.reshape(W, Q)
    glob_rows = (np.arange(W) // pn * pm)[:, None] + x
    assert np.array_equal(glob_rows, d["D_cm"].T)
    assert x.min() >= 0 and x.max() < pm
    win = x.reshape(W // pn, pn, Q)
    assert np.all(np.diff(win, axis=1) > 0)


@pytest.mark.parametrize("Ns", [32, 64, 128])
def test_low_is_the_blocked_transpose(oracle, Ns):
    d = datagen.init_data(4, 256, 128, 2, 4, seed=11)
    W, Q = d["W"], d["Q"]
    Qs = Ns // 32
    x = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(x, W, Q, Ns)
    want = d["DT"].reshape(W, Q // Qs, Qs).transpose(1, 0, 2)  # numpy's own transpose
    assert np.array_equal(x, want.reshape(-1))
    if Ns == 32:
        assert np.array_equal(x.reshape(Q, W), d["DT"].T)


@pytest.mark.parametrize("n,m,times", [(1, 8, 3), (2, 8, 3), (4, 32, 1), (8, 32, 1), (2, 4, 3)])
@pytest.mark.parametrize("Ns", [32, 64, 128])
def test_high_by_brute_force(oracle, n, m, times, Ns):
    N, K = 256, 256
    d = datagen.init_data(4, N, K, n, m, seed=13 + Ns)
    W, Q = d["W"], d["Q"]
    x = d["DT"].reshape(-1).copy()
    pn, pm = n, m
    for _ in range(times):
        pn, pm = oracle.trans_index(x, W, Q, pn, pm)
    before = x.reshape(W, Q).copy()
    ci = oracle.preprocess_high(pm, pn, x, W, Q, Ns)
    Qs = Ns // 32
    nwin = W // pn
    ci = ci.reshape(Q // Qs, nwin, pm)
    after = x.reshape(Q // Qs, W, Qs)
    for jb in range(Q // Qs):
        for w in range(nwin):
            cell = before[w * pn:(w + 1) * pn, jb * Qs:(jb + 1) * Qs]
            used = sorted(set(cell.reshape(-1).tolist()))
            assert ci[jb, w, :len(used)].tolist() == used
            assert np.all(ci[jb, w, len(used):] == -1)
            ranks = after[jb, w * pn:(w + 1) * pn, :]
            assert np.array_equal(ci[jb, w][ranks], cell)  # gather round trip
    if Ns == 32:  # one vector per block: the list is the window's own indices, ranks are 0..pN-1
        assert np.array_equal(after.reshape(Q, nwin, pn), np.broadcast_to(np.arange(pn), (Q, nwin, pn)))
