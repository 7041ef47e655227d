"""The checker's row list (nm_oracle_row_index), pinned by an independent source: the generator's
own global row numbers D_cm, which are what the reference's CPU path multiplies with
(include/utils.h:60, D = local + window * pM).  Whatever the widening, the column-block width or
the layout (ranks through column_info, or plain window-local indices), entry (v, r) of the list
must be 1 + D_cm[v][r]; entries beyond W are 0.  A dropped term (the window base), a transposed
block index or a rank left unresolved fails this."""
import numpy as np
import pytest

from conftest import datagen, preprocess_with_oracle


def expected_list(d):
    W, Q = d["W"], d["Q"]
    G = (W + 15) // 16
    rows = np.zeros((Q, G * 16), np.int64)
    rows[:, :W] = d["D_cm"].astype(np.int64) + 1          # [v][r]
    # list order inside a group of 16 kept rows: position kq * 4 + t holds kept row 4 t + kq
    r = np.arange(16)
    perm = 4 * (r % 4) + r // 4
    return rows.reshape(Q, G, 16)[:, :, perm].reshape(-1).astype(np.int32)


@pytest.mark.parametrize("n,m", [(2, 4), (3, 8), (2, 8), (1, 8), (16, 32), (12, 32), (8, 32), (4, 32), (32, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_row_list_equals_the_generators_global_rows(oracle, n, m, Ns):
    d = datagen.init_data(4, 256, 512, n, m, seed=n * 100 + m + Ns)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    got = oracle.row_index(D, cinfo, d["W"], d["N"], window, kept, Ns)
    assert np.array_equal(got, expected_list(d))


def test_a_reduction_that_is_not_whole_groups(oracle):
    """3:8 with K = 96: W = 36 kept rows, two full groups and one of four rows; the other twelve
    entries of the last group are 0."""
    d = datagen.init_data(4, 128, 96, 3, 8, seed=5)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    got = oracle.row_index(D, cinfo, d["W"], d["N"], window, kept, 128)
    assert d["W"] == 36 and got.size == 4 * 3 * 16
    assert np.array_equal(got, expected_list(d))
    assert (got.reshape(4, 3, 16)[:, 2, :] == 0).sum() == 4 * 12
