"""GPU parity on seeded random shapes, through the C-ABI, against the CPU checker: row counts,
column counts, reduction lengths, patterns, column-block widths, vector lengths, reduction splits
and both storage orders of A drawn at random, so that combinations nobody listed by hand are
exercised too.  Same tolerance as the hand-picked cases (1e-4, scaled max error)."""
import os
import random

import numpy as np
import pytest

from conftest import REL_TOL, datagen, kernel_geometry, nmspmm, preprocess_with_oracle, scaled_max_error

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

LONG_PATTERNS = [(2, 4), (3, 8), (2, 8), (1, 8), (16, 32), (12, 32), (8, 32), (4, 32), (32, 32)]
SHORT_PATTERNS = [(2, 4), (1, 4), (3, 4), (1, 8), (2, 8), (3, 8), (4, 8)]
MAX_MACS = 1.2e8  # keeps the scalar checker at a fraction of a second per case
# NMSPMM_TEST_SEED=<n> draws another set of problems (the default set is the one every run checks)
SEED = int(os.environ.get("NMSPMM_TEST_SEED", "0")) * 100000


def draw_case(rng):
    """One random problem: (M, N, K, n, m, vec_len, Ns, split_k, row_major)."""
    while True:
        vec_len = rng.choice([32, 32, 32, 32, 16, 8, 4])
        n, m = rng.choice(LONG_PATTERNS if vec_len == 32 else SHORT_PATTERNS)
        Ns = rng.choice([128, 128, 64, 32])
        if vec_len < 32:
            window, kept = m, n
            k_unit = m
            N = Ns * rng.randint(1, 768 // Ns)
        else:
            window, kept, _ = kernel_geometry(n, m)
            k_unit = window
            N = Ns * rng.randint(1, 1024 // Ns)
        K = k_unit * rng.randint(1, 1536 // k_unit)
        M = rng.choice([rng.randint(1, 32), rng.randint(33, 128), rng.randint(129, 640)])
        W = K // window * kept
        if M * N * W > MAX_MACS:
            continue
        nwin = K // k_unit
        split_k = min(rng.choice([1, 1, 1, 2, 3, 5, 8]), nwin)
        row_major = vec_len == 32 and rng.random() < 0.3
        return M, N, K, n, m, vec_len, Ns, split_k, row_major


CASES = [draw_case(random.Random(SEED + 7000 + i)) for i in range(400)]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("case", CASES, ids=lambda c: "M%d-N%d-K%d-%dof%d-L%d-Ns%d-s%d-%s" % (c[:8] + ("rm" if c[8] else "cm",)))
def test_random_shape(oracle, case):
    M, N, K, n, m, vec_len, Ns, split_k, row_major = case
    d = datagen.init_data(M, N, K, n, m, vec_len=vec_len, seed=M * 31 + N + K + n)
    W = d["W"]
    if vec_len == 32:
        window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    else:
        window, kept, cinfo = m, n, None
        D = d["DT"].reshape(-1).copy()
        oracle.preprocess_low(D, W, d["Q"], Ns, vec_len)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    dcinfo = None if cinfo is None else dev(cinfo)
    if row_major:
        ws = torch.full((nmspmm.workspace_bytes_rowmajor(M, N, K, split_k) // 4,), float("nan"), dtype=torch.float32,
                        device="cuda")
        nmspmm.spmm_rowmajor(dev(d["A_km"].T), dev(d["BT"]), dev(D), dcinfo, C, M, N, K, W, window, kept, ws, vec_len,
                             Ns, split_k)
    else:
        ws = None
        if split_k > 1:
            ws = torch.full((nmspmm.workspace_bytes(M, N, split_k) // 4,), float("nan"), dtype=torch.float32, device="cuda")
        nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), dcinfo, C, M, N, K, W, window, kept, vec_len, Ns, split_k, ws)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() in ("mfma", "skinny", "short", "gather", "simt")
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, W,
                           vec_len).reshape(M, N)
    got = C.cpu().numpy()
    assert np.isfinite(got).all()
    assert scaled_max_error(got, want) <= REL_TOL


def draw_decode_case(rng, rows=(1, 32), row_major_share=0.3):
    """One random decode-sized problem on the row list: (M, N, K, n, m, Ns, flags, row_major, accumulate)."""
    while True:
        n, m = rng.choice([(2, 4), (3, 8), (2, 8), (1, 8), (8, 32), (4, 32)])
        window, kept, _ = kernel_geometry(n, m)
        Ns = rng.choice([128, 64, 32])
        N = Ns * rng.randint(1, 2048 // Ns)
        K = window * rng.choice([rng.randint(1, 24), rng.randint(24, 16384 // window)])
        M = rng.randint(*rows)
        W = K // window * kept
        if M * N * W > MAX_MACS:
            continue
        flags = rng.choice([0, 0, 2, 4, 4, 6])
        return M, N, K, n, m, Ns, flags, rng.random() < row_major_share, rng.random() < 0.3


# up to 32 rows the row list always takes the decode kernel; 33 to 64 rows (column-major A) it does
# where the library expects it to beat the tile kernel
DECODE_CASES = ([draw_decode_case(random.Random(SEED + 9000 + i)) for i in range(120)] +
                [draw_decode_case(random.Random(SEED + 9500 + i), (33, 64), 0.0) for i in range(60)])


@pytest.mark.parametrize("case", DECODE_CASES,
                         ids=lambda c: "M%d-N%d-K%d-%dof%d-Ns%d-f%d-%s-%s" % (c[:7] + ("rm" if c[7] else "cm", "acc" if c[8] else "st")))
def test_random_decode_shape(oracle, case):
    """Up to 64 rows on the row list, with the stream hint and the cut reductions drawn at random
    (long reductions on few column vectors are among the cases, so the cut is taken), both storage
    orders of A, storing and adding to C."""
    M, N, K, n, m, Ns, flags, row_major, accumulate = case
    d = datagen.init_data(M, N, K, n, m, seed=M * 17 + N + K + n, dist="normal", b_scale=0.05)
    W = d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    dD, dcinfo = dev(D), None if cinfo is None else dev(cinfo)
    R = torch.empty(nmspmm.row_index_ints(W, N), dtype=torch.int32, device="cuda")
    nmspmm.row_index_device(dD, dcinfo, W, N, window, kept, Ns, R)
    C0 = np.random.default_rng(M + N).standard_normal((M, N)).astype(np.float32) if accumulate else None
    C = dev(C0) if accumulate else torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    split_k = 2 if accumulate and K // window >= 2 else 1
    if accumulate and split_k == 1:
        C0 = None
        C.fill_(float("nan"))
    if accumulate and split_k > 1:
        flags |= nmspmm.ACCUMULATE
    if row_major:
        ws = torch.full((nmspmm.workspace_bytes_rowmajor(M, N, K, split_k) // 4,), float("nan"), dtype=torch.float32,
                        device="cuda")
        nmspmm.spmm_rowmajor(dev(d["A_km"].T), dev(d["BT"]), dD, dcinfo, C, M, N, K, W, window, kept, ws, 32, Ns, split_k,
                             R, flags)
    else:
        ws = None
        if split_k > 1:
            ws = torch.full((nmspmm.workspace_bytes(M, N, split_k) // 4,), float("nan"), dtype=torch.float32, device="cuda")
        nmspmm.spmm_ex(dev(d["A_km"]), dev(d["BT"]), dD, dcinfo, C, M, N, K, W, window, kept, 32, Ns, split_k, ws, flags, R)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() in (("decode",) if M <= 32 else ("decode", "mfma", "skinny"))
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, W, 32,
                           C=None if C0 is None else C0.reshape(-1).copy()).reshape(M, N)
    got = C.cpu().numpy()
    assert np.isfinite(got).all()
    assert scaled_max_error(got, want) <= REL_TOL
