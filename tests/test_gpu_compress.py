"""GPU parity of the dense <-> N:M vector-sparse conversion, through the C-ABI: values and indices
bit-exact against the CPU checker, round trips at full size, and the whole chain
compress -> transIndex -> preprocess -> multiply against a dense fp64 product."""
import numpy as np
import pytest

from conftest import REL_TOL, datagen, kernel_geometry, nmspmm, scaled_max_error

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def compress_gpu(dense, n, m, vl=32):
    K, N = dense.shape
    W = K // m * n
    BT = torch.full((W, N), float("nan"), dtype=torch.float32, device="cuda")
    DT = torch.full((W, N // vl), -7, dtype=torch.int32, device="cuda")
    nmspmm.compress_device(dense, K, N, n, m, BT, DT, vl)
    return BT, DT


@pytest.mark.parametrize("K,N,n,m,vl", [
    (64, 128, 2, 4, 32), (256, 512, 2, 4, 32), (512, 1120, 1, 8, 32), (256, 96, 3, 8, 32), (128, 288, 2, 8, 32),
    (128, 256, 4, 32, 32), (64, 64, 8, 32, 32), (96, 160, 12, 16, 32), (64, 64, 2, 4, 4), (64, 264, 1, 8, 8),
    (128, 48, 5, 16, 16), (64, 36, 3, 4, 4), (32, 40, 17, 32, 8),
    # 32-row windows with 32-column vectors (the kernels that cut the window into quarters): one kept
    # row, nearly all, a column count that leaves the last workgroup with one live vector of eight
    (96, 1120, 1, 32, 32), (64, 288, 31, 32, 32), (160, 2080, 16, 32, 32), (32, 32, 12, 32, 32),
])
def test_compress_bit_exact_vs_checker(oracle, K, N, n, m, vl):
    rng = np.random.default_rng(K + N + n)
    host = rng.standard_normal((K, N), dtype=np.float32)
    host[rng.random((K, N)) < 0.05] = 0.0
    BT, DT = compress_gpu(torch.from_numpy(host).cuda(), n, m, vl)
    want_BT, want_DT = oracle.compress(host, n, m, vl)
    assert np.array_equal(DT.cpu().numpy(), want_DT)
    assert np.array_equal(BT.cpu().numpy(), want_BT)


def test_ties_and_non_finite_scores(oracle):
    K, N, n, m = 32, 64, 3, 8
    host = np.ones((K, N), np.float32)
    host[1::2] *= -1.0
    host[13, 5] = np.inf
    host[22, 40] = np.nan
    BT, DT = compress_gpu(torch.from_numpy(host).cuda(), n, m)
    want_BT, want_DT = oracle.compress(host, n, m)
    assert np.array_equal(DT.cpu().numpy(), want_DT)
    assert np.array_equal(BT.cpu().numpy(), want_BT, equal_nan=True)
    assert want_DT[3:6, 0].tolist() == [0, 1, 5] and want_DT[6:9, 1].tolist() == [0, 1, 6]


def test_ties_and_non_finite_scores_in_32_row_windows(oracle):
    """Equal scores in different quarters of a window (the quarters are ranked by different waves)
    must still prefer the lower row; NaN and Inf scores rank above everything."""
    K, N, n, m = 64, 96, 5, 32
    host = np.ones((K, N), np.float32)
    host[::3] *= -1.0
    host[7, 40] = np.inf
    host[29, 70] = np.nan
    host[40:44, :32] = 2.0      # four equal larger rows in the second window's second quarter
    BT, DT = compress_gpu(torch.from_numpy(host).cuda(), n, m)
    want_BT, want_DT = oracle.compress(host, n, m)
    assert np.array_equal(DT.cpu().numpy(), want_DT)
    assert np.array_equal(BT.cpu().numpy(), want_BT, equal_nan=True)
    assert want_DT[:5, 0].tolist() == [0, 1, 2, 3, 4] and want_DT[5:10, 0].tolist() == [0, 8, 9, 10, 11]
    back = torch.empty((K, N), dtype=torch.float32, device="cuda")
    nmspmm.decompress_device(BT, DT, K, N, n, m, back)
    torch.cuda.synchronize()
    want_back = oracle.decompress(np.ascontiguousarray(want_BT.T).reshape(-1),
                                  np.ascontiguousarray((want_DT + (np.arange(want_DT.shape[0]) // n * m)[:, None]).T.astype(np.int32)).reshape(-1),
                                  K, N, want_BT.shape[0])
    assert np.array_equal(back.cpu().numpy(), want_back, equal_nan=True)


@pytest.mark.parametrize("n,m", [(2, 4), (3, 8), (2, 8), (1, 8), (8, 32)])
def test_round_trips_at_full_size(n, m):
    K = N = 4096
    g = torch.Generator(device="cuda").manual_seed(100 * n + m)
    dense = torch.randn((K, N), generator=g, dtype=torch.float32, device="cuda")
    BT, DT = compress_gpu(dense, n, m)
    # indices: ascending inside each window, inside the window
    d = DT.view(K // m, n, N // 32)
    assert int(d.min()) >= 0 and int(d.max()) < m
    if n > 1:
        assert bool((d[:, 1:] > d[:, :-1]).all())
    # expansion keeps exactly the selected rows and zeroes the rest
    back = torch.full((K, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.decompress_device(BT, DT, K, N, n, m, back)
    keep_rows = torch.zeros((K // m, m, N // 32), dtype=torch.bool, device="cuda")
    keep_rows.scatter_(1, d.long(), True)
    kept = keep_rows[..., None].expand(-1, -1, -1, 32).reshape(K, N)
    assert int(keep_rows.sum()) == K // m * n * (N // 32)
    assert torch.equal(back, torch.where(kept, dense, torch.zeros_like(dense)))
    # kept rows dominate dropped rows (fp64 score; fp32 pairwise rounding allowed for)
    score = dense.double().abs().view(K // m, m, N // 32, 32).sum(3)
    inf = torch.tensor(float("inf"), dtype=torch.float64, device="cuda")
    worst_kept = torch.where(keep_rows, score, inf).amin(1)
    best_dropped = torch.where(keep_rows, -inf, score).amax(1)
    assert bool((worst_kept >= best_dropped * (1 - 1e-5)).all())
    # compressing the expansion again changes nothing
    BT2, DT2 = compress_gpu(back, n, m)
    assert torch.equal(DT2, DT) and torch.equal(BT2, BT)


def test_decompress_bit_exact_vs_generator(oracle):
    for (K, N, n, m, vl) in ((256, 512, 2, 4, 32), (128, 96, 1, 8, 32), (64, 64, 2, 4, 4), (128, 192, 3, 8, 8),
                             (128, 96, 8, 32, 32), (64, 320, 4, 32, 32), (96, 2080, 16, 32, 32), (64, 32, 12, 32, 32),
                             (64, 544, 31, 32, 32), (64, 1056, 7, 8, 16), (64, 48, 4, 16, 4), (96, 64, 9, 32, 8)):
        d = datagen.init_data(4, N, K, n, m, vec_len=vl, seed=K + n)
        back = torch.empty((K, N), dtype=torch.float32, device="cuda")
        nmspmm.decompress_device(torch.from_numpy(d["BT"]).cuda(), torch.from_numpy(d["DT"]).cuda(), K, N, n, m, back, vl)
        want = oracle.decompress(d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), K, N, d["W"], vl)
        assert np.array_equal(back.cpu().numpy(), want)


@pytest.mark.parametrize("K,N,n,m,vl", [(64, 96, 2, 8, 32), (128, 1088, 8, 32, 32), (64, 320, 5, 32, 32), (64, 64, 3, 4, 4)])
def test_decompress_scatters_by_index(K, N, n, m, vl):
    """The expansion puts compressed row p of a window where its index says (the checker's scatter,
    oracle/nm_oracle.cpp nm_oracle_decompress): the indices of a window need not ascend.  An index
    outside the window stores nothing; the row it would have named stays zero."""
    rng = np.random.default_rng(K + N + n)
    W, Q, nwin = K // m * n, N // vl, K // m
    BT = rng.uniform(-1, 1, (W, N)).astype(np.float32)
    DT = np.empty((W, Q), dtype=np.int32)
    for w in range(nwin):
        for a in range(Q):
            DT[w * n:(w + 1) * n, a] = rng.permutation(m)[:n]          # distinct, in no order
    bad = rng.random((W, Q)) < 0.1
    DT_bad = np.where(bad, rng.choice([-1, m, m + 7, 1 << 20, -(1 << 31)], size=(W, Q)), DT).astype(np.int32)
    for table in (DT, DT_bad):
        want = np.zeros((K, N), dtype=np.float32)
        for w in range(nwin):
            for p in range(n):
                for a in range(Q):
                    r = int(table[w * n + p, a])
                    if 0 <= r < m:
                        want[w * m + r, a * vl:(a + 1) * vl] = BT[w * n + p, a * vl:(a + 1) * vl]
        back = torch.full((K, N), float("nan"), dtype=torch.float32, device="cuda")
        guard = torch.full((8, N), 7.0, dtype=torch.float32, device="cuda")   # allocated right behind: must stay
        nmspmm.decompress_device(torch.from_numpy(BT).cuda(), torch.from_numpy(table).cuda(), K, N, n, m, back, vl)
        torch.cuda.synchronize()
        assert np.array_equal(back.cpu().numpy(), want)
        assert bool((guard == 7.0).all())


@pytest.mark.parametrize("n,m", [(2, 4), (1, 8)])
def test_compress_preprocess_multiply_chain(n, m):
    M, K, N, Ns = 256, 1024, 512, 128
    g = torch.Generator(device="cuda").manual_seed(7 + n)
    dense = torch.randn((K, N), generator=g, dtype=torch.float32, device="cuda")
    A = torch.randn((K, M), generator=g, dtype=torch.float32, device="cuda")      # column-major M x K
    BT, DT = compress_gpu(dense, n, m)
    W, Q = BT.shape[0], N // 32
    window, kept, times = kernel_geometry(n, m)
    pn, pm = n, m
    DT = DT.reshape(-1).contiguous()
    for _ in range(times):
        pn, pm = nmspmm.trans_index_device(DT, W, N, Q, pn, pm)
    D = torch.empty_like(DT)
    cinfo = None
    if window == 64:
        cinfo = torch.empty(nmspmm.column_info_ints(W, pn, pm, N, Ns), dtype=torch.int32, device="cuda")
        nmspmm.preprocess_high_device(cinfo, pm, pn, DT, D, W, Q, N, Ns)
    else:
        nmspmm.preprocess_low_device(DT, D, W, Q, Ns)
    C = torch.empty((M, N), dtype=torch.float32, device="cuda")
    nmspmm.spmm(A, BT, D, cinfo, C, M, N, K, W, window, kept, 32, Ns, 1, None)
    pruned = torch.empty_like(dense)
    nmspmm.decompress_device(BT, compress_gpu(dense, n, m)[1], K, N, n, m, pruned)
    want = (A.t().double() @ pruned.double()).cpu().numpy()
    assert scaled_max_error(C.cpu().numpy(), want) <= REL_TOL


def test_bad_arguments_are_rejected():
    x = torch.zeros((64, 64), dtype=torch.float32, device="cuda")
    # buffers large enough for every case, so that the library's own checks are what refuses them
    bt = torch.zeros((64, 64), dtype=torch.float32, device="cuda")
    dt = torch.zeros((64, 64), dtype=torch.int32, device="cuda")
    for (K, N, n, m, vl) in ((64, 64, 4, 4, 32), (64, 64, 0, 4, 32), (64, 64, 2, 5, 32), (64, 64, 2, 4, 3), (63, 64, 2, 4, 32),
                             (64, 48, 2, 4, 32)):
        with pytest.raises(nmspmm.NmSpmmError):
            nmspmm.compress_device(x, K, N, n, m, bt, dt, vl)
        with pytest.raises(nmspmm.NmSpmmError):
            nmspmm.decompress_device(bt, dt, K, N, n, m, x, vl)
