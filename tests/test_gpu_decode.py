"""The row list (the decode-oriented index format) and the decode kernel that reads it, on the GPU
through the C-ABI.  The list must equal the checker's bit for bit; the multiplication must match
the checker's restatement of the reference's nmGEMM_on_cpu within the scaled max error 1e-4."""
import numpy as np
import pytest

from conftest import REL_TOL, datagen, nmspmm, preprocess_with_oracle, scaled_max_error

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def gpu_row_list(D, cinfo, W, N, window, kept, Ns):
    R = torch.full((nmspmm.row_index_ints(W, N),), -77, dtype=torch.int32, device="cuda")
    nmspmm.row_index_device(dev(D), None if cinfo is None else dev(cinfo), W, N, window, kept, Ns, R)
    torch.cuda.synchronize()
    return R


def want_c(oracle, d, C0=None):
    return oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), d["M"], d["N"], d["W"],
                           C=None if C0 is None else C0.reshape(-1).copy()).reshape(d["M"], d["N"])


def run_decode(oracle, d, Ns=128, flags=0, split_k=1, C0=None):
    M, N, K, W = d["M"], d["N"], d["K"], d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    R = gpu_row_list(D, cinfo, W, N, window, kept, Ns)
    assert np.array_equal(R.cpu().numpy(), oracle.row_index(D, cinfo, W, N, window, kept, Ns))
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda") if C0 is None else dev(C0)
    ws = None
    if split_k > 1:
        ws = torch.empty(nmspmm.workspace_bytes(M, N, split_k) // 4, dtype=torch.float32, device="cuda")
    nmspmm.spmm_ex(dev(d["A_km"]), dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, W, window,
                   kept, 32, Ns, split_k, ws, flags, R)
    torch.cuda.synchronize()
    return C.cpu().numpy(), nmspmm.last_kernel()


@pytest.mark.parametrize("n,m", [(2, 4), (3, 8), (2, 8), (1, 8), (16, 32), (12, 32), (8, 32), (4, 32), (32, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_row_list_bit_exact_every_pattern_and_block_width(oracle, n, m, Ns):
    d = datagen.init_data(4, 512, 1024, n, m, seed=n + m + Ns)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    got = gpu_row_list(D, cinfo, d["W"], d["N"], window, kept, Ns).cpu().numpy()
    assert np.array_equal(got, oracle.row_index(D, cinfo, d["W"], d["N"], window, kept, Ns))
    # and, independently of the checker, the generator's own global rows
    assert np.array_equal(np.sort(got.reshape(d["Q"], -1), axis=1)[:, -d["W"]:], np.sort(d["D_cm"] + 1, axis=1))


@pytest.mark.parametrize("N,K,n,m", [(8192, 8192, 1, 8), (8192, 8192, 2, 8), (14336, 4096, 1, 8), (14336, 4096, 2, 8),
                                     (4096, 11008, 2, 8), (4096, 4096, 3, 8)])
def test_row_list_bit_exact_at_full_size(oracle, N, K, n, m):
    d = datagen.init_data(1, N, K, n, m, seed=N + K + n)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    got = gpu_row_list(D, cinfo, d["W"], N, window, kept, 128).cpu().numpy()
    assert np.array_equal(got, oracle.row_index(D, cinfo, d["W"], N, window, kept, 128))


@pytest.mark.parametrize("M", [1, 2, 7, 8, 13, 16, 17, 24, 31, 32, 33, 34, 39, 48, 57, 62, 63, 64])
@pytest.mark.parametrize("n,m,K", [(1, 8, 1024), (2, 8, 1088), (2, 4, 1152), (3, 8, 96), (3, 8, 1120), (32, 32, 160), (4, 32, 960)])
def test_decode_kernel_every_row_count(oracle, M, n, m, K):
    """Row counts on both sides of 16, 32 and 64, odd ones included (17 to 32 rows take one 64-bit
    load of A per k-step when the row count is even, two 32-bit loads when it is odd, 33 to 64 rows
    one 128-bit load whatever the count); reductions that give the 16 waves of a workgroup unequal
    shares, some none, and (3:8 with K = 96: 36 kept rows) a last group of four rows."""
    d = datagen.init_data(M, 256, K, n, m, seed=M + K, dist="normal", b_scale=0.02)
    got, fam = run_decode(oracle, d)
    assert fam == "decode"
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M", [1, 3, 9, 16, 19, 26, 33, 41, 50, 61])
@pytest.mark.parametrize("n,m,K", [(2, 8, 1088), (3, 8, 96), (1, 8, 2048)])
def test_nothing_outside_a_leaks_into_c(oracle, M, n, m, K):
    """The lanes of a 16-row tile whose row of C does not exist read the last row that does, and
    the last group of a reduction that is not whole groups has entries without a row: neither may
    bring anything from outside A into C.  A lies in the middle of a buffer of NaNs."""
    d = datagen.init_data(M, 128, K, n, m, seed=3 * M + K, dist="normal", b_scale=0.02)
    N, W = d["N"], d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    R = gpu_row_list(D, cinfo, W, N, window, kept, 128)
    pad = 4096
    buf = torch.full((2 * pad + K * M,), float("nan"), dtype=torch.float32, device="cuda")
    buf[pad:pad + K * M] = dev(d["A_km"]).reshape(-1)
    A = buf[pad:pad + K * M]
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm_ex(A, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, W, window, kept, 32, 128,
                   1, None, 0, R)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "decode"
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL
    # and on the reference layout (no list)
    C.fill_(float("nan"))
    nmspmm.spmm(A, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, W, window, kept, 32, 128, 1, None)
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("Ns", [64, 32])
@pytest.mark.parametrize("M,n,m", [(5, 1, 8), (32, 2, 8), (16, 2, 4)])
def test_decode_kernel_with_lists_from_other_block_widths(oracle, Ns, M, n, m):
    d = datagen.init_data(M, 512, 512, n, m, seed=M + Ns)
    got, fam = run_decode(oracle, d, Ns=Ns)
    assert fam == "decode"
    assert scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M", [1, 8, 16, 32])
@pytest.mark.parametrize("n,m", [(1, 8), (2, 8)])
@pytest.mark.parametrize("K,N", [(8192, 8192), (4096, 14336)])
def test_decode_shapes_at_full_size_on_the_row_list(oracle, M, n, m, K, N):
    """The sixteen decode cases at full size, all of C against the checker, with and without the
    non-temporal hint for B (with the hint the reduction may be cut between the waves differently,
    so the two results agree to the tolerance, not to the bit)."""
    d = datagen.init_data(M, N, K, n, m, seed=140 + M + n, dist="normal", b_scale=0.02)
    got, fam = run_decode(oracle, d)
    assert fam == "decode"
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL
    streamed, fam = run_decode(oracle, d, flags=nmspmm.STREAM_B)
    assert fam == "decode" and np.isfinite(streamed).all()
    assert scaled_max_error(streamed, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M", [3, 16, 20, 32])
def test_decode_kernel_adds_to_c_when_asked_like_a_split_call_of_the_reference(oracle, M):
    """split_k has no effect on how this kernel computes (one launch, reduction in the workgroup),
    but a split call with NMSPMM_ACCUMULATE still adds to C, as the reference's split calls do."""
    d = datagen.init_data(M, 256, 1024, 2, 8, seed=M)
    rng = np.random.default_rng(M)
    C0 = rng.uniform(-3.0, 3.0, (M, 256)).astype(np.float32)
    got, fam = run_decode(oracle, d, flags=nmspmm.ACCUMULATE, split_k=4, C0=C0)
    assert fam == "decode" and scaled_max_error(got, want_c(oracle, d, C0)) <= REL_TOL
    got, _ = run_decode(oracle, d, flags=nmspmm.ACCUMULATE, split_k=1, C0=C0)
    assert scaled_max_error(got, want_c(oracle, d)) <= REL_TOL
    got, _ = run_decode(oracle, d, flags=0, split_k=4, C0=C0)
    assert scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M,N", [(200, 256), (129, 256), (65, 8192), (128, 8192)])
def test_larger_row_counts_ignore_the_list(oracle, M, N):
    """More than 128 rows, and 65 to 128 rows on more column vectors than their 32-row parts could
    share the compute units with."""
    d = datagen.init_data(M, N, 512, 2, 8, seed=3)
    got, fam = run_decode(oracle, d)
    assert fam in ("skinny", "mfma")
    assert scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M", [65, 77, 96, 100, 127, 128])
@pytest.mark.parametrize("n,m,K,N", [(2, 8, 1088, 256), (1, 8, 2048, 512), (2, 4, 1152, 2048), (3, 8, 96, 128)])
def test_65_to_128_rows_on_few_column_vectors_are_cut_into_parts(oracle, M, n, m, K, N):
    """With at most 64 column vectors (2048 columns) 65 to 128 rows run as 32-row parts on the row
    list, one workgroup per vector and part; the last part may be short or odd."""
    d = datagen.init_data(M, N, K, n, m, seed=M + K, dist="normal", b_scale=0.02)
    got, fam = run_decode(oracle, d)
    assert fam == "decode"
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M", [48, 64])
@pytest.mark.parametrize("n,m,K", [(1, 8, 8192), (2, 8, 8192), (1, 8, 256), (2, 8, 256)])
def test_33_to_64_rows_on_8192_columns_on_the_row_list(oracle, M, n, m, K):
    """Ncols = 8192 (one workgroup per vector fills the GPU, so the rows are not cut into parts), all
    of C against the checker, with and without the non-temporal hint.  With a short reduction the
    library takes the decode kernel's four-halves form; at K = 8192 that form and the tile kernel
    are within a few per cent of each other and either may be chosen."""
    d = datagen.init_data(M, 8192, K, n, m, seed=150 + M + n, dist="normal", b_scale=0.02)
    got, fam = run_decode(oracle, d)
    assert fam == "decode" if K == 256 else fam in ("decode", "mfma")
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL
    streamed, fam = run_decode(oracle, d, flags=nmspmm.STREAM_B)
    assert fam in ("decode", "mfma") and scaled_max_error(streamed, want_c(oracle, d)) <= REL_TOL


def test_a_list_off_a_sixteen_byte_boundary_is_rejected(oracle):
    d = datagen.init_data(4, 128, 256, 2, 8, seed=1)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    base = torch.zeros(nmspmm.row_index_ints(d["W"], 128) + 1, dtype=torch.int32, device="cuda")
    C = torch.zeros((4, 128), dtype=torch.float32, device="cuda")
    with pytest.raises(nmspmm.NmSpmmError, match="ALIGNMENT"):
        nmspmm.spmm_ex(dev(d["A_km"]), dev(d["BT"]), dev(D), dev(cinfo), C, 4, 128, 256, d["W"], window, kept, 32, 128, 1,
                       None, 0, base[1:])


def test_decode_kernel_with_131072_column_vectors(oracle):
    """Ncols = 2^22: 131072 workgroups, B rows 16 MiB apart."""
    M, N, K = 4, 1 << 22, 64
    d = datagen.init_data(M, N, K, 2, 4, seed=4445, dist="normal", b_scale=0.02)
    got, fam = run_decode(oracle, d)
    assert fam == "decode"
    assert scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M,n,m", [(8, 1, 8), (32, 2, 8), (50, 2, 8), (64, 1, 8)])
def test_graph_replays_of_the_decode_kernel_equal_eager_calls(oracle, M, n, m):
    N, K = 512, 1024
    d = datagen.init_data(M, N, K, n, m, seed=M, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    R = gpu_row_list(D, cinfo, d["W"], N, window, kept, 128)
    A, B, Dd, ci = dev(d["A_km"]), dev(d["BT"]), dev(D), dev(cinfo)
    C_g = torch.empty((M, N), dtype=torch.float32, device="cuda")
    C_e = torch.empty_like(C_g)

    def call(C):
        nmspmm.spmm_ex(A, B, Dd, ci, C, M, N, K, d["W"], window, kept, 32, 128, 1, None, 0, R)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(C_g)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(C_g)
    for rep in range(3):
        A.mul_(1.25)
        C_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        call(C_e)
        torch.cuda.synchronize()
        assert nmspmm.last_kernel() == "decode"
        assert torch.isfinite(C_g).all().item() and torch.equal(C_g, C_e), "replay %d" % rep


@pytest.mark.parametrize("M", [1, 3, 8, 9, 16, 21, 32])
@pytest.mark.parametrize("n,m", [(1, 8), (2, 4)])
def test_row_major_activations_on_the_row_list(oracle, M, n, m):
    """nmspmm_spmm_rowmajor_ex with the row list: up to 8 rows the decode kernel reads the
    row-major A in place, above that the column-major copy in the workspace (pitch padded to four
    floats for odd row counts)."""
    N, K = 256, 1024
    d = datagen.init_data(M, N, K, n, m, seed=M + n, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    R = gpu_row_list(D, cinfo, d["W"], N, window, kept, 128)
    A_rm = dev(d["A_km"].T)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.full((nmspmm.workspace_bytes_rowmajor(M, N, K, 1) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm_rowmajor(A_rm, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, d["W"], window,
                         kept, ws, 32, 128, 1, R)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "decode"
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and scaled_max_error(got, want_c(oracle, d)) <= REL_TOL


@pytest.mark.parametrize("M", [1, 7, 16, 19, 32, 45, 64])
@pytest.mark.parametrize("n,m,K,N", [(2, 8, 11008, 4096), (2, 8, 8192, 2048), (1, 8, 16384, 1024), (2, 4, 4096, 4096), (2, 4, 16384, 1024), (3, 8, 8192, 2048)])
def test_reductions_cut_across_workgroups(oracle, M, n, m, K, N):
    """NMSPMM_DECODE_SPLIT with fewer column vectors than compute units and a long reduction: two to
    eight workgroups per vector, the last one to arrive adds the partial tiles up.  Against the
    checker; then forty more launches, every one bit-identical to the first (the sum is taken in
    slice order whoever arrives last, and the arrival counters are left at zero)."""
    d = datagen.init_data(M, N, K, n, m, seed=M + K // 64, dist="normal", b_scale=0.02)
    W = d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    R = gpu_row_list(D, cinfo, W, N, window, kept, 128)
    A, B, Dd = dev(d["A_km"]), dev(d["BT"]), dev(D)
    ci = None if cinfo is None else dev(cinfo)
    want = want_c(oracle, d)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm_ex(A, B, Dd, ci, C, M, N, K, W, window, kept, 32, 128, 1, None, nmspmm.DECODE_SPLIT, R)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "decode"
    first = C.clone()
    assert np.isfinite(first.cpu().numpy()).all() and scaled_max_error(first.cpu().numpy(), want) <= REL_TOL
    for _ in range(40):
        C.fill_(float("nan"))
        nmspmm.spmm_ex(A, B, Dd, ci, C, M, N, K, W, window, kept, 32, 128, 1, None, nmspmm.DECODE_SPLIT, R)
    torch.cuda.synchronize()
    assert torch.equal(C, first)
    # the same call without the flag (one workgroup per vector) agrees within the bound
    nmspmm.spmm_ex(A, B, Dd, ci, C, M, N, K, W, window, kept, 32, 128, 1, None, 0, R)
    torch.cuda.synchronize()
    assert scaled_max_error(C.cpu().numpy(), want) <= REL_TOL
    # with the hint for streamed weights, and adding to C like a split call of the reference
    C0 = np.random.default_rng(M).standard_normal((M, N)).astype(np.float32)
    Cd = dev(C0)
    ws = torch.empty(nmspmm.workspace_bytes(M, N, 2) // 4, dtype=torch.float32, device="cuda")
    nmspmm.spmm_ex(A, B, Dd, ci, Cd, M, N, K, W, window, kept, 32, 128, 2, ws,
                   nmspmm.DECODE_SPLIT | nmspmm.STREAM_B | nmspmm.ACCUMULATE, R)
    torch.cuda.synchronize()
    assert scaled_max_error(Cd.cpu().numpy(), want_c(oracle, d, C0)) <= REL_TOL


def test_the_split_flag_changes_nothing_where_every_compute_unit_has_a_vector(oracle):
    """8192 columns are 256 vectors: nothing to gain, the flag is ignored and the result is the
    unsplit kernel's bit for bit."""
    M, N, K, n, m = 8, 8192, 2048, 2, 8
    d = datagen.init_data(M, N, K, n, m, seed=11, dist="normal", b_scale=0.02)
    W = d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    R = gpu_row_list(D, cinfo, W, N, window, kept, 128)
    A, B, Dd, ci = dev(d["A_km"]), dev(d["BT"]), dev(D), dev(cinfo)
    C1 = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    C2 = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm_ex(A, B, Dd, ci, C1, M, N, K, W, window, kept, 32, 128, 1, None, 0, R)
    nmspmm.spmm_ex(A, B, Dd, ci, C2, M, N, K, W, window, kept, 32, 128, 1, None, nmspmm.DECODE_SPLIT, R)
    torch.cuda.synchronize()
    assert torch.equal(C1, C2)


@pytest.mark.parametrize("M,N,K,n,m", [(136, 4096, 2048, 2, 4), (137, 4096, 4096, 2, 4), (150, 4096, 2048, 32, 32), (160, 4096, 4096, 2, 8),
                                       (280, 8192, 2048, 3, 8), (288, 8192, 2048, 2, 8), (520, 11008, 4096, 1, 8)])
@pytest.mark.parametrize("with_list", [False, True])
@pytest.mark.parametrize("Ns", [128, 32])
def test_last_rows_of_a_tile_kernel_call_on_the_decode_sized_kernels(oracle, M, N, K, n, m, with_list, Ns):
    """Row counts 8 to 32 above a multiple of 128 where the library expects an extra layer of 128-row
    workgroups to cost more than reading B again: the rows up to the multiple run on the tile kernel,
    the last ones on the decode kernel (with the row list) or the kernel on the reference layout
    (without).  Every row against the checker, the seam included; nothing outside C's M rows is
    written."""
    d = datagen.init_data(M, N, K, n, m, seed=M + N + K)
    W = d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    apart = nmspmm.rows_apart(M, N, W, kept)
    assert 8 <= apart <= 32 and apart == M % 128
    R = gpu_row_list(D, cinfo, W, N, window, kept, Ns) if with_list else None
    guard = 64
    Cbuf = torch.full(((M + guard) * N,), float("nan"), dtype=torch.float32, device="cuda")
    C = Cbuf[: M * N].view(M, N)
    nmspmm.spmm_ex(dev(d["A_km"]), dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, W, window,
                   kept, 32, Ns, 1, None, 0, R)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() in ("mfma", "skinny", "decode")
    assert bool(torch.isfinite(C).all()) and bool(torch.isnan(Cbuf[M * N:]).all())
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, W).reshape(M, N)
    assert scaled_max_error(C.cpu().numpy(), want) <= REL_TOL
    assert scaled_max_error(C[M - apart:].cpu().numpy(), want[M - apart:]) <= REL_TOL


@pytest.mark.parametrize("M,N,K,n,m", [(137, 4096, 4096, 2, 4), (150, 4096, 2048, 32, 32), (281, 8192, 2048, 3, 8)])
def test_last_rows_apart_with_row_major_activations(oracle, M, N, K, n, m):
    """The same hand-over behind the row-major entry point: the copy of A has a pitch of M rounded up
    to four floats, and the last rows start 128 or 256 floats into each of its rows."""
    d = datagen.init_data(M, N, K, n, m, seed=M + N)
    W = d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    assert nmspmm.rows_apart(M, N, W, kept) == M % 128
    X = dev(np.ascontiguousarray(d["A_km"].reshape(K, M).T))                         # M x K, K contiguous
    ws = torch.empty(nmspmm.workspace_bytes_rowmajor(M, N, K, 1) // 4, dtype=torch.float32, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm_rowmajor(X, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, W, window, kept, ws)
    torch.cuda.synchronize()
    assert scaled_max_error(C.cpu().numpy(), want_c(oracle, d)) <= REL_TOL

