"""GPU parity of the multiplication, through the C-ABI, against the CPU checker (the restatement
of the reference's nmGEMM_on_cpu) on the same seeded inputs.

Tolerance: scaled max error  max|c - c_ref| / max(|c_ref|, rms(c_ref)) <= 1e-4  (the north-star
bound for fp32 with reordered accumulation; the rms floor keeps it meaningful for signed data)."""
import numpy as np
import pytest

from conftest import REL_TOL, datagen, kernel_geometry, nmspmm, preprocess_with_oracle, scaled_max_error, widen

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_gpu(oracle, d, Ns, split_k=1, fill=float("nan")):
    """Preprocess on the checker, multiply on the GPU; returns (C, kernel family)."""
    M, N, K, W = d["M"], d["N"], d["K"], d["W"]
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    C = torch.full((M, N), fill, dtype=torch.float32, device="cuda")
    ws = None
    if split_k > 1:
        ws = torch.empty(nmspmm.workspace_bytes(M, N, split_k) // 4, dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, W,
                window, kept, d["vec_len"], Ns, split_k, ws)
    torch.cuda.synchronize()
    return C.cpu().numpy(), nmspmm.last_kernel()


def check(oracle, d, got):
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), d["M"], d["N"],
                           d["W"], d["vec_len"]).reshape(d["M"], d["N"])
    assert np.isfinite(got).all()
    err = scaled_max_error(got, want)
    assert err <= REL_TOL, err


PATTERNS = [(2, 4), (3, 8), (2, 8), (1, 8), (16, 32), (12, 32), (8, 32), (4, 32), (32, 32)]


@pytest.mark.parametrize("n,m", PATTERNS)
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_matrix_core_tiles_every_pattern(oracle, n, m, Ns):
    d = datagen.init_data(256, 256, 512, n, m, seed=100 * n + m + Ns)
    got, fam = run_gpu(oracle, d, Ns)
    assert fam == "mfma"
    check(oracle, d, got)


def test_config1_512_cubed_2of4(oracle):
    """The reference's own CPU-checkable case: M = Ncols = K = 512, 2:4, uniform(-1,1); also checked against the dense
    product with the decompressed operand in fp64."""
    d = datagen.init_data(512, 512, 512, 2, 4, seed=1001)
    got, fam = run_gpu(oracle, d, 128)
    assert fam == "mfma"
    check(oracle, d, got)
    dense = oracle.decompress(d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), 512, 512, d["W"])
    want = d["A_km"].T.astype(np.float64) @ dense.astype(np.float64)
    assert scaled_max_error(got, want) <= REL_TOL


@pytest.mark.parametrize("M", [33, 36, 37, 64, 100, 101, 131, 132, 192, 257, 328, 333, 448, 1001])
@pytest.mark.parametrize("n,m,Ns", [(2, 4, 128), (1, 8, 128), (2, 8, 64), (3, 8, 32)])
def test_ragged_row_counts(oracle, M, n, m, Ns):
    """Row counts that are not whole tiles, odd ones included: with a pitch of A that is not a multiple
    of four floats the 128-bit loads of the matrix-core kernels sit on 4-byte boundaries only."""
    d = datagen.init_data(M, 256, 256, n, m, seed=M + n)
    got, fam = run_gpu(oracle, d, Ns)
    assert fam == "mfma" if M > 128 else fam in ("mfma", "skinny")   # up to 128 rows the two kernels compete
    check(oracle, d, got)


@pytest.mark.parametrize("M", [34, 48, 64, 68, 96, 100, 128])
@pytest.mark.parametrize("n,m,Ns", [(1, 8, 128), (2, 8, 64), (2, 4, 32), (3, 8, 128)])
def test_decode_kernel_up_to_128_rows(oracle, M, n, m, Ns):
    """Two and four 32-row blocks per wave; K gives the waves of a workgroup unequal shares, some
    none.  The shape (many columns, a short reduction) is one where the run-time model prefers this
    kernel to the tile kernel: clearly at 1:8 and 2:8, by a hair at 2:4 and 3:8."""
    d = datagen.init_data(M, 8192, 256, n, m, seed=M + Ns, dist="normal", b_scale=0.02)
    got, fam = run_gpu(oracle, d, Ns)
    assert fam == "skinny" if m == 8 and n <= 2 else fam in ("skinny", "mfma")
    check(oracle, d, got)


def test_dense_pattern_above_32_rows_stays_on_the_tile_kernel(oracle):
    d = datagen.init_data(64, 128, 256, 32, 32, seed=5)
    got, fam = run_gpu(oracle, d, 128)
    assert fam == "mfma"
    check(oracle, d, got)


@pytest.mark.parametrize("split_k", [2, 3, 4, 8, 16])
@pytest.mark.parametrize("n,m,Ns", [(2, 4, 128), (1, 8, 128), (2, 8, 32)])
def test_split_k_through_workspace(oracle, split_k, n, m, Ns):
    d = datagen.init_data(160, 256, 1280, n, m, seed=split_k)  # 40 or 20 windows: uneven splits included
    got, _ = run_gpu(oracle, d, Ns, split_k)
    check(oracle, d, got)
    one, _ = run_gpu(oracle, d, Ns, 1)
    assert scaled_max_error(got, one) <= REL_TOL


@pytest.mark.parametrize("split_k", [1, 2, 4])
@pytest.mark.parametrize("M,N,K,n,m,family", [(160, 256, 1280, 2, 4, "mfma"), (256, 512, 1024, 1, 8, "mfma"),
                                             (132, 256, 768, 3, 8, "mfma"), (16, 256, 1024, 2, 8, "skinny"),
                                             (32, 512, 1024, 1, 8, "skinny"), (64, 8192, 512, 1, 8, "skinny"),
                                             (7, 256, 1152, 2, 4, "skinny")])
def test_split_k_adds_to_c_like_the_reference(oracle, M, N, K, n, m, family, split_k):
    """The reference kernels store with SPLIT_K == 1 and atomicAdd into the caller's C with
    SPLIT_K > 1 (src/kernel_64x128_8x8.cu:235-251).  With NMSPMM_ACCUMULATE, and through the named
    launchers, a split call on a non-zero C equals the checker's accumulate-into-C result, and an
    unsplit call overwrites; without the flag every call overwrites."""
    d = datagen.init_data(M, N, K, n, m, seed=7 * M + split_k)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    rng = np.random.default_rng(M + split_k)
    C0 = rng.uniform(-4.0, 4.0, (M, N)).astype(np.float32)
    A, B, Dd = dev(d["A_km"]), dev(d["BT"]), dev(D)
    ci = None if cinfo is None else dev(cinfo)
    ws = None
    if split_k > 1:
        ws = torch.full((nmspmm.workspace_bytes(M, N, split_k) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    args = (d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"])
    product = oracle.gemm_cpu(*args).reshape(M, N)
    added = oracle.gemm_cpu(*args, C=C0.reshape(-1).copy()).reshape(M, N)
    want = added if split_k > 1 else product
    sparsity = 1.0 - n / m

    C = dev(C0)
    nmspmm.spmm_ex(A, B, Dd, ci, C, M, N, K, d["W"], window, kept, 32, 128, split_k, ws, nmspmm.ACCUMULATE)
    torch.cuda.synchronize()
    if M <= 32 or M > 128:  # between, the two kernels compete and the split decides
        assert nmspmm.last_kernel() == family
    assert scaled_max_error(C.cpu().numpy(), want) <= REL_TOL

    C = dev(C0)
    if cinfo is None:
        nmspmm.gemm_low_sparsity(128, A, B, Dd, C, M, N, K, d["W"], sparsity, split_k)
    else:
        nmspmm.gemm_high_sparsity(128, A, B, Dd, ci, C, M, N, K, d["W"], sparsity, split_k)
    torch.cuda.synchronize()
    assert scaled_max_error(C.cpu().numpy(), want) <= REL_TOL

    C = dev(C0)
    nmspmm.spmm(A, B, Dd, ci, C, M, N, K, d["W"], window, kept, 32, 128, split_k, ws)
    torch.cuda.synchronize()
    assert scaled_max_error(C.cpu().numpy(), product) <= REL_TOL


def test_unknown_flag_bits_are_rejected():
    with pytest.raises(nmspmm.NmSpmmError, match="BAD_SHAPE"):
        x = torch.zeros(64 * 64, dtype=torch.float32, device="cuda")
        nmspmm.spmm_ex(x, x, x.int(), None, x, 32, 32, 32, 16, 32, 16, 32, 32, 1, None, 8)


@pytest.mark.parametrize("M", [1, 2, 8, 13, 16, 30, 32])
@pytest.mark.parametrize("n,m", [(1, 8), (2, 8), (2, 4), (3, 8), (32, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_decode_sized_rows_take_the_skinny_path(oracle, M, n, m, Ns):
    """The decode workload in miniature: M <= 32, B ~ N(0, 0.02^2); K gives every wave of the
    workgroup a different number of windows, some none."""
    K = 1024 if m == 8 else 1088 if m == 32 else 1152
    d = datagen.init_data(M, 256, K, n, m, seed=M + Ns, dist="normal", b_scale=0.02)
    for split_k in (1, 4):  # split_k is accepted and has no effect on this path
        got, fam = run_gpu(oracle, d, Ns, split_k)
        assert fam == "skinny"
        check(oracle, d, got)


@pytest.mark.parametrize("M", [1, 16, 256])
def test_operands_off_a_sixteen_byte_boundary_are_rejected(oracle, M):
    """The kernels read A and B with 64- and 128-bit loads: the C-ABI rejects a B that is only
    4-byte aligned instead of launching anything."""
    d = datagen.init_data(M, 256, 1024, 1, 8, seed=M, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    W = d["W"]
    base = torch.empty(W * 256 + 1, dtype=torch.float32, device="cuda")
    B_off = base[1:].view(W, 256)
    assert B_off.data_ptr() % 8 == 4
    C = torch.zeros((M, 256), dtype=torch.float32, device="cuda")
    with pytest.raises(nmspmm.NmSpmmError, match="ALIGNMENT"):
        nmspmm.spmm(dev(d["A_km"]), B_off, dev(D), dev(cinfo), C, M, 256, 1024, W, window, kept, 32, 128)


@pytest.mark.parametrize("M", [1, 8, 16, 32])
@pytest.mark.parametrize("n,m", [(1, 8), (2, 8)])
@pytest.mark.parametrize("K,N", [(8192, 8192), (4096, 14336)])
def test_decode_shapes_at_full_size(oracle, M, n, m, K, N):
    """The sixteen decode cases at full size (K = Ncols = 8192 and K = 4096, Ncols = 14336; 1:8 and
    2:8; B ~ N(0, 0.02^2)), all of C against the checker."""
    d = datagen.init_data(M, N, K, n, m, seed=40 + M + n, dist="normal", b_scale=0.02)
    got, fam = run_gpu(oracle, d, 128)
    assert fam == "skinny"
    check(oracle, d, got)


@pytest.mark.parametrize("vl,n,m", [(4, 3, 4), (8, 5, 8), (16, 7, 8)])
def test_short_vectors_on_the_generic_kernel(oracle, vl, n, m):
    """Per-vector length below 32 on shapes and patterns the matrix-core kernels do not take (64
    columns are too few for the expanding kernel, densities above one half are not for the gathering
    one): indices are used as generated (no widening), any window."""
    M, N, K = 64, 64, 256
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=vl)
    W, Q = d["W"], d["Q"]
    D = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(D, W, Q, 64, vl)
    C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, W, m, n, vl, 64)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "simt"
    check(oracle, d, C.cpu().numpy())


@pytest.mark.parametrize("vl,n,m,Ns", [(4, 2, 4, 128), (4, 1, 4, 32), (4, 3, 4, 64), (8, 1, 8, 128), (8, 2, 8, 64), (16, 3, 8, 128),
                                       (4, 4, 8, 128), (8, 2, 16, 32), (16, 4, 16, 64), (4, 8, 16, 128)])
@pytest.mark.parametrize("M,split_k", [(64, 1), (256, 1), (301, 2), (132, 3)])
def test_short_vectors_on_the_matrix_cores(oracle, vl, n, m, Ns, M, split_k):
    """Vector lengths 4, 8 and 16 with windows of 4, 8 and 16 rows: the gathering MFMA kernel up to a
    density of one half, the expanding one above."""
    N, K = 256, 512
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=vl + n + M)
    W, Q = d["W"], d["Q"]
    D = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(D, W, Q, Ns, vl)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.empty(max(nmspmm.workspace_bytes(M, N, split_k) // 4, 1), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, W, m, n, vl, Ns, split_k,
                ws if split_k > 1 else None)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == ("gather" if 2 * n <= m else "short")
    check(oracle, d, C.cpu().numpy())


@pytest.mark.parametrize("vl,n,m,Ns", [(4, 2, 4, 128), (8, 1, 8, 64), (16, 4, 16, 32), (4, 3, 4, 128)])
@pytest.mark.parametrize("M,split_k", [(64, 1), (301, 2)])
def test_short_vectors_on_the_expanding_kernel(oracle, vl, n, m, Ns, M, split_k):
    """A reduction that is whole 16-row chunks but not whole 64-row (32-row) chunks stays on the
    expanding kernel at any density."""
    N, K = 256, 528
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=vl + n + M)
    W, Q = d["W"], d["Q"]
    D = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(D, W, Q, Ns, vl)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.empty(max(nmspmm.workspace_bytes(M, N, split_k) // 4, 1), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, W, m, n, vl, Ns, split_k,
                ws if split_k > 1 else None)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "short"
    check(oracle, d, C.cpu().numpy())


@pytest.mark.parametrize("vl", [4, 8, 16])
@pytest.mark.parametrize("n,m", [(1, 4), (2, 4), (1, 8), (2, 8), (3, 8), (4, 8), (2, 16), (4, 16), (8, 16)])
@pytest.mark.parametrize("M,N,K,split_k", [(1, 64, 64, 1), (4, 64, 64, 1), (37, 192, 256, 1), (64, 256, 512, 4), (201, 320, 384, 3), (260, 1088, 128, 2)])
def test_gathering_kernel_every_pattern_and_vector_length(oracle, vl, n, m, M, N, K, split_k):
    """The gathering kernel on every pattern it is built for: row counts that are not whole 64-row
    tiles (from a single row, odd ones included), column counts that are not whole 256-column
    workgroups, reductions of one chunk, splits that leave slices unequal."""
    Ns = 64 if N % 128 else 128
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=vl + 3 * n + M)
    W, Q = d["W"], d["Q"]
    D = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(D, W, Q, Ns, vl)
    chunk = 32 if m == 4 else 64
    split_k = min(split_k, K // chunk)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.empty(max(nmspmm.workspace_bytes(M, N, split_k) // 4, 1), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, W, m, n, vl, Ns, split_k, ws if split_k > 1 else None)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "gather"
    check(oracle, d, C.cpu().numpy())


@pytest.mark.parametrize("sparsity,n,m", [(0.5, 16, 32), (0.625, 12, 32), (0.0, 32, 32), (0.75, 8, 32), (0.875, 4, 32)])
@pytest.mark.parametrize("tile", [128, 64, 32])
def test_named_entry_points_with_gpu_preprocessing(oracle, sparsity, n, m, tile):
    """The reference driver's sequence (tests/test_nmspmm.cu:72-97) with pruning_M = 32: preprocess
    (here on the GPU), then the named launcher chosen by sparsity."""
    M, N, K = 128, 256, 256
    d = datagen.init_data(M, N, K, n, m, seed=int(sparsity * 1000) + tile)
    W, Q = d["W"], d["Q"]
    A, B, C = dev(d["A_km"]), dev(d["BT"]), torch.zeros((M, N), dtype=torch.float32, device="cuda")
    DT = dev(d["DT"].reshape(-1))
    Dp = torch.empty_like(DT)
    if sparsity < 0.7:
        nmspmm.preprocess_low_device(DT, Dp, W, Q, tile)
        nmspmm.gemm_low_sparsity(tile, A, B, Dp, C, M, N, K, W, sparsity, 1)
    else:
        pn, pm = nmspmm.trans_index_device(DT, W, N, Q, n, m)
        ci = torch.empty(nmspmm.column_info_ints(W, pn, pm, N, tile), dtype=torch.int32, device="cuda")
        nmspmm.preprocess_high_device(ci, pm, pn, DT, Dp, W, Q, N, tile)
        nmspmm.gemm_high_sparsity(tile, A, B, Dp, ci, C, M, N, K, W, sparsity, 2)  # split 2 via cached workspace
    torch.cuda.synchronize()
    check(oracle, d, C.cpu().numpy())


@pytest.mark.parametrize("M,N,K,n,m,sparsity", [(160, 1024, 2048, 2, 4, 0.5), (256, 512, 4096, 2, 8, 0.75),
                                                 (512, 1024, 1024, 1, 8, 0.875), (2048, 2048, 512, 3, 8, 0.625),
                                                 (16, 512, 2048, 2, 8, 0.75)])
def test_auto_entry_point_chooses_the_split_itself(oracle, M, N, K, n, m, sparsity):
    d = datagen.init_data(M, N, K, n, m, seed=M + K)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.gemm_auto(dev(d["A_km"]), dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, d["W"],
                     sparsity)
    torch.cuda.synchronize()
    split = nmspmm.suggest_split_k(M, N, d["W"], kept)
    assert 1 <= split <= 16 and (d["W"] // kept) // split >= 1
    if M == 160 and K == 2048:
        # 16 tiles for 256 CUs: the reduction must be cut, between workgroups or inside them
        assert split > 1 or nmspmm.waves_along_k_rows(M, N, d["W"], kept) > 0
    if M == 2048 or M <= 32:
        assert split == 1
    check(oracle, d, C.cpu().numpy())


@pytest.mark.parametrize("M,N,K,n,m", [(8192, 4224, 1024, 2, 4), (4096, 8448, 1024, 3, 8), (8192, 4224, 2048, 2, 8)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_ragged_last_round_needs_no_workspace(oracle, M, N, K, n, m, Ns):
    """More tiles than the GPU holds at once and a ragged last round: the leftover tiles run as
    workgroups that share the reduction between their waves, in a launch of their own.  An unsplit
    call does not touch a workspace it is handed: same bits with and without one, and the
    workspace keeps what it held."""
    d = datagen.init_data(M, N, K, n, m, seed=M + N)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    A, B, Dd = dev(d["A_km"]), dev(d["BT"]), dev(D)
    ci = None if cinfo is None else dev(cinfo)
    ws = torch.full((1 << 20,), float("nan"), dtype=torch.float32, device="cuda")
    outs = []
    for scratch in (ws, None):
        C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        nmspmm.spmm(A, B, Dd, ci, C, M, N, K, d["W"], window, kept, 32, Ns, 1, scratch)
        torch.cuda.synchronize()
        assert nmspmm.last_kernel() == "mfma" and bool(torch.isfinite(C).all())
        outs.append(C)
    assert torch.equal(outs[0], outs[1]) and bool(torch.isnan(ws).all())
    for (r0, r1) in ((0, 24), (M // 2 - 8, M // 2 + 8), (M - 16, M)):
        want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"],
                               rows=(r0, r1)).reshape(M, N)[r0:r1]
        assert scaled_max_error(outs[0][r0:r1].cpu().numpy(), want) <= REL_TOL


def check_every_tile_once(oracle, M, N, K, n, m, Ns, **gen):
    """Unsplit multiplication on the tile kernel, checked three ways: every element of C against
    the dense fp64 product A x decompress(B) (the textbook meaning of the operation; sees any row
    or column that went to the wrong place inside a tile, which sums along one axis cannot), the
    row and column sums as checksums of their own, and the first and last rows and one interior
    row of every 32-row strip against the checker."""
    d = datagen.init_data(M, N, K, n, m, seed=M + K, **gen)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, d["W"], window,
                kept, 32, Ns, 1, None)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "mfma" and bool(torch.isfinite(C).all())
    dense = torch.zeros((K, N), dtype=torch.float64, device="cuda")
    rows = (torch.arange(d["W"], device="cuda") // n * m)[:, None] + dev(d["DT"]).long()
    dense[rows.repeat_interleave(32, dim=1), torch.arange(N, device="cuda")[None, :].expand(d["W"], -1)] = dev(d["BT"]).double()
    A64 = dev(d["A_km"]).double()                                # [K][M]
    scaled = lambda got, want: float(((got - want).abs() / want.abs().clamp_min(want.pow(2).mean().sqrt())).max())
    # checksums: C^T 1 = B^T (A^T 1) and C 1 = A (B 1)
    assert scaled(C.double().sum(dim=0), A64.sum(dim=1) @ dense) <= REL_TOL
    assert scaled(C.double().sum(dim=1), dense.sum(dim=1) @ A64) <= REL_TOL
    # every element, a band of rows at a time (bounds the fp64 temporaries)
    for r0 in range(0, M, 2048):
        want = A64[:, r0:r0 + 2048].t() @ dense
        assert scaled(C[r0:r0 + 2048].double(), want) <= REL_TOL, "rows %d.." % r0
        del want
    del dense, A64
    sample = sorted(set(list(range(16)) + list(range(M - 16, M)) + [32 * s + (7 * s + 5) % 32 for s in range(M // 32)]))
    got = C.cpu().numpy()
    ref = np.zeros(M * N, np.float32)  # the checker adds into the rows it is asked for: each sampled row once
    for r in sample:
        oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"], rows=(r, r + 1), C=ref)
    assert scaled_max_error(got[sample], ref.reshape(M, N)[sample]) <= REL_TOL


@pytest.mark.parametrize("M,N,K,n,m", [(4096, 8448, 256, 2, 4), (8192, 4224, 512, 1, 8), (2048, 11008, 256, 2, 4),
                                       (4096, 11008, 4096, 1, 8), (1024, 24576, 4096, 2, 8), (2000, 11008, 256, 2, 4)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_leftover_tiles_in_a_launch_of_their_own(oracle, M, N, K, n, m, Ns):
    """More tiles than the GPU holds at once, a ragged last round and too few windows to cut its
    tiles along K: the leftovers run as a second launch, whole (the first two shapes) or as two or
    four shorter pieces along M each (688 tiles of 256 rows on 512 slots: 176 leftovers in four
    pieces; 1376: 352 in two; 768: 256 in two; the last shape with a ragged row count as well).
    Every tile must still be computed exactly once, for every width of the column blocks (the
    workgroup is then 1 x 4, 2 x 2 or 4 x 1 waves and the tile 128, 64 or 32 columns wide)."""
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m", [(1024, 5120, 128, 2, 4), (2048, 5120, 512, 1, 8), (300, 2048, 256, 2, 8),
                                       (2048, 6656, 512, 1, 8), (1000, 6656, 256, 3, 8), (1024, 5120, 128, 32, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_last_layer_of_a_small_launch_in_pieces(oracle, M, N, K, n, m, Ns):
    """Fewer tiles than the GPU holds at once: the tiles beyond the last multiple of 256 are
    computed as two 64-row pieces each by the workgroups at the end of the same launch when they
    cover at most half of the CUs (320 tiles of 128 rows and four windows: 64 in pieces; 640: 128; 48 with a ragged
    row count: all of them, and the pieces beyond the last row store nothing; 832: 64 after three
    whole layers) and whole otherwise (416: 160 leftovers).  Every tile exactly once, for every
    width of the column blocks."""
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m", [(1024, 4096, 320, 1, 8), (1024, 4096, 64, 1, 8), (512, 4096, 320, 1, 8), (768, 4096, 128, 1, 8),
                                       (200, 4096, 448, 1, 8), (1024, 4096, 96, 2, 4), (1024, 4096, 32, 2, 4), (384, 4096, 160, 2, 4),
                                       (2048, 4096, 96, 3, 8), (512, 4096, 32, 3, 8), (2048, 4096, 160, 12, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_waves_that_load_b_two_windows_ahead(oracle, M, N, K, n, m, Ns):
    """64- and 128-row waves load their B operands two windows ahead: at 3:8 always, at 1:8 and 2:4
    in launches of at most one workgroup per CU (256 whole tiles; 128 or 96 tiles as 256 or 192
    pieces; 192 whole tiles; 64-row waves for a ragged row count).  The window loop is then
    unrolled by two: one, two, three, five and seven windows per workgroup.  Every tile exactly
    once, for every width of the column blocks."""
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m,rows", [(256, 2048, 512, 2, 4, 64), (512, 4096, 1024, 1, 8, 128), (192, 1024, 1024, 2, 8, 64),
                                            (1000, 2048, 1056, 3, 8, 128), (300, 1024, 352, 32, 32, 64), (132, 2048, 512, 2, 4, 64),
                                            (768, 4096, 2112, 1, 8, 64), (256, 8192, 2112, 2, 8, 128),
                                            (200, 4096, 1088, 2, 8, 128), (256, 4096, 1056, 2, 4, 128), (250, 4096, 1216, 1, 8, 128)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_reduction_shared_between_the_waves_of_a_workgroup(oracle, M, N, K, n, m, rows, Ns):
    """Problems of few tiles: one workgroup per 128 or 64 rows of one 32-column vector, its four
    waves each over a quarter of the windows (33 and eleven windows: unequal quarters), partial
    sums added in LDS; the last three cases are at most one 128-row workgroup per compute unit,
    which take eight waves (17, 33 and 19 windows).  Ragged row counts, every index layout, every width of the column blocks;
    every tile exactly once."""
    window, kept, _ = kernel_geometry(n, m)
    assert nmspmm.waves_along_k_rows(M, N, K // window * kept, kept) == rows
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m", [(100, 4096, 1088, 2, 8), (160, 2048, 1472, 2, 4), (192, 2048, 1216, 1, 8), (256, 2048, 1120, 3, 8),
                                       (96, 4096, 2048, 1, 8), (130, 1024, 544, 2, 4)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_eight_waves_along_k_where_every_workgroup_has_a_cu(oracle, M, N, K, n, m, Ns):
    """At most one 64-row workgroup per compute unit and at least sixteen windows: eight waves share
    the reduction (17, 46, 19, 35 and 17 windows: unequal eighths; 32: equal ones).  Every tile
    exactly once, every index layout, every width of the column blocks."""
    window, kept, _ = kernel_geometry(n, m)
    assert nmspmm.waves_along_k_rows(M, N, K // window * kept, kept) == 64
    assert -(-M // 64) * (N // 32) <= nmspmm.device_figures()[0] and K // window >= 16
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m", [(2048, 4096, 2112, 2, 8), (2000, 4096, 1056, 2, 4), (1024, 8192, 2240, 2, 8), (4096, 2048, 1120, 2, 4),
                                       (2048, 4096, 544, 32, 32), (2048, 4096, 2048, 2, 8), (1990, 4096, 2368, 8, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_two_sets_of_waves_where_every_workgroup_has_a_cu(oracle, M, N, K, n, m, Ns):
    """A whole problem of at most one workgroup of 256-row waves per compute unit and at least 512
    kept rows per vector: each workgroup runs two sets of four waves, one per half of the windows
    (33, 33, 35, 35, 17 and 37 windows: unequal halves; 32: equal ones; two ragged row counts),
    and the sets exchange half of their sums through LDS.  Every tile exactly once, every index
    layout, every width of the column blocks."""
    window, kept, _ = kernel_geometry(n, m)
    assert nmspmm.tile_wave_rows(M, N, K // window * kept, kept, Ns) == 256
    assert nmspmm.tile_wave_sets(M, N, K // window * kept, kept, Ns) == 2
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m,rows", [(620, 4096, 2112, 2, 4, 64), (1280, 2048, 1120, 2, 4, 64), (640, 4096, 4160, 2, 8, 64),
                                            (600, 4096, 4128, 3, 8, 64), (1270, 2048, 8256, 1, 8, 64), (760, 4096, 6208, 2, 8, 128),
                                            (750, 4096, 8256, 2, 4, 128), (768, 4096, 6144, 3, 8, 128), (384, 8192, 8192, 2, 8, 128)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_eight_waves_along_k_over_several_layers_of_workgroups(oracle, M, N, K, n, m, rows, Ns):
    """More than two layers of 64-row workgroups on at most 256 tiles: where the pricing of the four
    forms picks eight waves, a compute unit runs two 64-row or one 128-row workgroup at a time,
    layer after layer (five 64-row layers, a ragged last row of workgroups, and three layers of
    128-row ones; window counts that leave the eight waves unequal shares).  Every tile exactly
    once, every index layout, every width of the column blocks."""
    window, kept, _ = kernel_geometry(n, m)
    W = K // window * kept
    assert nmspmm.waves_along_k_rows(M, N, W, kept) == rows and nmspmm.waves_along_k_count(M, N, W, kept) == 8
    assert -(-M // 64) * (N // 32) > 2 * nmspmm.device_figures()[0]
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


def test_larger_problems_stay_on_whole_tiles():
    assert nmspmm.waves_along_k_count(2048, 4096, 2048, 16) == 0
    assert nmspmm.tile_wave_sets(2048, 8192, 512, 16) == 1         # 512 tiles of 256-row waves
    assert nmspmm.tile_wave_sets(2048, 4096, 256, 16) == 1         # 256 kept rows: too short along K
    assert nmspmm.tile_wave_sets(2048, 4096, 1024, 16, 128, 2) == 1
    assert nmspmm.tile_wave_sets(0, 4096, 1024, 16) == 0
    assert nmspmm.waves_along_k_rows(2048, 4096, 2048, 16) == 0    # 512 tiles
    assert nmspmm.waves_along_k_rows(256, 2048, 64, 16) == 0       # four windows: nothing to share
    assert nmspmm.waves_along_k_rows(0, 2048, 64, 16) == 0


@pytest.mark.parametrize("split_k", [2, 3])
@pytest.mark.parametrize("M,n,m", [(512, 3, 8), (256, 1, 8), (384, 2, 4)])
def test_split_slices_of_unequal_length_two_windows_ahead(oracle, M, n, m, split_k):
    """Seven windows (K = 448 at 1:8, whose windows are 64 rows; K = 224 otherwise) cut into two or
    three slices: slices of odd and even length on the window loop unrolled by two."""
    d = datagen.init_data(M, 1024, 448 if m == 8 and n == 1 else 224, n, m, seed=M + split_k)
    got, fam = run_gpu(oracle, d, 128, split_k=split_k)
    assert fam == "mfma"
    check(oracle, d, got)


@pytest.mark.parametrize("M,N,K,n,m", [(1024, 5120, 256, 2, 4), (1152, 4096, 1024, 2, 8), (1000, 4608, 352, 3, 8), (1280, 4096, 704, 1, 8),
                                       (1024, 4608, 288, 32, 32)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_last_layer_of_a_small_launch_with_the_reduction_shared(oracle, M, N, K, n, m, Ns):
    """257 to 320 tiles of 128 rows and at least eight windows: the tiles beyond the first 256 are
    computed by four workgroups each at the end of the same launch, 128 rows of one 32-column
    vector with the reduction shared between the four waves (eight, nine, eleven and sixteen
    windows; a ragged row count).  Every tile exactly once, for every width of the column blocks
    (the whole tile is then 128 x 128, 256 x 64 or 512 x 32)."""
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m", [(512, 11008, 1056, 2, 4), (1024, 5632, 1088, 2, 8), (1000, 5632, 608, 3, 8), (768, 7168, 1280, 1, 8),
                                       (1280, 4352, 544, 32, 32), (1024, 4352, 608, 3, 8), (1024, 8704, 1088, 2, 8),
                                       (1024, 12800, 544, 2, 4), (1000, 9216, 1280, 1, 8)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_last_layer_of_a_small_launch_as_eighths_of_tiles(oracle, M, N, K, n, m, Ns):
    """Up to 96 tiles of 128 rows after one, two or three whole layers of 256 (344, 352, 352, 336,
    340, 272, 544, 800 and 576 tiles) and at least sixteen windows: the tiles of the last layer are
    computed by eight workgroups each at the end of the same launch, 64 rows of one 32-column
    vector with the reduction shared between the four waves (33, 17, 19, 20, 17, 19, 17, 17 and 20
    windows; ragged row counts).  Every tile exactly once, for every width of the column blocks
    (the whole tile is then 128 x 128, 256 x 64 or 512 x 32; 1280 rows in tiles of 512 give 408
    tiles, which take another plan)."""
    window, kept, _ = kernel_geometry(n, m)
    assert nmspmm.tile_wave_rows(M, N, K // window * kept, kept, Ns) == 128 and K // window >= 16
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


@pytest.mark.parametrize("M,N,K,n,m", [(4096, 4224, 1024, 2, 8), (4096, 4480, 544, 2, 4), (1152, 14848, 1088, 1, 8), (2176, 15488, 608, 3, 8),
                                       (4000, 4352, 1280, 1, 8)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_leftover_tiles_as_workgroups_that_share_the_reduction(oracle, M, N, K, n, m, Ns):
    """A few tiles beyond full rounds (16, 48 and 32 tiles of 256 rows beyond 512; 20 and 9 tiles of
    128 rows beyond 1024 and 2048) and at least sixteen windows: the leftovers run in a launch of
    their own as sixteen or eight workgroups per tile, 64 rows of one 32-column vector each, the
    reduction shared between the four waves (16, 17, 17, 19 and 20 windows; a ragged row count).
    Every tile exactly once, for every width of the column blocks (other widths give other tile
    counts: some of them take the pieces along M instead)."""
    check_every_tile_once(oracle, M, N, K, n, m, Ns)


def test_llm_layer_shape_2of8(oracle):
    """One LLM-layer shape (M = 512, K = 4096, Ncols = 11008, 2:8, N(0,1) x N(0,0.02^2))."""
    d = datagen.init_data(512, 11008, 4096, 2, 8, seed=3001, dist="normal", b_scale=0.02)
    got, fam = run_gpu(oracle, d, 128)
    assert fam == "mfma"
    check(oracle, d, got)


@pytest.mark.parametrize("M", [512, 2048, 8192])
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 11008), (11008, 4096)])
def test_llm_layer_shapes_at_full_size(oracle, M, K, N):
    """The nine prefill-sized LLM-layer shapes at 2:8, A ~ N(0,1), B ~ N(0, 0.02^2).  K = 11008 is
    172 windows of 64 rows, not a power of two; Ncols = 11008 is 86 column blocks.  Column sums in
    fp64 touch every tile, the first and last rows are compared with the checker."""
    check_every_tile_once(oracle, M, N, K, 2, 8, 128, dist="normal", b_scale=0.02)


@pytest.mark.parametrize("n,m", [(4, 32), (8, 32), (16, 32), (3, 8)])
def test_full_size_4096_cubed_remaining_patterns(oracle, n, m):
    """The fine-grained patterns (windows of 32 as generated, one widening for 4:32 and 8:32) and
    3:8 at M = Ncols = K = 4096."""
    check_every_tile_once(oracle, 4096, 4096, 4096, n, m, 128)


@pytest.mark.parametrize("n,m", [(2, 4), (2, 8), (1, 8)])
def test_full_size_4096_cubed_with_vectors_of_four_columns(oracle, n, m):
    """2:4, 2:8 and 1:8 with index vectors of 4 columns at M = Ncols = K = 4096 (2:4: 2048 x 1024
    indices, 8 MiB), the gathering matrix-core kernel.  Column sums in fp64 over all of C; sampled
    rows against the checker."""
    M = N = K = 4096
    vl = 4
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=5004)
    W, Q = d["W"], d["Q"]
    DT = dev(d["DT"].reshape(-1))
    D = torch.empty_like(DT)
    nmspmm.preprocess_low_device(DT, D, W, Q, 128, vl)
    want_D = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(want_D, W, Q, 128, vl)
    assert np.array_equal(D.cpu().numpy(), want_D)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), D, None, C, M, N, K, W, m, n, vl, 128)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "gather" and bool(torch.isfinite(C).all())
    dense = torch.zeros((K, N), dtype=torch.float64, device="cuda")
    rows = (torch.arange(W, device="cuda") // n * m)[:, None] + dev(d["DT"]).long()
    dense[rows.repeat_interleave(vl, dim=1), torch.arange(N, device="cuda")[None, :].expand(W, -1)] = dev(d["BT"]).double()
    want = dev(d["A_km"]).double().sum(dim=1) @ dense
    got = C.double().sum(dim=0)
    assert float(((got - want).abs() / want.abs().clamp_min(want.pow(2).mean().sqrt())).max()) <= REL_TOL
    rows_s = np.array([0, 1, 127, 128, 2047, 2048, M - 129, M - 2, M - 1])
    A_rows = np.ascontiguousarray(d["A_km"][:, rows_s])
    ref = oracle.gemm_cpu(A_rows.reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), len(rows_s), N, W,
                          vl).reshape(len(rows_s), N)
    assert scaled_max_error(C[torch.from_numpy(rows_s).cuda()].cpu().numpy(), ref) <= REL_TOL


@pytest.mark.parametrize("n,m", [(2, 4), (2, 8), (1, 8)])
def test_full_size_4096_cubed_checksums_and_row_sample(oracle, n, m):
    """The headline square workload at full size.  The checker would need minutes for all of C, so: (1) rows
    [0,32) and [4064,4096) are compared with the checker; (2) checksums that hold for any size:
    C . 1 = A . (B_dense . 1) and 1^T . C = (1^T . A) . B_dense, evaluated in fp64 from the inputs."""
    M = N = K = 4096
    d = datagen.init_data(M, N, K, n, m, seed=2000 + n * 10 + m)
    got, fam = run_gpu(oracle, d, 128)
    assert fam == "mfma" and np.isfinite(got).all()
    A, B, D = d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1)
    for rows in ((0, 32), (M - 32, M)):
        want = oracle.gemm_cpu(A, B, D, M, N, d["W"], rows=rows).reshape(M, N)[rows[0]:rows[1]]
        assert scaled_max_error(got[rows[0]:rows[1]], want) <= REL_TOL
    dense = oracle.decompress(B, D, K, N, d["W"]).astype(np.float64)
    A64 = d["A_km"].T.astype(np.float64)  # M x K
    row_sums = A64 @ dense.sum(axis=1)
    col_sums = A64.sum(axis=0) @ dense
    g64 = got.astype(np.float64)
    scale = np.sqrt(d["W"] * N / 9.0)  # std of a row/column sum of C for uniform(-1,1) operands
    assert np.max(np.abs(g64.sum(axis=1) - row_sums)) <= 1e-4 * scale
    assert np.max(np.abs(g64.sum(axis=0) - col_sums)) <= 1e-4 * scale


def test_result_larger_than_four_gib(oracle):
    """C of 32768 x 32768 floats is 4 GiB: every row's byte offset from C needs more than 32 bits
    beyond row 32767 / 2.  A sample of rows from both halves is compared with the checker (rows are
    independent, so the checker multiplies just those rows of A)."""
    M = N = 32768
    K = 64
    free, _ = torch.cuda.mem_get_info()
    if free < 6 * 2**30:
        pytest.skip("needs 6 GiB of free device memory")
    d = datagen.init_data(M, N, K, 2, 4, seed=4242)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, d["W"], window, kept, 32, 128)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "mfma"
    rows = np.array([0, 1, 255, 256, 16383, 16384, 16385, 20000, 32511, 32512, 32766, 32767])
    got = C[torch.from_numpy(rows).cuda()].cpu().numpy()
    A_rows = np.ascontiguousarray(d["A_km"][:, rows])
    want = oracle.gemm_cpu(A_rows.reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), len(rows), N,
                           d["W"]).reshape(len(rows), N)
    assert np.isfinite(got).all() and scaled_max_error(got, want) <= REL_TOL
    # nothing was left unwritten anywhere
    assert not torch.isnan(C).any().item()


def test_split_k_workspace_larger_than_four_gib(oracle):
    """Four reduction slices of a 16384 x 16384 result: the slices sit up to 3 GiB beyond the
    workspace's start and the second pass walks more than 2^32 bytes."""
    M = N = 16384
    K, split_k = 256, 4
    free, _ = torch.cuda.mem_get_info()
    if free < 8 * 2**30:
        pytest.skip("needs 8 GiB of free device memory")
    d = datagen.init_data(M, N, K, 1, 8, seed=4343)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    need = nmspmm.workspace_bytes(M, N, split_k)
    assert need >= 4 * 2**30
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), dev(cinfo), C, M, N, K, d["W"], window, kept, 32, 128, split_k, ws)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "mfma"
    rows = np.array([0, 127, 128, 8191, 8192, 12345, 16255, 16383])
    got = C[torch.from_numpy(rows).cuda()].cpu().numpy()
    A_rows = np.ascontiguousarray(d["A_km"][:, rows])
    want = oracle.gemm_cpu(A_rows.reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), len(rows), N,
                           d["W"]).reshape(len(rows), N)
    assert np.isfinite(got).all() and scaled_max_error(got, want) <= REL_TOL
    assert not torch.isnan(C).any().item()


def test_decode_kernel_with_a_million_column_vectors(oracle):
    """Ncols = 2^22: 131072 workgroups of the decode kernel, B rows 16 MiB apart."""
    M, N, K = 4, 1 << 22, 64
    d = datagen.init_data(M, N, K, 2, 4, seed=4444, dist="normal", b_scale=0.02)
    got, fam = run_gpu(oracle, d, 128)
    assert fam == "skinny"
    check(oracle, d, got)


@pytest.mark.parametrize("M,family", [((1 << 22) - 4, "mfma"), ((1 << 22) + 4, "simt")])
def test_row_counts_either_side_of_the_tile_kernels_limit(oracle, M, family):
    """The tile kernel forms A offsets with 24-bit multiplies, which holds up to 2^22 - 1 rows;
    beyond that the generic kernel runs.  Sampled rows against the checker on both sides."""
    N, K = 128, 32
    free, _ = torch.cuda.mem_get_info()
    if free < 6 * 2**30:
        pytest.skip("needs 6 GiB of free device memory")
    d = datagen.init_data(M, N, K, 2, 4, seed=M % 1000)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, d["W"], window, kept, 32, 128)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == family
    rows = np.array([0, 1, 255, 256, M // 2, M // 2 + 1, M - 257, M - 2, M - 1])
    got = C[torch.from_numpy(rows).cuda()].cpu().numpy()
    A_rows = np.ascontiguousarray(d["A_km"][:, rows])
    want = oracle.gemm_cpu(A_rows.reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), len(rows), N,
                           d["W"]).reshape(len(rows), N)
    assert np.isfinite(got).all() and scaled_max_error(got, want) <= REL_TOL
    assert not torch.isnan(C).any().item()


@pytest.mark.parametrize("M,N,K,vl,n,m", [(2048, 11008, 256, 4, 3, 4), (4096, 5120, 528, 8, 1, 8), (1000, 24576, 272, 16, 3, 8)])
def test_short_vector_kernel_with_leftover_tiles(oracle, M, N, K, vl, n, m):
    """The short-vector kernel on more tiles than the GPU holds at once with a ragged last round:
    the leftovers run as a second launch, whole or as two 128-row pieces each.  Column sums in fp64
    touch every tile; sampled rows against the checker."""
    d = datagen.init_data(M, N, K, n, m, vec_len=vl, seed=M + vl)
    W, Q = d["W"], d["Q"]
    D = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(D, W, Q, 128, vl)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None, C, M, N, K, W, m, n, vl, 128)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "short" and bool(torch.isfinite(C).all())
    dense = torch.zeros((K, N), dtype=torch.float64, device="cuda")
    rows = (torch.arange(W, device="cuda") // n * m)[:, None] + dev(d["DT"]).long()
    dense[rows.repeat_interleave(vl, dim=1), torch.arange(N, device="cuda")[None, :].expand(W, -1)] = dev(d["BT"]).double()
    want = dev(d["A_km"]).double().sum(dim=1) @ dense
    got = C.double().sum(dim=0)
    assert float(((got - want).abs() / want.abs().clamp_min(want.pow(2).mean().sqrt())).max()) <= REL_TOL
    rows_s = np.array([0, 1, 127, 128, 255, 256, M // 2, M - 129, M - 2, M - 1])
    A_rows = np.ascontiguousarray(d["A_km"][:, rows_s])
    ref = oracle.gemm_cpu(A_rows.reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), len(rows_s), N, W,
                          vl).reshape(len(rows_s), N)
    assert scaled_max_error(C[torch.from_numpy(rows_s).cuda()].cpu().numpy(), ref) <= REL_TOL
