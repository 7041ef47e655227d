"""GPU parity of the row-major-A entry point, through the C-ABI: the transpose is an exact copy,
and the multiplication of row-major activations matches the CPU checker like the column-major
form does."""
import numpy as np
import pytest

from conftest import REL_TOL, datagen, nmspmm, preprocess_with_oracle, scaled_max_error

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("rows,cols", [(64, 64), (512, 4096), (4096, 512), (100, 260), (33, 7), (1, 128), (4, 4), (2052, 68),
                                       (130, 129)])
def test_transpose_is_an_exact_copy(rows, cols):
    g = torch.Generator(device="cuda").manual_seed(rows * 7 + cols)
    src = torch.randn((rows, cols), generator=g, dtype=torch.float32, device="cuda")
    dst = torch.full((cols, rows), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.transpose_device(src, rows, cols, dst)
    assert torch.equal(dst, src.t())


def test_transpose_of_an_unaligned_view():
    base = torch.randn(64 * 64 + 1, dtype=torch.float32, device="cuda")
    src = base[1:].view(64, 64)                      # 4 bytes off a 16-byte boundary: scalar path
    dst = torch.empty((64, 64), dtype=torch.float32, device="cuda")
    nmspmm.transpose_device(src, 64, 64, dst)
    assert torch.equal(dst, src.t())


@pytest.mark.parametrize("M,N,K,n,m,split_k", [(101, 256, 512, 2, 4, 1), (37, 128, 1024, 2, 8, 2), (1001, 256, 256, 1, 8, 1),
                                               (258, 384, 768, 3, 8, 1), (33, 128, 256, 2, 4, 1), (131, 256, 512, 2, 8, 2)])
def test_row_counts_that_are_not_multiples_of_four_stay_on_the_matrix_cores(oracle, M, N, K, n, m, split_k):
    """The copy of a row-major A is padded to a row pitch of a multiple of four floats, so any row
    count runs on the matrix-core kernels (the decode kernel up to 128 rows, the tile kernel above)."""
    d = datagen.init_data(M, N, K, n, m, seed=M + N)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    A_rm = dev(d["A_km"].T)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.full((nmspmm.workspace_bytes_rowmajor(M, N, K, split_k) // 4,), float("nan"), dtype=torch.float32,
                    device="cuda")
    nmspmm.spmm_rowmajor(A_rm, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, d["W"], window,
                         kept, ws, 32, 128, split_k)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() in (("mfma",) if M > 128 else ("mfma", "skinny"))
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"]).reshape(M, N)
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and scaled_max_error(got, want) <= REL_TOL


@pytest.mark.parametrize("M,N,K,n,m,split_k", [(128, 256, 512, 2, 4, 1), (256, 128, 1024, 2, 8, 2), (64, 512, 512, 1, 8, 1),
                                               (8, 256, 1024, 2, 8, 1), (512, 384, 768, 3, 8, 4)])
def test_row_major_activations(oracle, M, N, K, n, m, split_k):
    d = datagen.init_data(M, N, K, n, m, seed=M + N + split_k)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    A_rm = dev(d["A_km"].T)                          # M x K, K contiguous
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    need = nmspmm.workspace_bytes_rowmajor(M, N, K, split_k)
    assert need >= 4 * M * K + nmspmm.workspace_bytes(M, N, split_k)
    ws = torch.empty(need // 4, dtype=torch.float32, device="cuda")
    nmspmm.spmm_rowmajor(A_rm, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, d["W"], window,
                         kept, ws, 32, 128, split_k)
    torch.cuda.synchronize()
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"]).reshape(M, N)
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and scaled_max_error(got, want) <= REL_TOL
    # the same values as the column-major entry point, bit for bit: only the copy differs
    C2 = torch.empty_like(C)
    ws2 = torch.empty(max(nmspmm.workspace_bytes(M, N, split_k) // 4, 1), dtype=torch.float32, device="cuda")
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C2, M, N, K, d["W"], window,
                kept, 32, 128, split_k, ws2 if split_k > 1 else None)
    assert torch.equal(C, C2)
    with pytest.raises(nmspmm.NmSpmmError):
        nmspmm.spmm_rowmajor(A_rm, dev(d["BT"]), dev(D), None if cinfo is None else dev(cinfo), C, M, N, K, d["W"], window,
                             kept, ws[: need // 4 - 4], 32, 128, split_k)


@pytest.mark.parametrize("M", [1, 2, 3, 5, 8, 9, 16, 32])
@pytest.mark.parametrize("n,m,Ns", [(1, 8, 128), (2, 8, 64), (2, 4, 32), (3, 8, 128), (32, 32, 128)])
def test_decode_sized_row_major_activations(oracle, M, n, m, Ns):
    """Up to 8 rows the decode kernel reads the row-major A in place, above it reads the copy;
    either way the result is the column-major entry point's, bit for bit, and the checker's within
    tolerance.  The head of the workspace (where a copy would go) stays untouched in place."""
    K = 1024 if m == 8 else 1088 if m == 32 else 1152
    N = 256
    d = datagen.init_data(M, N, K, n, m, seed=3 * M + n, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, Ns)
    A_rm = dev(d["A_km"].T)
    dc = None if cinfo is None else dev(cinfo)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.full((nmspmm.workspace_bytes_rowmajor(M, N, K, 1) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm_rowmajor(A_rm, dev(d["BT"]), dev(D), dc, C, M, N, K, d["W"], window, kept, ws, 32, Ns, 1)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "skinny"
    assert torch.isnan(ws).all().item() == (M <= 8)
    C2 = torch.empty_like(C)
    nmspmm.spmm(dev(d["A_km"]), dev(d["BT"]), dev(D), dc, C2, M, N, K, d["W"], window, kept, 32, Ns)
    assert torch.equal(C, C2)
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, d["W"]).reshape(M, N)
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and scaled_max_error(got, want) <= REL_TOL
