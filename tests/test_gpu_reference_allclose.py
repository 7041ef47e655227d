"""The reference's own acceptance check on the reference's own kind of data.

The reference driver accepts a kernel when its `allclose` (include/utils.h:68-80:
|a - b| <= 1e-8 + 1e-5 |b|) passes between the GPU result and nmGEMM_on_cpu on operands drawn
from [0, 1] (include/utils.h:36,42; tests/test_nmspmm.cu:90-108).  Here the same call sequence
runs through the C++ drop-in symbols of libnmspmm.so (host-pointer preprocessing in place, the
eight launchers by name, default stream), and the compiled reference itself (oracle/_ref) is both
the CPU result and the judge of closeness.  That criterion is ten times tighter than the 1e-4
bound of the other tests and is relative to each element, which all-positive data makes
meaningful."""
import ctypes
import importlib
import os

import numpy as np
import pytest

from conftest import ROOT, datagen
from oracle.nm_oracle import Reference

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not Reference.available(), reason="oracle/_ref is not built")]
torch = pytest.importorskip("torch")

TILES = {"huge": 128, "large": 64, "medium": 64, "small": 32}
SPARSITIES = [0.0, 0.5, 0.625, 0.75, 0.875]


@pytest.fixture(scope="module")
def cxx():
    """The drop-in's C++ symbols (include/NM-SpMM.h), by their mangled names."""
    lib = ctypes.CDLL(os.path.join(ROOT, "nm-spmm_amd", "libnmspmm.so"))
    vp, ci, ip = ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int)
    fns = {}
    for tile in TILES:
        name = "nmGEMM_%s_matrices_low_sparsity" % tile
        f = getattr(lib, "_Z%d%sPfS_PiS_iiiifi" % (len(name), name))
        f.argtypes, f.restype = [vp] * 4 + [ci] * 4 + [ctypes.c_float, ci], None
        fns[(tile, False)] = f
        name = "nmGEMM_%s_matrices_high_sparsity" % tile
        f = getattr(lib, "_Z%d%sPfS_PiS0_S_iiiifi" % (len(name), name))
        f.argtypes, f.restype = [vp] * 5 + [ci] * 4 + [ctypes.c_float, ci], None
        fns[(tile, True)] = f
    fns["transIndex"] = lib._Z10transIndexPiiiiRiS0_
    fns["transIndex"].argtypes, fns["transIndex"].restype = [vp, ci, ci, ci, ip, ip], None
    fns["low"] = lib._Z26PreProcessing_low_sparsityPiiii
    fns["low"].argtypes, fns["low"].restype = [vp, ci, ci, ci], None
    fns["high"] = lib._Z27PreProcessing_high_sparsityPiiiS_iiii
    fns["high"].argtypes, fns["high"].restype = [vp, ci, ci, vp] + [ci] * 4, None
    return fns


def run_like_the_reference_driver(cxx, d, tile, sparsity, split_k):
    """tests/test_nmspmm.cu:72-98 with the drop-in: returns C from the GPU."""
    M, N, K, W, Q = d["M"], d["N"], d["K"], d["W"], d["Q"]
    Ns, pM, pN = TILES[tile], 32, d["n"]
    high = sparsity in (0.75, 0.875)
    DT = d["DT"].reshape(-1).copy()
    if high:
        column_info = np.zeros(((W // pN) * (N // Ns) + 1) * pM * 2, np.int32)
        n_ref, m_ref = ctypes.c_int(pN), ctypes.c_int(pM)
        cxx["transIndex"](DT.ctypes.data, W, N, Q, ctypes.byref(n_ref), ctypes.byref(m_ref))
        assert (n_ref.value, m_ref.value) == (2 * pN, 64)
        cxx["high"](column_info.ctypes.data, m_ref.value, n_ref.value, DT.ctypes.data, W, Q, N, Ns)
    else:
        cxx["low"](DT.ctypes.data, W, Q, Ns)
    A = torch.from_numpy(d["A_km"]).cuda()
    B = torch.from_numpy(d["BT"]).cuda()
    D = torch.from_numpy(DT).cuda()
    C = torch.zeros((M, N), dtype=torch.float32, device="cuda")  # the driver uploads a zeroed C
    torch.cuda.synchronize()
    if high:
        ci = torch.from_numpy(column_info).cuda()
        cxx[(tile, True)](A.data_ptr(), B.data_ptr(), D.data_ptr(), ci.data_ptr(), C.data_ptr(), M, N, K, W, sparsity, split_k)
    else:
        cxx[(tile, False)](A.data_ptr(), B.data_ptr(), D.data_ptr(), C.data_ptr(), M, N, K, W, sparsity, split_k)
    torch.cuda.synchronize()
    return C.cpu().numpy()


def operands(M, N, K, sparsity, seed):
    kept = int(round(32 * (1.0 - sparsity)))
    return datagen.init_data(M, N, K, kept, 32, seed=seed, dist="unit")


@pytest.mark.parametrize("sparsity", SPARSITIES)
@pytest.mark.parametrize("tile", list(TILES))
def test_eight_launchers_pass_the_references_allclose_at_512_cubed(cxx, tile, sparsity):
    ref = Reference()
    d = operands(512, 512, 512, sparsity, seed=int(1000 * sparsity) + len(tile))
    want = ref.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), 512, 512, 512, d["W"])
    got = run_like_the_reference_driver(cxx, d, tile, sparsity, 1).reshape(-1)
    assert ref.allclose(np.ascontiguousarray(got), want), "the reference's allclose rejects the GPU result"


@pytest.mark.parametrize("sparsity", [0.5, 0.875])
def test_split_k_passes_the_references_allclose(cxx, sparsity):
    """SPLIT_K = 4 as the reference driver may ask for it: added to the zeroed C."""
    ref = Reference()
    d = operands(512, 512, 512, sparsity, seed=7)
    want = ref.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), 512, 512, 512, d["W"])
    got = run_like_the_reference_driver(cxx, d, "huge", sparsity, 4).reshape(-1)
    assert ref.allclose(np.ascontiguousarray(got), want)


@pytest.mark.parametrize("sparsity", SPARSITIES)
def test_sample_of_rows_at_k_4096(cxx, sparsity):
    """M = Ncols = K = 4096 on the GPU; 64 rows spread over the matrix against the reference's CPU
    path on those rows (rows are independent: include/utils.h:86-87)."""
    ref = Reference()
    M = N = K = 4096
    d = operands(M, N, K, sparsity, seed=4096 + int(8 * sparsity))
    got = run_like_the_reference_driver(cxx, d, "huge", sparsity, 1)
    rows = np.arange(64) * 64 + (np.arange(64) * 37) % 64   # one per 64-row strip, at varying offsets
    A_sub = np.ascontiguousarray(d["A_km"][:, rows]).reshape(-1)
    want = ref.gemm_cpu(A_sub, d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), 64, N, K, d["W"])
    assert ref.allclose(np.ascontiguousarray(got[rows]).reshape(-1), want)


@pytest.mark.parametrize("M", [1, 16, 32])
@pytest.mark.parametrize("sparsity", [0.5, 0.75, 0.875])
def test_named_launchers_take_an_attached_row_list_at_decode_sizes(cxx, M, sparsity):
    """The reference's signatures have no argument for the row list.  A caller that built one
    attaches it to its D; from then on the C++ launchers run decode-sized calls on the kernel that
    reads the list (same bits as nmspmm_spmm_ex with the list), and on the reference-layout kernel
    again once it is detached.  Both pass the reference's allclose."""
    nmspmm = importlib.import_module("nm-spmm_amd")
    ref = Reference()
    N, K = 1024, 2048
    d = operands(M, N, K, sparsity, seed=50 + M)
    W, Q, Ns = d["W"], d["Q"], 128
    high = sparsity in (0.75, 0.875)
    want = ref.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N, K, W)
    DT = d["DT"].reshape(-1).copy()
    window, kept = 32, d["n"]
    ci = None
    if high:
        column_info = np.zeros(((W // kept) * (N // Ns) + 1) * 32 * 2, np.int32)
        n_ref, m_ref = ctypes.c_int(kept), ctypes.c_int(32)
        cxx["transIndex"](DT.ctypes.data, W, N, Q, ctypes.byref(n_ref), ctypes.byref(m_ref))
        kept, window = n_ref.value, m_ref.value
        cxx["high"](column_info.ctypes.data, window, kept, DT.ctypes.data, W, Q, N, Ns)
        ci = torch.from_numpy(column_info).cuda()
    else:
        cxx["low"](DT.ctypes.data, W, Q, Ns)
    A, B, D = torch.from_numpy(d["A_km"]).cuda(), torch.from_numpy(d["BT"]).cuda(), torch.from_numpy(DT).cuda()
    R = torch.empty(nmspmm.row_index_ints(W, N), dtype=torch.int32, device="cuda")
    nmspmm.row_index_device(D, ci, W, N, window, kept, Ns, R)
    torch.cuda.synchronize()

    def launch():
        C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        if high:
            cxx[("huge", True)](A.data_ptr(), B.data_ptr(), D.data_ptr(), ci.data_ptr(), C.data_ptr(), M, N, K, W, sparsity, 1)
        else:
            cxx[("huge", False)](A.data_ptr(), B.data_ptr(), D.data_ptr(), C.data_ptr(), M, N, K, W, sparsity, 1)
        torch.cuda.synchronize()
        return C, nmspmm.last_kernel()

    plain, family = launch()
    assert family in ("skinny", "mfma")
    nmspmm.row_index_attach(D, R)
    try:
        listed, family = launch()
        assert family == "decode"
        direct = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        nmspmm.spmm_ex(A, B, D, ci, direct, M, N, K, W, window, kept, 32, Ns, 1, None, 0, R)
        torch.cuda.synchronize()
        assert torch.equal(listed, direct)
    finally:
        nmspmm.row_index_attach(D, None)
    again, family = launch()
    assert family in ("skinny", "mfma") and torch.equal(again, plain)
    for got in (plain, listed):
        assert ref.allclose(np.ascontiguousarray(got.cpu().numpy()).reshape(-1), want)
