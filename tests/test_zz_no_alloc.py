"""nmspmm_spmm_noalloc: split-K with the slices in the library's fixed device-resident scratch (for
callers that cannot allocate).  Through the C-ABI, against nmspmm_spmm with a caller-owned
workspace: the same kernels run on the same slices, so C must be identical bit for bit; and against
the checker to the 1e-4 bound.  Two calls in a row, the second with a smaller input, so the second
finds the first call's slices in the scratch."""
import ctypes

import numpy as np
import pytest

from conftest import REL_TOL, datagen, nmspmm, preprocess_with_oracle, scaled_max_error

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def both_ways(oracle, M, N, K, n, m, split_k, seed):
    d = datagen.init_data(M, N, K, n, m, seed=seed)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    A, B, Dd = dev(d["A_km"]), dev(d["BT"]), dev(D)
    ci = None if cinfo is None else dev(cinfo)
    ws = None
    if split_k > 1:
        ws = torch.full((nmspmm.workspace_bytes(M, N, split_k) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    C_ws = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    C_na = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    nmspmm.spmm(A, B, Dd, ci, C_ws, M, N, K, d["W"], window, kept, 32, 128, split_k, ws)
    fam = nmspmm.last_kernel()
    torch.cuda.synchronize()
    # Nothing may be allocated by the call: not by torch (memory_allocated) and not by the library
    # behind torch's back (the device's free bytes as hipMemGetInfo reports them, which a hipMalloc
    # inside libnmspmm.so would lower).  One untimed call first, so that the code object and the
    # scratch's address are already resolved; the library's cached workspace is released before,
    # so that any use of it would have to allocate again and show.
    nmspmm.spmm_noalloc(A, B, Dd, ci, C_na, M, N, K, d["W"], window, kept, 32, 128, split_k)
    torch.cuda.synchronize()
    nmspmm.release()
    C_na.fill_(float("nan"))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    nmspmm.spmm_noalloc(A, B, Dd, ci, C_na, M, N, K, d["W"], window, kept, 32, 128, split_k)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated during the call"
    assert nmspmm.last_kernel() == fam
    assert torch.equal(C_na, C_ws), "differs from the call with a caller-owned workspace"
    want = oracle.gemm_cpu(d["A_km"].reshape(-1), d["B_cm"].reshape(-1), d["D_cm"].reshape(-1), M, N,
                           d["W"]).reshape(M, N)
    assert scaled_max_error(C_na.cpu().numpy(), want) <= REL_TOL


@pytest.mark.parametrize("n,m", [(2, 4), (1, 8)])
def test_two_calls_in_a_row_the_second_smaller(oracle, n, m):
    both_ways(oracle, 512, 1024, 2048, n, m, 4, seed=70 + n)   # 8 MiB of slices
    both_ways(oracle, 160, 256, 1280, n, m, 3, seed=80 + n)    # 480 KiB: finds the first call's slices there
    both_ways(oracle, 160, 256, 1280, n, m, 1, seed=90 + n)    # unsplit: no scratch involved


def test_a_split_that_fills_the_scratch_to_its_last_byte(oracle):
    assert nmspmm.workspace_bytes(512, 4096, 4) == nmspmm.NOALLOC_MAX_BYTES
    both_ways(oracle, 512, 4096, 512, 2, 4, 4, seed=99)


def test_sizes_beyond_the_scratch_are_rejected_before_any_launch():
    M, N, split_k = 1024, 4096, 4
    assert nmspmm.workspace_bytes(M, N, split_k) > nmspmm.NOALLOC_MAX_BYTES
    x = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    C = torch.full((M, N), 7.0, dtype=torch.float32, device="cuda")
    with pytest.raises(nmspmm.NmSpmmError, match="WORKSPACE"):
        nmspmm.spmm_noalloc(x, x, x.int(), None, C, M, N, 1024, 512, 32, 16, 32, 128, split_k)
    torch.cuda.synchronize()
    assert bool((C == 7.0).all())


def test_the_limit_is_the_headers():
    import os
    import re
    from conftest import ROOT
    text = open(os.path.join(ROOT, "include", "nmspmm.h")).read()
    m = re.search(r"#define NMSPMM_NOALLOC_MAX_BYTES \((\d+)u << (\d+)\)", text)
    assert m and int(m.group(1)) << int(m.group(2)) == nmspmm.NOALLOC_MAX_BYTES
