"""GPU parity of the index preprocessing kernels, through the C-ABI: bit-exact against the CPU
checker and the reference-written golden vectors."""
import glob
import os

import numpy as np
import pytest

from conftest import GOLDEN_DIR, datagen, kernel_geometry, nmspmm

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN_DIR, "preprocess_*.npz"))), ids=os.path.basename)
def test_device_forms_match_reference_golden(path):
    g = np.load(path)
    W, Q, N, n, m = int(g["W"]), int(g["Q"]), int(g["N"]), int(g["n"]), int(g["m"])
    for key in g.files:
        if key.startswith("low_Ns"):
            Ns = int(key[6:])
            src, dst = dev(g["DT_in"].reshape(-1)), torch.empty(W * Q, dtype=torch.int32, device="cuda")
            nmspmm.preprocess_low_device(src, dst, W, Q, Ns)
            assert np.array_equal(dst.cpu().numpy(), g[key]), key
    x = dev(g["DT_in"].reshape(-1))
    pn, pm, t = n, m, 0
    while "trans%d" % (t + 1) in g.files:
        pn, pm = nmspmm.trans_index_device(x, W, N, Q, pn, pm)
        t += 1
        assert np.array_equal(x.cpu().numpy(), g["trans%d" % t]), "trans%d" % t
    for key in g.files:
        if key.startswith("high_Ns") and key.endswith("_DT"):
            Ns = int(key[7:-3])
            want_ci = g["high_Ns%d_cinfo" % Ns]
            ci = torch.full((want_ci.size,), 7, dtype=torch.int32, device="cuda")
            dst = torch.empty(W * Q, dtype=torch.int32, device="cuda")
            nmspmm.preprocess_high_device(ci, pm, pn, x, dst, W, Q, N, Ns)
            assert np.array_equal(dst.cpu().numpy(), g[key]), key
            assert np.array_equal(ci.cpu().numpy(), want_ci), key


@pytest.mark.parametrize("N,K,n,m,vl,times", [
    (4096, 4096, 2, 4, 32, 3), (4096, 4096, 1, 8, 32, 3), (4096, 4096, 2, 8, 32, 3), (4096, 4096, 3, 8, 32, 2),
    (11008, 4096, 2, 8, 32, 3), (4096, 11008, 2, 8, 32, 3), (4096, 4096, 8, 32, 32, 1), (4096, 4096, 4, 32, 32, 1),
    (1024, 1024, 2, 4, 4, 3), (512, 512, 2, 4, 8, 4),
    (4096, 4096, 2, 4, 4, 0),   # 2:4 with vector length 4 at full size: the 2048 x 1024 (8 MiB) index buffer as generated
])
def test_full_size_index_buffers_bit_exact_vs_checker(oracle, N, K, n, m, vl, times):
    d = datagen.init_data(4, N, K, n, m, vec_len=vl, seed=N + K + n)
    W, Q = d["W"], d["Q"]
    host = d["DT"].reshape(-1).copy()
    x = dev(host)
    pn, pm = n, m
    for _ in range(times):
        pn, pm = nmspmm.trans_index_device(x, W, N, Q, pn, pm)
        oracle.trans_index(host, W, Q, pn // 2, pm // 2)
        assert np.array_equal(x.cpu().numpy(), host)
    for Ns in (32, 64, 128):
        if N % Ns or Ns % vl:
            continue
        dst = torch.empty(W * Q, dtype=torch.int32, device="cuda")
        nmspmm.preprocess_low_device(x, dst, W, Q, Ns, vl)
        want = host.copy()
        oracle.preprocess_low(want, W, Q, Ns, vl)
        assert np.array_equal(dst.cpu().numpy(), want)
        want = host.copy()
        want_ci = oracle.preprocess_high(pm, pn, want, W, Q, Ns, vl)
        ci = torch.empty(nmspmm.column_info_ints(W, pn, pm, N, Ns), dtype=torch.int32, device="cuda")
        assert ci.numel() == want_ci.size
        nmspmm.preprocess_high_device(ci, pm, pn, x, dst, W, Q, N, Ns, vl)
        assert np.array_equal(dst.cpu().numpy(), want)
        assert np.array_equal(ci.cpu().numpy(), want_ci)


@pytest.mark.parametrize("vl,n,m,Ns", [(4, 2, 4, 128), (4, 1, 8, 32), (8, 2, 8, 64), (16, 3, 8, 128), (8, 4, 16, 128)])
def test_one_kernel_preprocessing_of_short_vectors(oracle, vl, n, m, Ns):
    """With vectors of 4, 8 or 16 columns the window stays as generated: the one-kernel entry point
    re-blocks, reports (m, n) as the geometry and needs no column_info."""
    N, K = 512, 256
    d = datagen.init_data(4, N, K, n, m, vec_len=vl, seed=vl + n)
    W, Q = d["W"], d["Q"]
    src = torch.from_numpy(d["DT"].reshape(-1).copy()).cuda()
    out = torch.full_like(src, -5)
    assert nmspmm.preprocess_device(src, n, m, W, Q, N, Ns, out, None) == (m, n)
    torch.cuda.synchronize()
    want = d["DT"].reshape(-1).copy()
    oracle.preprocess_low(want, W, Q, Ns, vl)
    assert np.array_equal(out.cpu().numpy(), want)
    assert np.array_equal(src.cpu().numpy(), d["DT"].reshape(-1))


@pytest.mark.parametrize("n,m", [(2, 4), (3, 8), (2, 8), (1, 8), (16, 32), (12, 32), (8, 32), (4, 32), (32, 32), (1, 2), (4, 16)])
@pytest.mark.parametrize("Ns", [128, 64, 32])
def test_one_kernel_preprocessing_equals_the_separate_calls(oracle, n, m, Ns):
    """nmspmm_preprocess_device folds the transIndex doublings into the re-blocking / ranking pass:
    bit-exact against the checker's sequence and it leaves its input alone."""
    N, K = 1024, 1024 if m != 8 or n != 3 else 1536
    d = datagen.init_data(4, N, K, n, m, seed=10 * n + m + Ns)
    W, Q = d["W"], d["Q"]
    host = d["DT"].reshape(-1).copy()
    src = dev(host)
    window, kept, times = kernel_geometry(n, m)
    want = host.copy()
    pn, pm = n, m
    for _ in range(times):
        pn, pm = oracle.trans_index(want, W, Q, pn, pm)
    out = torch.full((W * Q,), -9, dtype=torch.int32, device="cuda")
    if window == 64:
        want_ci = oracle.preprocess_high(pm, pn, want, W, Q, Ns)
        ci = torch.full((want_ci.size,), -9, dtype=torch.int32, device="cuda")
    else:
        oracle.preprocess_low(want, W, Q, Ns)
        want_ci, ci = None, None
    got = nmspmm.preprocess_device(src, n, m, W, Q, N, Ns, out, ci)
    assert got == (window, kept)
    assert np.array_equal(out.cpu().numpy(), want)
    if want_ci is not None:
        assert np.array_equal(ci.cpu().numpy(), want_ci)
    assert np.array_equal(src.cpu().numpy(), host)


def test_host_pointer_forms_work_in_place(oracle):
    N, K, n, m = 512, 512, 1, 8
    d = datagen.init_data(4, N, K, n, m, seed=3)
    W, Q = d["W"], d["Q"]
    got, want = d["DT"].reshape(-1).copy(), d["DT"].reshape(-1).copy()
    pn, pm = n, m
    for _ in range(3):
        pn, pm = nmspmm.trans_index_host(got, W, N, Q, pn, pm)
        oracle.trans_index(want, W, Q, pn // 2, pm // 2)
    assert (pn, pm) == (8, 64) and np.array_equal(got, want)
    a, b = got.copy(), want.copy()
    nmspmm.preprocess_low_host(a, W, Q, 64)
    oracle.preprocess_low(b, W, Q, 64)
    assert np.array_equal(a, b)
    ci = np.full(nmspmm.column_info_ints(W, pn, pm, N, 128) + pm, -777, np.int32)  # reference-sized, with slack
    nmspmm.preprocess_high_host(ci, pm, pn, got, W, Q, N, 128)
    want_ci = oracle.preprocess_high(pm, pn, want, W, Q, 128)
    assert np.array_equal(got, want)
    assert np.array_equal(ci[:-pm], want_ci) and np.all(ci[-pm:] == -777)
