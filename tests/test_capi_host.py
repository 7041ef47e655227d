"""CPU-only checks of the C-ABI: the library loads, exports every symbol include/nmspmm.h
declares and every C++ drop-in function of include/NM-SpMM.h, and rejects bad arguments with the
documented status codes before touching the GPU."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import ROOT, nmspmm


def declared_c_symbols():
    text = open(os.path.join(ROOT, "include", "nmspmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nmspmm_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = nmspmm.lib()
    names = declared_c_symbols()
    assert len(names) >= 16
    for name in names:
        assert hasattr(lib, name), name
    assert lib.nmspmm_version() >= 100


def test_library_exports_the_cxx_drop_in_functions():
    out = subprocess.run(["nm", "-DC", nmspmm.LIB_PATH], check=True, capture_output=True, text=True).stdout
    wanted = ["transIndex(int*, int, int, int, int&, int&)", "PreProcessing_low_sparsity(int*, int, int, int)",
              "PreProcessing_high_sparsity(int*, int, int, int*, int, int, int, int)"]
    for size in ("huge", "large", "medium", "small"):
        wanted.append("nmGEMM_%s_matrices_low_sparsity(float*, float*, int*, float*, int, int, int, int, float, int)" % size)
        wanted.append("nmGEMM_%s_matrices_high_sparsity(float*, float*, int*, int*, float*, int, int, int, int, float, int)" % size)
    wanted.append("nmGEMM(float*, float*, int*, int*, float*, int, int, int, int, float)")
    for w in wanted:
        assert " T " + w in out, w


def test_split_suggestion():
    L = nmspmm.lib()
    assert L.nmspmm_suggest_split_k(4096, 4096, 2048, 16) == 1      # 4096 waves already
    assert L.nmspmm_suggest_split_k(160, 4096, 2048, 16) == 1       # 64 tiles, 128 windows: the four waves of a workgroup share the reduction
    assert L.nmspmm_suggest_split_k(2048, 12288, 16384, 16) == 1    # 1536 tiles fill the GPU
    assert L.nmspmm_suggest_split_k(64, 8192, 2048, 16) == 1        # the decode kernel needs no split
    assert L.nmspmm_suggest_split_k(512, 4096, 1024, 16) in (1, 2)  # 128 tiles: as 256 pieces along M, or two slices
    assert L.nmspmm_suggest_split_k(192, 512, 128, 16) in (1, 2, 4, 8)  # never more slices than windows
    assert L.nmspmm_suggest_split_k(4096, 4096, 16, 16) == 1        # one window cannot be split
    assert L.nmspmm_suggest_split_k(8, 8192, 1024, 8) == 1          # decode kernel reduces in the workgroup
    assert L.nmspmm_suggest_split_k(0, 8192, 1024, 8) == 0 and L.nmspmm_suggest_split_k(64, 64, 100, 16) == 0
    assert L.nmspmm_gemm_auto(FAKE, FAKE, FAKE, None, FAKE, 64, 128, 128, 16, 0.75, None) == 1   # column_info missing
    assert L.nmspmm_gemm_auto(FAKE, FAKE, FAKE, None, FAKE, 64, 128, 128, 64, 0.3, None) == 3


def test_device_figures_without_a_gpu_are_those_of_an_mi355x():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the figures are the device's")
    assert nmspmm.device_figures() == (256, 8, 2.4e9)


def test_wave_sets_of_the_tile_kernel():
    """Two sets of waves per workgroup only for a whole unsplit problem of at most one workgroup of
    256-row waves per compute unit (256 without a GPU) with at least 512 kept rows per vector."""
    import torch
    if torch.cuda.is_available() and nmspmm.device_figures()[0] != 256:
        pytest.skip("the shapes below are sized for 256 compute units")
    for Ns in (128, 64, 32):
        assert nmspmm.tile_wave_rows(2048, 4096, 1024, 16, Ns) == 256
        assert nmspmm.tile_wave_sets(2048, 4096, 1024, 16, Ns) == 2      # 256 workgroups
        assert nmspmm.tile_wave_sets(2048, 8192, 1024, 16, Ns) == 1      # 512 workgroups
        assert nmspmm.tile_wave_sets(2048, 4096, 256, 16, Ns) == 1       # short along K
        assert nmspmm.tile_wave_sets(2048, 4096, 1024, 16, Ns, 2) == 1   # split by the caller
    assert nmspmm.tile_wave_sets(2048, 4096, 512, 8) == 1                # 128-row waves
    assert nmspmm.tile_wave_sets(64, 4096, 1024, 16) == 0                # waves along K: another launch
    assert nmspmm.tile_wave_sets(0, 4096, 1024, 16) == 0 and nmspmm.tile_wave_sets(64, 4096, 1000, 16) == 0


def test_rows_apart():
    """The last rows of a row count a little above a multiple of 128 go to the decode-sized kernels only
    where an extra layer of 128-row workgroups is expected to cost more than reading B again."""
    import torch
    if torch.cuda.is_available() and nmspmm.device_figures()[0] != 256:
        pytest.skip("the shapes below are sized for 256 compute units")
    assert nmspmm.rows_apart(136, 4096, 1024, 16) == 8          # 4096 columns, K = 2048 at 2:4
    assert nmspmm.rows_apart(288, 8192, 512, 16) == 32
    assert nmspmm.rows_apart(136, 2048, 1024, 16) == 0          # both row tiles fit one layer of workgroups
    assert nmspmm.rows_apart(136, 4096, 512, 8) == 0            # eight kept rows per window: only from 512 rows on
    assert nmspmm.rows_apart(520, 11008, 512, 8) == 8
    assert nmspmm.rows_apart(168, 4096, 1024, 16) == 0          # 40 rows above the multiple
    assert nmspmm.rows_apart(128, 4096, 1024, 16) == 0 and nmspmm.rows_apart(100, 4096, 1024, 16) == 0
    assert nmspmm.rows_apart(136, 4096, 1000, 16) == 0          # invalid: W is not a multiple of kept


def test_pattern_table():
    assert nmspmm.pattern_from_sparsity(0.0) == (32, 32, False)
    assert nmspmm.pattern_from_sparsity(0.5) == (32, 16, False)
    assert nmspmm.pattern_from_sparsity(0.625) == (32, 12, False)
    assert nmspmm.pattern_from_sparsity(0.75) == (64, 16, True)
    assert nmspmm.pattern_from_sparsity(0.875) == (64, 8, True)
    with pytest.raises(nmspmm.NmSpmmError) as e:
        nmspmm.pattern_from_sparsity(0.3)
    assert e.value.status == 3


def test_sizes():
    assert nmspmm.workspace_bytes(64, 128, 1) == 0
    assert nmspmm.workspace_bytes(64, 128, 4) == 4 * 64 * 128 * 4
    assert nmspmm.workspace_bytes(3, 3, 2) == 2 * 12 * 4  # slices padded to 4 floats
    # payload of the reference's allocation rule (tests/test_nmspmm.cu:23) without its slack window
    assert nmspmm.column_info_ints(1024, 16, 64, 4096, 128) == 32 * 64 * 64
    assert nmspmm.column_info_ints(1024, 16, 64, 4096, 96) == 0


FAKE = 0x1000  # an aligned non-NULL address that is never dereferenced on the error paths


def spmm_status(**kw):
    a = dict(A=FAKE, B=FAKE, D=FAKE, ci=None, C=FAKE, M=128, N=128, K=128, W=64, window=32, kept=16, vl=32, Ns=128,
             split=1, ws=None, wsb=0)
    a.update(kw)
    return nmspmm.lib().nmspmm_spmm(a["A"], a["B"], a["D"], a["ci"], a["C"], a["M"], a["N"], a["K"], a["W"],
                                    a["window"], a["kept"], a["vl"], a["Ns"], a["split"], a["ws"], a["wsb"], None)


def test_spmm_rejects_bad_arguments_without_a_gpu():
    assert spmm_status(A=None) == 1
    assert spmm_status(C=None) == 1
    assert spmm_status(M=0) == 2
    assert spmm_status(N=96) == 2           # N % Ns
    assert spmm_status(W=60) == 2           # W % kept
    assert spmm_status(K=256) == 2          # K * kept != W * window
    assert spmm_status(vl=5) == 3
    assert spmm_status(kept=40) == 3        # kept > window
    assert spmm_status(split=0) == 5
    assert spmm_status(split=5) == 5        # more slices than windows (W / kept = 4)
    assert spmm_status(split=2) == 6        # no workspace
    assert spmm_status(split=2, ws=FAKE, wsb=16) == 6
    assert spmm_status(A=FAKE + 4) == 8


def test_noalloc_entry_rejects_bad_arguments_without_a_gpu():
    """The entry point that allocates nothing: same checks as nmspmm_spmm, and a split whose slices
    exceed the library's fixed scratch (NMSPMM_NOALLOC_MAX_BYTES, 32 MiB) is refused, all before
    the GPU is touched."""
    L = nmspmm.lib()
    call = lambda **kw: L.nmspmm_spmm_noalloc(kw.get("A", FAKE), FAKE, FAKE, None, FAKE, kw.get("M", 128),
                                              kw.get("N", 128), kw.get("K", 128), kw.get("W", 64), 32, 16, 32, 128,
                                              kw.get("split", 1), None)
    assert call(A=None) == 1
    assert call(N=96) == 2
    assert call(split=0) == 5 and call(split=5) == 5
    assert call(A=FAKE + 4) == 8
    assert nmspmm.workspace_bytes(1024, 4096, 4) > nmspmm.NOALLOC_MAX_BYTES
    assert call(M=1024, N=4096, K=1024, W=512, split=4) == 6
    assert call(M=1 << 20, N=4096, K=1024, W=512, split=16) == 6


def test_spmm_ex_rejects_unknown_flags_without_a_gpu():
    L = nmspmm.lib()
    args = [FAKE, FAKE, FAKE, None, None, FAKE, 128, 128, 128, 64, 32, 16, 32, 128, 1, None, 0]
    assert L.nmspmm_spmm_ex(*args, 8, None) == 2
    assert L.nmspmm_spmm_ex(FAKE, FAKE, FAKE, None, None, None, 128, 128, 128, 64, 32, 16, 32, 128, 1, None, 0, 1, None) == 1
    args[4] = FAKE + 4   # a row list that is not 16-byte aligned
    assert L.nmspmm_spmm_ex(*args, 0, None) == 8


def test_row_list_entry_points_reject_bad_arguments_without_a_gpu():
    L = nmspmm.lib()
    assert nmspmm.row_index_ints(1024, 8192) == 256 * 64 * 16
    assert nmspmm.row_index_ints(36, 128) == 4 * 3 * 16       # the last group is padded
    assert nmspmm.row_index_ints(0, 128) == 0 and nmspmm.row_index_ints(64, 100) == 0
    call = lambda **kw: L.nmspmm_row_index_device(kw.get("D", FAKE), FAKE, kw.get("W", 64), kw.get("N", 128),
                                                   kw.get("window", 64), kw.get("kept", 16), kw.get("Ns", 128),
                                                   kw.get("R", FAKE), None)
    assert call(D=None) == 1 and call(R=None) == 1
    assert call(kept=80) == 3
    assert call(W=60) == 2 and call(N=96) == 2 and call(Ns=48) == 2


def test_attaching_a_row_list_checks_its_arguments():
    """Without a device there is nothing to attach to (the registry is keyed by device), but the
    argument check comes first; nmspmm_release forgets attachments and never fails for that."""
    L = nmspmm.lib()
    assert L.nmspmm_row_index_attach(None, FAKE) == 1 and L.nmspmm_row_index_detach(None) == 1
    assert L.nmspmm_row_index_attach(FAKE, FAKE) in (0, 7)    # OK with a current device, NMSPMM_ERR_HIP without
    assert L.nmspmm_row_index_detach(FAKE) in (0, 7)
    assert L.nmspmm_release() == 0


def test_named_entry_points_reject_the_other_family():
    L = nmspmm.lib()
    low = lambda s, tile=128: L.nmspmm_gemm_low_sparsity(tile, FAKE, FAKE, FAKE, FAKE, 128, 128, 128, 64, s, 1, None)
    high = lambda s, ci=FAKE: L.nmspmm_gemm_high_sparsity(128, FAKE, FAKE, FAKE, ci, FAKE, 128, 128, 128, 32, s, 1, None)
    assert low(0.75) == 4 and low(0.875) == 4
    assert high(0.5) == 4 and high(0.625) == 4 and high(0.0) == 4
    assert low(0.3) == 3 and high(0.3) == 3
    assert low(0.5, tile=48) == 2
    assert high(0.75, ci=None) == 1


def test_preprocess_rejects_bad_arguments_without_a_gpu():
    L = nmspmm.lib()
    n, m = ctypes.c_int(2), ctypes.c_int(4)
    assert L.nmspmm_trans_index_host(None, 8, 64, 2, ctypes.byref(n), ctypes.byref(m)) == 1
    assert L.nmspmm_trans_index_host(FAKE, 6, 64, 2, ctypes.byref(n), ctypes.byref(m)) == 2  # odd window count
    assert (n.value, m.value) == (2, 4)
    assert L.nmspmm_preprocess_low_host(FAKE, 8, 3, 64, 32) == 2       # Q % Qs
    assert L.nmspmm_preprocess_low_host(FAKE, 8, 4, 64, 7) == 3
    assert L.nmspmm_preprocess_low_device(FAKE, FAKE, 8, 4, 64, 32, None) == 2  # in == out
    assert L.nmspmm_preprocess_high_host(None, 64, 16, FAKE, 32, 4, 128, 128, 32) == 1
    assert L.nmspmm_preprocess_high_host(FAKE, 2048, 16, FAKE, 32, 4, 128, 128, 32) == 3
    assert L.nmspmm_preprocess_high_host(FAKE, 64, 16, FAKE, 40, 4, 128, 128, 32) == 2  # W % pN
    assert L.nmspmm_status_string(4).decode().startswith("sparsity belongs")


def test_one_kernel_preprocessing_rejects_bad_arguments_without_a_gpu():
    L = nmspmm.lib()
    w, k = ctypes.c_int(0), ctypes.c_int(0)
    args = lambda **kw: [kw.get("src", FAKE), kw.get("n", 2), kw.get("m", 8), kw.get("W", 64), 4, 128, kw.get("Ns", 128),
                         kw.get("dst", FAKE + 4096), kw.get("ci", FAKE + 8192), ctypes.byref(w), ctypes.byref(k), None]
    assert L.nmspmm_preprocess_device(*args(src=None)) == 1
    assert L.nmspmm_preprocess_device(*args(ci=None)) == 1          # 2:8 needs column_info
    assert L.nmspmm_preprocess_device(*args(n=3, m=4)) == 3         # 3:4 is not a kernel sparsity
    assert L.nmspmm_preprocess_device(*args(n=3, m=24)) == 3        # 1:8, but 24 does not double to 64
    assert L.nmspmm_preprocess_device(*args(W=72)) == 2             # not whole 16-row windows
    assert L.nmspmm_preprocess_device(*args(dst=FAKE)) == 2         # in place
    assert L.nmspmm_preprocess_device(*args(Ns=96)) == 2


def test_compress_rejects_bad_arguments_without_a_gpu():
    L = nmspmm.lib()
    assert L.nmspmm_compress_device(None, 64, 64, 2, 4, 32, FAKE, FAKE, None) == 1
    assert L.nmspmm_compress_device(FAKE, 64, 64, 4, 4, 32, FAKE, FAKE, None) == 3   # n == m
    assert L.nmspmm_compress_device(FAKE, 64, 64, 2, 64, 32, FAKE, FAKE, None) == 3  # window not instantiated
    assert L.nmspmm_compress_device(FAKE, 66, 64, 2, 4, 32, FAKE, FAKE, None) == 2   # K % m
    assert L.nmspmm_decompress_device(FAKE, None, 64, 64, 2, 4, 32, FAKE, None) == 1
    assert L.nmspmm_decompress_device(FAKE, FAKE, 64, 40, 2, 4, 32, FAKE, None) == 2  # N % vec_len
    # a window of m rows is addressed through 32-bit byte offsets: m * N * 4 bytes stay below 4 GiB
    assert L.nmspmm_compress_device(FAKE, 32, (1 << 25) + 32, 8, 32, 32, FAKE, FAKE, None) == 2
    assert L.nmspmm_decompress_device(FAKE, FAKE, 8, (1 << 27) + 32, 2, 8, 32, FAKE, None) == 2


def test_rowmajor_entry_rejects_bad_arguments_without_a_gpu():
    L = nmspmm.lib()
    L.nmspmm_workspace_bytes_rowmajor.restype = ctypes.c_size_t
    assert L.nmspmm_workspace_bytes_rowmajor(64, 128, 256, 1) == 4 * 64 * 256
    assert L.nmspmm_workspace_bytes_rowmajor(61, 128, 256, 1) == 4 * 64 * 256      # row pitch rounded up to 4
    assert L.nmspmm_workspace_bytes_rowmajor(64, 128, 256, 2) == 4 * 64 * 256 + L.nmspmm_workspace_bytes(64, 128, 2)
    assert L.nmspmm_workspace_bytes_rowmajor(0, 128, 256, 1) == 0
    assert L.nmspmm_transpose_device(None, 4, 4, FAKE, None) == 1
    assert L.nmspmm_transpose_device(FAKE, 4, 0, FAKE + 64, None) == 2
    assert L.nmspmm_transpose_device(FAKE, 4, 4, FAKE, None) == 2                     # in place
    args = [FAKE, FAKE, FAKE, None, FAKE, 64, 128, 256, 128, 32, 16, 32, 128, 1]
    assert L.nmspmm_spmm_rowmajor(*args, None, 0, None) == 6                           # workspace is never optional
    assert L.nmspmm_spmm_rowmajor(*args, FAKE, 4 * 64 * 256 - 16, None) == 6


def test_split_rule_matches_reference_partition():
    """The reference kernels give the first (windows % SPLIT_K) slices one extra window
    (src/kernel_64x128_8x8.cu:20-37, '20 tasks over 8 slices: 3 3 3 3 2 2 2 2')."""
    src = open(os.path.join(ROOT, "nm-spmm_amd", "csrc", "internal.h")).read()
    assert "split_windows" in src
    p, q = divmod(20, 8)
    counts = [p + 1 if z < q else p for z in range(8)]
    begins = [z * (p + 1) if z < q else z * p + q for z in range(8)]
    assert counts == [3, 3, 3, 3, 2, 2, 2, 2]
    assert begins == list(np.cumsum([0] + counts[:-1]))


def test_python_wrappers_refuse_tensors_smaller_than_the_shape_arguments():
    """The C interface sees plain pointers; the Python mirror knows the tensors and raises before a
    kernel could read or write beyond one (nothing here reaches the GPU: CPU tensors, the check
    comes first)."""
    import torch
    M, N, K, W = 64, 128, 128, 64            # 2:4 on the (32, 16) geometry
    f = lambda n: torch.zeros(n, dtype=torch.float32)
    i = lambda n: torch.zeros(n, dtype=torch.int32)
    good = dict(A=f(K * M), B=f(W * N), D=i(W * N // 32), C=f(M * N))
    for short in ("A", "B", "D", "C"):
        t = dict(good)
        t[short] = t[short][:-1]
        with pytest.raises(ValueError, match=short):
            nmspmm.spmm(t["A"], t["B"], t["D"], None, t["C"], M, N, K, W, 32, 16)
        with pytest.raises(ValueError, match=short):
            nmspmm.spmm_ex(t["A"], t["B"], t["D"], None, t["C"], M, N, K, W, 32, 16)
    # A for 32 rows passed as 64: the mistake that reads K * 32 floats beyond the tensor
    with pytest.raises(ValueError, match="A holds"):
        nmspmm.spmm_ex(f(K * 32), good["B"], good["D"], None, good["C"], M, N, K, W, 32, 16)
    with pytest.raises(ValueError, match="row_index"):
        nmspmm.spmm_ex(good["A"], good["B"], good["D"], None, good["C"], M, N, K, W, 32, 16,
                       row_index=i(nmspmm.row_index_ints(W, N) - 1))
    with pytest.raises(ValueError, match="column_info"):   # 2:8 on the (64, 16) geometry, K = 256
        nmspmm.spmm(f(256 * M), good["B"], good["D"], i(nmspmm.column_info_ints(W, 16, 64, N, 128) - 1), good["C"],
                    M, N, 256, W, 64, 16)
    with pytest.raises(ValueError, match="dBT"):
        nmspmm.compress_device(f(K * N), K, N, 2, 4, f(W * N - 1), i(W * N // 32))
    with pytest.raises(ValueError, match="dDT_out"):
        nmspmm.preprocess_low_device(i(W * 4), i(W * 4 - 1), W, 4, 128)
    with pytest.raises(ValueError, match="dst"):
        nmspmm.transpose_device(f(M * K), M, K, f(M * K - 1))
