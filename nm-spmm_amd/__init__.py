"""ctypes binding of libnmspmm.so, the MI355X N:M sparse x dense fp32 library.

The product is the shared library (C-ABI in include/nmspmm.h, C++ drop-in in include/NM-SpMM.h);
this module only loads it and forwards torch device pointers, for the Python tests and the
benchmark.  There is no CPU fallback: if the library has not been built, importing works but
every call raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnmspmm.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

OK = 0
STATUS_NAMES = {
    0: "NMSPMM_OK", 1: "NMSPMM_ERR_NULL_POINTER", 2: "NMSPMM_ERR_BAD_SHAPE", 3: "NMSPMM_ERR_BAD_PATTERN",
    4: "NMSPMM_ERR_WRONG_PATH", 5: "NMSPMM_ERR_BAD_SPLIT", 6: "NMSPMM_ERR_WORKSPACE", 7: "NMSPMM_ERR_HIP",
    8: "NMSPMM_ERR_ALIGNMENT",
}
TILE_SMALL, TILE_MEDIUM, TILE_LARGE, TILE_HUGE = 32, 64, 64, 128
ACCUMULATE = 1  # flag of spmm_ex: with split_k > 1 the product is added to what C holds
STREAM_B = 2    # flag of spmm_ex: B is loaded with the non-temporal hint (decode kernel on the row list)
DECODE_SPLIT = 4  # flag of spmm_ex: the decode kernel may cut reductions across workgroups (library scratch)


class NmSpmmError(RuntimeError):
    def __init__(self, fn, status):
        self.status = status
        super().__init__("%s failed: %s" % (fn, STATUS_NAMES.get(status, status)))


_lib = None


def lib():
    """The loaded library; raises if it has not been built (no silent fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libnmspmm.so is not built: run `make -C %s` (or __graft_entry__.build())" % CSRC_DIR)
        L = ctypes.CDLL(LIB_PATH)
        c_int, c_void_p, c_float, c_size_t = ctypes.c_int, ctypes.c_void_p, ctypes.c_float, ctypes.c_size_t
        ip = ctypes.POINTER(ctypes.c_int)
        L.nmspmm_version.restype = c_int
        L.nmspmm_status_string.restype = ctypes.c_char_p
        L.nmspmm_status_string.argtypes = [c_int]
        L.nmspmm_last_kernel.restype = ctypes.c_char_p
        L.nmspmm_pattern_from_sparsity.argtypes = [c_float, ip, ip, ip]
        L.nmspmm_trans_index_host.argtypes = [c_void_p, c_int, c_int, c_int, ip, ip]
        L.nmspmm_trans_index_device.argtypes = [c_void_p, c_int, c_int, c_int, ip, ip, c_void_p]
        L.nmspmm_preprocess_low_host.argtypes = [c_void_p] + [c_int] * 4
        L.nmspmm_preprocess_low_device.argtypes = [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]
        L.nmspmm_preprocess_high_host.argtypes = [c_void_p, c_int, c_int, c_void_p] + [c_int] * 5
        L.nmspmm_preprocess_high_device.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p] + [c_int] * 5 + [c_void_p]
        L.nmspmm_compress_device.argtypes = [c_void_p] + [c_int] * 5 + [c_void_p, c_void_p, c_void_p]
        L.nmspmm_decompress_device.argtypes = [c_void_p, c_void_p] + [c_int] * 5 + [c_void_p, c_void_p]
        L.nmspmm_preprocess_device.argtypes = [c_void_p] + [c_int] * 6 + [c_void_p, c_void_p, ip, ip, c_void_p]
        L.nmspmm_column_info_ints.restype = c_size_t
        L.nmspmm_column_info_ints.argtypes = [c_int] * 5
        L.nmspmm_workspace_bytes.restype = c_size_t
        L.nmspmm_workspace_bytes.argtypes = [c_int] * 3
        L.nmspmm_spmm.argtypes = [c_void_p] * 5 + [c_int] * 9 + [c_void_p, c_size_t, c_void_p]
        L.nmspmm_spmm_ex.argtypes = [c_void_p] * 6 + [c_int] * 9 + [c_void_p, c_size_t, ctypes.c_uint, c_void_p]
        L.nmspmm_row_index_ints.restype = c_size_t
        L.nmspmm_row_index_ints.argtypes = [c_int] * 2
        L.nmspmm_row_index_device.argtypes = [c_void_p, c_void_p] + [c_int] * 5 + [c_void_p, c_void_p]
        L.nmspmm_row_index_attach.argtypes = [c_void_p, c_void_p]
        L.nmspmm_row_index_detach.argtypes = [c_void_p]
        L.nmspmm_spmm_noalloc.argtypes = [c_void_p] * 5 + [c_int] * 9 + [c_void_p]
        L.nmspmm_gemm_low_sparsity.argtypes = [c_int] + [c_void_p] * 4 + [c_int] * 4 + [c_float, c_int, c_void_p]
        L.nmspmm_gemm_high_sparsity.argtypes = [c_int] + [c_void_p] * 5 + [c_int] * 4 + [c_float, c_int, c_void_p]
        L.nmspmm_transpose_device.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p]
        L.nmspmm_workspace_bytes_rowmajor.restype = c_size_t
        L.nmspmm_workspace_bytes_rowmajor.argtypes = [c_int] * 4
        L.nmspmm_spmm_rowmajor.argtypes = [c_void_p] * 5 + [c_int] * 9 + [c_void_p, c_size_t, c_void_p]
        L.nmspmm_spmm_rowmajor_ex.argtypes = [c_void_p] * 6 + [c_int] * 9 + [c_void_p, c_size_t, ctypes.c_uint, c_void_p]
        L.nmspmm_suggest_split_k.argtypes = [c_int] * 4
        L.nmspmm_waves_along_k_rows.argtypes = [c_int] * 4
        L.nmspmm_waves_along_k_count.argtypes = [c_int] * 4
        L.nmspmm_rows_apart.argtypes = [c_int] * 4
        L.nmspmm_tile_wave_rows.argtypes = [c_int] * 6
        L.nmspmm_tile_wave_sets.argtypes = [c_int] * 6
        L.nmspmm_device_figures.argtypes = [ip, ip, ctypes.POINTER(ctypes.c_double)]
        L.nmspmm_gemm_auto.argtypes = [c_void_p] * 5 + [c_int] * 4 + [c_float, c_void_p]
        L.nmspmm_release.restype = c_int
        _lib = L
    return _lib


def _check(fn, status):
    if status != OK:
        raise NmSpmmError(fn, status)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(fn, **tensors):
    """The C interface takes plain pointers and cannot see how much memory lies behind them; a
    tensor smaller than the shape arguments imply would make a kernel read or write beyond it (a
    GPU memory fault).  name=(tensor, elements): raises ValueError when the tensor holds fewer.
    None and shapes the library rejects anyway (non-positive counts) are left to the library."""
    for name, (t, count) in tensors.items():
        if t is None or not isinstance(count, int) or count <= 0:
            continue
        if t.numel() < count:
            raise ValueError("%s: %s holds %d elements, the shape arguments need %d" % (fn, name, t.numel(), count))


def _spmm_need(fn, A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len, Ns, row_index=None, a_elems=None):
    ok = all(isinstance(v, int) and v > 0 for v in (M, N, K, W, window, kept, vec_len, Ns))
    if not ok:
        return
    _need(fn, A=(A, a_elems if a_elems is not None else K * M), B=(B, W * N), D=(D, W * (N // vec_len)),
          C=(C, M * N), column_info=(cinfo, int(lib().nmspmm_column_info_ints(W, kept, window, N, Ns))),
          row_index=(row_index, int(lib().nmspmm_row_index_ints(W, N))))


def pattern_from_sparsity(sparsity):
    w, k, h = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _check("nmspmm_pattern_from_sparsity",
           lib().nmspmm_pattern_from_sparsity(sparsity, ctypes.byref(w), ctypes.byref(k), ctypes.byref(h)))
    return w.value, k.value, bool(h.value)


def last_kernel():
    return lib().nmspmm_last_kernel().decode()


def row_index_attach(dD, row_index):
    """From now on the named launchers pass `row_index` on when they are handed this D (both stay
    alive and unchanged while attached); None detaches."""
    _check("nmspmm_row_index_attach", lib().nmspmm_row_index_attach(_ptr(dD), _ptr(row_index)))


def release():
    """Frees what the library keeps per device (cached workspaces, staging); the caller makes sure
    no launch that uses them is still pending."""
    _check("nmspmm_release", lib().nmspmm_release())


# ---- device-pointer forms: arguments are torch tensors on the GPU -----------------------------------

def trans_index_device(dDT, W, N, Q, pN, pM):
    _need("trans_index_device", dDT=(dDT, W * Q))
    n, m = ctypes.c_int(pN), ctypes.c_int(pM)
    _check("nmspmm_trans_index_device",
           lib().nmspmm_trans_index_device(_ptr(dDT), W, N, Q, ctypes.byref(n), ctypes.byref(m), _stream()))
    return n.value, m.value


def preprocess_low_device(dDT_in, dDT_out, W, Q, Ns, vec_len=32):
    _need("preprocess_low_device", dDT_in=(dDT_in, W * Q), dDT_out=(dDT_out, W * Q))
    _check("nmspmm_preprocess_low_device",
           lib().nmspmm_preprocess_low_device(_ptr(dDT_in), _ptr(dDT_out), W, Q, Ns, vec_len, _stream()))


def preprocess_high_device(d_cinfo, pM, pN, dDT_in, dDT_out, W, Q, N, Ns, vec_len=32):
    _need("preprocess_high_device", dDT_in=(dDT_in, W * Q), dDT_out=(dDT_out, W * Q),
          column_info=(d_cinfo, int(column_info_ints(W, pN, pM, N, Ns))))
    _check("nmspmm_preprocess_high_device",
           lib().nmspmm_preprocess_high_device(_ptr(d_cinfo), pM, pN, _ptr(dDT_in), _ptr(dDT_out), W, Q, N, Ns,
                                               vec_len, _stream()))


def compress_device(dB, K, N, n, m, dBT, dDT, vec_len=32):
    """Dense row-major float32[K][N] on the GPU -> BT float32[K*n/m][N], DT int32[K*n/m][N/vec_len]."""
    if min(K, N, n, m, vec_len) > 0:
        _need("compress_device", dB=(dB, K * N), dBT=(dBT, K // m * n * N), dDT=(dDT, K // m * n * (N // vec_len)))
    _check("nmspmm_compress_device",
           lib().nmspmm_compress_device(_ptr(dB), K, N, n, m, vec_len, _ptr(dBT), _ptr(dDT), _stream()))


def decompress_device(dBT, dDT, K, N, n, m, dB, vec_len=32):
    if min(K, N, n, m, vec_len) > 0:
        _need("decompress_device", dB=(dB, K * N), dBT=(dBT, K // m * n * N), dDT=(dDT, K // m * n * (N // vec_len)))
    _check("nmspmm_decompress_device",
           lib().nmspmm_decompress_device(_ptr(dBT), _ptr(dDT), K, N, n, m, vec_len, _ptr(dB), _stream()))


def preprocess_device(dDT_in, n, m, W, Q, N, Ns, dD_out, d_cinfo):
    """Widening + re-blocking (+ ranking) in one kernel; returns (window, kept)."""
    window, kept = ctypes.c_int(0), ctypes.c_int(0)
    _need("preprocess_device", dDT_in=(dDT_in, W * Q), dD_out=(dD_out, W * Q))
    _check("nmspmm_preprocess_device",
           lib().nmspmm_preprocess_device(_ptr(dDT_in), n, m, W, Q, N, Ns, _ptr(dD_out), _ptr(d_cinfo),
                                          ctypes.byref(window), ctypes.byref(kept), _stream()))
    return window.value, kept.value


def column_info_ints(W, pN, pM, N, Ns):
    return lib().nmspmm_column_info_ints(W, pN, pM, N, Ns)


def workspace_bytes(M, N, split_k):
    return lib().nmspmm_workspace_bytes(M, N, split_k)


def spmm(A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len=32, Ns=128, split_k=1, workspace=None):
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _spmm_need("spmm", A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len, Ns)
    _check("nmspmm_spmm",
           lib().nmspmm_spmm(_ptr(A), _ptr(B), _ptr(D), _ptr(cinfo), _ptr(C), M, N, K, W, window, kept, vec_len,
                             Ns, split_k, _ptr(workspace), ws_bytes, _stream()))


def spmm_ex(A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len=32, Ns=128, split_k=1, workspace=None, flags=0,
            row_index=None):
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _spmm_need("spmm_ex", A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len, Ns, row_index)
    _check("nmspmm_spmm_ex",
           lib().nmspmm_spmm_ex(_ptr(A), _ptr(B), _ptr(D), _ptr(cinfo), _ptr(row_index), _ptr(C), M, N, K, W, window,
                                kept, vec_len, Ns, split_k, _ptr(workspace), ws_bytes, flags, _stream()))


def row_index_ints(W, N):
    return lib().nmspmm_row_index_ints(W, N)


def row_index_device(D, cinfo, W, N, window, kept, Ns, row_index):
    """Row list for the decode kernel from the preprocessed D (and column_info)."""
    if min(W, N) > 0:
        _need("row_index_device", D=(D, W * (N // 32)), row_index=(row_index, int(row_index_ints(W, N))))
    _check("nmspmm_row_index_device",
           lib().nmspmm_row_index_device(_ptr(D), _ptr(cinfo), W, N, window, kept, Ns, _ptr(row_index), _stream()))


NOALLOC_MAX_BYTES = 32 << 20  # NMSPMM_NOALLOC_MAX_BYTES


def spmm_noalloc(A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len=32, Ns=128, split_k=1):
    """spmm with the split-K slices in the library's fixed device-resident scratch: allocates nothing."""
    _spmm_need("spmm_noalloc", A, B, D, cinfo, C, M, N, K, W, window, kept, vec_len, Ns)
    _check("nmspmm_spmm_noalloc",
           lib().nmspmm_spmm_noalloc(_ptr(A), _ptr(B), _ptr(D), _ptr(cinfo), _ptr(C), M, N, K, W, window, kept,
                                     vec_len, Ns, split_k, _stream()))


def gemm_low_sparsity(tile, A, B, D, C, M, N, K, W, sparsity, split_k=1):
    _need("gemm_low_sparsity", A=(A, K * M), B=(B, W * N), D=(D, W * (N // 32)), C=(C, M * N))
    _check("nmspmm_gemm_low_sparsity",
           lib().nmspmm_gemm_low_sparsity(tile, _ptr(A), _ptr(B), _ptr(D), _ptr(C), M, N, K, W, sparsity, split_k,
                                          _stream()))


def gemm_high_sparsity(tile, A, B, D, cinfo, C, M, N, K, W, sparsity, split_k=1):
    _need("gemm_high_sparsity", A=(A, K * M), B=(B, W * N), D=(D, W * (N // 32)), C=(C, M * N))
    _check("nmspmm_gemm_high_sparsity",
           lib().nmspmm_gemm_high_sparsity(tile, _ptr(A), _ptr(B), _ptr(D), _ptr(cinfo), _ptr(C), M, N, K, W,
                                           sparsity, split_k, _stream()))


# ---- host-pointer forms: arguments are C-contiguous numpy int32 arrays, updated in place ----------

def transpose_device(src, rows, cols, dst):
    _need("transpose_device", src=(src, rows * cols), dst=(dst, rows * cols))
    _check("nmspmm_transpose_device", lib().nmspmm_transpose_device(_ptr(src), rows, cols, _ptr(dst), _stream()))


def workspace_bytes_rowmajor(M, N, K, split_k):
    return lib().nmspmm_workspace_bytes_rowmajor(M, N, K, split_k)


def spmm_rowmajor(A_rm, B, D, cinfo, C, M, N, K, W, window, kept, workspace, vec_len=32, Ns=128, split_k=1,
                  row_index=None, flags=0):
    """A_rm is row-major M x K; `workspace` (float32 tensor) holds workspace_bytes_rowmajor() bytes."""
    _spmm_need("spmm_rowmajor", A_rm, B, D, cinfo, C, M, N, K, W, window, kept, vec_len, Ns, row_index)
    _check("nmspmm_spmm_rowmajor_ex",
           lib().nmspmm_spmm_rowmajor_ex(_ptr(A_rm), _ptr(B), _ptr(D), _ptr(cinfo), _ptr(row_index), _ptr(C), M, N, K, W,
                                         window, kept, vec_len, Ns, split_k, _ptr(workspace),
                                         workspace.numel() * workspace.element_size(), flags, _stream()))


def suggest_split_k(M, N, W, kept):
    return lib().nmspmm_suggest_split_k(M, N, W, kept)


def waves_along_k_rows(M, N, W, kept):
    """128 or 64 when an unsplit multiplication of this shape shares the reduction between the
    waves of a workgroup, 0 otherwise."""
    return lib().nmspmm_waves_along_k_rows(M, N, W, kept)


def rows_apart(M, N, W, kept):
    """Last rows (1 to 32) that an unsplit tile-kernel call of this shape hands to the decode-sized kernels, else 0."""
    return lib().nmspmm_rows_apart(M, N, W, kept)


def waves_along_k_count(M, N, W, kept):
    """Waves per workgroup (4 or 8) of the launch with waves along K, 0 where that launch is not taken."""
    return lib().nmspmm_waves_along_k_count(M, N, W, kept)


def device_figures():
    """(compute units, dies, clock in Hz) the library's planning assumes for the current device."""
    cus, dies, clock = ctypes.c_int(), ctypes.c_int(), ctypes.c_double()
    _check("nmspmm_device_figures", lib().nmspmm_device_figures(ctypes.byref(cus), ctypes.byref(dies), ctypes.byref(clock)))
    return cus.value, dies.value, clock.value


def tile_wave_rows(M, N, W, kept, Ns=128, split_k=1):
    """Rows per wave of the tile kernel for this call (256, 128, 64), 0 for the launch with waves along K."""
    return lib().nmspmm_tile_wave_rows(M, N, W, kept, Ns, split_k)


def tile_wave_sets(M, N, W, kept, Ns=128, split_k=1):
    """Sets of four waves per workgroup of the tile kernel for this call (2: each set takes half of the windows)."""
    return lib().nmspmm_tile_wave_sets(M, N, W, kept, Ns, split_k)


def gemm_auto(A, B, D, cinfo, C, M, N, K, W, sparsity):
    """Multiply with the library's own choice of split_k (indices preprocessed for Ns = 128)."""
    _need("gemm_auto", A=(A, K * M), B=(B, W * N), D=(D, W * (N // 32)), C=(C, M * N))
    _check("nmspmm_gemm_auto",
           lib().nmspmm_gemm_auto(_ptr(A), _ptr(B), _ptr(D), _ptr(cinfo), _ptr(C), M, N, K, W, sparsity, _stream()))


def _np_ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def trans_index_host(DT, W, N, Q, pN, pM):
    n, m = ctypes.c_int(pN), ctypes.c_int(pM)
    _check("nmspmm_trans_index_host",
           lib().nmspmm_trans_index_host(_np_ptr(DT), W, N, Q, ctypes.byref(n), ctypes.byref(m)))
    return n.value, m.value


def preprocess_low_host(DT, W, Q, Ns, vec_len=32):
    _check("nmspmm_preprocess_low_host", lib().nmspmm_preprocess_low_host(_np_ptr(DT), W, Q, Ns, vec_len))


def preprocess_high_host(cinfo, pM, pN, DT, W, Q, N, Ns, vec_len=32):
    _check("nmspmm_preprocess_high_host",
           lib().nmspmm_preprocess_high_host(_np_ptr(cinfo), pM, pN, _np_ptr(DT), W, Q, N, Ns, vec_len))
