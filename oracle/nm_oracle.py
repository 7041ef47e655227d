"""TEST INFRASTRUCTURE: ctypes doorway onto the CPU checker (never imported by the library).

`Oracle` wraps oracle/libnm_oracle.so, our restatement of the reference's host-side algorithm
(nm_oracle.cpp names the reference lines).  `Reference` wraps oracle/_ref/libnmref.so, the
reference project's own host code compiled as is by oracle/Makefile; it exists wherever that
library was built (it travels with the tree as a binary, the reference sources do not).

Layouts follow reference include/utils.h:10-66: A column-major M x K, B column-major W x N,
D column-major W x Q with global K indices, BT / DT row-major (DT window-local), C row-major.
All arrays here are flat, C-contiguous numpy buffers in exactly those element orders.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "libnm_oracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libnmref.so")

_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_int = ctypes.c_int
_intp = ctypes.POINTER(ctypes.c_int)


def build(force=False):
    """Compile the checker (and the reference half when /root/reference is present)."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


class Oracle:
    def __init__(self):
        if not os.path.exists(_ORACLE_SO):
            build()
        lib = ctypes.CDLL(_ORACLE_SO)
        lib.nm_oracle_threads.restype = _int
        lib.nm_oracle_trans_index.argtypes = [_i32p, _int, _int, _intp, _intp]
        lib.nm_oracle_preprocess_low.argtypes = [_i32p, _int, _int, _int, _int]
        lib.nm_oracle_preprocess_high.argtypes = [_i32p, _int, _int, _i32p, _int, _int, _int, _int]
        lib.nm_oracle_gemm_cpu.argtypes = [_f32p, _f32p, _i32p, _f32p] + [_int] * 6
        lib.nm_oracle_decompress.argtypes = [_f32p, _i32p, _f32p] + [_int] * 4
        lib.nm_oracle_compress.argtypes = [_f32p] + [_int] * 5 + [_f32p, _i32p]
        lib.nm_oracle_row_index.argtypes = [_i32p, ctypes.c_void_p] + [_int] * 5 + [_i32p]
        for f in ("trans_index", "preprocess_low", "preprocess_high", "gemm_cpu", "decompress", "compress", "row_index"):
            getattr(lib, "nm_oracle_" + f).restype = None
        self.lib = lib

    def threads(self):
        return self.lib.nm_oracle_threads()

    def trans_index(self, DT, W, Q, pN, pM):
        """In place on DT; returns the doubled (pN, pM)."""
        n, m = ctypes.c_int(pN), ctypes.c_int(pM)
        self.lib.nm_oracle_trans_index(DT, W, Q, ctypes.byref(n), ctypes.byref(m))
        return n.value, m.value

    def preprocess_low(self, DT, W, Q, Ns, vec_len=32):
        self.lib.nm_oracle_preprocess_low(DT, W, Q, Ns, vec_len)

    def preprocess_high(self, pM, pN, DT, W, Q, Ns, vec_len=32):
        """In place on DT; returns column_info int32[(Q/Qs) * (W/pN) * pM]."""
        Qs = Ns // vec_len
        ci = np.empty((Q // Qs) * (W // pN) * pM, np.int32)
        self.lib.nm_oracle_preprocess_high(ci, pM, pN, DT, W, Q, Ns, vec_len)
        return ci

    def gemm_cpu(self, A, B, D, M, N, W, vec_len=32, rows=None, C=None):
        """C (row-major M x N, zero unless given) += A . B over rows [rows[0], rows[1])."""
        if C is None:
            C = np.zeros(M * N, np.float32)
        r0, r1 = (0, M) if rows is None else rows
        self.lib.nm_oracle_gemm_cpu(A, B, D, C, M, N, W, vec_len, r0, r1)
        return C

    def row_index(self, D, cinfo, W, N, window, kept, Ns):
        """Row list int32[(N/32) * ceil(W/16) * 16] from the preprocessed D (and column_info or None)."""
        R = np.empty((N // 32) * ((W + 15) // 16) * 16, np.int32)
        ci = None if cinfo is None else cinfo.ctypes.data_as(ctypes.c_void_p)
        self.lib.nm_oracle_row_index(D, ci, W, N, window, kept, Ns, R)
        return R

    def decompress(self, B, D, K, N, W, vec_len=32):
        dense = np.empty(K * N, np.float32)
        self.lib.nm_oracle_decompress(B, D, dense, K, N, W, vec_len)
        return dense.reshape(K, N)


    def compress(self, dense, n, m, vec_len=32):
        """dense row-major float32[K][N] -> (BT float32[W][N], DT int32[W][N/vec_len])."""
        K, N = dense.shape
        W = K // m * n
        BT = np.empty((W, N), np.float32)
        DT = np.empty((W, N // vec_len), np.int32)
        self.lib.nm_oracle_compress(np.ascontiguousarray(dense, np.float32).reshape(-1), K, N, n, m, vec_len,
                                    BT.reshape(-1), DT.reshape(-1))
        return BT, DT


class Reference:
    """The reference's own host functions (VEC_LEN fixed at 32 by its header)."""

    @staticmethod
    def available():
        return os.path.exists(_REF_SO)

    def __init__(self):
        lib = ctypes.CDLL(_REF_SO)
        lib.nmref_vec_len.restype = _int
        lib.nmref_trans_index.argtypes = [_i32p, _int, _int, _int, _intp, _intp]
        lib.nmref_preprocess_low.argtypes = [_i32p, _int, _int, _int]
        lib.nmref_preprocess_high.argtypes = [_i32p, _int, _int, _i32p, _int, _int, _int, _int]
        lib.nmref_gemm_cpu.argtypes = [_f32p, _f32p, _i32p, _f32p] + [_int] * 4
        lib.nmref_allclose.argtypes = [_f32p, _f32p, _int]
        lib.nmref_allclose.restype = _int
        for f in ("trans_index", "preprocess_low", "preprocess_high", "gemm_cpu"):
            getattr(lib, "nmref_" + f).restype = None
        self.lib = lib
        assert lib.nmref_vec_len() == 32

    def trans_index(self, DT, W, N, Q, pN, pM):
        n, m = ctypes.c_int(pN), ctypes.c_int(pM)
        self.lib.nmref_trans_index(DT, W, N, Q, ctypes.byref(n), ctypes.byref(m))
        return n.value, m.value

    def preprocess_low(self, DT, W, Q, Ns):
        self.lib.nmref_preprocess_low(DT, W, Q, Ns)

    def preprocess_high(self, pM, pN, DT, W, Q, N, Ns, slack=True):
        """Returns column_info sized as the reference driver does (tests/test_nmspmm.cu:23 gives
        payload + one window of slack); the slack is pre-filled with a sentinel to show that the
        reference never writes it."""
        n = (W // pN) * (N // Ns) * pM
        ci = np.full(n + (pM if slack else 0), -12345, np.int32)
        self.lib.nmref_preprocess_high(ci, pM, pN, DT, W, Q, N, Ns)
        return ci

    def gemm_cpu(self, A, B, D, M, N, K, W, C=None):
        if C is None:
            C = np.zeros(M * N, np.float32)
        self.lib.nmref_gemm_cpu(A, B, D, C, M, N, K, W)
        return C

    def allclose(self, a, b):
        return bool(self.lib.nmref_allclose(a, b, a.size))
