"""A drop-in for torch.nn.Linear (inference) whose weight is N:M vector-sparse and whose forward
runs the library's kernels: dense weight -> compress -> widen / preprocess once at construction,
then one row-major multiplication per call.  PyTorch only supplies device memory and the stream.

The multiplication is registered with torch.library as the operator `nmspmm::sparse_linear`
(with a fake implementation that only derives the output's shape), so that tracing front ends
(torch.compile, torch.export) see one opaque node instead of a Python function they cannot follow.

The reference has no framework binding; its driver multiplies synthetic operands
(tests/test_nmspmm.cu:72-97).  The sequence of calls here is that driver's, on real weights.
"""
import importlib
from typing import Optional

import torch

_nm = importlib.import_module(__name__.rsplit(".", 1)[0])

# (n, m) reduced to lowest terms -> (window, kept) the kernels run the pattern at
# (reference launchers, src/kernel_64x128_8x8.cu:264-289,584-602)
_GEOMETRY = {(1, 2): (32, 16), (3, 8): (32, 12), (1, 4): (64, 16), (1, 8): (64, 8)}


def _geometry(n, m):
    from math import gcd
    g = gcd(n, m)
    if (n // g, m // g) not in _GEOMETRY:
        raise ValueError("pattern %d:%d is not one of 1:2, 3:8, 1:4, 1:8 (or a multiple of them)" % (n, m))
    window, kept = _GEOMETRY[(n // g, m // g)]
    if window % m != 0:
        raise ValueError("pattern window %d does not divide the kernel window %d" % (m, window))
    return window, kept


_plans = {}  # (M, N, K, W, kept) -> (split, workspace floats): two library calls per shape, not per forward


@torch.library.custom_op("nmspmm::sparse_linear", mutates_args=(), device_types="cuda")
def sparse_linear(x: torch.Tensor, values: torch.Tensor, indices: torch.Tensor, column_info: Optional[torch.Tensor],
                  row_index: Optional[torch.Tensor], bias: Optional[torch.Tensor], window: int, kept: int, Ns: int,
                  flags: int) -> torch.Tensor:
    """x [..., K] row-major times the compressed weight (values [W, N], preprocessed indices,
    column_info for 64-row windows, optional row list) plus bias: [..., N].  The library's own
    choice of kernel and split; the workspace comes from torch's caching allocator."""
    W, N = values.shape
    K = x.shape[-1]
    x2 = x.reshape(-1, K).contiguous()
    M = x2.shape[0]
    y = torch.empty((M, N), dtype=torch.float32, device=x.device)
    if M > 0:
        key = (M, N, K, W, kept)
        if key not in _plans:
            split = _nm.suggest_split_k(M, N, W, kept)
            _plans[key] = (split, _nm.workspace_bytes_rowmajor(M, N, K, split) // 4)
        split, need = _plans[key]
        workspace = torch.empty(max(need, 4), dtype=torch.float32, device=x.device)
        _nm.spmm_rowmajor(x2, values, indices, column_info, y, M, N, K, W, window, kept, workspace, 32, Ns, split,
                          row_index, flags)
        if bias is not None:
            y += bias
    return y.reshape(*x.shape[:-1], N)


@sparse_linear.register_fake
def _sparse_linear_fake(x, values, indices, column_info, row_index, bias, window, kept, Ns, flags):
    return x.new_empty((*x.shape[:-1], values.shape[1]))


class NMSparseLinear(torch.nn.Module):
    """y = x @ prune(weight).T + bias with an n:m pattern shared by 32 adjacent output features.

    weight: float32 CUDA tensor [out_features, in_features]; in_features % window == 0 and
    out_features % 32 == 0.  Leading dimensions of x are flattened into rows; any row count runs on
    the matrix-core kernels (the copy of x the row-major entry point makes is padded to a row pitch
    of a multiple of four floats).  single_stream=True promises that all forwards of such modules
    are issued on one stream at a time; up to 64 rows they may then use more of the GPU when
    out_features is small (fewer than 256 groups of 32).
    """

    def __init__(self, weight, n, m, bias=None, single_stream=False):
        super().__init__()
        # single_stream: the caller issues every forward of every such module on one stream at a
        # time, which lets decode-sized calls cut their reductions across workgroups through the
        # library's device-resident scratch (nmspmm.h: NMSPMM_DECODE_SPLIT)
        self.flags = _nm.DECODE_SPLIT if single_stream else 0
        if weight.dtype != torch.float32 or not weight.is_cuda or weight.dim() != 2:
            raise ValueError("weight must be a 2-D float32 CUDA tensor")
        self.out_features, self.in_features = weight.shape
        self.n, self.m = n, m
        self.window, self.kept = _geometry(n, m)
        N, K = self.out_features, self.in_features
        if K % self.window != 0 or N % 32 != 0:
            raise ValueError("in_features must be a multiple of %d and out_features of 32" % self.window)
        self.Ns = 128 if N % 128 == 0 else 64 if N % 64 == 0 else 32
        self.W, self.Q = K // m * n, N // 32
        dense = weight.t().contiguous()                                   # K x N, row-major
        BT = torch.empty((self.W, N), dtype=torch.float32, device=weight.device)
        DT = torch.empty((self.W, self.Q), dtype=torch.int32, device=weight.device)
        _nm.compress_device(dense, K, N, n, m, BT, DT)
        D = torch.empty_like(DT)
        cinfo = None
        if self.window == 64:
            cinfo = torch.empty(_nm.column_info_ints(self.W, self.kept, self.window, N, self.Ns), dtype=torch.int32,
                                device=weight.device)
        got = _nm.preprocess_device(DT, n, m, self.W, self.Q, N, self.Ns, D, cinfo)
        assert got == (self.window, self.kept)
        # the row list: the index form the decode kernel (up to 64 rows) reads
        rows = torch.empty(_nm.row_index_ints(self.W, N), dtype=torch.int32, device=weight.device)
        _nm.row_index_device(D, cinfo, self.W, N, self.window, self.kept, self.Ns, rows)
        self.register_buffer("values", BT)
        self.register_buffer("indices", D.reshape(-1))
        self.register_buffer("column_info", cinfo)
        self.register_buffer("row_index", rows)
        self.register_buffer("bias", None if bias is None else bias.detach().to(torch.float32))

    def dense_weight(self):
        """The pruned weight as a dense [out_features, in_features] tensor (for checking)."""
        # undo the preprocessing by compressing the expansion instead of storing DT twice: the kept
        # values are in `values`, their rows are recovered from a multiplication with the identity
        eye = torch.eye(self.in_features, dtype=torch.float32, device=self.values.device)
        return self.forward(eye, add_bias=False).t().contiguous()

    def forward(self, x, add_bias=True):
        if x.dtype != torch.float32 or not x.is_cuda or x.shape[-1] != self.in_features:
            raise ValueError("x must be a float32 CUDA tensor whose last dimension is in_features")
        return sparse_linear(x, self.values, self.indices, self.column_info, self.row_index,
                             self.bias if add_bias else None, self.window, self.kept, self.Ns, self.flags)

    def extra_repr(self):
        return "in_features=%d, out_features=%d, pattern=%d:%d, bias=%s" % (
            self.in_features, self.out_features, self.n, self.m, self.bias is not None)
