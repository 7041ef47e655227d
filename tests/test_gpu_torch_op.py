"""The nn.Linear stand-in on the GPU: its output equals a dense fp64 linear layer with the pruned
weight, and the pruning it applied is the library's compression rule."""
import importlib

import numpy as np
import pytest

from conftest import REL_TOL, nmspmm, scaled_max_error

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.mark.parametrize("out_f,in_f,n,m,lead,bias", [(256, 512, 2, 4, (64,), True), (384, 1024, 2, 8, (4, 32), False),
                                                      (128, 512, 1, 8, (8,), True), (96, 256, 3, 8, (2, 3, 4), True),
                                                      (512, 512, 2, 8, (1,), False), (256, 256, 2, 4, (7,), True)])
def test_linear_standin_matches_dense_layer_with_pruned_weight(oracle, out_f, in_f, n, m, lead, bias):
    op = importlib.import_module("nm-spmm_amd.torch_op")
    g = torch.Generator(device="cuda").manual_seed(out_f + in_f + n)
    w = torch.randn((out_f, in_f), generator=g, dtype=torch.float32, device="cuda") * 0.05
    b = torch.randn((out_f,), generator=g, dtype=torch.float32, device="cuda") if bias else None
    x = torch.randn((*lead, in_f), generator=g, dtype=torch.float32, device="cuda")
    layer = op.NMSparseLinear(w, n, m, b)
    y = layer(x)
    assert y.shape == (*lead, out_f)
    # the pruned weight, by the CPU checker's compression of the same matrix
    BT, DT = oracle.compress(w.t().contiguous().cpu().numpy(), n, m)
    K, N, W = in_f, out_f, BT.shape[0]
    pruned = np.zeros((K, N), np.float32)
    rows = (np.arange(W) // n * m)[:, None] + DT
    pruned[np.repeat(rows, 32, axis=1), np.broadcast_to(np.arange(N), (W, N))] = BT
    want = x.reshape(-1, K).double().cpu().numpy() @ pruned.astype(np.float64)
    if bias:
        want = want + b.double().cpu().numpy()
    assert scaled_max_error(y.reshape(-1, N).cpu().numpy(), want) <= REL_TOL
    # and the layer's own view of its weight is that pruned matrix, exactly
    assert np.array_equal(layer.dense_weight().cpu().numpy(), pruned.T)


def test_decode_sized_forward_of_a_layer_with_few_output_features_on_one_stream(oracle):
    """single_stream=True: a decode-sized forward of a layer with fewer than 256 groups of 32 output
    features and a long reduction cuts its reductions across workgroups; same result within the
    bound, and row-major activations are read in place (8 rows) or copied (24 and 48 rows; at 48
    rows the library chooses between the decode kernel and the tile kernel)."""
    op = importlib.import_module("nm-spmm_amd.torch_op")
    g = torch.Generator(device="cuda").manual_seed(5)
    w = torch.randn((2048, 8192), generator=g, dtype=torch.float32, device="cuda") * 0.05
    plain = op.NMSparseLinear(w, 2, 8)
    split = op.NMSparseLinear(w, 2, 8, single_stream=True)
    for rows in (1, 8, 24, 48):
        x = torch.randn((rows, 8192), generator=g, dtype=torch.float32, device="cuda")
        y0, y1 = plain(x), split(x)
        assert nmspmm.last_kernel() in (("decode",) if rows <= 32 else ("decode", "mfma"))
        want = x.double() @ plain.dense_weight().double().t()
        assert scaled_max_error(y1.cpu().numpy(), want.cpu().numpy()) <= REL_TOL
        assert scaled_max_error(y0.cpu().numpy(), want.cpu().numpy()) <= REL_TOL


def test_rejects_unsupported_layers():
    op = importlib.import_module("nm-spmm_amd.torch_op")
    w = torch.zeros((64, 80), dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError):
        op.NMSparseLinear(w, 2, 4)            # in_features not a multiple of the window
    with pytest.raises(ValueError):
        op.NMSparseLinear(torch.zeros((64, 128), dtype=torch.float32, device="cuda"), 3, 4)
    with pytest.raises(ValueError):
        op.NMSparseLinear(torch.zeros((48, 128), dtype=torch.float32, device="cuda"), 2, 4)
