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


class TwoLayers(torch.nn.Module):
    def __init__(self, first, second):
        super().__init__()
        self.first, self.second = first, second

    def forward(self, x):
        return self.second(torch.nn.functional.gelu(self.first(x)))


def test_registered_operator_traces_as_one_node(oracle):
    """The multiplication is the operator nmspmm::sparse_linear: torch.compile(fullgraph=True)
    and torch.export of a model that holds two such layers trace without a graph break, the
    exported graph holds the operator twice, and the compiled model's output equals the eager one
    bit for bit and the fp64 layers with the checker-pruned weights within the bound."""
    op = importlib.import_module("nm-spmm_amd.torch_op")
    g = torch.Generator(device="cuda").manual_seed(11)
    w1 = torch.randn((512, 256), generator=g, dtype=torch.float32, device="cuda") * 0.05
    w2 = torch.randn((128, 512), generator=g, dtype=torch.float32, device="cuda") * 0.05
    b1 = torch.randn((512,), generator=g, dtype=torch.float32, device="cuda")
    model = TwoLayers(op.NMSparseLinear(w1, 2, 4, b1), op.NMSparseLinear(w2, 1, 8))
    x = torch.randn((3, 40, 256), generator=g, dtype=torch.float32, device="cuda")
    eager = model(x)
    compiled = torch.compile(model, fullgraph=True, backend="aot_eager")
    got = compiled(x)
    assert got.shape == (3, 40, 128) and torch.equal(got, eager)
    got16 = compiled(x[:, :16])               # another row count: decode-sized (48 rows)
    assert torch.equal(got16, model(x[:, :16]))
    exported = torch.export.export(model, (x,))
    targets = [str(n.target) for n in exported.graph.nodes if n.op == "call_function"]
    assert sum("nmspmm.sparse_linear" in t for t in targets) == 2
    assert torch.equal(exported.module()(x), eager)

    def pruned(w, n, m):
        BT, DT = oracle.compress(w.t().contiguous().cpu().numpy(), n, m)
        K, N, W = w.shape[1], w.shape[0], BT.shape[0]
        dense = np.zeros((K, N), np.float64)
        rows = (np.arange(W) // n * m)[:, None] + DT
        dense[np.repeat(rows, 32, axis=1), np.broadcast_to(np.arange(N), (W, N))] = BT
        return torch.from_numpy(dense).cuda()

    h = torch.nn.functional.gelu(x.double().reshape(-1, 256) @ pruned(w1, 2, 4) + b1.double())
    want = h @ pruned(w2, 1, 8)
    assert scaled_max_error(got.reshape(-1, 128).cpu().numpy(), want.cpu().numpy()) <= REL_TOL


def test_operator_passes_torchs_own_registration_checks():
    op = importlib.import_module("nm-spmm_amd.torch_op")
    g = torch.Generator(device="cuda").manual_seed(3)
    layer = op.NMSparseLinear(torch.randn((128, 256), generator=g, dtype=torch.float32, device="cuda"), 2, 8)
    x = torch.randn((5, 256), generator=g, dtype=torch.float32, device="cuda")
    args = (x, layer.values, layer.indices, layer.column_info, layer.row_index, None, layer.window, layer.kept, layer.Ns, 0)
    torch.library.opcheck(torch.ops.nmspmm.sparse_linear.default, args,
                          test_utils=("test_schema", "test_faketensor"))
