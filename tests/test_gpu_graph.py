"""The multiplication entry points launch kernels and nothing else (no allocation, no memset, no
synchronisation), so a caller can capture them into a HIP graph - the way a serving loop removes
the per-launch cost of decode-sized calls.  Each replay is checked against an eager call on the
same inputs, with eager work and synchronisation between the replays."""
import numpy as np
import pytest

from conftest import datagen, nmspmm, preprocess_with_oracle

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("M,n,m,split_k,row_major", [(8, 1, 8, 1, False), (4, 2, 8, 1, True), (64, 2, 4, 1, True),
                                                     (256, 2, 4, 1, False), (256, 2, 8, 2, False), (192, 1, 8, 3, True)])
def test_graph_replays_equal_eager_calls(oracle, M, n, m, split_k, row_major):
    N, K = 512, 1024
    d = datagen.init_data(M, N, K, n, m, seed=M + split_k, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    W = d["W"]
    A = dev(d["A_km"].T) if row_major else dev(d["A_km"])
    B, Dd = dev(d["BT"]), dev(D)
    dc = None if cinfo is None else dev(cinfo)
    need = (nmspmm.workspace_bytes_rowmajor(M, N, K, split_k) if row_major else nmspmm.workspace_bytes(M, N, split_k)) // 4
    ws_g = torch.empty(max(need, 4), dtype=torch.float32, device="cuda")
    ws_e = torch.empty_like(ws_g)
    C_g = torch.empty((M, N), dtype=torch.float32, device="cuda")
    C_e = torch.empty_like(C_g)

    def call(C, ws):
        if row_major:
            nmspmm.spmm_rowmajor(A, B, Dd, dc, C, M, N, K, W, window, kept, ws, 32, 128, split_k)
        else:
            nmspmm.spmm(A, B, Dd, dc, C, M, N, K, W, window, kept, 32, 128, split_k, ws if split_k > 1 else None)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(C_g, ws_g)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(C_g, ws_g)
    for rep in range(4):
        A.mul_(1.25)                      # eager work between the replays; the graph reads A in place
        C_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        call(C_e, ws_e)
        torch.cuda.synchronize()
        assert torch.isfinite(C_g).all().item()
        assert torch.equal(C_g, C_e), "replay %d" % rep


def test_graph_replays_of_a_call_that_hands_its_last_rows_over(oracle):
    """136 rows on 4096 columns: the tile kernel computes 128 rows and the kernel on the reference
    layout the other eight, two launches that a graph holds like any other."""
    M, N, K, n, m = 136, 4096, 2048, 2, 4
    d = datagen.init_data(M, N, K, n, m, seed=M, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    W = d["W"]
    assert nmspmm.rows_apart(M, N, W, kept) == 8
    A, B, Dd = dev(d["A_km"]), dev(d["BT"]), dev(D)
    C_g = torch.empty((M, N), dtype=torch.float32, device="cuda")
    C_e = torch.empty_like(C_g)

    def call(C):
        nmspmm.spmm(A, B, Dd, None, C, M, N, K, W, window, kept, 32, 128, 1, None)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(C_g)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(C_g)
    for rep in range(3):
        A.mul_(1.25)
        C_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        call(C_e)
        torch.cuda.synchronize()
        assert torch.isfinite(C_g).all().item()
        assert torch.equal(C_g, C_e), "replay %d" % rep



@pytest.mark.parametrize("M", [1, 16, 32])
def test_graph_replays_of_cut_decode_reductions(oracle, M):
    """NMSPMM_DECODE_SPLIT inside a graph: the captured launch carries one epoch for its arrival
    words, and every replay presents it again, interleaved with eager launches that carry newer
    ones.  The words are zero between launches, so each replay finds what the first run found: C
    is written by the slice that arrives last, every time, identical to the eager call."""
    N, K, n, m = 4096, 11008, 2, 8
    d = datagen.init_data(M, N, K, n, m, seed=M + 3, dist="normal", b_scale=0.02)
    window, kept, D, cinfo = preprocess_with_oracle(oracle, d, 128)
    W = d["W"]
    A, B, Dd, dc = dev(d["A_km"]), dev(d["BT"]), dev(D), dev(cinfo)
    R = torch.empty(nmspmm.row_index_ints(W, N), dtype=torch.int32, device="cuda")
    nmspmm.row_index_device(Dd, dc, W, N, window, kept, 128, R)
    C_g = torch.empty((M, N), dtype=torch.float32, device="cuda")
    C_e = torch.empty_like(C_g)
    C_plain = torch.empty_like(C_g)

    def call(C, flags=nmspmm.DECODE_SPLIT):
        nmspmm.spmm_ex(A, B, Dd, dc, C, M, N, K, W, window, kept, 32, 128, 1, None, flags, R)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(C_g)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(C_g)
        call(C_g)   # twice in one graph: two epochs held by the same graph
    for rep in range(5):
        A.mul_(1.25)
        C_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        call(C_e)
        call(C_plain, 0)
        torch.cuda.synchronize()
        assert nmspmm.last_kernel() == "decode"
        assert torch.isfinite(C_g).all().item(), "replay %d left rows of C unwritten" % rep
        assert torch.equal(C_g, C_e), "replay %d" % rep
        scale = float(C_plain.abs().max())
        assert float((C_g - C_plain).abs().max()) <= 1e-4 * scale
