"""GPU parity of the tile kernel on seeded random LARGE shapes, where the CPU checker would need
minutes: operands are drawn on the GPU, the reference is the dense product with the decompressed
operand in fp64 (torch on the GPU - an independent formulation, not the checker's loop nest).  The
shapes cross every launch plan: fewer tiles than the GPU holds, several rounds, ragged last rounds
(leftover tiles in a launch of their own, whole or in pieces), ragged row counts, reduction splits,
both storage orders of A, all three widths of the column blocks.  Same tolerance as everywhere (1e-4, scaled max error)."""
import os
import random

import pytest

from conftest import REL_TOL, nmspmm

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

# NMSPMM_TEST_SEED=<n> draws another set of problems (the default set is the one every run checks)
SEED = int(os.environ.get("NMSPMM_TEST_SEED", "0")) * 100000
GEOMETRY = {(2, 4): (32, 16), (3, 8): (32, 12), (2, 8): (64, 16), (1, 8): (64, 8)}


def draw_case(rng):
    n, m = rng.choice(list(GEOMETRY))
    M = rng.choice([rng.randint(129, 700), 4 * rng.randint(150, 1500), 256 * rng.randint(2, 24)])
    N = 128 * rng.randint(4, 96)
    K = 64 * rng.randint(2, 40)
    while M * N * K > 3.5e10:  # keeps the fp64 reference to a fraction of a second
        N = 128 * max(4, N // 256)
    split_k = min(rng.choice([1, 1, 1, 2, 3, 4]), K // 64)
    return M, N, K, n, m, split_k, rng.random() < 0.3, rng.choice([128, 128, 64, 32])


def draw_few_tiles_case(rng):
    """At most 256 tiles of 128 or 256 rows and a long reduction: the launches with waves along K in
    their four forms (64 or 128 rows, four or eight waves), whole tiles on two sets of waves."""
    n, m = rng.choice(list(GEOMETRY))
    N = 128 * rng.choice([8, 16, 16, 24, 32, 32, 40, 64])
    M = rng.randint(129, (128 if rng.random() < 0.6 else 256) * (256 // (N // 128)))
    K = 64 * rng.randint(32, 130)
    while M * N * K > 3.5e10:
        K -= 64 * 8
    return M, N, K, n, m, 1, rng.random() < 0.2, rng.choice([128, 128, 64, 32])


CASES = [draw_case(random.Random(SEED + 9000 + i)) for i in range(60)] + \
        [draw_few_tiles_case(random.Random(SEED + 9500 + i)) for i in range(40)]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "M%d-N%d-K%d-%dof%d-s%d-%s-Ns%d" % (c[:6] + ("rm" if c[6] else "cm", c[7])))
def test_random_large_shape(case):
    M, N, K, n, m, split_k, row_major, Ns = case
    window, kept = GEOMETRY[(n, m)]
    g = torch.Generator(device="cuda").manual_seed(M * 7 + N + K)
    W, Q = K // m * n, N // 32
    BT = torch.randn((W, N), generator=g, dtype=torch.float32, device="cuda") * 0.05
    pick = torch.rand((K // m, Q, m), generator=g, device="cuda").argsort(dim=2)[:, :, :n].sort(dim=2).values
    DT = pick.permute(0, 2, 1).reshape(W, Q).to(torch.int32).contiguous()          # [W][Q], window-local rows
    X = torch.randn((M, K), generator=g, dtype=torch.float32, device="cuda")       # row-major activations
    # reference: scatter the kept values back to K x N and multiply in fp64
    rows = (torch.arange(W, device="cuda") // n * m)[:, None] + DT.long()
    dense = torch.zeros((K, N), dtype=torch.float64, device="cuda")
    dense[rows.repeat_interleave(32, dim=1), torch.arange(N, device="cuda")[None, :].expand(W, -1)] = BT.double()
    want = X.double() @ dense
    del dense
    # the library's own preprocessing of the pattern as generated
    D = torch.empty_like(DT)
    cinfo = None
    if window == 64:
        cinfo = torch.empty(nmspmm.column_info_ints(W, kept, window, N, Ns), dtype=torch.int32, device="cuda")
    assert nmspmm.preprocess_device(DT, n, m, W, Q, N, Ns, D, cinfo) == (window, kept)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    if row_major:
        ws = torch.empty(nmspmm.workspace_bytes_rowmajor(M, N, K, split_k) // 4, dtype=torch.float32, device="cuda")
        nmspmm.spmm_rowmajor(X, BT, D, cinfo, C, M, N, K, W, window, kept, ws, 32, Ns, split_k)
    else:
        A = X.t().contiguous()                                                      # K x M: column-major M x K
        ws = torch.empty(max(nmspmm.workspace_bytes(M, N, split_k) // 4, 4), dtype=torch.float32, device="cuda")
        nmspmm.spmm(A, BT, D, cinfo, C, M, N, K, W, window, kept, 32, Ns, split_k, ws if split_k > 1 else None)
    torch.cuda.synchronize()
    assert nmspmm.last_kernel() == "mfma"
    assert torch.isfinite(C).all().item()
    rms = want.pow(2).mean().sqrt()
    err = ((C.double() - want).abs() / want.abs().clamp_min(rms)).max().item()
    assert err <= REL_TOL, err
