import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle.nm_oracle import Oracle, Reference  # noqa: E402  (the checker; tests may use it)

nmspmm = importlib.import_module("nm-spmm_amd")
datagen = importlib.import_module("nm-spmm_amd.datagen")

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")

# The tests load what is built; only when nothing is do they build it (hipcc cross-compiles without
# a GPU).  The package itself never builds or falls back: it raises when the library is missing.
if not os.path.exists(nmspmm.LIB_PATH):
    import subprocess
    subprocess.run(["make", "-C", os.path.join(ROOT, "nm-spmm_amd", "csrc"), "-j8"], check=True)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    if not Reference.available():
        pytest.skip("oracle/_ref/libnmref.so not built (reference tree absent at build time)")
    return Reference()


# (n, m) of a pattern as generated -> (window, kept) the kernels run it at, and how many
# transIndex doublings take it there (reference launchers: src/kernel_64x128_8x8.cu:264-289,584-602).
def kernel_geometry(n, m):
    table = {(1, 1): (32, 32), (1, 2): (32, 16), (3, 8): (32, 12), (1, 4): (64, 16), (1, 8): (64, 8)}
    from math import gcd
    g = gcd(n, m)
    window, kept = table[(n // g, m // g)]
    times = 0
    mm = m
    while mm < window:
        mm *= 2
        times += 1
    assert mm == window, "pattern window larger than the kernel window"
    return window, kept, times


def widen(oracle, DT, W, Q, n, m, times):
    """Apply the oracle's transIndex `times` times to a copy of DT."""
    DT = DT.copy()
    for _ in range(times):
        n, m = oracle.trans_index(DT.reshape(-1), W, Q, n, m)
    return DT, n, m


def preprocess_with_oracle(oracle, data, Ns):
    """Widen + preprocess on the CPU checker: returns (window, kept, D_blocked, cinfo or None)."""
    window, kept, times = kernel_geometry(data["n"], data["m"])
    DT, n, m = widen(oracle, data["DT"], data["W"], data["Q"], data["n"], data["m"], times)
    assert (m, n) == (window, kept)
    flat = DT.reshape(-1).copy()
    if window == 64:
        cinfo = oracle.preprocess_high(window, kept, flat, data["W"], data["Q"], Ns, data["vec_len"])
        return window, kept, flat, cinfo
    oracle.preprocess_low(flat, data["W"], data["Q"], Ns, data["vec_len"])
    return window, kept, flat, None


def scaled_max_error(got, want):
    """max |got - want| / max(|want|, rms(want)): the relative error of the north-star bound,
    made well-conditioned for signed data whose exact result may be arbitrarily close to 0."""
    want = want.astype(np.float64)
    got = got.astype(np.float64)
    rms = np.sqrt(np.mean(want * want))
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), rms)))


REL_TOL = 1e-4  # north-star bound for C (fp32, reordered accumulation)
