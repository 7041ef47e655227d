"""Runs the C++ drop-in driver (tests/cxx/test_nmspmm_dropin, built by __graft_entry__.build()):
a program written against include/NM-SpMM.h exactly as a caller of the reference would write it —
host-pointer preprocessing in place, the eight launchers by name, default stream — checked inside
the program against the CPU checker."""
import os
import subprocess

import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu
BIN = os.path.join(ROOT, "tests", "cxx", "test_nmspmm_dropin")


@pytest.mark.parametrize("args", [
    ["256", "256", "256", "32", "0.5"],
    ["256", "384", "512", "32", "0.625", "2"],
    ["192", "256", "256", "32", "0.0"],
    ["256", "256", "512", "32", "0.75"],
    ["128", "256", "512", "32", "0.875", "4"],
    ["16", "256", "512", "32", "0.875"],
    ["16", "256", "512", "32", "0.75", "4"],           # decode-sized rows, split call: adds to C
    ["512", "512", "1024", "32", "0.5", "4", "2", "3"],  # the reference driver's nine-argument form
], ids=" ".join)
def test_reference_style_driver(args):
    assert os.path.exists(BIN), "build the driver first: make -C tests/cxx"
    out = subprocess.run([BIN] + args, capture_output=True, text=True, timeout=120)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "The result is right!" in out.stdout and "wrong" not in out.stdout
    assert out.stdout.count("The result is right!") >= 3  # small, medium, large (+ huge when 128 | N)


def test_wrong_family_prints_not_support_like_the_reference():
    """0.75 through a low-sparsity launcher: the reference prints 'Not support!' and launches
    nothing (src/kernel_64x128_8x8.cu:264-265); so does the drop-in.  Exercised through ctypes on
    the mangled C++ symbol with NULL operands, which the error path never dereferences."""
    import ctypes
    lib = ctypes.CDLL(os.path.join(ROOT, "nm-spmm_amd", "libnmspmm.so"))
    fn = getattr(lib, "_Z33nmGEMM_huge_matrices_low_sparsityPfS_PiS_iiiifi")
    fn.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.c_float, ctypes.c_int]
    fn.restype = None
    fn(None, None, None, None, 128, 128, 128, 32, 0.75, 1)  # prints to stdout, must not crash
