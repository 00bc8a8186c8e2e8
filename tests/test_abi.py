"""The C-ABI library loads and exports every symbol include/dapple_stage.h declares (no compute)."""
import os
import re

from dapple_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dapple_stage.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(ds_[a-z0-9_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert declared, "no declarations parsed"
    for name in declared:
        assert hasattr(lib, name), name
    # and the ctypes table covers exactly the header
    assert declared == set(_lib.PROTOTYPES), declared ^ set(_lib.PROTOTYPES)


def test_build_target_and_argument_errors_without_a_gpu():
    lib = _lib.load()
    assert lib.ds_build_target() == b"gfx950"
    # argument validation happens before any HIP call
    assert lib.ds_grad_accumulate(None, None, 16, 0, None) == -1
    assert b"null" in lib.ds_last_error()
    assert lib.ds_gemm(None, None) == -1
    d = _lib.GemmDesc()
    d.dtype, d.m, d.n, d.k = 1, 8, 8, 7
    d.a = d.b = d.c = 256
    d.lda = d.ldb = d.ldc = 8
    assert lib.ds_gemm(d, None) == -1 and b"multiple of 8" in lib.ds_last_error()
