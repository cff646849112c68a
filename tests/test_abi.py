"""The C-ABI library loads and exports every symbol include/ffk.h declares
(no compute calls: runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "ffk.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ffk_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(ffk):
    names = _declared_symbols()
    assert len(names) > 30
    handle = ctypes.CDLL(ffk.LIB_PATH)
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, missing


def test_python_signature_table_matches_header(ffk):
    assert sorted(ffk.SIGNATURES) == _declared_symbols()


def test_argument_checks_do_not_need_a_device(ffk):
    lib = ffk.lib()
    # preconditions are checked before any HIP call is made
    assert lib.ffk_linear_forward(None, ffk.FLOAT, 7, None, None, None, None, 1, 1, 1) == 1
    assert b"Unhandled activation" in lib.ffk_last_error()
    assert lib.ffk_dropout_forward(None, ffk.FLOAT, None, None, 10, 1.5, 0, 0) == 1
    assert lib.ffk_embedding_forward(None, ffk.INT32, ffk.FLOAT, ffk.FLOAT, None, None, None,
                                     ffk.AGGR_NONE, 4, 2, 8, 10) == 1
    assert lib.ffk_element_unary_forward(None, ffk.FLOAT, 9999, 0.0, 1, 1, 4) == 3
    assert lib.ffk_gemm(None, ffk.DOUBLE, 0, 0, 4, 4, 4, 1, 1, 1, 0) == 3
