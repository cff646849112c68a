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


def test_gemm_kernel_name_needs_no_device(ffk):
    """The dispatch answers which kernel a shape runs on without launching anything."""
    big = ffk.gemm_kernel_name(ffk.BF16, False, True, 4096, 4096, 1024, has_bias=True)
    assert big.startswith("gemm_bf16_pipe_kernel<256,256,") and big.endswith("false,true,0,false>")
    assert ffk.gemm_kernel_name(ffk.BF16, True, False, 1024, 1024, 4096).startswith("gemm_bf16_pipe_kernel<128,128,")
    assert ffk.gemm_kernel_name(ffk.FLOAT, False, True, 32, 128, 64, has_bias=True).startswith("gemm_f32_kernel")
    assert ffk.gemm_kernel_name(ffk.BF16, False, False, 51, 131, 251) == "gemm_bf16_plain_kernel"
    # an activation changes the instance, and the answer follows the option that forces a tile
    relu = ffk.gemm_kernel_name(ffk.BF16, False, True, 4096, 4096, 1024, True, ffk.ACT_RELU)
    assert relu != big
    ffk.set_option(ffk.OPTION_GEMM_VARIANT, 128)
    try:
        assert ffk.gemm_kernel_name(ffk.BF16, False, True, 4096, 4096, 1024, True).startswith("gemm_bf16_pipe_kernel<128,128,")
    finally:
        ffk.set_option(ffk.OPTION_GEMM_VARIANT, 0)
