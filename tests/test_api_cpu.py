"""CPU-side checks of the boundary: the shared library loads, exports every symbol
the header declares, and rejects bad requests with the reference's messages before
touching a device."""
import os
import re

import pytest

import ccglib_amd as cc
from ccglib_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
VT = cc.ValueType


def header_functions():
    text = open(os.path.join(ROOT, "include", "ccglib_amd.h")).read()
    return sorted(set(re.findall(r"\b(ccglib_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _capi.load()
    names = header_functions()
    assert len(names) >= 18
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_capi.SIGNATURES) == names


def test_version_and_dimensions():
    assert "gfx950" in cc.version()
    assert cc.GEMM.GetDimensions(VT.float16) == (128, 128, 32)
    assert cc.GEMM.GetDimensions(cc.Precision(VT.bfloat16, VT.bfloat16)) == (128, 128, 32)
    assert cc.GEMM.GetDimensions(VT.float8e4m3) == (128, 128, 64)
    assert cc.GEMM.GetDimensions(VT.float8e5m2, cc.Variant.basic) == (128, 128, 64)
    assert cc.GEMM.GetDimensions(cc.Precision(VT.int1, VT.int32)) == (128, 128, 512)
    with pytest.raises(RuntimeError, match="No kernel parameters available"):
        cc.GEMM.GetDimensions(cc.Precision(VT.int32, VT.int32))


def test_ceildiv():
    assert cc.ceildiv(10, 5) == 2 and cc.ceildiv(16, 5) == 4      # test/helper.cpp:7-9


def test_basic_variant_rejects_interleaved_output():
    with pytest.raises(RuntimeError, match="complex-interleaved output is not supported in basic variant"):
        cc.GEMM(16, 16, 16, 256, 0, 0, VT.float16, cc.Variant.basic,
                cc.ComplexAxisLocation.complex_interleaved)


@pytest.mark.parametrize("prec", [VT.float16, cc.Precision(VT.int1, VT.int32)])
def test_unsupported_matrix_layout(prec):
    # test/gemm/mma.cpp:598-643: A col-major (with B col-major) must fail with the
    # compile-error token in the message
    with pytest.raises(RuntimeError, match="HIPRTC_ERROR_COMPILATION"):
        cc.GEMM(16, 16, 16, 256, 0, 0, prec, cc.Variant.basic, cc.ComplexAxisLocation.complex_planar,
                cc.MemOrder.row_major, cc.MemOrder.col_major, cc.MemOrder.col_major)
    with pytest.raises(RuntimeError, match="HIPRTC_ERROR_COMPILATION"):
        cc.GEMM(16, 16, 16, 256, 0, 0, prec, cc.Variant.basic, cc.ComplexAxisLocation.complex_planar,
                cc.MemOrder.row_major, cc.MemOrder.row_major, cc.MemOrder.row_major)


def test_unpacking_rejects_interleaved():
    with pytest.raises(RuntimeError, match="complex-interleaved input is not supported in unpacking kernel"):
        cc.Packing(2048, cc.Direction.backward, 0, 0, cc.ComplexAxisLocation.complex_interleaved)


def test_transpose_argument_checks():
    with pytest.raises(RuntimeError, match="NBIT_IN must be 1, 8, 16, 32"):
        cc.Transpose(1, 16, 16, 16, 16, 4, 0, 0)
    with pytest.raises(RuntimeError, match="multiples of 32"):
        cc.Transpose(1, 16, 48, 16, 16, 1, 0, 0)


def test_unsupported_type_pair():
    with pytest.raises(RuntimeError, match="No kernel parameters available"):
        cc.GEMM(1, 16, 16, 16, 0, 0, cc.Precision(VT.float16, VT.bfloat16))


def test_null_handles_are_errors_not_crashes():
    lib = _capi.load()
    assert lib.ccglib_gemm_run(None, None, None, None) != 0
    assert b"null" in lib.ccglib_last_error()
    assert lib.ccglib_transpose_run(None, None, None) != 0
    assert lib.ccglib_transpose_run_pair(None, None, None, None, None, None) != 0
    assert b"null" in lib.ccglib_last_error()
    assert lib.ccglib_packing_run(None, None, None) != 0
    assert lib.ccglib_pipeline_run(None, None, None, None) != 0
    assert lib.ccglib_gemm_destroy(None) == 0
