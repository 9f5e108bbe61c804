"""Runs the C++ conformance caller (tests/cpp/conformance.cpp), which uses the
drop-in ccglib headers with native HIP handles the way the reference's HIP API
tests and example do. The binary is built by tests/cpp/Makefile."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "conformance")


@pytest.mark.gpu
def test_cpp_conformance():
    if not os.path.exists(BINARY):
        subprocess.check_call(["make", "-C", os.path.join(HERE, "cpp")])
    r = subprocess.run([BINARY], capture_output=True, text=True, timeout=300)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout


def test_headers_declare_the_reference_api():
    # the class and method names a ccglib user compiles against
    inc = os.path.join(os.path.dirname(HERE), "include", "ccglib")
    text = {n: open(os.path.join(inc, n)).read() for n in
            ["gemm/mma.h", "transpose/transpose.h", "packing/packing.h", "pipeline/pipeline.h",
             "common/types.h"]}
    assert "namespace ccglib::mma" in text["gemm/mma.h"] and "class GEMM" in text["gemm/mma.h"]
    assert "static dim3 GetDimensions(Precision precision, Variant variant = Variant::opt)" in text["gemm/mma.h"]
    assert "void Run(hipDeviceptr_t d_a, hipDeviceptr_t d_b, hipDeviceptr_t d_c)" in text["gemm/mma.h"]
    assert "class Transpose" in text["transpose/transpose.h"]
    assert "class Packing" in text["packing/packing.h"]
    assert "class Pipeline" in text["pipeline/pipeline.h"]
    for token in ["int1 = 0", "float32 = 6", "complex_interleaved = 1", "backward = 1",
                  "col_major = 1", "opt = 1"]:
        assert token in text["common/types.h"]
