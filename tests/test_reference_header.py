"""ccglib::reference::GEMM of the drop-in headers (include/ccglib/gemm/reference.h),
run on the CPU through tests/cpp/libreference_shim.so: the reference's known-answer
tests (test/gemm/reference.cpp:27-45, :73-80, :98-109, :121-133) and bit-for-bit
agreement with the oracle on random inputs of every type pair. No GPU needed."""
import ctypes
import json
import os
import subprocess

import numpy as np
import pytest

import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))


# the second build allows fused multiply-add wherever the compiler likes (-mfma
# -ffp-contract=fast): the header has to keep its float loop free of it by itself
@pytest.fixture(scope="module", params=["libreference_shim.so", "libreference_shim_fma.so"])
def shim(request):
    path = os.path.join(HERE, "cpp", request.param)
    subprocess.check_call(["make", "-C", os.path.join(HERE, "cpp"), request.param],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    lib = ctypes.CDLL(path)
    vp, sz, f = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float
    lib.reference_gemm.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, sz, sz, sz, ctypes.c_int,
                                   f, f, f, f]
    lib.reference_gemm.restype = ctypes.c_int
    return lib


def run(lib, a, b, M, N, K, tin, tout, order, alpha=1 + 0j, beta=0j, c_in=None):
    c = np.zeros(2 * M * N, dtype=orc._STORAGE[tout]) if c_in is None else c_in.copy()
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    rc = lib.reference_gemm(tin, tout, a.ctypes.data, b.ctypes.data, c.ctypes.data, M, N, K, order,
                            alpha.real, alpha.imag, beta.real, beta.imag)
    assert rc == 0
    return c


def enc(vals, vtype):
    v = np.asarray(vals, dtype=np.float32)
    if vtype == orc.FLOAT16:
        return v.astype(np.float16).view(np.uint16)
    if vtype == orc.BFLOAT16:
        return (v.view(np.uint32) >> 16).astype(np.uint16)
    return v


@pytest.mark.parametrize("vtype", [orc.FLOAT16, orc.BFLOAT16, orc.FLOAT32])
def test_kat_float(shim, vtype):
    k = KATS["float"]
    a, b = enc(k["a"], vtype), enc(k["b"], vtype)
    assert run(shim, a, b, k["M"], k["N"], k["K"], vtype, orc.FLOAT32, orc.ROW_MAJOR).tolist() == k["c_row_major"]
    assert run(shim, a, b, k["M"], k["N"], k["K"], vtype, orc.FLOAT32, orc.COL_MAJOR).tolist() == k["c_col_major"]


def test_kat_int1(shim):
    k = KATS["int1"]
    a, b = np.array(k["a"], dtype=np.uint32), np.array(k["b"], dtype=np.uint32)
    assert run(shim, a, b, k["M"], k["N"], k["K"], orc.INT1, orc.INT32, orc.ROW_MAJOR).tolist() == k["c_row_major"]
    assert run(shim, a, b, k["M"], k["N"], k["K"], orc.INT1, orc.INT32, orc.COL_MAJOR).tolist() == k["c_col_major"]


def test_kat_alpha_beta_fp16(shim):
    k = KATS["alpha_beta_float16"]
    c = run(shim, enc(k["a"], orc.FLOAT16), enc(k["b"], orc.FLOAT16), k["M"], k["N"], k["K"],
            orc.FLOAT16, orc.FLOAT32, orc.ROW_MAJOR, complex(*k["alpha"]), complex(*k["beta"]),
            np.array(k["c_in"], dtype=np.float32))
    assert c.tolist() == k["c_row_major"]


PAIRS = [(orc.FLOAT8E4M3, orc.FLOAT32), (orc.FLOAT8E5M2, orc.FLOAT32), (orc.FLOAT16, orc.FLOAT16),
         (orc.FLOAT16, orc.FLOAT32), (orc.FLOAT32, orc.FLOAT16), (orc.BFLOAT16, orc.BFLOAT16),
         (orc.BFLOAT16, orc.FLOAT32), (orc.FLOAT32, orc.BFLOAT16), (orc.FLOAT32, orc.FLOAT32)]


def random_operand(rng, n, vtype):
    if vtype in (orc.FLOAT8E4M3, orc.FLOAT8E5M2):
        # finite encodings only
        v = rng.integers(0, 0x78 if vtype == orc.FLOAT8E4M3 else 0x7C, n, dtype=np.uint8)
        return v | (rng.integers(0, 2, n, dtype=np.uint8) << 7)
    return enc(rng.uniform(-2, 2, n), vtype)


@pytest.mark.parametrize("tin,tout", PAIRS)
@pytest.mark.parametrize("order", [orc.ROW_MAJOR, orc.COL_MAJOR])
def test_matches_oracle_bit_for_bit(shim, tin, tout, order):
    rng = np.random.default_rng(tin * 16 + tout)
    M, N, K = 13, 9, 37
    a, b = random_operand(rng, 2 * M * K, tin), random_operand(rng, 2 * N * K, tin)
    c_in = random_operand(rng, 2 * M * N, tout)
    for alpha, beta in ((1 + 0j, 0j), (1.5 - 0.5j, 0j), (0.75 + 2j, -0.5 + 0.25j)):
        want = orc.gemm(a, b, M, N, K, tin, tout, order, alpha, beta, c_in if beta != 0 else None)
        got = run(shim, a, b, M, N, K, tin, tout, order, alpha, beta, c_in)
        assert np.array_equal(got.view(np.uint8), want.reshape(-1).view(np.uint8))


@pytest.mark.parametrize("K", [32, 100, 257])
@pytest.mark.parametrize("order", [orc.ROW_MAJOR, orc.COL_MAJOR])
def test_bits_match_oracle(shim, K, order):
    rng = np.random.default_rng(K)
    M, N, words = 7, 11, (K + 31) // 32
    a = rng.integers(0, 2**32, 2 * M * words, dtype=np.uint32)
    b = rng.integers(0, 2**32, 2 * N * words, dtype=np.uint32)
    c_in = rng.integers(-1000, 1000, 2 * M * N).astype(np.int32)
    for alpha, beta in ((1 + 0j, 0j), (2 - 3j, 1 + 2j), (1.9 + 0j, 0.9j)):
        want = orc.gemm(a, b, M, N, K, orc.INT1, orc.INT32, order, alpha, beta, c_in)
        got = run(shim, a, b, M, N, K, orc.INT1, orc.INT32, order, alpha, beta, c_in)
        assert np.array_equal(got, want.reshape(-1))
