"""CPU oracle for the complex-GEMM hot path: TEST INFRASTRUCTURE ONLY.

numpy front end of ``ccglib_oracle.c`` (see that file's header for what each
function restates and what pins it). Only tests, the smoke check and the
benchmark's CPU-baseline leg may import this package; the shipped library never
does.

Arrays are passed as raw bit patterns: fp16 / bf16 as ``uint16``, fp8 as
``uint8``, packed 1-bit samples as ``uint32``; float32 / int32 as themselves.
"""
import ctypes
import os
import subprocess

import numpy as np

# Enum values of the reference API (include/ccglib/common/value_type.h:14-22).
INT1, INT32, BFLOAT16, FLOAT8E4M3, FLOAT8E5M2, FLOAT16, FLOAT32 = range(7)
ROW_MAJOR, COL_MAJOR = 0, 1          # include/ccglib/gemm/mem_order.h:6
PLANAR, INTERLEAVED = 0, 1           # include/ccglib/common/complex_order.h:12

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libccglib_oracle.so")

_STORAGE = {
    FLOAT16: np.uint16, BFLOAT16: np.uint16, FLOAT8E4M3: np.uint8,
    FLOAT8E5M2: np.uint8, FLOAT32: np.float32, INT32: np.int32, INT1: np.uint32,
}


def build(force=False):
    """Compile the C oracle with the Makefile beside it."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"])
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, vp, f, i = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
        L.oracle_gemm_float.argtypes = [vp, vp, vp, sz, sz, sz, i, i, i, f, f, f, f]
        L.oracle_gemm_float.restype = None
        L.oracle_gemm_float64.argtypes = [vp, vp, vp, sz, sz, sz, i, i]
        L.oracle_gemm_float64.restype = None
        L.oracle_gemm_int1.argtypes = [vp, vp, vp, sz, sz, sz, i, f, f, f, f]
        L.oracle_gemm_int1.restype = None
        L.oracle_transpose.argtypes = [vp, vp, sz, sz, sz, sz, sz, sz, i]
        L.oracle_transpose.restype = None
        L.oracle_pack_bits.argtypes = [vp, vp, sz, i]
        L.oracle_pack_bits.restype = None
        L.oracle_unpack_bits.argtypes = [vp, vp, sz]
        L.oracle_unpack_bits.restype = None
        L.oracle_ceildiv.argtypes = [sz, sz]
        L.oracle_ceildiv.restype = sz
        L.oracle_reference_fixture.argtypes = [vp, vp, sz, ctypes.POINTER(ctypes.c_uint)]
        L.oracle_reference_fixture.restype = None
        for name, arg, res in [
            ("oracle_half_to_float", ctypes.c_uint16, f),
            ("oracle_bf16_to_float", ctypes.c_uint16, f),
            ("oracle_e4m3_to_float", ctypes.c_uint8, f),
            ("oracle_e5m2_to_float", ctypes.c_uint8, f),
            ("oracle_float_to_half", f, ctypes.c_uint16),
            ("oracle_float_to_bf16", f, ctypes.c_uint16),
        ]:
            getattr(L, name).argtypes = [arg]
            getattr(L, name).restype = res
        L.oracle_max_threads.restype = i
        L.oracle_set_threads.argtypes = [i]
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _check(a, dtype, size, name):
    if a.dtype != dtype or a.size != size or not a.flags["C_CONTIGUOUS"]:
        raise ValueError(f"{name}: need contiguous {np.dtype(dtype)} array of "
                         f"{size} elements, got {a.dtype} x {a.size}")


def ceildiv(a, b):
    return lib().oracle_ceildiv(a, b)


def max_threads():
    return lib().oracle_max_threads()


def set_threads(n):
    lib().oracle_set_threads(n)


def reference_fixture(n_a, n_b, words=False):
    """The inputs of the reference's GEMM tests (test/gemm/mma.cpp:144-217): n_a values
    for A, then n_b for B, from one libc rand_r sequence that starts at seed 0:
    rand_r / RAND_MAX as float32 in [0, 1], or (words=True, 1-bit input) the raw 31-bit
    values as packed words. Returns (a, b)."""
    seed = ctypes.c_uint(0)
    out = []
    for n in (n_a, n_b):
        x = np.empty(n, dtype=np.uint32 if words else np.float32)
        lib().oracle_reference_fixture(None if words else _ptr(x), _ptr(x) if words else None, n,
                                       ctypes.byref(seed))
        out.append(x)
    return out


def gemm(a, b, M, N, K, type_in, type_out=FLOAT32, c_order=ROW_MAJOR,
         alpha=1 + 0j, beta=0j, c_in=None, batch=None):
    """Batched complex GEMM C = alpha A B^T + beta C_in with the reference's CPU
    semantics; the batch loop is the caller's loop in the reference
    (test/gemm/verify.h:54-60) and lives here.

    a: [B][2][M][K'] b: [B][2][N][K'] (K' = K, or ceil(K/32) words for 1-bit).
    Returns c [B][2][M][N] (row major) or [B][2][N][M] (column major) in the
    storage type of ``type_out``. ``batch`` is only needed where the operands are
    empty (K = 0) and B cannot be read from their size.
    """
    alpha, beta = complex(alpha), complex(beta)
    kk = (K + 31) // 32 if type_in == INT1 else K
    B = batch if batch is not None else a.size // (2 * M * kk)
    _check(a, _STORAGE[type_in], B * 2 * M * kk, "a")
    _check(b, _STORAGE[type_in], B * 2 * N * kk, "b")
    out_dt = _STORAGE[type_out]
    shape = (B, 2, M, N) if c_order == ROW_MAJOR else (B, 2, N, M)
    if c_in is None:
        if beta != 0:
            raise ValueError("c_in must be given when beta != 0")
        c = np.zeros(shape, dtype=out_dt)
    else:
        _check(c_in, out_dt, B * 2 * M * N, "c_in")
        c = np.array(c_in, dtype=out_dt).reshape(shape).copy()
    a3 = a.reshape(B, 2 * M * kk)
    b3 = b.reshape(B, 2 * N * kk)
    L = lib()
    for i in range(B):
        ai, bi, ci = a3[i], b3[i], c[i]
        if type_in == INT1:
            L.oracle_gemm_int1(_ptr(ai), _ptr(bi), _ptr(ci), M, N, K, c_order,
                               alpha.real, alpha.imag, beta.real, beta.imag)
        else:
            L.oracle_gemm_float(_ptr(ai), _ptr(bi), _ptr(ci), M, N, K, type_in,
                                type_out, c_order, alpha.real, alpha.imag,
                                beta.real, beta.imag)
    return c


def gemm_float64(a, b, M, N, K, type_in, c_order=ROW_MAJOR):
    """Same product accumulated in float64 (the error-norm yardstick)."""
    B = a.size // (2 * M * K)
    _check(a, _STORAGE[type_in], B * 2 * M * K, "a")
    _check(b, _STORAGE[type_in], B * 2 * N * K, "b")
    shape = (B, 2, M, N) if c_order == ROW_MAJOR else (B, 2, N, M)
    c = np.zeros(shape, dtype=np.float64)
    a3, b3 = a.reshape(B, -1), b.reshape(B, -1)
    for i in range(B):
        lib().oracle_gemm_float64(_ptr(a3[i]), _ptr(b3[i]), _ptr(c[i]), M, N, K,
                                  type_in, c_order)
    return c


def transpose(x, B, M, N, Mc, Nc, nr_bits, input_axis=PLANAR):
    """Tiled-layout transpose; returns the flat output array, padded sizes."""
    packing = 32 if nr_bits == 1 else 1
    eb = 4 if nr_bits == 1 else nr_bits // 8
    if x.dtype.itemsize != eb:
        raise ValueError("element width does not match nr_bits")
    _check(x, x.dtype, B * 2 * M * (N // packing), "x")
    Mp = -(-M // Mc) * Mc
    Np = -(-N // Nc) * Nc
    out = np.empty(B * 2 * Mp * (Np // packing), dtype=x.dtype)
    lib().oracle_transpose(_ptr(x), _ptr(out), B, M, N, Mc, Nc, nr_bits, input_axis)
    return out


def pack_bits(x, input_axis=PLANAR):
    N = x.size
    _check(x, np.uint8, N, "x")
    out = np.empty((N + 31) // 32, dtype=np.uint32)
    lib().oracle_pack_bits(_ptr(x), _ptr(out), N, input_axis)
    return out


def unpack_bits(x, N):
    _check(x, np.uint32, (N + 31) // 32, "x")
    out = np.empty(N, dtype=np.uint8)
    lib().oracle_unpack_bits(_ptr(x), _ptr(out), N)
    return out


def to_float(x, vtype):
    """Decode an array of raw bit patterns to float32 with the oracle's decoders."""
    L = lib()
    fn = {FLOAT16: L.oracle_half_to_float, BFLOAT16: L.oracle_bf16_to_float,
          FLOAT8E4M3: L.oracle_e4m3_to_float, FLOAT8E5M2: L.oracle_e5m2_to_float}[vtype]
    flat = x.reshape(-1)
    return np.array([fn(int(v)) for v in flat], dtype=np.float32).reshape(x.shape)


def from_float(x, vtype):
    L = lib()
    fn = {FLOAT16: L.oracle_float_to_half, BFLOAT16: L.oracle_float_to_bf16}[vtype]
    flat = np.asarray(x, dtype=np.float32).reshape(-1)
    return np.array([fn(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(x))
