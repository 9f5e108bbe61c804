"""Pins the CPU oracle: the reference's own known-answer tests, closed forms,
independent library routines and brute force. No GPU needed."""
import itertools

import numpy as np
import pytest
import torch

import oracle as orc


def enc(vals, vtype):
    """Encode exactly representable python numbers into the storage type."""
    v = np.asarray(vals, dtype=np.float32)
    if vtype == orc.FLOAT16:
        return v.astype(np.float16).view(np.uint16)
    if vtype == orc.BFLOAT16:
        return (v.view(np.uint32) >> 16).astype(np.uint16)
    return v


# ---- reference known-answer tests (tests/golden/reference_kats.json) --------

import json
import os

KATS = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                   "reference_kats.json")))


@pytest.mark.parametrize("vtype", [orc.FLOAT16, orc.BFLOAT16, orc.FLOAT32])
def test_kat_float(vtype):
    k = KATS["float"]
    a, b = enc(k["a"], vtype), enc(k["b"], vtype)
    c = orc.gemm(a, b, k["M"], k["N"], k["K"], vtype, orc.FLOAT32, orc.ROW_MAJOR)
    assert c.reshape(-1).tolist() == k["c_row_major"]
    c = orc.gemm(a, b, k["M"], k["N"], k["K"], vtype, orc.FLOAT32, orc.COL_MAJOR)
    assert c.reshape(-1).tolist() == k["c_col_major"]


INT1_A = np.array(KATS["int1"]["a"], dtype=np.uint32)
INT1_B = np.array(KATS["int1"]["b"], dtype=np.uint32)


def test_kat_int1():
    k = KATS["int1"]
    c = orc.gemm(INT1_A, INT1_B, k["M"], k["N"], k["K"], orc.INT1, orc.INT32, orc.ROW_MAJOR,
                 c_in=np.zeros(8, np.int32))
    assert c.reshape(-1).tolist() == k["c_row_major"]
    c = orc.gemm(INT1_A, INT1_B, k["M"], k["N"], k["K"], orc.INT1, orc.INT32, orc.COL_MAJOR,
                 c_in=np.zeros(8, np.int32))
    assert c.reshape(-1).tolist() == k["c_col_major"]


def test_kat_alpha_beta_fp16():
    k = KATS["alpha_beta_float16"]
    c = orc.gemm(enc(k["a"], orc.FLOAT16), enc(k["b"], orc.FLOAT16), k["M"], k["N"], k["K"],
                 orc.FLOAT16, orc.FLOAT32, orc.ROW_MAJOR, alpha=complex(*k["alpha"]),
                 beta=complex(*k["beta"]), c_in=np.array(k["c_in"], dtype=np.float32))
    assert c.reshape(-1).tolist() == k["c_row_major"]


def test_kat_alpha_beta_int1():
    k = KATS["alpha_beta_int1"]
    c = orc.gemm(np.array(k["a"], dtype=np.uint32), np.array(k["b"], dtype=np.uint32), k["M"],
                 k["N"], k["K"], orc.INT1, orc.INT32, orc.ROW_MAJOR, alpha=complex(*k["alpha"]),
                 beta=complex(*k["beta"]), c_in=np.array(k["c_in"], dtype=np.int32))
    assert c.reshape(-1).tolist() == k["c_row_major"]


def test_reference_fixture_is_one_libc_rand_r_sequence_from_seed_zero():
    """test/gemm/mma.cpp:144-217: A then B from one sequence. The first value of glibc's
    rand_r at seed 0 is 1012484; the rest is checked against libc called directly."""
    import ctypes
    libc = ctypes.CDLL(None)
    libc.rand_r.argtypes = [ctypes.POINTER(ctypes.c_uint)]
    seed = ctypes.c_uint(0)
    raw = np.array([libc.rand_r(ctypes.byref(seed)) for _ in range(300)], dtype=np.int64)
    assert raw[0] == 1012484
    wa, wb = orc.reference_fixture(100, 200, words=True)
    assert np.array_equal(np.concatenate([wa, wb]), raw.astype(np.uint32))
    fa, fb = orc.reference_fixture(100, 200)
    want = raw.astype(np.float32) / np.float32(2 ** 31 - 1)   # RAND_MAX, converted to float
    assert np.array_equal(np.concatenate([fa, fb]), want)
    assert fa.min() >= 0 and fb.max() <= 1


def test_ceildiv():
    for a, b, want in KATS["ceildiv"]["cases"]:
        assert orc.ceildiv(a, b) == want


# ---- closed forms and independent routines -----------------------------------

def test_all_ones_closed_form():
    M, N, K = 5, 7, 40
    a = enc(np.ones(2 * M * K), orc.FLOAT16)
    b = enc(np.ones(2 * N * K), orc.FLOAT16)
    c = orc.gemm(a, b, M, N, K, orc.FLOAT16)
    assert np.all(c[0, 0] == 0) and np.all(c[0, 1] == 2 * K)               # test/hip/mma.cpp:76-77


@pytest.mark.parametrize("vtype", [orc.FLOAT16, orc.BFLOAT16, orc.FLOAT32])
@pytest.mark.parametrize("c_order", [orc.ROW_MAJOR, orc.COL_MAJOR])
def test_matches_complex128_matmul_exactly_on_small_integers(vtype, c_order):
    # Small integers keep every float product and partial sum exact, so the
    # float oracle must equal numpy's complex128 product bit for bit. A dropped
    # term, a wrong sign, a conjugate or transposed operand all fail here.
    rng = np.random.default_rng(11)
    B, M, N, K = 3, 9, 6, 13
    av = rng.integers(-4, 5, size=(B, 2, M, K))
    bv = rng.integers(-4, 5, size=(B, 2, N, K))
    cv = rng.integers(-8, 9, size=(B, 2, M, N))
    alpha, beta = 2 - 3j, -1 + 2j
    A = av[:, 0] + 1j * av[:, 1]
    Bm = bv[:, 0] + 1j * bv[:, 1]
    Cin = cv[:, 0] + 1j * cv[:, 1]
    want = alpha * np.einsum("bmk,bnk->bmn", A, Bm) + beta * Cin
    if c_order == orc.COL_MAJOR:
        want = want.transpose(0, 2, 1)
        cv = cv.transpose(0, 1, 3, 2)
    c = orc.gemm(enc(av.reshape(-1), vtype), enc(bv.reshape(-1), vtype), M, N, K,
                 vtype, orc.FLOAT32, c_order, alpha, beta,
                 c_in=np.ascontiguousarray(cv, dtype=np.float32).reshape(-1))
    assert np.array_equal(c[:, 0], want.real) and np.array_equal(c[:, 1], want.imag)


def _enc_any(vals, vtype):
    """Small integers / powers of two into the storage type, fp8 included."""
    v = np.asarray(vals, dtype=np.float32)
    if vtype == orc.FLOAT8E4M3:
        return torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    if vtype == orc.FLOAT8E5M2:
        return torch.from_numpy(v).to(torch.float8_e5m2).view(torch.uint8).numpy()
    return enc(v, vtype)


@pytest.mark.parametrize("vtype", [orc.FLOAT16, orc.BFLOAT16, orc.FLOAT32, orc.FLOAT8E4M3,
                                   orc.FLOAT8E5M2])
@pytest.mark.parametrize("c_order", [orc.ROW_MAJOR, orc.COL_MAJOR])
def test_float64_yardstick_matches_complex128_matmul_exactly(vtype, c_order):
    # The float64 product that the Frobenius criterion is measured against: on
    # exactly representable small integers every product and partial sum is
    # exact in double, so it must equal numpy's complex128 product bit for bit
    # (a dropped term, wrong sign, conjugate or transposed operand fails here).
    rng = np.random.default_rng(23)
    B, M, N, K = 2, 7, 5, 19
    # every value in [-4, 4] is exact in all five input types (e5m2 has two mantissa bits)
    av = rng.integers(-4, 5, size=(B, 2, M, K))
    bv = rng.integers(-4, 5, size=(B, 2, N, K))
    A = av[:, 0] + 1j * av[:, 1]
    Bm = bv[:, 0] + 1j * bv[:, 1]
    want = np.einsum("bmk,bnk->bmn", A, Bm)
    if c_order == orc.COL_MAJOR:
        want = want.transpose(0, 2, 1)
    a, b = _enc_any(av.reshape(-1), vtype), _enc_any(bv.reshape(-1), vtype)
    assert np.array_equal(orc.to_float(a, vtype) if vtype != orc.FLOAT32 else a,
                          av.reshape(-1).astype(np.float32))            # the encoding is exact
    c = orc.gemm_float64(a, b, M, N, K, vtype, c_order)
    assert c.dtype == np.float64
    assert np.array_equal(c[:, 0], want.real) and np.array_equal(c[:, 1], want.imag)


def test_float64_yardstick_keeps_what_float32_loses():
    # 2^13 * 2^13 + 1 - 2^26 = 1 in double, 0 in float: the yardstick accumulates in
    # double (and so can tell a float32 rounding error from a wrong result)
    a = enc([8192.0, 1.0, -8192.0, 0, 0, 0], orc.FLOAT16)   # re[3], im[3]
    b = enc([8192.0, 1.0, 8192.0, 0, 0, 0], orc.FLOAT16)
    c64 = orc.gemm_float64(a, b, 1, 1, 3, orc.FLOAT16)
    c32 = orc.gemm(a, b, 1, 1, 3, orc.FLOAT16)
    assert c64[0, 0, 0, 0] == 1.0 and c32[0, 0, 0, 0] == 0.0


def test_beta_zero_never_reads_c():
    a = enc(np.ones(2 * 2 * 4), orc.FLOAT16)
    c_in = np.full(2 * 2 * 2, np.nan, dtype=np.float32)
    c = orc.gemm(a, a.copy(), 2, 2, 4, orc.FLOAT16, c_in=c_in)
    assert np.isfinite(c).all()                                           # src/reference/GEMM.cpp:80-85


@pytest.mark.parametrize("type_out", [orc.FLOAT16, orc.BFLOAT16])
def test_narrow_output_is_rounded_float_result(type_out):
    rng = np.random.default_rng(5)
    M, N, K = 8, 8, 33
    a = rng.uniform(-1, 1, 2 * M * K).astype(np.float32)
    b = rng.uniform(-1, 1, 2 * N * K).astype(np.float32)
    wide = orc.gemm(a, b, M, N, K, orc.FLOAT32, orc.FLOAT32)
    narrow = orc.gemm(a, b, M, N, K, orc.FLOAT32, type_out)
    if type_out == orc.FLOAT16:
        want = wide.astype(np.float16).view(np.uint16)
    else:
        want = torch.from_numpy(wide).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(narrow, want)


@pytest.mark.parametrize("vtype,tdt", [(orc.FLOAT8E4M3, torch.float8_e4m3fn),
                                       (orc.FLOAT8E5M2, torch.float8_e5m2)])
def test_fp8_gemm_matches_float_gemm_on_decoded_inputs(vtype, tdt):
    rng = np.random.default_rng(7)
    M, N, K = 6, 5, 64
    a8 = rng.integers(0, 256, 2 * M * K, dtype=np.uint8)
    b8 = rng.integers(0, 256, 2 * N * K, dtype=np.uint8)
    # keep finite codes only
    dec = lambda x: torch.from_numpy(x).view(tdt).to(torch.float32).numpy()
    a8[~np.isfinite(dec(a8))] = 0
    b8[~np.isfinite(dec(b8))] = 0
    got = orc.gemm(a8, b8, M, N, K, vtype)
    want = orc.gemm(dec(a8), dec(b8), M, N, K, orc.FLOAT32)
    assert np.array_equal(got, want)


def test_decoders_exhaustive_against_independent_casts():
    codes8 = np.arange(256, dtype=np.uint8)
    for vtype, tdt in [(orc.FLOAT8E4M3, torch.float8_e4m3fn), (orc.FLOAT8E5M2, torch.float8_e5m2)]:
        want = torch.from_numpy(codes8).view(tdt).to(torch.float32).numpy()
        got = orc.to_float(codes8, vtype)
        assert np.array_equal(got, want, equal_nan=True)
    codes16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(orc.to_float(codes16, orc.FLOAT16),
                          codes16.view(np.float16).astype(np.float32), equal_nan=True)
    want = torch.from_numpy(codes16.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(orc.to_float(codes16, orc.BFLOAT16), want, equal_nan=True)


def test_encoders_against_independent_casts():
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 100,
        rng.standard_normal(20000).astype(np.float32) * 1e-6,
        np.array([0.0, -0.0, 65504, 65519.9, 65520, 70000, -70000, 6e-8, 2.98e-8, 3e-8,
                  6.1e-5, 6.0975e-5, np.inf, -np.inf, 1 + 2 ** -11, 1 + 3 * 2 ** -11], np.float32),
        # every half-way point between neighbouring halfs in [1, 2)
        (1 + (np.arange(1024) + 0.5) * 2.0 ** -10).astype(np.float32),
    ])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.from_float(x, orc.FLOAT16), want)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.from_float(x, orc.BFLOAT16), want)


# ---- 1-bit GEMM ---------------------------------------------------------------

def _bits_to_pm1(words, K):
    bits = np.unpackbits(words.view(np.uint8), bitorder="little").reshape(*words.shape[:-1], -1)
    return bits[..., :K].astype(np.int64) * 2 - 1


@pytest.mark.parametrize("K", [32, 64, 45, 100])
@pytest.mark.parametrize("c_order", [orc.ROW_MAJOR, orc.COL_MAJOR])
def test_int1_equals_pm1_integer_matmul(K, c_order):
    # bit 1 = +1, bit 0 = -1, LSB first; samples beyond K in the last word are
    # zero bits and must not contribute (src/reference/GEMM.cpp:163-183).
    rng = np.random.default_rng(K)
    B, M, N = 2, 5, 4
    kw = (K + 31) // 32
    mask = np.full(kw, 0xFFFFFFFF, dtype=np.uint32)
    if K % 32:
        mask[-1] = (1 << (K % 32)) - 1
    a = rng.integers(0, 2 ** 32, (B, 2, M, kw), dtype=np.uint32) & mask
    b = rng.integers(0, 2 ** 32, (B, 2, N, kw), dtype=np.uint32) & mask
    pa, pb = _bits_to_pm1(a, K), _bits_to_pm1(b, K)
    A = pa[:, 0] + 1j * pa[:, 1]
    Bm = pb[:, 0] + 1j * pb[:, 1]
    want = np.einsum("bmk,bnk->bmn", A, Bm)
    if c_order == orc.COL_MAJOR:
        want = want.transpose(0, 2, 1)
    c = orc.gemm(a.reshape(-1), b.reshape(-1), M, N, K, orc.INT1, orc.INT32, c_order,
                 c_in=np.zeros(B * 2 * M * N, np.int32))
    assert np.array_equal(c[:, 0], want.real) and np.array_equal(c[:, 1], want.imag)


def test_int1_brute_force_tiny():
    # every combination of a 1x1x2 problem (2 samples), checked sample by sample
    for ar, ai, br, bi in itertools.product(range(4), repeat=4):
        a = np.array([ar, ai], dtype=np.uint32)
        b = np.array([br, bi], dtype=np.uint32)
        c = orc.gemm(a, b, 1, 1, 2, orc.INT1, orc.INT32, c_in=np.zeros(2, np.int32))
        s = lambda w, k: 1 if (w >> k) & 1 else -1
        want = sum(complex(s(ar, k), s(ai, k)) * complex(s(br, k), s(bi, k)) for k in range(2))
        assert (c[0, 0, 0, 0], c[0, 1, 0, 0]) == (want.real, want.imag)


# ---- transpose ------------------------------------------------------------------

@pytest.mark.parametrize("axis", [orc.PLANAR, orc.INTERLEAVED])
@pytest.mark.parametrize("bits,dtype", [(8, np.uint8), (16, np.uint16), (32, np.uint32)])
@pytest.mark.parametrize("M,N,Mc,Nc", [(256, 128, 64, 64), (100, 40, 32, 16), (7, 5, 4, 4)])
def test_transpose_matches_numpy_reshape(axis, bits, dtype, M, N, Mc, Nc):
    rng = np.random.default_rng(M + N)
    B = 2
    x = rng.integers(1, np.iinfo(dtype).max, (B, 2, M, N), dtype=dtype)
    Mp, Np = -(-M // Mc) * Mc, -(-N // Nc) * Nc
    padded = np.zeros((B, 2, Mp, Np), dtype=dtype)
    padded[:, :, :M, :N] = x
    want = padded.reshape(B, 2, Mp // Mc, Mc, Np // Nc, Nc).transpose(0, 2, 4, 1, 3, 5)
    src = x if axis == orc.PLANAR else x.transpose(0, 2, 3, 1)
    got = orc.transpose(np.ascontiguousarray(src).reshape(-1), B, M, N, Mc, Nc, bits, axis)
    assert np.array_equal(got, want.reshape(-1))


def test_transpose_one_bit_moves_words():
    rng = np.random.default_rng(1)
    B, M, N, Mc, Nc = 2, 256, 128, 64, 64          # test/transpose/transpose.cpp:37-42
    x = rng.integers(0, 2 ** 32, (B, 2, M, N // 32), dtype=np.uint32)
    want = x.reshape(B, 2, M // Mc, Mc, N // Nc, Nc // 32).transpose(0, 2, 4, 1, 3, 5)
    got = orc.transpose(x.reshape(-1), B, M, N, Mc, Nc, 1, orc.PLANAR)
    assert np.array_equal(got, want.reshape(-1))


# ---- packing ---------------------------------------------------------------------

@pytest.mark.parametrize("N", [2048, 64, 100, 31])
def test_pack_matches_numpy_packbits(N):
    rng = np.random.default_rng(N)
    x = rng.integers(0, 2, N, dtype=np.uint8)
    pad = np.zeros((-N) % 32, dtype=np.uint8)
    want = np.packbits(np.concatenate([x, pad]), bitorder="little").view(np.uint32)
    assert np.array_equal(orc.pack_bits(x), want)
    assert np.array_equal(orc.unpack_bits(want, N), x)


def test_pack_treats_any_nonzero_byte_as_one():
    x = np.array([0, 7, 0, 255, 128, 0, 1, 2] * 4, dtype=np.uint8)
    assert orc.pack_bits(x)[0] == int("".join("1" if v else "0" for v in x[::-1]), 2)


def test_pack_interleaved_moves_reals_first():
    rng = np.random.default_rng(0)
    N = 2048                                        # test/packing/packing.cpp:158
    x = rng.integers(0, 2, N, dtype=np.uint8)
    planar = np.concatenate([x[0::2], x[1::2]])
    assert np.array_equal(orc.pack_bits(x, orc.INTERLEAVED), orc.pack_bits(planar))
