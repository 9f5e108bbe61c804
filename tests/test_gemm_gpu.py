"""GPU parity tests of the complex GEMM against the CPU oracle, through the C ABI
(ccglib_amd.GEMM / Transpose are thin ctypes bindings). Shapes and cases follow
the reference's test/gemm/mma.cpp."""
import json
import os

import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import (ORC_TYPE, check_float, dequantize, device_zeros, quantize, stream,
                      to_device, to_host, transpose_operand)

pytestmark = pytest.mark.gpu

VT = cc.ValueType
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved
ROW, COL = cc.MemOrder.row_major, cc.MemOrder.col_major
OUT_NP = {VT.float32: np.float32, VT.float16: np.uint16, VT.bfloat16: np.uint16, VT.int32: np.int32}

FLOAT_PAIRS = [(VT.float16, VT.float32), (VT.float16, VT.float16), (VT.bfloat16, VT.float32),
               (VT.bfloat16, VT.bfloat16), (VT.float8e4m3, VT.float32), (VT.float8e5m2, VT.float32),
               (VT.float32, VT.float32), (VT.float32, VT.float16), (VT.float32, VT.bfloat16)]


def run_gemm(qa, qb, B, M, N, K, tin, tout, variant, c_axis=PLANAR, c_order=ROW, alpha=1, beta=0,
             c_in=None):
    """Returns C as a numpy array in planar layout [B][2][rows][cols] of the
    output storage type, whatever layout the GPU wrote."""
    if variant == cc.Variant.opt:
        d_a = transpose_operand(qa, B, M, K, tin)
        d_b = transpose_operand(qb, B, N, K, tin)
    else:
        d_a, d_b = to_device(qa), to_device(qb)
    out_np = OUT_NP[tout]
    n_out = B * 2 * M * N
    if c_in is not None:
        c_dev_in = c_in
        if c_axis == INTERLEAVED:
            rows, cols = (M, N) if c_order == ROW else (N, M)
            c_dev_in = np.ascontiguousarray(c_in.reshape(B, 2, rows, cols).transpose(0, 2, 3, 1))
        d_c = to_device(c_dev_in.reshape(-1))
    else:
        # poison the output: every element must be written, none read
        d_c = to_device(np.full(n_out, 0x7fc0 if out_np == np.uint16 else -1, dtype=out_np)
                        if out_np != np.float32 else np.full(n_out, np.nan, dtype=np.float32))
    gemm = cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(tin, tout), variant, c_axis, c_order,
                   ROW, COL, alpha, beta)
    gemm.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    c = to_host(d_c, out_np)
    rows, cols = (M, N) if c_order == ROW else (N, M)
    if c_axis == INTERLEAVED:
        c = np.ascontiguousarray(c.reshape(B, rows, cols, 2).transpose(0, 3, 1, 2))
    return c.reshape(B, 2, rows, cols)


def reference_inputs(B, M, N, K, tin, signed, seed):
    rng = np.random.default_rng(seed)
    lo = -1.0 if signed else 0.0   # the reference's fixtures use [0, 1] (test/gemm/mma.cpp:144-217)
    a = rng.uniform(lo, 1.0, (B, 2, M, K)).astype(np.float32)
    b = rng.uniform(lo, 1.0, (B, 2, N, K)).astype(np.float32)
    return quantize(a, tin).reshape(-1), quantize(b, tin).reshape(-1)


def float_case(B, M, N, K, tin, tout, variant, c_axis, c_order, signed=True, alpha=1, beta=0, seed=0,
               inputs=None):
    qa, qb = inputs if inputs is not None else reference_inputs(B, M, N, K, tin, signed, seed)
    c_in = None
    if beta != 0:
        rng = np.random.default_rng(seed + 1)
        c32 = rng.uniform(0, 1, B * 2 * M * N).astype(np.float32)
        c_in = c32 if tout == VT.float32 else quantize(c32, tout)
    got = run_gemm(qa, qb, B, M, N, K, tin, tout, variant, c_axis, c_order, alpha, beta, c_in)
    want = orc.gemm(qa, qb, M, N, K, ORC_TYPE[tin], ORC_TYPE[tout], int(c_order), alpha, beta, c_in)
    gotf = dequantize(got, tout)
    wantf = dequantize(want, tout)
    want64 = orc.gemm_float64(qa, qb, M, N, K, ORC_TYPE[tin], int(c_order))
    if alpha != 1 or beta != 0:
        w = (want64[:, 0] + 1j * want64[:, 1]) * complex(alpha)
        if beta != 0:
            ci = dequantize(c_in, tout).reshape(want64.shape).astype(np.float64)
            w = w + complex(beta) * (ci[:, 0] + 1j * ci[:, 1])
        want64 = np.stack([w.real, w.imag], axis=1)
    return check_float(gotf, wantf, want64, tin, tout)


# ---- reference known answers, through the GPU --------------------------------------

# tests/golden/reference_kats.json: the vectors of the reference's test/gemm/reference.cpp
KATS = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                   "reference_kats.json")))
KAT_A, KAT_B = KATS["float"]["a"], KATS["float"]["b"]


@pytest.mark.parametrize("tin", [VT.float16, VT.bfloat16, VT.float32])
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
def test_kat_float(tin, variant):
    k = KATS["float"]
    qa, qb = quantize(np.array(k["a"]), tin), quantize(np.array(k["b"]), tin)
    c = run_gemm(qa, qb, 1, k["M"], k["N"], k["K"], tin, VT.float32, variant)
    assert c.reshape(-1).tolist() == k["c_row_major"]
    c = run_gemm(qa, qb, 1, k["M"], k["N"], k["K"], tin, VT.float32, variant, c_order=COL)
    assert c.reshape(-1).tolist() == k["c_col_major"]


def test_kat_alpha_beta_fp16():
    k = KATS["alpha_beta_float16"]
    c = run_gemm(quantize(np.array(k["a"]), VT.float16), quantize(np.array(k["b"]), VT.float16), 1,
                 k["M"], k["N"], k["K"], VT.float16, VT.float32, cc.Variant.basic,
                 alpha=complex(*k["alpha"]), beta=complex(*k["beta"]),
                 c_in=np.array(k["c_in"], dtype=np.float32))
    assert c.reshape(-1).tolist() == k["c_row_major"]


def test_all_ones_closed_form():
    # test/hip/mma.cpp:20-83: real part 0, imaginary part 2K
    B, M, N, K = 3, 512, 512, 512
    q = quantize(np.ones(B * 2 * M * K), VT.float16)
    c = run_gemm(q, q.copy(), B, M, N, K, VT.float16, VT.float32, cc.Variant.basic)
    assert np.all(c[:, 0] == 0) and np.all(c[:, 1] == 2 * K)


# ---- the reference's fixture: B = 16, aligned and ragged shapes ------------------------

SHAPES = [(128, 256, 64), (100, 60, 40)]   # test/gemm/mma.cpp:402-408


@pytest.mark.parametrize("tin,tout", FLOAT_PAIRS)
@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("c_order", [ROW, COL])
def test_basic(tin, tout, M, N, K, c_order):
    float_case(16, M, N, K, tin, tout, cc.Variant.basic, PLANAR, c_order, signed=False)
    float_case(16, M, N, K, tin, tout, cc.Variant.basic, PLANAR, c_order, signed=True, seed=3)


@pytest.mark.parametrize("tin,tout", FLOAT_PAIRS)
@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("c_order", [ROW, COL])
@pytest.mark.parametrize("c_axis", [PLANAR, INTERLEAVED])
def test_opt(tin, tout, M, N, K, c_order, c_axis):
    float_case(16, M, N, K, tin, tout, cc.Variant.opt, c_axis, c_order, signed=False)
    float_case(16, M, N, K, tin, tout, cc.Variant.opt, c_axis, c_order, signed=True, seed=5)


# The reference's own test inputs, literally (test/gemm/mma.cpp:144-217): 16 batches, A
# then B filled from one libc rand_r sequence that starts at seed 0, at the aligned and
# the unaligned shape of test/gemm/mma.cpp:402-408, for every pair of types it tests.
@pytest.mark.parametrize("tin,tout", FLOAT_PAIRS)
@pytest.mark.parametrize("M,N,K", [(128, 256, 64), (100, 60, 40)])
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
@pytest.mark.parametrize("c_order", [ROW, COL])
def test_reference_seeded_inputs(tin, tout, M, N, K, variant, c_order):
    B = 16
    a, b = orc.reference_fixture(B * 2 * M * K, B * 2 * N * K)
    float_case(B, M, N, K, tin, tout, variant, PLANAR, c_order,
               inputs=(quantize(a, tin), quantize(b, tin)))


def basic_variant(variant):
    """The basic variant copies operands with ragged rows (K·size not a multiple of 16
    bytes) into the tiled layout first; "basic_no_retile" switches that off, which
    leaves the kernel that loads ragged rows itself."""
    if variant == "basic_no_retile":
        cc.set_option(cc.Option.basic_retile, 0)
        return cc.Variant.basic
    return variant


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (17, 5, 3), (129, 131, 33), (64, 300, 1000),
                                   (257, 129, 72), (130, 2, 2049)])
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt, "basic_no_retile"])
def test_odd_shapes_fp16(M, N, K, variant):
    variant = basic_variant(variant)
    float_case(2, M, N, K, VT.float16, VT.float32, variant, PLANAR, ROW, seed=M + N + K)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (17, 5, 3), (129, 131, 33), (64, 300, 1000), (257, 129, 72)])
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt, "basic_no_retile"])
def test_odd_shapes_fp32(M, N, K, variant):
    # K not a multiple of the 16 values of a tile row, rows that are not whole 16-byte chunks
    variant = basic_variant(variant)
    float_case(2, M, N, K, VT.float32, VT.float32, variant, PLANAR, ROW, seed=M + N + K)


@pytest.mark.parametrize("c_order", [ROW, COL])
@pytest.mark.parametrize("tin", [VT.float16, VT.bfloat16, VT.float8e4m3])
def test_interleaved_c_alpha_only(tin, c_order):
    # beta = 0 and aligned rows: wave tiles inside C go through the LDS-staged wide
    # stores, the ragged right and bottom edges (M = 300, N = 328) through the direct ones
    float_case(3, 300, 328, 96, tin, VT.float32, cc.Variant.opt, INTERLEAVED, c_order,
               alpha=0.75 - 0.5j, seed=21)
    float_case(2, 256, 512, 64, tin, VT.float32, cc.Variant.opt, INTERLEAVED, c_order, seed=22)


@pytest.mark.parametrize("c_order", [ROW, COL])
@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float16), (VT.bfloat16, VT.bfloat16),
                                      (VT.float32, VT.float16), (VT.float32, VT.bfloat16)])
def test_narrow_planar_c_alpha_only(tin, tout, c_order):
    # 16-bit planar C, beta = 0, rows of whole 16-byte vectors: wave tiles inside C take the
    # LDS-staged stores, the ragged edges (M = 300, N = 328) the direct ones
    float_case(3, 300, 328, 96, tin, tout, cc.Variant.opt, PLANAR, c_order, alpha=0.75 - 0.5j, seed=23)
    float_case(2, 256, 512, 64, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=24)
    float_case(2, 256, 516, 64, tin, tout, cc.Variant.basic, PLANAR, c_order, seed=25)   # N % 8 != 0: direct


def test_opt_rejects_misaligned_tiles():
    # tiles go to LDS in 16-byte pieces: a tiled operand that is not 16-byte aligned is an
    # argument error, not a fault
    B, M, N, K = 1, 128, 128, 64
    q = quantize(np.ones(B * 2 * M * K), VT.float16)
    d_a, d_b = transpose_operand(q, B, M, K, VT.float16), transpose_operand(q, B, N, K, VT.float16)
    d_c = to_device(np.zeros(B * 2 * M * N, dtype=np.float32))
    gemm = cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(VT.float16, VT.float32), cc.Variant.opt)
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        gemm.Run(d_a.data_ptr() + 2, d_b.data_ptr(), d_c.data_ptr())
    gemm.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    c = to_host(d_c, np.float32).reshape(B, 2, M, N)
    assert np.all(c[:, 0] == 0) and np.all(c[:, 1] == 2 * K)


def test_fp32_alpha_beta_and_many_tiles():
    float_case(3, 256, 320, 96, VT.float32, VT.float32, cc.Variant.opt, INTERLEAVED, COL,
               alpha=0.75 - 0.5j, beta=0.5 - 0.25j)
    float_case(40, 256, 1024, 32, VT.float32, VT.float16, cc.Variant.opt, PLANAR, ROW, seed=13)


@pytest.mark.parametrize("tin", [VT.float8e4m3, VT.float8e5m2])
@pytest.mark.parametrize("K", [1, 63, 64, 65, 128, 192, 200])
def test_fp8_k_tails(tin, K):
    # an MFMA consumes two 64-value K tiles; odd tile counts and ragged tails
    float_case(2, 70, 50, K, tin, VT.float32, cc.Variant.basic, PLANAR, ROW, seed=K)
    with cc.option(cc.Option.basic_retile, 0):
        float_case(2, 70, 50, K, tin, VT.float32, cc.Variant.basic, PLANAR, ROW, seed=K)
    float_case(2, 70, 50, K, tin, VT.float32, cc.Variant.opt, PLANAR, COL, seed=K + 1)


@pytest.mark.parametrize("m", [255, 256])     # test/gemm/mma.cpp:645-711
@pytest.mark.parametrize("variant,c_axis", [(cc.Variant.basic, PLANAR), (cc.Variant.opt, PLANAR),
                                            (cc.Variant.opt, INTERLEAVED)])
def test_alpha_beta_fp16(m, variant, c_axis):
    float_case(16, m, 128, 256, VT.float16, VT.float32, variant, c_axis, ROW, signed=False,
               alpha=0.3 + 1.6j, beta=0.8 - 1.1j)


@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float16), (VT.bfloat16, VT.bfloat16)])
def test_alpha_beta_narrow_output(tin, tout):
    float_case(4, 100, 60, 40, tin, tout, cc.Variant.opt, PLANAR, COL, alpha=-0.5 + 0.25j,
               beta=1.5 + 0.5j)


@pytest.mark.parametrize("tin", [VT.float8e4m3, VT.float8e5m2])
@pytest.mark.parametrize("variant,c_axis,beta", [(cc.Variant.opt, PLANAR, 0), (cc.Variant.opt, PLANAR, 0.5 - 0.25j),
                                                 (cc.Variant.opt, INTERLEAVED, 0.5 - 0.25j),
                                                 (cc.Variant.basic, PLANAR, 0.5 - 0.25j)])
def test_alpha_beta_fp8(tin, variant, c_axis, beta):
    # whole 64 x 64 wave tiles inside C (wide stores through LDS when beta is 0) and ragged ones
    float_case(3, 256, 320, 192, tin, VT.float32, variant, c_axis, ROW, alpha=0.75 - 0.5j, beta=beta)
    float_case(2, 200, 130, 128, tin, VT.float32, variant, c_axis, COL, alpha=-1.25j, beta=beta, seed=5)


@pytest.mark.parametrize("tin", [VT.float16, VT.float8e4m3])
def test_more_c_tiles_than_resident_blocks(tin):
    # 1536 C tiles of 256 x 128 for at most 256 persistent blocks: every block
    # walks several tiles, with the copy running across the tile boundaries
    float_case(48, 256, 1024, 128, tin, VT.float32, cc.Variant.opt, PLANAR, ROW, seed=11)


@pytest.mark.parametrize("beta", [0, 0.5 - 0.25j])
@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float32), (VT.bfloat16, VT.bfloat16),
                                      (VT.float8e4m3, VT.float32), (VT.float32, VT.float32),
                                      (VT.int1, VT.int32)])
@pytest.mark.parametrize("c_order", [ROW, COL])
def test_k_zero_basic(tin, tout, beta, c_order):
    """An empty product: C = beta C (the basic variant, which writes planar C only; the
    tiled layout of the opt variant has no K = 0). beta = 0 must overwrite whatever C
    held."""
    B, M, N = 3, 70, 130
    rng = np.random.default_rng(4)
    if tout == VT.int32:
        beta = int(beta.real * 4) if beta else 0
        c_in = rng.integers(-1000, 1000, B * 2 * M * N).astype(np.int32)
    else:
        c32 = rng.uniform(-1, 1, B * 2 * M * N).astype(np.float32)
        c_in = c32 if tout == VT.float32 else quantize(c32, tout)
    d_c = to_device(c_in)
    d_ab = device_zeros(64)
    cc.GEMM(B, M, N, 0, 0, stream(), cc.Precision(tin, tout), cc.Variant.basic, PLANAR, c_order, ROW,
            COL, 1, beta).Run(d_ab.data_ptr(), d_ab.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_c, OUT_NP[tout])
    empty = np.zeros(0, dtype=np.uint32 if tin == VT.int1 else quantize(np.zeros(1), tin).dtype)
    want = orc.gemm(empty, empty, M, N, 0, ORC_TYPE[tin], ORC_TYPE[tout], int(c_order), 1, beta, c_in, batch=B)
    got = np.ascontiguousarray(got).reshape(want.shape)
    if tout == VT.int32:
        assert np.array_equal(got, want)
    else:   # beta C in float; a fused multiply-add may round the last bit differently
        gotf, wantf = dequantize(got, tout), dequantize(want, tout)
        if beta == 0:
            assert not gotf.any()
        ulp = {VT.float32: 2.0 ** -23, VT.bfloat16: 2.0 ** -7}[tout]
        assert np.abs(gotf - wantf).max() <= 2 * ulp


def test_beta_zero_ignores_nan_in_c():
    # run_gemm poisons C with NaN whenever beta == 0: every float case above covers
    # it; this one states the property on its own
    qa, qb = reference_inputs(1, 8, 8, 8, VT.float16, True, 0)
    c = run_gemm(qa, qb, 1, 8, 8, 8, VT.float16, VT.float32, cc.Variant.basic)
    assert np.isfinite(c).all()


def test_config1_reference_cpu_case():
    # batch 1, 256^3, fp16 in, fp32 out, U[-1, 1]
    for variant in (cc.Variant.basic, cc.Variant.opt):
        float_case(1, 256, 256, 256, VT.float16, VT.float32, variant, PLANAR, ROW, seed=1)


def test_batches_are_independent():
    qa, qb = reference_inputs(4, 96, 80, 64, VT.bfloat16, True, 9)
    full = run_gemm(qa, qb, 4, 96, 80, 64, VT.bfloat16, VT.float32, cc.Variant.opt)
    a4, b4 = qa.reshape(4, -1), qb.reshape(4, -1)
    for i in range(4):
        one = run_gemm(a4[i].copy(), b4[i].copy(), 1, 96, 80, 64, VT.bfloat16, VT.float32,
                       cc.Variant.opt)
        assert np.array_equal(one[0], full[i])


# ---- 1-bit ------------------------------------------------------------------------------

@pytest.fixture(params=["mfma", "popcount"])
def int1_kernel(request):
    """The 1-bit GEMM has two implementations behind one entry point: the fp4 MFMA
    kernel that expands the packed words in registers (default, where the layout
    allows it: tiled operands, planar rows of whole 16-byte chunks, other planar
    rows after re-tiling) and XOR + popcount on the vector ALUs (the fallback, which
    the option selects for everything). The option is read when the GEMM object is
    created."""
    if request.param == "popcount":
        cc.set_option(cc.Option.int1_popcount, 1)
    return request.param


def int1_case(B, M, N, K, variant, c_axis=PLANAR, c_order=ROW, alpha=1, beta=0, seed=0, inputs=None):
    rng = np.random.default_rng(seed)
    kw = (K + 31) // 32
    mask = np.full(kw, 0xFFFFFFFF, dtype=np.uint32)
    if K % 32:
        mask[-1] = (1 << (K % 32)) - 1
    if inputs is not None:
        a, b = inputs
    else:
        a = (rng.integers(0, 2 ** 32, (B, 2, M, kw), dtype=np.uint32) & mask).reshape(-1)
        b = (rng.integers(0, 2 ** 32, (B, 2, N, kw), dtype=np.uint32) & mask).reshape(-1)
    c_in = rng.integers(-2 ** 30, 2 ** 30, B * 2 * M * N).astype(np.int32)
    d_a = transpose_operand(a, B, M, K, VT.int1) if variant == cc.Variant.opt else to_device(a)
    d_b = transpose_operand(b, B, N, K, VT.int1) if variant == cc.Variant.opt else to_device(b)
    rows, cols = (M, N) if c_order == ROW else (N, M)
    c_dev = c_in.reshape(B, 2, rows, cols)
    if c_axis == INTERLEAVED:
        c_dev = c_dev.transpose(0, 2, 3, 1)
    d_c = to_device(np.ascontiguousarray(c_dev).reshape(-1))
    cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(VT.int1, VT.int32), variant, c_axis, c_order,
            ROW, COL, alpha, beta).Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_c, np.int32)
    if c_axis == INTERLEAVED:
        got = got.reshape(B, rows, cols, 2).transpose(0, 3, 1, 2)
    want = orc.gemm(a, b, M, N, K, orc.INT1, orc.INT32, int(c_order), alpha, beta, c_in)
    assert np.array_equal(got.reshape(want.shape), want)


@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
def test_kat_int1(variant, int1_kernel):
    for k, c_in, alpha, beta in [
            (KATS["int1"], np.zeros(8, np.int32), 1, 0),
            (KATS["alpha_beta_int1"], np.array(KATS["alpha_beta_int1"]["c_in"], dtype=np.int32),
             complex(*KATS["alpha_beta_int1"]["alpha"]), complex(*KATS["alpha_beta_int1"]["beta"]))]:
        a, b = np.array(k["a"], dtype=np.uint32), np.array(k["b"], dtype=np.uint32)
        if variant == cc.Variant.opt:
            d_a = transpose_operand(a, 1, k["M"], k["K"], VT.int1)
            d_b = transpose_operand(b, 1, k["N"], k["K"], VT.int1)
        else:
            d_a, d_b = to_device(a), to_device(b)
        d_c = to_device(c_in)
        cc.GEMM(1, k["M"], k["N"], k["K"], 0, stream(), cc.Precision(VT.int1, VT.int32), variant, PLANAR,
                ROW, ROW, COL, alpha, beta).Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
        torch.cuda.synchronize()
        assert to_host(d_c, np.int32).tolist() == k["c_row_major"]


@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
@pytest.mark.parametrize("c_order", [ROW, COL])
@pytest.mark.parametrize("M,N,K", [(64, 64, 256), (128, 128, 512), (100, 60, 1024), (130, 257, 96),
                                   (256, 128, 4096)])
def test_int1(variant, c_order, M, N, K, int1_kernel):
    int1_case(16 if M == 64 else 3, M, N, K, variant, PLANAR, c_order, seed=M)


# the reference's 1-bit test inputs: raw rand_r values as packed words, 16 batches of
# 64 x 64 x 256 (test/gemm/mma.cpp:204-213, 422-436)
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
@pytest.mark.parametrize("c_order", [ROW, COL])
def test_int1_reference_seeded_inputs(variant, c_order, int1_kernel):
    B, M, N, K = 16, 64, 64, 256
    inputs = orc.reference_fixture(B * 2 * M * K // 32, B * 2 * N * K // 32, words=True)
    int1_case(B, M, N, K, variant, c_order=c_order, inputs=inputs)


@pytest.mark.parametrize("c_order", [ROW, COL])
@pytest.mark.parametrize("K", [512, 160])
def test_int1_interleaved_output(c_order, K, int1_kernel):
    int1_case(2, 100, 60, K, cc.Variant.opt, INTERLEAVED, c_order)


@pytest.mark.parametrize("K", [45, 100, 1000])
def test_int1_k_not_multiple_of_32(K, int1_kernel):
    int1_case(2, 20, 30, K, cc.Variant.basic, seed=K)


@pytest.mark.parametrize("K", [32, 160, 1056])
def test_int1_k_not_multiple_of_a_tile(K, int1_kernel):
    # whole words, but neither whole 128-sample nor whole 512-sample tiles
    int1_case(2, 130, 70, K, cc.Variant.opt, seed=K + 1)
    int1_case(2, 130, 70, K, cc.Variant.basic, seed=K + 2)


def test_int1_largest_k_of_one_mfma_launch_and_beyond():
    # K = 2^22 is the largest K of one launch on the fp4 MFMA (sums up to 2 K = 2^23 stay
    # exact in fp32); identical operands give the extreme value im = 2 K in every element.
    # A longer K is multiplied in pieces of 2^22 samples that the integer epilogue adds up.
    for K in (1 << 22, (1 << 22) + 512):
        kw = K // 32
        rng = np.random.default_rng(K)
        row = rng.integers(0, 2 ** 32, kw, dtype=np.uint32)
        a = np.broadcast_to(row, (1, 2, 8, kw)).copy().reshape(-1)
        b = np.broadcast_to(row, (1, 2, 4, kw)).copy().reshape(-1)
        d_a, d_b = transpose_operand(a, 1, 8, K, VT.int1), transpose_operand(b, 1, 4, K, VT.int1)
        d_c = to_device(np.zeros(2 * 8 * 4, np.int32))
        cc.GEMM(1, 8, 4, K, 0, stream(), cc.Precision(VT.int1, VT.int32), cc.Variant.opt).Run(
            d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
        torch.cuda.synchronize()
        got = to_host(d_c, np.int32).reshape(2, 8, 4)
        assert (got[0] == 0).all() and (got[1] == 2 * K).all()


@pytest.mark.parametrize("K", [256, 96])
def test_int1_basic_word_aligned_pointers(K, int1_kernel):
    # planar rows that start at a word but not at a 16-byte boundary: no kernel may read
    # them in 16-byte pieces
    B, M, N = 2, 70, 90
    rng = np.random.default_rng(K)
    kw = K // 32
    a = rng.integers(0, 2 ** 32, B * 2 * M * kw, dtype=np.uint32)
    b = rng.integers(0, 2 ** 32, B * 2 * N * kw, dtype=np.uint32)
    d_a = to_device(np.concatenate([np.zeros(1, np.uint32), a]))
    d_b = to_device(np.concatenate([np.zeros(3, np.uint32), b]))
    d_c = to_device(np.zeros(B * 2 * M * N, np.int32))
    cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(VT.int1, VT.int32), cc.Variant.basic).Run(
        d_a.data_ptr() + 4, d_b.data_ptr() + 12, d_c.data_ptr())
    torch.cuda.synchronize()
    want = orc.gemm(a, b, M, N, K, orc.INT1, orc.INT32)
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)


@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
@pytest.mark.parametrize("K", [256, 1152])
def test_int1_several_c_tiles_per_block(variant, K):
    # 6 x 4 x 9 C tiles of 256 x 128 for at most 256 persistent blocks, with one and
    # three K tiles per C tile (fewer than the copy's lead, and more)
    int1_case(6, 1024, 1100, K, variant, seed=K)


@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
@pytest.mark.parametrize("K", [(1 << 22) + 128, 2 * (1 << 22) + 4096 + 96])
def test_int1_k_in_pieces(variant, K, int1_kernel):
    # two and three pieces, the last one a partial tile; alpha and beta applied once
    if variant == cc.Variant.basic and K % 128:
        K -= K % 128       # planar rows of whole 16-byte chunks (no tiled copy of 2 x 8 MiB rows)
    int1_case(2, 40, 24, K, variant, c_order=COL, alpha=2 - 1j, beta=1 + 3j, seed=K % 1000)


@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
def test_int1_alpha_beta(variant, int1_kernel):
    # test/gemm/mma.cpp:713-775
    int1_case(16, 256, 128, 256, variant, alpha=2 - 3j, beta=3 - 2j)


# ---- both block tiles of the MFMA kernels ------------------------------------------------

@pytest.mark.parametrize("block_tile", [1, 2])
@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float32), (VT.bfloat16, VT.bfloat16),
                                      (VT.float32, VT.float16), (VT.float8e4m3, VT.float32)])
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
def test_block_tiles(block_tile, tin, tout, variant):
    """The dispatch picks 256 x 128 or 128 x 128 block tiles by problem size (option
    GEMM_BLOCK_TILE = 0); here each is forced in turn on the same problems: one
    partial tile, many tiles with ragged edges, a long K, alpha / beta, column-major
    and (opt) interleaved C."""
    with cc.option(cc.Option.gemm_block_tile, block_tile):
        float_case(1, 70, 50, 40, tin, tout, variant, PLANAR, ROW, seed=1)
        float_case(2, 300, 520, 96, tin, tout, variant, PLANAR, COL, seed=2)
        float_case(1, 130, 260, 1064, tin, tout, variant, PLANAR, ROW, alpha=1.5 - 0.5j, beta=0.25 + 1j,
                   seed=3)
        if variant == cc.Variant.opt:
            float_case(3, 257, 129, 72, tin, tout, variant, INTERLEAVED, ROW, alpha=2j, seed=4)


@pytest.mark.parametrize("block_tile", [1, 2])
@pytest.mark.parametrize("variant", [cc.Variant.basic, cc.Variant.opt])
def test_block_tiles_int1(block_tile, variant):
    with cc.option(cc.Option.gemm_block_tile, block_tile):
        int1_case(2, 70, 50, 640, variant, seed=1)
        int1_case(3, 300, 520, 1536, variant, c_order=COL, alpha=2 - 1j, beta=1 + 3j, seed=2)
        int1_case(1, 257, 129, 4096 + 512, variant, seed=3)
        if variant == cc.Variant.opt:
            int1_case(2, 130, 260, 1024, variant, c_axis=INTERLEAVED, seed=4)


@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float32), (VT.float16, VT.float16),
                                      (VT.bfloat16, VT.float32), (VT.bfloat16, VT.bfloat16)])
@pytest.mark.parametrize("c_order", [ROW, COL])
def test_wide_block_tile(tin, tout, c_order):
    """GEMM_BLOCK_TILE = 3: the 192 x 256 block (16-bit tiled input, planar C without
    beta, M and N multiples of 64, K of more than one tile) against the
    oracle: tiles that lie inside C and tiles of which only one or two 64-column
    groups or some of the four 64-row pieces do, widths that end in one or two short
    tiles of 128 columns, two to many K tiles, more C tiles than compute units, and a K
    with a partial last tile."""
    with cc.option(cc.Option.gemm_block_tile, 3):
        float_case(2, 256, 192, 64, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=1)
        float_case(3, 320, 448, 96, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=2)
        float_case(1, 64, 64, 40, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=3)
        float_case(2, 512, 832, 1000, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=4)
        float_case(40, 256, 576, 72, tin, tout, cc.Variant.opt, PLANAR, c_order, signed=False, seed=5)
        # with a complex alpha (applied to the accumulators on their way out)
        float_case(3, 320, 448, 96, tin, tout, cc.Variant.opt, PLANAR, c_order, alpha=1.5 - 0.5j, seed=6)
        float_case(2, 256, 192, 2048, tin, tout, cc.Variant.opt, PLANAR, c_order, alpha=-0.25 + 2j, seed=7)
        # 448 = 192 + 2 x 128 columns: 90 full tiles and 180 short ones, more tiles than compute
        # units (blocks with a full tile and then a short one, blocks with one short tile); then
        # 150 full and 300 short tiles (blocks with two short tiles)
        n, m = (448, 256) if c_order == ROW else (256, 448)
        float_case(90, m, n, 96, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=8)
        float_case(150, m, n, 64, tin, tout, cc.Variant.opt, PLANAR, c_order, alpha=0.5 + 0.5j, seed=9)
        # 4224 = 20 x 192 + 3 x 128 columns although 192 divides 4224: with 12 rows of tiles, 23
        # tiles per row even out the work of the 256 blocks where 22 would not
        n, m = (4224, 512) if c_order == ROW else (512, 4224)
        float_case(6, m, n, 64, tin, tout, cc.Variant.opt, PLANAR, c_order, seed=10)


def test_wide_block_tile_falls_back():
    """GEMM_BLOCK_TILE = 3 where the 192 x 256 kernel does not apply (ragged M or N,
    beta, interleaved C, K of one tile, fp8): the other kernels compute it."""
    with cc.option(cc.Option.gemm_block_tile, 3):
        float_case(2, 300, 520, 96, VT.float16, VT.float32, cc.Variant.opt, PLANAR, ROW, seed=1)
        float_case(1, 256, 192, 64, VT.float16, VT.float32, cc.Variant.opt, PLANAR, ROW,
                   alpha=1.5 - 0.5j, beta=0.25 + 1j, seed=2)
        float_case(1, 256, 192, 64, VT.float16, VT.float32, cc.Variant.opt, PLANAR, ROW, beta=1, seed=7)
        float_case(1, 256, 192, 64, VT.float16, VT.float32, cc.Variant.opt, INTERLEAVED, ROW, seed=3)
        float_case(1, 256, 192, 32, VT.float16, VT.float32, cc.Variant.opt, PLANAR, ROW, seed=4)
        float_case(1, 256, 192, 128, VT.float8e4m3, VT.float32, cc.Variant.opt, PLANAR, ROW, seed=5)
        float_case(1, 256, 192, 64, VT.float16, VT.float32, cc.Variant.basic, PLANAR, ROW, seed=6)


@pytest.mark.parametrize("B,M,N,K", [(2, 384, 640, 256), (3, 512, 4096, 576), (1, 1024, 1216, 2048)])
@pytest.mark.parametrize("alpha", [1, 0.75 - 1.25j])
def test_block_tile_choice_is_invisible(B, M, N, K, alpha):
    """The same bits whichever block tile computes them (same K order per element, and
    per K tile the same order of the four real products; the same expression for alpha)."""
    rng = np.random.default_rng(11)
    qa = quantize(rng.standard_normal((B, 2, M, K)).astype(np.float32), VT.float16).reshape(-1)
    qb = quantize(rng.standard_normal((B, 2, N, K)).astype(np.float32), VT.float16).reshape(-1)
    results = []
    for block_tile in (0, 1, 2, 3):
        with cc.option(cc.Option.gemm_block_tile, block_tile):
            results.append(run_gemm(qa, qb, B, M, N, K, VT.float16, VT.float32, cc.Variant.opt, alpha=alpha))
    for r in results[1:]:
        assert np.array_equal(results[0], r)


def _same_bits_either_block_tile(B, M, N, K, seed, c_order=ROW, alpha=1):
    rng = np.random.default_rng(seed)
    qa = quantize(rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32), VT.float16).reshape(-1)
    qb = quantize(rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32), VT.float16).reshape(-1)
    results = []
    for block_tile in (1, 3):
        with cc.option(cc.Option.gemm_block_tile, block_tile):
            results.append(run_gemm(qa, qb, B, M, N, K, VT.float16, VT.float32, cc.Variant.opt, PLANAR, c_order,
                                    alpha))
    assert np.array_equal(results[0], results[1]), (B, M, N, K, c_order)
    return qa, qb, results[1]


def test_wide_block_tilings_of_many_shapes():
    """The 192 x 256 kernel covers the width of C with full tiles and short ones, and a block
    takes its short tiles before or after its full ones: seeded random shapes (M, N multiples
    of 64; from a few tiles to several per block, widths with none, one, two and more short
    tiles per row of tiles) give the bits of the 256 x 128 kernel, which the other tests
    compare with the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(14):
        rows, cols = 64 * int(rng.integers(1, 13)), 64 * int(rng.integers(1, 40))
        B = int(rng.integers(1, 1 + max(1, 2400 // ((rows + 255) // 256 * ((cols + 191) // 192)))))
        K = int(rng.choice([64, 96, 160, 288]))
        c_order = ROW if case % 3 else COL
        M, N = (rows, cols) if c_order == ROW else (cols, rows)
        _same_bits_either_block_tile(B, M, N, K, 100 + case, c_order, alpha=1 if case % 4 else 0.5 - 2j)


def test_wide_block_more_than_64_tiles_with_short_ones():
    """More than 64 tiles per block, short tiles among them (448 = 192 + 2 x 128 columns): the
    coordinates past a block's table of 64, for tiles of both kinds."""
    B, M, N, K = 6000, 64, 448, 64
    qa, qb, got = _same_bits_either_block_tile(B, M, N, K, 13)
    want = orc.gemm(qa[-3 * 2 * M * K:], qb[-3 * 2 * N * K:], M, N, K, ORC_TYPE[VT.float16], ORC_TYPE[VT.float32])
    assert np.allclose(got[-3:], want.reshape(3, 2, M, N), rtol=1e-3, atol=1e-3)


def test_wide_block_more_than_64_tiles_per_block():
    """A block of the 192 x 256 kernel looks the coordinates of its first 64 C tiles up in a
    table and works out the others one by one: 20000 one-tile batches are more than 64 tiles
    for each of the 256 persistent blocks. Same bits as the 256 x 128 kernel."""
    rng = np.random.default_rng(12)
    B, M, N, K = 20000, 64, 64, 64
    qa = quantize(rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32), VT.float16).reshape(-1)
    qb = quantize(rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32), VT.float16).reshape(-1)
    results = []
    for block_tile in (1, 3):
        with cc.option(cc.Option.gemm_block_tile, block_tile):
            results.append(run_gemm(qa, qb, B, M, N, K, VT.float16, VT.float32, cc.Variant.opt))
    assert np.array_equal(results[0], results[1])
    want = orc.gemm(qa[:4 * 2 * M * K], qb[:4 * 2 * N * K], M, N, K, ORC_TYPE[VT.float16],
                    ORC_TYPE[VT.float32])
    assert np.allclose(results[1][:4], want.reshape(4, 2, M, N), rtol=1e-3, atol=1e-3)
