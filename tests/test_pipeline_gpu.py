"""GPU parity tests of the pipeline wrapper (pack -> transpose -> GEMM) against the
CPU oracle; cases follow the reference's test/pipeline/pipeline.cpp."""

import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import ORC_TYPE, check_float, dequantize, quantize, stream, to_device, to_host

pytestmark = pytest.mark.gpu
VT = cc.ValueType
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved
ROW, COL = cc.MemOrder.row_major, cc.MemOrder.col_major


@pytest.mark.parametrize("variant", [cc.Variant.opt, cc.Variant.basic])
@pytest.mark.parametrize("host", [False, True])
def test_pipeline_float16(variant, host):
    # test/pipeline/pipeline.cpp:17-86
    B, M, N, K = 2, 300, 200, 100
    alpha, beta = 1.5 - 1.5j, 0.5 - 0.5j
    rng = np.random.default_rng(0)
    qa = quantize(rng.uniform(-10, 10, B * 2 * M * K), VT.float16)
    qb = quantize(rng.uniform(-10, 10, B * 2 * N * K), VT.float16)
    c_in = rng.uniform(-10, 10, B * 2 * M * N).astype(np.float32)
    p = cc.Pipeline(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW, VT.float16, VT.float32,
                    variant, alpha, beta)
    if host:
        got = c_in.copy()
        p.RunHost(qa.ctypes.data, qb.ctypes.data, got.ctypes.data)
    else:
        d_a, d_b, d_c = to_device(qa), to_device(qb), to_device(c_in)
        p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
        torch.cuda.synchronize()
        got = to_host(d_c, np.float32)
    want = orc.gemm(qa, qb, M, N, K, orc.FLOAT16, orc.FLOAT32, orc.ROW_MAJOR, alpha, beta, c_in)
    w64 = orc.gemm_float64(qa, qb, M, N, K, orc.FLOAT16)
    w = (w64[:, 0] + 1j * w64[:, 1]) * alpha + beta * (c_in.reshape(B, 2, M, N)[:, 0].astype(np.float64)
                                                       + 1j * c_in.reshape(B, 2, M, N)[:, 1])
    check_float(got.reshape(want.shape), want, np.stack([w.real, w.imag], 1), VT.float16, VT.float32)


def test_pipeline_interleaved_in_and_out():
    B, M, N, K = 3, 130, 70, 96
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32)
    qa, qb = quantize(a, VT.bfloat16), quantize(b, VT.bfloat16)
    qa_il = np.ascontiguousarray(qa.transpose(0, 2, 3, 1))
    qb_il = np.ascontiguousarray(qb.transpose(0, 2, 3, 1))
    p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, INTERLEAVED, ROW, COL, COL, VT.bfloat16,
                    VT.float32, cc.Variant.opt)
    d_a, d_b = to_device(qa_il.reshape(-1)), to_device(qb_il.reshape(-1))
    d_c = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32))
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_c, np.float32).reshape(B, N, M, 2).transpose(0, 3, 1, 2)
    want = orc.gemm(qa.reshape(-1), qb.reshape(-1), M, N, K, orc.BFLOAT16, orc.FLOAT32, orc.COL_MAJOR)
    w64 = orc.gemm_float64(qa.reshape(-1), qb.reshape(-1), M, N, K, orc.BFLOAT16, orc.COL_MAJOR)
    check_float(got, want, w64, VT.bfloat16, VT.float32)


def test_pipeline_fp32_interleaved_in():
    # 32-bit interleaved input is not consumed directly: it goes through the transposes
    B, M, N, K = 2, 130, 70, 50
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32)
    a_il = np.ascontiguousarray(a.transpose(0, 2, 3, 1))
    b_il = np.ascontiguousarray(b.transpose(0, 2, 3, 1))
    p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, ROW, VT.float32,
                    VT.float16, cc.Variant.opt)
    d_a, d_b = to_device(a_il.reshape(-1)), to_device(b_il.reshape(-1))
    d_c = to_device(np.full(B * 2 * M * N, 0x7fc0, dtype=np.uint16))
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = dequantize(to_host(d_c, np.uint16), VT.float16).reshape(B, 2, M, N)
    want = orc.gemm(a.reshape(-1), b.reshape(-1), M, N, K, orc.FLOAT32, orc.FLOAT16)
    w64 = orc.gemm_float64(a.reshape(-1), b.reshape(-1), M, N, K, orc.FLOAT32)
    check_float(got, dequantize(want, VT.float16), w64, VT.float32, VT.float16)


@pytest.mark.parametrize("variant", [cc.Variant.opt, cc.Variant.basic])
def test_pipeline_int1(variant):
    # test/pipeline/pipeline.cpp:88-187: one byte per sample in, packed inside
    B, M, N, K = 2, 512, 512, 512
    alpha, beta = 2 + 3j, 1 - 3j
    rng = np.random.default_rng(2)
    a_bits = rng.integers(0, 2, B * 2 * M * K, dtype=np.uint8)
    b_bits = rng.integers(0, 2, B * 2 * N * K, dtype=np.uint8)
    c_in = rng.integers(-2 ** 31, 2 ** 31, B * 2 * M * N).astype(np.int32)
    p = cc.Pipeline(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW, VT.int1, VT.int32,
                    variant, alpha, beta)
    d_a, d_b, d_c = to_device(a_bits), to_device(b_bits), to_device(c_in)
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    want = orc.gemm(orc.pack_bits(a_bits), orc.pack_bits(b_bits), M, N, K, orc.INT1, orc.INT32,
                    orc.ROW_MAJOR, alpha, beta, c_in)
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)


@pytest.mark.parametrize("mode", ["direct", "popcount"])
@pytest.mark.parametrize("M,N,K,c_order", [(130, 70, 992, ROW), (64, 200, 96, COL), (20, 30, 32, ROW),
                                           (256, 128, 2048, COL)])
def test_pipeline_int1_shapes(mode, M, N, K, c_order):
    # Planar one-byte-per-sample input is packed straight into the tiled 1-bit layout
    # in the GEMM's workspace ("direct"); with the vector-ALU kernel selected the
    # pipeline packs and transposes as the reference does. Any non-zero byte is a 1 bit.
    if mode == "popcount":
        cc.set_option(cc.Option.int1_popcount, 1)
    B = 3
    rng = np.random.default_rng(M + K)
    a_bits = rng.integers(0, 2, B * 2 * M * K, dtype=np.uint8)
    b_bits = rng.integers(0, 2, B * 2 * N * K, dtype=np.uint8)
    # other non-zero values count as 1 too
    a_in = a_bits * rng.integers(1, 256, a_bits.size, dtype=np.uint8)
    b_in = b_bits * rng.integers(1, 256, b_bits.size, dtype=np.uint8)
    alpha, beta = -1 + 2j, 3 + 1j
    c_in = rng.integers(-1000, 1000, B * 2 * M * N).astype(np.int32)
    p = cc.Pipeline(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, c_order, VT.int1, VT.int32,
                    cc.Variant.opt, alpha, beta)
    d_a, d_b, d_c = to_device(a_in), to_device(b_in), to_device(c_in)
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())     # beta != 0: applied twice
    torch.cuda.synchronize()
    pa, pb = pack_rows(a_bits, B, M, K), pack_rows(b_bits, B, N, K)
    once = orc.gemm(pa, pb, M, N, K, orc.INT1, orc.INT32, int(c_order), alpha, beta, c_in)
    want = orc.gemm(pa, pb, M, N, K, orc.INT1, orc.INT32, int(c_order), alpha, beta, once.reshape(-1))
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)


@pytest.mark.parametrize("mode", ["direct", "popcount"])
def test_pipeline_int1_unaligned_input(mode):
    # input buffers that start at an odd address: the kernels that read the bytes 16 at a
    # time use unaligned loads or fall back to byte loads
    if mode == "popcount":
        cc.set_option(cc.Option.int1_popcount, 1)
    B, M, N, K = 2, 150, 140, 1056
    rng = np.random.default_rng(5)
    a_bits = rng.integers(0, 2, B * 2 * M * K, dtype=np.uint8)
    b_bits = rng.integers(0, 2, B * 2 * N * K, dtype=np.uint8)
    d_a = to_device(np.concatenate([np.zeros(1, np.uint8), a_bits * 7]))
    d_b = to_device(np.concatenate([np.zeros(3, np.uint8), b_bits * 255]))
    d_c = to_device(np.zeros(B * 2 * M * N, dtype=np.int32))
    p = cc.Pipeline(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW, VT.int1, VT.int32,
                    cc.Variant.opt)
    p.Run(d_a.data_ptr() + 1, d_b.data_ptr() + 3, d_c.data_ptr())
    torch.cuda.synchronize()
    want = orc.gemm(pack_rows(a_bits, B, M, K), pack_rows(b_bits, B, N, K), M, N, K, orc.INT1, orc.INT32)
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)


def pack_rows(bits, B, rows, K):
    """One byte per sample [B][2][rows][K] -> rows of whole 32-bit words, LSB first."""
    kw = (K + 31) // 32
    padded = np.zeros((B * 2 * rows, kw * 32), dtype=np.uint8)
    padded[:, :K] = bits.reshape(B * 2 * rows, K)
    return np.packbits(padded, axis=1, bitorder="little").view(np.uint32).reshape(-1)


def interleaved(q, B, rows, K):
    return np.ascontiguousarray(q.reshape(B, 2, rows, K).transpose(0, 2, 3, 1)).reshape(-1)


def _host_buffer(a, pinned):
    """A host copy of `a` as a torch tensor (page-locked if asked) and its numpy view."""
    t = torch.empty(a.nbytes, dtype=torch.uint8, pin_memory=pinned)
    v = t.numpy().view(a.dtype)
    v[:] = a.reshape(-1)
    return t, v


@pytest.mark.parametrize("pinned", [False, True])
@pytest.mark.parametrize("B,M,N,K,axis,beta,chunk_bytes", [
    (6, 256, 1024, 128, PLANAR, 0.5 - 0.25j, None),      # default size: 2 chunks of 3 batches
    (8, 256, 512, 256, INTERLEAVED, 0, 1 << 20),         # 8 chunks of 1: every lane used again
    (7, 200, 1000, 104, INTERLEAVED, 0, 5 << 20)])       # 2.1 MB a batch: chunks of 2, 2, 2 and 1
def test_pipeline_host_run_in_chunks(pinned, B, M, N, K, axis, beta, chunk_bytes):
    """Host-pointer Run of a problem that takes the batch-chunked path over several
    streams: equal, bit for bit, to the device Run of the same object, and within the
    float bounds of the oracle."""
    if chunk_bytes:
        cc.set_option(cc.Option.host_chunk_bytes, chunk_bytes)
    alpha = 1.0 if beta == 0 else 2 - 1j
    rng = np.random.default_rng(11)
    qa = quantize(rng.uniform(-2, 2, B * 2 * M * K), VT.float16)
    qb = quantize(rng.uniform(-2, 2, B * 2 * N * K), VT.float16)
    c_in = rng.uniform(-10, 10, B * 2 * M * N).astype(np.float32)
    a_in = interleaved(qa, B, M, K) if axis == INTERLEAVED else qa
    b_in = interleaved(qb, B, N, K) if axis == INTERLEAVED else qb
    p = cc.Pipeline(B, M, N, K, 0, stream(), axis, PLANAR, ROW, COL, ROW, VT.float16, VT.float32,
                    cc.Variant.opt, alpha, beta)
    d_a, d_b, d_c = to_device(a_in), to_device(b_in), to_device(c_in)
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    from_device = to_host(d_c, np.float32)
    for _ in range(2):   # the second call re-uses the lanes
        ta, ha = _host_buffer(a_in, pinned)
        tb, hb = _host_buffer(b_in, pinned)
        tc, hc = _host_buffer(c_in, pinned)
        p.RunHost(ha.ctypes.data, hb.ctypes.data, hc.ctypes.data)
        assert np.array_equal(hc, from_device)
    want = orc.gemm(qa, qb, M, N, K, orc.FLOAT16, orc.FLOAT32, orc.ROW_MAJOR, alpha, beta, c_in)
    w64 = orc.gemm_float64(qa, qb, M, N, K, orc.FLOAT16)
    c4 = c_in.reshape(B, 2, M, N).astype(np.float64)
    w = (w64[:, 0] + 1j * w64[:, 1]) * alpha + beta * (c4[:, 0] + 1j * c4[:, 1])
    check_float(hc.reshape(want.shape), want, np.stack([w.real, w.imag], 1), VT.float16, VT.float32)


def pack_per_batch(bits, B, axis):
    """The oracle's packing of one-byte-per-sample input, batch by batch: for interleaved
    input ([rows][K][2] per batch) all real bits of a batch, then all its imaginary bits
    (kernels/packing_kernel.cu:15-22 applied to one batch), which is the planar layout
    [B][2][rows][K / 32] that the 1-bit GEMM reads."""
    per = bits.reshape(B, -1)
    return np.concatenate([orc.pack_bits(np.ascontiguousarray(x), int(axis)) for x in per])


@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
def test_pipeline_int1_host_run(axis):
    """1-bit host Run through the chunked path (2 chunks of 2 batches: 13 MiB in all), planar
    and interleaved input: the oracle's integers, from the device Run and from the host Run."""
    B, M, N, K = 4, 128, 256, 4096
    rng = np.random.default_rng(12)
    a_bits = rng.integers(0, 2, B * 2 * M * K, dtype=np.uint8)
    b_bits = rng.integers(0, 2, B * 2 * N * K, dtype=np.uint8)
    c = rng.integers(-1000, 1000, B * 2 * M * N).astype(np.int32)
    p = cc.Pipeline(B, M, N, K, 0, stream(), axis, PLANAR, ROW, COL, ROW, VT.int1, VT.int32,
                    cc.Variant.opt, 1.0, 1.0)
    d_a, d_b, d_c = to_device(a_bits), to_device(b_bits), to_device(c)
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = c.copy()
    p.RunHost(a_bits.ctypes.data, b_bits.ctypes.data, got.ctypes.data)
    want = orc.gemm(pack_per_batch(a_bits, B, axis), pack_per_batch(b_bits, B, axis), M, N, K,
                    orc.INT1, orc.INT32, orc.ROW_MAJOR, 1.0, 1.0, c)
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)
    assert np.array_equal(got.reshape(want.shape), want)


@pytest.mark.parametrize("kernel", ["mfma", "popcount"])
@pytest.mark.parametrize("variant", [cc.Variant.opt, cc.Variant.basic])
@pytest.mark.parametrize("B,M,N,K,c_order", [(1, 64, 48, 256, ROW), (1, 130, 70, 992, COL),
                                             (3, 64, 200, 96, ROW), (5, 20, 30, 1024, COL)])
def test_pipeline_int1_interleaved_input(kernel, variant, B, M, N, K, c_order):
    """1-bit pipeline with interleaved input (one byte per sample, [B][rows][K][2]): for one
    batch the reference's flat packing (kernels/packing_kernel.cu:15-22) is the planar
    layout; for several batches every batch is packed on its own. Device Run and host Run
    against the oracle's GEMM of the oracle's packing, bit for bit; any non-zero byte is a 1."""
    if kernel == "popcount":
        cc.set_option(cc.Option.int1_popcount, 1)
    rng = np.random.default_rng(B * 1000 + K)
    a_bits = rng.integers(0, 2, B * M * K * 2, dtype=np.uint8)
    b_bits = rng.integers(0, 2, B * N * K * 2, dtype=np.uint8)
    a_in = a_bits * rng.integers(1, 256, a_bits.size, dtype=np.uint8)
    b_in = b_bits * rng.integers(1, 256, b_bits.size, dtype=np.uint8)
    alpha, beta = 2 - 1j, -1 + 1j
    c_in = rng.integers(-1000, 1000, B * 2 * M * N).astype(np.int32)
    want = orc.gemm(pack_per_batch(a_bits, B, INTERLEAVED), pack_per_batch(b_bits, B, INTERLEAVED),
                    M, N, K, orc.INT1, orc.INT32, int(c_order), alpha, beta, c_in)
    p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, c_order, VT.int1,
                    VT.int32, variant, alpha, beta)
    d_a, d_b, d_c = to_device(a_in), to_device(b_in), to_device(c_in)
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)
    got = c_in.copy()
    p.RunHost(a_in.ctypes.data, b_in.ctypes.data, got.ctypes.data)
    assert np.array_equal(got.reshape(want.shape), want)


def test_pipeline_int1_interleaved_input_unaligned():
    # interleaved bytes at an odd address: the packing kernel's wide loads take any address
    B, M, N, K = 2, 96, 64, 512
    rng = np.random.default_rng(8)
    a_bits = rng.integers(0, 2, B * M * K * 2, dtype=np.uint8)
    b_bits = rng.integers(0, 2, B * N * K * 2, dtype=np.uint8)
    want = orc.gemm(pack_per_batch(a_bits, B, INTERLEAVED), pack_per_batch(b_bits, B, INTERLEAVED),
                    M, N, K, orc.INT1, orc.INT32, c_in=np.zeros(B * 2 * M * N, np.int32))
    d_a = to_device(np.concatenate([np.zeros(1, np.uint8), a_bits]))
    d_b = to_device(np.concatenate([np.zeros(5, np.uint8), b_bits]))
    d_c = to_device(np.zeros(B * 2 * M * N, np.int32))
    p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, ROW, VT.int1, VT.int32,
                    cc.Variant.opt)
    p.Run(d_a.data_ptr() + 1, d_b.data_ptr() + 5, d_c.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)


@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float32), (VT.float16, VT.float16),
                                      (VT.bfloat16, VT.float32), (VT.float8e4m3, VT.float32),
                                      (VT.float8e5m2, VT.float32)])
@pytest.mark.parametrize("K", [4, 100, 576, 102, 33])
@pytest.mark.parametrize("variant", [cc.Variant.opt, cc.Variant.basic])
def test_pipeline_interleaved_input(tin, tout, K, variant):
    # Interleaved input whose rows are whole 16-byte chunks is consumed by the GEMM
    # directly (no transposes); other K take the transpose route (either variant) - both
    # must give the oracle's numbers. K = 102 / 33: not whole chunks.
    B, M, N = 3, 200, 150
    rng = np.random.default_rng(K)
    qa = quantize(rng.uniform(-1, 1, B * 2 * M * K), tin)
    qb = quantize(rng.uniform(-1, 1, B * 2 * N * K), tin)
    alpha, beta = 0.75 - 0.5j, -0.25 + 1j
    c32 = rng.uniform(-1, 1, B * 2 * M * N).astype(np.float32)
    c_in = c32 if tout == VT.float32 else quantize(c32, tout)
    p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, ROW, tin, tout,
                    variant, alpha, beta)
    d_a, d_b, d_c = to_device(interleaved(qa, B, M, K)), to_device(interleaved(qb, B, N, K)), to_device(c_in)
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    from gpu_util import dequantize
    got = dequantize(to_host(d_c, c_in.dtype), tout).reshape(B, 2, M, N)
    want = orc.gemm(qa, qb, M, N, K, ORC_TYPE[tin], ORC_TYPE[tout], orc.ROW_MAJOR, alpha, beta, c_in)
    w64 = orc.gemm_float64(qa, qb, M, N, K, ORC_TYPE[tin])
    ci = dequantize(c_in, tout).reshape(B, 2, M, N).astype(np.float64)
    w = (w64[:, 0] + 1j * w64[:, 1]) * alpha + beta * (ci[:, 0] + 1j * ci[:, 1])
    check_float(got, dequantize(want, tout), np.stack([w.real, w.imag], 1), tin, tout)


@pytest.mark.parametrize("tin", [VT.float16, VT.float8e4m3])
@pytest.mark.parametrize("route", [1, 2])
def test_pipeline_interleaved_input_either_route(tin, route):
    # The opt pipeline reads interleaved rows in place or transposes them into tiles first,
    # whichever it expects to be faster (option PIPELINE_ROUTE forces one): same numbers.
    B, M, N, K = 1, 6144, 6144, 64
    rng = np.random.default_rng(31)
    qa = quantize(rng.uniform(-1, 1, B * 2 * M * K), tin)
    qb = quantize(rng.uniform(-1, 1, B * 2 * N * K), tin)
    with cc.option(cc.Option.pipeline_route, route):
        p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, ROW, tin, VT.float32,
                        cc.Variant.opt)
    assert p.ReadsInPlace() == (route == 1)
    d_a, d_b = to_device(interleaved(qa, B, M, K)), to_device(interleaved(qb, B, N, K))
    d_c = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32))
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_c, np.float32).reshape(B, 2, M, N)
    want = orc.gemm(qa, qb, M, N, K, ORC_TYPE[tin], orc.FLOAT32)
    check_float(got, want, orc.gemm_float64(qa, qb, M, N, K, ORC_TYPE[tin]), tin, VT.float32)


def _time_runs(pipe, a, b, c, budget_ms=30.0):
    cur = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        pipe.Run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    e0.record(cur)
    pipe.Run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    e1.record(cur)
    e1.synchronize()
    n = max(3, int(budget_ms / max(e0.elapsed_time(e1), 1e-3)))
    e0.record(cur)
    for _ in range(n):
        pipe.Run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    e1.record(cur)
    e1.synchronize()
    return e0.elapsed_time(e1) / n


@pytest.mark.parametrize("tin,tdt,axis", [(VT.float16, torch.float16, INTERLEAVED),
                                          (VT.float8e4m3, torch.float8_e4m3fn, INTERLEAVED),
                                          (VT.float16, torch.float16, PLANAR)])
def test_pipeline_takes_the_faster_route(tin, tdt, axis):
    """Either side of the break-even points in ccglib_pipeline_create (the sweep behind them:
    python -m ccglib_amd.tuning.pipeline_crossover): the route the default takes is timed
    against the other one (PIPELINE_ROUTE = 1 / 2, best of three alternations of about 30 ms
    each) and may be at most 5 % slower."""
    K = 1024
    gen = torch.Generator(device="cuda").manual_seed(9)
    taken = []
    for M, N in [(512, 4096), (2048, 2048), (3072, 3072), (5120, 5120), (8192, 8192), (12288, 12288)]:
        B = max(1, (1 << 27) // (M * N))
        il = axis == INTERLEAVED
        scale = 448.0 / 5.8 if tin == VT.float8e4m3 else 1.0
        a = (torch.randn((B, M, K, 2) if il else (B, 2, M, K), device="cuda", generator=gen) * scale).to(tdt)
        b = (torch.randn((B, N, K, 2) if il else (B, 2, N, K), device="cuda", generator=gen) * scale).to(tdt)
        c = torch.empty((B, 2, M, N), device="cuda")
        pipes = {}
        for route in (0, 1, 2):
            with cc.option(cc.Option.pipeline_route, route):
                pipes[route] = cc.Pipeline(B, M, N, K, 0, stream(), axis, PLANAR, ROW, COL, ROW, tin,
                                           VT.float32, cc.Variant.opt)
        assert pipes[1].ReadsInPlace() and not pipes[2].ReadsInPlace()
        best = {1: float("inf"), 2: float("inf")}
        for _ in range(3):
            for route in (1, 2):
                best[route] = min(best[route], _time_runs(pipes[route], a, b, c))
        chosen = 1 if pipes[0].ReadsInPlace() else 2
        taken.append(chosen)
        print("%s %s %dx%d: in place %.4f ms, transposed %.4f ms, default %s" % (
            tin.name, axis.name, M, N, best[1], best[2], "in place" if chosen == 1 else "transposed"), flush=True)
        assert best[chosen] <= 1.05 * best[3 - chosen], (M, N, best)
        del pipes, a, b, c
    assert taken[0] == 1 and taken[-1] == 2     # the sweep crosses the break-even point


def test_pipeline_basic_rejects_interleaved_output():
    with pytest.raises(RuntimeError, match="complex-interleaved output is not supported in basic variant"):
        cc.Pipeline(1, 16, 16, 16, 0, stream(), PLANAR, INTERLEAVED, ROW, COL, ROW, VT.float16,
                    VT.float32, cc.Variant.basic)


@pytest.mark.parametrize("block_tile", [1, 2])
@pytest.mark.parametrize("tin", [VT.float16, VT.float8e4m3])
def test_pipeline_interleaved_rows_read_in_place_with_either_block_tile(block_tile, tin):
    """8- and 16-bit interleaved input whose rows are whole 16-byte chunks is read by the
    GEMM in place; its kernel has the same two block tiles as the tiled one (option
    GEMM_BLOCK_TILE forces one)."""
    B, M, N, K = 3, 300, 260, 160
    rng = np.random.default_rng(7)
    qa = quantize(rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32), tin)
    qb = quantize(rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32), tin)
    qa_il = np.ascontiguousarray(qa.transpose(0, 2, 3, 1)).reshape(-1)
    qb_il = np.ascontiguousarray(qb.transpose(0, 2, 3, 1)).reshape(-1)
    with cc.option(cc.Option.gemm_block_tile, block_tile):
        p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, ROW, tin, VT.float32,
                        cc.Variant.opt, 0.5 + 1j)
    d_a, d_b = to_device(qa_il), to_device(qb_il)
    d_c = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32))
    p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_c, np.float32).reshape(B, 2, M, N)
    want = orc.gemm(qa.reshape(-1), qb.reshape(-1), M, N, K, ORC_TYPE[tin], orc.FLOAT32, orc.ROW_MAJOR,
                    0.5 + 1j)
    w64 = orc.gemm_float64(qa.reshape(-1), qb.reshape(-1), M, N, K, ORC_TYPE[tin])
    w = (w64[:, 0] + 1j * w64[:, 1]) * (0.5 + 1j)
    check_float(got, want, np.stack([w.real, w.imag], 1), tin, VT.float32)


@pytest.mark.parametrize("tin,K", [(VT.float16, 96), (VT.float8e5m2, 144), (VT.float32, 36)])
@pytest.mark.parametrize("skew", [0, 1])
def test_pipeline_planar_rows_read_in_place(tin, K, skew):
    """Planar input of the opt variant whose rows are whole 16-byte chunks is read by the
    GEMM in place when the two transposes would cost more than they save (small
    M N / (M + N)); the result has the bits of Transpose + opt GEMM on the same data.
    skew: buffers one element off a 16-byte boundary, for which the pipeline falls
    back to its transposes."""
    from gpu_util import transpose_operand
    B, M, N = 3, 200, 300
    tout = VT.float32
    rng = np.random.default_rng(K)
    qa = quantize(rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32), tin).reshape(-1)
    qb = quantize(rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32), tin).reshape(-1)
    pad = np.zeros(skew, dtype=qa.dtype)
    d_a, d_b = to_device(np.concatenate([pad, qa])), to_device(np.concatenate([pad, qb]))
    off = skew * qa.dtype.itemsize
    d_c = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32))
    p = cc.Pipeline(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW, tin, tout, cc.Variant.opt)
    p.Run(d_a.data_ptr() + off, d_b.data_ptr() + off, d_c.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_c, np.float32).reshape(B, 2, M, N)
    want = orc.gemm(qa, qb, M, N, K, ORC_TYPE[tin], orc.FLOAT32)
    check_float(got, want, orc.gemm_float64(qa, qb, M, N, K, ORC_TYPE[tin]), tin, tout)
    # the reference's sequence with separate objects
    t_a, t_b = transpose_operand(qa, B, M, K, tin), transpose_operand(qb, B, N, K, tin)
    d_c2 = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32))
    cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(tin, tout), cc.Variant.opt).Run(
        t_a.data_ptr(), t_b.data_ptr(), d_c2.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(got.reshape(-1), to_host(d_c2, np.float32))
    # and the host Run of the same object
    if skew == 0:
        host_c = np.full(B * 2 * M * N, np.nan, dtype=np.float32)
        p.RunHost(qa.ctypes.data, qb.ctypes.data, host_c.ctypes.data)
        assert np.array_equal(host_c, got.reshape(-1))


@pytest.mark.parametrize("tin,tout", [(VT.float16, VT.float32), (VT.float16, VT.float16),
                                      (VT.bfloat16, VT.float32), (VT.bfloat16, VT.bfloat16)])
@pytest.mark.parametrize("c_order", [ROW, COL])
def test_pipeline_interleaved_rows_wide_block(tin, tout, c_order):
    """GEMM_BLOCK_TILE = 3 for 16-bit interleaved rows read in place: the 192 x 256 block
    (planar C without beta, M and N multiples of 64, rows of whole 128-byte
    pieces, i.e. K a multiple of 32) against the oracle, and bit for bit against the
    256 x 128 block: tiles inside C and tiles of which only some 64-column groups or
    64-row pieces are, two to many K pieces, more C tiles than compute units."""
    for seed, (B, M, N, K, alpha) in enumerate([(2, 256, 192, 64, 1), (3, 320, 448, 96, 1),
                                                (2, 512, 832, 992, 1), (40, 256, 576, 64, 1),
                                                (1, 64, 64, 128, 1), (3, 320, 448, 96, 0.5 - 1.5j),
                                                (90, 256, 448, 96, 1), (90, 448, 256, 64, 1),
                                                (150, 256, 448, 64, 0.25 + 1j)]):
        rng = np.random.default_rng(40 + seed)
        qa = quantize(rng.uniform(-1, 1, (B, 2, M, K)).astype(np.float32), tin)
        qb = quantize(rng.uniform(-1, 1, (B, 2, N, K)).astype(np.float32), tin)
        d_a = to_device(np.ascontiguousarray(qa.transpose(0, 2, 3, 1)).reshape(-1))
        d_b = to_device(np.ascontiguousarray(qb.transpose(0, 2, 3, 1)).reshape(-1))
        out_np = np.float32 if tout == VT.float32 else np.uint16
        results = []
        for block_tile in (3, 1):
            with cc.option(cc.Option.gemm_block_tile, block_tile):
                p = cc.Pipeline(B, M, N, K, 0, stream(), INTERLEAVED, PLANAR, ROW, COL, c_order, tin, tout,
                                cc.Variant.opt, alpha)
            d_c = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32) if tout == VT.float32
                            else np.full(B * 2 * M * N, 0x7fc0, dtype=np.uint16))
            p.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
            torch.cuda.synchronize()
            results.append(to_host(d_c, out_np))
        want = orc.gemm(qa.reshape(-1), qb.reshape(-1), M, N, K, ORC_TYPE[tin], ORC_TYPE[tout], int(c_order),
                        alpha)
        w64 = orc.gemm_float64(qa.reshape(-1), qb.reshape(-1), M, N, K, ORC_TYPE[tin], int(c_order))
        w = (w64[:, 0] + 1j * w64[:, 1]) * complex(alpha)
        w64 = np.stack([w.real, w.imag], axis=1)
        check_float(dequantize(results[0], tout).reshape(want.shape), dequantize(want, tout), w64, tin, tout)
        assert np.array_equal(results[0], results[1]), (B, M, N, K)
