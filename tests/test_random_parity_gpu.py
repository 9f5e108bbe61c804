"""Seeded random sweep over dtype pairs, shapes (ragged and aligned), variants, C
layouts, alpha / beta and the three ways in (GEMM on prepared operands, pipeline with
planar input, pipeline with interleaved input), every case against the CPU oracle."""
import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import (ORC_TYPE, check_float, dequantize, quantize, stream, to_device, to_host,
                      transpose_operand)

pytestmark = pytest.mark.gpu
VT = cc.ValueType
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved
ROW, COL = cc.MemOrder.row_major, cc.MemOrder.col_major
PAIRS = [(VT.float16, VT.float32), (VT.float16, VT.float16), (VT.bfloat16, VT.float32),
         (VT.bfloat16, VT.bfloat16), (VT.float32, VT.float32), (VT.float32, VT.float16),
         (VT.float8e4m3, VT.float32), (VT.float8e5m2, VT.float32)]
MS = [1, 7, 16, 64, 100, 128, 129, 255, 256, 300, 512]
NS = [1, 5, 16, 64, 96, 128, 200, 256, 257, 384, 520]
KS = [1, 3, 8, 16, 31, 32, 33, 64, 65, 96, 100, 128, 200, 256, 577]


def interleave(q, B, rows, K):
    return np.ascontiguousarray(q.reshape(B, 2, rows, K).transpose(0, 2, 3, 1)).reshape(-1)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_cases(seed):
    rng = np.random.default_rng(seed)
    for case in range(40):
        tin, tout = PAIRS[rng.integers(len(PAIRS))]
        B = int(rng.integers(1, 5))
        M, N, K = int(rng.choice(MS)), int(rng.choice(NS)), int(rng.choice(KS))
        variant = cc.Variant.opt if rng.integers(2) else cc.Variant.basic
        c_order = ROW if rng.integers(2) else COL
        c_axis = INTERLEAVED if (variant == cc.Variant.opt and rng.integers(3) == 0) else PLANAR
        alpha = complex(1) if rng.integers(2) else complex(float(rng.integers(-2, 3)) + 0.5,
                                                            float(rng.integers(-2, 3)))
        beta = complex(0) if rng.integers(2) else complex(float(rng.integers(-2, 3)), 0.25)
        way = int(rng.integers(3))
        what = "seed %d case %d: %s->%s B=%d M=%d N=%d K=%d %s C %s %s alpha=%s beta=%s way %d" % (
            seed, case, tin.name, tout.name, B, M, N, K, variant.name,
            "row" if c_order == ROW else "col", "interleaved" if c_axis == INTERLEAVED else "planar",
            alpha, beta, way)
        print(what, flush=True)
        qa = quantize(rng.uniform(-1, 1, B * 2 * M * K), tin)
        qb = quantize(rng.uniform(-1, 1, B * 2 * N * K), tin)
        c32 = rng.uniform(-1, 1, B * 2 * M * N).astype(np.float32)
        c_in = c32 if tout == VT.float32 else quantize(c32, tout)
        d_c = to_device(c_in)
        if way == 0:
            gemm = cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(tin, tout), variant, c_axis, c_order,
                           ROW, COL, alpha, beta)
            if variant == cc.Variant.opt:
                d_a, d_b = transpose_operand(qa, B, M, K, tin), transpose_operand(qb, B, N, K, tin)
            else:
                d_a, d_b = to_device(qa), to_device(qb)
            gemm.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
        else:
            axis = INTERLEAVED if way == 2 else PLANAR
            pipe = cc.Pipeline(B, M, N, K, 0, stream(), axis, c_axis, ROW, COL, c_order, tin, tout,
                               variant, alpha, beta)
            d_a = to_device(interleave(qa, B, M, K) if way == 2 else qa)
            d_b = to_device(interleave(qb, B, N, K) if way == 2 else qb)
            pipe.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
        torch.cuda.synchronize()
        got = dequantize(to_host(d_c, c_in.dtype), tout)
        rows, cols = (M, N) if c_order == ROW else (N, M)
        # an interleaved C buffer is [B][rows][cols][2]; the oracle works on planar ones
        c_planar = (np.ascontiguousarray(c_in.reshape(B, rows, cols, 2).transpose(0, 3, 1, 2)).reshape(-1)
                    if c_axis == INTERLEAVED else c_in)
        want = orc.gemm(qa, qb, M, N, K, ORC_TYPE[tin], ORC_TYPE[tout], int(c_order), alpha, beta, c_planar)
        w64 = orc.gemm_float64(qa, qb, M, N, K, ORC_TYPE[tin], int(c_order))
        ci = dequantize(c_planar, tout).reshape(w64.shape).astype(np.float64)
        w = (w64[:, 0] + 1j * w64[:, 1]) * alpha + beta * (ci[:, 0] + 1j * ci[:, 1])
        w64 = np.stack([w.real, w.imag], 1)
        if c_axis == INTERLEAVED:
            got = got.reshape(B, rows, cols, 2).transpose(0, 3, 1, 2)
        check_float(got.reshape(w64.shape), dequantize(want, tout).reshape(w64.shape), w64, tin, tout)


def _pack_rows(bits, B, rows, K):
    """One byte per sample [B][2][rows][K] -> rows of whole 32-bit words, LSB first."""
    kw = (K + 31) // 32
    padded = np.zeros((B * 2 * rows, kw * 32), dtype=np.uint8)
    padded[:, :K] = bits.reshape(B * 2 * rows, K)
    return np.packbits(padded, axis=1, bitorder="little").view(np.uint32).reshape(-1)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_int1_cases(seed):
    """1-bit GEMM and pipeline, bit-exact: both variants, ragged shapes, integer alpha / beta,
    and the option that selects the popcount kernel."""
    rng = np.random.default_rng(seed)
    for case in range(40):
        B = int(rng.integers(1, 6))
        M = int(rng.choice([1, 16, 64, 100, 128, 130, 256, 300]))
        N = int(rng.choice([1, 8, 64, 70, 128, 200, 256, 384]))
        way = int(rng.integers(4))   # GEMM basic, GEMM opt, pipeline opt, pipeline basic
        K = (int(rng.choice([32, 64, 96, 512, 992, 1024, 2048, 4096])) if way in (1, 2)
             else int(rng.choice([1, 31, 32, 33, 100, 512, 1000, 2048, 4097])))
        if way == 3 and K % 32:
            K = 32 * (K // 32 + 1)   # the pipeline's flat packing needs rows of whole words
        c_order = ROW if rng.integers(2) else COL
        alpha = complex(int(rng.integers(-3, 4)), int(rng.integers(-3, 4)))
        beta = complex(int(rng.integers(-2, 3)), int(rng.integers(-2, 3))) if rng.integers(2) else 0j
        switch = int(rng.integers(3))   # 1: the vector-ALU kernel; else the default (MFMA)
        with cc.option(cc.Option.int1_popcount, 1 if switch == 1 else 0):
            print("seed %d case %d: B=%d M=%d N=%d K=%d way %d C %s alpha=%s beta=%s switch %d" % (
                seed, case, B, M, N, K, way, "row" if c_order == ROW else "col", alpha, beta, switch),
                flush=True)
            a_bits = rng.integers(0, 2, B * 2 * M * K, dtype=np.uint8)
            b_bits = rng.integers(0, 2, B * 2 * N * K, dtype=np.uint8)
            c_in = rng.integers(-1000, 1000, B * 2 * M * N).astype(np.int32)
            pa, pb = _pack_rows(a_bits, B, M, K), _pack_rows(b_bits, B, N, K)
            want = orc.gemm(pa, pb, M, N, K, orc.INT1, orc.INT32, int(c_order), alpha, beta, c_in)
            d_c = to_device(c_in)
            if way in (0, 1):
                variant = cc.Variant.opt if way == 1 else cc.Variant.basic
                gemm = cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(VT.int1, VT.int32), variant, PLANAR,
                               c_order, ROW, COL, alpha, beta)
                if way == 1:
                    d_a, d_b = transpose_operand(pa, B, M, K, VT.int1), transpose_operand(pb, B, N, K, VT.int1)
                else:
                    d_a, d_b = to_device(pa), to_device(pb)
                gemm.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
            else:
                variant = cc.Variant.opt if way == 2 else cc.Variant.basic
                pipe = cc.Pipeline(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, c_order, VT.int1,
                                   VT.int32, variant, alpha, beta)
                d_a, d_b = to_device(a_bits), to_device(b_bits)
                pipe.Run(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
            torch.cuda.synchronize()
            assert np.array_equal(to_host(d_c, np.int32).reshape(want.shape), want)
