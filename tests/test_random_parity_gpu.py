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
