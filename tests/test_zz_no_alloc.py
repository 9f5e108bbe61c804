"""GPU test of ccglib_pipeline_run_static, the stateless pipeline call that allocates nothing
(its scratch is a static device array): its output against that of the pipeline object
(ccglib_pipeline_create + ccglib_pipeline_run) on the same buffers, two calls in a row, the
second with a smaller input, so that what the first call left in the array is still there.
Integer results bit for bit; float results bit for bit where the object takes the same route
(transposes, then the tiled kernel) and within the float bounds of the oracle elsewhere; every
float case is also compared with the oracle itself.
The device's free memory is read on either side of every stateless call and must not move,
and the call is captured into a HIP graph and replayed."""
import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import (ORC_TYPE, capture_and_replay, check_float, dequantize, quantize, stream,
                      to_device, to_host)

pytestmark = pytest.mark.gpu

VT = cc.ValueType
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved
ROW, COL = cc.MemOrder.row_major, cc.MemOrder.col_major
OUT_NP = {VT.float32: np.float32, VT.float16: np.uint16, VT.bfloat16: np.uint16, VT.int32: np.int32}


@pytest.fixture(autouse=True, scope="module")
def scratch_in_place():
    """The first call on a GPU is when the HIP runtime loads the code object that holds the
    static array, and the array comes to exist (its 32 MiB leave the device's free memory
    then, once). One small call up front, so that every call a test measures is a later one."""
    d = torch.zeros(2 * 2 * 32 * 32, dtype=torch.float32, device="cuda")
    cc.pipeline_run_static(1, 32, 32, 32, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW, VT.float16,
                           VT.float32, cc.Variant.opt, 1, 0, d.data_ptr(), d.data_ptr(), d.data_ptr())
    torch.cuda.synchronize()


def _inputs(B, M, N, K, tin, axis, seed):
    rng = np.random.default_rng(seed)
    if tin == VT.int1:
        a = rng.integers(0, 2, B * 2 * M * K, dtype=np.uint8) * rng.integers(1, 256, B * 2 * M * K, dtype=np.uint8)
        b = rng.integers(0, 2, B * 2 * N * K, dtype=np.uint8) * rng.integers(1, 256, B * 2 * N * K, dtype=np.uint8)
        return a, b, None, None      # one byte per sample, in the layout `axis` names
    qa = quantize(rng.uniform(-2, 2, (B, 2, M, K)), tin)
    qb = quantize(rng.uniform(-2, 2, (B, 2, N, K)), tin)
    pa, pb = qa.reshape(-1), qb.reshape(-1)      # planar, as the oracle takes them
    if axis == INTERLEAVED:
        qa = np.ascontiguousarray(qa.transpose(0, 2, 3, 1))
        qb = np.ascontiguousarray(qb.transpose(0, 2, 3, 1))
    return qa.reshape(-1), qb.reshape(-1), pa, pb


def _both(B, M, N, K, tin, tout, axis, c_axis, c_order, variant, alpha, beta, seed):
    """Runs the object and the stateless call on the same inputs; returns both outputs and,
    for float input, what the oracle says (its float result and the float64 product, both
    as planar float64 [B][2][rows][cols])."""
    a, b, pa, pb = _inputs(B, M, N, K, tin, axis, seed)
    rng = np.random.default_rng(seed + 1)
    n_out = B * 2 * M * N
    if tout == VT.int32:
        c_in = rng.integers(-1000, 1000, n_out).astype(np.int32)
    else:
        c_in = quantize(rng.uniform(-4, 4, n_out), tout)
    d_a, d_b = to_device(a), to_device(b)
    d_c1, d_c2 = to_device(c_in), to_device(c_in)
    pipe = cc.Pipeline(B, M, N, K, 0, stream(), axis, c_axis, ROW, COL, c_order, tin, tout, variant,
                       alpha, beta)
    pipe.Run(d_a.data_ptr(), d_b.data_ptr(), d_c1.data_ptr())
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]      # hipMemGetInfo: the device's, not torch's pool
    cc.pipeline_run_static(B, M, N, K, 0, stream(), axis, c_axis, ROW, COL, c_order, tin, tout,
                           variant, alpha, beta, d_a.data_ptr(), d_b.data_ptr(), d_c2.data_ptr())
    free_enqueued = torch.cuda.mem_get_info()[0]
    torch.cuda.synchronize()
    assert free_enqueued == free_before and torch.cuda.mem_get_info()[0] == free_before
    oracle = None
    if pa is not None:
        order = int(c_order)
        rows, cols = (M, N) if c_order == ROW else (N, M)
        c_planar = c_in
        if c_axis == INTERLEAVED:
            c_planar = np.ascontiguousarray(c_in.reshape(B, rows, cols, 2).transpose(0, 3, 1, 2)).reshape(-1)
        want = orc.gemm(pa, pb, M, N, K, ORC_TYPE[tin], ORC_TYPE[tout], order, alpha, beta,
                        c_planar if complex(beta) != 0 else None)
        w64 = orc.gemm_float64(pa, pb, M, N, K, ORC_TYPE[tin], order)
        w = (w64[:, 0] + 1j * w64[:, 1]) * complex(alpha)
        if complex(beta) != 0:
            ci = dequantize(c_planar, tout).reshape(w64.shape).astype(np.float64)
            w = w + complex(beta) * (ci[:, 0] + 1j * ci[:, 1])
        oracle = (dequantize(want, tout).astype(np.float64), np.stack([w.real, w.imag], axis=1))
    return to_host(d_c1, OUT_NP[tout]), to_host(d_c2, OUT_NP[tout]), oracle


# (first call, second and smaller call) per case
CASES = [
    # planar fp16, opt: the object transposes too -> identical bits
    dict(tin=VT.float16, tout=VT.float32, axis=PLANAR, c_axis=PLANAR, c_order=ROW, variant=cc.Variant.opt,
         alpha=1, beta=0, shapes=[(3, 300, 200, 100), (2, 130, 70, 40)], exact=True),
    # interleaved fp16 (the object reads the rows in place: other rounding order), alpha and beta
    dict(tin=VT.float16, tout=VT.float32, axis=INTERLEAVED, c_axis=INTERLEAVED, c_order=COL,
         variant=cc.Variant.opt, alpha=1.5 - 1.5j, beta=0.5 - 0.5j,
         shapes=[(2, 300, 200, 104), (1, 100, 60, 40)], exact=False),
    # fp8, basic variant (the object reads planar rows in place: same arithmetic, same bits)
    dict(tin=VT.float8e4m3, tout=VT.float32, axis=PLANAR, c_axis=PLANAR, c_order=ROW,
         variant=cc.Variant.basic, alpha=1, beta=0, shapes=[(2, 256, 128, 192), (1, 70, 50, 65)], exact=False),
    # bf16 -> bf16
    dict(tin=VT.bfloat16, tout=VT.bfloat16, axis=PLANAR, c_axis=PLANAR, c_order=COL, variant=cc.Variant.opt,
         alpha=1, beta=0, shapes=[(2, 257, 129, 72), (2, 64, 64, 32)], exact=True),
    # 1-bit, planar bytes and interleaved bytes (several batches)
    dict(tin=VT.int1, tout=VT.int32, axis=PLANAR, c_axis=PLANAR, c_order=ROW, variant=cc.Variant.opt,
         alpha=2 - 1j, beta=1 + 1j, shapes=[(3, 130, 70, 992), (2, 64, 48, 256)], exact=True),
    dict(tin=VT.int1, tout=VT.int32, axis=INTERLEAVED, c_axis=PLANAR, c_order=COL, variant=cc.Variant.opt,
         alpha=1, beta=0, shapes=[(3, 64, 200, 1024), (2, 20, 30, 96)], exact=True),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s-%s-%s" % (c["tin"].name, c["axis"].name, c["variant"].name))
def test_static_pipeline_matches_pipeline_object(case):
    for n, (B, M, N, K) in enumerate(case["shapes"]):
        print("static pipeline call %d: B=%d M=%d N=%d K=%d %s" % (n, B, M, N, K, case["tin"].name), flush=True)
        tin, tout = case["tin"], case["tout"]
        obj, static, oracle = _both(B, M, N, K, tin, tout, case["axis"], case["c_axis"], case["c_order"],
                                    case["variant"], case["alpha"], case["beta"], seed=17 + n)
        if case["exact"]:
            assert np.array_equal(obj, static)
        else:
            # same bounds as the library's other float paths, the object's output standing in
            # for the oracle's float product and float64 product
            o = dequantize(obj, tout).astype(np.float64)
            check_float(dequantize(static, tout), o, o, tin, tout)
        if oracle is not None:
            # and against the oracle itself (planar view of what the call wrote)
            rows, cols = (M, N) if case["c_order"] == ROW else (N, M)
            got = dequantize(static, tout)
            got = (got.reshape(B, rows, cols, 2).transpose(0, 3, 1, 2) if case["c_axis"] == INTERLEAVED
                   else got.reshape(B, 2, rows, cols))
            check_float(np.ascontiguousarray(got), oracle[0], oracle[1], tin, tout)


def test_static_pipeline_against_oracle():
    # and once against the oracle itself, so that the two entry points cannot be wrong together
    B, M, N, K = 2, 96, 200, 72
    rng = np.random.default_rng(3)
    qa = quantize(rng.standard_normal((B, 2, M, K)), VT.float16).reshape(-1)
    qb = quantize(rng.standard_normal((B, 2, N, K)), VT.float16).reshape(-1)
    d_a, d_b = to_device(qa), to_device(qb)
    d_c = to_device(np.full(B * 2 * M * N, np.nan, dtype=np.float32))
    cc.pipeline_run_static(B, M, N, K, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW, VT.float16,
                           VT.float32, cc.Variant.opt, 1, 0, d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    want = orc.gemm(qa, qb, M, N, K, orc.FLOAT16)
    w64 = orc.gemm_float64(qa, qb, M, N, K, orc.FLOAT16)
    check_float(to_host(d_c, np.float32).reshape(want.shape), want, w64, VT.float16, VT.float32)


class _StaticCall:
    """pipeline_run_static behind the Run(a, b, c) of an object, for capture_and_replay."""

    def __init__(self, stream_handle, *dims_and_layout):
        self.stream, self.args = stream_handle, dims_and_layout

    def Run(self, d_a, d_b, d_c):
        B, M, N, K, axis, c_axis, tin, tout = self.args
        cc.pipeline_run_static(B, M, N, K, 0, self.stream, axis, c_axis, ROW, COL, ROW, tin, tout,
                               cc.Variant.opt, 1, 0, d_a, d_b, d_c)


@pytest.mark.parametrize("tin,tout,axis", [(VT.float16, VT.float32, INTERLEAVED),
                                           (VT.int1, VT.int32, PLANAR)])
def test_static_pipeline_in_a_graph(tin, tout, axis):
    """The callers this entry point is for: captured once, replayed on changed input, every
    replay equal to the eager call."""
    B, M, N, K = 3, 200, 330, 96
    int1 = tin == VT.int1
    a = torch.zeros(B * 2 * M * K, dtype=torch.uint8 if int1 else torch.float16, device="cuda")
    b = torch.zeros(B * 2 * N * K, dtype=torch.uint8 if int1 else torch.float16, device="cuda")

    def fill(r):
        g = torch.Generator(device="cuda").manual_seed(300 + r)
        for t in (a, b):
            if int1:
                t.copy_(torch.randint(0, 2, t.shape, generator=g, device="cuda", dtype=torch.uint8))
            else:
                t.copy_(torch.randn(t.shape, generator=g, device="cuda").to(torch.float16))

    capture_and_replay(lambda s: _StaticCall(s, B, M, N, K, axis, PLANAR, tin, tout), [a, b], fill,
                       (B * 2 * M * N,), torch.int32 if int1 else torch.float32)


def test_static_pipeline_rejects_what_does_not_fit():
    assert cc.static_scratch_bytes() == 32 << 20    # the default build
    # 2 x (2 x 4096 x 4096 x 2 bytes) of tiles = 128 MiB > the 32 MiB array: refused, nothing runs
    d = to_device(np.zeros(16, np.uint8))
    with pytest.raises(RuntimeError, match="static scratch"):
        cc.pipeline_run_static(1, 4096, 4096, 4096, 0, stream(), PLANAR, PLANAR, ROW, COL, ROW,
                               VT.float16, VT.float32, cc.Variant.opt, 1, 0, d.data_ptr(),
                               d.data_ptr(), d.data_ptr())
    with pytest.raises(RuntimeError, match="not supported in basic variant"):
        cc.pipeline_run_static(1, 64, 64, 64, 0, stream(), PLANAR, INTERLEAVED, ROW, COL, ROW,
                               VT.float16, VT.float32, cc.Variant.basic, 1, 0, d.data_ptr(),
                               d.data_ptr(), d.data_ptr())
