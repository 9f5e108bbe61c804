"""Run() only enqueues work on the stream the object was created with and allocates
nothing, so it can be captured into a HIP graph: the graph is replayed several times
on changed input, with eager work and synchronisations in between, and every replay
is compared with the eager result."""
import numpy as np
import pytest
import torch

import ccglib_amd as cc
from gpu_util import capture_and_replay, quantize, to_device, transpose_operand

pytestmark = pytest.mark.gpu
VT = cc.ValueType
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved
ROW, COL = cc.MemOrder.row_major, cc.MemOrder.col_major


def test_graph_gemm_fp16_opt():
    B, M, N, K = 4, 256, 384, 128
    a = transpose_operand(quantize(np.zeros(B * 2 * M * K), VT.float16), B, M, K, VT.float16)
    b = transpose_operand(quantize(np.zeros(B * 2 * N * K), VT.float16), B, N, K, VT.float16)

    def fill(r):
        g = torch.Generator(device="cuda").manual_seed(100 + r)
        for t in (a, b):   # any bit pattern of small fp16 numbers, tile padding included
            t.copy_(torch.randint(0, 64, t.shape, generator=g, device="cuda", dtype=torch.uint8))

    capture_and_replay(lambda s: cc.GEMM(B, M, N, K, 0, s, cc.Precision(VT.float16, VT.float32),
                                          cc.Variant.opt),
                        [a, b], fill, (B * 2 * M * N,), torch.float32)


def test_graph_pipeline_fp16_interleaved():
    B, M, N, K = 3, 256, 512, 96
    a = torch.zeros(B * M * K * 2, dtype=torch.float16, device="cuda")
    b = torch.zeros(B * N * K * 2, dtype=torch.float16, device="cuda")

    def fill(r):
        g = torch.Generator(device="cuda").manual_seed(200 + r)
        for t in (a, b):
            t.copy_(torch.randn(t.shape, generator=g, device="cuda").to(torch.float16))

    capture_and_replay(lambda s: cc.Pipeline(B, M, N, K, 0, s, INTERLEAVED, PLANAR, ROW, COL, ROW,
                                              VT.float16, VT.float32, cc.Variant.opt),
                        [a, b], fill, (B * 2 * M * N,), torch.float32)


@pytest.mark.parametrize("what", ["pipeline", "packing_transpose_gemm"])
def test_graph_int1(what):
    # 16 batches of 32 C tiles: the 1-bit GEMM expands and multiplies in two groups, the
    # expansions on the object's second stream, forked from and joined into the captured one
    B, M, N, K = 16, 1024, 1024, 256
    a = torch.zeros(B * 2 * M * K, dtype=torch.uint8, device="cuda")
    b = torch.zeros(B * 2 * N * K, dtype=torch.uint8, device="cuda")

    def fill(r):
        g = torch.Generator(device="cuda").manual_seed(300 + r)
        for t in (a, b):
            t.copy_(torch.randint(0, 2, t.shape, generator=g, device="cuda", dtype=torch.uint8))

    if what == "pipeline":
        make = lambda s: cc.Pipeline(B, M, N, K, 0, s, PLANAR, PLANAR, ROW, COL, ROW, VT.int1, VT.int32,
                                     cc.Variant.opt)
    else:
        class Steps:
            """Packing -> Transpose -> GEMM as separate objects on one stream."""
            def __init__(self, s):
                prec = cc.Precision(VT.int1, VT.int32)
                mb, nb, kc = cc.GEMM.GetDimensions(prec)
                self.pk = [cc.Packing(B * 2 * rows * K, cc.Direction.forward, 0, s) for rows in (M, N)]
                self.tr = [cc.Transpose(B, rows, K, mb, kc, 1, 0, s) for rows in (M, N)]
                self.packed = [torch.zeros(B * 2 * rows * K // 32, dtype=torch.int32, device="cuda")
                               for rows in (M, N)]
                # the tiled layout holds whole tiles: rows padded to mb / nb, K to kc (512 samples)
                kp = cc.ceildiv(K, kc) * kc
                self.tiled = [torch.zeros(B * 2 * (cc.ceildiv(rows, t) * t) * kp // 32, dtype=torch.int32,
                                          device="cuda") for rows, t in ((M, mb), (N, nb))]
                self.gemm = cc.GEMM(B, M, N, K, 0, s, prec, cc.Variant.opt)

            def Run(self, pa, pb, pc):
                for i, src in enumerate((pa, pb)):
                    self.pk[i].Run(src, self.packed[i].data_ptr())
                    self.tr[i].Run(self.packed[i].data_ptr(), self.tiled[i].data_ptr())
                self.gemm.Run(self.tiled[0].data_ptr(), self.tiled[1].data_ptr(), pc)
        make = Steps

    capture_and_replay(make, [a, b], fill, (B * 2 * M * N,), torch.int32)


def _capture(side, run):
    """Captures run() on the stream `side` without any Run before it; returns the graph."""
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run()
    return graph


@pytest.mark.parametrize("expect_unaligned", [0, 1])
def test_graph_basic_gemm_meets_unaligned_operands_during_capture(expect_unaligned):
    """A basic-variant GEMM allocates its re-tiling workspace at the first Run that meets
    operands which are not 16-byte aligned - but not while the stream is being captured
    (the allocation would invalidate the capture): there it reads the rows through
    registers. With the option EXPECT_UNALIGNED the workspace exists from construction
    on. Either way the first such Run can be the captured one, and the replays give the
    oracle's result."""
    import oracle as orc
    from gpu_util import ORC_TYPE
    B, M, N, K = 2, 96, 200, 72
    rng = np.random.default_rng(31)
    qa = quantize(rng.uniform(-1, 1, B * 2 * M * K).astype(np.float32), VT.float16)
    qb = quantize(rng.uniform(-1, 1, B * 2 * N * K).astype(np.float32), VT.float16)
    skew = 1   # one fp16 element: 2 bytes off a 16-byte boundary
    d_a = to_device(np.concatenate([np.zeros(skew, np.uint16), qa]))
    d_b = to_device(np.concatenate([np.zeros(skew, np.uint16), qb]))
    d_c = torch.zeros(B * 2 * M * N, dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with cc.option(cc.Option.expect_unaligned, expect_unaligned):
        gemm = cc.GEMM(B, M, N, K, 0, side.cuda_stream, cc.Precision(VT.float16, VT.float32),
                       cc.Variant.basic)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    graph = _capture(side, lambda: gemm.Run(d_a.data_ptr() + 2 * skew, d_b.data_ptr() + 2 * skew,
                                            d_c.data_ptr()))
    assert torch.cuda.mem_get_info()[0] >= free_before, "Run allocated during the capture"
    want = orc.gemm(qa, qb, M, N, K, ORC_TYPE[VT.float16], ORC_TYPE[VT.float32])
    for _ in range(2):
        d_c.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = d_c.cpu().numpy().reshape(want.shape)
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3


def test_graph_fused_pipeline_meets_unaligned_buffers_during_capture():
    """A pipeline that reads rows in place creates the pipeline with transposes for
    unaligned buffers at the first Run that meets them; during a capture that Run reports
    an error instead of allocating, and with the option EXPECT_UNALIGNED the fallback
    exists from construction on and the captured Run works."""
    import oracle as orc
    from gpu_util import ORC_TYPE
    B, M, N, K = 2, 64, 128, 72
    rng = np.random.default_rng(32)
    a = rng.standard_normal((B, 2, M, K)).astype(np.float16)
    b = rng.standard_normal((B, 2, N, K)).astype(np.float16)
    skew = 2
    il = lambda x: np.concatenate([np.zeros(skew, np.uint16),
                                   np.ascontiguousarray(x.transpose(0, 2, 3, 1)).view(np.uint16).reshape(-1)])
    d_a, d_b = to_device(il(a)), to_device(il(b))
    d_c = torch.zeros(B * 2 * M * N, dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    make = lambda: cc.Pipeline(B, M, N, K, 0, side.cuda_stream, INTERLEAVED, PLANAR, ROW, COL, ROW,
                               VT.float16, VT.float32, cc.Variant.opt)
    run = lambda p: p.Run(d_a.data_ptr() + 2 * skew, d_b.data_ptr() + 2 * skew, d_c.data_ptr())
    # default: the Run inside the capture refuses
    pipe = make()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        try:
            with pytest.raises(RuntimeError, match="cannot be allocated while the stream is being captured"):
                run(pipe)
        finally:
            graph.capture_end()
    torch.cuda.synchronize()
    del graph
    # with the option: captured and replayed
    with cc.option(cc.Option.expect_unaligned, 1):
        pipe = make()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    graph = _capture(side, lambda: run(pipe))
    assert torch.cuda.mem_get_info()[0] >= free_before, "Run allocated during the capture"
    want = orc.gemm(a.view(np.uint16).reshape(-1), b.view(np.uint16).reshape(-1), M, N, K,
                    ORC_TYPE[VT.float16], ORC_TYPE[VT.float32])
    for _ in range(2):
        d_c.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = d_c.cpu().numpy().reshape(want.shape)
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3
