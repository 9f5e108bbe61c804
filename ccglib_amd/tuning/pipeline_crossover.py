"""Where reading rows in place stops paying: Pipeline.Run with the GEMM reading the caller's
rows in place (option PIPELINE_ROUTE = 1) against the two transposes followed by the GEMM on
tiles (PIPELINE_ROUTE = 2), for shapes on either side of the break-even points that
ccglib_pipeline_create uses (M N / (M + N): what the GEMM's work grows with, over what the
transposes' grows with), and the route the default picks.

    python -m ccglib_amd.tuning.pipeline_crossover [--k 256] [--rounds 3]

One MI355X, synthetic operands (N(0, 1); fp8 scaled into range), device buffers; every
(shape, route) is warmed up and then timed over about 40 ms of back-to-back Runs between
two events, `rounds` times in alternation; the table holds the medians.
"""
import argparse
import statistics

import torch

import ccglib_amd as cc

VT, AX, MO = cc.ValueType, cc.ComplexAxisLocation, cc.MemOrder
FAMILIES = [
    ("fp16 interleaved rows", VT.float16, torch.float16, AX.complex_interleaved),
    ("fp8 e4m3 interleaved rows", VT.float8e4m3, torch.float8_e4m3fn, AX.complex_interleaved),
    ("fp16 planar rows", VT.float16, torch.float16, AX.complex_planar),
]
# (M, N): squares across the break-even points, and rectangles to check that M N / (M + N) is
# the right abscissa
SHAPES = [(2048, 2048), (3072, 3072), (4096, 4096), (5120, 5120), (6144, 6144), (7168, 7168),
          (8192, 8192), (12288, 12288), (2048, 16384), (4096, 16384), (4096, 32768), (512, 4096)]


def time_runs(pipe, a, b, c, budget_ms=40.0):
    stream = torch.cuda.current_stream()
    for _ in range(3):
        pipe.Run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    pipe.Run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    e1.record(stream)
    e1.synchronize()
    n = max(3, int(budget_ms / max(e0.elapsed_time(e1), 1e-3)))
    e0.record(stream)
    for _ in range(n):
        pipe.Run(a.data_ptr(), b.data_ptr(), c.data_ptr())
    e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) / n


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--k", type=int, default=256)
    ap.add_argument("--rounds", type=int, default=3)
    args = ap.parse_args()
    K = args.k
    s = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(1)
    print("Pipeline.Run, opt variant, planar fp32 C, K = %d; B fills the compute units" % K)
    for name, vt, tdt, axis in FAMILIES:
        print("\n%s" % name)
        print("%-16s %4s %10s   %12s %12s   %8s   %s" % ("M x N", "B", "MN/(M+N)", "in place ms", "transposed ms",
                                                       "ratio", "default route"))
        for M, N in SHAPES:
            B = max(1, (1 << 27) // (M * N))
            shape_a = (B, M, K, 2) if axis == AX.complex_interleaved else (B, 2, M, K)
            shape_b = (B, N, K, 2) if axis == AX.complex_interleaved else (B, 2, N, K)
            scale = 448.0 / 5.8 if vt == VT.float8e4m3 else 1.0
            a = (torch.randn(shape_a, device="cuda", generator=gen) * scale).to(tdt)
            b = (torch.randn(shape_b, device="cuda", generator=gen) * scale).to(tdt)
            c = torch.empty((B, 2, M, N), device="cuda")
            pipes = {}
            for route in (0, 1, 2):
                with cc.option(cc.Option.pipeline_route, route):
                    pipes[route] = cc.Pipeline(B, M, N, K, 0, s, axis, AX.complex_planar, MO.row_major,
                                               MO.col_major, MO.row_major, vt, VT.float32, cc.Variant.opt)
            assert pipes[1].ReadsInPlace() and not pipes[2].ReadsInPlace()
            times = {1: [], 2: []}
            for _ in range(args.rounds):
                for route in (1, 2):
                    times[route].append(time_runs(pipes[route], a, b, c))
            t1, t2 = statistics.median(times[1]), statistics.median(times[2])
            print("%-16s %4d %10.0f   %12.4f %12.4f   %8.3f   %s" % (
                "%d x %d" % (M, N), B, M * N / (M + N), t1, t2, t1 / t2,
                "in place" if pipes[0].ReadsInPlace() else "transposed"), flush=True)
            del pipes, a, b, c


if __name__ == "__main__":
    main()
