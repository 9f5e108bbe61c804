"""Benchmark of the hot path on one MI355X.

A step is one pass over one batch of synthetic input of the beamformer-shaped
workload: interleaved fp16 A [64][512][576][2] (unit-magnitude random phases)
and B [64][4096][576][2] (complex Gaussian, sigma 1) are brought into the tiled
layout by Transpose and multiplied by the opt complex GEMM into planar fp32
C [64][2][512][4096]. Inputs are resident in HBM before the timed region.

Prints one JSON line. `value` is 8*B*M*N*K / (time per step): the whole step,
transposes included. The `roofline` object is about the GEMM kernel alone.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = {"f16": 2516.6, "bf16": 2516.6, "fp8": 5033.2}
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (B, M, N, K, type_in)
    "beamformer": (64, 512, 4096, 576, "float16"),
}


def time_kernel(fn, iters, torch):
    """Average duration in ms of fn() over `iters` back-to-back launches, from
    events recorded on the stream the kernels run on (torch's current stream)."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def cpu_baseline(B, M, N, K, orc, np):
    """The CPU oracle (a port of the reference's CPU path) timed on this host's
    cores on one batch of the same workload."""
    rng = np.random.default_rng(2)
    a = rng.standard_normal((1, 2, M, K)).astype(np.float16).view(np.uint16).reshape(-1)
    b = rng.standard_normal((1, 2, N, K)).astype(np.float16).view(np.uint16).reshape(-1)
    n_rows = N
    t0 = time.perf_counter()
    orc.gemm(a, b, M, n_rows, K, orc.FLOAT16)
    dt = time.perf_counter() - t0
    flops = 8.0 * M * n_rows * K
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": orc.max_threads(),
            "kind": "port",
            "sample": "1 of %d batches (M=%d N=%d K=%d fp16->fp32), %.2f s" % (B, M, n_rows, K, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="beamformer", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 1 GiB device copy (for scaling rocprofv3 HBM counters)")
    ap.add_argument("--isolated", action="store_true",
                    help="also time the GEMM launched back to back outside the step")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the batch axis "
                 "would shard with no exchange); run with --gpus 1")

    import numpy as np
    import torch
    import ccglib_amd as cc

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    VT, AX, MO = cc.ValueType, cc.ComplexAxisLocation, cc.MemOrder

    B, M, N, K, _ = WORKLOADS[args.workload]
    gen = torch.Generator(device="cuda").manual_seed(2)
    phase = torch.rand((B, M, K), device="cuda", generator=gen) * (2 * np.pi)
    a_il = torch.stack([torch.cos(phase), torch.sin(phase)], dim=-1).to(torch.float16).contiguous()
    del phase
    b_il = torch.randn((B, N, K, 2), device="cuda", generator=gen).to(torch.float16).contiguous()

    mb, nb, kc = cc.GEMM.GetDimensions(VT.float16)
    mp, np_, kp = cc.ceildiv(M, mb) * mb, cc.ceildiv(N, nb) * nb, cc.ceildiv(K, kc) * kc
    a_t = torch.empty(B * 2 * mp * kp, dtype=torch.float16, device="cuda")
    b_t = torch.empty(B * 2 * np_ * kp, dtype=torch.float16, device="cuda")
    c = torch.empty((B, 2, M, N), dtype=torch.float32, device="cuda")

    tr_a = cc.Transpose(B, M, K, mb, kc, 16, 0, stream, AX.complex_interleaved)
    tr_b = cc.Transpose(B, N, K, nb, kc, 16, 0, stream, AX.complex_interleaved)
    gemm = cc.GEMM(B, M, N, K, 0, stream, VT.float16, cc.Variant.opt, AX.complex_planar,
                   MO.row_major)

    def step():
        tr_a.Run(a_il.data_ptr(), a_t.data_ptr())
        tr_b.Run(b_il.data_ptr(), b_t.data_ptr())
        gemm.Run(a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    if args.copy_calibration:
        # a copy kernel of known size: reads 1 GiB and writes 1 GiB per launch
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # Timed region: `steps` passes, bracketed by synchronisation for the wall-clock
    # figure. Inside it every kernel is also bracketed by events recorded on the
    # stream the kernels are launched on, which gives each kernel's duration in
    # the situation that counts (the GEMM right after the transposes).
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        ev[i][0].record()
        tr_a.Run(a_il.data_ptr(), a_t.data_ptr())
        ev[i][1].record()
        tr_b.Run(b_il.data_ptr(), b_t.data_ptr())
        ev[i][2].record()
        gemm.Run(a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
        ev[i][3].record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    flops = 8.0 * B * M * N * K
    value = flops / (ms_per_step * 1e-3) / 1e12
    tra_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    trb_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    gemm_ms = sum(e[2].elapsed_time(e[3]) for e in ev) / args.steps
    gemm_tflops = flops / (gemm_ms * 1e-3) / 1e12
    trb_bytes = 2.0 * B * 2 * N * K * 2      # read + write, reference's definition
    tra_bytes = 2.0 * B * 2 * M * K * 2

    isolated = None
    if args.isolated:
        # the GEMM launched back to back on its own (inputs and caches warm)
        iters = max(args.steps, 10)
        iso_ms = time_kernel(lambda: gemm.Run(a_t.data_ptr(), b_t.data_ptr(), c.data_ptr()), iters, torch)
        isolated = {"gemm_ms": iso_ms, "gemm_tflops": flops / (iso_ms * 1e-3) / 1e12}

    traffic = None
    tpath = os.path.join(ROOT, "profiles", "gemm_f16_beamformer_traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get("hbm_bytes_per_launch")

    result = {
        "metric": "complex TFLOP/s (8 flop/cMAC) on 1 MI355X + % of dtype MFMA peak",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "beamformer-shaped batched complex GEMM: fp16 in, fp32 out, "
                               "B=64 M=512 N=4096 K=576; interleaved input -> Transpose -> opt "
                               "GEMM -> planar C (transposes inside the step)",
                   "B": B, "M": M, "N": N, "K": K, "variant": "opt"},
        "pct_of_mfma_peak": 100.0 * value / MFMA_PEAK_TFLOPS["f16"],
        "roofline": {"kernel": "complex_gemm_mfma<f16->f32, tiled>", "bound": "mfma",
                     "achieved": gemm_tflops, "peak": MFMA_PEAK_TFLOPS["f16"], "unit": "TFLOP/s",
                     "frac": gemm_tflops / MFMA_PEAK_TFLOPS["f16"], "traffic": traffic,
                     "kernel_ms": gemm_ms},
        "kernels": {"gemm_ms": gemm_ms, "gemm_tflops": gemm_tflops,
                    "transpose_a_ms": tra_ms, "transpose_a_gbs": tra_bytes / tra_ms / 1e6,
                    "transpose_b_ms": trb_ms, "transpose_b_gbs": trb_bytes / trb_ms / 1e6,
                    "transpose_b_frac_of_hbm_peak": trb_bytes / trb_ms / 1e6 / HBM_PEAK_GBS},
    }
    if isolated:
        result["isolated"] = isolated

    if not args.no_check:
        # one batch against a float64 product computed by an independent library
        bi = B - 1
        a64 = torch.complex(a_il[bi, ..., 0].double(), a_il[bi, ..., 1].double())
        b64 = torch.complex(b_il[bi, ..., 0].double(), b_il[bi, ..., 1].double())
        ref = a64 @ b64.T
        got = torch.complex(c[bi, 0].double(), c[bi, 1].double())
        result["check"] = {"rel_frobenius_vs_float64": float((got - ref).norm() / ref.norm()),
                           "bound": 1e-3, "batch": bi}

    if not args.no_cpu_baseline:
        import oracle as orc
        result["cpu_baseline"] = cpu_baseline(B, M, N, K, orc, np)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
