"""Benchmark of the hot path on one MI355X.

Default workload (the configuration the reference's headline metric is quoted on):
a step is one pass over one batch of synthetic input of the beamformer-shaped
problem: interleaved fp16 A [64][512][576][2] (unit-magnitude random phases) and
B [64][4096][576][2] (complex Gaussian, sigma 1) are brought into the tiled layout
by Transpose and multiplied by the opt complex GEMM into planar fp32
C [64][2][512][4096]. Inputs are resident in HBM before the timed region.

Prints one JSON line. `value` is 8*B*M*N*K / (time per step): the whole step, data
preparation kernels (transpose, packing) included. The `roofline` object is about the
GEMM kernel alone, timed with events on the launch stream inside the timed region.

Other workloads (`--workload`): the reference's other benchmark configurations, for
per-kernel measurements; a run without flags does not use them.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# published dense peaks of MI355X
MFMA_PEAK_TFLOPS = {"f16": 2516.6, "bf16": 2516.6, "fp8": 5033.2}
HBM_PEAK_GBS = 8000.0
# The 1-bit GEMM runs on the fp4 MFMA (the packed words are expanded to +-1
# nibbles in registers, inside the GEMM kernel): published fp4 dense peak
FP4_PEAK_TOPS = 10066.3

WORKLOADS = {
    # name: (B, M, N, K, input type, output type, input axis, description)
    "beamformer": (64, 512, 4096, 576, "float16", "float32", "interleaved",
                   "beamformer-shaped batched complex GEMM: fp16 in, fp32 out, B=64 M=512 N=4096 "
                   "K=576; interleaved input -> Transpose -> opt GEMM -> planar C"),
    "square_bf16": (1, 8192, 8192, 8192, "bfloat16", "float32", "planar",
                    "large square complex GEMM: bf16 in, fp32 out, B=1 M=N=K=8192, planar in/out; "
                    "Transpose -> opt GEMM"),
    "square_bf16_out": (1, 8192, 8192, 8192, "bfloat16", "bfloat16", "planar",
                        "as square_bf16 with bf16-downcast output"),
    "fp8_e4m3": (16, 4096, 4096, 8192, "float8e4m3", "float32", "planar",
                 "fp8 e4m3 complex GEMM, fp32 out: B=16 M=N=4096 K=8192, planar; per-matrix scale "
                 "into the e4m3 range; Transpose -> opt GEMM"),
    "fp8_e5m2": (16, 4096, 4096, 8192, "float8e5m2", "float32", "planar",
                 "as fp8_e4m3 with e5m2"),
    "correlator_int1": (32, 1024, 1024, 65536, "int1", "int32", "planar",
                        "1-bit correlator-style complex GEMM: one byte per sample -> Packing -> "
                        "Transpose -> 1-bit GEMM -> int32; B=32 M=N=1024 K=65536"),
}


def cpu_baseline(B, M, N, K, orc, np):
    """The CPU oracle (a port of the reference's CPU path) timed on this host's
    cores on a few batches of the default workload (about 10 s of CPU work)."""
    nb = min(B, 6)
    rng = np.random.default_rng(2)
    a = rng.standard_normal((nb, 2, M, K)).astype(np.float16).view(np.uint16).reshape(-1)
    b = rng.standard_normal((nb, 2, N, K)).astype(np.float16).view(np.uint16).reshape(-1)
    t0 = time.perf_counter()
    orc.gemm(a, b, M, N, K, orc.FLOAT16)
    dt = time.perf_counter() - t0
    flops = 8.0 * nb * M * N * K
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": orc.max_threads(),
            "kind": "port",
            "sample": "%d of %d batches (M=%d N=%d K=%d fp16->fp32), %.2f s" % (nb, B, M, N, K, dt)}


def make_inputs(name, torch, np):
    """Synthetic inputs of a workload, resident on the GPU, in the storage layout the
    first kernel of the step reads. Returns (a, b, info)."""
    B, M, N, K, tin, _, axis, _ = WORKLOADS[name]
    gen = torch.Generator(device="cuda").manual_seed({"beamformer": 2, "square_bf16": 3,
                                                      "square_bf16_out": 3, "fp8_e4m3": 4,
                                                      "fp8_e5m2": 4, "correlator_int1": 5}[name])
    info = {}
    if name == "beamformer":
        phase = torch.rand((B, M, K), device="cuda", generator=gen) * (2 * np.pi)
        a = torch.stack([torch.cos(phase), torch.sin(phase)], dim=-1).to(torch.float16).contiguous()
        del phase
        b = torch.randn((B, N, K, 2), device="cuda", generator=gen).to(torch.float16).contiguous()
    elif tin == "bfloat16":
        a = torch.randn((B, 2, M, K), device="cuda", generator=gen).to(torch.bfloat16)
        b = torch.randn((B, 2, N, K), device="cuda", generator=gen).to(torch.bfloat16)
    elif tin in ("float8e4m3", "float8e5m2"):
        dt, fmax = ((torch.float8_e4m3fn, 448.0) if tin == "float8e4m3"
                    else (torch.float8_e5m2, 57344.0))
        out = []
        for rows in (M, N):
            x = torch.randn((B, 2, rows, K), device="cuda", generator=gen)
            scale = fmax / float(x.abs().max())
            out.append((x * scale).clamp_(-fmax, fmax).to(dt))
            info.setdefault("scales", []).append(scale)
            del x
        a, b = out
    else:  # one byte per 1-bit sample
        a = torch.randint(0, 2, (B, 2, M, K), device="cuda", generator=gen, dtype=torch.uint8)
        b = torch.randint(0, 2, (B, 2, N, K), device="cuda", generator=gen, dtype=torch.uint8)
    return a, b, info


def check_result(name, a, b, c, torch):
    """One batch against an independent library's product of the same inputs."""
    B, M, N, K, tin, tout, axis, _ = WORKLOADS[name]
    bi = B - 1
    if tin == "int1":
        # bit 1 = +1, bit 0 = -1; exact in fp32 (|sums| <= 2K < 2^24)
        sa = a[bi].float() * 2 - 1
        sb = b[bi].float() * 2 - 1
        re = sa[0] @ sb[0].T - sa[1] @ sb[1].T
        im = sa[0] @ sb[1].T + sa[1] @ sb[0].T
        ok = bool(torch.equal(c[bi, 0].float(), re) and torch.equal(c[bi, 1].float(), im))
        return {"bit_exact_vs_pm1_matmul": ok, "batch": bi}
    if axis == "interleaved":
        a64 = torch.complex(a[bi, ..., 0].double(), a[bi, ..., 1].double())
        b64 = torch.complex(b[bi, ..., 0].double(), b[bi, ..., 1].double())
    else:
        a64 = torch.complex(a[bi, 0].double(), a[bi, 1].double())
        b64 = torch.complex(b[bi, 0].double(), b[bi, 1].double())
    ref = a64 @ b64.T
    got = torch.complex(c[bi, 0].double(), c[bi, 1].double())
    bound = 2e-2 if tin.startswith("float8") else (2.0 ** -8 if tout == "bfloat16" else 1e-3)
    return {"rel_frobenius_vs_float64": float((got - ref).norm() / ref.norm()), "bound": bound,
            "batch": bi}


def sample_core_clock(run, torch, load_s=1.2):
    """The core clock while `run` is enqueued over and over: rocm-smi is asked once, from a
    thread, about a third into `load_s` seconds of load. Returns MHz, or None when rocm-smi
    is not there or says nothing that parses (the figure is reported, not relied on)."""
    import re
    import shutil
    import subprocess
    import threading
    tool = shutil.which("rocm-smi") or "/opt/rocm/bin/rocm-smi"
    if not os.path.exists(tool):
        return None
    command = [tool, "--showclocks"]
    try:
        # rocm-smi is a Python script behind "#!/usr/bin/env python3": started with this
        # interpreter directly, the child process is one program from start to end (under a
        # profiler whose preloaded library touches the GPU in every process, the hop from
        # env to python3 would replace a program that has initialised the GPU)
        with open(tool, "rb") as f:
            first = f.readline()
        if first.startswith(b"#!") and b"python" in first:
            command = [sys.executable, os.path.realpath(tool), "--showclocks"]
    except OSError:
        pass
    found = []

    def ask():
        time.sleep(load_s / 3)
        try:
            out = subprocess.run(command, capture_output=True, text=True, timeout=20).stdout
            m = re.search(r"sclk clock level:\s*\d+:\s*\((\d+)Mhz\)", out)
            if m:
                found.append(float(m.group(1)))
        except Exception:
            pass

    t = threading.Thread(target=ask)
    t.start()
    t0 = time.perf_counter()
    while t.is_alive() or time.perf_counter() - t0 < load_s:
        for _ in range(16):
            run()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 > 30:
            break
    t.join()
    return found[0] if found else None


def measure(name, steps, warmup, settle_ms, torch, np, cc, isolated=False, copy_calibration=False,
            check=True, clock=False):
    """Builds the step of a workload, settles, times `steps` steps and checks the result.
    Returns a dict of figures plus what the optional extra measurements need."""
    stream = torch.cuda.current_stream().cuda_stream
    VT, AX, MO = cc.ValueType, cc.ComplexAxisLocation, cc.MemOrder
    B, M, N, K, tin_name, tout_name, axis_name, description = WORKLOADS[name]
    tin, tout = VT[tin_name], VT[tout_name]
    axis = AX.complex_interleaved if axis_name == "interleaved" else AX.complex_planar
    a_in, b_in, info = make_inputs(name, torch, np)

    prec = cc.Precision(tin, tout)
    bits = prec.GetInputBits()
    mb, nb, kc = cc.GEMM.GetDimensions(prec)
    mp, np_, kp = cc.ceildiv(M, mb) * mb, cc.ceildiv(N, nb) * nb, cc.ceildiv(K, kc) * kc
    out_dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16,
                 "int32": torch.int32}[tout_name]
    c = torch.empty((B, 2, M, N), dtype=out_dtype, device="cuda")

    # ---- the step: a list of (label, callable, algorithmic bytes) + the GEMM ----------
    kernels = []
    a_cur, b_cur = a_in, b_in
    if tin == VT.int1:
        na, nb_ = B * 2 * M * K, B * 2 * N * K
        a_p = torch.empty(na // 32, dtype=torch.int32, device="cuda")
        b_p = torch.empty(nb_ // 32, dtype=torch.int32, device="cuda")
        pk_a = cc.Packing(na, cc.Direction.forward, 0, stream)
        pk_b = cc.Packing(nb_, cc.Direction.forward, 0, stream)
        kernels.append(("packing_a", lambda s=a_cur, d=a_p: pk_a.Run(s.data_ptr(), d.data_ptr()),
                        na + na / 8))
        kernels.append(("packing_b", lambda s=b_cur, d=b_p: pk_b.Run(s.data_ptr(), d.data_ptr()),
                        nb_ + nb_ / 8))
        a_cur, b_cur = a_p, b_p
    a_t = torch.empty(B * 2 * mp * kp * bits // 8, dtype=torch.uint8, device="cuda")
    b_t = torch.empty(B * 2 * np_ * kp * bits // 8, dtype=torch.uint8, device="cuda")
    tr_a = cc.Transpose(B, M, K, mb, kc, bits, 0, stream, axis)
    tr_b = cc.Transpose(B, N, K, nb, kc, bits, 0, stream, axis)
    # both operands through one call (what Pipeline.Run does too); each on its own is
    # timed after the steps, see `standalone` below
    bytes_a, bytes_b = 2.0 * B * 2 * M * K * bits / 8, 2.0 * B * 2 * N * K * bits / 8
    kernels.append(("transposes", lambda sa=a_cur, sb=b_cur: cc.Transpose.RunPair(
        tr_a, sa.data_ptr(), a_t.data_ptr(), tr_b, sb.data_ptr(), b_t.data_ptr()), bytes_a + bytes_b))
    standalone = [("transpose_a", lambda s=a_cur: tr_a.Run(s.data_ptr(), a_t.data_ptr()), bytes_a),
                  ("transpose_b", lambda s=b_cur: tr_b.Run(s.data_ptr(), b_t.data_ptr()), bytes_b),
                  ("transposes_back_to_back", kernels[-1][1], bytes_a + bytes_b)]
    gemm = cc.GEMM(B, M, N, K, 0, stream, prec, cc.Variant.opt, AX.complex_planar, MO.row_major)
    run_gemm = lambda: gemm.Run(a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())

    def step():
        for _, fn, _ in kernels:
            fn()
        run_gemm()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # Settle phase, sized by duration as the reference's benchmark protocol sizes its warm-up
    # (benchmark/benchmark_gemm.cpp:262-298): the part runs under a power limit whose
    # controller needs tens of milliseconds of continuous load to reach its steady clock,
    # whatever --warmup says. The same step, untimed, until `settle_ms` have passed.
    settle_steps, settled = 0, 0.0
    if settle_ms > 0:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        while settled < settle_ms:
            e0.record()
            for _ in range(8):
                step()
            e1.record()
            e1.synchronize()
            settled += e0.elapsed_time(e1)
            settle_steps += 8

    if copy_calibration:
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
    # the situation that counts (the GEMM right after the data preparation).
    nk = len(kernels)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(nk + 2)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        ev[i][0].record()
        for j, (_, fn, _) in enumerate(kernels):
            fn()
            ev[i][j + 1].record()
        run_gemm()
        ev[i][nk + 1].record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    flops = 8.0 * B * M * N * K
    gemm_ms = sum(e[nk].elapsed_time(e[nk + 1]) for e in ev) / steps
    gemm_tflops = flops / (gemm_ms * 1e-3) / 1e12
    per_kernel = {"gemm_ms": gemm_ms, "gemm_tflops": gemm_tflops}
    for j, (label, _, nbytes) in enumerate(kernels):
        ms = sum(e[j].elapsed_time(e[j + 1]) for e in ev) / steps
        per_kernel[label + "_ms"] = ms
        per_kernel[label + "_gbs"] = nbytes / ms / 1e6
        per_kernel[label + "_frac_of_hbm_peak"] = nbytes / ms / 1e6 / HBM_PEAK_GBS

    # The two transposes as separate launches, each 20 times back to back between
    # two events (an event pair around a single 30 us launch adds some 4 us to it).
    for label, fn, nbytes in standalone:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        e0.record()
        for _ in range(20):
            fn()
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1) / 20
        per_kernel[label + "_ms"] = ms
        per_kernel[label + "_gbs"] = nbytes / ms / 1e6
        per_kernel[label + "_frac_of_hbm_peak"] = nbytes / ms / 1e6 / HBM_PEAK_GBS
    # What an event pair adds to the interval it brackets: 20 empty intervals on the same
    # stream. (The in-step figures contain it once per interval; the back-to-back ones
    # spread it over 20 launches.)
    empty = [torch.cuda.Event(enable_timing=True) for _ in range(21)]
    for e in empty:
        e.record()
    empty[-1].synchronize()
    overhead_ms = sum(empty[i].elapsed_time(empty[i + 1]) for i in range(20)) / 20
    per_kernel["event_interval_overhead_ms"] = overhead_ms
    for label, _, nbytes in kernels:
        net = per_kernel[label + "_ms"] - overhead_ms
        if net > 0:
            per_kernel[label + "_frac_net_of_event_overhead"] = nbytes / net / 1e6 / HBM_PEAK_GBS
    # Two launches of the same kernel on operands of different size give its fixed cost per
    # launch and its asymptotic rate: ms = fixed + bytes / rate.
    sizes = {label: nbytes for label, _, nbytes in standalone}
    if "transpose_a" in sizes and "transpose_b" in sizes and \
            max(sizes["transpose_a"], sizes["transpose_b"]) >= 2 * min(sizes["transpose_a"], sizes["transpose_b"]):
        (la, lb) = ("transpose_a", "transpose_b") if sizes["transpose_a"] < sizes["transpose_b"] else \
            ("transpose_b", "transpose_a")
        rate = (sizes[lb] - sizes[la]) / (per_kernel[lb + "_ms"] - per_kernel[la + "_ms"])   # bytes per ms
        fixed_ms = per_kernel[la + "_ms"] - sizes[la] / rate
        per_kernel["transpose_launch_fixed_cost_us"] = fixed_ms * 1e3
        per_kernel["transpose_asymptotic_gbs"] = rate / 1e6
        per_kernel["transpose_asymptotic_frac_of_hbm_peak"] = rate / 1e6 / HBM_PEAK_GBS
    per_kernel["method"] = ("gemm, transposes (both operands through ccglib_transpose_run_pair: one "
                            "launch when one operand is small, else two) and packing_*: event pairs "
                            "inside the timed steps; transpose_a / transpose_b / "
                            "transposes_back_to_back (the pair call again): 20 back to back between "
                            "two events after the steps; event_interval_overhead_ms: what an empty "
                            "interval between two events measures on this stream (contained once in "
                            "every in-step figure; *_frac_net_of_event_overhead subtracts it); "
                            "transpose_launch_fixed_cost_us / transpose_asymptotic_*: from the two "
                            "stand-alone transposes of different size, ms = fixed + bytes / rate")

    # (the library says which of its kernels the GEMM object launches)
    kernel_name = "%s <%s -> %s>" % (gemm.KernelName(), tin_name, tout_name)
    if tin == VT.int1:
        dtype, peak, unit = "fp4 (+-1, exact int32 result)", FP4_PEAK_TOPS, "TOP/s"
        kernel_name += " (fp4 MFMA, bits expanded in registers)"
    else:
        dtype = {"float16": "f16", "bfloat16": "bf16"}.get(tin_name, "fp8")
        peak, unit = MFMA_PEAK_TFLOPS[dtype], "TFLOP/s"

    out = {"name": name, "description": description, "shape": (B, M, N, K), "flops": flops,
           "ms_per_step": ms_per_step, "value": flops / (ms_per_step * 1e-3) / 1e12,
           "gemm_ms": gemm_ms, "gemm_tflops": gemm_tflops, "per_kernel": per_kernel,
           "dtype": dtype, "peak": peak, "unit": unit, "kernel_name": kernel_name,
           "settle_ms": settled, "settle_steps": settle_steps, "info": info,
           "check": check_result(name, a_in, b_in, c, torch) if check else None}
    if isolated:
        # the GEMM launched back to back on its own (inputs and caches warm)
        iters = max(steps, 10)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        run_gemm()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(iters):
            run_gemm()
        e1.record()
        torch.cuda.synchronize()
        iso_ms = e0.elapsed_time(e1) / iters
        out["isolated"] = {"gemm_ms": iso_ms, "gemm_tflops": flops / (iso_ms * 1e-3) / 1e12}
    if clock:
        # core clock under this workload's steps, after everything that is timed
        out["sclk_mhz"] = sample_core_clock(step, torch)
    out["_buffers"] = (a_in, b_in, c)    # for the optional pipeline measurements of the caller
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    # The part runs under a power limit whose controller takes about 30 ms of continuous
    # load to settle (GEMM launches of the default workload go 0.55 -> 0.70 -> 0.56 ms over
    # the first 35 steps). Whatever --warmup says, the same step is repeated, untimed, for
    # this many milliseconds before the timed region, and the JSON line says so.
    ap.add_argument("--settle-ms", type=float, default=150.0)
    ap.add_argument("--workload", default="beamformer", choices=sorted(WORKLOADS))
    ap.add_argument("--other-steps", type=int, default=20,
                    help="timed steps of each of the other workloads that a default run reports "
                         "in `other_workloads` (0: skip them)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--no-clock", action="store_true",
                    help="do not sample the core clock under load with rocm-smi after the timed steps")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 1 GiB device copy (for scaling rocprofv3 HBM counters)")
    ap.add_argument("--isolated", action="store_true",
                    help="also time the GEMM launched back to back outside the step")
    ap.add_argument("--host", action="store_true",
                    help="also time Pipeline's host-pointer Run on page-locked buffers (copies over "
                         "PCIe in both directions included; never part of `value`)")
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

    name = args.workload
    B, M, N, K, tin_name, tout_name, axis_name, description = WORKLOADS[name]
    tin, tout = VT[tin_name], VT[tout_name]
    m = measure(name, args.steps, args.warmup, args.settle_ms, torch, np, cc,
                isolated=args.isolated, copy_calibration=args.copy_calibration,
                check=not args.no_check, clock=not args.no_clock)
    a_in, b_in, c = m.pop("_buffers")
    flops, value, ms_per_step = m["flops"], m["value"], m["ms_per_step"]
    gemm_ms, gemm_tflops, peak = m["gemm_ms"], m["gemm_tflops"], m["peak"]

    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "gemm_f16_beamformer_traffic.json")
    if name == "beamformer" and os.path.exists(tpath):
        traffic = json.load(open(tpath)).get("hbm_bytes_per_launch")
        traffic_source = ("constant read from profiles/gemm_f16_beamformer_traffic.json: rocprofv3 "
                          "--pmc FETCH_SIZE / WRITE_SIZE of this command in an earlier run, scaled "
                          "by a copy kernel; not measured in this run")

    result = {
        "metric": "complex TFLOP/s (8 flop/cMAC) on 1 MI355X + % of dtype MFMA peak",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_ms": m["settle_ms"], "settle_steps": m["settle_steps"],
        "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": m["dtype"], "data": "synthetic",
        "config": {"workload": description + " (data preparation kernels inside the step)",
                   "name": name, "B": B, "M": M, "N": N, "K": K, "variant": "opt"},
        "pct_of_peak": 100.0 * value / peak,
        "roofline": {"kernel": m["kernel_name"], "bound": "mfma", "achieved": gemm_tflops,
                     "peak": peak, "unit": m["unit"], "frac": gemm_tflops / peak,
                     "traffic": traffic, "traffic_source": traffic_source, "kernel_ms": gemm_ms},
        "kernels": m["per_kernel"],
    }
    if m.get("sclk_mhz"):
        # The published peak is CUs x flop per clock and CU x 2.4 GHz; at the clock the part
        # actually runs under this load (power limit) the same formula gives a lower roof.
        sclk = m["sclk_mhz"]
        result["roofline"]["sclk_mhz_under_load"] = sclk
        result["roofline"]["peak_at_measured_clock"] = peak * sclk / 2400.0
        result["roofline"]["frac_of_peak_at_measured_clock"] = gemm_tflops / (peak * sclk / 2400.0)
    result.update(m["info"])
    if "isolated" in m:
        result["isolated"] = m["isolated"]

    if axis_name == "interleaved":
        # The same job through ccglib's Pipeline wrapper, which here feeds the interleaved
        # buffers to the GEMM directly (one kernel, no transposes, no intermediate buffers).
        # Reported beside the headline figure, which keeps the explicit Transpose launches.
        c2 = torch.empty_like(c)
        pipe = cc.Pipeline(B, M, N, K, 0, stream, AX.complex_interleaved, AX.complex_planar,
                           MO.row_major, MO.col_major, MO.row_major, tin, tout, cc.Variant.opt)
        for _ in range(args.warmup + m["settle_steps"]):
            pipe.Run(a_in.data_ptr(), b_in.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            pipe.Run(a_in.data_ptr(), b_in.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        fused_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        result["fused_pipeline"] = {
            "ms_per_step": fused_ms, "tflops": flops / (fused_ms * 1e-3) / 1e12,
            "max_abs_diff_vs_unfused": float((c2 - c).abs().max())}

    if tin == VT.int1:
        # The same job through Pipeline.Run, which packs the one-byte-per-sample input
        # straight into the tiled 1-bit layout (no packed, untransposed intermediate).
        c2 = torch.empty_like(c)
        pipe = cc.Pipeline(B, M, N, K, 0, stream, AX.complex_planar, AX.complex_planar,
                           MO.row_major, MO.col_major, MO.row_major, tin, tout, cc.Variant.opt)
        for _ in range(args.warmup + m["settle_steps"]):
            pipe.Run(a_in.data_ptr(), b_in.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            pipe.Run(a_in.data_ptr(), b_in.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        fused_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        result["fused_pipeline"] = {
            "ms_per_step": fused_ms, "tops": flops / (fused_ms * 1e-3) / 1e12,
            "identical_to_unfused": bool(torch.equal(c2, c))}
        del pipe, c2

    if args.host:
        # Host buffers in, host buffer out: the pipeline's host-pointer Run, which moves
        # chunks of batches over a few streams so that copies in, kernels and copies out overlap.
        in_axis = AX.complex_interleaved if axis_name == "interleaved" else AX.complex_planar
        pipe = cc.Pipeline(B, M, N, K, 0, stream, in_axis, AX.complex_planar, MO.row_major,
                           MO.col_major, MO.row_major, tin, tout, cc.Variant.opt)
        h_a = torch.empty(a_in.numel() * a_in.element_size(), dtype=torch.uint8, pin_memory=True)
        h_b = torch.empty(b_in.numel() * b_in.element_size(), dtype=torch.uint8, pin_memory=True)
        h_c = torch.empty(c.numel() * c.element_size(), dtype=torch.uint8, pin_memory=True)
        h_a.copy_(a_in.view(torch.uint8).reshape(-1))
        h_b.copy_(b_in.view(torch.uint8).reshape(-1))
        torch.cuda.synchronize()
        reps = 3
        pipe.RunHost(h_a.data_ptr(), h_b.data_ptr(), h_c.data_ptr())
        t0 = time.perf_counter()
        for _ in range(reps):
            pipe.RunHost(h_a.data_ptr(), h_b.data_ptr(), h_c.data_ptr())
        host_ms = (time.perf_counter() - t0) * 1e3 / reps
        moved = h_a.numel() + h_b.numel() + h_c.numel()
        c_dev = torch.empty_like(c)
        pipe.Run(a_in.data_ptr(), b_in.data_ptr(), c_dev.data_ptr())
        torch.cuda.synchronize()
        same = bool(torch.equal(h_c, c_dev.view(torch.uint8).reshape(-1).cpu()))
        del c_dev
        result["host_pipeline"] = {
            "ms_per_run": host_ms, "tflops": flops / (host_ms * 1e-3) / 1e12,
            "host_bytes_in": h_a.numel() + h_b.numel(), "host_bytes_out": h_c.numel(),
            "pcie_gbs_both_directions": moved / host_ms / 1e6,
            "identical_to_device_run": same}
        del pipe, h_a, h_b, h_c

    if not args.no_check:
        result["check"] = m["check"]

    if name == "beamformer" and args.other_steps > 0:
        # The reference's other benchmark configurations under the same clock: the same
        # protocol (warm-up, settle phase, events around the GEMM inside the step), fewer
        # steps; the buffers of one workload are freed before the next one is built.
        del a_in, b_in, c, m
        torch.cuda.empty_cache()
        others = {}
        for other in ("square_bf16", "square_bf16_out", "fp8_e4m3", "fp8_e5m2", "correlator_int1"):
            o = measure(other, args.other_steps, 3, args.settle_ms, torch, np, cc,
                        check=not args.no_check, clock=not args.no_clock)
            o.pop("_buffers")
            others[other] = {
                "kernel": o["kernel_name"], "shape": dict(zip("BMNK", o["shape"])),
                "steps": args.other_steps, "settle_ms": o["settle_ms"],
                "kernel_ms": o["gemm_ms"], "achieved": o["gemm_tflops"], "peak": o["peak"],
                "unit": o["unit"], "frac": o["gemm_tflops"] / o["peak"],
                "ms_per_step": o["ms_per_step"], "step_rate": o["value"],
                "kernels": o["per_kernel"], "check": o["check"]}
            if o.get("sclk_mhz"):
                others[other]["sclk_mhz_under_load"] = o["sclk_mhz"]
                others[other]["frac_of_peak_at_measured_clock"] = \
                    o["gemm_tflops"] / (o["peak"] * o["sclk_mhz"] / 2400.0)
            del o
            torch.cuda.empty_cache()
        result["other_workloads"] = others

    if not args.no_cpu_baseline and name == "beamformer":
        import oracle as orc
        result["cpu_baseline"] = cpu_baseline(B, M, N, K, orc, np)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
