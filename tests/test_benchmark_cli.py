"""The benchmark programs in ccglib_amd/benchmark/ take the options of the
reference's benchmarks (benchmark/benchmark_gemm.cpp:16-47,
benchmark_transpose.cpp:16-42, benchmark_packing.cpp:15-32) and print its CSV
columns. They are built by ccglib_amd/benchmark/Makefile (and by build())."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BENCH = os.path.join(os.path.dirname(HERE), "ccglib_amd", "benchmark")


def run(name, *args):
    return subprocess.run([os.path.join(BENCH, name), *args], capture_output=True, text=True, timeout=300)


def built(name):
    return os.path.exists(os.path.join(BENCH, name))


@pytest.mark.parametrize("name,options", [
    ("benchmark_gemm", ["-b", "-m", "-n", "-k", "--pad", "--nr_benchmarks", "--benchmark_duration", "--csv",
                        "--precision_in", "--precision_out", "--variant", "--complex_axis", "--device"]),
    ("benchmark_transpose", ["-b", "-m", "-n", "--pad", "--nr_benchmarks", "--benchmark_duration", "--csv",
                             "--precision", "--variant", "--complex_axis", "--device"]),
    ("benchmark_packing", ["-n", "--nr_benchmarks", "--benchmark_duration", "--csv", "--direction", "--device"]),
])
def test_help_lists_the_reference_options(name, options):
    if not built(name):
        pytest.skip("benchmark programs not built")
    r = run(name, "--help")
    assert r.returncode == 0
    for o in options:
        assert o + " " in r.stdout or o + "\t" in r.stdout, o


def test_missing_required_option():
    if not built("benchmark_gemm"):
        pytest.skip("benchmark programs not built")
    r = run("benchmark_gemm", "-m", "128", "-n", "128")
    assert r.returncode != 0 and "Required argument missing: k" in r.stderr


@pytest.mark.gpu
def test_gemm_csv():
    r = run("benchmark_gemm", "-b", "2", "-m", "256,100", "-n", "256", "-k", "64,40", "--precision_in", "float16",
            "--benchmark_duration", "0.05", "--csv")
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == "#M,N,K,runtime_ms,tops"
    assert [l.split(",")[:3] for l in lines[1:]] == [["256", "256", "64"], ["100", "256", "40"]]
    assert all(float(l.split(",")[4]) > 0 for l in lines[1:])


@pytest.mark.gpu
def test_gemm_int1_and_basic_variant():
    r = run("benchmark_gemm", "-m", "128", "-n", "128", "-k", "1024", "--precision_in", "int1", "--precision_out",
            "int32", "--variant", "basic", "--benchmark_duration", "0.05")
    assert r.returncode == 0, r.stderr
    assert "TOps/s" in r.stdout and "128x128x1024" in r.stdout


@pytest.mark.gpu
def test_transpose_and_packing_csv():
    r = run("benchmark_transpose", "-b", "4", "-m", "300", "-n", "200", "--pad", "--precision", "float16",
            "--complex_axis", "interleaved", "--benchmark_duration", "0.05", "--csv")
    assert r.returncode == 0, r.stderr
    assert r.stdout.splitlines()[0] == "#M,N,runtime_ms,gbytes" and r.stdout.splitlines()[1].startswith("300,200,")
    for direction in ("pack", "unpack"):
        r = run("benchmark_packing", "-n", "1000000,4096", "--direction", direction, "--benchmark_duration", "0.05",
                "--csv")
        assert r.returncode == 0, r.stderr
        assert r.stdout.splitlines()[0] == "#N,runtime_ms,gbytes" and len(r.stdout.splitlines()) == 3


TUNE = os.path.join(os.path.dirname(HERE), "ccglib_amd", "tuning", "tune_gemm")


@pytest.mark.gpu
def test_tuner_sweeps_its_configurations():
    """The kernel-configuration sweep (the counterpart of the reference's tuning/tune_gemm.py:316-363)
    runs every configuration on a small shape and prints one timed line per configuration."""
    if not os.path.exists(TUNE):
        pytest.skip("tuner not built")
    r = subprocess.run([TUNE, "2", "256", "256", "64"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0].startswith("configuration") and "B=2 M=256 N=256 K=64" in lines[0]
    rows = [l for l in lines[1:] if "%" in l]
    assert len(rows) >= 10
    # the configurations that the library's dispatch uses are among them
    names = " | ".join(rows)
    for want in ("f16 256x128 w64x64 s3 m16 xt", "fp8 256x128 w64x64 s3 m32", "int1 256x128 w64x64 s3 m32",
                 "f16 planar 256x128 w64x64 s3 m16 xt", "f16 interleaved 256x128 w64x64 s3 m16"):
        assert want in names, want
    hashes = {}
    for l in rows:
        # "<name>  <ms>  <rate>  <percent>%   C <hash of C's bits>"
        fields = l.split()
        assert fields[-2] == "C" and fields[-3].endswith("%")
        ms, rate = float(fields[-5]), float(fields[-4])
        assert ms > 0 and rate > 0
        hashes[" ".join(fields[:-5])] = fields[-1]
    # the same operands, layout and MFMA shape: the same bits, whatever the block shape,
    # the epilogue or the ring
    assert hashes["f16 256x128 w64x64 s3 m16 xt"] == hashes["f16 128x256 w64x64 s3 m16 xt"]
    assert hashes["f16 256x128 w64x64 s3 m16 xt"] == hashes["f16 128x256 w64x64 y3 x4 m16 xt"]
    # a filter selects configurations by name
    r = subprocess.run([TUNE, "2", "256", "256", "64", "bf16"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and all("bf16" in l for l in r.stdout.strip().splitlines()[1:])
