"""GPU parity tests of the tiled-layout transpose: bit-exact against the CPU oracle.
Cases follow the reference's test/transpose/transpose.cpp (B=2, 256x128, 64x64
chunks, planar and interleaved, 8/16-bit and 1-bit) and add ragged shapes."""
import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import device_zeros, stream, to_device, to_host

pytestmark = pytest.mark.gpu
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved
NP = {8: np.uint8, 16: np.uint16, 32: np.uint32, 1: np.uint32}


def run_case(B, M, N, Mc, Nc, bits, axis, seed=0, host=False, skew=0):
    rng = np.random.default_rng(seed)
    dt = NP[bits]
    nw = N // 32 if bits == 1 else N
    x = rng.integers(1, np.iinfo(dt).max, B * 2 * M * nw, dtype=dt, endpoint=True)
    want = orc.transpose(x, B, M, N, Mc, Nc, bits, int(axis))
    d_out = to_device(np.full(want.size, 0xA5 if bits == 8 else 0xA5A5, dtype=dt))  # poison
    t = cc.Transpose(B, M, N, Mc, Nc, bits, 0, stream(), axis)
    if host:
        t.RunHost(x.ctypes.data, d_out.data_ptr())
    else:
        # skew: the input starts `skew` elements past a 16-byte boundary
        d_in = to_device(np.concatenate([np.zeros(skew, dtype=dt), x]))
        t.Run(d_in.data_ptr() + skew * dt().itemsize, d_out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_out, dt), want)


@pytest.mark.parametrize("bits", [8, 16, 32])
@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
def test_reference_fixture(bits, axis):
    run_case(2, 256, 128, 64, 64, bits, axis)          # test/transpose/transpose.cpp:37-42


def test_reference_fixture_one_bit():
    run_case(2, 256, 128, 64, 64, 1, PLANAR)           # :209-212
    run_case(2, 256, 1024, 128, 512, 1, PLANAR)
    run_case(2, 100, 1056, 128, 512, 1, PLANAR)        # ragged in words
    run_case(2, 100, 96, 128, 512, 1, INTERLEAVED)


@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
@pytest.mark.parametrize("bits,kc", [(16, 32), (8, 64)])
@pytest.mark.parametrize("M,N", [(128, 64), (100, 40), (300, 100), (512, 576), (1, 8), (129, 1000),
                                 (77, 33), (5, 7)])
def test_gemm_chunks(axis, bits, kc, M, N):
    # chunk sizes the GEMM asks for; shapes with ragged rows, ragged columns and
    # rows that are not whole 16-byte vectors (scalar kernel)
    run_case(3, M, N, 128, kc, bits, axis, seed=M + N)


@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
@pytest.mark.parametrize("bits,kc", [(16, 32), (8, 64), (32, 16)])
@pytest.mark.parametrize("M,N,skew", [(130, 1001, 0), (64, 257, 3), (200, 96, 1), (3, 15, 5), (97, 8001, 0)])
def test_ragged_rows(axis, bits, kc, M, N, skew):
    # rows of any length at any element-aligned address: whole vectors are moved
    # with wide loads wherever they lie, the end of a row element by element
    run_case(2, M, N, 128, kc, bits, axis, seed=N + skew, skew=skew)


@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
def test_odd_chunks(axis):
    run_case(2, 50, 36, 16, 12, 16, axis)              # chunk rows are not whole vectors
    run_case(2, 7, 5, 4, 4, 8, axis)
    run_case(1, 64, 64, 8, 16, 32, axis)


def test_host_input():
    # Run(const void *h_input, ...) does nothing in the reference
    # (src/transpose/Transpose.cpp:147-154); here it must transpose
    run_case(2, 100, 40, 128, 32, 16, PLANAR, host=True)


def test_empty():
    t = cc.Transpose(0, 16, 16, 16, 16, 16, 0, stream())
    t.Run(0, 0)


@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
@pytest.mark.parametrize("bits,kc,Ma,Mb,N,Mca,Mcb,skew", [
    # (one launch for both when one operand has at most a quarter of the other's rows)
    (16, 32, 512, 4096, 576, 128, 128, 0),    # beamformer operands: rows of 72 vectors
    (16, 32, 70, 300, 1000, 128, 64, 0),      # ragged rows and columns, different row tiles
    (16, 32, 100, 300, 1000, 128, 64, 0),     # the same as two launches
    (8, 64, 30, 130, 257, 128, 128, 0),       # rows that are not whole vectors
    (8, 64, 77, 130, 257, 128, 128, 0),
    (32, 16, 50, 200, 96, 128, 128, 0),
    (32, 16, 64, 200, 96, 128, 128, 0),
    (16, 32, 129, 30, 264, 128, 128, 1),      # first operand not 16-byte aligned: two launches
    (1, 512, 300, 64, 1056, 128, 128, 0),     # 1-bit words, the small operand second
    (1, 512, 100, 256, 1056, 128, 128, 0),
    (16, 32, 5, 7, 7, 128, 128, 0),           # scalar kernel for both
])
def test_pair_matches_oracle(axis, bits, kc, Ma, Mb, N, Mca, Mcb, skew):
    """ccglib_transpose_run_pair: both operands as the oracle transposes each."""
    B = 3
    rng = np.random.default_rng(Ma + Mb + N)
    dt = NP[bits]
    nw = N // 32 if bits == 1 else N
    outs, args, keep = [], [], []
    for M, Mc, sk in ((Ma, Mca, skew), (Mb, Mcb, 0)):
        x = rng.integers(1, np.iinfo(dt).max, B * 2 * M * nw, dtype=dt, endpoint=True)
        want = orc.transpose(x, B, M, N, Mc, kc, bits, int(axis))
        d_out = to_device(np.full(want.size, 0xA5, dtype=dt))
        d_in = to_device(np.concatenate([np.zeros(sk, dtype=dt), x]))
        t = cc.Transpose(B, M, N, Mc, kc, bits, 0, stream(), axis)
        keep.append((d_in, t))
        args += [t, d_in.data_ptr() + sk * dt().itemsize, d_out.data_ptr()]
        outs.append((d_out, want))
    cc.Transpose.RunPair(*args)
    torch.cuda.synchronize()
    for d_out, want in outs:
        assert np.array_equal(to_host(d_out, dt), want)


def test_pair_of_different_rows_falls_back():
    """Operands whose rows differ in length cannot share a launch: still both done."""
    rng = np.random.default_rng(5)
    outs, args, keep = [], [], []
    for M, N in ((64, 128), (32, 256)):
        x = rng.integers(1, 65535, 2 * 2 * M * N, dtype=np.uint16, endpoint=True)
        want = orc.transpose(x, 2, M, N, 64, 32, 16, int(PLANAR))
        d_out, d_in = to_device(np.zeros(want.size, dtype=np.uint16)), to_device(x)
        t = cc.Transpose(2, M, N, 64, 32, 16, 0, stream(), PLANAR)
        keep.append((d_in, t))
        args += [t, d_in.data_ptr(), d_out.data_ptr()]
        outs.append((d_out, want))
    cc.Transpose.RunPair(*args)
    torch.cuda.synchronize()
    for d_out, want in outs:
        assert np.array_equal(to_host(d_out, np.uint16), want)
