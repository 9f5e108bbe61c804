"""GPU parity tests of bit packing / unpacking: bit-exact against the CPU oracle.
Cases follow the reference's test/packing/packing.cpp (N = 2048; pack, unpack,
round trip, interleaved) and add ragged sizes and unaligned buffers."""
import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import stream, to_device, to_host

pytestmark = pytest.mark.gpu
PLANAR, INTERLEAVED = cc.ComplexAxisLocation.complex_planar, cc.ComplexAxisLocation.complex_interleaved

SIZES = [2048, 64, 32, 31, 1, 100, 2048 + 17, 1 << 20, (1 << 20) + 40, 4096 * 3 + 64]


@pytest.mark.parametrize("N", SIZES)
def test_pack(N):
    rng = np.random.default_rng(N)
    x = rng.integers(0, 2, N, dtype=np.uint8)
    d_in = to_device(x)
    words = (N + 31) // 32
    d_out = to_device(np.full(words + 4, 0xDEADBEEF, dtype=np.uint32))
    cc.Packing(N, cc.Direction.forward, 0, stream()).Run(d_in.data_ptr(), d_out.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_out, np.uint32)
    assert np.array_equal(got[:words], orc.pack_bits(x))
    assert np.all(got[words:] == 0xDEADBEEF)          # nothing written past the end


def test_pack_any_nonzero_byte_is_one():
    rng = np.random.default_rng(1)
    x = rng.integers(0, 256, 1 << 16, dtype=np.uint8)
    x[rng.random(x.size) < 0.5] = 0
    d_in, d_out = to_device(x), to_device(np.zeros(x.size // 32, dtype=np.uint32))
    cc.Packing(x.size, cc.Direction.forward, 0, stream()).Run(d_in.data_ptr(), d_out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_out, np.uint32), orc.pack_bits(x))


@pytest.mark.parametrize("N", SIZES)
def test_unpack(N):
    rng = np.random.default_rng(N)
    words = (N + 31) // 32
    w = rng.integers(0, 2 ** 32, words, dtype=np.uint32)
    d_in = to_device(w)
    d_out = to_device(np.full(N + 16, 7, dtype=np.uint8))
    cc.Packing(N, cc.Direction.backward, 0, stream()).Run(d_in.data_ptr(), d_out.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_out, np.uint8)
    assert np.array_equal(got[:N], orc.unpack_bits(w, N))
    assert np.all(got[N:] == 7)


@pytest.mark.parametrize("N", [2048, 100, 1 << 18])
def test_round_trip(N):
    rng = np.random.default_rng(N)
    x = rng.integers(0, 2, N, dtype=np.uint8)
    d_in = to_device(x)
    d_packed = to_device(np.zeros((N + 31) // 32, dtype=np.uint32))
    d_out = to_device(np.full(N, 9, dtype=np.uint8))
    cc.Packing(N, cc.Direction.forward, 0, stream()).Run(d_in.data_ptr(), d_packed.data_ptr())
    cc.Packing(N, cc.Direction.backward, 0, stream()).Run(d_packed.data_ptr(), d_out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_out, np.uint8), x)


@pytest.mark.parametrize("N", [2048, 64, 128, 100, 2, 62, 1 << 20, (1 << 20) + 64, (1 << 16) + 2])
def test_pack_interleaved(N):
    rng = np.random.default_rng(N)
    x = rng.integers(0, 2, N, dtype=np.uint8)
    d_in = to_device(x)
    words = (N + 31) // 32
    d_out = to_device(np.full(words + 4, 0xDEADBEEF, dtype=np.uint32))
    cc.Packing(N, cc.Direction.forward, 0, stream(), INTERLEAVED).Run(d_in.data_ptr(), d_out.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_out, np.uint32)
    assert np.array_equal(got[:words], orc.pack_bits(x, orc.INTERLEAVED))
    assert np.all(got[words:] == 0xDEADBEEF)


def test_unaligned_buffers():
    rng = np.random.default_rng(5)
    N = 4096 + 13
    x = rng.integers(0, 2, N + 3, dtype=np.uint8)
    d_in = to_device(x)
    d_out = to_device(np.zeros((N + 31) // 32, dtype=np.uint32))
    cc.Packing(N, cc.Direction.forward, 0, stream()).Run(d_in.data_ptr() + 3, d_out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_out, np.uint32), orc.pack_bits(x[3:].copy()))
    d_bytes = to_device(np.zeros(N + 8, dtype=np.uint8))
    cc.Packing(N, cc.Direction.backward, 0, stream()).Run(d_out.data_ptr(), d_bytes.data_ptr() + 5)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_bytes, np.uint8)[5:5 + N], x[3:])


@pytest.mark.parametrize("offset", [1, 4, 15])
@pytest.mark.parametrize("axis", [PLANAR, INTERLEAVED])
def test_unaligned_large_buffers(offset, axis):
    # buffers at odd addresses take the same wide-access kernels (one 16-byte access at any
    # address), also beyond one grid of blocks' worth of data
    rng = np.random.default_rng(offset)
    N = (1 << 21) + 64 + (13 if axis == PLANAR else 0)
    x = rng.integers(0, 2, N + offset, dtype=np.uint8)
    d_in = to_device(x)
    words = (N + 31) // 32
    d_out = to_device(np.full(words + 2, 0xDEADBEEF, dtype=np.uint32))
    cc.Packing(N, cc.Direction.forward, 0, stream(), axis).Run(d_in.data_ptr() + offset, d_out.data_ptr())
    torch.cuda.synchronize()
    got = to_host(d_out, np.uint32)
    assert np.array_equal(got[:words], orc.pack_bits(x[offset:].copy(), int(axis)))
    assert np.all(got[words:] == 0xDEADBEEF)
    if axis == PLANAR:
        d_bytes = to_device(np.full(N + 32, 9, dtype=np.uint8))
        cc.Packing(N, cc.Direction.backward, 0, stream()).Run(d_out.data_ptr(), d_bytes.data_ptr() + offset)
        torch.cuda.synchronize()
        back = to_host(d_bytes, np.uint8)
        assert np.array_equal(back[offset:offset + N], x[offset:])
        assert np.all(back[:offset] == 9) and np.all(back[offset + N:] == 9)


def test_host_input():
    rng = np.random.default_rng(6)
    N = 2048
    x = rng.integers(0, 2, N, dtype=np.uint8)
    d_out = to_device(np.zeros(N // 32, dtype=np.uint32))
    cc.Packing(N, cc.Direction.forward, 0, stream()).RunHost(x.ctypes.data, d_out.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(to_host(d_out, np.uint32), orc.pack_bits(x))
