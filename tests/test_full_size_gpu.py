"""The reference's benchmark configurations at their full sizes. The CPU oracle cannot finish these
in reasonable time, so they are checked through properties that do not depend on size:
one batch against an independent float64 (or exact +-1) product computed by torch on
the GPU, CPU-oracle spot blocks with the full K, bit-exact transposes against torch's
own permutation, and pack -> unpack round trips."""
import numpy as np
import pytest
import torch

import ccglib_amd as cc
import oracle as orc
from gpu_util import ORC_TYPE, stream

pytestmark = pytest.mark.gpu
VT, AX, MO = cc.ValueType, cc.ComplexAxisLocation, cc.MemOrder


def tiled(x, B, rows, K, vtype, axis=AX.complex_planar):
    prec = cc.Precision(vtype, VT.int32 if vtype == VT.int1 else VT.float32)
    mb, nb, kc = cc.GEMM.GetDimensions(prec)
    bits = prec.GetInputBits()
    rp, kp = cc.ceildiv(rows, mb) * mb, cc.ceildiv(K, kc) * kc
    out = torch.empty(B * 2 * rp * kp * bits // 8, dtype=torch.uint8, device="cuda")
    cc.Transpose(B, rows, K, mb, kc, bits, 0, stream(), axis).Run(x.data_ptr(), out.data_ptr())
    return out


def rel_err_vs_float64(a, b, c, batch, interleaved=False):
    if interleaved:
        a64 = torch.complex(a[batch, ..., 0].double(), a[batch, ..., 1].double())
        b64 = torch.complex(b[batch, ..., 0].double(), b[batch, ..., 1].double())
    else:
        a64 = torch.complex(a[batch, 0].double(), a[batch, 1].double())
        b64 = torch.complex(b[batch, 0].double(), b[batch, 1].double())
    ref = a64 @ b64.T
    got = torch.complex(c[batch, 0].double(), c[batch, 1].double())
    return float((got - ref).norm() / ref.norm())


def oracle_spot_block(a_planar_np, b_planar_np, c, batch, M, N, K, vtype, m0, n0, size=32):
    """CPU oracle on a size x size block of C with the full K; per-element rule of the
    reference's tests (test/gemm/fpequals.h:38-53)."""
    a_blk = np.ascontiguousarray(a_planar_np[:, m0:m0 + size, :]).reshape(-1)
    b_blk = np.ascontiguousarray(b_planar_np[:, n0:n0 + size, :]).reshape(-1)
    want = orc.gemm(a_blk, b_blk, size, size, K, ORC_TYPE[vtype])[0]
    got = c[batch, :, m0:m0 + size, n0:n0 + size].float().cpu().numpy()
    eps = {VT.float16: 2.0 ** -10, VT.bfloat16: 2.0 ** -7, VT.float8e4m3: 0.125, VT.float8e5m2: 0.25}[vtype]
    rel = np.abs(got - want) / (np.abs(got) + np.abs(want) + 1.0)
    assert rel.max() <= 10 * eps


def test_beamformer_fp16():
    # B=64 M=512 N=4096 K=576, interleaved in -> Transpose -> opt GEMM -> planar fp32
    B, M, N, K = 64, 512, 4096, 576
    gen = torch.Generator(device="cuda").manual_seed(2)
    phase = torch.rand((B, M, K), device="cuda", generator=gen) * (2 * np.pi)
    a = torch.stack([torch.cos(phase), torch.sin(phase)], dim=-1).half().contiguous()
    b = torch.randn((B, N, K, 2), device="cuda", generator=gen).half().contiguous()
    a_t = tiled(a, B, M, K, VT.float16, AX.complex_interleaved)
    b_t = tiled(b, B, N, K, VT.float16, AX.complex_interleaved)
    # the transposes, bit-exact against torch's own permutation (whole tensors)
    want_a = a.view(B, M // 128, 128, K // 32, 32, 2).permute(0, 1, 3, 5, 2, 4).contiguous()
    assert torch.equal(a_t.view(torch.float16), want_a.view(-1))
    want_b = b.view(B, N // 128, 128, K // 32, 32, 2).permute(0, 1, 3, 5, 2, 4).contiguous()
    assert torch.equal(b_t.view(torch.float16), want_b.view(-1))
    del want_a, want_b
    c = torch.full((B, 2, M, N), float("nan"), device="cuda")
    cc.GEMM(B, M, N, K, 0, stream(), VT.float16, cc.Variant.opt).Run(
        a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    assert torch.isfinite(c).all()
    for batch in (0, 31, 63):
        assert rel_err_vs_float64(a, b, c, batch, interleaved=True) <= 1e-3
    a_np = a[5].permute(2, 0, 1).contiguous().cpu().numpy().view(np.uint16)
    b_np = b[5].permute(2, 0, 1).contiguous().cpu().numpy().view(np.uint16)
    oracle_spot_block(a_np, b_np, c, 5, M, N, K, VT.float16, 480, 4064)
    oracle_spot_block(a_np, b_np, c, 5, M, N, K, VT.float16, 0, 1000)


@pytest.mark.parametrize("tout", [VT.float32, VT.bfloat16])
def test_square_bf16(tout):
    # B=1 M=N=K=8192 planar; fp32 output and bf16-downcast output
    M = N = K = 8192
    gen = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randn((1, 2, M, K), device="cuda", generator=gen).bfloat16()
    b = torch.randn((1, 2, N, K), device="cuda", generator=gen).bfloat16()
    a_t, b_t = tiled(a, 1, M, K, VT.bfloat16), tiled(b, 1, N, K, VT.bfloat16)
    dt = torch.float32 if tout == VT.float32 else torch.bfloat16
    c = torch.empty((1, 2, M, N), dtype=dt, device="cuda")
    cc.GEMM(1, M, N, K, 0, stream(), cc.Precision(VT.bfloat16, tout), cc.Variant.opt).Run(
        a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    err = rel_err_vs_float64(a, b, c, 0)
    assert err <= (1e-3 if tout == VT.float32 else 2.0 ** -8)
    if tout == VT.float32:
        # the basic variant on the planar input gives the same numbers up to fp32 rounding order
        c2 = torch.empty_like(c)
        cc.GEMM(1, M, N, K, 0, stream(), VT.bfloat16, cc.Variant.basic).Run(
            a.data_ptr(), b.data_ptr(), c2.data_ptr())
        torch.cuda.synchronize()
        assert float((c - c2).norm() / c.norm()) <= 1e-5
        a_np = a[0].view(torch.int16).cpu().numpy().view(np.uint16)
        b_np = b[0].view(torch.int16).cpu().numpy().view(np.uint16)
        oracle_spot_block(a_np, b_np, c, 0, M, N, K, VT.bfloat16, 8160, 4096)


@pytest.mark.parametrize("vtype,tdt,fmax", [(VT.float8e4m3, torch.float8_e4m3fn, 448.0),
                                            (VT.float8e5m2, torch.float8_e5m2, 57344.0)])
def test_fp8(vtype, tdt, fmax):
    # B=16 M=N=4096 K=8192 planar; per-matrix scale into the fp8 range, then quantised
    B, M, N, K = 16, 4096, 4096, 8192
    gen = torch.Generator(device="cuda").manual_seed(4)
    mats = []
    for rows in (M, N):
        x = torch.randn((B, 2, rows, K), device="cuda", generator=gen)
        mats.append((x * (fmax / float(x.abs().max()))).clamp_(-fmax, fmax).to(tdt))
        del x
    a, b = mats
    a_t, b_t = tiled(a, B, M, K, vtype), tiled(b, B, N, K, vtype)
    c = torch.empty((B, 2, M, N), device="cuda")
    cc.GEMM(B, M, N, K, 0, stream(), vtype, cc.Variant.opt).Run(a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    for batch in (0, 15):
        assert rel_err_vs_float64(a, b, c, batch) <= 2e-2
    a_np = a[7].view(torch.uint8).cpu().numpy()
    b_np = b[7].view(torch.uint8).cpu().numpy()
    oracle_spot_block(a_np, b_np, c, 7, M, N, K, vtype, 4064, 0, size=16)


def test_correlator_int1():
    # B=32 M=N=1024 K=65536: one byte per sample -> Packing -> Transpose -> 1-bit GEMM
    B, M, N, K = 32, 1024, 1024, 65536
    gen = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(0, 2, (B, 2, M, K), device="cuda", generator=gen, dtype=torch.uint8)
    b = torch.randint(0, 2, (B, 2, N, K), device="cuda", generator=gen, dtype=torch.uint8)
    n_samples = a.numel()                      # 2^32: the index arithmetic must be 64-bit
    assert n_samples == 1 << 32
    a_p = torch.empty(n_samples // 32, dtype=torch.int32, device="cuda")
    b_p = torch.empty(n_samples // 32, dtype=torch.int32, device="cuda")
    cc.Packing(n_samples, cc.Direction.forward, 0, stream()).Run(a.data_ptr(), a_p.data_ptr())
    cc.Packing(n_samples, cc.Direction.forward, 0, stream()).Run(b.data_ptr(), b_p.data_ptr())
    # packing, bit-exact against torch on the whole tensor
    w = (1 << torch.arange(8, device="cuda", dtype=torch.int32)).to(torch.uint8)
    want_bytes = (a.view(-1, 8) * w).sum(dim=1, dtype=torch.uint8)
    assert torch.equal(a_p.view(torch.uint8), want_bytes)
    del want_bytes
    # round trip back to bytes
    back = torch.empty_like(a)
    cc.Packing(n_samples, cc.Direction.backward, 0, stream()).Run(a_p.data_ptr(), back.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(back, a)
    del back
    a_t, b_t = tiled(a_p, B, M, K, VT.int1), tiled(b_p, B, N, K, VT.int1)
    c = torch.empty((B, 2, M, N), dtype=torch.int32, device="cuda")
    cc.GEMM(B, M, N, K, 0, stream(), cc.Precision(VT.int1, VT.int32), cc.Variant.opt).Run(
        a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    # bit 1 = +1, bit 0 = -1: exact integer product in fp32 (|sums| <= 2K < 2^24), every batch
    for batch in range(B):
        sa, sb = a[batch].float() * 2 - 1, b[batch].float() * 2 - 1
        re = sa[0] @ sb[0].T - sa[1] @ sb[1].T
        im = sa[0] @ sb[1].T + sa[1] @ sb[0].T
        assert torch.equal(c[batch, 0].float(), re) and torch.equal(c[batch, 1].float(), im)
    # CPU oracle spot block with the full K
    a_np = a_p.view(B, 2, M, K // 32)[3][:, 100:116].contiguous().cpu().numpy().view(np.uint32)
    b_np = b_p.view(B, 2, N, K // 32)[3][:, 900:916].contiguous().cpu().numpy().view(np.uint32)
    want = orc.gemm(a_np.reshape(-1), b_np.reshape(-1), 16, 16, K, orc.INT1, orc.INT32,
                    c_in=np.zeros(2 * 16 * 16, np.int32))[0]
    assert np.array_equal(c[3, :, 100:116, 900:916].cpu().numpy(), want)


def complex_c(c, batch, interleaved):
    if interleaved:
        return torch.complex(c[batch, ..., 0].double(), c[batch, ..., 1].double())
    return torch.complex(c[batch, 0].double(), c[batch, 1].double())


@pytest.mark.parametrize("c_axis", [AX.complex_planar, AX.complex_interleaved])
def test_beamformer_fp16_alpha_beta(c_axis):
    """The beamformer shape with beta != 0: the kernel reads the 1 GiB C it then
    overwrites. Three batches against complex128."""
    B, M, N, K = 64, 512, 4096, 576
    alpha, beta = 0.5 + 0.25j, -0.75 + 0.5j
    il = c_axis == AX.complex_interleaved
    gen = torch.Generator(device="cuda").manual_seed(12)
    a = torch.randn((B, 2, M, K), device="cuda", generator=gen).half()
    b = torch.randn((B, 2, N, K), device="cuda", generator=gen).half()
    c = torch.randn((B, M, N, 2) if il else (B, 2, M, N), device="cuda", generator=gen)
    keep = {batch: complex_c(c, batch, il) for batch in (0, 37, 63)}
    a_t, b_t = tiled(a, B, M, K, VT.float16), tiled(b, B, N, K, VT.float16)
    cc.GEMM(B, M, N, K, 0, stream(), VT.float16, cc.Variant.opt, c_axis, MO.row_major, MO.row_major,
            MO.col_major, alpha, beta).Run(a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    for batch, c_in in keep.items():
        a64 = torch.complex(a[batch, 0].double(), a[batch, 1].double())
        b64 = torch.complex(b[batch, 0].double(), b[batch, 1].double())
        want = alpha * (a64 @ b64.T) + beta * c_in
        assert float((complex_c(c, batch, il) - want).norm() / want.norm()) <= 1e-3


def one_batch_alone(a_t, b_t, batch, B, M, N, K, vtype, c_axis):
    """The same product for one batch by itself, from the tiles of that batch: the
    numbers a batched launch must reproduce bit for bit wherever the batch sits."""
    c1 = torch.empty((M, N, 2) if c_axis == AX.complex_interleaved else (2, M, N), device="cuda")
    cc.GEMM(1, M, N, K, 0, stream(), vtype, cc.Variant.opt, c_axis).Run(
        a_t.data_ptr() + batch * (a_t.numel() // B), b_t.data_ptr() + batch * (b_t.numel() // B),
        c1.data_ptr())
    torch.cuda.synchronize()
    return c1


def check_batches(a, b, a_t, b_t, c, B, M, N, K, vtype, c_axis, bound):
    il = c_axis == AX.complex_interleaved
    for batch in (0, B // 2, B - 1):
        a64 = torch.complex(a[batch, 0].double(), a[batch, 1].double())
        b64 = torch.complex(b[batch, 0].double(), b[batch, 1].double())
        want = a64 @ b64.T
        del a64, b64
        err = float((complex_c(c, batch, il) - want).norm() / want.norm())
        del want
        assert err <= bound, (batch, err)
        assert torch.equal(c[batch], one_batch_alone(a_t, b_t, batch, B, M, N, K, vtype, c_axis)), batch


# Offsets beyond 2^32 bytes and 2^31 elements. Block tiles (option GEMM_BLOCK_TILE): 1 is
# 256 x 128, 2 is 128 x 128, 3 is 192 x 256 (16-bit input and planar C only; elsewhere
# it means the default choice).
@pytest.mark.parametrize("block_tile", [1, 2, 3])
@pytest.mark.parametrize("c_axis", [AX.complex_planar, AX.complex_interleaved])
@pytest.mark.parametrize("vtype,tdt,bound", [(VT.float16, torch.float16, 1e-3),
                                             (VT.float8e4m3, torch.float8_e4m3fn, 2e-2)])
def test_c_larger_than_4_gib(vtype, tdt, bound, c_axis, block_tile):
    B, M, N, K = 5, 16384, 16384, 64          # C: 5 x 2 GiB, 2.7e9 elements
    cc.set_option(cc.Option.gemm_block_tile, block_tile)
    gen = torch.Generator(device="cuda").manual_seed(13)
    a = torch.randn((B, 2, M, K), device="cuda", generator=gen).to(tdt)
    b = torch.randn((B, 2, N, K), device="cuda", generator=gen).to(tdt)
    a_t, b_t = tiled(a, B, M, K, vtype), tiled(b, B, N, K, vtype)
    il = c_axis == AX.complex_interleaved
    c = torch.full((B, M, N, 2) if il else (B, 2, M, N), float("nan"), device="cuda")
    assert c.numel() > 2 ** 31
    cc.GEMM(B, M, N, K, 0, stream(), vtype, cc.Variant.opt, c_axis).Run(
        a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    cc.set_option(cc.Option.gemm_block_tile, 0)
    check_batches(a, b, a_t, b_t, c, B, M, N, K, vtype, c_axis, bound)


@pytest.mark.parametrize("block_tile", [1, 2, 3])
@pytest.mark.parametrize("c_axis", [AX.complex_planar, AX.complex_interleaved])
@pytest.mark.parametrize("vtype,tdt,N,bound", [(VT.float16, torch.float16, 4096, 1e-3),
                                               (VT.float8e4m3, torch.float8_e4m3fn, 8192, 2e-2)])
def test_tiled_operand_larger_than_4_gib(vtype, tdt, N, bound, c_axis, block_tile):
    B, M, K = 3, 128, 98304                   # the N-row operand: 4.8e9 bytes, > 2^31 elements
    cc.set_option(cc.Option.gemm_block_tile, block_tile)
    gen = torch.Generator(device="cuda").manual_seed(14)
    a = torch.randn((B, 2, M, K), device="cuda", generator=gen).to(tdt)
    b = torch.empty((B, 2, N, K), dtype=tdt, device="cuda")
    for batch in range(B):                    # in pieces: the float32 draw is 4 x the size
        b[batch] = torch.randn((2, N, K), device="cuda", generator=gen).to(tdt)
    a_t, b_t = tiled(a, B, M, K, vtype), tiled(b, B, N, K, vtype)
    assert b_t.numel() > 2 ** 32 and b.numel() > 2 ** 31
    # the transpose itself, bit-exact, at the far end of the operand
    kc = 64 // b.element_size()
    want_last = b[B - 1].view(torch.uint8 if b.element_size() == 1 else torch.int16) \
        .view(2, N // 128, 128, K // kc, kc).permute(1, 3, 0, 2, 4).contiguous().view(-1)
    got_last = b_t.view(want_last.dtype)[(B - 1) * want_last.numel():]
    assert torch.equal(got_last, want_last)
    del want_last
    il = c_axis == AX.complex_interleaved
    c = torch.full((B, M, N, 2) if il else (B, 2, M, N), float("nan"), device="cuda")
    cc.GEMM(B, M, N, K, 0, stream(), vtype, cc.Variant.opt, c_axis).Run(
        a_t.data_ptr(), b_t.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    cc.set_option(cc.Option.gemm_block_tile, 0)
    check_batches(a, b, a_t, b_t, c, B, M, N, K, vtype, c_axis, bound)
