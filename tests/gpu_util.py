"""Helpers shared by the GPU parity tests: input generation in the storage
formats of the library, device buffers through torch, and the comparison rules."""
import numpy as np
import torch

import ccglib_amd as cc
import oracle as orc

ORC_TYPE = {cc.ValueType.float16: orc.FLOAT16, cc.ValueType.bfloat16: orc.BFLOAT16,
            cc.ValueType.float8e4m3: orc.FLOAT8E4M3, cc.ValueType.float8e5m2: orc.FLOAT8E5M2,
            cc.ValueType.float32: orc.FLOAT32, cc.ValueType.int1: orc.INT1,
            cc.ValueType.int32: orc.INT32}

# per-element tolerance of the reference's own tests (test/gemm/fpequals.h:15-53)
EPSILON = {cc.ValueType.float8e4m3: 0.125, cc.ValueType.float8e5m2: 0.25,
           cc.ValueType.float16: 0.000976562, cc.ValueType.bfloat16: 0.0078125,
           # the reference runs float32 input as tf32 and tests it with the fp16 epsilon; the
           # products here are true fp32, so the Frobenius bound below is the tight one
           cc.ValueType.float32: 0.000976562}
# relative Frobenius error bound against float64
FROBENIUS = {cc.ValueType.float16: 1e-3, cc.ValueType.bfloat16: 1e-3,
             cc.ValueType.float8e4m3: 2e-2, cc.ValueType.float8e5m2: 2e-2,
             cc.ValueType.float32: 1e-5}


def quantize(x, vtype):
    """float32 array -> storage bit patterns (round to nearest even, fp8 saturating)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    t = torch.from_numpy(x)
    if vtype == cc.ValueType.float32:
        return x
    if vtype == cc.ValueType.float16:
        return x.astype(np.float16).view(np.uint16)
    if vtype == cc.ValueType.bfloat16:
        return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    if vtype == cc.ValueType.float8e4m3:
        return t.clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    if vtype == cc.ValueType.float8e5m2:
        return t.clamp(-57344, 57344).to(torch.float8_e5m2).view(torch.uint8).numpy()
    raise ValueError(vtype)


def dequantize(q, vtype):
    t = torch.from_numpy(np.ascontiguousarray(q))
    if vtype == cc.ValueType.float16:
        return q.view(np.float16).astype(np.float32)
    if vtype == cc.ValueType.bfloat16:
        return t.view(torch.int16).view(torch.bfloat16).to(torch.float32).numpy()
    if vtype == cc.ValueType.float8e4m3:
        return t.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    if vtype == cc.ValueType.float8e5m2:
        return t.view(torch.float8_e5m2).to(torch.float32).numpy()
    if vtype == cc.ValueType.float32:
        return np.asarray(q, dtype=np.float32)
    raise ValueError(vtype)


_SIGNED = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32, np.dtype(np.uint8): np.uint8}


def to_device(a):
    """numpy array -> torch CUDA tensor holding the same bytes."""
    a = np.ascontiguousarray(a)
    if a.dtype in _SIGNED:
        a = a.view(_SIGNED[a.dtype])
    return torch.from_numpy(a).cuda()


def to_host(t, dtype):
    """torch CUDA tensor -> numpy array of `dtype` with the same bytes."""
    return t.cpu().numpy().view(dtype)


def stream():
    return torch.cuda.current_stream().cuda_stream


def device_zeros(nbytes):
    return torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")


def transpose_operand(q, B, rows, K, vtype, axis=cc.ComplexAxisLocation.complex_planar):
    """Runs the library's Transpose with the chunk sizes GetDimensions reports and
    returns the device tensor holding the tiled operand."""
    prec = cc.Precision(vtype, cc.ValueType.int32 if vtype == cc.ValueType.int1 else cc.ValueType.float32)
    mb, nb, kc = cc.GEMM.GetDimensions(prec)
    bits = prec.GetInputBits()
    rp, kp = cc.ceildiv(rows, mb) * mb, cc.ceildiv(K, kc) * kc
    d_in = to_device(q)
    d_out = device_zeros(B * 2 * rp * kp * bits // 8)
    cc.Transpose(B, rows, K, mb, kc, bits, 0, stream(), axis).Run(d_in.data_ptr(), d_out.data_ptr())
    return d_out


def check_float(got, want32, want64, type_in, type_out):
    """got: float array from the GPU; want32: float-accumulating oracle; want64:
    float64 product. Applies the reference's per-element rule against the oracle
    and the relative Frobenius bound against float64."""
    got = got.astype(np.float64)
    narrow = type_out != cc.ValueType.float32
    tol = (100 if narrow else 10) * EPSILON[type_in]
    rel = np.abs(got - want32) / (np.abs(got) + np.abs(want32) + 1.0)
    assert rel.max() <= tol, f"per-element error {rel.max()} > {tol}"
    frob = np.linalg.norm(got - want64) / max(np.linalg.norm(want64), 1e-30)
    bound = FROBENIUS[type_in]
    if narrow:  # the output rounding itself is 2^-11 (half) or 2^-8 (bfloat16) relative
        bound = max(bound, 2.0 ** -8 if type_out == cc.ValueType.bfloat16 else 2.0 ** -10)
    assert frob <= bound, f"relative Frobenius error {frob} > {bound}"
    return frob


def capture_and_replay(make_object, inputs, fill_inputs, out_shape, out_dtype, rounds=3):
    """make_object(stream) -> object with Run(a, b, c); inputs: list of device tensors the
    graph reads; fill_inputs(round) writes new contents into them."""
    side = torch.cuda.Stream()
    obj = make_object(side.cuda_stream)
    d_c = torch.zeros(out_shape, dtype=out_dtype, device="cuda")
    fill_inputs(0)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):           # warm-up outside the capture
        obj.Run(inputs[0].data_ptr(), inputs[1].data_ptr(), d_c.data_ptr())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        obj.Run(inputs[0].data_ptr(), inputs[1].data_ptr(), d_c.data_ptr())
    for r in range(1, rounds + 1):
        fill_inputs(r)
        torch.cuda.synchronize()
        d_c.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = d_c.clone()
        d_c.zero_()
        torch.cuda.synchronize()            # `side` does not wait for the stream zero_() ran on
        with torch.cuda.stream(side):
            obj.Run(inputs[0].data_ptr(), inputs[1].data_ptr(), d_c.data_ptr())
        torch.cuda.synchronize()
        assert torch.equal(got, d_c), "replay %d differs from the eager run" % r
        assert bool(d_c.ne(0).any())
