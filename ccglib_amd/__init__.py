"""MI355X (gfx950) complex-GEMM library with the ccglib operator interface.

Python mirror of the reference's C++ classes (same names, argument order and
error behaviour), bound to the C ABI of libccglib_amd.so:

    ccglib::mma::GEMM            -> GEMM            (include/ccglib/gemm/mma.h:27-68)
    ccglib::transpose::Transpose -> Transpose       (include/ccglib/transpose/transpose.h:14-54)
    ccglib::packing::Packing     -> Packing         (include/ccglib/packing/packing.h:25-54)
    ccglib::pipeline::Pipeline   -> Pipeline        (include/ccglib/pipeline/pipeline.h:28-73)

Device buffers are passed as integer device addresses (e.g. ``tensor.data_ptr()``),
streams as integer ``hipStream_t`` handles (0 = default stream). Every ``Run``
only enqueues work on the stream. Errors raise ``RuntimeError`` with the
library's message, as the reference throws ``std::runtime_error``.
"""
import contextlib
import ctypes
import enum

from . import _capi

__all__ = ["ValueType", "ComplexAxisLocation", "Direction", "MemOrder", "Variant",
           "Precision", "GEMM", "Transpose", "Packing", "Pipeline", "ceildiv", "version"]


class ValueType(enum.IntEnum):          # include/ccglib/common/value_type.h:14-22
    int1 = 0
    int32 = 1
    bfloat16 = 2
    float8e4m3 = 3
    float8e5m2 = 4
    float16 = 5
    float32 = 6


class ComplexAxisLocation(enum.IntEnum):  # include/ccglib/common/complex_order.h:12
    complex_planar = 0
    complex_interleaved = 1


class Direction(enum.IntEnum):          # include/ccglib/common/direction.h:6
    forward = 0
    backward = 1


class MemOrder(enum.IntEnum):           # include/ccglib/gemm/mem_order.h:6
    row_major = 0
    col_major = 1


class Variant(enum.IntEnum):            # include/ccglib/gemm/variant.h:6
    basic = 0
    opt = 1


_BITS = {ValueType.int1: 1, ValueType.float8e4m3: 8, ValueType.float8e5m2: 8,
         ValueType.bfloat16: 16, ValueType.float16: 16, ValueType.float32: 32,
         ValueType.int32: 32}


class Precision:
    """Input/output value types; output defaults to float32
    (include/ccglib/common/precision.h:13-37)."""

    def __init__(self, input_type, output_type=ValueType.float32):
        self.input_type = ValueType(input_type)
        self.output_type = ValueType(output_type)

    def GetInputBits(self):
        return _BITS[self.input_type]

    def GetOutputBits(self):
        return _BITS[self.output_type]


def _as_precision(p):
    return p if isinstance(p, Precision) else Precision(p)


def ceildiv(a, b):
    """include/ccglib/common/helper.h:6-9"""
    return a // b + (a % b != 0)


def version():
    return _capi.load().ccglib_version().decode()


class Option(enum.IntEnum):
    """Process-wide options of the library (include/ccglib_amd.h; no counterpart in
    the reference). Read when an object is created."""
    int1_popcount = 0
    basic_retile = 1
    host_chunk_bytes = 2
    gemm_block_tile = 3
    expect_unaligned = 4
    pipeline_route = 5


def set_option(option, value):
    _capi.check(_capi.load().ccglib_amd_set_option(int(option), int(value)))


def get_option(option):
    out = ctypes.c_size_t(0)
    _capi.check(_capi.load().ccglib_amd_get_option(int(option), ctypes.byref(out)))
    return out.value


@contextlib.contextmanager
def option(option, value):
    """Sets an option for the duration of a with block."""
    old = get_option(option)
    set_option(option, value)
    try:
        yield
    finally:
        set_option(option, old)


def _ptr(x):
    return ctypes.c_void_p(int(x))


class _Handle:
    _destroy = None

    def __init__(self):
        self._h = ctypes.c_void_p()

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and h.value and _capi is not None and ctypes is not None:
            getattr(_capi.load(), self._destroy)(h)   # (modules are None at interpreter exit)
            self._h = ctypes.c_void_p()


class GEMM(_Handle):
    """C[b] = alpha * A[b] * B[b]^T + beta * C[b] on complex planar data.

    Argument order is that of the reference constructor (note c_mem_order
    before a_mem_order)."""
    _destroy = "ccglib_gemm_destroy"

    def __init__(self, B, M, N, K, device, stream, precision, variant=Variant.opt,
                 c_complex_axis_location=ComplexAxisLocation.complex_planar,
                 c_mem_order=MemOrder.row_major, a_mem_order=MemOrder.row_major,
                 b_mem_order=MemOrder.col_major, alpha=1 + 0j, beta=0j):
        super().__init__()
        precision = _as_precision(precision)
        alpha, beta = complex(alpha), complex(beta)
        _capi.check(_capi.load().ccglib_gemm_create(
            ctypes.byref(self._h), B, M, N, K, int(device), _ptr(stream),
            int(precision.input_type), int(precision.output_type), int(variant),
            int(c_complex_axis_location), int(c_mem_order), int(a_mem_order), int(b_mem_order),
            alpha.real, alpha.imag, beta.real, beta.imag))

    def Run(self, d_a, d_b, d_c):
        _capi.check(_capi.load().ccglib_gemm_run(self._h, _ptr(d_a), _ptr(d_b), _ptr(d_c)))

    def KernelName(self):
        """Which kernel Run launches for 16-byte aligned buffers (no counterpart in
        the reference)."""
        buf = ctypes.create_string_buffer(160)
        _capi.check(_capi.load().ccglib_gemm_kernel_name(self._h, buf, len(buf)))
        return buf.value.decode()

    @staticmethod
    def GetDimensions(precision, variant=Variant.opt):
        """(m_per_block, n_per_block, k_chunk) of the opt layout."""
        precision = _as_precision(precision)
        m, n, k = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_uint()
        _capi.check(_capi.load().ccglib_gemm_get_dimensions(
            int(precision.input_type), int(precision.output_type), int(variant),
            ctypes.byref(m), ctypes.byref(n), ctypes.byref(k)))
        return m.value, n.value, k.value


class Transpose(_Handle):
    _destroy = "ccglib_transpose_destroy"

    def __init__(self, B, M, N, M_chunk, N_chunk, nr_bits, device, stream,
                 input_complex_axis_location=ComplexAxisLocation.complex_planar):
        super().__init__()
        _capi.check(_capi.load().ccglib_transpose_create(
            ctypes.byref(self._h), B, M, N, M_chunk, N_chunk, nr_bits, int(device),
            _ptr(stream), int(input_complex_axis_location)))

    def Run(self, d_input, d_output):
        _capi.check(_capi.load().ccglib_transpose_run(self._h, _ptr(d_input), _ptr(d_output)))

    def RunHost(self, h_input, d_output):
        """Run(const void *h_input, hipDeviceptr_t d_output) of the reference."""
        _capi.check(_capi.load().ccglib_transpose_run_host(self._h, _ptr(h_input),
                                                          _ptr(d_output)))

    @staticmethod
    def RunPair(transpose_a, d_input_a, d_output_a, transpose_b, d_input_b, d_output_b):
        """Both operands of one GEMM, in one kernel launch where they take the
        same kernel (no counterpart in the reference)."""
        _capi.check(_capi.load().ccglib_transpose_run_pair(
            transpose_a._h, _ptr(d_input_a), _ptr(d_output_a),
            transpose_b._h, _ptr(d_input_b), _ptr(d_output_b)))


class Packing(_Handle):
    _destroy = "ccglib_packing_destroy"

    def __init__(self, N, direction, device, stream,
                 input_complex_axis_location=ComplexAxisLocation.complex_planar):
        super().__init__()
        _capi.check(_capi.load().ccglib_packing_create(
            ctypes.byref(self._h), N, int(direction), int(device), _ptr(stream),
            int(input_complex_axis_location)))

    def Run(self, d_input, d_output):
        _capi.check(_capi.load().ccglib_packing_run(self._h, _ptr(d_input), _ptr(d_output)))

    def RunHost(self, h_input, d_output):
        _capi.check(_capi.load().ccglib_packing_run_host(self._h, _ptr(h_input), _ptr(d_output)))


class Pipeline(_Handle):
    _destroy = "ccglib_pipeline_destroy"

    def __init__(self, B, M, N, K, device, stream, input_complex_axis_location,
                 output_complex_axis_location, a_mem_order, b_mem_order, c_mem_order,
                 input_precision, output_precision, variant=Variant.opt, alpha=1 + 0j, beta=0j):
        super().__init__()
        alpha, beta = complex(alpha), complex(beta)
        _capi.check(_capi.load().ccglib_pipeline_create(
            ctypes.byref(self._h), B, M, N, K, int(device), _ptr(stream),
            int(input_complex_axis_location), int(output_complex_axis_location),
            int(a_mem_order), int(b_mem_order), int(c_mem_order), int(input_precision),
            int(output_precision), int(variant), alpha.real, alpha.imag, beta.real, beta.imag))

    def Run(self, d_a, d_b, d_c):
        _capi.check(_capi.load().ccglib_pipeline_run(self._h, _ptr(d_a), _ptr(d_b), _ptr(d_c)))

    def ReadsInPlace(self):
        """Whether the GEMM of this pipeline reads the caller's rows in place (no transposes);
        no counterpart in the reference (see Option.pipeline_route)."""
        out = ctypes.c_int(0)
        _capi.check(_capi.load().ccglib_pipeline_reads_in_place(self._h, ctypes.byref(out)))
        return bool(out.value)

    def RunHost(self, h_a, h_b, h_c):
        _capi.check(_capi.load().ccglib_pipeline_run_host(self._h, _ptr(h_a), _ptr(h_b),
                                                         _ptr(h_c)))


def static_scratch_bytes():
    """Size of the static device array behind pipeline_run_static in the loaded library
    (build option CCGLIB_AMD_STATIC_SCRATCH_BYTES, 32 MiB unless the build says otherwise)."""
    return _capi.load().ccglib_amd_static_scratch_bytes()


def pipeline_run_static(B, M, N, K, device, stream, input_complex_axis_location,
                        output_complex_axis_location, a_mem_order, b_mem_order, c_mem_order,
                        input_precision, output_precision, variant, alpha, beta, d_a, d_b, d_c):
    """The pipeline as one stateless call that allocates nothing: its scratch is a static
    device array (ccglib_pipeline_run_static; no counterpart in the reference)."""
    alpha, beta = complex(alpha), complex(beta)
    _capi.check(_capi.load().ccglib_pipeline_run_static(
        B, M, N, K, device, _ptr(stream), int(input_complex_axis_location),
        int(output_complex_axis_location), int(a_mem_order), int(b_mem_order), int(c_mem_order),
        int(input_precision), int(output_precision), int(variant), alpha.real, alpha.imag,
        beta.real, beta.imag, _ptr(d_a), _ptr(d_b), _ptr(d_c)))
