"""ctypes binding of libccglib_amd.so (the C ABI declared in include/ccglib_amd.h)."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# CCGLIB_AMD_LIBRARY may point at another build of the same library
LIB_PATH = os.environ.get("CCGLIB_AMD_LIBRARY") or os.path.join(HERE, "libccglib_amd.so")

_sz, _vp, _i, _f = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_pvp = ctypes.POINTER(ctypes.c_void_p)
_pu = ctypes.POINTER(ctypes.c_uint)

# name -> (restype, argtypes); one entry per function declared in the header
SIGNATURES = {
    "ccglib_last_error": (ctypes.c_char_p, []),
    "ccglib_version": (ctypes.c_char_p, []),
    "ccglib_amd_set_option": (_i, [_i, _sz]),
    "ccglib_amd_get_option": (_i, [_i, ctypes.POINTER(ctypes.c_size_t)]),
    "ccglib_amd_static_scratch_bytes": (_sz, []),
    "ccglib_gemm_create": (_i, [_pvp, _sz, _sz, _sz, _sz, _i, _vp, _i, _i, _i, _i, _i, _i, _i,
                                _f, _f, _f, _f]),
    "ccglib_gemm_run": (_i, [_vp, _vp, _vp, _vp]),
    "ccglib_gemm_kernel_name": (_i, [_vp, ctypes.c_char_p, _sz]),
    "ccglib_gemm_destroy": (_i, [_vp]),
    "ccglib_gemm_get_dimensions": (_i, [_i, _i, _i, _pu, _pu, _pu]),
    "ccglib_transpose_create": (_i, [_pvp, _sz, _sz, _sz, _sz, _sz, _sz, _i, _vp, _i]),
    "ccglib_transpose_run": (_i, [_vp, _vp, _vp]),
    "ccglib_transpose_run_host": (_i, [_vp, _vp, _vp]),
    "ccglib_transpose_run_pair": (_i, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "ccglib_transpose_destroy": (_i, [_vp]),
    "ccglib_packing_create": (_i, [_pvp, _sz, _i, _i, _vp, _i]),
    "ccglib_packing_run": (_i, [_vp, _vp, _vp]),
    "ccglib_packing_run_host": (_i, [_vp, _vp, _vp]),
    "ccglib_packing_destroy": (_i, [_vp]),
    "ccglib_pipeline_create": (_i, [_pvp, _sz, _sz, _sz, _sz, _i, _vp, _i, _i, _i, _i, _i, _i, _i,
                                    _i, _f, _f, _f, _f]),
    "ccglib_pipeline_run": (_i, [_vp, _vp, _vp, _vp]),
    "ccglib_pipeline_run_host": (_i, [_vp, _vp, _vp, _vp]),
    "ccglib_pipeline_reads_in_place": (_i, [_vp, ctypes.POINTER(_i)]),
    "ccglib_pipeline_destroy": (_i, [_vp]),
    "ccglib_pipeline_run_static": (_i, [_sz, _sz, _sz, _sz, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _i,
                                        _f, _f, _f, _f, _vp, _vp, _vp]),
}

_lib = None


def load():
    """Loads the shared library. There is no fallback: without the built HIP
    library every operation of this package raises."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libccglib_amd.so is not built (expected at %s); run "
                "`python -m ccglib_amd.build`" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status):
    if status != 0:
        raise RuntimeError(load().ccglib_last_error().decode())
