// Every instantiation of the one-wave-per-SIMD GEMM kernel that the library
// launches, and nothing else: tests/test_kernel_asm.py compiles this file to
// assembly and scans it (see there).
#define CCGLIB_GEMM_MFMA_PART 99   // none of gemm_mfma.hip's own instantiations
#include "../../ccglib_amd/csrc/gemm_mfma.hip"

namespace ccglib_amd {
namespace {
#define CCGLIB_WIDE(...) \
  template __global__ void complex_gemm_mfma_wide<__VA_ARGS__>(const KernelArgs);
// (type in, type out, interleaved rows, alpha)
CCGLIB_WIDE(kFloat16, kFloat32, false, false)
CCGLIB_WIDE(kFloat16, kFloat32, false, true)
CCGLIB_WIDE(kFloat16, kFloat32, true, false)
CCGLIB_WIDE(kFloat16, kFloat32, true, true)
CCGLIB_WIDE(kFloat16, kFloat16, false, false)
CCGLIB_WIDE(kFloat16, kFloat16, false, true)
CCGLIB_WIDE(kFloat16, kFloat16, true, false)
CCGLIB_WIDE(kFloat16, kFloat16, true, true)
CCGLIB_WIDE(kBfloat16, kFloat32, false, false)
CCGLIB_WIDE(kBfloat16, kFloat32, false, true)
CCGLIB_WIDE(kBfloat16, kFloat32, true, false)
CCGLIB_WIDE(kBfloat16, kFloat32, true, true)
CCGLIB_WIDE(kBfloat16, kBfloat16, false, false)
CCGLIB_WIDE(kBfloat16, kBfloat16, false, true)
CCGLIB_WIDE(kBfloat16, kBfloat16, true, false)
CCGLIB_WIDE(kBfloat16, kBfloat16, true, true)
#undef CCGLIB_WIDE
}  // namespace
}  // namespace ccglib_amd
