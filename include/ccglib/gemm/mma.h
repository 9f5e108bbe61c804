// ccglib::mma::GEMM for gfx950: same constructor, Run and GetDimensions as the
// reference class with native HIP handles (include/ccglib/gemm/mma.h:42-50 there),
// implemented as an inline wrapper over the C ABI in ccglib_amd.h.
#ifndef CCGLIB_GEMM_MMA_H_
#define CCGLIB_GEMM_MMA_H_

#include <complex>

#include <hip/hip_runtime.h>

#include <ccglib/common/error.h>
#include <ccglib/common/types.h>

namespace ccglib::mma {

class GEMM {
 public:
  // Note the order: C's memory order comes before A's and B's.
  GEMM(size_t B, size_t M, size_t N, size_t K, hipDevice_t &device, hipStream_t &stream,
       Precision precision, Variant variant = Variant::opt,
       ComplexAxisLocation c_complex_axis_location = ComplexAxisLocation::complex_planar,
       MemOrder c_mem_order = MemOrder::row_major, MemOrder a_mem_order = MemOrder::row_major,
       MemOrder b_mem_order = MemOrder::col_major, std::complex<float> alpha = {1, 0},
       std::complex<float> beta = {0, 0}) {
    detail::check(ccglib_gemm_create(&handle_, B, M, N, K, detail::ordinal(device), stream,
                                     static_cast<ValueType>(precision.input_type),
                                     static_cast<ValueType>(precision.output_type), variant,
                                     c_complex_axis_location, c_mem_order, a_mem_order,
                                     b_mem_order, alpha.real(), alpha.imag(), beta.real(),
                                     beta.imag()));
  }
  GEMM(const GEMM &) = delete;
  GEMM &operator=(const GEMM &) = delete;
  ~GEMM() { ccglib_gemm_destroy(handle_); }

  // Enqueues C = alpha A B^T + beta C on the stream given at construction.
  void Run(hipDeviceptr_t d_a, hipDeviceptr_t d_b, hipDeviceptr_t d_c) {
    detail::check(ccglib_gemm_run(handle_, d_a, d_b, d_c));
  }

  // (m_per_block, n_per_block, k_chunk): chunk sizes of the opt input layout.
  static dim3 GetDimensions(Precision precision, Variant variant = Variant::opt) {
    unsigned m = 0, n = 0, k = 0;
    detail::check(ccglib_gemm_get_dimensions(static_cast<ValueType>(precision.input_type),
                                             static_cast<ValueType>(precision.output_type),
                                             variant, &m, &n, &k));
    return dim3(m, n, k);
  }

 private:
  ccglib_gemm_t handle_ = nullptr;
};

}  // namespace ccglib::mma
#endif  // CCGLIB_GEMM_MMA_H_
