// ccglib::transpose::Transpose for gfx950 (reference:
// include/ccglib/transpose/transpose.h:26-31), an inline wrapper over the C ABI.
#ifndef CCGLIB_TRANSPOSE_TRANSPOSE_H_
#define CCGLIB_TRANSPOSE_TRANSPOSE_H_

#include <hip/hip_runtime.h>

#include <ccglib/common/error.h>
#include <ccglib/common/types.h>

namespace ccglib::transpose {

class Transpose {
 public:
  Transpose(size_t B, size_t M, size_t N, size_t M_chunk, size_t N_chunk, size_t nr_bits,
            hipDevice_t &device, hipStream_t &stream,
            ComplexAxisLocation input_complex_axis_location = ComplexAxisLocation::complex_planar) {
    detail::check(ccglib_transpose_create(&handle_, B, M, N, M_chunk, N_chunk, nr_bits,
                                          detail::ordinal(device), stream,
                                          input_complex_axis_location));
  }
  Transpose(const Transpose &) = delete;
  Transpose &operator=(const Transpose &) = delete;
  ~Transpose() { ccglib_transpose_destroy(handle_); }

  void Run(hipDeviceptr_t d_input, hipDeviceptr_t d_output) {
    detail::check(ccglib_transpose_run(handle_, d_input, d_output));
  }
  // Host input: copied to the device on the stream, then transposed.
  void Run(const void *h_input, hipDeviceptr_t d_output) {
    detail::check(ccglib_transpose_run_host(handle_, h_input, d_output));
  }

 private:
  ccglib_transpose_t handle_ = nullptr;
};

}  // namespace ccglib::transpose
#endif  // CCGLIB_TRANSPOSE_TRANSPOSE_H_
