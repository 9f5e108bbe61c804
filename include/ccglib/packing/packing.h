// ccglib::packing::Packing for gfx950 (reference:
// include/ccglib/packing/packing.h:35-40), an inline wrapper over the C ABI.
#ifndef CCGLIB_PACKING_PACKING_H_
#define CCGLIB_PACKING_PACKING_H_

#include <hip/hip_runtime.h>

#include <ccglib/common/error.h>
#include <ccglib/common/types.h>

namespace ccglib::packing {

class Packing {
 public:
  Packing(size_t N, Direction direction, hipDevice_t &device, hipStream_t &stream,
          ComplexAxisLocation input_complex_axis_location = ComplexAxisLocation::complex_planar) {
    detail::check(ccglib_packing_create(&handle_, N, direction, detail::ordinal(device), stream,
                                        input_complex_axis_location));
  }
  Packing(const Packing &) = delete;
  Packing &operator=(const Packing &) = delete;
  ~Packing() { ccglib_packing_destroy(handle_); }

  void Run(hipDeviceptr_t d_input, hipDeviceptr_t d_output) {
    detail::check(ccglib_packing_run(handle_, d_input, d_output));
  }
  void Run(unsigned char *h_input, hipDeviceptr_t d_output) {
    detail::check(ccglib_packing_run_host(handle_, h_input, d_output));
  }

 private:
  ccglib_packing_t handle_ = nullptr;
};

}  // namespace ccglib::packing
#endif  // CCGLIB_PACKING_PACKING_H_
