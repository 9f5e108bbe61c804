// ccglib::pipeline::Pipeline for gfx950 (reference:
// include/ccglib/pipeline/pipeline.h:44-54), an inline wrapper over the C ABI.
#ifndef CCGLIB_PIPELINE_PIPELINE_H_
#define CCGLIB_PIPELINE_PIPELINE_H_

#include <complex>

#include <hip/hip_runtime.h>

#include <ccglib/common/error.h>
#include <ccglib/common/types.h>

namespace ccglib::pipeline {

class Pipeline {
 public:
  Pipeline(size_t B, size_t M, size_t N, size_t K, hipDevice_t &device, hipStream_t &stream,
           ComplexAxisLocation input_complex_axis_location,
           ComplexAxisLocation output_complex_axis_location, mma::MemOrder a_mem_order,
           mma::MemOrder b_mem_order, mma::MemOrder c_mem_order, ValuePrecision input_precision,
           ValuePrecision output_precision, mma::Variant variant = mma::Variant::opt,
           std::complex<float> alpha = {1, 0}, std::complex<float> beta = {0, 0}) {
    detail::check(ccglib_pipeline_create(
        &handle_, B, M, N, K, detail::ordinal(device), stream, input_complex_axis_location,
        output_complex_axis_location, a_mem_order, b_mem_order, c_mem_order,
        static_cast<ValueType>(input_precision), static_cast<ValueType>(output_precision), variant,
        alpha.real(), alpha.imag(), beta.real(), beta.imag()));
  }
  Pipeline(const Pipeline &) = delete;
  Pipeline &operator=(const Pipeline &) = delete;
  ~Pipeline() { ccglib_pipeline_destroy(handle_); }

  // Device buffers: [pack] -> [transpose] -> GEMM on the stream, no synchronisation.
  void Run(hipDeviceptr_t d_a, hipDeviceptr_t d_b, hipDeviceptr_t d_c) {
    detail::check(ccglib_pipeline_run(handle_, d_a, d_b, d_c));
  }
  // Host buffers: copies in, runs, copies C back and synchronises the stream
  // (the reference offers this for its own host-memory class only).
  void RunHost(const void *h_a, const void *h_b, void *h_c) {
    detail::check(ccglib_pipeline_run_host(handle_, h_a, h_b, h_c));
  }

 private:
  ccglib_pipeline_t handle_ = nullptr;
};

}  // namespace ccglib::pipeline
#endif  // CCGLIB_PIPELINE_PIPELINE_H_
