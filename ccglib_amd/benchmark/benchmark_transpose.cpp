// Transpose benchmark with the command line and the output of the reference's
// benchmark/benchmark_transpose.cpp (options :16-42, "#M,N,runtime_ms,gbytes"
// :215-221, gbytes = 2 * bytes / t :268-270), on plain HIP.
#include <iomanip>

#include "bench_common.h"

int main(int argc, const char *argv[]) {
  bench::Options opt(argv[0], "Transpose benchmark");
  opt.add("b", "Size of batch axis", "1");
  opt.add("m", "Size(s) of M axis", "", true);
  opt.add("n", "Size(s) of N axis", "", true);
  opt.add_flag("pad", "Pad input when not multiple of tile size");
  opt.add("nr_benchmarks", "Number of benchmarks", "1");
  opt.add("benchmark_duration", "Approximate benchmark duration (seconds)", "4");
  opt.add_flag("csv", "Format output to CSV");
  opt.add("precision", "GEMM precision (float32, float16, bfloat16, float8e4m3, float8e5m2 or int1)", "", true);
  opt.add("variant", "GEMM kernel variant (basic or opt)", "opt");
  opt.add("complex_axis", "Location of complex axis (planar or interleaved)", "planar");
  opt.add("device", "GPU device ID", "0");
  opt.parse(argc, argv);

  try {
    const size_t B = opt.size("b");
    std::vector<size_t> M_in = opt.sizes("m"), N_in = opt.sizes("n");
    const auto &names = bench::precision_names();
    if (!names.count(opt.str("precision"))) {
      std::cerr << "Invalid precision provided: " << opt.str("precision") << std::endl;
      return EXIT_FAILURE;
    }
    const ccglib::ValueType type = names.at(opt.str("precision"));
    const ccglib::Precision precision(type, type == ccglib::int1 ? ccglib::int32 : ccglib::float32);
    const std::map<std::string, ccglib::mma::Variant> variants{{"basic", ccglib::mma::basic},
                                                               {"opt", ccglib::mma::opt}};
    const std::map<std::string, ccglib::ComplexAxisLocation> axes{
        {"planar", ccglib::complex_planar}, {"interleaved", ccglib::complex_interleaved}};
    const ccglib::mma::Variant variant = variants.at(opt.str("variant"));
    const ccglib::ComplexAxisLocation axis = axes.at(opt.str("complex_axis"));

    const size_t count = std::max(M_in.size(), N_in.size());
    bench::broadcast(M_in, count);
    bench::broadcast(N_in, count);
    if (M_in.size() != count || N_in.size() != count) throw std::runtime_error("m, n must be the same length");
    const size_t nr_benchmarks = opt.size("nr_benchmarks");
    const float duration = opt.real("benchmark_duration");
    std::cerr << "Estimated benchmark duration: " << nr_benchmarks * duration * (count + 1) << " s" << std::endl;

    bench::Gpu gpu((unsigned)opt.size("device"));
    const dim3 tile = ccglib::mma::GEMM::GetDimensions(precision, variant);
    const size_t bits = precision.GetInputBits();
    std::vector<size_t> M = M_in, N = N_in;
    if (opt.flag("pad")) {
      for (size_t i = 0; i < count; ++i) {
        M[i] = bench::align(M_in[i], tile.x);
        N[i] = bench::align(N_in[i], tile.z);
      }
    } else if (bits == 1) {
      // rows of packed samples are whole 32-bit words
      for (size_t i = 0; i < count; ++i) {
        if (N[i] % 32 != 0) throw std::runtime_error("all n must be a multiple of 32");
      }
    }
    size_t in_elems = 0, out_elems = 0;
    for (size_t i = 0; i < count; ++i) {
      in_elems = std::max(in_elems, M[i] * N[i]);
      out_elems = std::max(out_elems, bench::align(M[i], tile.x) * bench::align(N[i], tile.z));
    }
    hipDeviceptr_t d_in = gpu.alloc(B * 2 * in_elems * bits / 8, 0xAA);
    hipDeviceptr_t d_out = gpu.alloc(B * 2 * out_elems * bits / 8, 0xBB);

    const bool csv = opt.flag("csv");
    if (csv) std::cout << "#M,N,runtime_ms,gbytes" << std::endl;
    for (size_t bench_nr = 0; bench_nr < nr_benchmarks; ++bench_nr) {
      for (size_t i = 0; i < count; ++i) {
        ccglib::transpose::Transpose transpose(B, M[i], N[i], tile.x, tile.z, bits, gpu.device, gpu.stream, axis);
        const double ms = gpu.measure([&] { transpose.Run(d_in, d_out); }, duration, bench_nr == 0 && i == 0);
        const size_t bytes = B * 2 * M[i] * N[i] * bits / 8;
        const double gbytes = 2.0 * (double)bytes / ms * 1e-6;
        if (csv) {
          std::cout << M_in[i] << "," << N_in[i] << "," << ms << "," << gbytes << std::endl;
        } else {
          const std::string shape = std::to_string(M_in[i]) + "x" + std::to_string(N_in[i]);
          std::cout << std::setw(20) << shape << " " << std::setw(7) << ms << " ms, " << std::setw(7) << gbytes
                    << " GByte/s" << std::endl;
        }
      }
    }
  } catch (const std::exception &e) {
    std::cerr << "benchmark_transpose: " << e.what() << std::endl;
    return EXIT_FAILURE;
  }
  return EXIT_SUCCESS;
}
