// GEMM benchmark with the command line and the output of the reference's
// benchmark/benchmark_gemm.cpp (options :16-47, "#M,N,K,runtime_ms,tops" :247-252,
// tops = 8 B M N K / t :79-82), on plain HIP. Added: bfloat16 as a precision name.
#include <iomanip>

#include "bench_common.h"

int main(int argc, const char *argv[]) {
  bench::Options opt(argv[0], "GEMM benchmark");
  opt.add("b", "Size of batch axis", "1");
  opt.add("m", "Size(s) of M axis", "", true);
  opt.add("n", "Size(s) of N axis", "", true);
  opt.add("k", "Size(s) of K axis", "", true);
  opt.add_flag("pad", "Pad input when not multiple of tile size");
  opt.add("nr_benchmarks", "Number of benchmarks", "1");
  opt.add("benchmark_duration", "Approximate benchmark duration (seconds)", "4");
  opt.add_flag("csv", "Format output to CSV");
  opt.add("precision_in", "GEMM input precision (float32, float16, bfloat16, float8e4m3, float8e5m2, or int1)",
          "float32", true);
  opt.add("precision_out", "GEMM output precision (float32, float16, bfloat16 or int32)", "float32");
  opt.add("variant", "GEMM kernel variant (basic or opt)", "opt");
  opt.add("complex_axis", "Location of complex axis of the output (planar or interleaved)", "planar");
  opt.add("device", "GPU device ID", "0");
  opt.parse(argc, argv);

  try {
    const size_t B = opt.size("b");
    std::vector<size_t> M_in = opt.sizes("m"), N_in = opt.sizes("n"), K_in = opt.sizes("k");
    const auto &names = bench::precision_names();
    if (!names.count(opt.str("precision_in")) || !names.count(opt.str("precision_out"))) {
      std::cerr << "Invalid precision provided: input=" << opt.str("precision_in")
                << ", output=" << opt.str("precision_out") << std::endl;
      return EXIT_FAILURE;
    }
    const ccglib::Precision precision(names.at(opt.str("precision_in")), names.at(opt.str("precision_out")));
    const std::map<std::string, ccglib::mma::Variant> variants{{"basic", ccglib::mma::basic},
                                                               {"opt", ccglib::mma::opt}};
    const std::map<std::string, ccglib::ComplexAxisLocation> axes{
        {"planar", ccglib::complex_planar}, {"interleaved", ccglib::complex_interleaved}};
    const ccglib::mma::Variant variant = variants.at(opt.str("variant"));
    const ccglib::ComplexAxisLocation axis = axes.at(opt.str("complex_axis"));

    const size_t count = std::max({M_in.size(), N_in.size(), K_in.size()});
    bench::broadcast(M_in, count);
    bench::broadcast(N_in, count);
    bench::broadcast(K_in, count);
    if (M_in.size() != count || N_in.size() != count || K_in.size() != count) {
      throw std::runtime_error("m, n, k must be the same length");
    }
    const size_t nr_benchmarks = opt.size("nr_benchmarks");
    const float duration = opt.real("benchmark_duration");
    std::cerr << "Estimated benchmark duration: " << nr_benchmarks * duration * (count + 1) << " s" << std::endl;

    bench::Gpu gpu((unsigned)opt.size("device"));
    const dim3 tile = ccglib::mma::GEMM::GetDimensions(precision, variant);
    std::vector<size_t> M = M_in, N = N_in, K = K_in;
    if (opt.flag("pad")) {
      for (size_t i = 0; i < count; ++i) {
        M[i] = bench::align(M_in[i], tile.x);
        N[i] = bench::align(N_in[i], tile.y);
        K[i] = bench::align(K_in[i], tile.z);
      }
    }
    // (unlike the reference, the 1-bit kernels here take any M, N, K)

    size_t num_a = 0, num_b = 0, num_c = 0;
    for (size_t i = 0; i < count; ++i) {
      // the opt variant reads whole tiles
      const size_t mp = bench::align(M[i], tile.x), np = bench::align(N[i], tile.y), kp = bench::align(K[i], tile.z);
      num_a = std::max(num_a, mp * kp);
      num_b = std::max(num_b, np * kp);
      num_c = std::max(num_c, M[i] * N[i]);
    }
    const size_t in_bits = precision.GetInputBits(), out_bits = precision.GetOutputBits();
    hipDeviceptr_t d_a = gpu.alloc(B * 2 * num_a * in_bits / 8, 0xAA);
    hipDeviceptr_t d_b = gpu.alloc(B * 2 * num_b * in_bits / 8, 0xBB);
    hipDeviceptr_t d_c = gpu.alloc(B * 2 * num_c * out_bits / 8, 0);

    const bool csv = opt.flag("csv");
    if (csv) std::cout << "#M,N,K,runtime_ms,tops" << std::endl;
    for (size_t bench_nr = 0; bench_nr < nr_benchmarks; ++bench_nr) {
      for (size_t i = 0; i < count; ++i) {
        ccglib::mma::GEMM gemm(B, M[i], N[i], K[i], gpu.device, gpu.stream, precision, variant, axis);
        const double ms = gpu.measure([&] { gemm.Run(d_a, d_b, d_c); }, duration, bench_nr == 0 && i == 0);
        const double tops = 8e-9 * (double)B * M_in[i] * N_in[i] * K_in[i] / ms;
        if (csv) {
          std::cout << M_in[i] << "," << N_in[i] << "," << K_in[i] << "," << ms << "," << tops << std::endl;
        } else {
          const std::string shape =
              std::to_string(M_in[i]) + "x" + std::to_string(N_in[i]) + "x" + std::to_string(K_in[i]);
          std::cout << std::setw(20) << shape << " " << std::setw(7) << ms << " ms, " << std::setw(7) << tops
                    << " TOps/s" << std::endl;
        }
      }
    }
  } catch (const std::exception &e) {
    std::cerr << "benchmark_gemm: " << e.what() << std::endl;
    return EXIT_FAILURE;
  }
  return EXIT_SUCCESS;
}
