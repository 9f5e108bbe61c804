// Packing benchmark with the command line and the output of the reference's
// benchmark/benchmark_packing.cpp (options :15-32, "#N,runtime_ms,gbytes" :120-126,
// gbytes = (N + N / 8) / t :172-177), on plain HIP. The buffers are sized for
// the chosen direction (one byte per sample on the unpacked side).
#include <algorithm>
#include <iomanip>

#include "bench_common.h"

int main(int argc, const char *argv[]) {
  bench::Options opt(argv[0], "Packing benchmark");
  opt.add("n", "Size(s) of N axis", "", true);
  opt.add("nr_benchmarks", "Number of benchmarks", "1");
  opt.add("benchmark_duration", "Approximate benchmark duration (seconds)", "4");
  opt.add_flag("csv", "Format output to CSV");
  opt.add("direction", "Packing direction (pack or unpack)", "pack");
  opt.add("device", "GPU device ID", "0");
  opt.parse(argc, argv);

  try {
    const std::vector<size_t> N = opt.sizes("n");
    const std::map<std::string, ccglib::Direction> directions{{"pack", ccglib::forward},
                                                              {"unpack", ccglib::backward}};
    if (!directions.count(opt.str("direction"))) throw std::runtime_error("direction must be pack or unpack");
    const ccglib::Direction direction = directions.at(opt.str("direction"));
    const size_t nr_benchmarks = opt.size("nr_benchmarks");
    const float duration = opt.real("benchmark_duration");
    std::cerr << "Estimated benchmark duration: " << nr_benchmarks * duration * (N.size() + 1) << " s" << std::endl;

    bench::Gpu gpu((unsigned)opt.size("device"));
    const size_t n_max = *std::max_element(N.begin(), N.end());
    const size_t unpacked_bytes = n_max, packed_bytes = ccglib::helper::ceildiv(n_max, (size_t)32) * 4;
    hipDeviceptr_t d_unpacked = gpu.alloc(unpacked_bytes, direction == ccglib::forward ? 0x01 : 0xBB);
    hipDeviceptr_t d_packed = gpu.alloc(packed_bytes, 0xAA);
    hipDeviceptr_t d_in = direction == ccglib::forward ? d_unpacked : d_packed;
    hipDeviceptr_t d_out = direction == ccglib::forward ? d_packed : d_unpacked;

    const bool csv = opt.flag("csv");
    if (csv) std::cout << "#N,runtime_ms,gbytes" << std::endl;
    for (size_t bench_nr = 0; bench_nr < nr_benchmarks; ++bench_nr) {
      for (size_t i = 0; i < N.size(); ++i) {
        ccglib::packing::Packing packing(N[i], direction, gpu.device, gpu.stream);
        const double ms = gpu.measure([&] { packing.Run(d_in, d_out); }, duration, bench_nr == 0 && i == 0);
        const double gbytes = ((double)N[i] + (double)N[i] / 8) / ms * 1e-6;
        if (csv) {
          std::cout << N[i] << "," << ms << "," << gbytes << std::endl;
        } else {
          std::cout << std::setw(20) << N[i] << " " << std::setw(7) << ms << " ms, " << std::setw(7) << gbytes
                    << " GByte/s" << std::endl;
        }
      }
    }
  } catch (const std::exception &e) {
    std::cerr << "benchmark_packing: " << e.what() << std::endl;
    return EXIT_FAILURE;
  }
  return EXIT_SUCCESS;
}
