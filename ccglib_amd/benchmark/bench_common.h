// Shared pieces of the benchmark programs: a small command line parser that
// accepts the option names of the reference's benchmarks
// (benchmark/benchmark_gemm.cpp:13-50, benchmark_transpose.cpp:13-43,
// benchmark_packing.cpp:12-33 there), and the timing protocol those use (one
// run to size the loop, a warm-up loop before the first measurement, then
// HIP events around back-to-back runs on one stream).
#ifndef CCGLIB_AMD_BENCH_COMMON_H_
#define CCGLIB_AMD_BENCH_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <functional>
#include <iostream>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include <ccglib/ccglib.hpp>

namespace bench {

inline void hip_check(hipError_t e, const char *what) {
  if (e != hipSuccess) {
    throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
  }
}

struct OptionSpec {
  std::string name, help, default_value;
  bool is_flag, required;
};

// Options are given as "--name value", "--name=value" or, for one-letter
// names, "-n value"; lists are comma separated or the option is repeated.
class Options {
 public:
  Options(std::string program, std::string title) : program_(std::move(program)), title_(std::move(title)) {}
  void add(const std::string &name, const std::string &help, const std::string &default_value = "",
           bool required = false) {
    specs_.push_back({name, help, default_value, false, required});
  }
  void add_flag(const std::string &name, const std::string &help) {
    specs_.push_back({name, help, "false", true, false});
  }

  void parse(int argc, const char *argv[]) {
    for (int i = 1; i < argc; ++i) {
      std::string arg = argv[i];
      if (arg == "-h" || arg == "--help") {
        print_help();
        std::exit(EXIT_SUCCESS);
      }
      if (arg.size() < 2 || arg[0] != '-') fail("unexpected argument " + arg);
      std::string name = arg.substr(arg[1] == '-' ? 2 : 1), value;
      bool have_value = false;
      const size_t eq = name.find('=');
      if (eq != std::string::npos) {
        value = name.substr(eq + 1);
        name = name.substr(0, eq);
        have_value = true;
      }
      const OptionSpec *spec = find(name);
      if (!spec) fail("unknown option " + arg);
      if (spec->is_flag) {
        if (!have_value) {
          // "--csv" or "--csv true"
          if (i + 1 < argc && (std::string(argv[i + 1]) == "true" || std::string(argv[i + 1]) == "false")) {
            value = argv[++i];
          } else {
            value = "true";
          }
        }
      } else if (!have_value) {
        if (i + 1 >= argc) fail("option " + arg + " needs a value");
        value = argv[++i];
      }
      std::string &slot = values_[name];
      slot = (slot.empty() || spec->is_flag) ? value : slot + "," + value;
    }
    for (const OptionSpec &s : specs_) {
      if (s.required && !values_.count(s.name)) {
        std::cerr << "Required argument missing: " << s.name << std::endl;
        std::cerr << "Run " << program_ << " -h for help" << std::endl;
        std::exit(EXIT_FAILURE);
      }
    }
  }

  std::string str(const std::string &name) const {
    auto it = values_.find(name);
    if (it != values_.end()) return it->second;
    const OptionSpec *s = find(name);
    return s ? s->default_value : std::string();
  }
  bool flag(const std::string &name) const { return str(name) == "true" || str(name) == "1"; }
  size_t size(const std::string &name) const { return std::stoull(str(name)); }
  float real(const std::string &name) const { return std::stof(str(name)); }
  std::vector<size_t> sizes(const std::string &name) const {
    std::vector<size_t> out;
    const std::string s = str(name);
    size_t pos = 0;
    while (pos <= s.size() && !s.empty()) {
      const size_t comma = s.find(',', pos);
      const std::string item = s.substr(pos, comma == std::string::npos ? std::string::npos : comma - pos);
      if (!item.empty()) out.push_back(std::stoull(item));
      if (comma == std::string::npos) break;
      pos = comma + 1;
    }
    return out;
  }

 private:
  const OptionSpec *find(const std::string &name) const {
    for (const OptionSpec &s : specs_) {
      if (s.name == name) return &s;
    }
    return nullptr;
  }
  [[noreturn]] void fail(const std::string &message) const {
    std::cerr << "Error parsing commandline: " << message << std::endl;
    std::exit(EXIT_FAILURE);
  }
  void print_help() const {
    std::cout << title_ << "\nUsage: " << program_ << " [options]\n";
    for (const OptionSpec &s : specs_) {
      std::cout << "  " << (s.name.size() == 1 ? "-" : "--") << s.name << (s.is_flag ? "" : " arg") << "\t" << s.help;
      if (!s.default_value.empty() && !s.is_flag) std::cout << " (default: " << s.default_value << ")";
      if (s.required) std::cout << " (required)";
      std::cout << "\n";
    }
    std::cout << "  -h, --help\tPrint help" << std::endl;
  }

  std::string program_, title_;
  std::vector<OptionSpec> specs_;
  std::map<std::string, std::string> values_;
};

inline const std::map<std::string, ccglib::ValueType> &precision_names() {
  static const std::map<std::string, ccglib::ValueType> names{
      {"float32", ccglib::ValueType::float32},       {"float16", ccglib::ValueType::float16},
      {"bfloat16", ccglib::ValueType::bfloat16},     {"float8e4m3", ccglib::ValueType::float8e4m3},
      {"float8e5m2", ccglib::ValueType::float8e5m2}, {"int32", ccglib::ValueType::int32},
      {"int1", ccglib::ValueType::int1}};
  return names;
}

// A single-valued size list is repeated to the common length.
inline void broadcast(std::vector<size_t> &v, size_t n) {
  if (v.size() == 1) v.resize(n, v[0]);
}

inline size_t align(size_t a, size_t b) { return ccglib::helper::ceildiv(a, b) * b; }

// Device, stream and the two events of a benchmark program.
struct Gpu {
  explicit Gpu(unsigned id) {
    hip_check(hipInit(0), "hipInit");
    hip_check(hipDeviceGet(&device, (int)id), "hipDeviceGet");
    hip_check(hipSetDevice((int)id), "hipSetDevice");
    hip_check(hipStreamCreate(&stream), "hipStreamCreate");
    hip_check(hipEventCreate(&start), "hipEventCreate");
    hip_check(hipEventCreate(&end), "hipEventCreate");
  }
  ~Gpu() {
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(end);
    (void)hipStreamDestroy(stream);
  }
  hipDeviceptr_t alloc(size_t bytes, unsigned char fill) {
    void *p = nullptr;
    hip_check(hipMalloc(&p, bytes ? bytes : 1), "hipMalloc");
    hip_check(hipMemsetAsync(p, fill, bytes, stream), "hipMemsetAsync");
    hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    owned.push_back(p);
    return p;
  }
  float elapsed_ms(const std::function<void()> &body, size_t iterations) {
    hip_check(hipEventRecord(start, stream), "hipEventRecord");
    for (size_t i = 0; i < iterations; ++i) body();
    hip_check(hipEventRecord(end, stream), "hipEventRecord");
    hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
    float ms = 0.f;
    hip_check(hipEventElapsedTime(&ms, start, end), "hipEventElapsedTime");
    return ms;
  }
  // Average run time in milliseconds over about `duration_s` seconds of runs.
  double measure(const std::function<void()> &body, float duration_s, bool warm_up) {
    const float once = elapsed_ms(body, 1);
    const size_t iterations = (size_t)((1000.f * duration_s) / (once > 1e-6f ? once : 1e-6f)) + 1;
    if (warm_up) (void)elapsed_ms(body, iterations);
    return (double)elapsed_ms(body, iterations) / (double)iterations;
  }

  hipDevice_t device;
  hipStream_t stream;
  hipEvent_t start, end;
  std::vector<void *> owned;   // freed by the driver at process exit
};

}  // namespace bench
#endif  // CCGLIB_AMD_BENCH_COMMON_H_
