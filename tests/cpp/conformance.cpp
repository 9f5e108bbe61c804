// C++ conformance caller for the drop-in headers: exercises ccglib::mma::GEMM,
// transpose::Transpose, packing::Packing and pipeline::Pipeline with native HIP
// handles, the way the reference's own HIP API tests and example do
// (test/hip/mma.cpp, test/hip/packing.cpp, test/hip/transpose.cpp,
// test/hip/pipeline.cpp, example/example.hip). Expected values come from closed
// forms and from loops written out here, on inputs whose arithmetic is exact.
#include <complex>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <ccglib/ccglib.hpp>

static int failures = 0;
#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) {                                                           \
      ++failures;                                                            \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
    }                                                                        \
  } while (0)
#define HIP(x)                                                               \
  do {                                                                       \
    hipError_t e_ = (x);                                                     \
    if (e_ != hipSuccess) {                                                  \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                          \
    }                                                                        \
  } while (0)

template <typename T> struct DeviceBuffer {
  T *ptr = nullptr;
  size_t n;
  explicit DeviceBuffer(size_t count) : n(count) { HIP(hipMalloc(&ptr, count * sizeof(T) + 64)); }
  ~DeviceBuffer() { (void)hipFree(ptr); }
  void upload(const std::vector<T> &h) { HIP(hipMemcpy(ptr, h.data(), n * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> download() {
    std::vector<T> h(n);
    HIP(hipMemcpy(h.data(), ptr, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
  hipDeviceptr_t dev() { return reinterpret_cast<hipDeviceptr_t>(ptr); }
};

// all inputs one: real part 0, imaginary part 2K (test/hip/mma.cpp:76-77)
static void test_all_ones(hipDevice_t device, hipStream_t stream) {
  const size_t B = 3, M = 512, N = 512, K = 512;
  std::vector<__half> ones(B * 2 * M * K, __float2half(1.0f));
  DeviceBuffer<__half> a(B * 2 * M * K), b(B * 2 * N * K);
  DeviceBuffer<float> c(B * 2 * M * N);
  a.upload(ones);
  b.upload(ones);
  ccglib::mma::GEMM gemm(B, M, N, K, device, stream, ccglib::ValueType::float16, ccglib::mma::basic);
  gemm.Run(a.dev(), b.dev(), c.dev());
  HIP(hipStreamSynchronize(stream));
  const std::vector<float> h = c.download();
  bool ok = true;
  for (size_t bb = 0; bb < B; ++bb)
    for (size_t i = 0; i < M * N; ++i) {
      ok = ok && h[(bb * 2) * M * N + i] == 0.0f && h[(bb * 2 + 1) * M * N + i] == 2.0f * K;
    }
  CHECK(ok);
}

// Transpose with GetDimensions chunks, then the opt GEMM, against a loop on
// small integers (every product and sum is exact in fp32).
static void test_opt_with_transpose(hipDevice_t device, hipStream_t stream) {
  const size_t B = 2, M = 100, N = 60, K = 40;
  const std::complex<float> alpha(2, -1), beta(-1, 3);
  std::mt19937 rng(7);
  std::uniform_int_distribution<int> dist(-3, 3);
  std::vector<__half> ha(B * 2 * M * K), hb(B * 2 * N * K);
  std::vector<float> fa(ha.size()), fb(hb.size()), hc(B * 2 * M * N);
  for (size_t i = 0; i < ha.size(); ++i) ha[i] = __float2half(fa[i] = (float)dist(rng));
  for (size_t i = 0; i < hb.size(); ++i) hb[i] = __float2half(fb[i] = (float)dist(rng));
  for (auto &v : hc) v = (float)dist(rng);

  const ccglib::Precision precision(ccglib::ValueType::float16, ccglib::ValueType::float32);
  const dim3 dims = ccglib::mma::GEMM::GetDimensions(precision, ccglib::mma::opt);
  const size_t Mp = ccglib::helper::ceildiv(M, (size_t)dims.x) * dims.x;
  const size_t Np = ccglib::helper::ceildiv(N, (size_t)dims.y) * dims.y;
  const size_t Kp = ccglib::helper::ceildiv(K, (size_t)dims.z) * dims.z;
  DeviceBuffer<__half> a(ha.size()), b(hb.size()), at(B * 2 * Mp * Kp), bt(B * 2 * Np * Kp);
  DeviceBuffer<float> c(hc.size());
  a.upload(ha);
  b.upload(hb);
  c.upload(hc);
  ccglib::transpose::Transpose ta(B, M, K, dims.x, dims.z, 16, device, stream);
  ccglib::transpose::Transpose tb(B, N, K, dims.y, dims.z, 16, device, stream);
  ta.Run(a.dev(), at.dev());
  tb.Run(b.dev(), bt.dev());
  ccglib::mma::GEMM gemm(B, M, N, K, device, stream, precision, ccglib::mma::opt,
                         ccglib::complex_planar, ccglib::mma::row_major, ccglib::mma::row_major,
                         ccglib::mma::col_major, alpha, beta);
  gemm.Run(at.dev(), bt.dev(), c.dev());
  HIP(hipStreamSynchronize(stream));
  const std::vector<float> got = c.download();
  bool ok = true;
  for (size_t bb = 0; bb < B; ++bb)
    for (size_t m = 0; m < M; ++m)
      for (size_t n = 0; n < N; ++n) {
        std::complex<float> sum(0, 0);
        for (size_t k = 0; k < K; ++k) {
          const std::complex<float> x(fa[((bb * 2) * M + m) * K + k], fa[((bb * 2 + 1) * M + m) * K + k]);
          const std::complex<float> y(fb[((bb * 2) * N + n) * K + k], fb[((bb * 2 + 1) * N + n) * K + k]);
          sum += x * y;
        }
        const std::complex<float> cin(hc[((bb * 2) * M + m) * N + n], hc[((bb * 2 + 1) * M + m) * N + n]);
        const std::complex<float> want = alpha * sum + beta * cin;
        ok = ok && got[((bb * 2) * M + m) * N + n] == want.real() &&
             got[((bb * 2 + 1) * M + m) * N + n] == want.imag();
      }
  CHECK(ok);
  // and against the host-side class, batch by batch, as the reference's tests
  // verify (test/gemm/verify.h:54-60)
  ccglib::reference::GEMM host;
  std::vector<float> want_host = hc;
  for (size_t bb = 0; bb < B; ++bb) {
    host.Run(ha.data() + bb * 2 * M * K, hb.data() + bb * 2 * N * K, want_host.data() + bb * 2 * M * N,
             M, N, K, ccglib::mma::row_major, alpha, beta);
  }
  CHECK(want_host == got);
}

// pack, unpack and the round trip on N = 2048 (test/hip/packing.cpp)
static void test_packing(hipDevice_t device, hipStream_t stream) {
  const size_t N = 2048;
  std::mt19937 rng(1);
  std::vector<unsigned char> in(N);
  for (auto &v : in) v = rng() & 1;
  DeviceBuffer<unsigned char> d_in(N), d_back(N);
  DeviceBuffer<unsigned> d_packed(N / 32);
  d_in.upload(in);
  ccglib::packing::Packing pack(N, ccglib::forward, device, stream);
  ccglib::packing::Packing unpack(N, ccglib::backward, device, stream);
  pack.Run(d_in.dev(), d_packed.dev());
  unpack.Run(d_packed.dev(), d_back.dev());
  HIP(hipStreamSynchronize(stream));
  const std::vector<unsigned> packed = d_packed.download();
  bool ok = true;
  for (size_t i = 0; i < N; ++i) ok = ok && ((packed[i / 32] >> (i % 32)) & 1u) == in[i];
  CHECK(ok);
  CHECK(d_back.download() == in);
}

// every element lands where the tiling formula says (test/hip/transpose.cpp)
static void test_transpose(hipDevice_t device, hipStream_t stream) {
  const size_t B = 2, M = 256, N = 128, Mc = 64, Nc = 64;
  std::vector<uint16_t> in(B * 2 * M * N);
  for (size_t i = 0; i < in.size(); ++i) in[i] = (uint16_t)(i * 2654435761u >> 16);
  for (int interleaved = 0; interleaved < 2; ++interleaved) {
    DeviceBuffer<uint16_t> d_in(in.size()), d_out(in.size());
    d_in.upload(in);
    ccglib::transpose::Transpose t(B, M, N, Mc, Nc, 16, device, stream,
                                   interleaved ? ccglib::complex_interleaved : ccglib::complex_planar);
    t.Run(d_in.dev(), d_out.dev());
    HIP(hipStreamSynchronize(stream));
    const std::vector<uint16_t> out = d_out.download();
    bool ok = true;
    for (size_t b = 0; b < B; ++b)
      for (size_t c = 0; c < 2; ++c)
        for (size_t m = 0; m < M; ++m)
          for (size_t n = 0; n < N; ++n) {
            const size_t i = interleaved ? ((b * M + m) * N + n) * 2 + c : ((b * 2 + c) * M + m) * N + n;
            const size_t o = ((((b * (M / Mc) + m / Mc) * (N / Nc) + n / Nc) * 2 + c) * Mc + m % Mc) * Nc + n % Nc;
            ok = ok && in[i] == out[o];
          }
    CHECK(ok);
  }
}

// 1-bit pipeline: one byte per sample in, packed and transposed inside; bit 1 is
// +1 and bit 0 is -1 (test/hip/pipeline.cpp, test/pipeline/pipeline.cpp:88-187)
static void test_pipeline_int1(hipDevice_t device, hipStream_t stream) {
  const size_t B = 2, M = 64, N = 48, K = 1024;
  std::mt19937 rng(3);
  std::vector<unsigned char> ha(B * 2 * M * K), hb(B * 2 * N * K);
  for (auto &v : ha) v = rng() & 1;
  for (auto &v : hb) v = rng() & 1;
  DeviceBuffer<unsigned char> a(ha.size()), b(hb.size());
  DeviceBuffer<int> c(B * 2 * M * N);
  a.upload(ha);
  b.upload(hb);
  HIP(hipMemset(c.ptr, 0, c.n * sizeof(int)));
  ccglib::pipeline::Pipeline pipe(B, M, N, K, device, stream, ccglib::complex_planar,
                                  ccglib::complex_planar, ccglib::mma::row_major,
                                  ccglib::mma::col_major, ccglib::mma::row_major, ccglib::int1,
                                  ccglib::int32, ccglib::mma::opt);
  pipe.Run(a.dev(), b.dev(), c.dev());
  HIP(hipStreamSynchronize(stream));
  const std::vector<int> got = c.download();
  bool ok = true;
  for (size_t bb = 0; bb < B; ++bb)
    for (size_t m = 0; m < M; ++m)
      for (size_t n = 0; n < N; ++n) {
        int re = 0, im = 0;
        for (size_t k = 0; k < K; ++k) {
          const int ar = ha[((bb * 2) * M + m) * K + k] ? 1 : -1, ai = ha[((bb * 2 + 1) * M + m) * K + k] ? 1 : -1;
          const int br = hb[((bb * 2) * N + n) * K + k] ? 1 : -1, bi = hb[((bb * 2 + 1) * N + n) * K + k] ? 1 : -1;
          re += ar * br - ai * bi;
          im += ar * bi + ai * br;
        }
        ok = ok && got[((bb * 2) * M + m) * N + n] == re && got[((bb * 2 + 1) * M + m) * N + n] == im;
      }
  CHECK(ok);
}

// construction errors are std::runtime_error with the reference's wording
static void test_errors(hipDevice_t device, hipStream_t stream) {
  auto message = [&](auto make) -> std::string {
    try {
      make();
    } catch (const std::runtime_error &e) {
      return e.what();
    }
    return "";
  };
  CHECK(message([&] {
          ccglib::mma::GEMM g(16, 16, 16, 256, device, stream, ccglib::ValueType::float16,
                              ccglib::mma::basic, ccglib::complex_interleaved);
        }).find("complex-interleaved output is not supported in basic variant") != std::string::npos);
  CHECK(message([&] {
          ccglib::mma::GEMM g(16, 16, 16, 256, device, stream, ccglib::ValueType::float16,
                              ccglib::mma::basic, ccglib::complex_planar, ccglib::mma::row_major,
                              ccglib::mma::col_major, ccglib::mma::col_major);
        }).find("HIPRTC_ERROR_COMPILATION") != std::string::npos);
  CHECK(message([&] {
          ccglib::packing::Packing p(2048, ccglib::backward, device, stream, ccglib::complex_interleaved);
        }).find("complex-interleaved input is not supported in unpacking kernel") != std::string::npos);
}

int main() {
  HIP(hipInit(0));
  hipDevice_t device;
  HIP(hipDeviceGet(&device, 0));
  hipStream_t stream;
  HIP(hipStreamCreate(&stream));
  test_all_ones(device, stream);
  test_opt_with_transpose(device, stream);
  test_packing(device, stream);
  test_transpose(device, stream);
  test_pipeline_int1(device, stream);
  test_errors(device, stream);
  HIP(hipStreamDestroy(stream));
  std::printf(failures ? "conformance: %d check(s) failed\n" : "conformance: all checks passed\n", failures);
  return failures ? 1 : 0;
}
