// C entry points around ccglib::reference::GEMM (include/ccglib/gemm/reference.h)
// so that the Python tests can run it on the CPU and compare it with the oracle.
#include <complex>
#include <cstddef>

#include <ccglib/gemm/reference.h>

// type codes: the integer values of ccglib::ValueType
enum { kInt1 = 0, kInt32 = 1, kBf16 = 2, kE4m3 = 3, kE5m2 = 4, kF16 = 5, kF32 = 6 };

extern "C" int reference_gemm(int type_in, int type_out, const void *a, const void *b, void *c,
                              size_t M, size_t N, size_t K, int c_order, float alpha_re,
                              float alpha_im, float beta_re, float beta_im) {
  ccglib::reference::GEMM gemm;
  const auto order = c_order == 0 ? ccglib::mma::row_major : ccglib::mma::col_major;
  const std::complex<float> alpha(alpha_re, alpha_im), beta(beta_re, beta_im);
#define PAIR(TI, TO, CI, CO)                                                                   \
  if (type_in == CI && type_out == CO) {                                                       \
    gemm.Run(static_cast<const TI *>(a), static_cast<const TI *>(b), static_cast<TO *>(c), M,  \
             N, K, order, alpha, beta);                                                        \
    return 0;                                                                                  \
  }
  PAIR(fp8_e4m3, float, kE4m3, kF32)
  PAIR(fp8_e5m2, float, kE5m2, kF32)
  PAIR(half, half, kF16, kF16)
  PAIR(half, float, kF16, kF32)
  PAIR(float, half, kF32, kF16)
  PAIR(bf16, bf16, kBf16, kBf16)
  PAIR(bf16, float, kBf16, kF32)
  PAIR(float, bf16, kF32, kBf16)
  PAIR(float, float, kF32, kF32)
  PAIR(unsigned, int, kInt1, kInt32)
#undef PAIR
  return 1;
}
