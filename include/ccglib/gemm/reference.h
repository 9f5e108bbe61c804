// ccglib::reference::GEMM: the host-side complex GEMM that callers of the
// reference check device results against (reference:
// include/ccglib/gemm/reference.h:12-54, src/reference/GEMM.cpp:15-91 for the
// floating-point pairs, :106-224 for 1-bit input). Header-only here, plain
// loops on the calling thread; the GPU library never calls it.
//
// One batch per call. a is [2][M][K], b is [2][N][K] (planar, K contiguous), c is
// [2][M][N] (row_major) or [2][N][M] (col_major):
//   c = alpha * a * b^T + beta * c     (complex, no conjugate)
// Arithmetic of the floating-point pairs: float, k ascending, the four real
// products of one k combined before they are added to the sums; alpha is
// applied only if it differs from (1, 0), and c is read only if beta differs
// from (0, 0); the result is rounded to the output type on store.
// 1-bit input: K counts samples, rows hold ceil(K / 32) words, bit 1 is +1 and
// bit 0 is -1; the bits that pad the last word count as the reference counts
// them (the real part sees them in both of its terms, the imaginary part is
// corrected for them); alpha and beta are truncated to integers, alpha is
// always applied and c is always read; integer arithmetic wraps modulo 2^32.
#ifndef CCGLIB_GEMM_REFERENCE_H_
#define CCGLIB_GEMM_REFERENCE_H_

#include <complex>
#include <cstddef>
#include <cstdint>

#include <ccglib/bf16.h>
#include <ccglib/fp16.h>
#include <ccglib/fp8.h>
#include <ccglib/gemm/mem_order.h>

namespace ccglib::reference {

namespace detail {

inline float to_float(float v) { return v; }
inline float to_float(half v) { return __half2float(v); }
inline float to_float(bf16 v) { return __bfloat162float(v); }
inline float to_float(fp8_e4m3 v) { return static_cast<float>(v); }
inline float to_float(fp8_e5m2 v) { return static_cast<float>(v); }

inline void from_float(float v, float *out) { *out = v; }
inline void from_float(float v, half *out) { *out = __float2half(v); }
inline void from_float(float v, bf16 *out) { *out = __float2bfloat16(v); }

// A float product that is rounded before anything is added to it, whatever the
// compiler and its flags (-mfma with -ffp-contract=fast fuses across statements
// and, in clang, past `#pragma clang fp contract(off)` too): the value passes
// through an empty asm statement, which no optimiser looks into, so there is no
// multiply left next to an add that could become a fused multiply-add.
inline float rounded_product(float x, float y) {
  float p = x * y;
#if defined(__x86_64__)
  __asm__ volatile("" : "+x"(p));
#elif defined(__aarch64__)
  __asm__ volatile("" : "+w"(p));
#else
  __asm__ volatile("" : "+m"(p));
#endif
  return p;
}

template <typename Tin, typename Tout>
void gemm_float(const Tin *a, const Tin *b, Tout *c, size_t M, size_t N, size_t K,
                ccglib::mma::MemOrder order, std::complex<float> alpha, std::complex<float> beta) {
  const Tin *a_im = a + M * K, *b_im = b + N * K;
  Tout *c_im = c + M * N;
  const bool scale = alpha != std::complex<float>(1.f, 0.f);
  const bool add_c = beta != std::complex<float>(0.f, 0.f);
  for (size_t m = 0; m < M; ++m) {
    for (size_t n = 0; n < N; ++n) {
      float re = 0.f, im = 0.f;
      for (size_t k = 0; k < K; ++k) {
        const float ar = to_float(a[m * K + k]), ai = to_float(a_im[m * K + k]);
        const float br = to_float(b[n * K + k]), bi = to_float(b_im[n * K + k]);
        const float t_re = rounded_product(ar, br) - rounded_product(ai, bi);
        const float t_im = rounded_product(ar, bi) + rounded_product(ai, br);
        re += t_re;
        im += t_im;
      }
      if (scale) {
        const float r = re;
        re = rounded_product(alpha.real(), r) - rounded_product(alpha.imag(), im);
        im = rounded_product(alpha.imag(), r) + rounded_product(alpha.real(), im);
      }
      const size_t at = order == ccglib::mma::row_major ? m * N + n : n * M + m;
      if (add_c) {
        const float cr = to_float(c[at]), ci = to_float(c_im[at]);
        re += rounded_product(beta.real(), cr) - rounded_product(beta.imag(), ci);
        im += rounded_product(beta.imag(), cr) + rounded_product(beta.real(), ci);
      }
      from_float(re, &c[at]);
      from_float(im, &c_im[at]);
    }
  }
}

inline unsigned ones(std::uint32_t x) {
  unsigned count = 0;
  for (; x; x &= x - 1) ++count;
  return count;
}

inline void gemm_bits(const unsigned *a, const unsigned *b, int *c, size_t M, size_t N, size_t K,
                      ccglib::mma::MemOrder order, std::complex<float> alpha,
                      std::complex<float> beta) {
  const size_t words = (K + 31) / 32, padded = words * 32, padding = padded - K;
  const unsigned *a_im = a + M * words, *b_im = b + N * words;
  int *c_im = c + M * N;
  const std::uint32_t al_re = (std::uint32_t)(std::int32_t)alpha.real(),
                      al_im = (std::uint32_t)(std::int32_t)alpha.imag(),
                      be_re = (std::uint32_t)(std::int32_t)beta.real(),
                      be_im = (std::uint32_t)(std::int32_t)beta.imag();
  for (size_t m = 0; m < M; ++m) {
    for (size_t n = 0; n < N; ++n) {
      std::int64_t differ_re = 0, differ_im = 0;
      for (size_t w = 0; w < words; ++w) {
        const std::uint32_t ar = a[m * words + w], ai = a_im[m * words + w];
        const std::uint32_t br = b[n * words + w], bi = b_im[n * words + w];
        differ_re += ones(ar ^ br) + ones(ai ^ ~bi);
        differ_im += ones(ar ^ bi) + ones(ai ^ br);
      }
      const std::uint32_t s_re = 2u * (std::uint32_t)((std::int64_t)padded - differ_re);
      const std::uint32_t s_im =
          2u * (std::uint32_t)((std::int64_t)padded - (std::int64_t)padding - differ_im);
      const size_t at = order == ccglib::mma::row_major ? m * N + n : n * M + m;
      const std::uint32_t cr = (std::uint32_t)c[at], ci = (std::uint32_t)c_im[at];
      c[at] = (int)(al_re * s_re - al_im * s_im + be_re * cr - be_im * ci);
      c_im[at] = (int)(al_im * s_re + al_re * s_im + be_im * cr + be_re * ci);
    }
  }
}

}  // namespace detail

class GEMM {
public:
  virtual ~GEMM() = default;

#define CCGLIB_REFERENCE_RUN(TIN, TOUT)                                                          \
  virtual void Run(const TIN *a, const TIN *b, TOUT *c, size_t M, size_t N, size_t K,            \
                   ccglib::mma::MemOrder output_mem_order = ccglib::mma::row_major,              \
                   std::complex<float> alpha = {1, 0}, std::complex<float> beta = {0, 0}) {      \
    detail::gemm_float(a, b, c, M, N, K, output_mem_order, alpha, beta);                         \
  }
  CCGLIB_REFERENCE_RUN(fp8_e4m3, float)
  CCGLIB_REFERENCE_RUN(fp8_e5m2, float)
  CCGLIB_REFERENCE_RUN(half, half)
  CCGLIB_REFERENCE_RUN(half, float)
  CCGLIB_REFERENCE_RUN(float, half)
  CCGLIB_REFERENCE_RUN(bf16, bf16)
  CCGLIB_REFERENCE_RUN(bf16, float)
  CCGLIB_REFERENCE_RUN(float, bf16)
  CCGLIB_REFERENCE_RUN(float, float)
#undef CCGLIB_REFERENCE_RUN

  virtual void Run(const unsigned *a, const unsigned *b, int *c, size_t M, size_t N, size_t K,
                   ccglib::mma::MemOrder output_mem_order = ccglib::mma::row_major,
                   std::complex<float> alpha = {1, 0}, std::complex<float> beta = {0, 0}) {
    detail::gemm_bits(a, b, c, M, N, K, output_mem_order, alpha, beta);
  }
};

}  // namespace ccglib::reference

#endif  // CCGLIB_GEMM_REFERENCE_H_
