/*
 * CPU oracle for the complex-GEMM hot path: TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms of the reference library's CPU
 * path and of its data-movement kernels, so that the HIP kernels can be checked
 * against them on the same inputs. Nothing in the shipped library links, loads
 * or calls it; only tests, the smoke check and the benchmark's CPU-baseline leg
 * may use it, and only as the checker.
 *
 * Each function cites the reference file:line (relative to the reference tree)
 * whose behaviour it follows.
 *
 * Pinning status (what fixes each function besides its own formula):
 *   oracle_gemm_float   pinned: reference known-answer tests
 *                       test/gemm/reference.cpp:27-45 (3x2x2, row+col, half /
 *                       bf16 / float inputs) and :98-109 (alpha/beta, K=8);
 *                       complex128 matmul identity; all-ones closed form
 *                       (test/hip/mma.cpp:76-77).
 *   oracle_gemm_int1    pinned: reference known-answer tests
 *                       test/gemm/reference.cpp:73-80 and :121-133; +-1 integer
 *                       matmul identity; brute force on tiny shapes.
 *   oracle_transpose    pinned: closed-form index map restated independently
 *                       with numpy reshape/transpose
 *                       (test/transpose/transpose.cpp:120-146).
 *   oracle_pack_bits / oracle_unpack_bits
 *                       pinned: numpy.packbits(bitorder="little") identity and
 *                       the reference's own check test/packing/packing.cpp:56-63,
 *                       :190-203; round trip.
 *   fp8 / fp16 / bf16 decode and encode
 *                       pinned: exhaustive comparison with an independent
 *                       library's casts (all 256 fp8 codes, all 65536 fp16 and
 *                       bf16 codes).
 */
#define _POSIX_C_SOURCE 200809L   /* rand_r */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* Enum values are those of the reference API
 * (include/ccglib/common/value_type.h:14-22, gemm/mem_order.h:6,
 * common/complex_order.h:12). */
enum {
  CCG_INT1 = 0,
  CCG_INT32 = 1,
  CCG_BFLOAT16 = 2,
  CCG_FLOAT8E4M3 = 3,
  CCG_FLOAT8E5M2 = 4,
  CCG_FLOAT16 = 5,
  CCG_FLOAT32 = 6
};
enum { CCG_ROW_MAJOR = 0, CCG_COL_MAJOR = 1 };
enum { CCG_PLANAR = 0, CCG_INTERLEAVED = 1 };

/* ---------------------------------------------------------------------- */
/* Narrow float formats <-> float. The reference gets these from the vendor  */
/* headers (include/ccglib/fp16.h, bf16.h, fp8.h:35-37: OCP fp8 on this       */
/* target). They are restated here bit by bit.                               */
/* ---------------------------------------------------------------------- */

static float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

static uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  return u;
}

/* Generic small IEEE-like format decode: 1 sign, E exponent, Mn mantissa bits.
 * ocp_e4m3 selects the OCP e4m3 rule: no infinities, only S.1111.111 is NaN. */
static float small_to_float(uint32_t v, int E, int Mn, int ocp_e4m3) {
  const int bias = (1 << (E - 1)) - 1;
  const uint32_t sign = (v >> (E + Mn)) & 1u;
  const uint32_t e = (v >> Mn) & ((1u << E) - 1u);
  const uint32_t m = v & ((1u << Mn) - 1u);
  float mag;
  if (e == 0) {
    mag = ldexpf((float)m, 1 - bias - Mn); /* subnormal or zero */
  } else if (e == (1u << E) - 1u && !ocp_e4m3) {
    mag = m ? NAN : INFINITY;
  } else if (ocp_e4m3 && e == 15 && m == 7) {
    mag = NAN;
  } else {
    mag = ldexpf((float)(m | (1u << Mn)), (int)e - bias - Mn);
  }
  return sign ? -mag : mag;
}

float oracle_half_to_float(uint16_t h) { return small_to_float(h, 5, 10, 0); }
float oracle_bf16_to_float(uint16_t h) {
  return bits_to_float((uint32_t)h << 16);
}
float oracle_e4m3_to_float(uint8_t v) { return small_to_float(v, 4, 3, 1); }
float oracle_e5m2_to_float(uint8_t v) { return small_to_float(v, 5, 2, 0); }

/* float -> half, round to nearest even, overflow to infinity. */
uint16_t oracle_float_to_half(float f) {
  const uint32_t u = float_to_bits(f);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t absu = u & 0x7fffffffu;
  if (absu > 0x7f800000u) {
    return (uint16_t)(sign | 0x7e00u); /* NaN */
  }
  if (absu >= 0x47800000u) { /* >= 65536: infinity (65520 rounds up below) */
    return (uint16_t)(sign | 0x7c00u);
  }
  const float a = bits_to_float(absu);
  if (absu < 0x38800000u) { /* below the smallest normal half, 2^-14 */
    /* subnormal half: value = n * 2^-24, n rounded to nearest even */
    const float scaled = a * 16777216.0f; /* exact: 2^24 */
    const float r = nearbyintf(scaled);   /* default mode = nearest even */
    return (uint16_t)(sign | (uint16_t)r);
  }
  /* normal: round the 23-bit mantissa to 10 bits */
  uint32_t v = absu - 0x38000000u; /* rebias 127 -> 15 */
  const uint32_t lsb = (v >> 13) & 1u;
  v += 0x0fffu + lsb;
  return (uint16_t)(sign | (uint16_t)(v >> 13));
}

/* float -> bfloat16, round to nearest even. */
uint16_t oracle_float_to_bf16(float f) {
  uint32_t u = float_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  }
  const uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

static float load_as_float(const void *p, size_t idx, int type) {
  switch (type) {
  case CCG_FLOAT16:
    return oracle_half_to_float(((const uint16_t *)p)[idx]);
  case CCG_BFLOAT16:
    return oracle_bf16_to_float(((const uint16_t *)p)[idx]);
  case CCG_FLOAT8E4M3:
    return oracle_e4m3_to_float(((const uint8_t *)p)[idx]);
  case CCG_FLOAT8E5M2:
    return oracle_e5m2_to_float(((const uint8_t *)p)[idx]);
  case CCG_FLOAT32:
  default:
    return ((const float *)p)[idx];
  }
}

static void store_from_float(void *p, size_t idx, int type, float v) {
  switch (type) {
  case CCG_FLOAT16:
    ((uint16_t *)p)[idx] = oracle_float_to_half(v);
    break;
  case CCG_BFLOAT16:
    ((uint16_t *)p)[idx] = oracle_float_to_bf16(v);
    break;
  case CCG_FLOAT32:
  default:
    ((float *)p)[idx] = v;
    break;
  }
}

/* ---------------------------------------------------------------------- */
/* Float complex GEMM, one batch per call.                                   */
/* Follows src/reference/GEMM.cpp:15-91:                                     */
/*   - compute type is float for every supported pair (:22-27);              */
/*   - a is [2][M][K], b is [2][N][K], c is [2][M][N] or [2][N][M] (:28-35); */
/*   - (m,n) loops parallel, k sequential ascending, the four products       */
/*     combined per k before accumulation (:45-62);                          */
/*   - alpha applied only when alpha != (1,0) (:69-73);                      */
/*   - beta term reads c only when beta != (0,0) (:80-85);                   */
/*   - result converted to the output type on store (:87-88).                */
/* ---------------------------------------------------------------------- */
void oracle_gemm_float(const void *a, const void *b, void *c, size_t M,
                       size_t N, size_t K, int type_in, int type_out,
                       int c_order, float alpha_re, float alpha_im,
                       float beta_re, float beta_im) {
  const size_t a_plane = M * K;
  const size_t b_plane = N * K;
  const size_t c_plane = M * N;
  const size_t c_major_len = (c_order == CCG_ROW_MAJOR) ? N : M;

#pragma omp parallel for collapse(2)
  for (size_t m = 0; m < M; ++m) {
    for (size_t n = 0; n < N; ++n) {
      float sum_re = 0.0f;
      float sum_im = 0.0f;
      for (size_t k = 0; k < K; ++k) {
        const float ar = load_as_float(a, m * K + k, type_in);
        const float ai = load_as_float(a, a_plane + m * K + k, type_in);
        const float br = load_as_float(b, n * K + k, type_in);
        const float bi = load_as_float(b, b_plane + n * K + k, type_in);
        const float term_re = ar * br - ai * bi;
        const float term_im = ar * bi + ai * br;
        sum_re += term_re;
        sum_im += term_im;
      }
      if (alpha_re != 1.0f || alpha_im != 0.0f) {
        const float keep = sum_re;
        sum_re = alpha_re * sum_re - alpha_im * sum_im;
        sum_im = alpha_im * keep + alpha_re * sum_im;
      }
      const size_t major = (c_order == CCG_ROW_MAJOR) ? m : n;
      const size_t minor = (c_order == CCG_ROW_MAJOR) ? n : m;
      const size_t idx = major * c_major_len + minor;
      if (beta_re != 0.0f || beta_im != 0.0f) {
        const float cr = load_as_float(c, idx, type_out);
        const float ci = load_as_float(c, c_plane + idx, type_out);
        sum_re += beta_re * cr - beta_im * ci;
        sum_im += beta_im * cr + beta_re * ci;
      }
      store_from_float(c, idx, type_out, sum_re);
      store_from_float(c, c_plane + idx, type_out, sum_im);
    }
  }
}

/* Same product accumulated in double, output double [2][M][N] or [2][N][M].
 * Not a restatement of the reference: it is the float64 yardstick that the
 * relative-Frobenius-error criterion is measured against. */
void oracle_gemm_float64(const void *a, const void *b, double *c, size_t M,
                         size_t N, size_t K, int type_in, int c_order) {
  const size_t a_plane = M * K;
  const size_t b_plane = N * K;
  const size_t c_plane = M * N;
  const size_t c_major_len = (c_order == CCG_ROW_MAJOR) ? N : M;
#pragma omp parallel for collapse(2)
  for (size_t m = 0; m < M; ++m) {
    for (size_t n = 0; n < N; ++n) {
      double sum_re = 0.0;
      double sum_im = 0.0;
      for (size_t k = 0; k < K; ++k) {
        const double ar = load_as_float(a, m * K + k, type_in);
        const double ai = load_as_float(a, a_plane + m * K + k, type_in);
        const double br = load_as_float(b, n * K + k, type_in);
        const double bi = load_as_float(b, b_plane + n * K + k, type_in);
        sum_re += ar * br - ai * bi;
        sum_im += ar * bi + ai * br;
      }
      const size_t major = (c_order == CCG_ROW_MAJOR) ? m : n;
      const size_t minor = (c_order == CCG_ROW_MAJOR) ? n : m;
      c[major * c_major_len + minor] = sum_re;
      c[c_plane + major * c_major_len + minor] = sum_im;
    }
  }
}

/* ---------------------------------------------------------------------- */
/* 1-bit complex GEMM, one batch per call.                                   */
/* Follows src/reference/GEMM.cpp:106-224:                                   */
/*   - K counts 1-bit samples; rows hold ceil(K/32) words (:111-114);        */
/*   - bit 1 is +1, bit 0 is -1, so a product is XOR and a sum is a popcount */
/*     (:131-183); the popcount itself is bit-serial (:97-104);              */
/*   - sum_re = popc(ar^br) + popc(ai^~bi), sum_im = popc(ar^bi)+popc(ai^br) */
/*     (:193-196); re = 2*(Kpadded - sum_re),                                */
/*     im = 2*(Kpadded - padding - sum_im) (:199-200);                       */
/*   - alpha, beta truncated to int, alpha always applied, c always read     */
/*     (:202-221).                                                           */
/* Integer arithmetic wraps modulo 2^32 (unsigned is used to keep that       */
/* well defined in C).                                                       */
/* ---------------------------------------------------------------------- */
static int popcount_serial(uint32_t x) {
  int count = 0;
  while (x) {
    count += (int)(x & 1u);
    x >>= 1;
  }
  return count;
}

void oracle_gemm_int1(const uint32_t *a, const uint32_t *b, int32_t *c,
                      size_t M, size_t N, size_t K, int c_order, float alpha_re,
                      float alpha_im, float beta_re, float beta_im) {
  const size_t k_packed = (K + 31) / 32;
  const size_t k_padded = k_packed * 32;
  const size_t k_padding = k_padded - K;
  const size_t a_plane = M * k_packed;
  const size_t b_plane = N * k_packed;
  const size_t c_plane = M * N;
  const size_t c_major_len = (c_order == CCG_ROW_MAJOR) ? N : M;
  const uint32_t al_re = (uint32_t)(int32_t)alpha_re;
  const uint32_t al_im = (uint32_t)(int32_t)alpha_im;
  const uint32_t be_re = (uint32_t)(int32_t)beta_re;
  const uint32_t be_im = (uint32_t)(int32_t)beta_im;

#pragma omp parallel for collapse(2)
  for (size_t m = 0; m < M; ++m) {
    for (size_t n = 0; n < N; ++n) {
      int pop_re = 0;
      int pop_im = 0;
      for (size_t k = 0; k < k_packed; ++k) {
        const uint32_t ar = a[m * k_packed + k];
        const uint32_t ai = a[a_plane + m * k_packed + k];
        const uint32_t br = b[n * k_packed + k];
        const uint32_t bi = b[b_plane + n * k_packed + k];
        pop_re += popcount_serial(ar ^ br) + popcount_serial(ai ^ ~bi);
        pop_im += popcount_serial(ar ^ bi) + popcount_serial(ai ^ br);
      }
      const uint32_t s_re = 2u * (uint32_t)((int64_t)k_padded - pop_re);
      const uint32_t s_im =
          2u * (uint32_t)((int64_t)k_padded - (int64_t)k_padding - pop_im);
      const uint32_t r_re = al_re * s_re - al_im * s_im;
      const uint32_t r_im = al_im * s_re + al_re * s_im;
      const size_t major = (c_order == CCG_ROW_MAJOR) ? m : n;
      const size_t minor = (c_order == CCG_ROW_MAJOR) ? n : m;
      const size_t idx = major * c_major_len + minor;
      const uint32_t cr = (uint32_t)c[idx];
      const uint32_t ci = (uint32_t)c[c_plane + idx];
      c[idx] = (int32_t)(r_re + be_re * cr - be_im * ci);
      c[c_plane + idx] = (int32_t)(r_im + be_im * cr + be_re * ci);
    }
  }
}

/* ---------------------------------------------------------------------- */
/* Transpose into the tiled layout of the optimised GEMM.                    */
/* Follows kernels/transpose_kernel.cu:40-82:                                */
/*   in  [B][2][M][Nw]           (planar)      or [B][M][Nw][2] (interleaved)*/
/*   out [B][Mp/Mc][Np/Nc][2][Mc][Ncw]                                       */
/* where for 1-bit data Nw = N/32 and Ncw = Nc/32 count 32-bit words          */
/* (:33,57-59), otherwise Nw = N, Ncw = Nc; elements beyond M or N are zero  */
/* (:69-80). elem_bytes is the width moved (1, 2 or 4: :20-30).              */
/* ---------------------------------------------------------------------- */
void oracle_transpose(const void *in, void *out, size_t B, size_t M, size_t N,
                      size_t Mc, size_t Nc, size_t nr_bits, int input_axis) {
  const size_t packing = (nr_bits == 1) ? 32 : 1;
  const size_t eb = (nr_bits == 1) ? 4 : nr_bits / 8;
  const size_t Mp = (M + Mc - 1) / Mc * Mc;
  const size_t Np = (N + Nc - 1) / Nc * Nc;
  const size_t Nw = N / packing;
  const size_t Npw = Np / packing;
  const size_t Ncw = Nc / packing;
  const size_t n_tiles = Npw / Ncw;
  const uint8_t *src = (const uint8_t *)in;
  uint8_t *dst = (uint8_t *)out;

#pragma omp parallel for collapse(2)
  for (size_t b = 0; b < B; ++b) {
    for (size_t m = 0; m < Mp; ++m) {
      for (size_t n = 0; n < Npw; ++n) {
        const size_t mt = m / Mc, mc = m % Mc;
        const size_t nt = n / Ncw, nc = n % Ncw;
        for (size_t z = 0; z < 2; ++z) {
          const size_t o =
              ((((b * (Mp / Mc) + mt) * n_tiles + nt) * 2 + z) * Mc + mc) *
                  Ncw +
              nc;
          if (m < M && n < Nw) {
            const size_t i = (input_axis == CCG_PLANAR)
                                 ? ((b * 2 + z) * M + m) * Nw + n
                                 : ((b * M + m) * Nw + n) * 2 + z;
            memcpy(dst + o * eb, src + i * eb, eb);
          } else {
            memset(dst + o * eb, 0, eb);
          }
        }
      }
    }
  }
}

/* ---------------------------------------------------------------------- */
/* Bit packing. Follows kernels/packing_kernel.cu:7-49 (pack) and :51-62     */
/* (unpack): output bit t of the flat bit stream, LSB first within each      */
/* 32-bit word, is (input byte != 0) at index t (planar) or, for interleaved  */
/* input, at index 2t, minus (N-1) when that is >= N (:15-22), which moves    */
/* all real parts in front of all imaginary parts. Bits beyond N in the last */
/* word are zero.                                                            */
/* ---------------------------------------------------------------------- */
void oracle_pack_bits(const uint8_t *in, uint32_t *out, size_t N,
                      int input_axis) {
  const size_t words = (N + 31) / 32;
#pragma omp parallel for
  for (size_t w = 0; w < words; ++w) {
    uint32_t v = 0;
    for (size_t bit = 0; bit < 32; ++bit) {
      const size_t t = w * 32 + bit;
      if (t >= N) {
        break;
      }
      size_t idx = t;
      if (input_axis == CCG_INTERLEAVED) {
        idx = 2 * t;
        if (idx >= N) {
          idx -= N - 1;
        }
      }
      if (in[idx] != 0) {
        v |= (1u << bit);
      }
    }
    out[w] = v;
  }
}

void oracle_unpack_bits(const uint32_t *in, uint8_t *out, size_t N) {
#pragma omp parallel for
  for (size_t t = 0; t < N; ++t) {
    out[t] = (uint8_t)((in[t / 32] >> (t % 32)) & 1u);
  }
}

/* ceildiv as in include/ccglib/common/helper.h:6-9 (positive operands). */
size_t oracle_ceildiv(size_t a, size_t b) { return a / b + (a % b != 0); }

/*
 * The inputs of the reference's GEMM tests (test/gemm/mma.cpp:144-217): A, then
 * B, filled element by element from ONE rand_r sequence that starts at seed 0 -
 * rand_r / RAND_MAX in float (then converted to the input type by the caller),
 * or the raw value for packed 1-bit words. glibc's rand_r is a fixed algorithm,
 * so this reproduces the reference's numbers. `seed` carries the state from the
 * call for A to the call for B. Exactly one of `values` / `words` is non-null.
 */
void oracle_reference_fixture(float *values, uint32_t *words, size_t n, unsigned *seed) {
  for (size_t i = 0; i < n; ++i) {
    const int r = rand_r(seed);
    if (values) values[i] = (float)r / (float)RAND_MAX;
    if (words) words[i] = (uint32_t)r;
  }
}

/* Number of OpenMP threads the loops above will use. */
#ifdef _OPENMP
#include <omp.h>
int oracle_max_threads(void) { return omp_get_max_threads(); }
void oracle_set_threads(int n) { omp_set_num_threads(n); }
#else
int oracle_max_threads(void) { return 1; }
void oracle_set_threads(int n) { (void)n; }
#endif
