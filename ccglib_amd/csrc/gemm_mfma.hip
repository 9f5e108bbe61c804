// Complex GEMM on the gfx950 matrix cores for fp16, bf16, fp32 and fp8
// (e4m3/e5m2) input with fp32 accumulation, and for 1-bit input (+-1 values on
// the fp4 instruction, exact integer sums; kernels/gemm_kernel_int1.cu:64-356).
//
// Stands in for the reference's wmma_complex_gemm_basic / wmma_complex_gemm_opt
// (kernels/gemm_kernel_float.cu:35-181, :186-355) and its epilogue helpers
// (kernels/matrix_operations.h:38-178). The math is the same four real
// products per complex product (gemm_kernel_float.cu:293-303); everything
// else is laid out for 64-wide wavefronts:
//
//  * One persistent block owns a sequence of BX x BY patches of C and walks K in
//    tiles of 64 bytes per row. Tiles go global -> LDS directly
//    (global_load_lds_dwordx4) through a ring of LDS slots, two iterations ahead
//    of the math: for the tiled (opt) layout, for planar (basic) rows that are
//    whole aligned 16-byte chunks, and for the pipeline's interleaved rows. Only
//    planar rows that are neither (and have no tiled copy) are staged through
//    registers by a second kernel, whose element-wise loads do their bounds
//    checks and zero fill.
//  * LDS rows are 64 bytes with the 16-byte chunk index XORed by a function of
//    the row that suits the fragment shape of the MFMA in use (measured free of
//    bank conflicts; see complex_gemm_mfma_dtl).
//  * 16-bit and 32-bit input: 16x16x32 (16x16x4 for fp32) MFMA; fp8: the
//    32x32x64 f8f6f4 MFMA, which runs at twice the rate of the legacy fp8
//    instruction; 1-bit input: the same instruction on fp4 +-1 values expanded
//    from the packed words in registers.
//  * The four products of a complex MAC reuse the same fragments; the minus
//    sign of Re -= Xi*Yi is a sign-bit flip of the Yi fragment registers.
//  * Workgroup ids are remapped so that consecutive tiles land on the same
//    XCD (shared L2), in groups that reuse both operands.
#include <atomic>
#include <type_traits>
#include <utility>

#include "gemm_device.h"

// Timing-only builds for the kernel-configuration sweep (never for the library):
// a bit mask of parts of the kernels to leave out, which gives wrong numbers and
// shows what each part costs. 1: the C stores (of the register-direct epilogues of
// 16-bit input); 2: the matrix instructions (16-row shapes); 4: the global -> LDS
// copies; 8: the barrier of the K loop.
#ifndef CCGLIB_ABLATE
#define CCGLIB_ABLATE 0
#endif

namespace ccglib_amd {
namespace {

constexpr bool kAblateStores = (CCGLIB_ABLATE & 1) != 0, kAblateMfma = (CCGLIB_ABLATE & 2) != 0,
               kAblateCopies = (CCGLIB_ABLATE & 4) != 0, kAblateBarrier = (CCGLIB_ABLATE & 8) != 0;

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef int int8_t_ __attribute__((ext_vector_type(8)));
typedef unsigned short ushort4_t __attribute__((ext_vector_type(4)));

// K tiles consumed by one MFMA: one for 16-bit input (16x16x32), two for fp8
// (16x16x128: 32 bytes per lane, 16 from each of two K tiles).
template <int DT> struct DtypeTraits {
  static constexpr int kTilesPerMfma = (DT == kFloat8e4m3 || DT == kFloat8e5m2) ? 2 : 1;
  static constexpr int kElemBytes = (DT == kFloat8e4m3 || DT == kFloat8e5m2) ? 1
                                    : (DT == kFloat32)                       ? 4
                                                                             : 2;
  static constexpr unsigned kSignMask = (DT == kFloat8e4m3 || DT == kFloat8e5m2) ? 0x80808080u
                                        : (DT == kFloat32)                         ? 0x80000000u
                                                                                   : 0x80008000u;
};

template <int DT> struct Fragment {
  int4_t v[DtypeTraits<DT>::kTilesPerMfma];
};

template <int DT>
__device__ __forceinline__ float4_t mfma(const Fragment<DT> &a, const Fragment<DT> &b,
                                         float4_t acc) {
  if constexpr (kAblateMfma) {
    // (timing-only build: the operands are still fetched)
    asm volatile("" : "+v"(acc) : "v"(a.v[0]), "v"(b.v[0]));
    return acc;
  }
  if constexpr (DT == kFloat16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(half8_t, a.v[0]), __builtin_bit_cast(half8_t, b.v[0]), acc, 0, 0, 0);
  } else if constexpr (DT == kBfloat16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8_t, a.v[0]), __builtin_bit_cast(bf16x8_t, b.v[0]), acc, 0, 0, 0);
  } else if constexpr (DT == kFloat32) {
    // fp32 input (true fp32 products, no tf32 on this part): a lane's 16-byte
    // chunk is four K values; 16x16x4 takes one value per lane, and which K a
    // lane supplies does not matter as long as both operands agree.
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // (copies first: a bit cast applied to a vector element expression
      // directly reads element 0 whatever the index)
      const int ae = a.v[0][e], be = b.v[0][e];
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, ae),
                                                 __builtin_bit_cast(float, be), acc, 0, 0, 0);
    }
    return acc;
  } else {
    int8_t_ av, bv;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      av[i] = a.v[0][i];
      av[4 + i] = a.v[1][i];
      bv[i] = b.v[0][i];
      bv[4 + i] = b.v[1][i];
    }
    // format code 0 = e4m3, 1 = e5m2; scale exponent 127 = 2^0
    constexpr int fmt = (DT == kFloat8e4m3) ? 0 : 1;
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc, fmt, fmt, 0, 0x7f, 0,
                                                            0x7f);
  }
}

template <int DT>
__device__ __forceinline__ Fragment<DT> negate(const Fragment<DT> &f) {
  Fragment<DT> r;
#pragma unroll
  for (int t = 0; t < DtypeTraits<DT>::kTilesPerMfma; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r.v[t][i] = f.v[t][i] ^ (int)DtypeTraits<DT>::kSignMask;
    }
  }
  return r;
}

// The 32-row MFMAs. A lane holds 32 bytes of one row of the K tile (two
// 16-byte chunks) and 16 accumulators per 32x32 tile. fp8 (32x32x64) eats the
// whole 64-byte row in one instruction, 16-bit input (32x32x16) takes one
// chunk per instruction. One wave alone keeps the MFMA pipe full with these,
// which the 16-row shapes do not on this part (measured 58 % for 16x16x32),
// so the second wave of a SIMD covers the other's LDS and barrier waits.
typedef float float16_t_ __attribute__((ext_vector_type(16)));
struct Fragment32 {
  int4_t v[2];
};

template <int DT>
__device__ __forceinline__ float16_t_ mfma32(const Fragment32 &a, const Fragment32 &b,
                                             float16_t_ acc) {
  if constexpr (DT == kFloat16) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a.v[u]),
                                                   __builtin_bit_cast(half8_t, b.v[u]), acc, 0, 0, 0);
    }
    return acc;
  } else if constexpr (DT == kBfloat16) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a.v[u]),
                                                    __builtin_bit_cast(bf16x8_t, b.v[u]), acc, 0, 0, 0);
    }
    return acc;
  } else {
    int8_t_ av, bv;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      av[i] = a.v[0][i];
      av[4 + i] = a.v[1][i];
      bv[i] = b.v[0][i];
      bv[4 + i] = b.v[1][i];
    }
    constexpr int fmt = (DT == kFloat8e4m3) ? 0 : 1;
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc, fmt, fmt, 0, 0x7f, 0,
                                                           0x7f);
  }
}

// Accumulator of one MFMA tile and how the output is spread over a wave, for
// both MFMA shapes (MS = 16 or 32 rows) and for the 16-row shape with the
// operand roles exchanged (kAcc16T: X is the MFMA "B" operand and tile i of a
// wave holds the columns x = 4 (lane % 16) + i, see complex_gemm_mfma_dtl).
// A lane holds "pieces" of four consecutive x (the contiguous C axis) at one y:
//   MS 16:   piece (jj, ii) at x = 16 ii + 4 (lane / 16), y = 16 jj + lane % 16
//   MS 32:   piece (jj, ii) at x = 32 (ii / 4) + 8 (ii % 4) + 4 (lane / 32), y = 32 jj + lane % 32
//   kAcc16T: piece (jj, ii) at x = 4 (lane % 16), y = 16 jj + 4 (lane / 16) + ii; its four
//            elements are register ii of the four tiles of tile row jj
constexpr int kAcc16T = 116;
template <int MS> struct AccType { using type = float4_t; };
template <> struct AccType<32> { using type = float16_t_; };

template <int MS> __device__ __forceinline__ unsigned piece_x(int ii, int lane) {
  if constexpr (MS == kAcc16T) return (lane & 15) * 4;
  return MS == 16 ? ii * 16 + (lane >> 4) * 4 : (ii >> 2) * 32 + (ii & 3) * 8 + (lane >> 5) * 4;
}
template <int MS> __device__ __forceinline__ unsigned piece_y(int jj, int ii, int lane) {
  if constexpr (MS == kAcc16T) return jj * 16 + (lane >> 4) * 4 + ii;
  return MS == 16 ? jj * 16 + (lane & 15) : jj * 32 + (lane & 31);
}
// (TILE0: kAcc16T only, the first of the four tiles when a wave's tile rows hold more)
template <int MS, int TILE0 = 0, typename Acc>
__device__ __forceinline__ float piece_elem(const Acc &acc, int jj, int ii, int e) {
  if constexpr (MS == kAcc16T) {
    return acc[jj][TILE0 + e][ii];
  } else if constexpr (MS == 16) {
    return acc[jj][ii][e];
  } else {
    return acc[jj][ii >> 2][(ii & 3) * 4 + e];
  }
}

template <int TOUT> struct OutType;
template <> struct OutType<kFloat32> { using type = float; };
template <> struct OutType<kFloat16> { using type = _Float16; };
template <> struct OutType<kBfloat16> { using type = __bf16; };
template <> struct OutType<kInt32> { using type = int; };

// One K tile (or two for fp8) of math for a wave: reads its X and Y fragments
// from the LDS slot(s) and issues the four real products of the complex MAC.
// slot[u] points at the K tile u of this MFMA step: [X re][X im][Y re][Y im].
template <int DT, int BX, int BY, int TX, int TY, typename Mid>
__device__ __forceinline__ void mma_step(const char *const (&slot)[DtypeTraits<DT>::kTilesPerMfma],
                                         int x_frag_off, int y_frag_off,
                                         float4_t (&acc_re)[TY][TX], float4_t (&acc_im)[TY][TX],
                                         Mid &&mid) {
  constexpr int KPM = DtypeTraits<DT>::kTilesPerMfma;
  Fragment<DT> xr[TX], xi[TX];
#pragma unroll
  for (int i = 0; i < TX; ++i) {
#pragma unroll
    for (int u = 0; u < KPM; ++u) {
      const char *p = slot[u] + x_frag_off + i * 16 * kTileRowBytes;
      xr[i].v[u] = *reinterpret_cast<const int4_t *>(p);
      xi[i].v[u] = *reinterpret_cast<const int4_t *>(p + BX * kTileRowBytes);
    }
  }
#pragma unroll
  for (int j = 0; j < TY; ++j) {
    Fragment<DT> yr, yi;
#pragma unroll
    for (int u = 0; u < KPM; ++u) {
      const char *p = slot[u] + y_frag_off + j * 16 * kTileRowBytes;
      yr.v[u] = *reinterpret_cast<const int4_t *>(p);
      yi.v[u] = *reinterpret_cast<const int4_t *>(p + BY * kTileRowBytes);
    }
    const Fragment<DT> yin = negate<DT>(yi);
#pragma unroll
    for (int i = 0; i < TX; ++i) acc_re[j][i] = mfma<DT>(xr[i], yr, acc_re[j][i]);
#pragma unroll
    for (int i = 0; i < TX; ++i) acc_im[j][i] = mfma<DT>(xr[i], yi, acc_im[j][i]);
#pragma unroll
    for (int i = 0; i < TX; ++i) acc_re[j][i] = mfma<DT>(xi[i], yin, acc_re[j][i]);
#pragma unroll
    for (int i = 0; i < TX; ++i) acc_im[j][i] = mfma<DT>(xi[i], yr, acc_im[j][i]);
    if (j == 0) mid();
  }
}

// The same step with every LDS read placed by hand, for one K tile per MFMA and
// a 4 x 4 wave tile. Right after the barrier all waves of the block want their
// fragments at once and the LDS serves them one read at a time; if a wave asks
// for all ten fragments of the first tile row before its first MFMA, the matrix
// cores wait for the whole queue. Here a wave reads what its first MFMA needs,
// keeps about three reads in flight ahead of their use, and fetches the Y
// fragments of the next tile row during the current one.
// xo[i] is the lane's offset of the X fragment of tile i. XT: the operand roles
// of the MFMA are exchanged (Y supplies the instruction's "A" rows, X its "B"
// columns), which transposes what a lane holds of every 16 x 16 tile.
// FIRST: the first K tile of a C tile; the sums start from zero.
// xa[i] / ya: the lane's LDS address of the X fragment of tile i / of the Y
// fragment of tile row 0 in the current slots. late(): called among the MFMAs
// of the last tile row, for whatever the next iteration needs computed (its
// addresses, the slot numbers): work placed there is hidden behind MFMAs, work
// left between the last MFMA and the barrier is not.
template <int DT, int BX, int BY, bool XT, bool FIRST, typename Mid, typename Late>
__device__ __forceinline__ void mma_step_ordered(const unsigned (&xa)[4], unsigned ya,
                                                 float4_t (&acc_re)[4][4], float4_t (&acc_im)[4][4],
                                                 Mid &&mid, Late &&late) {
  static_assert(DtypeTraits<DT>::kTilesPerMfma == 1, "one K tile per MFMA");
  // (LDS addresses as 32-bit numbers: the read's address register is the number itself)
  typedef __attribute__((address_space(3))) const int4_t lds_int4_t;
  auto rd = [](unsigned address) {
    Fragment<DT> f;
    f.v[0] = *reinterpret_cast<lds_int4_t *>(address);
    return f;
  };
  auto mm = [](const Fragment<DT> &x, const Fragment<DT> &y, float4_t acc) {
    return XT ? mfma<DT>(y, x, acc) : mfma<DT>(x, y, acc);
  };
  auto c0 = [](const float4_t &acc) { return FIRST ? float4_t{0.f, 0.f, 0.f, 0.f} : acc; };
  constexpr int ROW16 = 16 * kTileRowBytes, XP = BX * kTileRowBytes, YP = BY * kTileRowBytes;
#define CCGLIB_PIN __builtin_amdgcn_sched_barrier(0)
  Fragment<DT> xr[4], xi[4], yr, yi, yin, yr_next, yi_next;
  yr = rd(ya);
  xr[0] = rd(xa[0]);
  xr[1] = rd(xa[1]);
  xr[2] = rd(xa[2]);
  CCGLIB_PIN;
  acc_re[0][0] = mm(xr[0], yr, c0(acc_re[0][0]));
  xr[3] = rd(xa[3]);
  CCGLIB_PIN;
  acc_re[0][1] = mm(xr[1], yr, c0(acc_re[0][1]));
  yi = rd(ya + YP);
  CCGLIB_PIN;
  acc_re[0][2] = mm(xr[2], yr, c0(acc_re[0][2]));
  xi[0] = rd(xa[0] + XP);
  CCGLIB_PIN;
  acc_re[0][3] = mm(xr[3], yr, c0(acc_re[0][3]));
  xi[1] = rd(xa[1] + XP);
  CCGLIB_PIN;
  acc_im[0][0] = mm(xr[0], yi, c0(acc_im[0][0]));
  xi[2] = rd(xa[2] + XP);
  CCGLIB_PIN;
  acc_im[0][1] = mm(xr[1], yi, c0(acc_im[0][1]));
  xi[3] = rd(xa[3] + XP);
  CCGLIB_PIN;
  acc_im[0][2] = mm(xr[2], yi, c0(acc_im[0][2]));
  yin = negate<DT>(yi);
  CCGLIB_PIN;
  acc_im[0][3] = mm(xr[3], yi, c0(acc_im[0][3]));
  yr_next = rd(ya + ROW16);
  CCGLIB_PIN;
  acc_re[0][0] = mm(xi[0], yin, acc_re[0][0]);
  yi_next = rd(ya + YP + ROW16);
  CCGLIB_PIN;
  acc_im[0][0] = mm(xi[0], yr, acc_im[0][0]);
#pragma unroll
  for (int i = 1; i < 4; ++i) {
    acc_re[0][i] = mm(xi[i], yin, acc_re[0][i]);
    acc_im[0][i] = mm(xi[i], yr, acc_im[0][i]);
  }
  CCGLIB_PIN;
  mid();
  CCGLIB_PIN;
#pragma unroll
  for (int j = 1; j < 4; ++j) {
    yr = yr_next;
    yi = yi_next;
    yin = negate<DT>(yi);
    CCGLIB_PIN;
    // from one MFMA to the next only one of the two operands changes (measured 1-2 %
    // faster on random data than four MFMAs per Y fragment in a row: the part is
    // power limited, and this order toggles fewer operand bits)
    acc_re[j][0] = mm(xr[0], yr, c0(acc_re[j][0]));
    acc_im[j][0] = mm(xr[0], yi, c0(acc_im[j][0]));
    acc_im[j][1] = mm(xr[1], yi, c0(acc_im[j][1]));
    acc_re[j][1] = mm(xr[1], yr, c0(acc_re[j][1]));
    if (j < 3) yr_next = rd(ya + (j + 1) * ROW16);
    CCGLIB_PIN;
    acc_re[j][2] = mm(xr[2], yr, c0(acc_re[j][2]));
    acc_im[j][2] = mm(xr[2], yi, c0(acc_im[j][2]));
    acc_im[j][3] = mm(xr[3], yi, c0(acc_im[j][3]));
    acc_re[j][3] = mm(xr[3], yr, c0(acc_re[j][3]));
    if (j < 3) yi_next = rd(ya + YP + (j + 1) * ROW16);
    CCGLIB_PIN;
    if (j == 3) {
      late();
      CCGLIB_PIN;
    }
    acc_im[j][0] = mm(xi[0], yr, acc_im[j][0]);
    acc_re[j][0] = mm(xi[0], yin, acc_re[j][0]);
    acc_re[j][1] = mm(xi[1], yin, acc_re[j][1]);
    acc_im[j][1] = mm(xi[1], yr, acc_im[j][1]);
    acc_im[j][2] = mm(xi[2], yr, acc_im[j][2]);
    acc_re[j][2] = mm(xi[2], yin, acc_re[j][2]);
    acc_re[j][3] = mm(xi[3], yin, acc_re[j][3]);
    acc_im[j][3] = mm(xi[3], yr, acc_im[j][3]);
    CCGLIB_PIN;
  }
#undef CCGLIB_PIN
}

// The same on the 32-row MFMAs: TX x TY tiles of 32x32, one K tile per step.
// off[0] and off[1] are the lane's two 16-byte chunks of its row.
template <int DT, int BX, int BY, int TX, int TY, typename Mid>
__device__ __forceinline__ void mma_step32(const char *slot, const int (&x_off)[2],
                                           const int (&y_off)[2], float16_t_ (&acc_re)[TY][TX],
                                           float16_t_ (&acc_im)[TY][TX], Mid &&mid) {
  constexpr int D = TX > TY ? TX : TY;
  Fragment32 xr[TX], xi[TX], yr[TY], yi[TY], yin[TY];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    if (d < TX) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const char *p = slot + x_off[u] + d * 32 * kTileRowBytes;
        xr[d].v[u] = *reinterpret_cast<const int4_t *>(p);
        xi[d].v[u] = *reinterpret_cast<const int4_t *>(p + BX * kTileRowBytes);
      }
    }
    if (d < TY) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const char *p = slot + y_off[u] + d * 32 * kTileRowBytes;
        yr[d].v[u] = *reinterpret_cast<const int4_t *>(p);
        yi[d].v[u] = *reinterpret_cast<const int4_t *>(p + BY * kTileRowBytes);
      }
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d) {
    __builtin_amdgcn_sched_barrier(0);
    if (d < TY) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int w = 0; w < 4; ++w) yin[d].v[u][w] = yi[d].v[u][w] ^ (int)DtypeTraits<DT>::kSignMask;
      }
    }
    int ti[TX + TY], tj[TX + TY], n = 0;
    if (d < TX) {
#pragma unroll
      for (int j = 0; j < d && j < TY; ++j) ti[n] = d, tj[n] = j, ++n;
    }
    if (d < TY) {
#pragma unroll
      for (int i = 0; i <= d && i < TX; ++i) ti[n] = i, tj[n] = d, ++n;
    }
#pragma unroll
    for (int t = 0; t < n; ++t)
      acc_re[tj[t]][ti[t]] = mfma32<DT>(xr[ti[t]], yr[tj[t]], acc_re[tj[t]][ti[t]]);
#pragma unroll
    for (int t = 0; t < n; ++t)
      acc_im[tj[t]][ti[t]] = mfma32<DT>(xr[ti[t]], yi[tj[t]], acc_im[tj[t]][ti[t]]);
#pragma unroll
    for (int t = 0; t < n; ++t)
      acc_re[tj[t]][ti[t]] = mfma32<DT>(xi[ti[t]], yin[tj[t]], acc_re[tj[t]][ti[t]]);
#pragma unroll
    for (int t = 0; t < n; ++t)
      acc_im[tj[t]][ti[t]] = mfma32<DT>(xi[ti[t]], yr[tj[t]], acc_im[tj[t]][ti[t]]);
    if (d == 0) {
      __builtin_amdgcn_sched_barrier(0);
      mid();
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

// The 32-row step for a 2 x 2 wave tile with the LDS reads in order of need
// (see mma_step_ordered): two 16-byte reads per fragment.
template <int DT, int BX, int BY, typename Mid>
__device__ __forceinline__ void mma_step32_ordered(const char *slot, const int (&x_off)[2],
                                                   const int (&y_off)[2], float16_t_ (&acc_re)[2][2],
                                                   float16_t_ (&acc_im)[2][2], Mid &&mid) {
  auto rd = [&](const int (&off)[2], int extra) {
    Fragment32 f;
    f.v[0] = *reinterpret_cast<const int4_t *>(slot + off[0] + extra);
    f.v[1] = *reinterpret_cast<const int4_t *>(slot + off[1] + extra);
    return f;
  };
  auto neg = [](const Fragment32 &f) {
    Fragment32 r;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int w = 0; w < 4; ++w) r.v[u][w] = f.v[u][w] ^ (int)DtypeTraits<DT>::kSignMask;
    }
    return r;
  };
  constexpr int ROW32 = 32 * kTileRowBytes, XP = BX * kTileRowBytes, YP = BY * kTileRowBytes;
#define CCGLIB_PIN __builtin_amdgcn_sched_barrier(0)
  Fragment32 x0r, x0i, x1r, x1i, y0r, y0i, y0n, y1r, y1i, y1n;
  y0r = rd(y_off, 0);
  x0r = rd(x_off, 0);
  y0i = rd(y_off, YP);
  CCGLIB_PIN;
  acc_re[0][0] = mfma32<DT>(x0r, y0r, acc_re[0][0]);
  x0i = rd(x_off, XP);
  CCGLIB_PIN;
  acc_im[0][0] = mfma32<DT>(x0r, y0i, acc_im[0][0]);
  y0n = neg(y0i);
  x1r = rd(x_off, ROW32);
  CCGLIB_PIN;
  acc_re[0][0] = mfma32<DT>(x0i, y0n, acc_re[0][0]);
  x1i = rd(x_off, XP + ROW32);
  CCGLIB_PIN;
  acc_im[0][0] = mfma32<DT>(x0i, y0r, acc_im[0][0]);
  CCGLIB_PIN;
  mid();
  CCGLIB_PIN;
  acc_re[0][1] = mfma32<DT>(x1r, y0r, acc_re[0][1]);
  y1r = rd(y_off, ROW32);
  CCGLIB_PIN;
  acc_im[0][1] = mfma32<DT>(x1r, y0i, acc_im[0][1]);
  y1i = rd(y_off, YP + ROW32);
  CCGLIB_PIN;
  acc_re[0][1] = mfma32<DT>(x1i, y0n, acc_re[0][1]);
  acc_im[0][1] = mfma32<DT>(x1i, y0r, acc_im[0][1]);
  CCGLIB_PIN;
  acc_re[1][0] = mfma32<DT>(x0r, y1r, acc_re[1][0]);
  acc_im[1][0] = mfma32<DT>(x0r, y1i, acc_im[1][0]);
  y1n = neg(y1i);
  CCGLIB_PIN;
  acc_re[1][0] = mfma32<DT>(x0i, y1n, acc_re[1][0]);
  acc_im[1][0] = mfma32<DT>(x0i, y1r, acc_im[1][0]);
  acc_re[1][1] = mfma32<DT>(x1r, y1r, acc_re[1][1]);
  acc_im[1][1] = mfma32<DT>(x1r, y1i, acc_im[1][1]);
  acc_re[1][1] = mfma32<DT>(x1i, y1n, acc_re[1][1]);
  acc_im[1][1] = mfma32<DT>(x1i, y1r, acc_im[1][1]);
  CCGLIB_PIN;
#undef CCGLIB_PIN
}

// 1-bit samples, multiplied on the fp4 MFMA straight from the packed words.
// A 64-byte row of a slot holds 512 samples; a lane reads its two 16-byte
// chunks of a row as for the other 32-row MFMAs, and each of the eight words
// it then holds feeds one 32x32x64 MFMA (64 samples of K: 32 from each half of
// the wave). A word becomes the MFMA's four operand registers with seven
// vector-ALU instructions: nibble i of register j is 0x2 | bit (4 i + j) << 3,
// i.e. fp4 +1.0 for a 0 bit and -1.0 for a 1 bit. Which sample lands in which
// K position of the instruction does not matter as long as X and Y agree, and
// neither does the sign convention (bit 1 = +1 in src/reference/GEMM.cpp:131-200):
// negating X and Y together leaves every product as it is. The expansion of the
// fragment that is needed two to four MFMAs later is placed behind each MFMA,
// in whose shadow the vector ALU is otherwise idle; the MFMAs are issued so
// that only one operand changes from one to the next.
// Samples past K (zero bits in both operands, which the tiled layout and the
// zero tile guarantee) add 0 to every real and +2 to every imaginary sum; the
// epilogue takes that off (KernelArgs::im_excess), which is the reference's
// K_PADDING correction (kernels/gemm_kernel_int1.cu:64-196).
__device__ __forceinline__ int4_t expand_bits(int word) {
  const unsigned w = (unsigned)word;
  int4_t o;
  // (a & b) | c in one instruction (truth table 0xEA)
  o[0] = (int)__builtin_amdgcn_bitop3_b32(w << 3, 0x88888888u, 0x22222222u, 0xEA);
  o[1] = (int)__builtin_amdgcn_bitop3_b32(w << 2, 0x88888888u, 0x22222222u, 0xEA);
  o[2] = (int)__builtin_amdgcn_bitop3_b32(w << 1, 0x88888888u, 0x22222222u, 0xEA);
  o[3] = (int)__builtin_amdgcn_bitop3_b32(w, 0x88888888u, 0x22222222u, 0xEA);
  return o;
}

__device__ __forceinline__ float16_t_ mfma_fp4(const int4_t &a, const int4_t &b, float16_t_ acc) {
  // format code 4 = fp4 (only the low four registers are read); scale 2^0
  const int8_t_ av = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
  const int8_t_ bv = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc, 4, 4, 0, 0x7f, 0, 0x7f);
}

template <int BX, int BY, typename Mid>
__device__ __forceinline__ void mma_step32_bits(const char *slot, const int (&x_off)[2],
                                                const int (&y_off)[2], float16_t_ (&acc_re)[2][2],
                                                float16_t_ (&acc_im)[2][2], Mid &&mid) {
  constexpr int ROW32 = 32 * kTileRowBytes, XP = BX * kTileRowBytes, YP = BY * kTileRowBytes;
  // fragments: 0 x0r, 1 x0i, 2 x1r, 3 x1i, 4 y0r, 5 y0i, 6 y1r, 7 y1i
  enum { X0R, X0I, X1R, X1I, Y0R, Y0I, Y1R, Y1I };
  int4_t raw[8];    // the chunk (four words, one per MFMA step) in use
  auto rd = [&](int f, int u) {
    const int off = (f < 4 ? x_off[u] : y_off[u]) + ((f & 1) ? (f < 4 ? XP : YP) : 0) +
                    ((f & 2) ? ROW32 : 0);
    raw[f] = *reinterpret_cast<const int4_t *>(slot + off);
  };
  auto neg = [](const int4_t &f) {
    int4_t r;
#pragma unroll
    for (int w = 0; w < 4; ++w) r[w] = f[w] ^ (int)0x88888888u;
    return r;
  };
#define CCGLIB_PIN __builtin_amdgcn_sched_barrier(0)
  // in order of first use
  rd(X0R, 0);
  rd(Y0R, 0);
  rd(Y0I, 0);
  rd(Y1I, 0);
  rd(Y1R, 0);
  rd(X1R, 0);
  rd(X1I, 0);
  rd(X0I, 0);
  CCGLIB_PIN;
  int4_t x0r = expand_bits(raw[X0R][0]), y0r = expand_bits(raw[Y0R][0]),
         y0i = expand_bits(raw[Y0I][0]);
  int4_t x0i, x1r, x1i, y1r, y1i, y0n, y1n, x0r_next, y0r_next, y0i_next;
  CCGLIB_PIN;
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const int w = s & 3;
    // after a chunk's last word has been taken, the next chunk of the row is read
    // into the same registers (its first word is needed sixteen MFMAs later)
    const bool reload = (s == 3);
    const bool reload_next = (s == 2);   // for the fragments expanded one step ahead
    acc_re[0][0] = mfma_fp4(x0r, y0r, acc_re[0][0]);
    y1i = expand_bits(raw[Y1I][w]);
    if (reload) rd(Y1I, 1);
    CCGLIB_PIN;
    acc_im[0][0] = mfma_fp4(x0r, y0i, acc_im[0][0]);
    y1r = expand_bits(raw[Y1R][w]);
    if (reload) rd(Y1R, 1);
    CCGLIB_PIN;
    acc_im[1][0] = mfma_fp4(x0r, y1i, acc_im[1][0]);
    x1r = expand_bits(raw[X1R][w]);
    if (reload) rd(X1R, 1);
    CCGLIB_PIN;
    acc_re[1][0] = mfma_fp4(x0r, y1r, acc_re[1][0]);
    x1i = expand_bits(raw[X1I][w]);
    if (reload) rd(X1I, 1);
    CCGLIB_PIN;
    if (s == 0) {
      mid();
      CCGLIB_PIN;
    }
    acc_re[1][1] = mfma_fp4(x1r, y1r, acc_re[1][1]);
    y0n = neg(y0i);
    CCGLIB_PIN;
    acc_im[1][1] = mfma_fp4(x1r, y1i, acc_im[1][1]);
    y1n = neg(y1i);
    CCGLIB_PIN;
    acc_im[0][1] = mfma_fp4(x1r, y0i, acc_im[0][1]);
    x0i = expand_bits(raw[X0I][w]);
    if (reload) rd(X0I, 1);
    CCGLIB_PIN;
    acc_re[0][1] = mfma_fp4(x1r, y0r, acc_re[0][1]);
    CCGLIB_PIN;
    acc_im[0][1] = mfma_fp4(x1i, y0r, acc_im[0][1]);
    CCGLIB_PIN;
    acc_re[0][1] = mfma_fp4(x1i, y0n, acc_re[0][1]);
    if (s < 7) x0r_next = expand_bits(raw[X0R][(s + 1) & 3]);
    if (reload_next) rd(X0R, 1);
    CCGLIB_PIN;
    acc_re[1][1] = mfma_fp4(x1i, y1n, acc_re[1][1]);
    if (s < 7) y0r_next = expand_bits(raw[Y0R][(s + 1) & 3]);
    if (reload_next) rd(Y0R, 1);
    CCGLIB_PIN;
    acc_im[1][1] = mfma_fp4(x1i, y1r, acc_im[1][1]);
    if (s < 7) y0i_next = expand_bits(raw[Y0I][(s + 1) & 3]);
    if (reload_next) rd(Y0I, 1);
    CCGLIB_PIN;
    acc_im[1][0] = mfma_fp4(x0i, y1r, acc_im[1][0]);
    acc_re[1][0] = mfma_fp4(x0i, y1n, acc_re[1][0]);
    acc_re[0][0] = mfma_fp4(x0i, y0n, acc_re[0][0]);
    acc_im[0][0] = mfma_fp4(x0i, y0r, acc_im[0][0]);
    CCGLIB_PIN;
    if (s < 7) {
      x0r = x0r_next;
      y0r = y0r_next;
      y0i = y0i_next;
    }
  }
#undef CCGLIB_PIN
}

// The same for interleaved operands (rows of (re, im) pairs, as the caller's
// buffers hold them). With K running over the 2K real numbers of a row,
//   Re = sum X~ . Y1,  Y1 = (yr, -yi, ...)   and   Im = sum X~ . Y2,  Y2 = (yi, yr, ...)
// so the raw X fragment is used as it is and both Y variants come from the raw
// Y fragment in registers: a sign flip of the odd elements and a swap inside
// each pair. Two MFMAs per fragment pair over half as many complex values:
// the same MFMA and LDS work per complex MAC as with planar operands.
template <int DT, int BX, int BY, int TX, int TY, typename Mid>
__device__ __forceinline__ void mma_step_interleaved(const char *slot, const int (&x_off)[2],
                                                     const int (&y_off)[2],
                                                     float4_t (&acc_re)[TY][TX],
                                                     float4_t (&acc_im)[TY][TX], Mid &&mid) {
  // The slot holds 128 bytes of every row; x_off / y_off are the lane's two
  // 16-byte chunks of its row. fp8 takes both in one MFMA, 16-bit input one
  // per MFMA (two passes over the slot).
  constexpr int KPM = DtypeTraits<DT>::kTilesPerMfma;
  constexpr int PASSES = 2 / KPM;
  constexpr bool kBytes = DtypeTraits<DT>::kElemBytes == 1;
#pragma unroll
  for (int h = 0; h < PASSES; ++h) {
    Fragment<DT> x[TX];
#pragma unroll
    for (int i = 0; i < TX; ++i) {
#pragma unroll
      for (int u = 0; u < KPM; ++u) {
        x[i].v[u] = *reinterpret_cast<const int4_t *>(slot + x_off[h * KPM + u] + i * 16 * 128);
      }
    }
#pragma unroll
    for (int j = 0; j < TY; ++j) {
      Fragment<DT> y1, y2;
#pragma unroll
      for (int u = 0; u < KPM; ++u) {
        const int4_t raw =
            *reinterpret_cast<const int4_t *>(slot + y_off[h * KPM + u] + j * 16 * 128);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const unsigned v = (unsigned)raw[w];
          y1.v[u][w] = (int)(v ^ (kBytes ? 0x80008000u : 0x80000000u));
          y2.v[u][w] = kBytes ? (int)__builtin_amdgcn_perm(v, v, 0x02030001u)
                              : (int)__builtin_amdgcn_alignbit(v, v, 16);
        }
      }
#pragma unroll
      for (int i = 0; i < TX; ++i) acc_re[j][i] = mfma<DT>(x[i], y1, acc_re[j][i]);
#pragma unroll
      for (int i = 0; i < TX; ++i) acc_im[j][i] = mfma<DT>(x[i], y2, acc_im[j][i]);
      if (h == 0 && j == 0) mid();
    }
  }
}

// The interleaved step for 16-bit input and a 4 x 4 wave tile with every LDS
// read and every derived fragment placed by hand (see mma_step_ordered). The
// slot is walked as eight tile rows (two halves of K x four rows of Y). The raw
// Y fragment of a row is read two rows ahead; its two variants are computed
// during the previous row, two instructions behind each of that row's last
// four MFMAs, where they issue in the shadow of the matrix instruction instead
// of holding up the next row; the X fragments of the second half are fetched
// during rows 2 and 3.
template <int DT, int BX, int BY, typename Mid>
__device__ __forceinline__ void mma_step_interleaved_ordered(const char *slot, const int (&x_off)[2],
                                                             const int (&y_off)[2],
                                                             float4_t (&acc_re)[4][4],
                                                             float4_t (&acc_im)[4][4], Mid &&mid) {
  static_assert(DtypeTraits<DT>::kTilesPerMfma == 1 && DtypeTraits<DT>::kElemBytes == 2,
                "16-bit input");
  auto rd = [&](int off) {
    Fragment<DT> f;
    f.v[0] = *reinterpret_cast<const int4_t *>(slot + off);
    return f;
  };
  // words w0, w0 + 1 of (yr, -yi, ...) and of (yi, yr, ...) from the raw (yr, yi, ...).
  // The empty asm statement takes the result where it is computed: without it,
  // arithmetic whose result is first used in the next row is sunk there before
  // the instructions are scheduled. (The arithmetic itself stays ordinary code,
  // so the compiler keeps track of the wait states the MFMAs need.)
  auto flip2 = [](Fragment<DT> &f, const Fragment<DT> &raw, int w0) {
#pragma unroll
    for (int w = w0; w < w0 + 2; ++w) {
      int o = (int)((unsigned)raw.v[0][w] ^ 0x80000000u);
      asm volatile("" : "+v"(o));
      f.v[0][w] = o;
    }
  };
  auto swap2 = [](Fragment<DT> &f, const Fragment<DT> &raw, int w0) {
#pragma unroll
    for (int w = w0; w < w0 + 2; ++w) {
      const unsigned v = (unsigned)raw.v[0][w];
      int o = (int)__builtin_amdgcn_alignbit(v, v, 16);
      asm volatile("" : "+v"(o));
      f.v[0][w] = o;
    }
  };
  constexpr int ROW16 = 16 * 128;
  auto y_row_off = [&](int r) { return y_off[r >> 2] + (r & 3) * ROW16; };
#define CCGLIB_PIN __builtin_amdgcn_sched_barrier(0)
  Fragment<DT> xa[4], xb[4], raw[2], y1, y2, y1n, y2n;
  raw[0] = rd(y_row_off(0));
  xa[0] = rd(x_off[0]);
  xa[1] = rd(x_off[0] + ROW16);
  raw[1] = rd(y_row_off(1));
  xa[2] = rd(x_off[0] + 2 * ROW16);
  CCGLIB_PIN;
  flip2(y1, raw[0], 0);
  flip2(y1, raw[0], 2);
  swap2(y2, raw[0], 0);
  swap2(y2, raw[0], 2);
  CCGLIB_PIN;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int j = r & 3;
    Fragment<DT>(&x)[4] = r < 4 ? xa : xb;
    const Fragment<DT> &next_raw = raw[(r + 1) & 1];
    acc_re[j][0] = mfma<DT>(x[0], y1, acc_re[j][0]);
    if (r == 0) xa[3] = rd(x_off[0] + 3 * ROW16);
    if (r + 2 < 8) raw[r & 1] = rd(y_row_off(r + 2));   // this row's raw fragment is used up
    CCGLIB_PIN;
    acc_im[j][0] = mfma<DT>(x[0], y2, acc_im[j][0]);
    if (r == 2 || r == 3) xb[2 * (r - 2)] = rd(x_off[1] + 2 * (r - 2) * ROW16);
    CCGLIB_PIN;
    // (from one MFMA to the next only one of the two operands changes)
    acc_im[j][1] = mfma<DT>(x[1], y2, acc_im[j][1]);
    if (r == 2 || r == 3) xb[2 * (r - 2) + 1] = rd(x_off[1] + (2 * (r - 2) + 1) * ROW16);
    CCGLIB_PIN;
    acc_re[j][1] = mfma<DT>(x[1], y1, acc_re[j][1]);
    CCGLIB_PIN;
    acc_re[j][2] = mfma<DT>(x[2], y1, acc_re[j][2]);
    if (r + 1 < 8) flip2(y1n, next_raw, 0);
    CCGLIB_PIN;
    acc_im[j][2] = mfma<DT>(x[2], y2, acc_im[j][2]);
    if (r + 1 < 8) flip2(y1n, next_raw, 2);
    CCGLIB_PIN;
    acc_im[j][3] = mfma<DT>(x[3], y2, acc_im[j][3]);
    if (r + 1 < 8) swap2(y2n, next_raw, 0);
    CCGLIB_PIN;
    acc_re[j][3] = mfma<DT>(x[3], y1, acc_re[j][3]);
    if (r + 1 < 8) swap2(y2n, next_raw, 2);
    CCGLIB_PIN;
    if (r == 0) {
      mid();
      CCGLIB_PIN;
    }
    y1 = y1n;
    y2 = y2n;
  }
#undef CCGLIB_PIN
}

// Interleaved 8-bit operands on the 32-row MFMA: a 2 x 2 wave tile of 32 x 32
// tiles; the slot holds 128 bytes (64 (re, im) pairs) of every row, walked in two
// halves of 64 bytes, one MFMA step each. off[h][u] are the lane's two 16-byte
// chunks of its row in half h. As for 16-bit input the raw X fragment is used
// as it is and both Y variants come from the raw Y fragment: a sign flip of the
// odd bytes and a swap inside each byte pair. LDS reads are placed by hand, a
// fragment being fetched about four MFMAs (of 32 cycles) ahead of its use.
template <int DT, int BX, int BY, typename Mid>
__device__ __forceinline__ void mma_step32_interleaved(const char *slot, const int (&x_off)[2][2],
                                                       const int (&y_off)[2][2],
                                                       float16_t_ (&acc_re)[2][2],
                                                       float16_t_ (&acc_im)[2][2], Mid &&mid) {
  static_assert(DtypeTraits<DT>::kElemBytes == 1, "8-bit input");
  auto rd = [&](const int (&off)[2], int extra) {
    Fragment32 f;
    f.v[0] = *reinterpret_cast<const int4_t *>(slot + off[0] + extra);
    f.v[1] = *reinterpret_cast<const int4_t *>(slot + off[1] + extra);
    return f;
  };
  auto flip = [](const Fragment32 &raw) {      // (yr, -yi, ...)
    Fragment32 f;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int w = 0; w < 4; ++w) f.v[u][w] = (int)((unsigned)raw.v[u][w] ^ 0x80008000u);
    }
    return f;
  };
  auto swap = [](const Fragment32 &raw) {      // (yi, yr, ...)
    Fragment32 f;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const unsigned v = (unsigned)raw.v[u][w];
        f.v[u][w] = (int)__builtin_amdgcn_perm(v, v, 0x02030001u);
      }
    }
    return f;
  };
  constexpr int ROW32 = 32 * 128;
#define CCGLIB_PIN __builtin_amdgcn_sched_barrier(0)
  Fragment32 x0, x1, raw0, raw1, ya, yb;
  raw0 = rd(y_off[0], 0);
  x0 = rd(x_off[0], 0);
  x1 = rd(x_off[0], ROW32);
  CCGLIB_PIN;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    ya = flip(raw0);
    yb = swap(raw0);
    CCGLIB_PIN;
    acc_re[0][0] = mfma32<DT>(x0, ya, acc_re[0][0]);
    raw1 = rd(y_off[h], ROW32);
    CCGLIB_PIN;
    acc_im[0][0] = mfma32<DT>(x0, yb, acc_im[0][0]);
    CCGLIB_PIN;
    if (h == 0) {
      mid();
      CCGLIB_PIN;
    }
    acc_re[0][1] = mfma32<DT>(x1, ya, acc_re[0][1]);
    if (h == 0) raw0 = rd(y_off[1], 0);
    CCGLIB_PIN;
    acc_im[0][1] = mfma32<DT>(x1, yb, acc_im[0][1]);
    ya = flip(raw1);
    yb = swap(raw1);
    CCGLIB_PIN;
    acc_re[1][0] = mfma32<DT>(x0, ya, acc_re[1][0]);
    acc_im[1][0] = mfma32<DT>(x0, yb, acc_im[1][0]);
    if (h == 0) x0 = rd(x_off[1], 0);
    CCGLIB_PIN;
    acc_re[1][1] = mfma32<DT>(x1, ya, acc_re[1][1]);
    acc_im[1][1] = mfma32<DT>(x1, yb, acc_im[1][1]);
    if (h == 0) x1 = rd(x_off[1], ROW32);
    CCGLIB_PIN;
  }
#undef CCGLIB_PIN
}

// Epilogue of one wave: alpha * acc + beta * C, conversion, bounds-checked
// store, piece by piece (four consecutive elements of the contiguous C axis).
template <int TOUT, int TX, int TY, int MS = 16, int TILE0 = 0, typename Acc>
__device__ __forceinline__ void store_wave_tile(const KernelArgs &args, unsigned b, unsigned x_wave,
                                                unsigned y_wave, int lane, const Acc &acc_re,
                                                const Acc &acc_im) {
  // TX, TY count MFMA tiles; pieces per tile row: 1 (MS 16) or 4 (MS 32)
  constexpr int NPX = MS == 32 ? TX * 4 : TX;
  using Tout = typename OutType<TOUT>::type;
  const unsigned nx = args.nx, ny = args.ny;
  const bool have_alpha = args.have_alpha, have_beta = args.have_beta;
  const float ar = args.alpha_re, ai = args.alpha_im, br = args.beta_re, bi = args.beta_im;
  Tout *cbase = reinterpret_cast<Tout *>(args.c) + (size_t)b * 2 * nx * ny;
  const bool vec_ok = (nx % 4 == 0) && args.c_vector_ok;
#pragma unroll
  for (int j = 0; j < TY; ++j) {
#pragma unroll
    for (int i = 0; i < NPX; ++i) {
      const unsigned y = y_wave + piece_y<MS>(j, i, lane);
      const unsigned x = x_wave + piece_x<MS>(i, lane);
      if (y >= ny || x >= nx) continue;
      float re[4], im[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        re[e] = piece_elem<MS, TILE0>(acc_re, j, i, e);
        im[e] = piece_elem<MS, TILE0>(acc_im, j, i, e);
        if (have_alpha) {
          const float r0 = re[e];
          re[e] = alpha_times_re(ar, ai, r0, im[e]);
          im[e] = alpha_times_im(ar, ai, r0, im[e]);
        }
      }
      const bool full = vec_ok && (x + 4 <= nx);
      if (!args.c_interleaved) {
        Tout *pr = cbase + (size_t)y * nx + x;
        Tout *pi = pr + (size_t)nx * ny;
        if (have_beta) {
          // (whole pieces: C comes in with one wide load per plane)
          Tout cr4[4], ci4[4];
          if (full) {
            typedef Tout Piece __attribute__((ext_vector_type(4)));
            const Piece vr = *reinterpret_cast<const Piece *>(pr), vi = *reinterpret_cast<const Piece *>(pi);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              cr4[e] = vr[e];
              ci4[e] = vi[e];
            }
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (full || x + e < nx) {
              const float cr = full ? (float)cr4[e] : (float)pr[e];
              const float ci = full ? (float)ci4[e] : (float)pi[e];
              re[e] += br * cr - bi * ci;
              im[e] += bi * cr + br * ci;
            }
          }
        }
        if (full) {
          if constexpr (TOUT == kFloat32) {
            *reinterpret_cast<float4_t *>(pr) = float4_t{re[0], re[1], re[2], re[3]};
            *reinterpret_cast<float4_t *>(pi) = float4_t{im[0], im[1], im[2], im[3]};
          } else {
            Tout r4[4] = {(Tout)re[0], (Tout)re[1], (Tout)re[2], (Tout)re[3]};
            Tout i4[4] = {(Tout)im[0], (Tout)im[1], (Tout)im[2], (Tout)im[3]};
            *reinterpret_cast<ushort4_t *>(pr) = __builtin_bit_cast(ushort4_t, r4);
            *reinterpret_cast<ushort4_t *>(pi) = __builtin_bit_cast(ushort4_t, i4);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (x + e < nx) {
              pr[e] = (Tout)re[e];
              pi[e] = (Tout)im[e];
            }
          }
        }
      } else {
        Tout *p = cbase + ((size_t)y * nx + x) * 2;
        if (have_beta) {
          Tout c8[8];
          if (full) {
            typedef Tout Piece __attribute__((ext_vector_type(8)));
            const Piece v = *reinterpret_cast<const Piece *>(p);
#pragma unroll
            for (int e = 0; e < 8; ++e) c8[e] = v[e];
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (full || x + e < nx) {
              const float cr = full ? (float)c8[2 * e] : (float)p[2 * e];
              const float ci = full ? (float)c8[2 * e + 1] : (float)p[2 * e + 1];
              re[e] += br * cr - bi * ci;
              im[e] += bi * cr + br * ci;
            }
          }
        }
        if (full) {
          if constexpr (TOUT == kFloat32) {
            reinterpret_cast<float4_t *>(p)[0] = float4_t{re[0], im[0], re[1], im[1]};
            reinterpret_cast<float4_t *>(p)[1] = float4_t{re[2], im[2], re[3], im[3]};
          } else {
            Tout v8[8] = {(Tout)re[0], (Tout)im[0], (Tout)re[1], (Tout)im[1],
                          (Tout)re[2], (Tout)im[2], (Tout)re[3], (Tout)im[3]};
            *reinterpret_cast<int4_t *>(p) = __builtin_bit_cast(int4_t, v8);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (x + e < nx) {
              p[2 * e] = (Tout)re[e];
              p[2 * e + 1] = (Tout)im[e];
            }
          }
        }
      }
    }
  }
}

// Epilogue of the 1-bit GEMM on the MFMA path: the accumulators hold exact
// integers (sums of +-1 products); alpha and beta are truncated to integers and
// everything wraps modulo 2^32, as in the popcount kernel.
template <int TX, int TY, int MS, typename Acc>
__device__ __forceinline__ void store_wave_tile_int32(const KernelArgs &args, unsigned b,
                                                      unsigned x_wave, unsigned y_wave, int lane,
                                                      const Acc &acc_re, const Acc &acc_im) {
  constexpr int NPX = MS == 32 ? TX * 4 : TX;
  const unsigned nx = args.nx, ny = args.ny;
  const unsigned ar = (unsigned)(int)args.alpha_re, ai = (unsigned)(int)args.alpha_im;
  const unsigned br = (unsigned)(int)args.beta_re, bi = (unsigned)(int)args.beta_im;
  const bool have_beta = args.have_beta;
  unsigned *cbase = reinterpret_cast<unsigned *>(args.c) + (size_t)b * 2 * nx * ny;
  const bool vec_ok = (nx % 4 == 0) && args.c_vector_ok;
#pragma unroll
  for (int j = 0; j < TY; ++j) {
#pragma unroll
    for (int i = 0; i < NPX; ++i) {
      const unsigned y = y_wave + piece_y<MS>(j, i, lane);
      const unsigned x = x_wave + piece_x<MS>(i, lane);
      if (y >= ny || x >= nx) continue;
      unsigned re[4], im[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned sr = (unsigned)(int)piece_elem<MS>(acc_re, j, i, e);
        const unsigned si = (unsigned)(int)piece_elem<MS>(acc_im, j, i, e) - args.im_excess;
        re[e] = ar * sr - ai * si;
        im[e] = ai * sr + ar * si;
      }
      const bool full = vec_ok && (x + 4 <= nx);
      if (!args.c_interleaved) {
        unsigned *pr = cbase + (size_t)y * nx + x, *pi = pr + (size_t)nx * ny;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (have_beta && x + e < nx) {
            const unsigned cr = pr[e], ci = pi[e];
            re[e] += br * cr - bi * ci;
            im[e] += bi * cr + br * ci;
          }
        }
        if (full) {
          *reinterpret_cast<int4_t *>(pr) = int4_t{(int)re[0], (int)re[1], (int)re[2], (int)re[3]};
          *reinterpret_cast<int4_t *>(pi) = int4_t{(int)im[0], (int)im[1], (int)im[2], (int)im[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (x + e < nx) {
              pr[e] = re[e];
              pi[e] = im[e];
            }
          }
        }
      } else {
        unsigned *p = cbase + ((size_t)y * nx + x) * 2;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (have_beta && x + e < nx) {
            const unsigned cr = p[2 * e], ci = p[2 * e + 1];
            re[e] += br * cr - bi * ci;
            im[e] += bi * cr + br * ci;
          }
        }
        if (full) {
          reinterpret_cast<int4_t *>(p)[0] = int4_t{(int)re[0], (int)im[0], (int)re[1], (int)im[1]};
          reinterpret_cast<int4_t *>(p)[1] = int4_t{(int)re[2], (int)im[2], (int)re[3], (int)im[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (x + e < nx) {
              p[2 * e] = re[e];
              p[2 * e + 1] = im[e];
            }
          }
        }
      }
    }
  }
}

// Epilogue of the exchanged-roles layout (kAcc16T) for the common case (planar
// C, beta = 0, wave tile entirely inside C, vector-aligned rows): register e of
// the four tiles of a tile row are four consecutive x, so a lane writes 16 bytes
// (8 for fp16 / bf16 C) and a store instruction four whole 256-byte row segments,
// straight from the accumulators.
template <int TOUT, int TY>
__device__ __forceinline__ void store_wave_tile_rows(const KernelArgs &args, unsigned b,
                                                     unsigned x_wave, unsigned y_wave, int lane,
                                                     float4_t (&acc_re)[TY][4],
                                                     float4_t (&acc_im)[TY][4]) {
  using Tout = typename OutType<TOUT>::type;
  const unsigned nx = args.nx, ny = args.ny;
  const bool have_alpha = args.have_alpha;
  const float ar = args.alpha_re, ai = args.alpha_im;
  Tout *out = reinterpret_cast<Tout *>(args.c) + (size_t)b * 2 * nx * ny +
              (size_t)(y_wave + (lane >> 4) * 4) * nx + x_wave + (lane & 15) * 4;
#pragma unroll
  for (int plane = 0; plane < 2; ++plane) {
#pragma unroll
    for (int j = 0; j < TY; ++j) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float re = acc_re[j][i][e], im = acc_im[j][i][e];
          v[i] = plane == 0 ? (have_alpha ? alpha_times_re(ar, ai, re, im) : re)
                            : (have_alpha ? alpha_times_im(ar, ai, re, im) : im);
        }
        Tout *p = out + (size_t)plane * nx * ny + (size_t)(j * 16 + e) * nx;
        if constexpr (kAblateStores) {
          if (v[0] == 12345.678f) *p = (Tout)v[1];   // (timing-only build)
        } else if constexpr (TOUT == kFloat32) {
          *reinterpret_cast<float4_t *>(p) = float4_t{v[0], v[1], v[2], v[3]};
        } else {
          Tout t[4] = {(Tout)v[0], (Tout)v[1], (Tout)v[2], (Tout)v[3]};
          *reinterpret_cast<ushort4_t *>(p) = __builtin_bit_cast(ushort4_t, t);
        }
      }
    }
  }
}

// Epilogue through LDS for the common case (planar fp32 C, beta = 0, wave tile
// entirely inside C, 64 columns wide): the accumulators of 16 rows are written
// to a wave-private LDS patch and read back row-wise, so that every store
// instruction writes four contiguous 256-byte row segments instead of sixteen
// 64-byte ones. `patch` is 16 rows of 272 bytes (the 16-byte pad keeps both
// the column-wise writes and the row-wise reads free of bank conflicts).
constexpr int kStagePatchBytes = 16 * 272;

template <int TX, int TY>
__device__ __forceinline__ void store_wave_tile_staged(const KernelArgs &args, unsigned b,
                                                       unsigned x_wave, unsigned y_wave, int lane,
                                                       char *patch, float4_t (&acc_re)[TY][TX],
                                                       float4_t (&acc_im)[TY][TX]) {
  static_assert(TX == 4, "patch rows hold 64 columns");
  const unsigned nx = args.nx, ny = args.ny;
  const bool have_alpha = args.have_alpha;
  const float ar = args.alpha_re, ai = args.alpha_im;
  float *cbase = reinterpret_cast<float *>(args.c) + (size_t)b * 2 * nx * ny;
  char *wr = patch + (lane & 15) * 272 + (lane >> 4) * 16;   // [y = lane%16][x = (lane/16)*4 ..]
  const char *rd = patch + (lane >> 4) * 272 + (lane & 15) * 16;  // [row lane/16][x = (lane%16)*4 ..]
  float *out = cbase + (size_t)(y_wave + (lane >> 4)) * nx + x_wave + (lane & 15) * 4;
#pragma unroll
  for (int plane = 0; plane < 2; ++plane) {
#pragma unroll
    for (int j = 0; j < TY; ++j) {
#pragma unroll
      for (int i = 0; i < TX; ++i) {
        float4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float re = acc_re[j][i][e], im = acc_im[j][i][e];
          v[e] = plane == 0 ? (have_alpha ? alpha_times_re(ar, ai, re, im) : re)
                            : (have_alpha ? alpha_times_im(ar, ai, re, im) : im);
        }
        *reinterpret_cast<float4_t *>(wr + i * 64) = v;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float4_t v = *reinterpret_cast<const float4_t *>(rd + r * 4 * 272);
        *reinterpret_cast<float4_t *>(out + (size_t)plane * nx * ny + (size_t)(j * 16 + r * 4) * nx) = v;
      }
    }
  }
}

// The same for planar fp16 / bf16 C: a tile row of 16 x 64 values is 16 rows of
// 128 bytes (stride 144 in the patch: conflict-free 8-byte writes down a column,
// 16-byte aligned reads along a row); every store instruction writes eight whole
// 128-byte row segments instead of sixteen 32-byte pieces.
template <int TOUT, int TX, int TY>
__device__ __forceinline__ void store_wave_tile_staged_narrow(const KernelArgs &args, unsigned b,
                                                              unsigned x_wave, unsigned y_wave,
                                                              int lane, char *patch,
                                                              float4_t (&acc_re)[TY][TX],
                                                              float4_t (&acc_im)[TY][TX]) {
  static_assert(TX == 4, "patch rows hold 64 columns");
  using Tout = typename OutType<TOUT>::type;
  const unsigned nx = args.nx, ny = args.ny;
  const bool have_alpha = args.have_alpha;
  const float ar = args.alpha_re, ai = args.alpha_im;
  Tout *cbase = reinterpret_cast<Tout *>(args.c) + (size_t)b * 2 * nx * ny;
  char *wr = patch + (lane & 15) * 144 + (lane >> 4) * 8;        // [y = lane%16][x = (lane/16)*4 ..]
  const char *rd = patch + (lane >> 3) * 144 + (lane & 7) * 16;  // [row lane/8][x = (lane%8)*8 ..]
  Tout *out = cbase + (size_t)(y_wave + (lane >> 3)) * nx + x_wave + (lane & 7) * 8;
#pragma unroll
  for (int plane = 0; plane < 2; ++plane) {
#pragma unroll
    for (int j = 0; j < TY; ++j) {
#pragma unroll
      for (int i = 0; i < TX; ++i) {
        Tout v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float re = acc_re[j][i][e], im = acc_im[j][i][e];
          v[e] = (Tout)(plane == 0 ? (have_alpha ? alpha_times_re(ar, ai, re, im) : re)
                                   : (have_alpha ? alpha_times_im(ar, ai, re, im) : im));
        }
        *reinterpret_cast<ushort4_t *>(wr + i * 32) = __builtin_bit_cast(ushort4_t, v);
      }
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int4_t v = *reinterpret_cast<const int4_t *>(rd + r * 8 * 144);
        *reinterpret_cast<int4_t *>(out + (size_t)plane * nx * ny + (size_t)(j * 16 + r * 8) * nx) = v;
      }
    }
  }
}

// The same for interleaved fp32 C: 16 rows of 32 (re, im) pairs at a time (half
// the width of the wave tile, again 256 bytes per row) go through the patch.
template <int TX, int TY>
__device__ __forceinline__ void store_wave_tile_staged_il(const KernelArgs &args, unsigned b,
                                                          unsigned x_wave, unsigned y_wave, int lane,
                                                          char *patch, float4_t (&acc_re)[TY][TX],
                                                          float4_t (&acc_im)[TY][TX]) {
  static_assert(TX == 4, "two halves of 32 columns");
  const unsigned nx = args.nx, ny = args.ny;
  const bool have_alpha = args.have_alpha;
  const float ar = args.alpha_re, ai = args.alpha_im;
  float *cbase = reinterpret_cast<float *>(args.c) + (size_t)b * 2 * nx * ny;
  char *wr = patch + (lane & 15) * 272 + (lane >> 4) * 32;   // [y = lane%16][pair (lane/16)*4 ..]
  const char *rd = patch + (lane >> 4) * 272 + (lane & 15) * 16;  // [row lane/16][pairs 2 (lane%16) ..]
  float *out = cbase + ((size_t)(y_wave + (lane >> 4)) * nx + x_wave) * 2 + (lane & 15) * 4;
#pragma unroll
  for (int j = 0; j < TY; ++j) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 2 * h; i < 2 * h + 2; ++i) {
        float re[4], im[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float r0 = acc_re[j][i][e], i0 = acc_im[j][i][e];
          re[e] = have_alpha ? alpha_times_re(ar, ai, r0, i0) : r0;
          im[e] = have_alpha ? alpha_times_im(ar, ai, r0, i0) : i0;
        }
        char *w = wr + (i - 2 * h) * 128;
        *reinterpret_cast<float4_t *>(w) = float4_t{re[0], im[0], re[1], im[1]};
        *reinterpret_cast<float4_t *>(w + 16) = float4_t{re[2], im[2], re[3], im[3]};
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float4_t v = *reinterpret_cast<const float4_t *>(rd + r * 4 * 272);
        *reinterpret_cast<float4_t *>(out + ((size_t)(j * 16 + r * 4) * nx + h * 32) * 2) = v;
      }
    }
  }
}

// The same for the 32-row MFMA layout: one 32 x 32 tile at a time goes through
// a patch of 32 rows of 144 bytes (128 + 16 of padding), and every store
// instruction writes eight whole 128-byte row segments.
constexpr int kStagePatch32Bytes = 32 * 144;

template <int TX, int TY, bool INT = false>
__device__ __forceinline__ void store_wave_tile_staged32(const KernelArgs &args, unsigned b,
                                                         unsigned x_wave, unsigned y_wave, int lane,
                                                         char *patch, float16_t_ (&acc_re)[TY][TX],
                                                         float16_t_ (&acc_im)[TY][TX]) {
  const unsigned nx = args.nx, ny = args.ny;
  const bool have_alpha = args.have_alpha;
  const float ar = args.alpha_re, ai = args.alpha_im;
  float *cbase = reinterpret_cast<float *>(args.c) + (size_t)b * 2 * nx * ny;
  char *wr = patch + (lane & 31) * 144 + (lane >> 5) * 16;        // [y = lane%32][x = 8k + 4 (lane/32) ..]
  const char *rd = patch + (lane >> 3) * 144 + (lane & 7) * 16;   // [row lane/8 (+8q)][x = 4 (lane%8) ..]
  float *out = cbase + (size_t)(y_wave + (lane >> 3)) * nx + x_wave + (lane & 7) * 4;
#pragma unroll
  for (int plane = 0; plane < 2; ++plane) {
#pragma unroll
    for (int j = 0; j < TY; ++j) {
#pragma unroll
      for (int i = 0; i < TX; ++i) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float4_t v;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float re = acc_re[j][i][4 * k + e], im = acc_im[j][i][4 * k + e];
            if constexpr (INT) {
              // exact integers; alpha truncated, arithmetic modulo 2^32
              const unsigned sr = (unsigned)(int)re, si = (unsigned)(int)im - args.im_excess;
              const unsigned iar = (unsigned)(int)ar, iai = (unsigned)(int)ai;
              const unsigned o = plane == 0 ? iar * sr - iai * si : iai * sr + iar * si;
              v[e] = __builtin_bit_cast(float, o);
            } else {
              v[e] = plane == 0 ? (have_alpha ? alpha_times_re(ar, ai, re, im) : re)
                                : (have_alpha ? alpha_times_im(ar, ai, re, im) : im);
            }
          }
          *reinterpret_cast<float4_t *>(wr + k * 32) = v;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4_t v = *reinterpret_cast<const float4_t *>(rd + q * 8 * 144);
          *reinterpret_cast<float4_t *>(out + (size_t)plane * nx * ny +
                                        (size_t)(j * 32 + q * 8) * nx + i * 32) = v;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Register-staged kernel: global -> registers -> LDS, two LDS stages. Used for
// planar (basic) input whose rows are not whole aligned 16-byte chunks: its
// element-wise loads do the bounds checks and the zero fill.
// ---------------------------------------------------------------------------
template <int DT, int TOUT, int BX, int BY, int WX, int WY, int KT, int LOADER, int WAVES_PER_EU>
__global__ __launch_bounds__(64 * (BX / WX) * (BY / WY), WAVES_PER_EU) void complex_gemm_mfma(
    const KernelArgs args) {
  constexpr int NWX = BX / WX, NWY = BY / WY;
  constexpr int NTHREADS = 64 * NWX * NWY;
  constexpr int TX = WX / 16, TY = WY / 16;
  constexpr int KPM = DtypeTraits<DT>::kTilesPerMfma;
  constexpr int EB = DtypeTraits<DT>::kElemBytes;
  static_assert(KT % KPM == 0, "stage must hold whole MFMAs");
  constexpr int X_KTILE_BYTES = 2 * BX * kTileRowBytes;
  constexpr int Y_KTILE_BYTES = 2 * BY * kTileRowBytes;
  constexpr int KTILE_BYTES = X_KTILE_BYTES + Y_KTILE_BYTES;
  constexpr int STAGE_BYTES = KT * KTILE_BYTES;
  constexpr int X_CHUNKS = KT * 2 * BX * 4;
  constexpr int Y_CHUNKS = KT * 2 * BY * 4;
  static_assert(X_CHUNKS % NTHREADS == 0 && Y_CHUNKS % NTHREADS == 0, "chunks per thread");
  constexpr int CX = X_CHUNKS / NTHREADS, CY = Y_CHUNKS / NTHREADS;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wx = wave % NWX, wy = wave / NWX;

  const TileCoord tc = tile_coord(args, blockIdx.x);
  const unsigned b = tc.b, block_x = tc.block_x, block_y = tc.block_y;

  OperandView xv{args.x + (size_t)b * args.x_batch_bytes, args.nx, args.x_tiles, block_x * BX};
  OperandView yv{args.y + (size_t)b * args.y_batch_bytes, args.ny, args.y_tiles, block_y * BY};
  const unsigned k_tiles = args.k_tiles;
  const unsigned k_bytes = args.k_bytes;

  int4_t xs[CX], ys[CY];
  auto fetch = [&](unsigned kt0) {
#pragma unroll
    for (int i = 0; i < CX; ++i) {
      const int gidx = tid + i * NTHREADS;
      const int kk = gidx / (2 * BX * 4), rem = gidx % (2 * BX * 4);
      xs[i] = load_chunk<EB, LOADER>(xv, kt0 + kk, k_tiles, k_bytes, rem / (BX * 4),
                                     (rem / 4) % BX, rem % 4);
    }
#pragma unroll
    for (int i = 0; i < CY; ++i) {
      const int gidx = tid + i * NTHREADS;
      const int kk = gidx / (2 * BY * 4), rem = gidx % (2 * BY * 4);
      ys[i] = load_chunk<EB, LOADER>(yv, kt0 + kk, k_tiles, k_bytes, rem / (BY * 4),
                                     (rem / 4) % BY, rem % 4);
    }
  };
  auto stash = [&](int stage) {
    char *s = lds + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < CX; ++i) {
      const int gidx = tid + i * NTHREADS;
      const int kk = gidx / (2 * BX * 4), rem = gidx % (2 * BX * 4);
      const int plane = rem / (BX * 4), row = (rem / 4) % BX, c = rem % 4;
      *reinterpret_cast<int4_t *>(s + kk * KTILE_BYTES + plane * BX * kTileRowBytes +
                                  swizzled_row_offset(row, c)) = xs[i];
    }
#pragma unroll
    for (int i = 0; i < CY; ++i) {
      const int gidx = tid + i * NTHREADS;
      const int kk = gidx / (2 * BY * 4), rem = gidx % (2 * BY * 4);
      const int plane = rem / (BY * 4), row = (rem / 4) % BY, c = rem % 4;
      *reinterpret_cast<int4_t *>(s + kk * KTILE_BYTES + X_KTILE_BYTES +
                                  plane * BY * kTileRowBytes + swizzled_row_offset(row, c)) =
          ys[i];
    }
  };

  float4_t acc_re[TY][TX], acc_im[TY][TX];
#pragma unroll
  for (int j = 0; j < TY; ++j) {
#pragma unroll
    for (int i = 0; i < TX; ++i) {
      acc_re[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};
      acc_im[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
  }

  const int lane_off = swizzled_row_offset(lane & 15, lane >> 4);
  const int x_frag_off = (wx * WX) * kTileRowBytes + lane_off;
  const int y_frag_off = X_KTILE_BYTES + (wy * WY) * kTileRowBytes + lane_off;

  auto compute = [&](int stage) {
    const char *s = lds + stage * STAGE_BYTES;
#pragma unroll
    for (int kk = 0; kk < KT; kk += KPM) {
      const char *slot[KPM];
#pragma unroll
      for (int u = 0; u < KPM; ++u) slot[u] = s + (kk + u) * KTILE_BYTES;
      mma_step<DT, BX, BY, TX, TY>(slot, x_frag_off, y_frag_off, acc_re, acc_im, [] {});
    }
  };

  const unsigned stages = (k_tiles + KT - 1) / KT;
  fetch(0);
  stash(0);
  if (stages > 1) fetch(KT);
  __syncthreads();
  for (unsigned s = 0; s < stages; ++s) {
    const int cur = s & 1;
    if (s + 1 < stages) stash(cur ^ 1);
    if (s + 2 < stages) fetch((s + 2) * KT);
    compute(cur);
    __syncthreads();
  }

  store_wave_tile<TOUT, TX, TY>(args, b, block_x * BX + wx * WX, block_y * BY + wy * WY, lane,
                                acc_re, acc_im);
}

// ---------------------------------------------------------------------------
// Direct-to-LDS kernel for the tiled (opt) layout, and for planar input with
// 16-byte aligned rows (where each lane brings its own address instead of an
// offset into a contiguous tile). Operand tiles of the tiled layout are
// contiguous 16 KiB blocks; the copy into LDS needs no registers: every wave issues
// global_load_lds_dwordx4, each of which moves 16 rows x 64 bytes (1 KiB)
// straight into LDS. The hardware writes lane L's 16 bytes at LDS offset
// base + 16 L; the XOR swizzle of the LDS layout is obtained by letting lane L
// fetch the chunk that belongs there (a permutation inside each 64-byte row,
// so the global access stays fully coalesced).
//
// LDS is a ring of SLOTS K tiles (X and Y may have rings of different depth).
// Iteration i waits for its own tile with s_waitcnt vmcnt(n) - n being the
// loads issued for later iterations - then passes one barrier, issues the loads
// SLOTS - 1 iterations ahead into the slot that the previous iteration just
// released (after its first group of MFMAs), and does the math.
//
// Blocks are persistent: each walks a sequence of C tiles, and the copy simply
// runs on into the next C tile, so its first K tiles are in flight while the
// current tile's results are stored, and those stores drain under the next
// tile's math. Loads past the end of K (rows whose last K tile is partial) or
// past the last C tile are pointed at a zero tile, which keeps the number of
// outstanding loads the same in every iteration.
// ---------------------------------------------------------------------------
__device__ __attribute__((aligned(256))) char g_zero_tile[kTileBytes];

template <int N> __device__ __forceinline__ void wait_vmcnt_then_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  if constexpr (kAblateBarrier) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
  }
}

// Both copy helpers write m0 (the LDS base of the copy) and say so in their
// clobber lists, so that the compiler never assumes a value it put there
// survives them; clang warns about any mention of m0 there, which is the point.
// The compiler does not look into an asm statement for the wait states its
// instructions need after what it placed in front of it: the scalar base of the
// first helper may have come out of a vector register right before (a spilled
// scalar register read back with v_readlane), and a vector memory instruction
// may read such a register five wait states later at the earliest. The helper
// therefore hands the base on through a scalar move: the scalar ALU may read the
// register at once, and what it writes the memory instruction may read at once.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load_1k_to_lds(const char *base, unsigned lane_offset,
                                               unsigned lds_address) {
  if constexpr (kAblateCopies) return;
  unsigned long long base_here;
  asm volatile(
      "s_mov_b64 %0, %3\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %2, %0"
      : "=&s"(base_here)
      : "s"(lds_address), "v"(lane_offset), "s"(base)
      : "memory", "m0");
}

// Same, with a full address per lane (planar layout: the 16 rows of a row block
// are not contiguous in memory).
__device__ __forceinline__ void load_1k_to_lds_by_lane(const char *lane_address,
                                                       unsigned lds_address) {
  if constexpr (kAblateCopies) return;
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off"
      :
      : "s"(lds_address), "v"(lane_address)
      : "memory", "m0");
}
#pragma clang diagnostic pop

#include "gemm_mfma_wide.h"

template <int DT, int TOUT, int BX, int BY, int WX, int WY, int SLOTS, int WAVES_PER_EU, int LOADER,
          int MS, bool XT, int XSLOTS>
__global__ __launch_bounds__(64 * (BX / WX) * (BY / WY), WAVES_PER_EU) void complex_gemm_mfma_dtl(
    const KernelArgs args) {
  constexpr int NWX = BX / WX, NWY = BY / WY, NW = NWX * NWY;
  constexpr int TX = WX / MS, TY = WY / MS;          // MFMA tiles of a wave
  static_assert(MS == 32 || DtypeTraits<DT>::kTilesPerMfma == 1,
                "one K tile per iteration: fp8 input runs on the 32-row MFMA here");
  constexpr int KPM = 1;
  static_assert(MS == 16 || LOADER != kLoadInterleavedVec || DtypeTraits<DT>::kElemBytes == 1,
                "interleaved operands on the 32-row MFMAs: 8-bit input only");
  // interleaved operands: one plane of (re, im) rows
  // (their slots hold 128 bytes of every row, fetched as whole cache lines)
  constexpr bool IL = (LOADER == kLoadInterleavedVec);
  constexpr int PLANES = IL ? 1 : 2;
  constexpr int RB = IL ? 128 : kTileRowBytes;      // bytes of a row in one slot
  constexpr int RPB = 1024 / RB;                    // rows moved by one 1 KiB copy instruction
  constexpr int CPR = RB / 16;                      // 16-byte chunks per row
  constexpr int X_BYTES = PLANES * BX * RB, Y_BYTES = PLANES * BY * RB;
  constexpr int SLOT_BYTES = X_BYTES + Y_BYTES;
  // 1 KiB row blocks (16 rows x 64 bytes or 8 x 128) of the X and the Y part of a K tile
  constexpr int X_ROW_BLOCKS = X_BYTES / 1024, Y_ROW_BLOCKS = Y_BYTES / 1024;
  static_assert(X_ROW_BLOCKS % NW == 0 && Y_ROW_BLOCKS % NW == 0,
                "row blocks must divide evenly over the waves");
  constexpr int XL = X_ROW_BLOCKS / NW, YL = Y_ROW_BLOCKS / NW;   // loads per wave per K tile
  constexpr int LPW = XL + YL;
  // XT: the X fragments feed the "B" side of the 16-row MFMA and tile i of a wave
  // holds the columns x = 4 (lane % 16) + i of its 64, so that a lane ends up with
  // 16 consecutive bytes of four C rows per register index and the C stores need no
  // regrouping through LDS. For that, the rows of every 16-row block of X sit in
  // LDS in the order [4 a + (i ^ a)] <- row 4 a + i, with their 16-byte chunks XORed
  // with 3 (block & 1): fragment reads of rows 4 r + i are then free of bank
  // conflicts (measured), and a copy instruction still moves the contiguous 1 KiB.
  static_assert(!XT || (MS == 16 && TX == 4 && TY == 4 && !IL && WX == 64 && NW % 2 == 0 &&
                        (BX / 16) % 2 == 0),
                "exchanged roles: 16-row MFMA, 4 x 4 tiles per wave");
  // The ring. SLOTS K tiles of Y and XSLOTS >= SLOTS K tiles of X: X tiles are
  // requested XLEAD iterations before their use, Y tiles YLEAD iterations. With
  // equal counts a slot is [X | Y] as one piece of LDS; with more X slots the
  // two rings lie one after the other (X is then the operand to make the narrower
  // one: more of its K tiles fit, and a longer wait for memory is covered).
  static_assert(SLOTS >= 2 && XSLOTS >= SLOTS, "ring must hold at least two iterations");
  constexpr bool SPLIT = XSLOTS != SLOTS;
  constexpr int XLEAD = XSLOTS - 1, YLEAD = SLOTS - 1;
  // The counter of outstanding copies retires in order. In every iteration a wave
  // requests its Y blocks first and then its X blocks; the K tile of iteration k is
  // complete when nothing older than the last request for it is outstanding, which
  // leaves the requests of the YLEAD - 1 iterations since, and the X blocks that
  // followed Y(k) in its own iteration when X runs further ahead.
  constexpr int kOutstandingOk = (XLEAD > YLEAD ? XL : 0) + (YLEAD - 1) * LPW;
  static_assert(kOutstandingOk < 64, "vmcnt range");
  auto x_slot_off = [](unsigned s) { return SPLIT ? s * X_BYTES : s * SLOT_BYTES; };
  auto y_slot_off = [](unsigned s) {
    return SPLIT ? XSLOTS * X_BYTES + s * Y_BYTES : s * SLOT_BYTES + X_BYTES;
  };

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wx = wave % NWX, wy = wave / NWX;
  // slots along K (the host counts 64-byte pieces of a row)
  const unsigned k_tiles = IL ? (args.k_tiles + 1) / 2 : args.k_tiles;
  const unsigned total = args.blocks_x * args.blocks_y * args.batch;
  // bytes of one operand row in memory (planar: one plane's row)
  const unsigned row_bytes = IL ? 2 * args.k_bytes : args.k_bytes;
  // ... and the distance between rows (larger when the launch covers a piece of K)
  const unsigned row_stride = IL ? 2 * args.row_stride_bytes : args.row_stride_bytes;

  // ---- this wave's share of the copy: XL + YL row blocks of every K tile --
  // Row block q of an operand's part of a K tile: re plane, im plane, 16 rows
  // each. What depends on the lane (its row and swizzled chunk inside the row
  // block) is the same for every C tile; the wave-uniform tile pointers are set
  // per C tile.
  const unsigned lane_off = (lane >> 2) * kTileRowBytes +
                            (((lane & 3) ^ (MS == 32 ? (lane >> 4) & 3 : (lane >> 3) & 3)) * 16);
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char *)lds;
  const int r = lane / CPR;                                   // row inside the row block
  // chunk that belongs at lane*16: the XOR pattern that makes the fragment
  // reads of the MFMA shape in use free of bank conflicts (measured)
  // (interleaved rows on the 32-row MFMAs: XOR with (row >> 1) & 7, which also
  // depends on the parity of the 8-row row block, see c_of below)
  const int c = (lane % CPR) ^ (IL ? r & 7 : MS == 32 ? (r >> 2) & 3 : (r >> 1) & 3);
  auto c_of = [&](int rb) {   // chunk this lane fetches for row block rb of an operand
    return (IL && MS == 32) ? ((lane % CPR) ^ (((rb & 1) << 2) | ((r >> 1) & 3))) : c;
  };
  // (XT) row and chunk this lane fetches of an X row block (a wave's X row blocks
  // all have the parity of the wave number)
  const int xt_row = 4 * (lane >> 4) + (((lane >> 2) & 3) ^ (lane >> 4));
  const int xt_chunk = (lane & 3) ^ (3 * (wave & 1));
  const unsigned lane_off_x = XT ? xt_row * kTileRowBytes + xt_chunk * 16 : lane_off;

  // One operand's side of the copy: where its next K tile comes from. The copy
  // walks the same sequence of C tiles as the math, X ahead of Y when its ring
  // is deeper; past the last C tile it re-reads the last one (never used).
  struct Stream {
    unsigned tile, kt;          // C tile and K tile of the request issued last
  };
  Stream xs{blockIdx.x, 0}, ys{blockIdx.x, 0};
  unsigned x_tile_off[XL], y_tile_off[YL];   // wave-uniform: the row block inside its operand tile
  unsigned x_lds[XL], y_lds[YL];             // wave-uniform: LDS byte address inside slot 0 of the ring
  const char *x_src[XL], *y_src[YL];         // wave-uniform: K tile 0 of the operand tile (tiled layout)
  const char *x_lane_src[XL], *y_lane_src[YL];   // planar layouts: this lane's chunk of K tile 0
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int q = i * NW + wave, plane = q / (BX / RPB), rb = q % (BX / RPB);
    x_tile_off[i] = plane * kTilePlaneBytes + ((rb * RPB) % kTileRows) * kTileRowBytes;
    x_lds[i] = lds_base + x_slot_off(0) + q * 1024;
  }
#pragma unroll
  for (int i = 0; i < YL; ++i) {
    const int q = i * NW + wave, plane = q / (BY / RPB), rb = q % (BY / RPB);
    y_tile_off[i] = plane * kTilePlaneBytes + ((rb * RPB) % kTileRows) * kTileRowBytes;
    y_lds[i] = lds_base + y_slot_off(0) + q * 1024;
  }
  // Points one side of the copy at the operand tile of C tile vt.
  auto point_x = [&](unsigned vt) {
    if (vt >= total) return;
    const TileCoord tc = tile_coord(args, vt);
    const char *op = args.x + (size_t)tc.b * args.x_batch_bytes;
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const int q = i * NW + wave, plane = q / (BX / RPB), rb = q % (BX / RPB);
      const unsigned row0 = tc.block_x * BX + rb * RPB;
      if constexpr (LOADER == kLoadTiled) {
        unsigned tile = row0 / kTileRows;
        tile = tile < args.x_tiles ? tile : args.x_tiles - 1;   // rows past the end: never stored
        x_src[i] = op + (size_t)tile * args.k_tile_stride * kTileBytes;
      } else {
        unsigned row = row0 + (XT ? xt_row : r);
        row = row < args.nx ? row : args.nx - 1;   // likewise
        x_lane_src[i] = op + ((size_t)plane * args.nx + row) * row_stride +
                        (XT ? xt_chunk : c_of(rb)) * 16;
      }
    }
  };
  auto point_y = [&](unsigned vt) {
    if (vt >= total) return;
    const TileCoord tc = tile_coord(args, vt);
    const char *op = args.y + (size_t)tc.b * args.y_batch_bytes;
#pragma unroll
    for (int i = 0; i < YL; ++i) {
      const int q = i * NW + wave, plane = q / (BY / RPB), rb = q % (BY / RPB);
      const unsigned row0 = tc.block_y * BY + rb * RPB;
      if constexpr (LOADER == kLoadTiled) {
        unsigned tile = row0 / kTileRows;
        tile = tile < args.y_tiles ? tile : args.y_tiles - 1;
        y_src[i] = op + (size_t)tile * args.k_tile_stride * kTileBytes;
      } else {
        unsigned row = row0 + r;
        row = row < args.ny ? row : args.ny - 1;
        y_lane_src[i] = op + ((size_t)plane * args.ny + row) * row_stride + c_of(rb) * 16;
      }
    }
  };
  // issue_*: straight-line code (it is placed between MFMAs, and a branch there
  // would let the compiler sink those MFMAs below it); advance_*: the
  // bookkeeping, with the branches of the tile change.
  auto issue_x = [&](unsigned slot) {
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const unsigned dst = x_lds[i] + (x_slot_off(slot) - x_slot_off(0));
      if constexpr (LOADER == kLoadTiled) {
        load_1k_to_lds(x_src[i] + (size_t)xs.kt * kTileBytes + x_tile_off[i], lane_off_x, dst);
      } else {
        // rows are whole 16-byte chunks: a chunk is either inside K or reads zeros
        const int q = i * NW + wave, rb = q % (BX / RPB);
        const int chunk = XT ? xt_chunk : c_of(rb);
        const bool inside = (xs.kt * RB + chunk * 16 + 16 <= row_bytes);
        load_1k_to_lds_by_lane(inside ? x_lane_src[i] + (size_t)xs.kt * RB : g_zero_tile + lane * 16,
                               dst);
      }
    }
  };
  auto issue_y = [&](unsigned slot) {
#pragma unroll
    for (int i = 0; i < YL; ++i) {
      const unsigned dst = y_lds[i] + (y_slot_off(slot) - y_slot_off(0));
      if constexpr (LOADER == kLoadTiled) {
        load_1k_to_lds(y_src[i] + (size_t)ys.kt * kTileBytes + y_tile_off[i], lane_off, dst);
      } else {
        const int q = i * NW + wave, rb = q % (BY / RPB);
        const bool inside = (ys.kt * RB + c_of(rb) * 16 + 16 <= row_bytes);
        load_1k_to_lds_by_lane(inside ? y_lane_src[i] + (size_t)ys.kt * RB : g_zero_tile + lane * 16,
                               dst);
      }
    }
  };
  auto advance_x = [&] {
    if (++xs.kt == k_tiles) {
      xs.kt = 0;
      xs.tile += gridDim.x;
      point_x(xs.tile);
    }
  };
  auto advance_y = [&] {
    if (++ys.kt == k_tiles) {
      ys.kt = 0;
      ys.tile += gridDim.x;
      point_y(ys.tile);
    }
  };

  const int frag_lane_off = swizzled_row_offset(lane & 15, lane >> 4);
  const int x_frag_off = (wx * WX) * kTileRowBytes + frag_lane_off;
  const int y_frag_off = X_BYTES + (wy * WY) * kTileRowBytes + frag_lane_off;
  int xo[4];   // X fragment of tile i (16-row MFMA)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r16 = lane & 15, g = lane >> 4;
    xo[i] = XT ? (wx * WX + 4 * r16 + (i ^ (r16 & 3))) * kTileRowBytes +
                     ((g ^ (3 * ((r16 >> 2) & 1))) * 16)
               : x_frag_off + i * 16 * kTileRowBytes;
  }
  // 32-row MFMA: row lane % 32, chunks lane / 32 and lane / 32 + 2 (any split
  // of K over the lanes is fine as long as X and Y use the same one)
  const int row32 = lane & 31, sw32 = (row32 >> 2) & 3;
  const int frag32_off[2] = {row32 * kTileRowBytes + (((lane >> 5) ^ sw32) * 16),
                             row32 * kTileRowBytes + ((((lane >> 5) | 2) ^ sw32) * 16)};
  const int x32_off[2] = {(wx * WX) * kTileRowBytes + frag32_off[0],
                          (wx * WX) * kTileRowBytes + frag32_off[1]};
  const int y32_off[2] = {X_BYTES + (wy * WY) * kTileRowBytes + frag32_off[0],
                          X_BYTES + (wy * WY) * kTileRowBytes + frag32_off[1]};
  // interleaved rows of 128 bytes: row lane % 16, chunks lane / 16 and lane / 16 + 4
  const int il_row = lane & 15;
  const int il_off[2] = {il_row * 128 + (((lane >> 4) ^ (il_row & 7)) * 16),
                         il_row * 128 + ((((lane >> 4) | 4) ^ (il_row & 7)) * 16)};
  const int xil_off[2] = {(wx * WX) * 128 + il_off[0], (wx * WX) * 128 + il_off[1]};
  const int yil_off[2] = {X_BYTES + (wy * WY) * 128 + il_off[0],
                          X_BYTES + (wy * WY) * 128 + il_off[1]};
  // interleaved rows on the 32-row MFMAs: row lane % 32, half h of the 128 bytes, chunks
  // 4 h + 2 (lane / 32) and the next one
  int xil32_off[2][2], yil32_off[2][2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int row = lane & 31, chunk = 4 * h + 2 * (lane >> 5) + u;
      const int off = row * 128 + ((chunk ^ ((row >> 1) & 7)) * 16);
      xil32_off[h][u] = (wx * WX) * 128 + off;
      yil32_off[h][u] = X_BYTES + (wy * WY) * 128 + off;
    }
  }
  // wide stores through LDS: no beta term, vector-aligned rows (interleaved C
  // only with the 16-row layout)
  const bool staged_ok = (MS == 16 || !args.c_interleaved) && !args.have_beta &&
                         args.c_vector_ok && (args.nx % 4 == 0);

  // ---- pipeline ----------------------------------------------------------
  point_x(xs.tile);
  point_y(ys.tile);
  // The bookkeeping of the copy (advance_*, which branches) is done at the top of
  // an iteration for the copies issued inside it, so that nothing but
  // straight-line code follows the barrier. Before the first iteration: the
  // requests that iterations -XLEAD .. -1 would have made, in their order.
#pragma unroll
  for (int t = -XLEAD; t < 0; ++t) {
    if (t + YLEAD >= 0) {
      if (t + YLEAD > 0) advance_y();
      issue_y(t + YLEAD);
    }
    if (t + XLEAD > 0) advance_x();
    issue_x(t + XLEAD);
  }
  unsigned x_slot = 0, y_slot = 0;         // slots of the current iteration
  // (hand-ordered 16-row step) the lane's fragment addresses in the current slots
  unsigned xa[4], ya = lds_base + y_slot_off(0) + (y_frag_off - X_BYTES);
#pragma unroll
  for (int i = 0; i < 4; ++i) xa[i] = lds_base + x_slot_off(0) + xo[i];
  const unsigned iters = k_tiles;
  for (unsigned vt = blockIdx.x; vt < total; vt += gridDim.x) {
    typename AccType<MS>::type acc_re[TY][TX], acc_im[TY][TX];
    // (the hand-ordered step of the 16-row MFMAs starts its first iteration from zero itself)
    constexpr bool kStepClears = !IL && DT != kInt1 && MS == 16 && TX == 4 && TY == 4;
    static_assert(!SPLIT || kStepClears, "separate X and Y rings: hand-ordered 16-row step only");
    if constexpr (!kStepClears) {
#pragma unroll
      for (int j = 0; j < TY; ++j) {
#pragma unroll
        for (int i = 0; i < TX; ++i) {
          acc_re[j][i] = 0.f;
          acc_im[j][i] = 0.f;
        }
      }
    }
    for (unsigned it = 0; it < iters; ++it) {
      advance_y();
      advance_x();
      // After the first C tile, the K tiles of the first YLEAD iterations were
      // already waited for before the previous epilogue (see below), so these
      // iterations only need the barrier; waiting on the counter here would
      // wait for the previous tile's C stores, which are younger than them.
      if (vt != blockIdx.x && it < (unsigned)YLEAD) {
        asm volatile("s_barrier" ::: "memory");
      } else {
        wait_vmcnt_then_barrier<kOutstandingOk>();
      }
      // The slots of the previous iteration are free now: refill them with the
      // K tiles that are XLEAD / YLEAD iterations ahead (of this C tile or the
      // next). The copy instructions go out after the first group of MFMAs: right
      // after the barrier every wave of the block would otherwise be busy with
      // their address arithmetic and the matrix cores would have nothing to do.
      auto refill_slots = [&] {
        unsigned x_refill = x_slot + XLEAD, y_refill = y_slot + YLEAD;
        x_refill = x_refill >= XSLOTS ? x_refill - XSLOTS : x_refill;
        y_refill = y_refill >= SLOTS ? y_refill - SLOTS : y_refill;
        issue_y(y_refill);
        issue_x(x_refill);
      };
      const unsigned x_next = x_slot + 1 == XSLOTS ? 0 : x_slot + 1;
      const unsigned y_next = y_slot + 1 == SLOTS ? 0 : y_slot + 1;
      if constexpr (kStepClears) {
        // (the first iteration of a C tile starts its sums from zero instead of
        // from accumulators that would have to be cleared first; the fragment
        // addresses of the next iteration are worked out among the last MFMAs
        // of this one, so that only the wait and the barrier stand between two
        // iterations' MFMAs)
        // (no fragment is read after the step calls this, so it overwrites in place)
        auto next_addresses = [&] {
#pragma unroll
          for (int i = 0; i < 4; ++i) xa[i] = lds_base + x_slot_off(x_next) + xo[i];
          ya = lds_base + y_slot_off(y_next) + (y_frag_off - X_BYTES);
        };
        if (it == 0) {
          mma_step_ordered<DT, BX, BY, XT, true>(xa, ya, acc_re, acc_im, refill_slots,
                                                 next_addresses);
        } else {
          mma_step_ordered<DT, BX, BY, XT, false>(xa, ya, acc_re, acc_im, refill_slots,
                                                  next_addresses);
        }
      } else {
        const char *slot_ptr = lds + x_slot_off(x_slot);
        if constexpr (IL && MS == 32) {
          static_assert(TX == 2 && TY == 2, "2 x 2 tiles of 32 x 32 per wave");
          mma_step32_interleaved<DT, BX, BY>(slot_ptr, xil32_off, yil32_off, acc_re, acc_im,
                                             refill_slots);
        } else if constexpr (IL && DtypeTraits<DT>::kElemBytes == 2 && TX == 4 && TY == 4) {
          mma_step_interleaved_ordered<DT, BX, BY>(slot_ptr, xil_off, yil_off, acc_re, acc_im,
                                                   refill_slots);
        } else if constexpr (IL) {
          mma_step_interleaved<DT, BX, BY, TX, TY>(slot_ptr, xil_off, yil_off, acc_re, acc_im,
                                                   refill_slots);
        } else {
          const char *tile[KPM] = {slot_ptr};
          if constexpr (DT == kInt1) {
            static_assert(MS == 32 && TX == 2 && TY == 2, "2 x 2 tiles of 32 x 32 per wave");
            mma_step32_bits<BX, BY>(tile[0], x32_off, y32_off, acc_re, acc_im, refill_slots);
          } else if constexpr (MS == 32 && TX == 2 && TY == 2) {
            mma_step32_ordered<DT, BX, BY>(tile[0], x32_off, y32_off, acc_re, acc_im, refill_slots);
          } else if constexpr (MS == 32) {
            mma_step32<DT, BX, BY, TX, TY>(tile[0], x32_off, y32_off, acc_re, acc_im, refill_slots);
          } else {
            mma_step<DT, BX, BY, TX, TY>(tile, x_frag_off, y_frag_off, acc_re, acc_im, refill_slots);
          }
        }
      }
      x_slot = x_next;
      y_slot = y_next;
    }
    // The stores below are not waited for here: they drain while the next C
    // tile is being computed. The counter cannot tell loads from stores, so
    // the next tile's first K tiles, which are already on their way, are waited
    // for now; the first wait that has to include the stores then comes YLEAD
    // iterations into the next tile.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const TileCoord tc = tile_coord(args, vt);
    const unsigned x_wave = tc.block_x * BX + wx * WX, y_wave = tc.block_y * BY + wy * WY;
    bool staged = false;
    if constexpr (XT) {
      // the accumulators already hold whole row segments
      if (staged_ok && !args.c_interleaved && x_wave + WX <= args.nx && y_wave + WY <= args.ny) {
        store_wave_tile_rows<TOUT, TY>(args, tc.b, x_wave, y_wave, lane, acc_re, acc_im);
      } else {
        store_wave_tile<TOUT, TX, TY, kAcc16T>(args, tc.b, x_wave, y_wave, lane, acc_re, acc_im);
      }
      staged = true;
    }
    if constexpr (!XT && MS == 16 && TOUT == kFloat32 && TX == 4 &&
                  !SPLIT && NW * kStagePatchBytes <= SLOT_BYTES) {
      if (staged_ok) {
        // The slot consumed last is free until the next refill, but other waves
        // may still be reading it: one barrier, then every wave uses its own
        // patch of it. (Uniform per block, so the barrier is safe.)
        // ([X | Y] slots here: the rings are one)
        unsigned free_slot = y_slot + YLEAD;
        free_slot = free_slot >= SLOTS ? free_slot - SLOTS : free_slot;
        asm volatile("s_barrier" ::: "memory");
        if (x_wave + WX <= args.nx && y_wave + WY <= args.ny) {
          char *patch = lds + free_slot * SLOT_BYTES + wave * kStagePatchBytes;
          if (args.c_interleaved) {
            store_wave_tile_staged_il<TX, TY>(args, tc.b, x_wave, y_wave, lane, patch, acc_re, acc_im);
          } else {
            store_wave_tile_staged<TX, TY>(args, tc.b, x_wave, y_wave, lane, patch, acc_re, acc_im);
          }
          staged = true;
        }
      }
    }
    if constexpr (!XT && MS == 16 && (TOUT == kFloat16 || TOUT == kBfloat16) && TX == 4 &&
                  !SPLIT && NW * kStagePatchBytes <= SLOT_BYTES) {
      if (staged_ok && !args.c_interleaved && args.nx % 8 == 0) {
        // ([X | Y] slots here: the rings are one)
        unsigned free_slot = y_slot + YLEAD;
        free_slot = free_slot >= SLOTS ? free_slot - SLOTS : free_slot;
        asm volatile("s_barrier" ::: "memory");
        if (x_wave + WX <= args.nx && y_wave + WY <= args.ny) {
          store_wave_tile_staged_narrow<TOUT, TX, TY>(
              args, tc.b, x_wave, y_wave, lane,
              lds + free_slot * SLOT_BYTES + wave * kStagePatchBytes, acc_re, acc_im);
          staged = true;
        }
      }
    }
    if constexpr (MS == 32 && (TOUT == kFloat32 || TOUT == kInt32) &&
                  !SPLIT && NW * kStagePatch32Bytes <= SLOT_BYTES) {
      if (staged_ok) {
        // ([X | Y] slots here: the rings are one)
        unsigned free_slot = y_slot + YLEAD;
        free_slot = free_slot >= SLOTS ? free_slot - SLOTS : free_slot;
        asm volatile("s_barrier" ::: "memory");
        if (x_wave + WX <= args.nx && y_wave + WY <= args.ny) {
          store_wave_tile_staged32<TX, TY, TOUT == kInt32>(args, tc.b, x_wave, y_wave, lane,
                                           lds + free_slot * SLOT_BYTES + wave * kStagePatch32Bytes,
                                           acc_re, acc_im);
          staged = true;
        }
      }
    }
    if (!staged) {
      if constexpr (TOUT == kInt32) {
        store_wave_tile_int32<TX, TY, MS>(args, tc.b, x_wave, y_wave, lane, acc_re, acc_im);
      } else {
        store_wave_tile<TOUT, TX, TY, MS>(args, tc.b, x_wave, y_wave, lane, acc_re, acc_im);
      }
    }
  }
  // nothing may still be writing into LDS when the block gives it back
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

inline hipError_t check_grid(size_t total) {
  return total > 0x7fffffffu ? hipErrorInvalidValue : hipSuccess;
}

// LDS beyond 64 KiB has to be requested once per kernel and device. `done`
// is the caller's per-kernel record (one flag per device ordinal).
constexpr int kMaxDevices = 64;
template <typename Kernel>
hipError_t allow_lds(Kernel kernel, int bytes, std::atomic<bool> (&done)[kMaxDevices]) {
  if (bytes <= 64 * 1024) return hipSuccess;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked && done[dev].load(std::memory_order_acquire)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && tracked) done[dev].store(true, std::memory_order_release);
  return e;
}

template <int DT, int TOUT, int BX, int BY, int WX, int WY, int KT, int LOADER, int WPE>
hipError_t launch_config(const GemmParams &p, hipStream_t stream) {
  constexpr int NTHREADS = 64 * (BX / WX) * (BY / WY);
  constexpr int LDS_BYTES = 2 * KT * 2 * (BX + BY) * kTileRowBytes;
  const KernelArgs a = make_kernel_args(p, BX, BY);
  const size_t total = (size_t)a.blocks_x * a.blocks_y * p.batch;
  if (total == 0) return hipSuccess;
  if (hipError_t e = check_grid(total)) return e;
  auto kernel = complex_gemm_mfma<DT, TOUT, BX, BY, WX, WY, KT, LOADER, WPE>;
  static std::atomic<bool> lds_allowed[kMaxDevices];
  if (hipError_t e = allow_lds(kernel, LDS_BYTES, lds_allowed)) return e;
  hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(NTHREADS), LDS_BYTES, stream, a);
  return hipGetLastError();
}

// Number of compute units of the current device (queried once).
inline int compute_units() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0) {
      cus = 256;
    }
    return cus;
  }();
  return n;
}

template <int DT, int TOUT, int BX, int BY, int WX, int WY, int SLOTS, int WPE,
          int LOADER = kLoadTiled, int MS = 16, bool XT = false, int XSLOTS = SLOTS>
hipError_t launch_dtl(const GemmParams &p, hipStream_t stream) {
  constexpr int NTHREADS = 64 * (BX / WX) * (BY / WY);
  constexpr int LDS_BYTES = 2 * (XSLOTS * BX + SLOTS * BY) * kTileRowBytes;
  constexpr int kLdsPerCu = 160 * 1024;
  constexpr int BLOCKS_PER_CU = (kLdsPerCu / LDS_BYTES) < (WPE * 256 / NTHREADS)
                                    ? (kLdsPerCu / LDS_BYTES)
                                    : (WPE * 256 / NTHREADS);
  static_assert(BLOCKS_PER_CU >= 1, "configuration does not fit a CU");
  const KernelArgs a = make_kernel_args(p, BX, BY);
  const size_t total = (size_t)a.blocks_x * a.blocks_y * p.batch;
  if (total == 0) return hipSuccess;
  if (hipError_t e = check_grid(total)) return e;
  auto kernel = complex_gemm_mfma_dtl<DT, TOUT, BX, BY, WX, WY, SLOTS, WPE, LOADER, MS, XT, XSLOTS>;
  static std::atomic<bool> lds_allowed[kMaxDevices];
  if (hipError_t e = allow_lds(kernel, LDS_BYTES, lds_allowed)) return e;
  // persistent blocks: as many as are resident at once, each walking C tiles
  // with a stride of the grid size (a multiple of the XCD count)
  const size_t resident = (size_t)compute_units() * BLOCKS_PER_CU / kNumXcd * kNumXcd;
  const unsigned grid = (unsigned)(total < resident ? total : resident);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(NTHREADS), LDS_BYTES, stream, a);
  return hipGetLastError();
}

// How the 192 x 256 kernel covers the width of C: tiles of 192 columns, the last of
// which may hang over the edge, or - where 64 divides the width - full tiles
// followed by short ones of 128 columns, which take two thirds of the matrix
// instructions: as many as make the width come out even (4096 = 20 x 192 + 2 x 128),
// or three more for two full ones less as long as that shortens the work of the
// block that finishes last (8192 = 32 x 192 + 16 x 128: with 32 rows of tiles every
// one of 256 blocks gets 4 full and 2 short tiles, 5 1/3 full tiles' worth, where
// 42 x 192 + 128 would give 64 of them 6 full tiles). The short tiles are the last
// ones in the kernel's numbering; `rounds` is that longest block's work in full
// tiles, with a charge for the change of kind.
struct WideTiling {
  unsigned full_x, short_x, grid;
  double rounds;
};
// (the tuner switches the short tiles off for a row of its table)
static bool g_wide_short_tiles = true;
inline WideTiling wide_tiling(const GemmParams &p) {
  const size_t resident = (size_t)compute_units() / kNumXcd * kNumXcd;
  const size_t rows = ceil_div((size_t)p.ny, (size_t)kWideBY) * p.batch;
  WideTiling best;
  best.full_x = (unsigned)ceil_div((size_t)p.nx, (size_t)kWideBX);
  best.short_x = 0;
  const size_t plain_total = best.full_x * rows;
  best.grid = (unsigned)(plain_total < resident ? plain_total : resident);
  best.rounds = best.grid ? (double)ceil_div(plain_total, (size_t)best.grid) : 0.0;
  const size_t units = p.nx / 64;
  if (!g_wide_short_tiles || p.nx % 64 != 0 || plain_total == 0) return best;
  const double short_work = (double)kWideShortBX / kWideBX, change = 0.05;
  for (size_t n_short = units % 3 == 0 ? 3 : units % 3 == 2 ? 1 : 2; 3 + 2 * n_short <= units; n_short += 3) {
    WideTiling mixed;
    mixed.full_x = (unsigned)((units - 2 * n_short) / 3);
    mixed.short_x = (unsigned)n_short;
    const size_t full_total = mixed.full_x * rows, total = full_total + n_short * rows;
    mixed.grid = (unsigned)(total < resident ? total : resident);
    // block i computes the tiles i, i + grid, ...
    mixed.rounds = 0.0;
    for (size_t i = 0; i < mixed.grid; ++i) {
      const size_t mine = (total - i + mixed.grid - 1) / mixed.grid;
      const size_t full = i < full_total ? (full_total - i + mixed.grid - 1) / mixed.grid : 0;
      const double work =
          (double)full + short_work * (double)(mine - full) + (full > 0 && mine > full ? change : 0.0);
      mixed.rounds = work > mixed.rounds ? work : mixed.rounds;
    }
    if (mixed.rounds < best.rounds - 1e-9) best = mixed;
  }
  return best;
}

// The 192 x 256 block of gemm_mfma_wide.h (16-bit input; tiled layout, or IL: the
// pipeline's interleaved rows): one persistent block per compute unit.
template <int DT, int TOUT, bool IL = false>
hipError_t launch_wide(const GemmParams &p, hipStream_t stream) {
  KernelArgs a = make_kernel_args(p, kWideBX, kWideBY);
  const WideTiling tiling = wide_tiling(p);
  a.blocks_x = tiling.full_x;
  a.short_x = tiling.short_x;
  const size_t total = (size_t)(a.blocks_x + a.short_x) * a.blocks_y * p.batch;
  if (total == 0) return hipSuccess;
  if (hipError_t e = check_grid(total)) return e;
  const unsigned grid = tiling.grid;
  if (p.have_alpha) {
    auto kernel = complex_gemm_mfma_wide<DT, TOUT, IL, true>;
    static std::atomic<bool> lds_allowed[kMaxDevices];
    if (hipError_t e = allow_lds(kernel, kWideLdsBytes, lds_allowed)) return e;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), kWideLdsBytes, stream, a);
  } else {
    auto kernel = complex_gemm_mfma_wide<DT, TOUT, IL, false>;
    static std::atomic<bool> lds_allowed[kMaxDevices];
    if (hipError_t e = allow_lds(kernel, kWideLdsBytes, lds_allowed)) return e;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), kWideLdsBytes, stream, a);
  }
  return hipGetLastError();
}

// Whether 128 x 128 block tiles beat 256 x 128 ones for this problem: they do
// when the larger tiles would leave compute units without work (fewer tiles
// than units, or a last round that is mostly empty), although the smaller
// block moves a third more bytes from L2 to LDS per flop (`penalty`: how much
// slower per flop it measured once every unit is busy). Estimated from the
// fraction of unit-rounds that hold a tile under either tiling.
inline bool small_tiles_pay(const GemmParams &p, double penalty) {
  if (p.block_tile == 1 || p.block_tile == 2) return p.block_tile == 2;
  const size_t units = (size_t)compute_units();
  auto busy = [&](size_t bx, size_t by) {
    const size_t tiles = (size_t)p.batch * ceil_div((size_t)p.nx, bx) * ceil_div((size_t)p.ny, by);
    return (double)tiles / (double)(units * ceil_div(tiles, units));
  };
  return busy(128, 128) / penalty > busy(256, 128);
}

// Whether the 192 x 256 block of gemm_mfma_wide.h can compute this problem (what
// its stores and its K loop assume), and whether it pays: per flop it measured
// about 7 % faster than the 256 x 128 block once every compute unit is busy
// (B=64 512x4096x576: 0.519 against 0.558 ms), but its tiles are 1.5 times as
// large, so more of the last round of tiles can stay empty - which the short
// tiles of wide_tiling even out where the width allows (8192^3: 5 1/3 tiles for
// every block, 2.75 against 2.78 ms).
inline bool wide_tiles_apply(const GemmParams &p) {
  if (p.c_interleaved || p.have_beta || (uintptr_t)p.c % 16 != 0 ||
      p.nx % 64 != 0 || p.ny % 64 != 0 || p.k_in_memory) {
    return false;
  }
  if (p.input_interleaved) {
    // rows of whole 128-byte pieces (32 complex values), at least two of them; a
    // lane's offset inside a copy of 8 rows is a 32-bit number
    const size_t row_bytes = (size_t)2 * p.k * bits_of(p.type_in) / 8;
    return bits_of(p.type_in) == 16 && row_bytes % 128 == 0 && row_bytes >= 256 &&
           row_bytes < ((size_t)1 << 28) && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 16 == 0;
  }
  return p.variant == kOpt && p.k_tiles >= 2;
}
inline bool wide_tiles_pay(const GemmParams &p) {
  if (p.block_tile != 0) return p.block_tile == 3;
  const size_t units = (size_t)compute_units();
  // fraction of the unit-rounds' tile area that holds elements of C
  auto useful = [&](size_t bx, size_t by) {
    const size_t cols = ceil_div((size_t)p.nx, bx), rows = ceil_div((size_t)p.ny, by);
    const size_t tiles = (size_t)p.batch * cols * rows;
    return (double)p.batch * p.nx * p.ny / (double)(units * ceil_div(tiles, units) * bx * by);
  };
  const double wide_useful =
      (double)p.batch * p.nx * p.ny / ((double)units * wide_tiling(p).rounds * kWideBX * kWideBY);
  const double other = useful(256, 128) > useful(128, 128) / 1.15 ? useful(256, 128)
                                                                   : useful(128, 128) / 1.15;
  return wide_useful * 1.075 > other;
}

template <int DT, int TOUT>
hipError_t launch_typed(const GemmParams &p, hipStream_t stream) {
  constexpr int KPM = DtypeTraits<DT>::kTilesPerMfma;
  const size_t k_bytes = (size_t)p.k * bits_of(p.type_in) / 8;
  // planar rows made of whole, aligned 16-byte chunks can be copied straight
  // into LDS as well; anything else goes through the register-staged kernel
  const bool planar_direct = (p.variant == kBasic) && (k_bytes >= 16) && (k_bytes % 16 == 0) &&
                             ((uintptr_t)p.x % 16 == 0) && ((uintptr_t)p.y % 16 == 0);
  if (p.input_interleaved) {
    // raw (re, im) rows straight from the caller: the host side only takes this
    // path for 8- and 16-bit input whose rows are whole aligned 16-byte chunks
    if constexpr (DT == kFloat32) {
      return hipErrorInvalidValue;
    } else if constexpr (KPM == 1) {
      if constexpr (DtypeTraits<DT>::kElemBytes == 2) {
        if (wide_tiles_apply(p) && wide_tiles_pay(p)) return launch_wide<DT, TOUT, true>(p, stream);
      }
      if (small_tiles_pay(p, 1.15)) {
        return launch_dtl<DT, TOUT, 128, 128, 64, 32, 4, 2, kLoadInterleavedVec>(p, stream);
      }
      return launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadInterleavedVec>(p, stream);
    } else {
      if (small_tiles_pay(p, 1.05)) {
        return launch_dtl<DT, TOUT, 128, 128, 64, 64, 2, 2, kLoadInterleavedVec, 32>(p, stream);
      }
      return launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadInterleavedVec, 32>(p, stream);
    }
  }
  if (p.variant == kOpt || planar_direct) {
    if constexpr (KPM == 1 && DtypeTraits<DT>::kElemBytes == 2) {
      // 16-bit input, tiled operands, planar C without beta: 192 x 256 block, 4 waves
      // of 192 x 64 (one per SIMD), where that pays
      if (wide_tiles_apply(p) && wide_tiles_pay(p)) return launch_wide<DT, TOUT>(p, stream);
    }
    if constexpr (KPM == 1) {
      // 16- and 32-bit input: 256 x 128 block, 8 waves of 64 x 64 (two per SIMD), 3-slot ring.
      // Interleaved fp32 C: in the exchanged-roles layout a lane's (re, im) pairs of
      // a row lie 32 bytes apart, so every store instruction would write half
      // cache lines; the other layout regroups the tile through LDS into whole
      // rows of pairs (measured 5 % faster at B=64 512x4096x576).
      if constexpr (TOUT == kFloat32) {
        if (p.variant == kOpt && p.c_interleaved) {
          return launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadTiled, 16, false>(p, stream);
        }
      }
      // problems too small to give every compute unit a 256 x 128 tile: 128 x 128
      // blocks, 8 waves of 64 x 32, 4-slot ring
      if (small_tiles_pay(p, 1.15)) {
        return p.variant == kOpt
                   ? launch_dtl<DT, TOUT, 128, 128, 64, 32, 4, 2, kLoadTiled, 16>(p, stream)
                   : launch_dtl<DT, TOUT, 128, 128, 64, 32, 4, 2, kLoadPlanarVec, 16>(p, stream);
      }
      return p.variant == kOpt
                 ? launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadTiled, 16, true>(p, stream)
                 : launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 16, true>(p, stream);
    } else {
      // fp8: the 32x32x64 MFMA takes one K tile per instruction, which lets the
      // same block shape and ring as for 16-bit input fit into LDS
      // (small problems: 128 x 128 blocks, 4 waves of 64 x 64, two blocks a unit)
      if (small_tiles_pay(p, 1.05)) {
        return p.variant == kOpt
                   ? launch_dtl<DT, TOUT, 128, 128, 64, 64, 2, 2, kLoadTiled, 32>(p, stream)
                   : launch_dtl<DT, TOUT, 128, 128, 64, 64, 2, 2, kLoadPlanarVec, 32>(p, stream);
      }
      return p.variant == kOpt
                 ? launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>(p, stream)
                 : launch_dtl<DT, TOUT, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 32>(p, stream);
    }
  }
  // fp8 stages are twice as large (two K tiles per MFMA): one wave per SIMD
  // with the full register file
  constexpr int WPE = (KPM == 2) ? 1 : 2;
  return launch_config<DT, TOUT, 128, 128, 64, 64, KPM, kLoadPlanarElem, WPE>(p, stream);
}

}  // namespace

// The instantiations are spread over several translation units so that they
// compile in parallel: gemm_mfma_<part>.hip define CCGLIB_GEMM_MFMA_PART and
// include this file (1 fp16, 2 bf16, 3 fp32, 4 fp8, 5 1-bit input; 0 the
// dispatch below). Included without the macro (the tuning program), the file
// holds everything.
#ifndef CCGLIB_GEMM_MFMA_PART
#define CCGLIB_GEMM_MFMA_PART -1
#endif
#define CCGLIB_GEMM_MFMA_HAS(part) (CCGLIB_GEMM_MFMA_PART == -1 || CCGLIB_GEMM_MFMA_PART == (part))

hipError_t launch_gemm_mfma_f16(const GemmParams &p, hipStream_t stream);
hipError_t launch_gemm_mfma_bf16(const GemmParams &p, hipStream_t stream);
hipError_t launch_gemm_mfma_f32(const GemmParams &p, hipStream_t stream);
hipError_t launch_gemm_mfma_fp8(const GemmParams &p, hipStream_t stream);
hipError_t launch_gemm_mfma_int1(const GemmParams &p, hipStream_t stream);

#if CCGLIB_GEMM_MFMA_HAS(1)
hipError_t launch_gemm_mfma_f16(const GemmParams &p, hipStream_t stream) {
  if (p.type_out == kFloat32) return launch_typed<kFloat16, kFloat32>(p, stream);
  if (p.type_out == kFloat16) return launch_typed<kFloat16, kFloat16>(p, stream);
  return hipErrorInvalidValue;
}
#endif

#if CCGLIB_GEMM_MFMA_HAS(2)
hipError_t launch_gemm_mfma_bf16(const GemmParams &p, hipStream_t stream) {
  if (p.type_out == kFloat32) return launch_typed<kBfloat16, kFloat32>(p, stream);
  if (p.type_out == kBfloat16) return launch_typed<kBfloat16, kBfloat16>(p, stream);
  return hipErrorInvalidValue;
}
#endif

#if CCGLIB_GEMM_MFMA_HAS(3)
hipError_t launch_gemm_mfma_f32(const GemmParams &p, hipStream_t stream) {
  if (p.type_out == kFloat32) return launch_typed<kFloat32, kFloat32>(p, stream);
  if (p.type_out == kFloat16) return launch_typed<kFloat32, kFloat16>(p, stream);
  if (p.type_out == kBfloat16) return launch_typed<kFloat32, kBfloat16>(p, stream);
  return hipErrorInvalidValue;
}
#endif

#if CCGLIB_GEMM_MFMA_HAS(4)
hipError_t launch_gemm_mfma_fp8(const GemmParams &p, hipStream_t stream) {
  if (p.type_out != kFloat32) return hipErrorInvalidValue;
  return p.type_in == kFloat8e4m3 ? launch_typed<kFloat8e4m3, kFloat32>(p, stream)
                                  : launch_typed<kFloat8e5m2, kFloat32>(p, stream);
}
#endif

#if CCGLIB_GEMM_MFMA_HAS(5)
hipError_t launch_gemm_mfma_int1(const GemmParams &p, hipStream_t stream) {
  // packed 1-bit samples expanded in registers; the caller has checked that
  // planar rows are whole aligned 16-byte chunks and that K fits fp32 sums
  if (p.type_out != kInt32 || p.input_interleaved) return hipErrorInvalidValue;
  if (small_tiles_pay(p, 1.0)) {
    return p.variant == kOpt
               ? launch_dtl<kInt1, kInt32, 128, 128, 64, 64, 2, 2, kLoadTiled, 32>(p, stream)
               : launch_dtl<kInt1, kInt32, 128, 128, 64, 64, 2, 2, kLoadPlanarVec, 32>(p, stream);
  }
  return p.variant == kOpt
             ? launch_dtl<kInt1, kInt32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>(p, stream)
             : launch_dtl<kInt1, kInt32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 32>(p, stream);
}
#endif

#if CCGLIB_GEMM_MFMA_HAS(0)
// Which kernel launch_gemm_mfma starts for these parameters (the decisions of
// launch_typed, in words).
const char *describe_gemm_mfma(const GemmParams &p) {
  const bool bits8 = p.type_in == kFloat8e4m3 || p.type_in == kFloat8e5m2;
  const bool bits16 = p.type_in == kFloat16 || p.type_in == kBfloat16;
  const bool int1 = p.type_in == kInt1;
  const size_t k_bytes = (size_t)p.k * bits_of(p.type_in) / 8;
  const bool planar_direct = (p.variant == kBasic) && (k_bytes >= 16) && (k_bytes % 16 == 0) &&
                             ((uintptr_t)p.x % 16 == 0) && ((uintptr_t)p.y % 16 == 0);
  const double penalty = int1 ? 1.0 : bits8 ? 1.05 : 1.15;
  if (p.input_interleaved) {
    if (bits16 && wide_tiles_apply(p) && wide_tiles_pay(p)) {
      return "complex_gemm_mfma_wide, 192x256 block, one wave per SIMD, interleaved rows";
    }
    return small_tiles_pay(p, penalty) ? "complex_gemm_mfma_dtl, 128x128 block, interleaved rows"
                                       : "complex_gemm_mfma_dtl, 256x128 block, interleaved rows";
  }
  if (p.variant == kOpt || planar_direct || int1) {
    if (bits16 && wide_tiles_apply(p) && wide_tiles_pay(p)) {
      return "complex_gemm_mfma_wide, 192x256 block, one wave per SIMD";
    }
    if (p.variant == kOpt) {
      return small_tiles_pay(p, penalty) ? "complex_gemm_mfma_dtl, 128x128 block, tiled operands"
                                         : "complex_gemm_mfma_dtl, 256x128 block, tiled operands";
    }
    return small_tiles_pay(p, penalty) ? "complex_gemm_mfma_dtl, 128x128 block, planar rows"
                                       : "complex_gemm_mfma_dtl, 256x128 block, planar rows";
  }
  return "complex_gemm_mfma, 128x128 block, planar rows through registers";
}

hipError_t launch_gemm_mfma(const GemmParams &p, hipStream_t stream) {
  switch (p.type_in) {
    case kFloat16: return launch_gemm_mfma_f16(p, stream);
    case kBfloat16: return launch_gemm_mfma_bf16(p, stream);
    case kFloat32: return launch_gemm_mfma_f32(p, stream);
    case kFloat8e4m3:
    case kFloat8e5m2: return launch_gemm_mfma_fp8(p, stream);
    case kInt1: return launch_gemm_mfma_int1(p, stream);
    default: return hipErrorInvalidValue;
  }
}
#endif

}  // namespace ccglib_amd
