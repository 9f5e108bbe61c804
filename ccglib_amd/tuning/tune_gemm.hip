// Offline sweep over kernel configurations of the complex GEMM on one gfx950
// device: the counterpart of the reference's tuning/tune_gemm.py (which sweeps
// block and warp tile sizes of its kernel through a JIT tuner).
// The configurations here are template instantiations of the library's own
// kernels (block tile, wave tile, ring slots, MFMA shape, operand layout), timed
// back to back on operands of the given shape; the library's dispatch
// (launch_typed in ../csrc/gemm_mfma.hip) uses the winners.
//
//   make && ./tune_gemm [--fill=baseline|legacy|zero] [B M N K [filter]]
//                                            e.g.  ./tune_gemm 64 512 4096 576 f16
//
// --fill=baseline (default): the operand distributions of the benchmark
//   configurations - real and imaginary parts N(0, 1) for fp16 / bf16 / fp32
//   (for B=64 M=512 N=4096 K=576, the beamformer shape, the M-row operand holds
//   unit-magnitude random phases), N(0, 1) scaled into the fp8 range (x 448 / 5.8
//   for e4m3: the largest of 10^8 normal samples is about 5.8) and quantised,
//   Bernoulli(0.5) bits for 1-bit input. The part is power limited, and what the
//   operands hold decides how fast a kernel runs.
// --fill=legacy: the fill of earlier sweeps (a 2 MiB pattern of numbers with three
//   exponents; fp8 without sign bit), kept for comparison with their files.
// --fill=zero: all-zero operands (no power limit).
// `make ABLATE=n` builds timing-only variants (see CCGLIB_ABLATE in gemm_mfma.hip).
//
//   ./tune_gemm --probe=mfma|mix|fill|l2read [--fill=...]
// Small probes of the machine that the kernels' floors are argued from: the rate
// of matrix instructions issued from registers alone (1 or 2 waves per SIMD, the
// operands changing from instruction to instruction), what an instruction between
// two matrix instructions costs a wave that has the SIMD to itself, the rate of a
// plain fill of 1 GiB, and the rate at which all compute units read a window of a
// given size over and over (L2 and memory-side cache).
// TUNE_GEMM_SMALL (make SMALL=1): only the 16-bit rows of the beamformer sweep - the
// kernels one works on most - for a build of under a minute.
#ifdef TUNE_GEMM_SMALL
#define CCGLIB_GEMM_MFMA_PART 99   // none of the library's own instantiations
#endif
#include "../csrc/gemm_mfma.hip"
#ifndef TUNE_GEMM_SMALL
#include "../csrc/gemm_int1.hip"
#endif

#include <hip/hip_fp8.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

using namespace ccglib_amd;

#define CHECK(x)                                                                      \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
      std::exit(1);                                                                   \
    }                                                                                 \
  } while (0)

typedef hipError_t (*LaunchFn)(const GemmParams &, hipStream_t);
struct Config {
  const char *name;
  LaunchFn launch;
  int type_in, type_out;
  int layout = kLoadTiled;   // operand layout the configuration reads
  double peak = 0;           // what "of peak" refers to (0: the input type's MFMA peak)
};

#ifndef TUNE_GEMM_SMALL
// the 1-bit GEMM on the vector ALUs (XOR + population count), whatever the layout
static hipError_t launch_popcount(const GemmParams &p, hipStream_t stream) {
  GemmParams q = p;
  q.int1_direct = 0;
  return launch_gemm_int1(q, stream);
}
#endif
// 256 CUs x 64 lane-operations per clock x 2.4 GHz, 8 lane-operations (4 XOR, 4
// counts) per 32 complex products of 8 "operations" each
constexpr double kPopcountRoof = 256 * 64 * 2.4e9 * 32 / 1e12;   // 1258 TOP/s

// the 192 x 256 kernel with tiles of 192 columns only (the last one hanging over the edge)
template <int DT, int TOUT, bool IL>
hipError_t launch_wide_full_tiles(const GemmParams &p, hipStream_t stream) {
  g_wide_short_tiles = false;
  const hipError_t e = launch_wide<DT, TOUT, IL>(p, stream);
  g_wide_short_tiles = true;
  return e;
}

// name: type, [operand layout,] block BX x BY, wave WX x WY, ring slots, MFMA rows
static const std::vector<Config> kConfigs = {
#ifndef TUNE_GEMM_SMALL
    {"f16 256x128 w64x64 s3 m16", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16>, kFloat16, kFloat32},
#endif
    {"f16 256x128 w64x64 s3 m16 xt", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16, true>, kFloat16, kFloat32},
    {"f16 128x256 w64x64 s3 m16 xt", launch_dtl<kFloat16, kFloat32, 128, 256, 64, 64, 3, 2, kLoadTiled, 16, true>, kFloat16, kFloat32},
    {"f16 128x256 w64x64 y3 x4 m16 xt", launch_dtl<kFloat16, kFloat32, 128, 256, 64, 64, 3, 2, kLoadTiled, 16, true, 4>, kFloat16, kFloat32},
    {"f16 192x256 w192x64 x3 y2 m16 xt 1wave", launch_wide<kFloat16, kFloat32, false>, kFloat16, kFloat32},
    {"f16 192x256 ... 1wave, full tiles only", launch_wide_full_tiles<kFloat16, kFloat32, false>, kFloat16, kFloat32},
    {"bf16 256x128 w64x64 s3 m16 xt", launch_dtl<kBfloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16, true>, kBfloat16, kFloat32},
    {"bf16 192x256 w192x64 x3 y2 m16 xt 1wave", launch_wide<kBfloat16, kFloat32, false>, kBfloat16, kFloat32},
#ifndef TUNE_GEMM_SMALL
    {"f16 256x128 w64x64 s3 m32", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>, kFloat16, kFloat32},
    {"f16 128x128 w64x64 s2 m16", launch_dtl<kFloat16, kFloat32, 128, 128, 64, 64, 2, 2, kLoadTiled, 16>, kFloat16, kFloat32},
    {"f16 128x128 w64x32 s4 m16", launch_dtl<kFloat16, kFloat32, 128, 128, 64, 32, 4, 2, kLoadTiled, 16>, kFloat16, kFloat32},
    {"f32 256x128 w64x64 s3 m16", launch_dtl<kFloat32, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16>, kFloat32, kFloat32},
    {"fp8 256x128 w64x64 s3 m32", launch_dtl<kFloat8e4m3, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>, kFloat8e4m3, kFloat32},
    {"fp8 128x128 w64x64 s2 m32", launch_dtl<kFloat8e4m3, kFloat32, 128, 128, 64, 64, 2, 2, kLoadTiled, 32>, kFloat8e4m3, kFloat32},
    {"fp8 128x128 w64x32 s4 m32", launch_dtl<kFloat8e4m3, kFloat32, 128, 128, 64, 32, 4, 2, kLoadTiled, 32>, kFloat8e4m3, kFloat32},
    {"int1 128x128 w64x64 s2 m32", launch_dtl<kInt1, kInt32, 128, 128, 64, 64, 2, 2, kLoadTiled, 32>, kInt1, kInt32},
    {"int1 256x128 w64x64 s3 m32", launch_dtl<kInt1, kInt32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>, kInt1, kInt32},
    // the 1-bit GEMM on the vector ALUs; "of peak" is of its issue roof
    {"int1 popcount 128x128 (vector ALU)", launch_popcount, kInt1, kInt32, kLoadTiled, kPopcountRoof},
    {"int1 popcount planar 128x128 (vector ALU)", launch_popcount, kInt1, kInt32, kLoadPlanarVec, kPopcountRoof},
#endif
    // planar rows (basic variant) and raw interleaved rows (the pipeline's fused mode)
#ifndef TUNE_GEMM_SMALL
    {"f16 planar 256x128 w64x64 s3 m16", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 16>, kFloat16, kFloat32, kLoadPlanarVec},
#endif
#ifndef TUNE_GEMM_SMALL
    {"f16 planar 256x128 w64x64 s3 m16 xt", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 16, true>, kFloat16, kFloat32, kLoadPlanarVec},
#endif
    {"f16 interleaved 256x128 w64x64 s3 m16", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadInterleavedVec, 16>, kFloat16, kFloat32, kLoadInterleavedVec},
    {"f16 interleaved 192x256 w192x64 x3 y2 m16 xt 1wave", launch_wide<kFloat16, kFloat32, true>, kFloat16, kFloat32, kLoadInterleavedVec},
    {"f16 interleaved 192x256 ... 1wave, full tiles only", launch_wide_full_tiles<kFloat16, kFloat32, true>, kFloat16, kFloat32, kLoadInterleavedVec},
    {"bf16 interleaved 192x256 w192x64 x3 y2 m16 xt 1wave", launch_wide<kBfloat16, kFloat32, true>, kBfloat16, kFloat32, kLoadInterleavedVec},
#ifndef TUNE_GEMM_SMALL
    {"fp8 planar 256x128 w64x64 s3 m32", launch_dtl<kFloat8e4m3, kFloat32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 32>, kFloat8e4m3, kFloat32, kLoadPlanarVec},
#endif
#ifndef TUNE_GEMM_SMALL
    {"fp8 interleaved 256x128 w64x64 s3 m32", launch_dtl<kFloat8e4m3, kFloat32, 256, 128, 64, 64, 3, 2, kLoadInterleavedVec, 32>, kFloat8e4m3, kFloat32, kLoadInterleavedVec},
#endif
};

static double peak_of(int type) {
  switch (type) {
    case kFloat32: return 157.3;
    case kInt1: return 10066.3;
    case kFloat8e4m3:
    case kFloat8e5m2: return 5033.2;
    default: return 2516.6;
  }
}

// ---- operand fills ----------------------------------------------------------------
// A counter-based generator: what an element holds depends on its index and the
// seed only.
__device__ __forceinline__ unsigned mix32(unsigned long long x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdull;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ull;
  x ^= x >> 33;
  return (unsigned)x;
}
__device__ __forceinline__ float uniform01(unsigned r) { return (r >> 8) * (1.0f / 16777216.0f) + 0x1p-25f; }

template <typename T> __device__ __forceinline__ T to_type(float v);
template <> __device__ __forceinline__ _Float16 to_type<_Float16>(float v) { return (_Float16)v; }
template <> __device__ __forceinline__ __bf16 to_type<__bf16>(float v) { return (__bf16)v; }
template <> __device__ __forceinline__ float to_type<float>(float v) { return v; }
template <> __device__ __forceinline__ unsigned char to_type<unsigned char>(float v) {
  // e4m3, saturating, round to nearest even; N(0, 1) scaled into the type's range
  return (unsigned char)__hip_cvt_float_to_fp8(v * (448.0f / 5.8f), __HIP_SATFINITE, __HIP_E4M3);
}

// Pair i of an operand is the (re, im) of one complex element; `pos` maps it to
// the two element offsets of the layout in use. PHASES: unit magnitude, random
// phase; otherwise both parts N(0, 1).
struct PairLayout {
  int layout;
  unsigned long long plane;   // tiled: elements of one tile plane; planar: of one operand plane
};
template <typename T, bool PHASES>
__global__ void fill_pairs(T *out, unsigned long long pairs, PairLayout pl, unsigned long long seed) {
  for (unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x; i < pairs;
       i += (unsigned long long)gridDim.x * blockDim.x) {
    const float u = uniform01(mix32(2 * i + seed)), w = uniform01(mix32(2 * i + 1 + seed));
    const float angle = 6.2831853f * w;
    const float radius = PHASES ? 1.0f : sqrtf(-2.0f * logf(u));
    const float re = radius * cosf(angle), im = radius * sinf(angle);
    unsigned long long ire, iim;
    if (pl.layout == kLoadInterleavedVec) {
      ire = 2 * i;
      iim = 2 * i + 1;
    } else {   // a re plane followed by an im plane, per tile or per batch
      ire = (i / pl.plane) * 2 * pl.plane + i % pl.plane;
      iim = ire + pl.plane;
    }
    out[ire] = to_type<T>(re);
    out[iim] = to_type<T>(im);
  }
}
__global__ void fill_words(unsigned *out, unsigned long long words, unsigned long long seed) {
  for (unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x; i < words;
       i += (unsigned long long)gridDim.x * blockDim.x) {
    out[i] = mix32(i + seed);
  }
}

static void fill_baseline(void *d, size_t bytes, int type, int layout, size_t plane_elems, bool phases,
                          unsigned long long seed) {
  const dim3 grid(4096), block(256);
  if (type == kInt1) {
    hipLaunchKernelGGL(fill_words, grid, block, 0, 0, (unsigned *)d, (unsigned long long)(bytes / 4), seed);
    return;
  }
  const size_t elem = (size_t)bits_of(type) / 8;
  const unsigned long long pairs = bytes / elem / 2;
  const PairLayout pl{layout, (unsigned long long)plane_elems};
#define FILL(T)                                                                                     \
  if (phases) {                                                                                     \
    hipLaunchKernelGGL((fill_pairs<T, true>), grid, block, 0, 0, (T *)d, pairs, pl, seed);           \
  } else {                                                                                          \
    hipLaunchKernelGGL((fill_pairs<T, false>), grid, block, 0, 0, (T *)d, pairs, pl, seed);          \
  }
  if (type == kFloat16) {
    FILL(_Float16)
  } else if (type == kBfloat16) {
    FILL(__bf16)
  } else if (type == kFloat32) {
    FILL(float)
  } else {
    FILL(unsigned char)
  }
#undef FILL
}

// The fill of earlier sweeps: random operand bytes that are ordinary numbers in the
// given type, a 2 MiB pattern repeated over the operand.
static void fill_legacy(void *d, size_t bytes, int type) {
  std::vector<unsigned short> h(1 << 20);
  std::srand(1);
  for (auto &v : h) {
    const unsigned r = (unsigned)std::rand();
    if (type == kFloat16 || type == kBfloat16) {
      const int e = (type == kFloat16 ? 13 : 125) + (int)(r % 3);
      v = (unsigned short)(((r >> 8 & 1) << 15) | (e << (type == kFloat16 ? 10 : 7)) | (r >> 9 & (type == kFloat16 ? 0x3ff : 0x7f)));
    } else if (type == kInt1) {
      v = (unsigned short)(r >> 4);
    } else {
      v = (unsigned short)((r & 0x3f3f) | 0x2020);
    }
  }
  if (type == kFloat32) {
    float *f = reinterpret_cast<float *>(h.data());
    for (size_t i = 0; i < h.size() / 2; ++i) f[i] = (std::rand() / (float)RAND_MAX) * 4.f - 2.f;
  }
  for (size_t o = 0; o < bytes; o += h.size() * 2)
    CHECK(hipMemcpy((char *)d + o, h.data(), std::min(h.size() * 2, bytes - o), hipMemcpyHostToDevice));
}


// ---- probes ------------------------------------------------------------------------
typedef float f16v_t __attribute__((ext_vector_type(16)));

// MFMAs from registers only. SHAPE 16: 16x16x32, 32: 32x32x16 (fp16). Four A and
// four B operand sets take turns so that the inputs change as in a GEMM.
template <int SHAPE, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES / 4) void probe_mfma(const int4_t *in, float *out, int iters) {
  extern __shared__ char probe_lds[];
  int4_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = in[(threadIdx.x % 64) * 8 + i];
    b[i] = in[(threadIdx.x % 64) * 8 + 4 + i];
  }
  constexpr int NACC = SHAPE == 16 ? 16 : 8;
  typename AccType<SHAPE>::type acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 64; ++n) {
      if constexpr (SHAPE == 16) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[n % NACC]) : "v"(a[n % 4]), "v"(b[(n / 4) % 4]));
      } else {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[n % NACC]) : "v"(a[n % 4]), "v"(b[(n / 4) % 4]));
      }
    }
  }
  asm volatile("s_nop 15\n\ts_nop 15");
  float s = 0;
#pragma unroll
  for (int i = 0; i < NACC; ++i) s += acc[i][0] + acc[i][3];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// What an instruction between two 16x16x32 MFMAs costs one wave per SIMD. MODE 0:
// none; 1 / 2: one / two vector-ALU instructions behind every MFMA; 3: four in a row
// behind every fourth; 4: a ds_read_b128 behind every eighth; 5: a 1 KiB global ->
// LDS copy behind every twelfth; 6: four such copies in a row behind every 48th.
template <int MODE>
__global__ __launch_bounds__(256, 1) void probe_mix(const int4_t *in, float *out, int iters) {
  extern __shared__ __attribute__((aligned(1024))) char probe_lds[];
  int4_t a = in[(threadIdx.x % 64) * 8], b = in[(threadIdx.x % 64) * 8 + 4];
  float4_t acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  int x0 = a[0], x1 = a[1], x2 = a[2], x3 = a[3];
  int4_t l = {0, 0, 0, 0};
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char *)probe_lds;
  const unsigned la = lds_base + 65536 + (threadIdx.x % 64) * 16;
  const unsigned wave = (unsigned)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / 64));
  const char *src = reinterpret_cast<const char *>(in);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 96; ++n) {
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[n % 16]) : "v"(a), "v"(b));
      if (MODE == 1 || MODE == 2) asm volatile("v_xor_b32 %0, 0x80008000, %0" : "+v"(x0));
      if (MODE == 2) asm volatile("v_xor_b32 %0, 0x80008000, %0" : "+v"(x1));
      if (MODE == 3 && (n & 3) == 3) {
        asm volatile("v_xor_b32 %0, 0x80008000, %0\n\tv_xor_b32 %1, 0x80008000, %1\n\t"
                     "v_xor_b32 %2, 0x80008000, %2\n\tv_xor_b32 %3, 0x80008000, %3"
                     : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));
      }
      if (MODE == 4 && (n & 7) == 7) asm volatile("ds_read_b128 %0, %1" : "=v"(l) : "v"(la));
      if (MODE == 5 && n % 12 == 11) load_1k_to_lds(src, (threadIdx.x % 64) * 16, lds_base + wave * 8192 + (n / 12) * 1024);
      if (MODE == 6 && n % 48 == 47) {
#pragma unroll
        for (int c = 0; c < 4; ++c) load_1k_to_lds(src, (threadIdx.x % 64) * 16, lds_base + wave * 8192 + c * 1024);
      }
    }
    if (MODE == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(l));
    if (MODE == 5 || MODE == 6) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  asm volatile("s_nop 15\n\ts_nop 15");
  float s = x0 + x1 + x2 + x3 + l[0];
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i][0];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ void probe_fill(float4_t *out, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    out[i] = float4_t{1.f, 2.f, 3.f, 4.f};
  }
}
// every block reads the whole window `rounds` times, each block starting elsewhere
__global__ void probe_window_read(const int4_t *in, size_t n, int rounds, int *sink) {
  int4_t s = {0, 0, 0, 0};
  const size_t start = (blockIdx.x * 977u % 1024u) * (n / 1024);
  for (int r = 0; r < rounds; ++r) {
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
      size_t j = i + start;
      j = j >= n ? j - n : j;
      const int4_t v = in[j];
      s[0] ^= v[0];
      s[1] ^= v[1];
      s[2] ^= v[2];
      s[3] ^= v[3];
    }
  }
  if ((s[0] ^ s[1] ^ s[2] ^ s[3]) == 0x12345678) *sink = 1;
}

template <typename F> static float time_launches(F &&launch, int reps) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  float ms = 0;
  for (int round = 0; round < 2; ++round) {   // the second round is the settled one
    CHECK(hipEventRecord(e0));
    for (int i = 0; i < reps; ++i) launch();
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    CHECK(hipEventElapsedTime(&ms, e0, e1));
  }
  return ms / reps;
}

static int run_probe(const std::string &probe, const std::string &fill) {
  int4_t *in;
  float *out;
  CHECK(hipMalloc(&in, 1 << 20));
  CHECK(hipMalloc(&out, 256 * 512 * 4));
  if (fill == "zero") {
    CHECK(hipMemset(in, 0, 1 << 20));
  } else {
    fill_baseline(in, 1 << 20, kFloat16, kLoadInterleavedVec, 1, false, 7);
  }
  CHECK(hipDeviceSynchronize());
  const int iters = 4000;
  if (probe == "mfma") {
    std::printf("matrix instructions from registers only, %s operands (four A and four B sets in turn), fp16\n", fill.c_str());
    auto run = [&](const char *name, auto kernel, int waves, double flop_per_mfma) {
      CHECK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));
      const float ms = time_launches([&] { hipLaunchKernelGGL(kernel, dim3(256), dim3(64 * waves), 100 * 1024, 0, in, out, iters); }, 10);
      const double tflops = 64.0 * flop_per_mfma * iters * waves * 256 / (ms * 1e-3) / 1e12;
      std::printf("%-32s %8.3f ms %8.1f TFLOP/s  %5.1f%% of 2516.6\n", name, ms, tflops, 100 * tflops / 2516.6);
    };
    run("16x16x32, 1 wave per SIMD", probe_mfma<16, 4>, 4, 2.0 * 16 * 16 * 32);
    run("16x16x32, 2 waves per SIMD", probe_mfma<16, 8>, 8, 2.0 * 16 * 16 * 32);
    run("32x32x16, 1 wave per SIMD", probe_mfma<32, 4>, 4, 2.0 * 32 * 32 * 16);
    run("32x32x16, 2 waves per SIMD", probe_mfma<32, 8>, 8, 2.0 * 32 * 32 * 16);
  } else if (probe == "mix") {
    std::printf("one wave per SIMD issuing 16x16x32 MFMAs and, between them (%s operands):\n", fill.c_str());
    auto run = [&](const char *name, auto kernel) {
      CHECK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));
      const float ms = time_launches([&] { hipLaunchKernelGGL(kernel, dim3(256), dim3(256), 100 * 1024, 0, in, out, iters); }, 10);
      const double tflops = 96.0 * 2 * 16 * 16 * 32 * iters * 4 * 256 / (ms * 1e-3) / 1e12;
      std::printf("%-52s %8.3f ms %8.1f TFLOP/s  %5.1f%% of 2516.6\n", name, ms, tflops, 100 * tflops / 2516.6);
    };
    run("nothing", probe_mix<0>);
    run("one v_xor behind every MFMA", probe_mix<1>);
    run("two v_xor behind every MFMA", probe_mix<2>);
    run("four v_xor in a row behind every 4th MFMA", probe_mix<3>);
    run("a ds_read_b128 behind every 8th MFMA", probe_mix<4>);
    run("a 1 KiB global -> LDS copy behind every 12th MFMA", probe_mix<5>);
    run("four such copies in a row behind every 48th MFMA", probe_mix<6>);
  } else if (probe == "fill") {
    for (size_t mib : {16, 256, 1024}) {
      float4_t *buf;
      CHECK(hipMalloc(&buf, mib << 20));
      const size_t n = (mib << 20) / 16;
      const float ms = time_launches([&] { hipLaunchKernelGGL(probe_fill, dim3(8192), dim3(256), 0, 0, buf, n); }, 20);
      std::printf("fill of %5zu MiB: %8.4f ms  %6.2f TB/s\n", mib, ms, (double)(mib << 20) / (ms * 1e-3) / 1e12);
      CHECK(hipFree(buf));
    }
  } else if (probe == "l2read") {
    int *sink;
    CHECK(hipMalloc(&sink, 4));
    for (size_t kib : {1024, 2048, 4096, 16384, 65536, 262144}) {
      int4_t *buf;
      CHECK(hipMalloc(&buf, kib << 10));
      CHECK(hipMemset(buf, 1, kib << 10));
      const size_t n = (kib << 10) / 16;
      const int rounds = (int)std::max<size_t>(1, (64 << 10) / kib);
      const float ms = time_launches([&] { hipLaunchKernelGGL(probe_window_read, dim3(1024), dim3(256), 0, 0, buf, n, rounds, sink); }, 5);
      std::printf("1024 blocks reading a window of %7zu KiB: %8.4f ms  %6.2f TB/s\n", kib, ms,
                  1024.0 * rounds * (kib << 10) / (ms * 1e-3) / 1e12);
      CHECK(hipFree(buf));
    }
  } else {
    std::printf("unknown probe '%s' (mfma, mix, fill or l2read)\n", probe.c_str());
    return 1;
  }
  return 0;
}

int main(int argc, char **argv) {
  unsigned B = 64, M = 512, N = 4096, K = 576;
  std::string fill = std::getenv("ZERO") ? "zero" : "baseline", probe;
  std::vector<const char *> pos;
  for (int i = 1; i < argc; ++i) {
    if (std::strncmp(argv[i], "--fill=", 7) == 0) {
      fill = argv[i] + 7;
    } else if (std::strncmp(argv[i], "--probe=", 8) == 0) {
      probe = argv[i] + 8;
    } else {
      pos.push_back(argv[i]);
    }
  }
  if (fill != "baseline" && fill != "legacy" && fill != "zero") {
    std::printf("unknown fill '%s' (baseline, legacy or zero)\n", fill.c_str());
    return 1;
  }
  if (!probe.empty()) return run_probe(probe, fill);
  if (pos.size() >= 4) {
    B = (unsigned)std::atoi(pos[0]);
    M = (unsigned)std::atoi(pos[1]);
    N = (unsigned)std::atoi(pos[2]);
    K = (unsigned)std::atoi(pos[3]);
  }
  const char *filter = pos.size() > 4 ? pos[4] : (pos.size() == 1 ? pos[0] : nullptr);
  const bool beamformer = B == 64 && M == 512 && N == 4096 && K == 576;
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  std::printf("%-44s %10s %12s %10s   (B=%u M=%u N=%u K=%u, %s operands%s)\n", "configuration", "ms", "TFLOP/s",
              "of peak", B, M, N, K, fill.c_str(), CCGLIB_ABLATE ? ", TIMING-ONLY BUILD" : "");
  if (CCGLIB_ABLATE) std::printf("CCGLIB_ABLATE = %d: parts of the kernels are left out, C is wrong\n", CCGLIB_ABLATE);
  for (const Config &c : kConfigs) {
    if (filter && !std::strstr(c.name, filter)) continue;
    GemmParams p;
    const int kpt = k_per_tile(c.type_in);
    p.batch = B;
    p.nx = N;
    p.ny = M;
    p.k = K;
    p.k_tiles = ((c.layout == kLoadInterleavedVec ? 2 * K : K) + kpt - 1) / kpt;
    p.x_tiles = (N + kTileRows - 1) / kTileRows;
    p.y_tiles = (M + kTileRows - 1) / kTileRows;
    p.type_in = c.type_in;
    p.type_out = c.type_out;
    p.variant = c.layout == kLoadPlanarVec ? kBasic : kOpt;
    p.c_interleaved = 0;
    p.input_interleaved = c.layout == kLoadInterleavedVec;
    p.alpha_re = 1;
    p.alpha_im = 0;
    p.beta_re = 0;
    p.beta_im = 0;
    p.have_alpha = 0;
    p.have_beta = 0;
    if (std::strstr(c.name, "192x256") != nullptr) {
      if (!wide_tiles_apply(p)) {
        std::printf("%-44s (not applicable to this shape)\n", c.name);
        continue;
      }
    }
    // whole tiles: at least as large as the planar and interleaved layouts
    const unsigned k_tiles_planar = (K + kpt - 1) / kpt;
    const size_t x_bytes = (size_t)B * p.x_tiles * k_tiles_planar * kTileBytes;
    const size_t y_bytes = (size_t)B * p.y_tiles * k_tiles_planar * kTileBytes;
    const size_t c_bytes = (size_t)B * 2 * M * N * 4;
    void *dx, *dy, *dc;
    CHECK(hipMalloc(&dx, x_bytes));
    CHECK(hipMalloc(&dy, y_bytes));
    CHECK(hipMalloc(&dc, c_bytes));
    if (fill == "zero") {
      CHECK(hipMemset(dx, 0, x_bytes));
      CHECK(hipMemset(dy, 0, y_bytes));
    } else if (fill == "legacy") {
      fill_legacy(dx, x_bytes, c.type_in);
      fill_legacy(dy, y_bytes, c.type_in);
    } else {
      // elements of one plane: of a tile (tiled layout) or of one batch's operand plane
      const size_t elem_bits = (size_t)bits_of(c.type_in);
      const size_t tile_plane = (size_t)kTilePlaneBytes * 8 / elem_bits;
      const size_t xp = c.layout == kLoadTiled ? tile_plane : (size_t)N * K;
      const size_t yp = c.layout == kLoadTiled ? tile_plane : (size_t)M * K;
      fill_baseline(dx, x_bytes, c.type_in, c.layout, xp, false, 1);
      fill_baseline(dy, y_bytes, c.type_in, c.layout, yp, beamformer && c.type_in != kInt1, 2);
      CHECK(hipDeviceSynchronize());
    }
    p.x = dx;
    p.y = dy;
    p.c = dc;
    // The part runs under a power limit whose controller needs about 30 ms of
    // continuous load to settle: warm up for 60 ms, then time 100 ms.
    CHECK(c.launch(p, 0));
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0));
    CHECK(c.launch(p, 0));
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float one = 0;
    CHECK(hipEventElapsedTime(&one, e0, e1));
    const int warm = std::max(3, (int)(60.f / one)), iters = std::max(5, (int)(100.f / one));
    for (int i = 0; i < warm; ++i) CHECK(c.launch(p, 0));
    CHECK(hipEventRecord(e0));
    for (int i = 0; i < iters; ++i) CHECK(c.launch(p, 0));
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float best;
    CHECK(hipEventElapsedTime(&best, e0, e1));
    best /= iters;
    const double tflops = 8.0 * B * M * N * K / (best * 1e-3) / 1e12;
    // a hash of C's bits: configurations that multiply the same operands in the same
    // layout must agree
    std::vector<unsigned> hc(c_bytes / 4);
    CHECK(hipMemcpy(hc.data(), dc, c_bytes, hipMemcpyDeviceToHost));
    unsigned long long hash = 1469598103934665603ull;
    for (unsigned v : hc) hash = (hash ^ v) * 1099511628211ull;
    std::printf("%-44s %10.4f %12.1f %9.1f%%   C %016llx\n", c.name, best, tflops,
                100 * tflops / (c.peak > 0 ? c.peak : peak_of(c.type_in)), hash);
    std::fflush(stdout);
    CHECK(hipFree(dx));
    CHECK(hipFree(dy));
    CHECK(hipFree(dc));
  }
  return 0;
}
