// Transpose into the tiled layout of the optimised GEMM:
//   in  [B][2][M][N] (planar) or [B][M][N][2] (interleaved)
//   out [B][Mp/Mc][Np/Nc][2][Mc][Nc], zero where m >= M or n >= N.
// Stands in for the reference's transpose kernel
// (kernels/transpose_kernel.cu:50-82), which moves one element pair per
// thread. This one is bandwidth-shaped: a thread moves 16-byte vectors (both
// planes of 2 rows), lanes of a wave run along N across tile boundaries, so
// loads are contiguous runs of 128 or 256 bytes per row and stores are
// contiguous runs of rows inside each output tile. Both sides are streamed once, so the
// accesses carry the non-temporal hint (measured +5 to +10 % on this part).
// A scalar kernel covers shapes whose rows are not whole 16-byte vectors.
#include "common.h"

namespace ccglib_amd {
namespace {

typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned short ushort8_t __attribute__((ext_vector_type(8)));
typedef unsigned char uchar16_t __attribute__((ext_vector_type(16)));

struct TransposeArgs {
  const char *in;
  char *out;
  size_t m, n;              // logical sizes in elements
  size_t m_chunk, n_chunk;  // tile sizes in elements
  size_t m_tiles, n_tiles;
  size_t n_vecs_padded;     // 16-byte vectors per padded row
  size_t vecs_per_tile_row;
};

// De-interleaves two 16-byte vectors holding (re, im) pairs.
template <int EB>
__device__ __forceinline__ void deinterleave(uint4_t a, uint4_t b, uint4_t &re, uint4_t &im) {
  if constexpr (EB == 4) {
    re = uint4_t{a[0], a[2], b[0], b[2]};
    im = uint4_t{a[1], a[3], b[1], b[3]};
  } else if constexpr (EB == 2) {
    const ushort8_t x = __builtin_bit_cast(ushort8_t, a), y = __builtin_bit_cast(ushort8_t, b);
    re = __builtin_bit_cast(uint4_t, __builtin_shufflevector(x, y, 0, 2, 4, 6, 8, 10, 12, 14));
    im = __builtin_bit_cast(uint4_t, __builtin_shufflevector(x, y, 1, 3, 5, 7, 9, 11, 13, 15));
  } else {
    const uchar16_t x = __builtin_bit_cast(uchar16_t, a), y = __builtin_bit_cast(uchar16_t, b);
    re = __builtin_bit_cast(uint4_t, __builtin_shufflevector(x, y, 0, 2, 4, 6, 8, 10, 12, 14, 16,
                                                             18, 20, 22, 24, 26, 28, 30));
    im = __builtin_bit_cast(uint4_t, __builtin_shufflevector(x, y, 1, 3, 5, 7, 9, 11, 13, 15, 17,
                                                             19, 21, 23, 25, 27, 29, 31));
  }
}

// 16 bytes at an address that is aligned to the element size only (global
// memory takes any alignment on this target).
typedef uint4_t uint4_unaligned_t __attribute__((aligned(1)));

template <int EB> struct ElementOf;
template <> struct ElementOf<1> { typedef unsigned char type; };
template <> struct ElementOf<2> { typedef unsigned short type; };
template <> struct ElementOf<4> { typedef unsigned type; };

// The output vector of elements n0 .. n0 + 16/EB - 1 of one input row that ends
// at element n (n0 < n): whole vectors with wide loads from wherever they lie,
// the vector that holds the end of the row element by element, zero beyond.
// p points at element n0 (planar) or at pair n0 (interleaved).
template <int EB, bool INTERLEAVED>
__device__ __forceinline__ void load_ragged(const char *p, size_t plane_stride_bytes, size_t n0,
                                            size_t n, uint4_t &re, uint4_t &im) {
  constexpr int V = 16 / EB;
  typedef typename ElementOf<EB>::type T;
  if (n0 + V <= n) {
    if constexpr (!INTERLEAVED) {
      re = *reinterpret_cast<const uint4_unaligned_t *>(p);
      im = *reinterpret_cast<const uint4_unaligned_t *>(p + plane_stride_bytes);
    } else {
      const uint4_t x = *reinterpret_cast<const uint4_unaligned_t *>(p);
      const uint4_t y = *reinterpret_cast<const uint4_unaligned_t *>(p + 16);
      deinterleave<EB>(x, y, re, im);
    }
    return;
  }
  struct Vec { T e[V]; };
  Vec r = {}, i = {};
  const T *q = reinterpret_cast<const T *>(p);
  const T *qi = reinterpret_cast<const T *>(p + plane_stride_bytes);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    if (n0 + e < n) {
      r.e[e] = INTERLEAVED ? q[2 * e] : q[e];
      i.e[e] = INTERLEAVED ? q[2 * e + 1] : qi[e];
    }
  }
  re = __builtin_bit_cast(uint4_t, r);
  im = __builtin_bit_cast(uint4_t, i);
}

constexpr int kRowsPerThread = 2;

// grid: (ceil(n_vecs_padded / VPR), ceil(Mp / rows per block) [of both operands], B); block: 256
// threads as VPR vectors x 256 / VPR rows, each thread doing rows r and
// r + 256 / VPR (two rows a thread measured best over the operand shapes of the
// benchmark configurations: one row is as good for 16-bit but slower for 8-bit
// elements, four are 2-7 % slower, eight halve the rate). VPR is 16 (256 bytes
// of a row per block) or, for padded rows that are a multiple of 8 but not of
// 16 vectors, 8: no lanes without work at the end of a row (K = 576 halfs is
// 72 vectors: with 16 a tenth of the threads would idle).
// RAGGED: input rows of any length at any element-aligned address (the output
// tiles still hold whole vectors per row).
// One launch can serve two operands with rows of the same length (the A and B
// of one GEMM): block rows below y_split belong to the first, the others to
// the second, which spares a small operand its own launch, ramp-up and tail.
struct TransposePairArgs {
  TransposeArgs op[2];
  unsigned y_split;
};

template <int EB, bool INTERLEAVED, bool RAGGED, int VPR>
__global__ __launch_bounds__(256) void transpose_vec(const TransposePairArgs pair) {
  constexpr int V = 16 / EB;  // elements per vector
  constexpr int RS = 256 / VPR;   // rows between the two rows of a thread
  const bool second = blockIdx.y >= pair.y_split;
  const TransposeArgs &a = pair.op[second ? 1 : 0];
  const size_t nvec = (size_t)blockIdx.x * VPR + (threadIdx.x % VPR);
  const size_t m_base = (size_t)(blockIdx.y - (second ? pair.y_split : 0u)) * (RS * kRowsPerThread) +
                        (threadIdx.x / VPR);
  const size_t b = blockIdx.z;
  const size_t m_padded = a.m_tiles * a.m_chunk;
  if (nvec >= a.n_vecs_padded) return;
  const size_t n0 = nvec * V;
  const bool n_ok = n0 < a.n;  // (not RAGGED: rows are whole vectors, inside or outside)
  const size_t nt = nvec / a.vecs_per_tile_row, v = nvec % a.vecs_per_tile_row;
  const size_t plane_bytes = a.m_chunk * a.n_chunk * EB;

  uint4_t re[kRowsPerThread], im[kRowsPerThread];
#pragma unroll
  for (int i = 0; i < kRowsPerThread; ++i) {
    const size_t m = m_base + RS * i;
    re[i] = uint4_t{0, 0, 0, 0};
    im[i] = uint4_t{0, 0, 0, 0};
    if (m < a.m && n_ok) {
      if constexpr (RAGGED) {
        const char *p = INTERLEAVED ? a.in + ((b * a.m + m) * a.n + n0) * 2 * EB
                                    : a.in + (((b * 2) * a.m + m) * a.n + n0) * EB;
        load_ragged<EB, INTERLEAVED>(p, a.m * a.n * EB, n0, a.n, re[i], im[i]);
      } else if constexpr (!INTERLEAVED) {
        const char *p = a.in + (((b * 2) * a.m + m) * a.n + n0) * EB;
        re[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p));
        im[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p + a.m * a.n * EB));
      } else {
        const char *p = a.in + ((b * a.m + m) * a.n + n0) * 2 * EB;
        const uint4_t x = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p));
        const uint4_t y = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p + 16));
        deinterleave<EB>(x, y, re[i], im[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kRowsPerThread; ++i) {
    const size_t m = m_base + RS * i;
    if (m < m_padded) {
      const size_t mt = m / a.m_chunk, mr = m % a.m_chunk;
      char *q = a.out + (((b * a.m_tiles + mt) * a.n_tiles + nt) * 2) * plane_bytes +
                (mr * a.n_chunk) * EB + v * 16;
      __builtin_nontemporal_store(re[i], reinterpret_cast<uint4_t *>(q));
      __builtin_nontemporal_store(im[i], reinterpret_cast<uint4_t *>(q + plane_bytes));
    }
  }
}

// One thread per output element pair; any shape.
template <typename T, bool INTERLEAVED>
__global__ __launch_bounds__(256) void transpose_scalar(const TransposeArgs a, size_t batch) {
  const size_t n_padded = a.n_tiles * a.n_chunk;
  const size_t m_padded = a.m_tiles * a.m_chunk;
  const size_t per_batch = m_padded * n_padded;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_batch * batch) return;
  const size_t b = idx / per_batch;
  const size_t m = (idx % per_batch) / n_padded, n = idx % n_padded;
  const T *in = reinterpret_cast<const T *>(a.in);
  T *out = reinterpret_cast<T *>(a.out);
  T re = 0, im = 0;
  if (m < a.m && n < a.n) {
    if constexpr (!INTERLEAVED) {
      re = in[((b * 2) * a.m + m) * a.n + n];
      im = in[((b * 2 + 1) * a.m + m) * a.n + n];
    } else {
      re = in[((b * a.m + m) * a.n + n) * 2];
      im = in[((b * a.m + m) * a.n + n) * 2 + 1];
    }
  }
  const size_t mt = m / a.m_chunk, mr = m % a.m_chunk;
  const size_t nt = n / a.n_chunk, nr = n % a.n_chunk;
  const size_t plane = a.m_chunk * a.n_chunk;
  const size_t o = (((b * a.m_tiles + mt) * a.n_tiles + nt) * 2) * plane + mr * a.n_chunk + nr;
  out[o] = re;
  out[o + plane] = im;
}

// What a launch of the vector kernel needs to know about one operand.
template <int EB> struct VecPlan {
  TransposeArgs a;
  bool out_vec_ok, in_vec_ok, narrow;
  size_t y_blocks;
};

template <int EB> VecPlan<EB> plan_operand(const TransposeParams &p) {
  VecPlan<EB> v;
  TransposeArgs &a = v.a;
  a.in = static_cast<const char *>(p.in);
  a.out = static_cast<char *>(p.out);
  a.m = p.m;
  a.n = p.n;
  a.m_chunk = p.m_chunk;
  a.n_chunk = p.n_chunk;
  a.m_tiles = ceil_div(p.m, p.m_chunk);
  a.n_tiles = ceil_div(p.n, p.n_chunk);
  constexpr size_t V = 16 / EB;
  const size_t m_padded = a.m_tiles * a.m_chunk, n_padded = a.n_tiles * a.n_chunk;
  // whole vectors per output tile row; the input may be ragged
  v.narrow = (n_padded / V) % 16 != 0 && (n_padded / V) % 8 == 0;
  const size_t rows_per_block = 256 / (v.narrow ? 8 : 16) * kRowsPerThread;
  v.y_blocks = ceil_div(m_padded, rows_per_block);
  v.out_vec_ok = (p.n_chunk % V == 0) && ((uintptr_t)p.out % 16 == 0) &&
                 ((uintptr_t)p.in % EB == 0) && p.batch <= 65535 && v.y_blocks <= 65535;
  v.in_vec_ok = (p.n % V == 0) && ((uintptr_t)p.in % 16 == 0);
  a.n_vecs_padded = v.out_vec_ok ? n_padded / V : 0;
  a.vecs_per_tile_row = v.out_vec_ok ? p.n_chunk / V : 0;
  return v;
}

// p1 == nullptr: one operand. Otherwise the caller has checked that both take
// the same kernel (same batch, row length, tile width, layout and raggedness).
template <int EB>
hipError_t launch_vec(const TransposeParams &p0, const VecPlan<EB> &v0, const VecPlan<EB> *v1,
                      hipStream_t stream) {
  TransposePairArgs pair;
  pair.op[0] = v0.a;
  pair.op[1] = v1 ? v1->a : v0.a;
  pair.y_split = (unsigned)v0.y_blocks;
  const size_t vpr = v0.narrow ? 8 : 16;
  const dim3 grid((unsigned)ceil_div(v0.a.n_vecs_padded, vpr),
                  (unsigned)(v0.y_blocks + (v1 ? v1->y_blocks : 0)), (unsigned)p0.batch);
  auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, pair); };
  const bool narrow = v0.narrow;
  if (p0.interleaved) {
    if (v0.in_vec_ok) {
      narrow ? launch(transpose_vec<EB, true, false, 8>) : launch(transpose_vec<EB, true, false, 16>);
    } else {
      narrow ? launch(transpose_vec<EB, true, true, 8>) : launch(transpose_vec<EB, true, true, 16>);
    }
  } else {
    if (v0.in_vec_ok) {
      narrow ? launch(transpose_vec<EB, false, false, 8>) : launch(transpose_vec<EB, false, false, 16>);
    } else {
      narrow ? launch(transpose_vec<EB, false, true, 8>) : launch(transpose_vec<EB, false, true, 16>);
    }
  }
  return hipGetLastError();
}

template <int EB, typename T>
hipError_t launch_width(const TransposeParams &p, hipStream_t stream) {
  const VecPlan<EB> v = plan_operand<EB>(p);
  const TransposeArgs &a = v.a;
  const size_t m_padded = a.m_tiles * a.m_chunk, n_padded = a.n_tiles * a.n_chunk;
  if (p.batch == 0 || m_padded == 0 || n_padded == 0) return hipSuccess;
  if (v.out_vec_ok) return launch_vec<EB>(p, v, nullptr, stream);
  const size_t total = p.batch * m_padded * n_padded;
  const size_t blocks = ceil_div(total, 256);
  if (blocks > 0x7fffffffu) return hipErrorInvalidValue;
  if (p.interleaved) {
    hipLaunchKernelGGL((transpose_scalar<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream, a,
                       p.batch);
  } else {
    hipLaunchKernelGGL((transpose_scalar<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       a, p.batch);
  }
  return hipGetLastError();
}

template <int EB>
bool try_launch_pair(const TransposeParams &p0, const TransposeParams &p1, hipStream_t stream,
                     hipError_t &result) {
  if (p0.batch != p1.batch || p0.n != p1.n || p0.n_chunk != p1.n_chunk ||
      p0.interleaved != p1.interleaved || p0.batch == 0 || p0.n == 0 || p0.m == 0 || p1.m == 0) {
    return false;
  }
  // One launch pays when one operand is small (it is spared its own launch, ramp-up
  // and tail: B=64, 512 and 4096 rows of 576 halfs take 0.231 ms together against
  // 0.234 ms one after the other). Two operands of similar size are 1-3 % faster as
  // two launches (fp8 B=16 4096 x 8192 twice: 0.753 against 0.775 ms; 1-bit words
  // B=32 1024 x 2048 twice: 0.376 against 0.384 ms).
  const size_t small = p0.m < p1.m ? p0.m : p1.m, large = p0.m < p1.m ? p1.m : p0.m;
  if (small * 4 > large) return false;
  const VecPlan<EB> v0 = plan_operand<EB>(p0), v1 = plan_operand<EB>(p1);
  if (!v0.out_vec_ok || !v1.out_vec_ok || v0.in_vec_ok != v1.in_vec_ok ||
      v0.y_blocks + v1.y_blocks > 65535) {
    return false;
  }
  result = launch_vec<EB>(p0, v0, &v1, stream);
  return true;
}

}  // namespace

hipError_t launch_transpose(const TransposeParams &p, hipStream_t stream) {
  switch (p.elem_bytes) {
    case 1: return launch_width<1, unsigned char>(p, stream);
    case 2: return launch_width<2, unsigned short>(p, stream);
    case 4: return launch_width<4, unsigned>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

// Both operands of one GEMM. One launch when they take the same vector kernel and
// one of them is at most a quarter of the other, otherwise one launch each.
hipError_t launch_transpose_pair(const TransposeParams &p0, const TransposeParams &p1,
                                 hipStream_t stream) {
  hipError_t e = hipSuccess;
  bool done = false;
  if (p0.elem_bytes == p1.elem_bytes) {
    switch (p0.elem_bytes) {
      case 1: done = try_launch_pair<1>(p0, p1, stream, e); break;
      case 2: done = try_launch_pair<2>(p0, p1, stream, e); break;
      case 4: done = try_launch_pair<4>(p0, p1, stream, e); break;
      default: return hipErrorInvalidValue;
    }
  }
  if (done) return e;
  e = launch_transpose(p0, stream);
  return e == hipSuccess ? launch_transpose(p1, stream) : e;
}

}  // namespace ccglib_amd
