// 1-bit complex GEMM.
//
// Stands in for the reference's int1 wmma_complex_gemm_basic / _opt
// (kernels/gemm_kernel_int1.cu:64-196, :198-356), which exist for NVIDIA's
// binary tensor-core op only; gfx950 has no 1-bit matrix instruction. This file
// holds the launcher, which picks one of two ways to the same integers:
//  * the fp4 MFMA kernel on the packed words as they are (in the file of the MFMA
//    kernels; tiled operands and planar rows of whole aligned 16-byte chunks),
//  * XOR + population count on the vector ALU (complex_gemm_int1 below; the
//    fallback for everything else),
// and the kernel that packs one byte per sample straight into 1-bit tiles for
// the pipeline.
//
// The popcount kernel builds the dot products from v_xor_b32 and
// v_bcnt_u32_b32 (whose add operand does the accumulation). With bit 1 = +1 and bit 0 = -1 a product is an XOR
// and a sum a popcount (src/reference/GEMM.cpp:131-200):
//   pop_re = popc(xr ^ yr) + popc(xi ^ ~yi)
//   pop_im = popc(xr ^ yi) + popc(xi ^ yr)
//   re = 2 * (Kp - pop_re),  im = 2 * (Kp - pad - pop_im)
// where Kp is the K the kernel actually walks (whole 512-sample tiles, zero
// filled) and pad = Kp - K.
//
// One block of 256 threads owns a 128 x 128 patch of C; each thread keeps an
// 8 x 8 register tile (x = tx + 16 i, y = ty + 16 j), so every LDS read of a
// row is reused 8 times. Operand tiles have the same
// 128-row x 64-byte geometry as the floating-point kernels and go through
// the same global -> registers -> LDS double buffer.
#include <algorithm>

#include "gemm_device.h"

namespace ccglib_amd {
namespace {

template <int LOADER>
__global__ __launch_bounds__(256, 2) void complex_gemm_int1(const KernelArgs args) {
  constexpr int BX = 128, BY = 128, NTHREADS = 256;
  constexpr int X_BYTES = 2 * BX * kTileRowBytes;
  constexpr int STAGE_BYTES = X_BYTES + 2 * BY * kTileRowBytes;
  constexpr int CX = 2 * BX * 4 / NTHREADS, CY = 2 * BY * 4 / NTHREADS;

  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE_BYTES];

  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;

  const TileCoord tc = tile_coord(args, blockIdx.x);
  const unsigned b = tc.b, block_x = tc.block_x, block_y = tc.block_y;
  OperandView xv{args.x + (size_t)b * args.x_batch_bytes, args.nx, args.x_tiles, block_x * BX};
  OperandView yv{args.y + (size_t)b * args.y_batch_bytes, args.ny, args.y_tiles, block_y * BY};
  const unsigned k_tiles = args.k_tiles, k_bytes = args.k_bytes;

  int4_t xs[CX], ys[CY];
  auto fetch = [&](unsigned kt) {
#pragma unroll
    for (int i = 0; i < CX; ++i) {
      const int g = tid + i * NTHREADS;
      xs[i] = load_chunk<4, LOADER>(xv, kt, k_tiles, k_bytes, g / (BX * 4), (g / 4) % BX, g % 4);
    }
#pragma unroll
    for (int i = 0; i < CY; ++i) {
      const int g = tid + i * NTHREADS;
      ys[i] = load_chunk<4, LOADER>(yv, kt, k_tiles, k_bytes, g / (BY * 4), (g / 4) % BY, g % 4);
    }
  };
  auto stash = [&](int stage) {
    char *s = lds + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < CX; ++i) {
      const int g = tid + i * NTHREADS;
      *reinterpret_cast<int4_t *>(s + (g / (BX * 4)) * BX * kTileRowBytes +
                                  swizzled_row_offset((g / 4) % BX, g % 4)) = xs[i];
    }
#pragma unroll
    for (int i = 0; i < CY; ++i) {
      const int g = tid + i * NTHREADS;
      *reinterpret_cast<int4_t *>(s + X_BYTES + (g / (BY * 4)) * BY * kTileRowBytes +
                                  swizzled_row_offset((g / 4) % BY, g % 4)) = ys[i];
    }
  };

  int pop_re[8][8], pop_im[8][8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pop_re[j][i] = 0;
      pop_im[j][i] = 0;
    }
  }

  typedef int int2_t __attribute__((ext_vector_type(2)));
  auto compute = [&](int stage) {
    const char *s = lds + stage * STAGE_BYTES;
    // 8 bytes (64 samples) of every row at a time keeps the register tile
    // within the budget of two waves per SIMD
#pragma unroll 1
    for (int h = 0; h < 8; ++h) {
      const int c = h >> 1, sub = (h & 1) * 8;
      int2_t xr[8], xi[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const char *p = s + swizzled_row_offset(tx + 16 * i, c) + sub;
        xr[i] = *reinterpret_cast<const int2_t *>(p);
        xi[i] = *reinterpret_cast<const int2_t *>(p + BX * kTileRowBytes);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const char *p = s + X_BYTES + swizzled_row_offset(ty + 16 * j, c) + sub;
        const int2_t yr = *reinterpret_cast<const int2_t *>(p);
        const int2_t yi = *reinterpret_cast<const int2_t *>(p + BY * kTileRowBytes);
        const int2_t nyi = ~yi;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
          for (int w = 0; w < 2; ++w) {
            pop_re[j][i] += __builtin_popcount((unsigned)(xr[i][w] ^ yr[w]));
            pop_re[j][i] += __builtin_popcount((unsigned)(xi[i][w] ^ nyi[w]));
            pop_im[j][i] += __builtin_popcount((unsigned)(xr[i][w] ^ yi[w]));
            pop_im[j][i] += __builtin_popcount((unsigned)(xi[i][w] ^ yr[w]));
          }
        }
      }
    }
  };

  fetch(0);
  stash(0);
  if (k_tiles > 1) fetch(1);
  __syncthreads();
  for (unsigned s = 0; s < k_tiles; ++s) {
    const int cur = s & 1;
    if (s + 1 < k_tiles) stash(cur ^ 1);
    if (s + 2 < k_tiles) fetch(s + 2);
    compute(cur);
    __syncthreads();
  }

  // ---- epilogue (integer arithmetic wraps modulo 2^32) ----------------------
  const unsigned nx = args.nx, ny = args.ny;
  const unsigned k_walked = k_tiles * (kTileRowBytes * 8);
  const unsigned pad = k_walked - args.k;
  const unsigned ar = (unsigned)(int)args.alpha_re, ai = (unsigned)(int)args.alpha_im;
  const unsigned br = (unsigned)(int)args.beta_re, bi = (unsigned)(int)args.beta_im;
  const bool have_beta = args.have_beta;
  unsigned *cbase = reinterpret_cast<unsigned *>(args.c) + (size_t)b * 2 * nx * ny;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const unsigned y = block_y * BY + ty + 16 * j;
    if (y >= ny) continue;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const unsigned x = block_x * BX + tx + 16 * i;
      if (x >= nx) continue;
      const unsigned s_re = 2u * (k_walked - (unsigned)pop_re[j][i]);
      const unsigned s_im = 2u * (k_walked - pad - (unsigned)pop_im[j][i]);
      unsigned re = ar * s_re - ai * s_im;
      unsigned im = ai * s_re + ar * s_im;
      unsigned *pr, *pi;
      if (!args.c_interleaved) {
        pr = cbase + (size_t)y * nx + x;
        pi = pr + (size_t)nx * ny;
      } else {
        pr = cbase + ((size_t)y * nx + x) * 2;
        pi = pr + 1;
      }
      if (have_beta) {
        const unsigned cr = *pr, ci = *pi;
        re += br * cr - bi * ci;
        im += bi * cr + br * ci;
      }
      *pr = re;
      *pi = im;
    }
  }
}

template <int LOADER>
hipError_t launch_loader(const GemmParams &p, hipStream_t stream) {
  const KernelArgs a = make_kernel_args(p, 128, 128);
  const size_t total = (size_t)a.blocks_x * a.blocks_y * p.batch;
  if (total == 0) return hipSuccess;
  if (total > 0x7fffffffu) return hipErrorInvalidValue;
  hipLaunchKernelGGL(complex_gemm_int1<LOADER>, dim3((unsigned)total), dim3(256), 0, stream, a);
  return hipGetLastError();
}

typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

// One byte per sample straight into the tiled 1-bit layout that the opt variant
// reads ([batch][rows/128][K/512][2][128 rows][64 bytes]; rows and samples past
// the end are zero bits): Packing and Transpose of the reference's pipeline
// (src/pipeline/Pipeline.cpp:111-121) in one pass without the packed intermediate.
// A wave takes 16 rows of a tile, two at a time: lane = (row of the two, 16-byte
// piece p of the 512 samples of a tile row), so that a load instruction reads two
// runs of 512 contiguous bytes; a thread has eight loads in flight. A thread's
// 16 bytes are half an output word: of every two loads, lane pairs exchange one
// half, after which the even lane holds word p / 2 of the first load's row and
// the odd lane that of the second's, so that a store instruction of a wave
// writes four whole tile rows, 256 contiguous bytes.
// Inside a half word the 16 samples are stored transposed (sample 4 d + j at bit
// 4 j + d), which saves the bit gathering per 4 bytes: both operands of the GEMM
// are packed by this kernel, and a sum over K does not see a permutation of K
// that is the same in X and Y.
__device__ __forceinline__ unsigned nonzero_bits_transposed(uint4_t v) {
  unsigned c = 0;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned nz = (((v[d] & 0x7f7f7f7fu) + 0x7f7f7f7fu) | v[d]) & 0x80808080u;
    c |= nz >> (7 - d);
  }
  // byte j of c holds samples j, 4 + j, 8 + j, 12 + j in its low four bits
  const unsigned t = c | (c >> 4);
  return (t & 0xffu) | ((t >> 8) & 0xff00u);
}

constexpr int kPackLoads = 4;   // loads in flight per thread (two rows each per wave)
template <bool VEC>
__global__ __launch_bounds__(256) void pack_bytes_to_tiles(const unsigned char *__restrict__ src,
                                                           char *__restrict__ dst, unsigned rows,
                                                           unsigned row_tiles, unsigned k,
                                                           unsigned k1_tiles) {
  // blockIdx: x = four K tiles of 512 samples (one per wave: a block reads 2 KiB
  // contiguous of each of its rows), y = block of 2 kPackLoads rows, z = (batch, plane)
  const unsigned lane = threadIdx.x & 63;
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const unsigned p = lane & 31;                 // 16-byte piece of the 512 samples of a tile row
  constexpr unsigned RPW = 2 * kPackLoads, WPT = kTileRows / RPW;   // rows per wave, waves per tile
  const unsigned rt = blockIdx.y / WPT;
  const size_t b = blockIdx.z >> 1;
  const unsigned plane = blockIdx.z & 1;
  const unsigned kt = blockIdx.x * 4 + wave;
  if (kt >= k1_tiles) return;
  const unsigned k0 = kt * 512 + p * 16;
  const unsigned row0_in_tile = (blockIdx.y % WPT) * RPW + (lane >> 5);   // + 2 i
  const unsigned block_row0 = rt * kTileRows + (blockIdx.y % WPT) * RPW;
  unsigned half[kPackLoads];
  // the same for all threads of a wave: all its rows and all 512 samples exist
  if (VEC && block_row0 + RPW <= rows && kt * 512 + 512 <= k) {
    const unsigned char *p0 =
        src + ((b * 2 + plane) * rows + rt * kTileRows + row0_in_tile) * (size_t)k + k0;
    uint4_t v[kPackLoads];
#pragma unroll
    for (int i = 0; i < kPackLoads; ++i) {
      v[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p0 + (size_t)(2 * i) * k));
    }
#pragma unroll
    for (int i = 0; i < kPackLoads; ++i) half[i] = nonzero_bits_transposed(v[i]);
  } else {
#pragma unroll
    for (int i = 0; i < kPackLoads; ++i) {
      const unsigned r = rt * kTileRows + row0_in_tile + 2 * i;
      const unsigned char *row_ptr = src + ((b * 2 + plane) * rows + (r < rows ? r : 0)) * (size_t)k;
      const unsigned n = (r < rows && k0 < k) ? (k - k0 < 16 ? k - k0 : 16) : 0;
      unsigned bits = 0;
      for (unsigned e = 0; e < n; ++e) {
        bits |= (row_ptr[k0 + e] != 0 ? 1u : 0u) << (4 * (e & 3) + (e >> 2));
      }
      half[i] = bits;
    }
  }
  // Lane pairs hold the two halves of word p / 2 of each row: of every two rows
  // the even lane takes the word of the first and the odd lane that of the second.
  const bool odd = (lane & 1) != 0;
  char *out = dst + ((b * row_tiles + rt) * k1_tiles + kt) * kTileBytes +
              plane * kTilePlaneBytes + (row0_in_tile + (odd ? 2 : 0)) * kTileRowBytes + 4 * (p >> 1);
#pragma unroll
  for (int m = 0; m < kPackLoads / 2; ++m) {
    const unsigned give = odd ? half[2 * m] : half[2 * m + 1];
    const unsigned got = (unsigned)__builtin_amdgcn_update_dpp(0, (int)give, 0xB1, 0xf, 0xf, false);
    const unsigned word = odd ? (got | (half[2 * m + 1] << 16)) : (half[2 * m] | (got << 16));
    *reinterpret_cast<unsigned *>(out + 4 * m * kTileRowBytes) = word;
  }
}

// Largest K for which every partial sum (at most 2 K in magnitude) is exact in fp32.
constexpr unsigned kMaxMfmaK = 1u << 22;

// The packed words as they are: tiled operands always (16-byte aligned, which
// the caller has checked), planar rows when they are whole aligned 16-byte
// chunks (K a multiple of 128).
bool direct_ok(const GemmParams &p) {
  if (!p.int1_direct || p.k == 0 || p.input_interleaved) return false;
  if (((uintptr_t)p.x | (uintptr_t)p.y) % 16 != 0) return false;
  if (p.variant == kOpt) return true;
  const size_t k_bytes = ceil_div(p.k, 32) * 4;
  return k_bytes % 16 == 0;
}

hipError_t launch_int1_on_mfma(const GemmParams &p, hipStream_t stream, bool *done) {
  *done = false;
  if (direct_ok(p)) {
    *done = true;
    if (p.k <= kMaxMfmaK) return launch_gemm_mfma(p, stream);
    // A longer K in pieces whose sums stay exact in fp32, each piece added to C
    // by the integer epilogue: C = alpha S1 + beta C, then C += alpha S2, ...
    // (whole tiles per piece; the operands' rows and row tiles keep the distances
    // of the whole K)
    const unsigned tiles_per_piece = kMaxMfmaK / 512;
    for (unsigned t0 = 0; t0 < p.k_tiles; t0 += tiles_per_piece) {
      GemmParams q = p;
      q.k_in_memory = p.k;
      q.k_tiles = std::min(tiles_per_piece, p.k_tiles - t0);
      q.k = (t0 + q.k_tiles == p.k_tiles) ? p.k - t0 * 512 : q.k_tiles * 512;
      const size_t offset = p.variant == kOpt ? (size_t)t0 * kTileBytes : (size_t)t0 * kTileRowBytes;
      q.x = static_cast<const char *>(p.x) + offset;
      q.y = static_cast<const char *>(p.y) + offset;
      if (t0 > 0) {
        q.beta_re = 1.f;
        q.beta_im = 0.f;
        q.have_beta = 1;
      }
      if (hipError_t e = launch_gemm_mfma(q, stream)) return e;
    }
    return hipSuccess;
  }
  return hipSuccess;   // not done: the caller runs the vector-ALU kernel
}

// The same for interleaved input ([batch][rows][K][2] bytes, (re, im) pairs): a
// wave takes eight rows of one K tile, a whole row of 512 samples (1 KiB) per
// load instruction, eight loads in flight. A lane's 16 bytes are eight pairs:
// eight real and eight imaginary bits, a quarter word of each plane; the four
// lanes of a quad exchange theirs (three DPP moves) and the first two of them
// store the real and the imaginary word, so a store instruction of a wave
// writes one 64-byte tile row in each plane. Samples keep their order here
// (sample k of a row's tile is bit k % 32 of word k / 32): both operands of a
// pipeline have the same layout and are packed by the same kernel.
__device__ __forceinline__ unsigned nonzero_nibble(unsigned x) {
  const unsigned nz = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
  return (((nz >> 7) * 0x00204081u) >> 21) & 0xfu;
}

// 8 (re, im) byte pairs -> real bits in bits 0-7, imaginary bits in bits 8-15
__device__ __forceinline__ unsigned pair_bits(uint4_t v) {
  const unsigned re_lo = __builtin_amdgcn_perm(v[1], v[0], 0x06040200u);
  const unsigned re_hi = __builtin_amdgcn_perm(v[3], v[2], 0x06040200u);
  const unsigned im_lo = __builtin_amdgcn_perm(v[1], v[0], 0x07050301u);
  const unsigned im_hi = __builtin_amdgcn_perm(v[3], v[2], 0x07050301u);
  return nonzero_nibble(re_lo) | (nonzero_nibble(re_hi) << 4) | (nonzero_nibble(im_lo) << 8) |
         (nonzero_nibble(im_hi) << 12);
}

constexpr unsigned kPairRowsPerWave = 8;
template <bool VEC>
__global__ __launch_bounds__(256) void pack_pairs_to_tiles(const unsigned char *__restrict__ src,
                                                           char *__restrict__ dst, unsigned rows,
                                                           unsigned row_tiles, unsigned k,
                                                           unsigned k1_tiles) {
  // blockIdx: x = four K tiles of 512 samples (one per wave: a block reads 4 KiB
  // contiguous of each of its rows), y = block of eight rows, z = batch
  const unsigned lane = threadIdx.x & 63;
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr unsigned RPW = kPairRowsPerWave, WPT = kTileRows / RPW;
  const unsigned rt = blockIdx.y / WPT;
  const unsigned row0_in_tile = (blockIdx.y % WPT) * RPW;
  const size_t b = blockIdx.z;
  const unsigned kt = blockIdx.x * 4 + wave;
  if (kt >= k1_tiles) return;
  const unsigned k0 = kt * 512 + lane * 8;      // first of this lane's eight samples
  unsigned bits[RPW];
  // the same for all threads of a wave: all its rows and all 512 samples exist
  if (VEC && rt * kTileRows + row0_in_tile + RPW <= rows && kt * 512 + 512 <= k) {
    const unsigned char *p0 = src + ((b * rows + rt * kTileRows + row0_in_tile) * (size_t)k + k0) * 2;
    uint4_t v[RPW];
#pragma unroll
    for (unsigned i = 0; i < RPW; ++i) {
      v[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p0 + (size_t)i * k * 2));
    }
#pragma unroll
    for (unsigned i = 0; i < RPW; ++i) bits[i] = pair_bits(v[i]);
  } else {
#pragma unroll
    for (unsigned i = 0; i < RPW; ++i) {
      const unsigned r = rt * kTileRows + row0_in_tile + i;
      const unsigned char *row_ptr = src + (b * rows + (r < rows ? r : 0)) * (size_t)k * 2;
      const unsigned n = (r < rows && k0 < k) ? (k - k0 < 8 ? k - k0 : 8) : 0;
      unsigned re = 0, im = 0;
      for (unsigned e = 0; e < n; ++e) {
        re |= (row_ptr[2 * (size_t)(k0 + e)] != 0 ? 1u : 0u) << e;
        im |= (row_ptr[2 * (size_t)(k0 + e) + 1] != 0 ? 1u : 0u) << e;
      }
      bits[i] = re | (im << 8);
    }
  }
  // lanes 4 w .. 4 w + 3 hold the four bytes of word w of either plane
  const unsigned plane = lane & 1;
  char *out = dst + ((b * row_tiles + rt) * k1_tiles + kt) * kTileBytes + plane * kTilePlaneBytes +
              row0_in_tile * kTileRowBytes + 4 * (lane >> 2);
#pragma unroll
  for (unsigned i = 0; i < RPW; ++i) {
    const int mine = (int)bits[i];
    const unsigned q0 = (unsigned)__builtin_amdgcn_update_dpp(0, mine, 0x00, 0xf, 0xf, false);
    const unsigned q1 = (unsigned)__builtin_amdgcn_update_dpp(0, mine, 0x55, 0xf, 0xf, false);
    const unsigned q2 = (unsigned)__builtin_amdgcn_update_dpp(0, mine, 0xAA, 0xf, 0xf, false);
    const unsigned q3 = (unsigned)__builtin_amdgcn_update_dpp(0, mine, 0xFF, 0xf, 0xf, false);
    const unsigned sh = plane * 8;
    const unsigned word = ((q0 >> sh) & 0xffu) | (((q1 >> sh) & 0xffu) << 8) |
                          (((q2 >> sh) & 0xffu) << 16) | (((q3 >> sh) & 0xffu) << 24);
    if ((lane & 3) < 2) *reinterpret_cast<unsigned *>(out + i * kTileRowBytes) = word;
  }
}

}  // namespace

bool gemm_int1_can_take_bytes(const GemmParams &p) {
  if (!p.int1_direct || !p.workspace || p.k == 0 || p.k > kMaxMfmaK) return false;
  if (p.workspace_bytes < gemm_int1_tiles_bytes(p.batch, p.nx, p.ny, p.k)) return false;
  return p.batch <= 32767 && 16 * (size_t)p.x_tiles <= 65535 && 16 * (size_t)p.y_tiles <= 65535;
}

hipError_t launch_gemm_int1_from_bytes(const GemmParams &p, hipStream_t stream) {
  if (!gemm_int1_can_take_bytes(p)) return hipErrorInvalidValue;
  // pack into the tiled 1-bit layout and multiply the packed words as they are
  const unsigned k1_tiles = (unsigned)ceil_div(p.k, 512);
  const size_t x_bytes = (size_t)p.batch * p.x_tiles * k1_tiles * kTileBytes;
  char *ws_x = static_cast<char *>(p.workspace), *ws_y = ws_x + x_bytes;
  for (int which = 0; which < 2; ++which) {
    const unsigned rows = which ? p.ny : p.nx, row_tiles = which ? p.y_tiles : p.x_tiles;
    const unsigned char *src = static_cast<const unsigned char *>(which ? p.y : p.x);
    if (p.input_interleaved) {
      // (re, im) byte pairs
      const dim3 grid((unsigned)ceil_div(k1_tiles, 4), (kTileRows / kPairRowsPerWave) * row_tiles, p.batch);
      const bool vec = (p.k % 8 == 0) && ((uintptr_t)src % 16 == 0);
      if (vec) {
        hipLaunchKernelGGL(pack_pairs_to_tiles<true>, grid, dim3(256), 0, stream, src,
                           which ? ws_y : ws_x, rows, row_tiles, p.k, k1_tiles);
      } else {
        hipLaunchKernelGGL(pack_pairs_to_tiles<false>, grid, dim3(256), 0, stream, src,
                           which ? ws_y : ws_x, rows, row_tiles, p.k, k1_tiles);
      }
      continue;
    }
    const dim3 grid((unsigned)ceil_div(k1_tiles, 4), (kTileRows / (2 * kPackLoads)) * row_tiles, 2 * p.batch);
    const bool vec = (p.k % 16 == 0) && ((uintptr_t)src % 16 == 0);
    if (vec) {
      hipLaunchKernelGGL(pack_bytes_to_tiles<true>, grid, dim3(256), 0, stream, src,
                         which ? ws_y : ws_x, rows, row_tiles, p.k, k1_tiles);
    } else {
      hipLaunchKernelGGL(pack_bytes_to_tiles<false>, grid, dim3(256), 0, stream, src,
                         which ? ws_y : ws_x, rows, row_tiles, p.k, k1_tiles);
    }
  }
  if (hipError_t e = hipGetLastError()) return e;
  GemmParams q = p;
  q.x = ws_x;
  q.y = ws_y;
  q.variant = kOpt;
  q.input_interleaved = 0;   // (the tiles are planar whatever the bytes were)
  q.k_tiles = k1_tiles;
  return launch_gemm_mfma(q, stream);
}

size_t gemm_int1_tiles_bytes(size_t batch, size_t m, size_t n, size_t k) {
  if (k == 0 || k > kMaxMfmaK) return 0;
  return batch * (ceil_div(m, kTileRows) + ceil_div(n, kTileRows)) * ceil_div(k, 512) * kTileBytes;
}

hipError_t launch_gemm_int1(const GemmParams &p, hipStream_t stream) {
  if (p.type_in != kInt1 || p.type_out != kInt32) return hipErrorInvalidValue;
  bool done = false;
  if (hipError_t e = launch_int1_on_mfma(p, stream, &done)) return e;
  if (done) return hipSuccess;
  if (p.variant == kOpt) return launch_loader<kLoadTiled>(p, stream);
  const size_t k_bytes = ceil_div(p.k, 32) * 4;
  const bool aligned = (k_bytes >= 16) && (k_bytes % 16 == 0) && ((uintptr_t)p.x % 16 == 0) &&
                       ((uintptr_t)p.y % 16 == 0);
  return aligned ? launch_loader<kLoadPlanarVec>(p, stream)
                 : launch_loader<kLoadPlanarElem>(p, stream);
}

}  // namespace ccglib_amd
