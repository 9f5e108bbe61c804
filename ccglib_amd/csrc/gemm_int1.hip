// 1-bit complex GEMM: XOR + population count on the vector ALU.
//
// Stands in for the reference's int1 wmma_complex_gemm_basic / _opt
// (kernels/gemm_kernel_int1.cu:64-196, :198-356), which exist for NVIDIA's
// binary tensor-core op only; gfx950 has no 1-bit matrix instruction, so the
// dot products are built from v_xor_b32 and v_bcnt_u32_b32 (whose add operand
// does the accumulation). With bit 1 = +1 and bit 0 = -1 a product is an XOR
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

}  // namespace

hipError_t launch_gemm_int1(const GemmParams &p, hipStream_t stream) {
  if (p.type_in != kInt1 || p.type_out != kInt32) return hipErrorInvalidValue;
  if (p.variant == kOpt) return launch_loader<kLoadTiled>(p, stream);
  const size_t k_bytes = ceil_div(p.k, 32) * 4;
  const bool aligned = (k_bytes >= 16) && (k_bytes % 16 == 0) && ((uintptr_t)p.x % 16 == 0) &&
                       ((uintptr_t)p.y % 16 == 0);
  return aligned ? launch_loader<kLoadPlanarVec>(p, stream)
                 : launch_loader<kLoadPlanarElem>(p, stream);
}

}  // namespace ccglib_amd
