// Device-side helpers shared by the complex GEMM kernels: the LDS swizzle, the
// operand loaders for the tiled and the planar layouts, the kernel argument
// block and the workgroup-to-tile mapping.
#ifndef CCGLIB_AMD_GEMM_DEVICE_H_
#define CCGLIB_AMD_GEMM_DEVICE_H_

#include "common.h"

namespace ccglib_amd {

typedef int int4_t __attribute__((ext_vector_type(4)));
// 16 bytes at an address that is aligned to the element size only: one wide
// load (global memory takes any alignment on this target).
typedef int4_t int4_unaligned_t __attribute__((aligned(1)));

enum Loader { kLoadTiled = 0, kLoadPlanarVec = 1, kLoadPlanarElem = 2, kLoadInterleavedVec = 3 };

constexpr int kNumXcd = 8;

// LDS rows are 64 bytes; XORing the 16-byte chunk index with (row >> 1) & 3
// keeps linear 16-byte writes and 16-row column reads free of bank conflicts.
__device__ __forceinline__ int swizzled_row_offset(int row, int chunk) {
  return row * kTileRowBytes + ((chunk ^ ((row >> 1) & 3)) << 4);
}

// Description of one operand as the loader sees it.
struct OperandView {
  const char *base;   // start of this batch's data
  unsigned rows;      // logical rows
  unsigned tiles;     // 128-row tiles (tiled layout)
  unsigned row0;      // first row of this block
};

// Loads the 16-byte chunk (k tile kt, plane, row, chunk c) of an operand.
// Out-of-range chunks read a clamped, valid address and are then replaced by
// zero, so the vector paths issue their loads without branches.
template <int EB, int LOADER>
__device__ __forceinline__ int4_t load_chunk(const OperandView &op, unsigned kt, unsigned k_tiles,
                                             unsigned k_bytes, int plane, int row, int c) {
  const int4_t zero = {0, 0, 0, 0};
  const unsigned grow = op.row0 + row;
  if constexpr (LOADER == kLoadTiled) {
    const unsigned tile = grow / kTileRows;
    const bool valid = (kt < k_tiles) && (tile < op.tiles);
    const unsigned tile_c = tile < op.tiles ? tile : op.tiles - 1;
    const unsigned kt_c = kt < k_tiles ? kt : k_tiles - 1;
    const size_t off = ((size_t)tile_c * k_tiles + kt_c) * kTileBytes + plane * kTilePlaneBytes +
                       (grow % kTileRows) * kTileRowBytes + c * 16;
    const int4_t v = *reinterpret_cast<const int4_t *>(op.base + off);
    return valid ? v : zero;
  } else {
    const unsigned kb = kt * kTileRowBytes + c * 16;
    if constexpr (LOADER == kLoadPlanarVec) {
      const bool valid = (grow < op.rows) && (kb + 16 <= k_bytes);
      const unsigned row_c = grow < op.rows ? grow : op.rows - 1;
      const unsigned kb_c = (kb + 16 <= k_bytes) ? kb : 0;
      const char *p = op.base + ((size_t)plane * op.rows + row_c) * k_bytes + kb_c;
      const int4_t v = *reinterpret_cast<const int4_t *>(p);
      return valid ? v : zero;
    } else {
      int4_t v = zero;
      if (grow >= op.rows || kb >= k_bytes) return v;
      const char *p = op.base + ((size_t)plane * op.rows + grow) * k_bytes + kb;
      if (kb + 16 <= k_bytes) return *reinterpret_cast<const int4_unaligned_t *>(p);
      // the chunk that holds the end of the row, element by element
      if constexpr (EB == 2) {
        const unsigned short *q = reinterpret_cast<const unsigned short *>(p);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          unsigned s = (kb + 2 * e < k_bytes) ? q[e] : 0u;
          v[e / 2] |= (int)(s << (16 * (e % 2)));
        }
      } else if constexpr (EB == 4) {
        const unsigned *q = reinterpret_cast<const unsigned *>(p);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = (kb + 4 * e < k_bytes) ? (int)q[e] : 0;
        }
      } else {
        const unsigned char *q = reinterpret_cast<const unsigned char *>(p);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          unsigned s = (kb + e < k_bytes) ? q[e] : 0u;
          v[e / 4] |= (int)(s << (8 * (e % 4)));
        }
      }
      return v;
    }
  }
}

struct KernelArgs {
  const char *x;
  const char *y;
  char *c;
  unsigned batch, nx, ny, k, k_tiles, k_bytes, x_tiles, y_tiles;
  // distance between consecutive rows of a planar operand (bytes) and between
  // consecutive row tiles of a tiled one (K tiles): those of the whole operand
  // in memory, of which this launch may cover a piece of K
  unsigned row_stride_bytes, k_tile_stride;
  unsigned blocks_x, blocks_y;
  // 192 x 256 kernel only: tiles of 128 columns that follow the blocks_x full ones of a row
  unsigned short_x;
  size_t x_batch_bytes, y_batch_bytes;
  float alpha_re, alpha_im, beta_re, beta_im;
  int have_alpha, have_beta, c_interleaved;
  int c_vector_ok;  // C base is 16-byte aligned: wide stores allowed
  // 1-bit samples on the MFMA: what the zero bits past K add to every imaginary sum
  unsigned im_excess;
};

// alpha * (re + i im), one part at a time. The fused operation is written out, so that
// every kernel that applies alpha rounds alike whatever the compiler would contract,
// and the float result is taken by an empty asm statement: a conversion to fp16 that
// follows is then a rounding of that float (as in the reference, which stores the
// float sum into a half) and cannot be merged into the fused operation, which would
// round the exact sum once.
__device__ __forceinline__ float alpha_times_re(float ar, float ai, float re, float im) {
  float r = __builtin_fmaf(ar, re, -(ai * im));
  asm("" : "+v"(r));
  return r;
}
__device__ __forceinline__ float alpha_times_im(float ar, float ai, float re, float im) {
  float r = __builtin_fmaf(ai, re, ar * im);
  asm("" : "+v"(r));
  return r;
}

// Maps the hardware workgroup id to a logical tile id such that the ids that
// one XCD receives (every 8th workgroup) are consecutive.
__device__ __forceinline__ unsigned xcd_remap(unsigned wg, unsigned total) {
  const unsigned xcd = wg % kNumXcd;
  const unsigned idx = wg / kNumXcd;
  const unsigned q = total / kNumXcd, r = total % kNumXcd;
  const unsigned start = xcd * q + (xcd < r ? xcd : r);
  return start + idx;
}


// n / d for wave-uniform n < 2^20 through the float reciprocal: the product is within 0.2 of
// the true quotient there (23-bit reciprocal, 24-bit product), so truncation is
// off by at most one, which the remainder shows. An integer division by a
// run-time value costs several times as many instructions on this target.
__device__ __forceinline__ unsigned small_div(unsigned n, unsigned d, unsigned *rem) {
  // (n and d are the same in every lane; the float arithmetic runs on the vector
  // ALU, and the result goes back to a scalar register)
  unsigned q = (unsigned)__builtin_amdgcn_readfirstlane(
      (int)(unsigned)((float)n * __builtin_amdgcn_rcpf((float)d)));
  unsigned r = n - q * d;
  if ((int)r < 0) {
    --q;
    r += d;
  } else if (r >= d) {
    ++q;
    r -= d;
  }
  *rem = r;
  return q;
}

// Splits the logical tile id into (batch, block_x, block_y). Inside a batch,
// tiles are walked in groups of 4 block rows with y fastest, so the 32
// consecutive tiles that one XCD works on touch 4 Y panels and 8 X panels.
// (Persistent blocks call this once per C tile, between two K iterations: with
// fewer than 2^20 tiles in all it takes the short divisions above.)
struct TileCoord {
  unsigned b, block_x, block_y;
};
__device__ __forceinline__ TileCoord tile_coord(const KernelArgs &args, unsigned wg) {
  const unsigned per_batch = args.blocks_x * args.blocks_y;
  const unsigned total = per_batch * args.batch;
  const unsigned logical = xcd_remap(wg, total);
  const bool small = total < (1u << 20);
  TileCoord tc;
  unsigned t;
  if (small) {
    tc.b = small_div(logical, per_batch, &t);
  } else {
    tc.b = logical / per_batch;
    t = logical % per_batch;
  }
  constexpr unsigned GROUP = 4;
  const unsigned group_size = GROUP * args.blocks_x;
  unsigned in_group;
  const unsigned g = small ? small_div(t, group_size, &in_group) : t / group_size;
  if (!small) in_group = t - g * group_size;
  const unsigned first_y = g * GROUP;
  const unsigned rows_in_group =
      (args.blocks_y - first_y) < GROUP ? (args.blocks_y - first_y) : GROUP;
  if (rows_in_group == GROUP) {
    tc.block_y = first_y + in_group % GROUP;
    tc.block_x = in_group / GROUP;
  } else if (small) {
    unsigned y;
    tc.block_x = small_div(in_group, rows_in_group, &y);
    tc.block_y = first_y + y;
  } else {
    tc.block_y = first_y + in_group % rows_in_group;
    tc.block_x = in_group / rows_in_group;
  }
  // wave-uniform by construction; say so, so that addresses built from them stay scalar
  tc.b = (unsigned)__builtin_amdgcn_readfirstlane((int)tc.b);
  tc.block_x = (unsigned)__builtin_amdgcn_readfirstlane((int)tc.block_x);
  tc.block_y = (unsigned)__builtin_amdgcn_readfirstlane((int)tc.block_y);
  return tc;
}

// Fills the kernel argument block from the launch parameters for a BX x BY
// block tile.
inline KernelArgs make_kernel_args(const GemmParams &p, int bx, int by) {
  KernelArgs a;
  a.x = static_cast<const char *>(p.x);
  a.y = static_cast<const char *>(p.y);
  a.c = static_cast<char *>(p.c);
  a.batch = p.batch;
  a.nx = p.nx;
  a.ny = p.ny;
  a.k = p.k;
  a.k_tiles = p.k_tiles;
  // bytes of K per row of a planar operand: 1-bit samples are stored in whole
  // 32-bit words
  a.k_bytes = (p.type_in == kInt1) ? (unsigned)(ceil_div(p.k, 32) * 4)
                                   : (unsigned)((size_t)p.k * bits_of(p.type_in) / 8);
  a.x_tiles = p.x_tiles;
  a.y_tiles = p.y_tiles;
  const unsigned k_mem = p.k_in_memory ? p.k_in_memory : p.k;
  a.row_stride_bytes = (p.type_in == kInt1) ? (unsigned)(ceil_div(k_mem, 32) * 4)
                                            : (unsigned)((size_t)k_mem * bits_of(p.type_in) / 8);
  a.k_tile_stride = p.k_in_memory ? (unsigned)ceil_div(k_mem, (size_t)k_per_tile(p.type_in)) : p.k_tiles;
  a.blocks_x = (unsigned)ceil_div(p.nx, bx);
  a.blocks_y = (unsigned)ceil_div(p.ny, by);
  a.short_x = 0;
  if (p.variant == kOpt && !p.input_interleaved) {
    a.x_batch_bytes = (size_t)p.x_tiles * a.k_tile_stride * kTileBytes;
    a.y_batch_bytes = (size_t)p.y_tiles * a.k_tile_stride * kTileBytes;
  } else {
    a.x_batch_bytes = (size_t)2 * p.nx * a.row_stride_bytes;
    a.y_batch_bytes = (size_t)2 * p.ny * a.row_stride_bytes;
  }
  a.alpha_re = p.alpha_re;
  a.alpha_im = p.alpha_im;
  a.beta_re = p.beta_re;
  a.beta_im = p.beta_im;
  a.have_alpha = p.have_alpha;
  a.have_beta = p.have_beta;
  a.c_interleaved = p.c_interleaved;
  a.c_vector_ok = ((uintptr_t)p.c % 16 == 0);
  a.im_excess = (p.type_in == kInt1) ? 2u * (p.k_tiles * (unsigned)k_per_tile(kInt1) - p.k) : 0u;
  return a;
}

}  // namespace ccglib_amd
#endif  // CCGLIB_AMD_GEMM_DEVICE_H_
