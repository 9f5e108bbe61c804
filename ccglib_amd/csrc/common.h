// Shared definitions of the gfx950 complex-GEMM library: enum values, launch
// parameter blocks handed from the C ABI layer to the kernel launchers, and
// the tile geometry every kernel agrees on.
#ifndef CCGLIB_AMD_COMMON_H_
#define CCGLIB_AMD_COMMON_H_

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace ccglib_amd {

// Values of the reference enums (include/ccglib/common/value_type.h:14-22).
enum ValueType : int {
  kInt1 = 0,
  kInt32 = 1,
  kBfloat16 = 2,
  kFloat8e4m3 = 3,
  kFloat8e5m2 = 4,
  kFloat16 = 5,
  kFloat32 = 6
};
enum : int { kPlanar = 0, kInterleaved = 1 };
enum : int { kForward = 0, kBackward = 1 };
enum : int { kRowMajor = 0, kColMajor = 1 };
enum : int { kBasic = 0, kOpt = 1 };

// Tile geometry of the optimised layout. Every operand tile is 128 rows of
// 64 bytes of K (32 half/bfloat16 values, 64 fp8 values or 512 one-bit
// samples), real plane then imaginary plane: 16 KiB that are contiguous in
// memory, so a block copies a tile into LDS with plain 16-byte loads.
constexpr int kTileRows = 128;
constexpr int kTileRowBytes = 64;
constexpr int kTilePlaneBytes = kTileRows * kTileRowBytes;  // 8 KiB
constexpr int kTileBytes = 2 * kTilePlaneBytes;             // 16 KiB

inline size_t ceil_div(size_t a, size_t b) { return a / b + (a % b != 0); }

inline int bits_of(int type) {
  switch (type) {
    case kInt1: return 1;
    case kFloat8e4m3:
    case kFloat8e5m2: return 8;
    case kBfloat16:
    case kFloat16: return 16;
    case kFloat32:
    case kInt32: return 32;
    default: return 0;
  }
}

// K values (samples) held by one 64-byte tile row.
inline int k_per_tile(int type_in) { return kTileRowBytes * 8 / bits_of(type_in); }

// Problem description for one GEMM launch, in kernel terms. The kernel
// computes D[y][x] = sum_k X[x][k] * Y[y][k] with x the contiguous output
// axis: for a row-major C, X is the caller's B (N rows) and Y the caller's A
// (M rows); for a column-major C the two are exchanged by the host, which is
// valid because the complex product commutes.
struct GemmParams {
  const void *x;        // operand whose rows index the contiguous C axis
  const void *y;        // operand whose rows index the strided C axis
  void *c;
  unsigned batch;
  unsigned nx, ny;      // logical (un-padded) rows of X and Y
  unsigned k;           // logical K in samples
  unsigned k_tiles;     // number of 64-byte K tiles (ceil)
  // When a launch covers only a piece of K (x and y then point at the piece's
  // first tile or byte of row 0): K of the whole operand in memory, which sets
  // the distance between rows and between row tiles. 0: the same as k.
  unsigned k_in_memory = 0;
  unsigned x_tiles, y_tiles;  // 128-row tiles per operand (ceil)
  int type_in, type_out;
  int variant;          // kBasic: planar rows; kOpt: tiled layout
  int input_interleaved;  // operands are rows of (re, im) pairs; k_tiles counts 64-byte
                          // pieces of those rows (used by the pipeline only)
  int c_interleaved;    // 0 planar, 1 interleaved
  float alpha_re, alpha_im, beta_re, beta_im;
  int have_alpha, have_beta;
  // 1-bit pipeline only: device memory for both operands in the tiled 1-bit
  // layout, which the caller's bytes are packed into (may be null)
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  // 1-bit GEMM only: the MFMA kernel may multiply the packed words (0: the
  // vector-ALU kernel runs whatever the layout)
  int int1_direct = 1;
  int block_tile = 0;      // 0: chosen per problem; 1: 256 x 128 blocks; 2: 128 x 128; 3: 192 x 256
};

// Bytes of both operands in the tiled 1-bit layout (what the pipeline packs the
// caller's bytes into when the GEMM multiplies the packed words as they are).
size_t gemm_int1_tiles_bytes(size_t batch, size_t m, size_t n, size_t k);

// 1-bit GEMM whose operands p.x / p.y are one byte per sample, planar
// [batch][2][rows][k] (the pipeline's input): packed straight into 1-bit tiles
// in the workspace and multiplied on the fp4 MFMA. Only when gemm_int1_can_take_bytes.
bool gemm_int1_can_take_bytes(const GemmParams &p);
hipError_t launch_gemm_int1_from_bytes(const GemmParams &p, hipStream_t stream);

hipError_t launch_gemm_mfma(const GemmParams &p, hipStream_t stream);
const char *describe_gemm_mfma(const GemmParams &p);
hipError_t launch_gemm_int1(const GemmParams &p, hipStream_t stream);

struct TransposeParams {
  const void *in;
  void *out;
  size_t batch, m, n;        // n in elements of elem_bytes (words for 1 bit)
  size_t m_chunk, n_chunk;   // likewise
  int elem_bytes;            // 1, 2 or 4
  int interleaved;
};
hipError_t launch_transpose(const TransposeParams &p, hipStream_t stream);
// The two operands of one GEMM (rows of the same length): one launch where both
// take the same kernel.
hipError_t launch_transpose_pair(const TransposeParams &p0, const TransposeParams &p1,
                                 hipStream_t stream);

// Interleaved input may be `segments` buffers of n samples each, one after the
// other, each packed on its own into ceil(n / 32) words (real bits, then
// imaginary bits).
hipError_t launch_pack_bits(const unsigned char *in, unsigned *out, size_t n,
                            int interleaved, hipStream_t stream, size_t segments = 1);
hipError_t launch_unpack_bits(const unsigned *in, unsigned char *out, size_t n,
                              hipStream_t stream);

}  // namespace ccglib_amd
#endif  // CCGLIB_AMD_COMMON_H_
