// Wide-block variant of the direct-to-LDS complex GEMM for 16-bit input in the
// tiled (opt) layout - or, as a second instantiation, in the caller's rows of
// (re, im) pairs, see IL below: a 192 x 256 patch of C per block, four waves (one
// per SIMD, the whole register file each) of 192 x 64, i.e. 12 x 4 MFMA tiles of
// 16 x 16 and 384 accumulator registers per lane.
//
// Compared with the 256 x 128 block of complex_gemm_mfma_dtl this moves 22 % fewer
// bytes from L2 to LDS per flop (448 operand rows per 49152 products instead of
// 384 per 32768), passes one barrier per 3072 instead of per 2048 matrix-core
// cycles, and gives a K tile that much longer to arrive.
//
//  * One wave per SIMD has to keep the matrix core busy by itself: whatever else
//    the wave issues goes between two matrix instructions, a few instructions at a
//    time, and nothing may make it wait in the middle of the K loop.
//  * X (the operand along the contiguous axis of C) is shared by the four waves:
//    a ring of three 24 KiB slots in LDS, one barrier per K iteration. X is the
//    instruction's "B" operand in the exchanged-roles layout of
//    complex_gemm_mfma_dtl, so register e of four neighbouring tiles holds four
//    consecutive x and C rows are stored straight from the accumulators.
//  * Y is private: wave w multiplies rows 64 w .. 64 w + 63 of the block's Y and
//    nobody else reads them, so the wave copies exactly those rows itself; its own
//    s_waitcnt covers them and no barrier is involved. The wave holds the eight Y
//    fragments of a K tile in registers for the whole iteration, so a Y slot is
//    free as soon as they are read: two slots give the copy the same two
//    iterations of lead as X has with three.
//  * The iteration boundary lies inside the last X tile of an iteration: once the
//    wave's last read of the current X slot has returned it waits for its copies
//    of the next K tile, passes the barrier, and reads the next iteration's first
//    X fragments and - each into the registers of its predecessor, right behind
//    that one's last use - the next Y fragments, all behind the remaining matrix
//    instructions of the tile. The next iteration starts with its operands in
//    registers.
//  * The order of a tile's 16 matrix instructions (two Y tile rows at a time) is
//    chosen so that the Y fragments die one by one over the tile; for every sum it
//    keeps the order of complex_gemm_mfma_dtl (Xr Yr before Xi Yi, Xr Yi before
//    Xi Yr), so both kernels produce the same bits.
//
//  * Where 192 does not divide the width of C, the last one or two tiles of a row
//    of tiles can be short ones of 128 columns (see WideTile): 8 instead of 12 X
//    tiles per K iteration, with a K loop of their own.
//
// Included by gemm_mfma.hip inside its namespaces, after the helpers it uses.
#ifndef CCGLIB_AMD_GEMM_MFMA_WIDE_H_
#define CCGLIB_AMD_GEMM_MFMA_WIDE_H_

constexpr int kWideBX = 192, kWideBY = 256;
constexpr int kWideXSlots = 3, kWideYSlots = 2;
constexpr int kWideLdsBytes =
    (kWideXSlots * 2 * kWideBX + kWideYSlots * 2 * kWideBY) * kTileRowBytes;   // 136 KiB
constexpr int kWideTX = kWideBX / 16;   // X tiles of a wave
constexpr int kWideShortBX = 128;       // columns of a short tile: the first eight X tiles

// The MFMA as an inline-asm statement with the register file of the accumulator
// spelled out. The compiler puts the accumulators of all matrix instructions of a
// function into the AccVGPR half of the register file; with 384 of them it would
// keep 128 in the other half and copy them in and out around every instruction
// that uses them. Here the accumulators of the first eight X tiles are declared
// as AccVGPRs (all 256) and those of the last four as ordinary VGPRs, and stay
// where they are. What the compiler no longer does for these statements: the
// wait states between a matrix instruction and a dependent read of its result by
// another kind of instruction - the epilogue waits explicitly
// (wait_for_mfma_results) - and the wait states between a vector-ALU write of an
// operand register and the matrix instruction that reads it: every value derived
// from a fragment is therefore pinned several matrix instructions ahead of its
// use (flip_sign, swap_pairs), and tests/test_kernel_asm.py scans the generated
// code for a vector-ALU write right in front of a matrix instruction that reads
// it. (An s_nop in front of every matrix instruction would do as well and
// measured 6 % slower.) A matrix instruction that adds to the result of the one
// before needs none.
// ZERO: the sum starts from zero (first K tile of a C tile).
template <int DT, bool ACC_IN_AGPR, bool ZERO>
__device__ __forceinline__ void mfma16_asm(float4_t &acc, const int4_t &a, const int4_t &b) {
  if constexpr (kAblateMfma) {
    // (timing-only build: the accumulator and the operands stay where they are)
    if constexpr (ACC_IN_AGPR) {
      asm volatile("" : "+a"(acc) : "v"(a), "v"(b));
    } else {
      asm volatile("" : "+v"(acc) : "v"(a), "v"(b));
    }
    return;
  }
#define CCGLIB_MFMA_ASM(OPCODE)                                                                    \
  if constexpr (ACC_IN_AGPR) {                                                                     \
    if constexpr (ZERO) {                                                                          \
      asm volatile(OPCODE " %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));                          \
    } else {                                                                                       \
      asm volatile(OPCODE " %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));                         \
    }                                                                                              \
  } else {                                                                                         \
    if constexpr (ZERO) {                                                                          \
      asm volatile(OPCODE " %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));                         \
    } else {                                                                                       \
      asm volatile(OPCODE " %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));                         \
    }                                                                                              \
  }
  if constexpr (DT == kFloat16) {
    CCGLIB_MFMA_ASM("v_mfma_f32_16x16x32_f16")
  } else {
    static_assert(DT == kBfloat16, "16-bit input");
    CCGLIB_MFMA_ASM("v_mfma_f32_16x16x32_bf16")
  }
#undef CCGLIB_MFMA_ASM
}

// Results of the matrix instructions issued last may be read by other instructions
// only after up to 18 wait states.
__device__ __forceinline__ void wait_for_mfma_results() {
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
}

// Register e of the four tiles of a 64-column group are four consecutive x of a
// C row: a lane writes 16 bytes (8 for fp16 / bf16 C) and a store instruction four
// whole row segments, straight from the accumulators. This empty asm statement
// takes four accumulators where they are at this point of the instruction stream.
template <bool ACC_IN_AGPR>
__device__ __forceinline__ void take_accumulators(float4_t &a, float4_t &b, float4_t &c, float4_t &d) {
  if constexpr (ACC_IN_AGPR) {
    asm volatile("" : "+a"(a), "+a"(b), "+a"(c), "+a"(d));
  } else {
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
  }
}

// The C tiles of a launch: args.blocks_x tiles of 192 columns per row of tiles,
// followed - where 192 does not divide the width of C and the host found that it
// pays - by args.short_x tiles of 128 columns (4096 = 20 x 192 + 2 x 128) instead of
// one tile that hangs over the edge. All full tiles come first in the numbering,
// in the order of tile_coord; the short ones follow, so that a block, which walks
// the numbering with the stride of the grid, meets its full tiles before its short
// ones. A tile is named by its batch, its first column and its row of tiles.
struct WideTile {
  unsigned b, x0, block_y;
};
// BY_LANE: the tile id differs from lane to lane (plain divisions).
template <bool BY_LANE>
__device__ __forceinline__ WideTile wide_tile(const KernelArgs &args, unsigned id) {
  const unsigned full = args.blocks_x * args.blocks_y * args.batch;
  WideTile w;
  if (id >= full) {
    // short tiles of one row of tiles are neighbours; rows of a batch follow each other
    const unsigned r = xcd_remap(id - full, args.short_x * args.blocks_y * args.batch);
    const unsigned row = r / args.short_x;
    w.x0 = args.blocks_x * kWideBX + (r % args.short_x) * kWideShortBX;
    w.block_y = row % args.blocks_y;
    w.b = row / args.blocks_y;
    if constexpr (!BY_LANE) {
      w.b = (unsigned)__builtin_amdgcn_readfirstlane((int)w.b);
      w.x0 = (unsigned)__builtin_amdgcn_readfirstlane((int)w.x0);
      w.block_y = (unsigned)__builtin_amdgcn_readfirstlane((int)w.block_y);
    }
    return w;
  }
  if constexpr (!BY_LANE) {
    const TileCoord tc = tile_coord(args, id);
    return WideTile{tc.b, tc.block_x * kWideBX, tc.block_y};
  }
  const unsigned per_batch = args.blocks_x * args.blocks_y;
  const unsigned logical = xcd_remap(id, full);
  w.b = logical / per_batch;
  const unsigned t = logical % per_batch;
  constexpr unsigned GROUP = 4;
  const unsigned group_size = GROUP * args.blocks_x;
  const unsigned g = t / group_size, in_group = t % group_size;
  const unsigned first_y = g * GROUP;
  const unsigned rows_in_group = (args.blocks_y - first_y) < GROUP ? (args.blocks_y - first_y) : GROUP;
  w.block_y = first_y + in_group % rows_in_group;
  w.x0 = in_group / rows_in_group * kWideBX;
  return w;
}


// IL: the operands are the caller's rows of (re, im) pairs (the pipeline's
// interleaved input), read in place. A K iteration then covers 128 bytes of every
// row - 32 complex values, as with the two 64-byte planes of a tile - and, with k
// running over the 64 numbers of such a piece,
//   Re = sum (xr, -xi, ...) . (yr, yi, ...)     Im = sum (xi, xr, ...) . (yr, yi, ...)
// so the Y fragments are used as they are and both variants of an X fragment
// come from the raw one in registers (a sign flip of the odd elements, a swap
// inside each pair: 16 vector instructions per 16 matrix instructions, two behind
// each of a tile's last eight). The matrix instructions, the rings, the barrier
// and the stores are those of the tiled layout. In LDS a slot is a sequence of 1 KiB
// blocks of 8 rows, [the first 64 bytes of each row | the second 64 bytes]: a copy
// instruction fetches 8 whole 128-byte lines, and every fragment read touches
// the banks exactly as in the tiled layout (64-byte rows, 256 bytes apart every
// four), so the chunk swizzles of that layout carry over.
// ALPHA: the result is multiplied by the complex alpha of the arguments on its way
// out (both parts of an element sit in the same lane, in acc_re and acc_im).
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in this order.
template <int... Is, class F>
__device__ __forceinline__ void static_for_each(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_each(std::make_integer_sequence<int, N>{}, f);
}

// (the lambdas of the kernel: left to its cost estimate, the compiler keeps the larger
// ones as functions in some instantiations, and the accumulators then live in memory)
#define CCGLIB_INLINE __attribute__((always_inline))
template <int DT, int TOUT, bool IL, bool ALPHA>
__global__ __launch_bounds__(256, 1) void complex_gemm_mfma_wide(const KernelArgs args) {
  static_assert(DtypeTraits<DT>::kTilesPerMfma == 1 && DtypeTraits<DT>::kElemBytes == 2,
                "16-bit input");
  constexpr int BX = kWideBX, BY = kWideBY, TX = kWideTX;
  constexpr int XSLOTS = kWideXSlots, YSLOTS = kWideYSlots;
  static_assert(XSLOTS == 3 && YSLOTS == 2, "both operands are requested two iterations ahead");
  constexpr int XP = BX * kTileRowBytes, YP = BY * kTileRowBytes;   // one plane of a slot
  constexpr int X_BYTES = 2 * XP, Y_BYTES = 2 * YP;
  constexpr int Y_RING = XSLOTS * X_BYTES;
  // 1 KiB copies a wave issues per K tile: 6 row blocks of X and its own 8 of Y
  constexpr int kCopies = 14;
  // 16 and 64 rows of a slot, and the distance from the first to the second
  // fragment of a tile (im plane; second half of the 128 bytes)
  constexpr unsigned TILE16 = IL ? 2048 : 16 * kTileRowBytes;
  constexpr unsigned GROUP = 4 * TILE16;
  constexpr unsigned X2ND = IL ? 512 : XP, Y2ND = IL ? 512 : YP;

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // (interleaved rows: the host counts 64-byte pieces and only launches this
  // kernel for rows of whole 128-byte pieces)
  const unsigned k_tiles = IL ? args.k_tiles / 2 : args.k_tiles;
  const unsigned row_stride = 2 * args.row_stride_bytes;   // IL: bytes from row to row
  const unsigned full_total = args.blocks_x * args.blocks_y * args.batch;
  const unsigned total = full_total + args.short_x * args.blocks_y * args.batch;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char *)lds;

  // ---- the C tiles of this block -------------------------------------------------
  // The block's C tiles are blockIdx.x + k gridDim.x; the short tiles are the last
  // ones in the numbering, so these are full tiles up to some k and short ones from
  // there. Lane n works out the
  // coordinates of tile n once (the first 64; a block with more takes the slow
  // way for the rest), and the wave fetches them with a lane read at every tile
  // change: with one wave per SIMD the divisions would otherwise stand in the
  // middle of the MFMA stream.
  const unsigned first_tile = blockIdx.x, tile_stride = gridDim.x;
  const unsigned my_tiles = (total - first_tile + tile_stride - 1) / tile_stride;
  const unsigned my_full_tiles =
      first_tile < full_total ? (full_total - first_tile + tile_stride - 1) / tile_stride : 0;
  // The order in which the block takes them: its short tiles before its full ones
  // or after them, in turn for every four blocks of an XCD (the short tiles of one
  // row of tiles and of a batch's neighbouring rows, which share operands). A short
  // tile moves as many operand bytes as a full one for two thirds of the products:
  // all of them at once, behind the full tiles, would wait for memory.
  const unsigned short_begin = ((blockIdx.x / kNumXcd / 4) & 1) ? 0 : my_full_tiles;
  const unsigned short_end = short_begin + (my_tiles - my_full_tiles);
  auto tile_id = [&](unsigned n) {
    const unsigned k = n < short_begin ? n : n < short_end ? my_full_tiles + (n - short_begin) : n - (short_end - short_begin);
    return first_tile + k * tile_stride;
  };
  unsigned table_b, table_x, table_y;
  {
    unsigned vt = tile_id((unsigned)lane);
    vt = vt < total ? vt : first_tile;
    const WideTile tc = wide_tile<true>(args, vt);
    table_b = tc.b;
    table_x = tc.x0;
    table_y = tc.block_y;
  }
  auto coords = [&](unsigned n) {   // past the last tile: the last one again (copied, never used)
    n = n < my_tiles ? n : my_tiles - 1;
    WideTile tc;
    if (n < 64) {
      tc.b = (unsigned)__builtin_amdgcn_readlane((int)table_b, (int)n);
      tc.x0 = (unsigned)__builtin_amdgcn_readlane((int)table_x, (int)n);
      tc.block_y = (unsigned)__builtin_amdgcn_readlane((int)table_y, (int)n);
    } else {
      tc = wide_tile<false>(args, tile_id(n));
    }
    return tc;
  };

  // ---- the copy --------------------------------------------------------------
  // What a lane fetches of a 1 KiB row block (16 rows x 64 bytes) so that the
  // hardware's linear write (lane L at 16 L) produces the swizzled LDS layout:
  // Y: chunk XOR (row >> 1) & 3; X: the exchanged-roles order of rows and chunks,
  // whose chunk XOR depends on the parity of the row block
  // (see complex_gemm_mfma_dtl).
  const unsigned lane_off_y = (lane >> 2) * kTileRowBytes + (((lane & 3) ^ ((lane >> 3) & 3)) * 16);
  const int xt_row = 4 * (lane >> 4) + (((lane >> 2) & 3) ^ (lane >> 4));
  const unsigned lane_off_x_even = xt_row * kTileRowBytes + (lane & 3) * 16;
  const unsigned lane_off_x_odd = xt_row * kTileRowBytes + ((lane & 3) ^ 3) * 16;
  // IL: lane L of a copy writes chunk position L & 3 of row slot (L >> 2) & 7 in
  // half L >> 5 of an 8-row block. Y: row = slot, chunk XOR (row >> 1) & 3. X: the
  // exchanged-roles order, in which slot 4 a + (i ^ a) of a 16-row block holds row
  // 4 a + i and the chunks are XORed with 3 (16-row block & 1): for the 8-row block
  // q = 6 wave + i of the slot that is a = 2 (i & 1) + (slot >> 2) and 16-row
  // block parity ((i >> 1) + wave) & 1.
  const int cs = (lane >> 2) & 7, ch = lane >> 5, cpos = lane & 3;
  const unsigned il_off_y = cs * row_stride + (4 * ch + (cpos ^ ((cs >> 1) & 3))) * 16;
  unsigned il_off_x[2][2];   // [i & 1][(i >> 1) & 1]
#pragma unroll
  for (int qp = 0; qp < 2; ++qp) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int a = 2 * qp + (cs >> 2), row = 4 * (cs >> 2) + ((cs & 3) ^ a);
      const int bp = (e + wave) & 1;
      il_off_x[qp][e] = row * row_stride + (4 * ch + (cpos ^ (3 * bp))) * 16;
    }
  }

  // Wave w copies the row blocks 6 (w & 1) .. + 5 of plane w / 2 of X (consecutive
  // KiB of the slot) and the 64 rows of Y that it multiplies (4 consecutive KiB in
  // either plane).
  const unsigned x_plane = wave >> 1, x_rb0 = 6 * (wave & 1);
  const unsigned x_lds = lds_base + x_plane * XP + x_rb0 * 1024;
  const unsigned y_lds = lds_base + Y_RING + wave * (IL ? 64 * 128 : 64 * kTileRowBytes);
  struct Stream {
    unsigned n, kt;   // tile of the block and K tile of the request issued last
  };
  Stream xs{0, 0}, ys{0, 0};
  // wave-uniform: K tile 0 of the operand tile that holds row block i of the wave's
  // six of X; K tile 0 of the wave's rows of Y (re plane)
  const char *x_src[6], *y_src = nullptr;
  auto point_x = [&](unsigned n) CCGLIB_INLINE {
    const WideTile tc = coords(n);
    if constexpr (IL) {
      const char *op = args.x + (size_t)tc.b * args.x_batch_bytes;
#pragma unroll
      for (int i = 0; i < 6; ++i) {
        unsigned row0 = tc.x0 + (6 * wave + i) * 8;
        row0 = row0 < args.nx ? row0 : args.nx - 8;   // rows past the end: never stored
        x_src[i] = op + (size_t)row0 * row_stride;
      }
      return;
    }
    const char *op = args.x + (size_t)tc.b * args.x_batch_bytes + x_plane * kTilePlaneBytes;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      const unsigned row0 = tc.x0 + (x_rb0 + i) * 16;
      unsigned tile = row0 / kTileRows;
      tile = tile < args.x_tiles ? tile : args.x_tiles - 1;   // rows past the end: never stored
      x_src[i] = op + (size_t)tile * args.k_tile_stride * kTileBytes +
                 (row0 % kTileRows) * kTileRowBytes;
    }
  };
  auto point_y = [&](unsigned n) CCGLIB_INLINE {
    const WideTile tc = coords(n);
    const unsigned row0 = tc.block_y * BY + wave * 64;
    if constexpr (IL) {
      y_src = args.y + (size_t)tc.b * args.y_batch_bytes +
              (size_t)(row0 < args.ny ? row0 : args.ny - 64) * row_stride;
      return;
    }
    unsigned tile = row0 / kTileRows;
    tile = tile < args.y_tiles ? tile : args.y_tiles - 1;
    y_src = args.y + (size_t)tc.b * args.y_batch_bytes +
            (size_t)tile * args.k_tile_stride * kTileBytes + (row0 % kTileRows) * kTileRowBytes;
  };
  // Copy c of the 14 of a K tile: 0 - 7 the wave's rows of Y (re plane, then im),
  // 8 - 13 its row blocks of X. One at a time and well apart: every vector memory
  // instruction occupies the compute unit's address unit for 16 cycles, and a wave
  // that issues the next one earlier waits - with its matrix instructions behind it.
  auto issue = [&](int c, unsigned x_slot, unsigned y_slot) CCGLIB_INLINE {
    if constexpr (IL) {
      // 0 - 7: rows 8 c .. 8 c + 7 of the wave's 64 of Y; 8 - 13: its 8-row blocks of X
      if (c < 8) {
        load_1k_to_lds(y_src + (size_t)ys.kt * 128 + (size_t)(8 * c) * row_stride, il_off_y,
                       y_lds + y_slot * Y_BYTES + c * 1024);
      } else {
        const int i = c - 8;
        load_1k_to_lds(x_src[i] + (size_t)xs.kt * 128, il_off_x[i & 1][(i >> 1) & 1],
                       x_lds + x_slot * X_BYTES + i * 1024);
      }
      return;
    }
    if (c < 8) {
      const int plane = c >> 2, blk = c & 3;
      load_1k_to_lds(y_src + (size_t)ys.kt * kTileBytes + plane * kTilePlaneBytes + blk * 1024,
                     lane_off_y, y_lds + y_slot * Y_BYTES + plane * YP + blk * 1024);
    } else {
      const int i = c - 8;
      load_1k_to_lds(x_src[i] + (size_t)xs.kt * kTileBytes, (i & 1) ? lane_off_x_odd : lane_off_x_even,
                     x_lds + x_slot * X_BYTES + i * 1024);
    }
  };
  auto advance_x = [&]() CCGLIB_INLINE {
    if (++xs.kt == k_tiles) {
      xs.kt = 0;
      point_x(++xs.n);
    }
  };
  auto advance_y = [&]() CCGLIB_INLINE {
    if (++ys.kt == k_tiles) {
      ys.kt = 0;
      point_y(++ys.n);
    }
  };

  // ---- fragments ---------------------------------------------------------------
  typedef __attribute__((address_space(3))) const int4_t lds_int4_t;
  auto rd = [](unsigned address) { return *reinterpret_cast<lds_int4_t *>(address); };
  const int r16 = lane & 15, g4 = lane >> 4;
  unsigned xo[4];   // X fragment of tile i of a 64-row group, inside a slot
  // (IL: row slot S of a group lies at (S >> 3) KiB + 64 (S & 7) of the group's 8 KiB)
  auto row_address = [](int slot) {
    return IL ? (slot >> 3) * 1024 + (slot & 7) * 64 : slot * kTileRowBytes;
  };
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    xo[i] = lds_base + row_address(4 * r16 + (i ^ (r16 & 3))) + ((g4 ^ (3 * ((r16 >> 2) & 1))) * 16);
  }
  const unsigned yo = y_lds + (IL ? row_address(r16) + ((g4 ^ ((r16 >> 1) & 3)) * 16)
                                  : swizzled_row_offset(r16, g4));

  // ---- pipeline ------------------------------------------------------------------
  point_x(0);
  point_y(0);
  // the requests that iterations -2 and -1 would have made
#pragma unroll
  for (int c = 0; c < kCopies; ++c) issue(c, 0, 0);
  advance_y();
  advance_x();
#pragma unroll
  for (int c = 0; c < kCopies; ++c) issue(c, 1, 1);

  unsigned x_slot = 0, y_slot = 0;   // slots of the current iteration
  // the Y fragments of the current K tile (re and im; IL: first and second half of the 128 bytes)
  int4_t yr[4], yi[4];
  // X fragments of the current and the next tile: re, im, -im;
  // IL: xr, xi the two halves with the odd elements negated, xn, xm the halves with
  // the elements of each pair exchanged
  int4_t xr[2], xi[2], xn[2], xm[2];
  constexpr int kOddSign = (int)0x80000000u;
  // Values derived from a fragment are taken by an empty asm statement where they
  // are computed. Without it the compiler may sink the computation to just before
  // the matrix instruction that reads the result (it does so across the branches
  // around the C stores) - and for a matrix instruction in an asm statement it
  // does not insert the wait states that such a read needs after a vector-ALU
  // write: the instruction then sees the old register contents. With it, every
  // derived value is written several matrix instructions before its first use.
  auto swap_pairs = [](int v) CCGLIB_INLINE {
    int o = (int)__builtin_amdgcn_alignbit((unsigned)v, (unsigned)v, 16);
    asm volatile("" : "+v"(o));
    return o;
  };
  auto flip_sign = [](int v, int mask) CCGLIB_INLINE {
    int o = v ^ mask;
    asm volatile("" : "+v"(o));
    return o;
  };
  auto flip = [&](const int4_t &v) CCGLIB_INLINE {
    int4_t o;
#pragma unroll
    for (int w = 0; w < 4; ++w) o[w] = flip_sign(v[w], (int)DtypeTraits<DT>::kSignMask);
    return o;
  };
  // what the last tile of "iteration -1" would have done for iteration 0
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kCopies) : "memory");
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    yr[j] = rd(yo + j * TILE16);
    yi[j] = rd(yo + Y2ND + j * TILE16);
  }
  if constexpr (!kAblateBarrier) asm volatile("s_barrier" ::: "memory");
  xr[0] = rd(xo[0]);
  xi[0] = rd(xo[0] + X2ND);
  if constexpr (IL) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      xn[0][w] = swap_pairs(xr[0][w]);
      xm[0][w] = swap_pairs(xi[0][w]);
      xr[0][w] = flip_sign(xr[0][w], kOddSign);
      xi[0][w] = flip_sign(xi[0][w], kOddSign);
    }
    // (the first matrix instruction reads xr[0] right away)
    asm volatile("s_nop 7" ::: "memory");
  } else {
    xn[0] = flip(xi[0]);
  }

  // ---- the C stores ----------------------------------------------------------------
  // A wave's 192 x 64 patch leaves in 96 store instructions of four 256-byte row
  // segments (see store_piece), none of them after the K loop (but for a block's last
  // tile of a kind): they are issued one every other matrix instruction behind those
  // of the tile's LAST K iteration and of the next tile's FIRST one, as the
  // accumulators become final and before they are started again:
  //   group 0 (X tiles 0 - 3, final behind tile 3 of the last iteration): last iteration;
  //   group 1 (tiles 4 - 7): half in the last iteration, half in the next first one
  //   (which starts these accumulators again with its tile 4);
  //   group 2 (tiles 8 - 11): the next first iteration, before its tile 8.
  // (A short tile, 128 x 64 per wave: group 0 in its last iteration, group 1 in the
  // next first one.)
  // The host only launches this kernel for planar C without beta, with
  // 16-byte aligned rows and nx, ny multiples of 64: a 64 x 64 piece of a tile is
  // either inside C or outside.
  using Tout = typename OutType<TOUT>::type;
  struct StoreTarget {
    char *base;        // wave-uniform: row y_wave, column x_block of the tile's re plane
    bool inside[3];    // the wave's rows and the group's columns are inside C
    bool all;          // all three: every store of the tile is issued
  };
  StoreTarget target{nullptr, {false, false, false}, false};
  const unsigned lane_store_off =
      (unsigned)((((lane >> 4) * 4) * (size_t)args.nx + (lane & 15) * 4) * sizeof(Tout));
  const size_t plane_bytes = (size_t)args.nx * args.ny * sizeof(Tout);
  auto aim_stores = [&](unsigned n, bool short_tile) CCGLIB_INLINE {
    const WideTile tc = coords(n);
    const unsigned x_block = tc.x0, y_wave = tc.block_y * BY + wave * 64;
    target.base = args.c + ((size_t)tc.b * 2 * args.nx * args.ny + (size_t)y_wave * args.nx + x_block) *
                               sizeof(Tout);
    const bool y_in = y_wave < args.ny;
    target.inside[0] = y_in;
    target.inside[1] = y_in && x_block + 64 < args.nx;
    target.inside[2] = y_in && !short_tile && x_block + 128 < args.nx;
    target.all = short_tile ? target.inside[1] : target.inside[2];
  };
  // ---- the body: full tiles or short ones --------------------------------------------
  // A block computes its full tiles and its short ones one kind after the other, and
  // each kind has its own copy of what follows, with its own accumulators; the copies of the operands
  // run on from one to the other. All 256 AccVGPRs and 128 VGPRs are taken: where
  // two chains of updates of the same accumulators met (one loop over tiles of both
  // kinds, or short tiles that take over the stores of a full one) the compiler
  // would have to fit the registers of one into the gaps of the other - it copies
  // accumulators around instead, right behind matrix instructions whose wait states
  // it does not know.
  using Yes = std::true_type;
  using No = std::false_type;
  auto body = [&](auto narrow, unsigned n_begin, unsigned n_end) CCGLIB_INLINE {
  constexpr bool SHORT = decltype(narrow)::value;
  constexpr int TXK = SHORT ? kWideShortBX / 16 : TX;   // X tiles of a C tile
  float4_t acc_re[4][TXK], acc_im[4][TXK];

  // Store s (0 .. 31) of group g: tile row j = s / 8, plane (s / 4) % 2, register e =
  // s % 4 of the group's four tiles, which are four consecutive x of row 16 j + 4
  // (lane / 16) + e. The empty asm statement takes the accumulators where they are,
  // here and now: without it the compiler may read them right behind the matrix
  // instruction that wrote them, whose wait states it does not know.
  auto store_piece = [&](int g, int s) CCGLIB_INLINE {
    if (!target.inside[g] || (SHORT && g >= 2)) return;
    const int j = s >> 3, plane = (s >> 2) & 1, e = s & 3;
    float v[4];
    if constexpr (ALPHA) {
      // both parts of the four elements, through the helpers that every kernel's
      // epilogue uses, so that every block tile gives the same bits
      if (g < 2) {
        take_accumulators<true>(acc_re[j][4 * g], acc_re[j][4 * g + 1], acc_re[j][4 * g + 2], acc_re[j][4 * g + 3]);
        take_accumulators<true>(acc_im[j][4 * g], acc_im[j][4 * g + 1], acc_im[j][4 * g + 2], acc_im[j][4 * g + 3]);
      } else if constexpr (!SHORT) {
        take_accumulators<false>(acc_re[j][4 * g], acc_re[j][4 * g + 1], acc_re[j][4 * g + 2], acc_re[j][4 * g + 3]);
        take_accumulators<false>(acc_im[j][4 * g], acc_im[j][4 * g + 1], acc_im[j][4 * g + 2], acc_im[j][4 * g + 3]);
      }
      const float ar = args.alpha_re, ai = args.alpha_im;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float re = acc_re[j][4 * g + i][e], im = acc_im[j][4 * g + i][e];
        v[i] = plane == 0 ? alpha_times_re(ar, ai, re, im) : alpha_times_im(ar, ai, re, im);
      }
    } else {
      float4_t(&acc)[4][TXK] = plane == 0 ? acc_re : acc_im;
      if (g < 2) {
        take_accumulators<true>(acc[j][4 * g], acc[j][4 * g + 1], acc[j][4 * g + 2], acc[j][4 * g + 3]);
      } else if constexpr (!SHORT) {
        take_accumulators<false>(acc[j][4 * g], acc[j][4 * g + 1], acc[j][4 * g + 2], acc[j][4 * g + 3]);
      }
      v[0] = acc[j][4 * g][e];
      v[1] = acc[j][4 * g + 1][e];
      v[2] = acc[j][4 * g + 2][e];
      v[3] = acc[j][4 * g + 3][e];
    }
    if constexpr (!ALPHA) {
      // The four values are gathered in ordinary registers. Left to itself the
      // compiler gathers them in a tuple of AccVGPRs, and where every AccVGPR holds
      // an accumulator it moves four of those out of the way and back - reading
      // them right behind matrix instructions whose wait states it does not know.
      asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
    }
    char *p = target.base + plane * plane_bytes +
              ((size_t)(j * 16 + e) * args.nx + g * 64) * sizeof(Tout) + lane_store_off;
    if constexpr (kAblateStores) {
      if (v[0] == 12345.678f) *reinterpret_cast<Tout *>(p) = (Tout)v[1];   // (timing-only build)
    } else if constexpr (TOUT == kFloat32) {
      // (C is written once and not read again by this kernel: stores marked
      // non-temporal measured 0.4 % faster at B=64 512x4096x576)
      __builtin_nontemporal_store(float4_t{v[0], v[1], v[2], v[3]}, reinterpret_cast<float4_t *>(p));
    } else {
      Tout t4[4] = {(Tout)v[0], (Tout)v[1], (Tout)v[2], (Tout)v[3]};
      __builtin_nontemporal_store(__builtin_bit_cast(ushort4_t, t4), reinterpret_cast<ushort4_t *>(p));
    }
  };
  constexpr int kStoresPerIteration = 4 * TXK;   // half of a tile's stores

  // One K iteration. `first`: the first one of a C tile (sums start from zero);
  // written out on its own, so that the accumulators have one definition there and
  // one chain of updates in the loop over the middle ones. It also issues the
  // remaining stores of the previous C tile; for the block's first tile the target
  // is still the empty one and every store is skipped (a second variant without
  // the stores would meet this one where the loop begins - two chains of
  // definitions, see above). `last`: the last one of a C tile, which issues the
  // first half of its stores.
  // A short tile: the first eight X tiles only, the same 14 copies (the X rows past
  // the tile are fetched and not used) one every 8 instead of 12 matrix
  // instructions, the boundary inside X tile 7; its stores are those of group 0 in
  // the last iteration and those of group 1 in the next first one.
  auto iteration = [&](auto first, auto last) CCGLIB_INLINE {
    constexpr bool FIRST = decltype(first)::value, CARRY = FIRST, LAST = decltype(last)::value;
    constexpr int TXI = TXK;
    constexpr int kCopyEvery = SHORT ? 8 : 12;
    // the bookkeeping (which branches at a C tile change) of the copies issued
    // inside this iteration: K tile + 2 of both operands
    advance_y();
    advance_x();
    const unsigned x_next = x_slot + 1 == XSLOTS ? 0 : x_slot + 1;
    const unsigned x_refill = x_slot >= 1 ? x_slot - 1 : XSLOTS - 1;   // (x_slot + 2) % 3
    const unsigned xa = x_slot * X_BYTES, xa_next = x_next * X_BYTES;
    const unsigned ya_next = yo + (y_slot ^ 1) * Y_BYTES;
#define CCGLIB_PIN __builtin_amdgcn_sched_barrier(0)
    // what else is issued behind MFMA p of tile t
    auto behind = [&](int t, int p) CCGLIB_INLINE {
      const int s = t & 1;
      if (t + 1 < TXI) {
        // the next tile's X fragments into the other register set
        if (p == 0) {
          const unsigned a = xo[(t + 1) & 3] + xa + ((t + 1) >> 2) * GROUP;
          xr[s ^ 1] = rd(a);
          xi[s ^ 1] = rd(a + X2ND);
          CCGLIB_PIN;
        }
        if (!IL && p >= 10 && p < 14) {
          // -im of the next tile, one instruction behind each of four MFMAs (four in a
          // row would hold up the next MFMA); pinned on both sides: moved up, it
          // would wait for the read just issued
          CCGLIB_PIN;
          xn[s ^ 1][p - 10] = flip_sign(xi[s ^ 1][p - 10], (int)DtypeTraits<DT>::kSignMask);
          CCGLIB_PIN;
        }
      }
      if (IL && p >= 8) {
        // both variants of the next tile's fragments (the next iteration's first
        // tile behind the last one), two instructions behind each of eight MFMAs;
        // the exchange reads the raw value, so it comes before the sign flip
        const int ns = t + 1 < TXI ? (s ^ 1) : 0, w = 2 * (p & 1);
        CCGLIB_PIN;
        if (p < 10) {
          xn[ns][w] = swap_pairs(xr[ns][w]);
          xn[ns][w + 1] = swap_pairs(xr[ns][w + 1]);
        } else if (p < 12) {
          xr[ns][w] = flip_sign(xr[ns][w], kOddSign);
          xr[ns][w + 1] = flip_sign(xr[ns][w + 1], kOddSign);
        } else if (p < 14) {
          xm[ns][w] = swap_pairs(xi[ns][w]);
          xm[ns][w + 1] = swap_pairs(xi[ns][w + 1]);
        } else {
          xi[ns][w] = flip_sign(xi[ns][w], kOddSign);
          xi[ns][w + 1] = flip_sign(xi[ns][w + 1], kOddSign);
        }
        CCGLIB_PIN;
      }
      {
        // C stores behind every other MFMA (the odd ones; the copies go behind even
        // ones), all of them before the last copy of the iteration
        const int idx = 16 * t + p;
        if (LAST && (idx & 1) && idx >= 65 && idx < 65 + 2 * kStoresPerIteration) {
          const int s = (idx - 65) / 2;
          store_piece(s < 32 ? 0 : 1, s < 32 ? s : s - 32);
          CCGLIB_PIN;
        }
        if (CARRY && (idx & 1) && idx < 1 + 2 * kStoresPerIteration) {
          const int s = (idx - 1) / 2;
          if (SHORT) {
            store_piece(1, s);
          } else {
            store_piece(s < 16 ? 1 : 2, s < 16 ? 16 + s : s - 16);
          }
          CCGLIB_PIN;
        }
      }
      {
        // The copy of K tile + 2, one instruction every 12 (8) MFMAs from tile 1 on: the
        // Y slot whose fragments this iteration holds in registers, and the X slot
        // that the barrier of the previous iteration's last tile released.
        const int m = 16 * t + p - 16;
        if (m >= 0 && m % kCopyEvery == 6 && m / kCopyEvery < kCopies) {
          issue(m / kCopyEvery, x_refill, y_slot);
          CCGLIB_PIN;
        }
      }
      if (t == TXI - 1) {
        // The iteration boundary. MFMA 4 of the last tile has waited for the
        // wave's last fragment read from this X slot (IL: MFMA 0 has, whose operand
        // was computed from it; the boundary is at MFMA 1 there, so that the two
        // variants of the next fragments can be made behind MFMAs 8 - 15 as in
        // every other tile). Copy c goes out behind MFMA 22 + 12 c (22 + 8 c) of the
        // iteration: 14 of them before the boundary, or 13 (IL), or 12 (short tile) -
        // the rest of this iteration's copies is then still to come.
        constexpr int kBoundary = IL ? 1 : 4;
        constexpr int kAllBefore = (16 * (TXI - 1) + kBoundary - 22) / kCopyEvery + 1;
        constexpr int kCopiesBefore = kAllBefore < kCopies ? kAllBefore : kCopies;
        static_assert(kCopiesBefore == (SHORT ? 12 : IL ? 13 : 14), "copies issued before the boundary");
        static_assert(22 + kCopyEvery * (kCopies - 1) < 16 * TXI, "every copy inside the iteration");
        // stores of this iteration issued before the boundary: behind the odd MFMAs
        // from 65 (last iteration) or 1 (first) on, up to the boundary's own
        constexpr int kIdxBoundary = 16 * (TXI - 1) + kBoundary;
        constexpr int kLastOdd = kIdxBoundary % 2 ? kIdxBoundary : kIdxBoundary - 1;
        constexpr int kSoFar = (kLastOdd - (LAST ? 65 : 1)) / 2 + 1;
        constexpr int kStoresBefore = kSoFar < kStoresPerIteration ? kSoFar : kStoresPerIteration;
        static_assert(kStoresBefore == (!SHORT || !LAST ? kStoresPerIteration : IL ? 25 : 26), "stores before the boundary");
        if (p == kBoundary) {
          // This wave's copies of the next K tile are complete when nothing older
          // than the requests of this iteration is outstanding - which are its
          // copies and, in a first or last iteration of a tile that lies entirely
          // inside C, its stores so far (the counter retires loads in order and does
          // not tell them from stores; where stores may have been skipped, the
          // smaller number is the safe one and waits for more than it has to).
          if ((CARRY || LAST) && target.all) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kCopiesBefore + kStoresBefore) : "memory");
          } else {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kCopiesBefore) : "memory");
          }
          // every wave's part of the next X tile has landed, and nobody reads the
          // current X slot any more
          if constexpr (!kAblateBarrier) asm volatile("s_barrier" ::: "memory");
          xr[0] = rd(xo[0] + xa_next);
          xi[0] = rd(xo[0] + xa_next + X2ND);
          CCGLIB_PIN;
        }
        // each Y fragment of the next K tile into the registers of its
        // predecessor, behind that one's last use (in either order of the tile's
        // matrix instructions)
        if (p == 4) yr[0] = rd(ya_next);
        if (p == 5) yr[1] = rd(ya_next + TILE16);
        if (p == 6) yi[0] = rd(ya_next + Y2ND);
        if (p == 7) yi[1] = rd(ya_next + Y2ND + TILE16);
        if (p == 12) yr[2] = rd(ya_next + 2 * TILE16);
        if (p == 13) yr[3] = rd(ya_next + 3 * TILE16);
        if (p == 14) yi[2] = rd(ya_next + Y2ND + 2 * TILE16);
        if (p == 15) yi[3] = rd(ya_next + Y2ND + 3 * TILE16);
        if (p >= 4) CCGLIB_PIN;
        if (!IL && p >= 12) {
          xn[0][p - 12] = flip_sign(xi[0][p - 12], (int)DtypeTraits<DT>::kSignMask);
          CCGLIB_PIN;
        }
      }
    };
    // (one copy of the loop body per X tile, made by the template and not left to the
    // unroller: past a size limit that one leaves the loop as it is, and the
    // accumulators, then indexed at run time, would live in memory)
    static_for<TXI>([&](auto x_tile) CCGLIB_INLINE {
      constexpr int t = decltype(x_tile)::value;
      const int s = t & 1;
      // exchanged roles: Y supplies the instruction's "A" rows, X its "B" columns
#define CCGLIB_MM(ACC, Y, X, Z, P)                                                     \
  if (t < 8) {                                                                         \
    mfma16_asm<DT, true, Z>(ACC, Y, X);                                                \
  } else {                                                                             \
    mfma16_asm<DT, false, Z>(ACC, Y, X);                                               \
  }                                                                                    \
  behind(t, P);
      if constexpr (IL) {
        // first half of the 128 bytes, then the second, for two Y tile rows at a time
        CCGLIB_MM(acc_re[0][t], yr[0], xr[s], FIRST, 0)
        CCGLIB_MM(acc_re[1][t], yr[1], xr[s], FIRST, 1)
        CCGLIB_MM(acc_im[0][t], yr[0], xn[s], FIRST, 2)
        CCGLIB_MM(acc_im[1][t], yr[1], xn[s], FIRST, 3)
        CCGLIB_MM(acc_re[0][t], yi[0], xi[s], false, 4)
        CCGLIB_MM(acc_re[1][t], yi[1], xi[s], false, 5)
        CCGLIB_MM(acc_im[0][t], yi[0], xm[s], false, 6)
        CCGLIB_MM(acc_im[1][t], yi[1], xm[s], false, 7)
        CCGLIB_MM(acc_re[2][t], yr[2], xr[s], FIRST, 8)
        CCGLIB_MM(acc_re[3][t], yr[3], xr[s], FIRST, 9)
        CCGLIB_MM(acc_im[2][t], yr[2], xn[s], FIRST, 10)
        CCGLIB_MM(acc_im[3][t], yr[3], xn[s], FIRST, 11)
        CCGLIB_MM(acc_re[2][t], yi[2], xi[s], false, 12)
        CCGLIB_MM(acc_re[3][t], yi[3], xi[s], false, 13)
        CCGLIB_MM(acc_im[2][t], yi[2], xm[s], false, 14)
        CCGLIB_MM(acc_im[3][t], yi[3], xm[s], false, 15)
        return;
      }
      CCGLIB_MM(acc_re[0][t], yr[0], xr[s], FIRST, 0)
      CCGLIB_MM(acc_re[1][t], yr[1], xr[s], FIRST, 1)
      CCGLIB_MM(acc_im[0][t], yi[0], xr[s], FIRST, 2)
      CCGLIB_MM(acc_im[1][t], yi[1], xr[s], FIRST, 3)
      CCGLIB_MM(acc_im[0][t], yr[0], xi[s], false, 4)
      CCGLIB_MM(acc_im[1][t], yr[1], xi[s], false, 5)
      CCGLIB_MM(acc_re[0][t], yi[0], xn[s], false, 6)
      CCGLIB_MM(acc_re[1][t], yi[1], xn[s], false, 7)
      CCGLIB_MM(acc_re[2][t], yr[2], xr[s], FIRST, 8)
      CCGLIB_MM(acc_re[3][t], yr[3], xr[s], FIRST, 9)
      CCGLIB_MM(acc_im[2][t], yi[2], xr[s], FIRST, 10)
      CCGLIB_MM(acc_im[3][t], yi[3], xr[s], FIRST, 11)
      CCGLIB_MM(acc_im[2][t], yr[2], xi[s], false, 12)
      CCGLIB_MM(acc_im[3][t], yr[3], xi[s], false, 13)
      CCGLIB_MM(acc_re[2][t], yi[2], xn[s], false, 14)
      CCGLIB_MM(acc_re[3][t], yi[3], xn[s], false, 15)
#undef CCGLIB_MM
    });
#undef CCGLIB_PIN
    x_slot = x_next;
    y_slot ^= 1;
  };

  // (k_tiles >= 2: the host does not launch this kernel for a K of one tile)
  for (unsigned n = n_begin; n < n_end; ++n) {
    iteration(Yes{}, No{});
    for (unsigned it = 2; it < k_tiles; ++it) iteration(No{}, No{});
    aim_stores(n, SHORT);
    iteration(No{}, Yes{});
  }
  // the second half of the last tile's stores
  wait_for_mfma_results();
#pragma unroll
  for (int s = 0; s < kStoresPerIteration; ++s) {
    if (SHORT) {
      store_piece(1, s);
    } else {
      store_piece(s < 16 ? 1 : 2, s < 16 ? 16 + s : s - 16);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // (the next body's first iteration must not take these stores for its own)
  target = StoreTarget{nullptr, {false, false, false}, false};
  };   // body
  // (written out: in a loop over the two kinds everything would be live everywhere)
  if (short_begin == 0 && short_end > 0) body(Yes{}, 0, short_end);
  if (my_full_tiles > 0) {
    const unsigned first_full = short_begin == 0 ? short_end : 0;
    body(No{}, first_full, first_full + my_full_tiles);
  }
  if (short_begin != 0 && short_end > short_begin) body(Yes{}, short_begin, short_end);
  // nothing may still be writing into LDS when the block gives it back
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

#undef CCGLIB_INLINE

#endif  // CCGLIB_AMD_GEMM_MFMA_WIDE_H_
