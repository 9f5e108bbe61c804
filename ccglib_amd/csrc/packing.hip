// Bit packing and unpacking of 1-bit samples.
// Stands in for the reference's pack_bits / unpack_bits
// (kernels/packing_kernel.cu:7-49, :51-62): output bit t (LSB first in 32-bit
// words) is (input byte != 0) at index t, or for interleaved (re, im) input at
// index 2t, minus N-1 when that runs past the end, which puts all real bits in
// front of all imaginary bits.
//
// The reference reads one byte per thread and ballots. Here every lane reads
// 16 bytes with one load, turns them into 16 bits with integer arithmetic, and
// neighbouring lanes are merged with cross-lane moves, so a wave reads 1 KiB
// per load instruction and writes whole words.
#include "common.h"

namespace ccglib_amd {
namespace {

typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

// 4 bytes -> 4 bits (bit i = byte i != 0).
__device__ __forceinline__ unsigned nibble_of(unsigned x) {
  const unsigned nz = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
  return (((nz >> 7) * 0x00204081u) >> 21) & 0xfu;
}

// 16 bytes -> 16 bits.
__device__ __forceinline__ unsigned bits_of16(uint4_t v) {
  return nibble_of(v[0]) | (nibble_of(v[1]) << 4) | (nibble_of(v[2]) << 8) |
         (nibble_of(v[3]) << 12);
}

// 4 bits -> 4 bytes of 0/1.
__device__ __forceinline__ unsigned bytes_of_nibble(unsigned b) {
  return ((b & 0xfu) * 0x00204081u) & 0x01010101u;
}

// 16 bytes at any address: one wide load (global memory takes any alignment on
// this target; a load that straddles cache lines costs a little bandwidth).
typedef uint4_t uint4_unaligned_t __attribute__((aligned(1)));

template <bool ALIGNED> __device__ __forceinline__ uint4_t load16(const unsigned char *p) {
  if constexpr (ALIGNED) {
    return __builtin_nontemporal_load(reinterpret_cast<const uint4_t *>(p));
  } else {
    return *reinterpret_cast<const uint4_unaligned_t *>(p);
  }
}

// Planar: thread -> kPackPerThread times 16 input bytes, each half an output word;
// lane pairs merge. A wave takes 64 * kPackPerThread consecutive groups, so every
// load instruction reads 1 KiB contiguous and a thread has several in flight.
// n16 = number of whole 16-byte groups that make whole words (2 per word).
constexpr int kPackPerThread = 2;
template <bool ALIGNED>
__global__ __launch_bounds__(256) void pack_planar_vec(const unsigned char *__restrict__ in,
                                                       unsigned *__restrict__ out, size_t n16) {
  const size_t stride = (size_t)gridDim.x * 256 * kPackPerThread;
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // n16 and every item index base + 64 k are even, so a lane pair is in or out together
  for (size_t base = ((size_t)blockIdx.x * 4 + wave) * 64 * kPackPerThread; base < n16; base += stride) {
    uint4_t v[kPackPerThread];
#pragma unroll
    for (int k = 0; k < kPackPerThread; ++k) {
      const size_t gi = base + k * 64 + lane;
      v[k] = gi < n16 ? load16<ALIGNED>(in + gi * 16) : uint4_t{0, 0, 0, 0};
    }
#pragma unroll
    for (int k = 0; k < kPackPerThread; ++k) {
      const size_t gi = base + k * 64 + lane;
      const unsigned mine = bits_of16(v[k]);
      const unsigned next = __shfl_down(mine, 1);
      if ((lane & 1) == 0 && gi < n16) out[gi >> 1] = mine | (next << 16);
    }
  }
}

// Interleaved: thread -> 16 input bytes = 8 (re, im) pairs -> 8 real bits and
// 8 imaginary bits; four lanes merge into one real and one imaginary word. As
// in the planar kernel a wave takes 64 * kPackPerThread consecutive groups. The
// input is `segments` buffers of seg16 groups each, one after the other, every one
// packed on its own (all its real bits, then all its imaginary bits): one segment
// is the reference's packing of a whole buffer, one per batch is what the
// pipeline needs. A segment must hold a multiple of 64 samples, so that its
// imaginary half starts on a word boundary and four lanes never straddle two.
template <bool ALIGNED>
__global__ __launch_bounds__(256) void pack_interleaved_vec(const unsigned char *__restrict__ in,
                                                            unsigned *__restrict__ out,
                                                            size_t seg16) {
  // blockIdx.y: the segment (no division per item to find it)
  const size_t seg_words = seg16 / 2;        // packed words of one segment
  in += (size_t)blockIdx.y * seg16 * 16;
  unsigned *o_re = out + (size_t)blockIdx.y * seg_words, *o_im = o_re + seg_words / 2;
  const size_t stride = (size_t)gridDim.x * 256 * kPackPerThread;
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (size_t base = ((size_t)blockIdx.x * 4 + wave) * 64 * kPackPerThread; base < seg16; base += stride) {
    uint4_t v[kPackPerThread];
#pragma unroll
    for (int k = 0; k < kPackPerThread; ++k) {
      const size_t gi = base + k * 64 + lane;
      v[k] = gi < seg16 ? load16<ALIGNED>(in + gi * 16) : uint4_t{0, 0, 0, 0};
    }
#pragma unroll
    for (int k = 0; k < kPackPerThread; ++k) {
      const size_t gi = base + k * 64 + lane;
      // real parts are the even bytes, imaginary parts the odd ones: gather each
      // kind into two words first, then 4 bytes -> 4 bits as in the planar kernel
      const unsigned re_lo = __builtin_amdgcn_perm(v[k][1], v[k][0], 0x06040200u);
      const unsigned re_hi = __builtin_amdgcn_perm(v[k][3], v[k][2], 0x06040200u);
      const unsigned im_lo = __builtin_amdgcn_perm(v[k][1], v[k][0], 0x07050301u);
      const unsigned im_hi = __builtin_amdgcn_perm(v[k][3], v[k][2], 0x07050301u);
      const unsigned mine = nibble_of(re_lo) | (nibble_of(re_hi) << 4) | (nibble_of(im_lo) << 8) |
                            (nibble_of(im_hi) << 12);
      const unsigned l1 = __shfl_down(mine, 1), l2 = __shfl_down(mine, 2),
                     l3 = __shfl_down(mine, 3);
      if ((lane & 3) == 0 && gi < seg16) {
        const unsigned re = (mine & 0xffu) | ((l1 & 0xffu) << 8) | ((l2 & 0xffu) << 16) |
                            ((l3 & 0xffu) << 24);
        const unsigned im = ((mine >> 8) & 0xffu) | (((l1 >> 8) & 0xffu) << 8) |
                            (((l2 >> 8) & 0xffu) << 16) | (((l3 >> 8) & 0xffu) << 24);
        o_re[gi >> 2] = re;
        o_im[gi >> 2] = im;
      }
    }
  }
}

// Any N: one thread per output word, byte loads. For the end of a buffer that
// is not whole words and for interleaved segments that are not multiples of 64
// samples. Interleaved input is `segments` buffers of n samples each (see above);
// word w then counts the words of all segments, ceil(n / 32) each.
__global__ __launch_bounds__(256) void pack_scalar(const unsigned char *__restrict__ in,
                                                   unsigned *__restrict__ out, size_t n,
                                                   size_t first_word, size_t words,
                                                   int interleaved) {
  const size_t w = first_word + (size_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= words) return;
  const size_t seg_words = (n + 31) / 32;
  const size_t seg = interleaved ? w / seg_words : 0, lw = interleaved ? w % seg_words : w;
  const unsigned char *src = in + seg * n;
  unsigned v = 0;
  for (unsigned bit = 0; bit < 32; ++bit) {
    const size_t t = lw * 32 + bit;
    if (t >= n) break;
    size_t idx = t;
    if (interleaved) {
      idx = 2 * t;
      if (idx >= n) idx -= n - 1;
    }
    if (src[idx] != 0) v |= 1u << bit;
  }
  out[w] = v;
}

// thread -> four times 16 output bytes, each from half a word: four small loads
// in flight per thread (with one, the kernel waits on the latency of its reads),
// and every store instruction of a wave writes 1 KiB contiguous.
constexpr int kUnpackPerThread = 4;
template <bool ALIGNED>
__global__ __launch_bounds__(256) void unpack_vec(const unsigned *__restrict__ in,
                                                  unsigned char *__restrict__ out, size_t n16) {
  const size_t stride = (size_t)gridDim.x * 256 * kUnpackPerThread;
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (size_t base = ((size_t)blockIdx.x * 4 + wave) * 64 * kUnpackPerThread; base < n16;
       base += stride) {
    unsigned w[kUnpackPerThread];
#pragma unroll
    for (int k = 0; k < kUnpackPerThread; ++k) {
      const size_t g = base + k * 64 + lane;
      w[k] = g < n16 ? __builtin_nontemporal_load(in + (g >> 1)) : 0u;
    }
#pragma unroll
    for (int k = 0; k < kUnpackPerThread; ++k) {
      const size_t g = base + k * 64 + lane;
      if (g < n16) {
        const unsigned h = (w[k] >> ((g & 1) * 16)) & 0xffffu;
        const uint4_t v = {bytes_of_nibble(h), bytes_of_nibble(h >> 4), bytes_of_nibble(h >> 8),
                           bytes_of_nibble(h >> 12)};
        if constexpr (ALIGNED) {
          __builtin_nontemporal_store(v, reinterpret_cast<uint4_t *>(out) + g);
        } else {
          *reinterpret_cast<uint4_unaligned_t *>(out + g * 16) = v;   // one wide store at any address
        }
      }
    }
  }
}

__global__ __launch_bounds__(256) void unpack_scalar(const unsigned *__restrict__ in,
                                                     unsigned char *__restrict__ out,
                                                     size_t first, size_t n) {
  const size_t t = first + (size_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= n) return;
  out[t] = (unsigned char)((in[t / 32] >> (t % 32)) & 1u);
}

unsigned grid_for(size_t items, size_t per_thread) {
  // As many blocks as the items take at `per_thread` items a thread (few items
  // per thread measured fastest on this part: the streams are read or written
  // exactly once, with the non-temporal hint); the grid-stride loops only
  // matter beyond the cap.
  const size_t want = ceil_div(items, 256 * per_thread);
  const size_t cap = (size_t)1 << 30;
  size_t g = want < cap ? want : cap;
  if (g == 0) g = 1;
  return (unsigned)g;
}

}  // namespace

hipError_t launch_pack_bits(const unsigned char *in, unsigned *out, size_t n, int interleaved,
                            hipStream_t stream, size_t segments) {
  if (n == 0 || segments == 0) return hipSuccess;
  if (!interleaved) {
    n *= segments;   // planar packing is the same flat map whatever the batch structure
    segments = 1;
  }
  const size_t seg_words = ceil_div(n, 32), words = seg_words * segments;
  size_t vec_words = 0;  // words produced by the vector kernels
  const bool aligned = ((uintptr_t)in % 16 == 0);
  if (!interleaved) {
    vec_words = n / 32;
    if (vec_words) {
      const size_t n16 = vec_words * 2;
      const dim3 grid(grid_for(n16, kPackPerThread));
      if (aligned) {
        hipLaunchKernelGGL(pack_planar_vec<true>, grid, dim3(256), 0, stream, in, out, n16);
      } else {
        hipLaunchKernelGGL(pack_planar_vec<false>, grid, dim3(256), 0, stream, in, out, n16);
      }
    }
  } else if (n % 64 == 0) {
    vec_words = words;
    const size_t seg16 = n / 16;
    // one grid row per segment, at most 65535 rows a launch
    for (size_t first = 0; first < segments; first += 65535) {
      const size_t rows = segments - first < 65535 ? segments - first : 65535;
      const dim3 grid(grid_for(seg16, kPackPerThread), (unsigned)rows);
      const unsigned char *src = in + first * n;
      unsigned *dst = out + first * seg_words;
      if (aligned) {
        hipLaunchKernelGGL(pack_interleaved_vec<true>, grid, dim3(256), 0, stream, src, dst, seg16);
      } else {
        hipLaunchKernelGGL(pack_interleaved_vec<false>, grid, dim3(256), 0, stream, src, dst, seg16);
      }
    }
  }
  if (vec_words < words) {
    const size_t rest = words - vec_words;
    const size_t blocks = ceil_div(rest, 256);
    if (blocks > 0x7fffffffu) return hipErrorInvalidValue;
    hipLaunchKernelGGL(pack_scalar, dim3((unsigned)blocks), dim3(256), 0, stream, in, out, n,
                       vec_words, words, interleaved);
  }
  return hipGetLastError();
}

hipError_t launch_unpack_bits(const unsigned *in, unsigned char *out, size_t n,
                              hipStream_t stream) {
  if (n == 0) return hipSuccess;
  size_t done = 0;
  if (n >= 16) {
    const size_t n16 = n / 16;
    const dim3 grid(grid_for(n16, kUnpackPerThread));
    if ((uintptr_t)out % 16 == 0) {
      hipLaunchKernelGGL(unpack_vec<true>, grid, dim3(256), 0, stream, in, out, n16);
    } else {
      hipLaunchKernelGGL(unpack_vec<false>, grid, dim3(256), 0, stream, in, out, n16);
    }
    done = n16 * 16;
  }
  if (done < n) {
    const size_t blocks = ceil_div(n - done, 256);
    if (blocks > 0x7fffffffu) return hipErrorInvalidValue;
    hipLaunchKernelGGL(unpack_scalar, dim3((unsigned)blocks), dim3(256), 0, stream, in, out, done,
                       n);
  }
  return hipGetLastError();
}

}  // namespace ccglib_amd
