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

constexpr int kUnroll = 1;

// Planar: thread -> kPackPerThread times 16 input bytes, each half an output word;
// lane pairs merge. A wave takes 64 * kPackPerThread consecutive groups, so every
// load instruction reads 1 KiB contiguous and a thread has several in flight.
// n16 = number of whole 16-byte groups that make whole words (2 per word).
constexpr int kPackPerThread = 2;
__global__ __launch_bounds__(256) void pack_planar_vec(const uint4_t *__restrict__ in,
                                                       unsigned *__restrict__ out, size_t n16) {
  const size_t stride = (size_t)gridDim.x * 256 * kPackPerThread;
  const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // n16 and every item index base + 64 k are even, so a lane pair is in or out together
  for (size_t base = ((size_t)blockIdx.x * 4 + wave) * 64 * kPackPerThread; base < n16; base += stride) {
    uint4_t v[kPackPerThread];
#pragma unroll
    for (int k = 0; k < kPackPerThread; ++k) {
      const size_t gi = base + k * 64 + lane;
      v[k] = gi < n16 ? __builtin_nontemporal_load(in + gi) : uint4_t{0, 0, 0, 0};
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
// 8 imaginary bits; four lanes merge into one real and one imaginary word.
// Requires N % 64 == 0 so that the imaginary half starts on a word boundary.
__global__ __launch_bounds__(256) void pack_interleaved_vec(const uint4_t *__restrict__ in,
                                                            unsigned *__restrict__ out,
                                                            size_t n16, size_t imag_word0) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t g = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; g < n16; g += stride * kUnroll) {
    uint4_t v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const size_t gi = g + u * stride;
      v[u] = gi < n16 ? __builtin_nontemporal_load(in + gi) : uint4_t{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const size_t gi = g + u * stride;
      const unsigned b = bits_of16(v[u]);  // bit 2p = re of pair p, bit 2p+1 = im
      // gather even bits into the low byte, odd bits into the second byte
      unsigned e = b & 0x5555u, o = (b >> 1) & 0x5555u;
      e = (e | (e >> 1)) & 0x3333u;
      e = (e | (e >> 2)) & 0x0f0fu;
      e = (e | (e >> 4)) & 0x00ffu;
      o = (o | (o >> 1)) & 0x3333u;
      o = (o | (o >> 2)) & 0x0f0fu;
      o = (o | (o >> 4)) & 0x00ffu;
      const unsigned mine = e | (o << 8);
      const unsigned l1 = __shfl_down(mine, 1), l2 = __shfl_down(mine, 2),
                     l3 = __shfl_down(mine, 3);
      if ((threadIdx.x & 3) == 0 && gi < n16) {
        const unsigned re = (mine & 0xffu) | ((l1 & 0xffu) << 8) | ((l2 & 0xffu) << 16) |
                            ((l3 & 0xffu) << 24);
        const unsigned im = ((mine >> 8) & 0xffu) | (((l1 >> 8) & 0xffu) << 8) |
                            (((l2 >> 8) & 0xffu) << 16) | (((l3 >> 8) & 0xffu) << 24);
        out[gi >> 2] = re;
        out[imag_word0 + (gi >> 2)] = im;
      }
    }
  }
}

// Any N, any alignment: one thread per output word, byte loads.
__global__ __launch_bounds__(256) void pack_scalar(const unsigned char *__restrict__ in,
                                                   unsigned *__restrict__ out, size_t n,
                                                   size_t first_word, size_t words,
                                                   int interleaved) {
  const size_t w = first_word + (size_t)blockIdx.x * 256 + threadIdx.x;
  if (w >= words) return;
  unsigned v = 0;
  for (unsigned bit = 0; bit < 32; ++bit) {
    const size_t t = w * 32 + bit;
    if (t >= n) break;
    size_t idx = t;
    if (interleaved) {
      idx = 2 * t;
      if (idx >= n) idx -= n - 1;
    }
    if (in[idx] != 0) v |= 1u << bit;
  }
  out[w] = v;
}

// thread -> four times 16 output bytes, each from half a word: four small loads
// in flight per thread (with one, the kernel waits on the latency of its reads),
// and every store instruction of a wave writes 1 KiB contiguous.
constexpr int kUnpackPerThread = 4;
__global__ __launch_bounds__(256) void unpack_vec(const unsigned *__restrict__ in,
                                                  uint4_t *__restrict__ out, size_t n16) {
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
        __builtin_nontemporal_store(uint4_t{bytes_of_nibble(h), bytes_of_nibble(h >> 4),
                                            bytes_of_nibble(h >> 8), bytes_of_nibble(h >> 12)},
                                    out + g);
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
                            hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const size_t words = ceil_div(n, 32);
  size_t vec_words = 0;  // words produced by the vector kernel
  const bool aligned = ((uintptr_t)in % 16 == 0);
  if (aligned && !interleaved) {
    vec_words = n / 32;
    if (vec_words) {
      const size_t n16 = vec_words * 2;
      hipLaunchKernelGGL(pack_planar_vec, dim3(grid_for(n16, kPackPerThread)), dim3(256), 0, stream,
                         reinterpret_cast<const uint4_t *>(in), out, n16);
    }
  } else if (aligned && interleaved && n % 64 == 0) {
    vec_words = words;
    const size_t n16 = n / 16;
    hipLaunchKernelGGL(pack_interleaved_vec, dim3(grid_for(n16, kUnroll)), dim3(256), 0, stream,
                       reinterpret_cast<const uint4_t *>(in), out, n16, n / 64);
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
  if ((uintptr_t)out % 16 == 0 && n >= 16) {
    const size_t n16 = n / 16;
    hipLaunchKernelGGL(unpack_vec, dim3(grid_for(n16, kUnpackPerThread)), dim3(256), 0, stream, in,
                       reinterpret_cast<uint4_t *>(out), n16);
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
