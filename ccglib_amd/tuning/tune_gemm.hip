// Offline sweep over kernel configurations of the tiled-input complex GEMM on
// one gfx950 device: the counterpart of the reference's tuning/tune_gemm.py
// (which sweeps block and warp tile sizes of its kernel through a JIT tuner).
// The configurations here are template instantiations of the library's own
// kernel (block tile, wave tile, ring slots, MFMA shape), timed back to back on
// random operands of the given shape; the library's dispatch
// (launch_typed in ../csrc/gemm_mfma.hip) uses the winners.
//
//   make && ./tune_gemm [B M N K [filter]]       e.g.  ./tune_gemm 64 512 4096 576 f16
//   ZERO=1 ./tune_gemm ...                       all-zero operands (no power limit)
#include "../csrc/gemm_mfma.hip"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
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
};

// name: type, block BX x BY, wave WX x WY, ring slots, MFMA rows
static const std::vector<Config> kConfigs = {
    {"f16 256x128 w64x64 s3 m16", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16>, kFloat16, kFloat32},
    {"f16 256x128 w64x64 s3 m16 xt", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16, true>, kFloat16, kFloat32},
    {"f16 128x256 w64x64 s3 m16 xt", launch_dtl<kFloat16, kFloat32, 128, 256, 64, 64, 3, 2, kLoadTiled, 16, true>, kFloat16, kFloat32},
    {"f16 128x256 w64x64 y3 x4 m16 xt", launch_dtl<kFloat16, kFloat32, 128, 256, 64, 64, 3, 2, kLoadTiled, 16, true, 4>, kFloat16, kFloat32},
    {"f16 256x128 w64x64 s3 m32", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>, kFloat16, kFloat32},
    {"f16 128x128 w64x64 s2 m16", launch_dtl<kFloat16, kFloat32, 128, 128, 64, 64, 2, 2, kLoadTiled, 16>, kFloat16, kFloat32},
    {"f16 128x128 w64x32 s4 m16", launch_dtl<kFloat16, kFloat32, 128, 128, 64, 32, 4, 2, kLoadTiled, 16>, kFloat16, kFloat32},
    {"bf16 256x128 w64x64 s3 m16", launch_dtl<kBfloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16>, kBfloat16, kFloat32},
    {"f32 256x128 w64x64 s3 m16", launch_dtl<kFloat32, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 16>, kFloat32, kFloat32},
    {"fp8 256x128 w64x64 s3 m32", launch_dtl<kFloat8e4m3, kFloat32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>, kFloat8e4m3, kFloat32},
    {"fp8 128x128 w64x64 s2 m32", launch_dtl<kFloat8e4m3, kFloat32, 128, 128, 64, 64, 2, 2, kLoadTiled, 32>, kFloat8e4m3, kFloat32},
    {"fp8 128x128 w64x32 s4 m32", launch_dtl<kFloat8e4m3, kFloat32, 128, 128, 64, 32, 4, 2, kLoadTiled, 32>, kFloat8e4m3, kFloat32},
    {"int1 128x128 w64x64 s2 m32", launch_dtl<kInt1, kInt32, 128, 128, 64, 64, 2, 2, kLoadTiled, 32>, kInt1, kInt32},
    {"int1 256x128 w64x64 s3 m32", launch_dtl<kInt1, kInt32, 256, 128, 64, 64, 3, 2, kLoadTiled, 32>, kInt1, kInt32},
    // planar rows (basic variant) and raw interleaved rows (the pipeline's fused mode)
    {"f16 planar 256x128 w64x64 s3 m16", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 16>, kFloat16, kFloat32, kLoadPlanarVec},
    {"f16 planar 256x128 w64x64 s3 m16 xt", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 16, true>, kFloat16, kFloat32, kLoadPlanarVec},
    {"f16 interleaved 256x128 w64x64 s3 m16", launch_dtl<kFloat16, kFloat32, 256, 128, 64, 64, 3, 2, kLoadInterleavedVec, 16>, kFloat16, kFloat32, kLoadInterleavedVec},
    {"fp8 planar 256x128 w64x64 s3 m32", launch_dtl<kFloat8e4m3, kFloat32, 256, 128, 64, 64, 3, 2, kLoadPlanarVec, 32>, kFloat8e4m3, kFloat32, kLoadPlanarVec},
    {"fp8 interleaved 256x128 w64x64 s3 m32", launch_dtl<kFloat8e4m3, kFloat32, 256, 128, 64, 64, 3, 2, kLoadInterleavedVec, 32>, kFloat8e4m3, kFloat32, kLoadInterleavedVec},
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

// Random operand bytes that are ordinary numbers in the given type.
static void fill(std::vector<unsigned short> &h, int type) {
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
}

int main(int argc, char **argv) {
  unsigned B = 64, M = 512, N = 4096, K = 576;
  if (argc > 4) {
    B = (unsigned)std::atoi(argv[1]);
    M = (unsigned)std::atoi(argv[2]);
    N = (unsigned)std::atoi(argv[3]);
    K = (unsigned)std::atoi(argv[4]);
  }
  const char *filter = argc > 5 ? argv[5] : (argc == 2 ? argv[1] : nullptr);
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  std::printf("%-40s %10s %12s %10s   (B=%u M=%u N=%u K=%u%s)\n", "configuration", "ms", "TFLOP/s", "of peak", B, M, N, K,
              std::getenv("ZERO") ? ", zero operands" : "");
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
    // whole tiles: at least as large as the planar and interleaved layouts
    const unsigned k_tiles_planar = (K + kpt - 1) / kpt;
    const size_t x_bytes = (size_t)B * p.x_tiles * k_tiles_planar * kTileBytes;
    const size_t y_bytes = (size_t)B * p.y_tiles * k_tiles_planar * kTileBytes;
    const size_t c_bytes = (size_t)B * 2 * M * N * 4;
    void *dx, *dy, *dc;
    CHECK(hipMalloc(&dx, x_bytes));
    CHECK(hipMalloc(&dy, y_bytes));
    CHECK(hipMalloc(&dc, c_bytes));
    std::vector<unsigned short> h(1 << 20);
    fill(h, c.type_in);
    for (size_t o = 0; o < x_bytes; o += h.size() * 2)
      CHECK(hipMemcpy((char *)dx + o, h.data(), std::min(h.size() * 2, x_bytes - o), hipMemcpyHostToDevice));
    for (size_t o = 0; o < y_bytes; o += h.size() * 2)
      CHECK(hipMemcpy((char *)dy + o, h.data(), std::min(h.size() * 2, y_bytes - o), hipMemcpyHostToDevice));
    if (std::getenv("ZERO")) {
      CHECK(hipMemset(dx, 0, x_bytes));
      CHECK(hipMemset(dy, 0, y_bytes));
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
    // layout with the same MFMA shape must agree
    std::vector<unsigned> hc(c_bytes / 4);
    CHECK(hipMemcpy(hc.data(), dc, c_bytes, hipMemcpyDeviceToHost));
    unsigned long long hash = 1469598103934665603ull;
    for (unsigned v : hc) hash = (hash ^ v) * 1099511628211ull;
    std::printf("%-40s %10.4f %12.1f %9.1f%%   C %016llx\n", c.name, best, tflops,
                100 * tflops / peak_of(c.type_in), hash);
    std::fflush(stdout);
    CHECK(hipFree(dx));
    CHECK(hipFree(dy));
    CHECK(hipFree(dc));
  }
  return 0;
}
