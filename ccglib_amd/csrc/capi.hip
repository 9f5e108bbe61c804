// C ABI of the library (declared in include/ccglib_amd.h): argument checking,
// object state and stream plumbing around the kernel launchers. The host-side
// behaviour mirrors the reference classes it replaces: src/mma/GEMM.cpp,
// src/transpose/Transpose.cpp, src/packing/Packing.cpp,
// src/pipeline/Pipeline.cpp.
#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>

#include "../../include/ccglib_amd.h"
#include "common.h"

using namespace ccglib_amd;

namespace {

thread_local std::string g_last_error;

int fail(int code, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int fail_hip(hipError_t e, const char *what) {
  return fail(CCGLIB_ERROR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                   \
  do {                                                  \
    hipError_t e_ = (expr);                             \
    if (e_ != hipSuccess) return fail_hip(e_, #expr);   \
  } while (0)

// Makes `device` current for the lifetime of the guard.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) {
    if (hipGetDevice(&previous_) != hipSuccess) previous_ = -1;
    if (previous_ != device) {
      status_ = hipSetDevice(device);
      switched_ = (status_ == hipSuccess);
    }
  }
  ~DeviceGuard() {
    if (switched_ && previous_ >= 0) (void)hipSetDevice(previous_);
  }
  hipError_t status() const { return status_; }

 private:
  int previous_ = -1;
  bool switched_ = false;
  hipError_t status_ = hipSuccess;
};

int check_device(int device) {
  int count = 0;
  HIP_TRY(hipGetDeviceCount(&count));
  if (device < 0 || device >= count) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "device ordinal %d out of range (%d devices)",
                device, count);
  }
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strstr(prop.gcnArchName, "gfx950") == nullptr) {
    // same wording as the reference's check (src/mma/GEMM.cpp:128-130)
    return fail(CCGLIB_ERROR_UNSUPPORTED, "This architecture is not supported (%s; need gfx950)",
                prop.gcnArchName);
  }
  return CCGLIB_OK;
}

bool is_enum01(int v) { return v == 0 || v == 1; }

bool pair_supported(int in, int out) {
  switch (in) {
    case kFloat16: return out == kFloat32 || out == kFloat16;
    case kBfloat16: return out == kFloat32 || out == kBfloat16;
    case kFloat32: return out == kFloat32 || out == kFloat16 || out == kBfloat16;
    case kFloat8e4m3:
    case kFloat8e5m2: return out == kFloat32;
    case kInt1: return out == kInt32;
    default: return false;
  }
}

}  // namespace

struct ccglib_gemm {
  size_t B, M, N, K;
  int device;
  hipStream_t stream;
  int type_in, type_out, variant, c_axis, c_order;
  float alpha_re, alpha_im, beta_re, beta_im;
  // Set by the pipeline only: A and B are the caller's interleaved (re, im)
  // rows and are consumed as they are, without a transpose.
  bool input_interleaved = false;
  // Device memory the object owns (freed with it): the tiled copies of a
  // basic-variant GEMM (below), or, for the 1-bit pipeline, the 1-bit tiles
  // that the caller's bytes are packed into.
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
  // Basic variant whose planar rows direct-to-LDS copies cannot fetch (rows that
  // are not whole 16-byte chunks, or operands that are not 16-byte aligned): A
  // and B are first copied into the tiled layout (A at the start of
  // `workspace`, B at retile_b_offset) and the kernel of the opt variant runs on
  // the copies. retile_allowed: the option was on when the object was created.
  // (retile is set once, possibly by a Run: under lazy_lock, and read without it)
  std::atomic<bool> retile{false};
  bool retile_allowed = true;
  size_t retile_b_offset = 0;
  std::mutex lazy_lock;
  // 1-bit GEMM: the MFMA kernel multiplies the packed words (0: the option that
  // keeps it on the vector ALUs was set when the object was created)
  int int1_direct = 1;
  int block_tile = 0;
};

struct ccglib_transpose {
  size_t B, M, N, M_chunk, N_chunk, nr_bits;
  int device;
  hipStream_t stream;
  int axis;
  size_t input_bytes() const { return B * 2 * M * N * nr_bits / 8; }
};

struct ccglib_packing {
  size_t N;
  int direction, device, axis;
  hipStream_t stream;
  // Set by the pipeline only: interleaved input is this many buffers of
  // N / segments samples, one after the other, each packed on its own.
  size_t segments = 1;
};

struct ccglib_pipeline {
  size_t B, M, N, K;
  int device;
  hipStream_t stream;
  int type_in, type_out, c_axis;
  bool need_copyin_c;
  // 1-bit input, one byte per sample, planar: expanded straight into the GEMM's
  // workspace (no packed or transposed intermediates)
  bool int1_direct = false;
  // 8/16-bit interleaved input that the GEMM reads in place (no transposes);
  // `unfused` is the pipeline with transposes that takes over for buffers that
  // are not 16-byte aligned, created by the first Run that meets such buffers
  bool fused = false;
  std::atomic<ccglib_pipeline *> unfused{nullptr};   // (set once, under lazy_lock)
  std::mutex lazy_lock;
  ccglib_packing_t pack_a = nullptr, pack_b = nullptr;
  ccglib_transpose_t trans_a = nullptr, trans_b = nullptr;
  ccglib_gemm_t gemm = nullptr;
  void *d_a_packed = nullptr, *d_b_packed = nullptr, *d_a_trans = nullptr, *d_b_trans = nullptr;
  // What the object was created with, for the batch-chunked host path below.
  int in_axis = 0, a_order = 0, b_order = 0, c_order = 0, variant = 0;
  float alpha_re = 1, alpha_im = 0, beta_re = 0, beta_im = 0;
  // Host-pointer Run in chunks of whole batches on a few lanes, each a stream with
  // a pipeline of chunk_B batches and device buffers for one chunk, so that the
  // copies to the device, the kernels and the copies back of different chunks
  // overlap. Created by the first host Run that is large enough to use them.
  // (two: with three or four the copies of the 1.75 GB beamformer job took 25-35
  // ms instead of 23)
  static constexpr int kHostLanes = 2;
  size_t chunk_B = 0;
  ccglib_pipeline *lane[kHostLanes] = {};
  ccglib_pipeline *lane_tail = nullptr;   // for a last chunk of fewer batches
  hipStream_t lane_stream[kHostLanes] = {};
  void *lane_a[kHostLanes] = {}, *lane_b[kHostLanes] = {}, *lane_c[kHostLanes] = {};
  hipEvent_t caller_ready = nullptr;
};

namespace {

// Process-wide options (ccglib_amd_set_option), read when an object is created.
size_t g_options[CCGLIB_AMD_OPTION_COUNT] = {0, 1, 0, 0, 0, 0};

// Largest buffer of 1-bit tiles a pipeline allocates; beyond it the pipeline
// runs the reference's sequence of kernels on its packed / transposed buffers.
constexpr size_t kInt1TilesCap = (size_t)16 << 30;

// Bytes of A and of B in the tiled layout (whole tiles).
void tiled_bytes(const ccglib_gemm *g, size_t *bytes_a, size_t *bytes_b) {
  const size_t bits = (size_t)bits_of(g->type_in);
  const size_t kc = (size_t)k_per_tile(g->type_in);
  const size_t kp = ceil_div(g->K, kc) * kc;
  *bytes_a = g->B * 2 * ceil_div(g->M, kTileRows) * kTileRows * kp * bits / 8;
  *bytes_b = g->B * 2 * ceil_div(g->N, kTileRows) * kTileRows * kp * bits / 8;
}

// Gives a basic-variant GEMM the workspace for tiled copies of its operands.
// Failing to get the memory is not an error: the kernels that read planar rows
// in place then run.
void make_retile_workspace(ccglib_gemm *g) {
  if (g->workspace || !g->retile_allowed) return;
  size_t bytes_a = 0, bytes_b = 0;
  tiled_bytes(g, &bytes_a, &bytes_b);
  DeviceGuard guard(g->device);
  if (guard.status() == hipSuccess && hipMalloc(&g->workspace, bytes_a + bytes_b) == hipSuccess) {
    g->workspace_bytes = bytes_a + bytes_b;
    g->retile_b_offset = bytes_a;
    g->retile.store(true, std::memory_order_release);
  } else {
    g->workspace = nullptr;
    (void)hipGetLastError();
  }
}

// Whether work submitted to the stream is being recorded into a graph: nothing
// may be allocated then (an allocation would invalidate the capture).
bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

// Launch parameters of a GEMM object for the given buffers.
void fill_gemm_params(const ccglib_gemm *g, const void *d_a, const void *d_b, void *d_c,
                      GemmParams *out) {
  GemmParams &p = *out;
  // C[m][n] = sum_k A[m][k] B[n][k]. The kernel wants the operand of the
  // contiguous C axis as X: B for a row-major C, A for a column-major C (the
  // complex product commutes, so exchanging the operands transposes C).
  const bool row_major = (g->c_order == kRowMajor);
  p.x = row_major ? d_b : d_a;
  p.y = row_major ? d_a : d_b;
  p.nx = (unsigned)(row_major ? g->N : g->M);
  p.ny = (unsigned)(row_major ? g->M : g->N);
  p.c = d_c;
  p.batch = (unsigned)g->B;
  p.k = (unsigned)g->K;
  p.input_interleaved = g->input_interleaved;
  if (g->input_interleaved) {
    // a row holds K (re, im) pairs: twice the bytes, walked in 64-byte pieces
    p.k_tiles = (unsigned)ceil_div(2 * g->K, (size_t)k_per_tile(g->type_in));
  } else {
    p.k_tiles = (unsigned)ceil_div(g->K, (size_t)k_per_tile(g->type_in));
  }
  if (p.k_tiles == 0) p.k_tiles = 1;  // K = 0: one all-zero tile keeps the epilogue uniform
  p.x_tiles = (unsigned)ceil_div(p.nx, kTileRows);
  p.y_tiles = (unsigned)ceil_div(p.ny, kTileRows);
  p.type_in = g->type_in;
  p.type_out = g->type_out;
  p.variant = g->variant;
  p.c_interleaved = (g->c_axis == kInterleaved);
  p.alpha_re = g->alpha_re;
  p.alpha_im = g->alpha_im;
  p.beta_re = g->beta_re;
  p.beta_im = g->beta_im;
  // same switches as the reference's HAVE_ALPHA / HAVE_BETA (src/mma/GEMM.cpp:207-213)
  p.have_alpha = (g->alpha_re != 1.0f || g->alpha_im != 0.0f);
  p.have_beta = (g->beta_re != 0.0f || g->beta_im != 0.0f);
  p.workspace = g->workspace;
  p.workspace_bytes = g->workspace_bytes;
  p.int1_direct = g->int1_direct;
  p.block_tile = g->block_tile;
}

}  // namespace

namespace {

// Argument checks shared by the GEMM constructor and the stateless entry point,
// in the reference's order and with its wording.
int validate_gemm(size_t B, size_t M, size_t N, size_t K, int type_in, int type_out, int variant,
                  int c_complex_axis_location, int c_mem_order, int a_mem_order, int b_mem_order) {
  if (!is_enum01(variant) || !is_enum01(c_complex_axis_location) || !is_enum01(c_mem_order) ||
      !is_enum01(a_mem_order) || !is_enum01(b_mem_order)) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "enum argument out of range");
  }
  if (variant == kBasic && c_complex_axis_location == kInterleaved) {
    // src/mma/GEMM.cpp:77-80
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "complex-interleaved output is not supported in basic variant");
  }
  if (!pair_supported(type_in, type_out)) {
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "No kernel parameters available for selected precision (in %d, out %d)", type_in,
                type_out);
  }
  if (a_mem_order != kRowMajor || b_mem_order != kColMajor) {
    // The reference rejects these layouts when it compiles its kernel at
    // construction (kernels/gemm_kernel_float.cu:20-25); callers match on the
    // name of that failure (test/gemm/mma.cpp:598-627).
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "HIPRTC_ERROR_COMPILATION: GEMM supports only a row-major A matrix and a "
                "col-major B matrix");
  }
  if (B > 0xffffffffu || M > 0x7fffffffu || N > 0x7fffffffu || K > 0x7fffffffu) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "problem size out of range");
  }
  // the kernels address a row with 32-bit byte offsets, also when the pipeline
  // hands them interleaved rows (twice the bytes)
  if (2 * K * (size_t)bits_of(type_in) / 8 > 0xffffffffu) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT,
                "K = %zu: a row of the operands must stay below 2 GiB", K);
  }
  return CCGLIB_OK;
}

void init_gemm(ccglib_gemm *g, size_t B, size_t M, size_t N, size_t K, int device, void *stream,
               int type_in, int type_out, int variant, int c_complex_axis_location,
               int c_mem_order, float alpha_re, float alpha_im, float beta_re, float beta_im) {
  g->B = B;
  g->M = M;
  g->N = N;
  g->K = K;
  g->device = device;
  g->stream = static_cast<hipStream_t>(stream);
  g->type_in = type_in;
  g->type_out = type_out;
  g->variant = variant;
  g->c_axis = c_complex_axis_location;
  g->c_order = c_mem_order;
  g->alpha_re = alpha_re;
  g->alpha_im = alpha_im;
  g->beta_re = beta_re;
  g->beta_im = beta_im;
}

}  // namespace

extern "C" {

const char *ccglib_last_error(void) { return g_last_error.c_str(); }

const char *ccglib_version(void) { return "ccglib-amd 0.2.0 (gfx950)"; }

int ccglib_amd_set_option(int option, size_t value) {
  if (option < 0 || option >= CCGLIB_AMD_OPTION_COUNT) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "unknown option %d", option);
  }
  if (option == CCGLIB_AMD_OPTION_GEMM_BLOCK_TILE && value > 3) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "GEMM_BLOCK_TILE is 0, 1, 2 or 3 (got %zu)", value);
  }
  if (option == CCGLIB_AMD_OPTION_PIPELINE_ROUTE && value > 2) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "PIPELINE_ROUTE is 0, 1 or 2 (got %zu)", value);
  }
  g_options[option] = value;
  return CCGLIB_OK;
}

int ccglib_amd_get_option(int option, size_t *value) {
  if (option < 0 || option >= CCGLIB_AMD_OPTION_COUNT || !value) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "unknown option %d", option);
  }
  *value = g_options[option];
  return CCGLIB_OK;
}

/* ------------------------------- GEMM ---------------------------------- */

int ccglib_gemm_get_dimensions(int type_in, int type_out, int variant, unsigned *m_per_block,
                               unsigned *n_per_block, unsigned *k_chunk) {
  (void)variant;  // as in the reference, both variants report the same tiles
  if (!m_per_block || !n_per_block || !k_chunk) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null output pointer");
  }
  if (!pair_supported(type_in, type_out)) {
    // wording of src/mma/Kernel.cpp:38-40
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "No kernel parameters available for selected precision (in %d, out %d)", type_in,
                type_out);
  }
  *m_per_block = kTileRows;
  *n_per_block = kTileRows;
  *k_chunk = (unsigned)k_per_tile(type_in);
  return CCGLIB_OK;
}

int ccglib_gemm_create(ccglib_gemm_t *gemm, size_t B, size_t M, size_t N, size_t K, int device,
                       void *stream, int type_in, int type_out, int variant,
                       int c_complex_axis_location, int c_mem_order, int a_mem_order,
                       int b_mem_order, float alpha_re, float alpha_im, float beta_re,
                       float beta_im) {
  if (!gemm) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null handle pointer");
  *gemm = nullptr;
  if (int rc = validate_gemm(B, M, N, K, type_in, type_out, variant, c_complex_axis_location,
                             c_mem_order, a_mem_order, b_mem_order)) {
    return rc;
  }
  if (int rc = check_device(device)) return rc;
  ccglib_gemm *g = new (std::nothrow) ccglib_gemm;
  if (!g) return fail(CCGLIB_ERROR_RUNTIME, "out of host memory");
  init_gemm(g, B, M, N, K, device, stream, type_in, type_out, variant, c_complex_axis_location,
            c_mem_order, alpha_re, alpha_im, beta_re, beta_im);
  g->retile_allowed = g_options[CCGLIB_AMD_OPTION_BASIC_RETILE] != 0;
  g->int1_direct = g_options[CCGLIB_AMD_OPTION_INT1_POPCOUNT] == 0;
  g->block_tile = (int)g_options[CCGLIB_AMD_OPTION_GEMM_BLOCK_TILE];
  // Planar rows that direct-to-LDS copies cannot fetch in whole chunks (for 1-bit
  // input: rows of K / 32 words). Re-tiling them costs two bandwidth-bound passes
  // and a copy of A and B; the kernel for the tiled layout then runs several
  // times faster than the ones that load ragged rows through registers.
  // (Operands that are not 16-byte aligned get the same workspace at their first Run.)
  const size_t row_bytes = type_in == kInt1 ? ceil_div(K, 32) * 4 : K * (size_t)bits_of(type_in) / 8;
  if (variant == kBasic && B && M && N && K &&
      (row_bytes % 16 != 0 || g_options[CCGLIB_AMD_OPTION_EXPECT_UNALIGNED] != 0) &&
      (type_in != kInt1 || g->int1_direct)) {
    make_retile_workspace(g);
  }
  *gemm = g;
  return CCGLIB_OK;
}

int ccglib_gemm_run(ccglib_gemm_t g, const void *d_a, const void *d_b, void *d_c) {
  if (!g) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null GEMM handle");
  if (g->B == 0 || g->M == 0 || g->N == 0) return CCGLIB_OK;
  if (!d_a || !d_b || !d_c) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null device pointer");
  GemmParams p;
  fill_gemm_params(g, d_a, d_b, d_c, &p);
  if (g->input_interleaved && ((uintptr_t)d_a % 16 != 0 || (uintptr_t)d_b % 16 != 0)) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT,
                "interleaved pipeline input must be 16-byte aligned");
  }
  if (g->K == 0 && g->variant == kOpt) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "K = 0 has no tiled layout");
  }
  if (g->variant == kOpt && !g->input_interleaved &&
      ((uintptr_t)d_a % 16 != 0 || (uintptr_t)d_b % 16 != 0)) {
    // tiles are copied to LDS in 16-byte pieces (what Transpose writes into
    // hipMalloc'ed memory is aligned far beyond this)
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "tiled operands must be 16-byte aligned");
  }
  DeviceGuard guard(g->device);
  HIP_TRY(guard.status());
  bool retile_now = g->retile;
  if (g->variant == kBasic && g->K && (g->type_in != kInt1 || g->int1_direct)) {
    const size_t row_bytes = g->type_in == kInt1 ? ceil_div(g->K, 32) * 4
                                                 : g->K * (size_t)bits_of(g->type_in) / 8;
    const bool misaligned = (uintptr_t)d_a % 16 != 0 || (uintptr_t)d_b % 16 != 0;
    // Planar operands that are not 16-byte aligned cannot be copied to LDS in
    // place either: the object gets its workspace at the first such Run (the one
    // allocation a Run may make) and keeps it - unless the stream is being
    // captured into a graph, where the kernel that reads such rows through
    // registers runs instead (the option EXPECT_UNALIGNED makes the object
    // allocate at construction).
    if (misaligned && !g->retile.load(std::memory_order_acquire) && !stream_is_capturing(g->stream)) {
      // (two threads may Run one object: only one of them allocates)
      std::lock_guard<std::mutex> lock(g->lazy_lock);
      make_retile_workspace(g);
    }
    retile_now = g->retile.load(std::memory_order_acquire) && (misaligned || row_bytes % 16 != 0);
  }
  if (retile_now) {
    TransposeParams t;
    t.batch = g->B;
    // (1-bit rows are moved as 32-bit words)
    const bool words = (g->type_in == kInt1);
    t.n = words ? ceil_div(g->K, 32) : g->K;
    t.m_chunk = kTileRows;
    t.n_chunk = words ? (size_t)k_per_tile(kInt1) / 32 : (size_t)k_per_tile(g->type_in);
    t.elem_bytes = words ? 4 : bits_of(g->type_in) / 8;
    t.interleaved = 0;
    char *tiled_a = static_cast<char *>(g->workspace), *tiled_b = tiled_a + g->retile_b_offset;
    t.in = d_a;
    t.out = tiled_a;
    t.m = g->M;
    TransposeParams tb = t;
    tb.in = d_b;
    tb.out = tiled_b;
    tb.m = g->N;
    const hipError_t et = launch_transpose_pair(t, tb, g->stream);
    if (et != hipSuccess) return fail_hip(et, "re-tiling of ragged GEMM operands");
    fill_gemm_params(g, tiled_a, tiled_b, d_c, &p);
    p.variant = kOpt;
    p.workspace = nullptr;
    p.workspace_bytes = 0;
  }
  const hipError_t e = (g->type_in == kInt1) ? launch_gemm_int1(p, g->stream)
                                              : launch_gemm_mfma(p, g->stream);
  if (e != hipSuccess) return fail_hip(e, "GEMM kernel launch");
  return CCGLIB_OK;
}

int ccglib_gemm_kernel_name(ccglib_gemm_t g, char *name, size_t size) {
  if (!g || !name || size == 0) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null argument");
  // 16-byte aligned buffers assumed (what Run meets with memory from hipMalloc)
  GemmParams p;
  fill_gemm_params(g, nullptr, nullptr, nullptr, &p);
  const char *what;
  if (g->type_in == kInt1 && !g->int1_direct) {
    what = "complex_gemm_int1, 128x128 block, XOR + population count";
  } else if (g->retile) {
    p.variant = kOpt;
    what = describe_gemm_mfma(p);
  } else if (g->type_in == kInt1 && g->variant == kBasic && (ceil_div(g->K, 32) * 4) % 16 != 0) {
    what = "complex_gemm_int1, 128x128 block, XOR + population count";
  } else {
    what = describe_gemm_mfma(p);
  }
  std::snprintf(name, size, "%s%s", g->retile ? "transpose_vec (re-tiling) + " : "", what);
  return CCGLIB_OK;
}

int ccglib_gemm_destroy(ccglib_gemm_t g) {
  if (g && g->workspace) {
    DeviceGuard guard(g->device);
    (void)hipFree(g->workspace);   // waits for the kernels that still use it
  }
  delete g;
  return CCGLIB_OK;
}

/* ----------------------------- Transpose -------------------------------- */

int ccglib_transpose_create(ccglib_transpose_t *transpose, size_t B, size_t M, size_t N,
                            size_t M_chunk, size_t N_chunk, size_t nr_bits, int device,
                            void *stream, int input_complex_axis_location) {
  if (!transpose) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null handle pointer");
  *transpose = nullptr;
  if (!is_enum01(input_complex_axis_location)) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "enum argument out of range");
  }
  if (nr_bits != 1 && nr_bits != 8 && nr_bits != 16 && nr_bits != 32) {
    // kernels/transpose_kernel.cu:20-32
    return fail(CCGLIB_ERROR_UNSUPPORTED, "NBIT_IN must be 1, 8, 16, 32 (got %zu)", nr_bits);
  }
  if (M_chunk == 0 || N_chunk == 0) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "chunk sizes must be positive");
  }
  if (nr_bits == 1 && (N % 32 != 0 || N_chunk % 32 != 0)) {
    // one-bit samples move as whole 32-bit words (kernels/transpose_kernel.cu:33,57-59)
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "1-bit transpose needs N and N_chunk to be multiples of 32 (got %zu, %zu)", N,
                N_chunk);
  }
  if (int rc = check_device(device)) return rc;
  ccglib_transpose *t = new (std::nothrow) ccglib_transpose;
  if (!t) return fail(CCGLIB_ERROR_RUNTIME, "out of host memory");
  t->B = B;
  t->M = M;
  t->N = N;
  t->M_chunk = M_chunk;
  t->N_chunk = N_chunk;
  t->nr_bits = nr_bits;
  t->device = device;
  t->stream = static_cast<hipStream_t>(stream);
  t->axis = input_complex_axis_location;
  *transpose = t;
  return CCGLIB_OK;
}

static TransposeParams transpose_params(const ccglib_transpose *t, const void *d_input,
                                        void *d_output) {
  TransposeParams p;
  p.in = d_input;
  p.out = d_output;
  p.batch = t->B;
  p.m = t->M;
  p.m_chunk = t->M_chunk;
  if (t->nr_bits == 1) {
    p.elem_bytes = 4;
    p.n = t->N / 32;
    p.n_chunk = t->N_chunk / 32;
  } else {
    p.elem_bytes = (int)(t->nr_bits / 8);
    p.n = t->N;
    p.n_chunk = t->N_chunk;
  }
  p.interleaved = (t->axis == kInterleaved);
  return p;
}

int ccglib_transpose_run(ccglib_transpose_t t, const void *d_input, void *d_output) {
  if (!t) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null transpose handle");
  if (t->B == 0 || t->M == 0 || t->N == 0) return CCGLIB_OK;
  if (!d_input || !d_output) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null device pointer");
  const TransposeParams p = transpose_params(t, d_input, d_output);
  DeviceGuard guard(t->device);
  HIP_TRY(guard.status());
  const hipError_t e = launch_transpose(p, t->stream);
  if (e != hipSuccess) return fail_hip(e, "transpose kernel launch");
  return CCGLIB_OK;
}

int ccglib_transpose_run_pair(ccglib_transpose_t ta, const void *d_input_a, void *d_output_a,
                              ccglib_transpose_t tb, const void *d_input_b, void *d_output_b) {
  if (!ta || !tb) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null transpose handle");
  if (ta->device != tb->device || ta->stream != tb->stream) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT,
                "the two transposes of a pair must share their device and stream");
  }
  const bool empty_a = ta->B == 0 || ta->M == 0 || ta->N == 0;
  const bool empty_b = tb->B == 0 || tb->M == 0 || tb->N == 0;
  if (empty_a || empty_b) {
    const int rc = empty_a ? CCGLIB_OK : ccglib_transpose_run(ta, d_input_a, d_output_a);
    return rc != CCGLIB_OK || empty_b ? rc : ccglib_transpose_run(tb, d_input_b, d_output_b);
  }
  if (!d_input_a || !d_output_a || !d_input_b || !d_output_b) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null device pointer");
  }
  DeviceGuard guard(ta->device);
  HIP_TRY(guard.status());
  const hipError_t e = launch_transpose_pair(transpose_params(ta, d_input_a, d_output_a),
                                             transpose_params(tb, d_input_b, d_output_b), ta->stream);
  if (e != hipSuccess) return fail_hip(e, "transpose kernel launch");
  return CCGLIB_OK;
}

int ccglib_transpose_run_host(ccglib_transpose_t t, const void *h_input, void *d_output) {
  if (!t) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null transpose handle");
  if (!h_input || !d_output) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null pointer");
  const size_t bytes = t->input_bytes();
  if (bytes == 0) return CCGLIB_OK;
  DeviceGuard guard(t->device);
  HIP_TRY(guard.status());
  // stream-ordered staging buffer, as src/transpose/Transpose.cpp:51-56
  void *d_input = nullptr;
  HIP_TRY(hipMallocAsync(&d_input, bytes, t->stream));
  hipError_t e = hipMemcpyAsync(d_input, h_input, bytes, hipMemcpyHostToDevice, t->stream);
  int rc = CCGLIB_OK;
  if (e != hipSuccess) rc = fail_hip(e, "hipMemcpyAsync");
  if (rc == CCGLIB_OK) rc = ccglib_transpose_run(t, d_input, d_output);
  e = hipFreeAsync(d_input, t->stream);
  if (rc == CCGLIB_OK && e != hipSuccess) rc = fail_hip(e, "hipFreeAsync");
  return rc;
}

int ccglib_transpose_destroy(ccglib_transpose_t t) {
  delete t;
  return CCGLIB_OK;
}

/* ------------------------------ Packing --------------------------------- */

int ccglib_packing_create(ccglib_packing_t *packing, size_t N, int direction, int device,
                          void *stream, int input_complex_axis_location) {
  if (!packing) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null handle pointer");
  *packing = nullptr;
  if (!is_enum01(input_complex_axis_location)) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "enum argument out of range");
  }
  if (direction != kForward && direction != kBackward) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "Unknown packing direction");
  }
  if (direction == kBackward && input_complex_axis_location == kInterleaved) {
    // src/packing/Packing.cpp:49-53
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "complex-interleaved input is not supported in unpacking kernel");
  }
  if (direction == kForward && input_complex_axis_location == kInterleaved && N % 2 != 0) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT,
                "complex-interleaved input needs an even number of samples");
  }
  if (int rc = check_device(device)) return rc;
  ccglib_packing *k = new (std::nothrow) ccglib_packing;
  if (!k) return fail(CCGLIB_ERROR_RUNTIME, "out of host memory");
  k->N = N;
  k->direction = direction;
  k->device = device;
  k->axis = input_complex_axis_location;
  k->stream = static_cast<hipStream_t>(stream);
  *packing = k;
  return CCGLIB_OK;
}

int ccglib_packing_run(ccglib_packing_t k, const void *d_input, void *d_output) {
  if (!k) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null packing handle");
  if (k->N == 0) return CCGLIB_OK;
  if (!d_input || !d_output) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null device pointer");
  DeviceGuard guard(k->device);
  HIP_TRY(guard.status());
  hipError_t e;
  if (k->direction == kForward) {
    e = launch_pack_bits(static_cast<const unsigned char *>(d_input),
                         static_cast<unsigned *>(d_output), k->N / k->segments,
                         k->axis == kInterleaved, k->stream, k->segments);
  } else {
    e = launch_unpack_bits(static_cast<const unsigned *>(d_input),
                           static_cast<unsigned char *>(d_output), k->N, k->stream);
  }
  if (e != hipSuccess) return fail_hip(e, "packing kernel launch");
  return CCGLIB_OK;
}

int ccglib_packing_run_host(ccglib_packing_t k, const void *h_input, void *d_output) {
  if (!k) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null packing handle");
  if (!h_input || !d_output) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null pointer");
  // forward: N bytes of samples; backward: ceil(N/32) packed words
  const size_t bytes = (k->direction == kForward) ? k->N : ceil_div(k->N, 32) * 4;
  if (bytes == 0) return CCGLIB_OK;
  DeviceGuard guard(k->device);
  HIP_TRY(guard.status());
  void *d_input = nullptr;
  HIP_TRY(hipMallocAsync(&d_input, bytes, k->stream));
  hipError_t e = hipMemcpyAsync(d_input, h_input, bytes, hipMemcpyHostToDevice, k->stream);
  int rc = CCGLIB_OK;
  if (e != hipSuccess) rc = fail_hip(e, "hipMemcpyAsync");
  if (rc == CCGLIB_OK) rc = ccglib_packing_run(k, d_input, d_output);
  e = hipFreeAsync(d_input, k->stream);
  if (rc == CCGLIB_OK && e != hipSuccess) rc = fail_hip(e, "hipFreeAsync");
  return rc;
}

int ccglib_packing_destroy(ccglib_packing_t k) {
  delete k;
  return CCGLIB_OK;
}

/* ------------------------------ Pipeline -------------------------------- */

}  // extern "C"

namespace {

// Frees what the chunked host path of a pipeline holds.
void destroy_host_lanes(ccglib_pipeline *p) {
  if (!p->caller_ready && !p->lane_stream[0]) return;
  DeviceGuard guard(p->device);
  for (int l = 0; l < ccglib_pipeline::kHostLanes; ++l) {
    if (p->lane_stream[l]) (void)hipStreamSynchronize(p->lane_stream[l]);
  }
  ccglib_pipeline_destroy(p->lane_tail);
  p->lane_tail = nullptr;
  for (int l = 0; l < ccglib_pipeline::kHostLanes; ++l) {
    ccglib_pipeline_destroy(p->lane[l]);
    if (p->lane_a[l]) (void)hipFree(p->lane_a[l]);
    if (p->lane_b[l]) (void)hipFree(p->lane_b[l]);
    if (p->lane_c[l]) (void)hipFree(p->lane_c[l]);
    if (p->lane_stream[l]) (void)hipStreamDestroy(p->lane_stream[l]);
    p->lane[l] = nullptr;
    p->lane_a[l] = p->lane_b[l] = p->lane_c[l] = nullptr;
    p->lane_stream[l] = nullptr;
  }
  if (p->caller_ready) (void)hipEventDestroy(p->caller_ready);
  p->caller_ready = nullptr;
  p->chunk_B = 0;
}

}  // namespace

extern "C" {

int ccglib_pipeline_destroy(ccglib_pipeline_t p) {
  if (!p) return CCGLIB_OK;
  {
    DeviceGuard guard(p->device);
    if (p->d_a_packed) (void)hipFree(p->d_a_packed);
    if (p->d_b_packed) (void)hipFree(p->d_b_packed);
    if (p->d_a_trans) (void)hipFree(p->d_a_trans);
    if (p->d_b_trans) (void)hipFree(p->d_b_trans);
  }
  destroy_host_lanes(p);
  ccglib_pipeline_destroy(p->unfused.load());
  ccglib_packing_destroy(p->pack_a);
  ccglib_packing_destroy(p->pack_b);
  ccglib_transpose_destroy(p->trans_a);
  ccglib_transpose_destroy(p->trans_b);
  ccglib_gemm_destroy(p->gemm);
  delete p;
  return CCGLIB_OK;
}

}  // extern "C"

namespace {

// allow_fused: the GEMM may read interleaved input in place (false for the
// pipeline that stands in for it when the caller's buffers are not aligned).
int pipeline_create(ccglib_pipeline_t *pipeline, size_t B, size_t M, size_t N, size_t K,
                    int device, void *stream, int input_complex_axis_location,
                    int output_complex_axis_location, int a_mem_order, int b_mem_order,
                    int c_mem_order, int input_type, int output_type, int variant,
                    float alpha_re, float alpha_im, float beta_re, float beta_im,
                    bool allow_fused) {
  if (!pipeline) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null handle pointer");
  *pipeline = nullptr;
  if (!is_enum01(input_complex_axis_location) || !is_enum01(variant)) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "enum argument out of range");
  }
  if (variant == kBasic && output_complex_axis_location == kInterleaved) {
    // as the GEMM it wraps (src/mma/GEMM.cpp:77-80)
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "complex-interleaved output is not supported in basic variant");
  }
  ccglib_pipeline *p = new (std::nothrow) ccglib_pipeline;
  if (!p) return fail(CCGLIB_ERROR_RUNTIME, "out of host memory");
  p->B = B;
  p->M = M;
  p->N = N;
  p->K = K;
  p->device = device;
  p->stream = static_cast<hipStream_t>(stream);
  p->type_in = input_type;
  p->type_out = output_type;
  p->c_axis = output_complex_axis_location;
  p->need_copyin_c = (beta_re != 0.0f || beta_im != 0.0f);  // src/pipeline/Pipeline.cpp:138
  p->in_axis = input_complex_axis_location;
  p->a_order = a_mem_order;
  p->b_order = b_mem_order;
  p->c_order = c_mem_order;
  p->variant = variant;
  p->alpha_re = alpha_re;
  p->alpha_im = alpha_im;
  p->beta_re = beta_re;
  p->beta_im = beta_im;
  int rc = CCGLIB_OK;
  const bool packing = (input_type == kInt1);   // src/pipeline/Pipeline.cpp:52
  // Interleaved 8/16-bit input whose rows are whole 16-byte chunks is fed to the
  // GEMM as it is (the kernel de-interleaves in its arithmetic), which saves the
  // two transposes and their intermediate buffers for either variant.
  const size_t in_bits = (size_t)bits_of(input_type);
  // Reading rows in place costs the GEMM a few per cent against reading tiles; the
  // transposes cost two bandwidth-bound passes over A and B and two more launches.
  // The GEMM's work grows with M N and the transposes' with M + N, so reading in
  // place is the smaller price while
  //   M N / (M + N)  <  T (1 + c / (B K (M + N)))
  // with the break-even T of large problems and c the launches' fixed cost in
  // operand elements. Measured (python -m ccglib_amd.tuning.pipeline_crossover at
  // K = 256, 1024, 4096): 16-bit interleaved rows T = 3800 where the 192 x 256 kernel
  // reads them (planar C, no beta, alpha only with fp32 C, M and N multiples of 64, K of 32) and
  // 2800 elsewhere, 8-bit interleaved rows T = 2700, c = 1e7 for both.
  const double mn_over_sum = (M + N) ? (double)M * (double)N / (double)(M + N) : 0.0;
  const double operand_elements = (double)B * (double)K * (double)(M + N);
  // (option PIPELINE_ROUTE: 1 in place wherever possible, 2 never for the opt variant)
  const size_t route = g_options[CCGLIB_AMD_OPTION_PIPELINE_ROUTE];
  auto below = [&](double break_even, double fixed_cost) {
    return route == 1 ||
           (route == 0 && operand_elements > 0 &&
            mn_over_sum < break_even * (1.0 + fixed_cost / operand_elements));
  };
  const bool wide_rows = in_bits == 16 && output_complex_axis_location == kPlanar &&
                         beta_re == 0.f && beta_im == 0.f &&
                         M % 64 == 0 && N % 64 == 0 && K % 32 == 0 && K >= 64;
  const bool fused = allow_fused && !packing && input_complex_axis_location == kInterleaved && K > 0 &&
                     (in_bits == 8 || in_bits == 16) && (2 * K * in_bits / 8) % 16 == 0 &&
                     (variant == kBasic ||
                      below(in_bits == 8 ? 2700.0 : wide_rows ? 3800.0 : 2800.0, 1.0e7));
  // Planar input of the opt variant whose rows are whole 16-byte chunks: the GEMM
  // can read the rows in place as well (the basic variant's loader, same
  // arithmetic and K order as on tiles). That costs the GEMM more (the tiled
  // operands have the 192 x 256 kernel), so the break-even lies lower: T = 1500,
  // c = 6e6 (measured on squares; long rectangles at small K would still gain up to
  // 8 % from reading in place beyond it).
  const bool planar_in_place = allow_fused && !packing && variant == kOpt &&
                               input_complex_axis_location == kPlanar &&
                               output_complex_axis_location == kPlanar && K > 0 &&
                               (in_bits == 8 || in_bits == 16 || in_bits == 32) &&
                               (K * in_bits / 8) % 16 == 0 && below(1500.0, 6.0e6);
  // The reference transposes for the opt variant only (:53) and hands interleaved
  // input of the basic variant to a kernel that reads it as planar. Here such
  // input is always de-interleaved: in the GEMM's loader (fused) or, where that
  // cannot take the rows, by the transposes, with the tiled kernel behind them.
  const bool basic_needs_tiles = !packing && variant == kBasic &&
                                 input_complex_axis_location == kInterleaved && !fused;
  const bool transposing = ((variant == kOpt) && !fused && !planar_in_place) || basic_needs_tiles;
  // Packing moves the real samples of every batch in front of its imaginary ones
  // (below), so what follows it sees planar data. (The reference hands
  // input_complex_axis_location to its Transpose here too,
  // src/pipeline/Pipeline.cpp:78-84, which then de-interleaves packed words.)
  const int axis_after_packing = packing ? kPlanar : input_complex_axis_location;
  do {
    if (packing && B && M && N && K % 32 == 0) {
      // (K in whole words, as the packed layout of the other route needs it.)
      // The 1-bit GEMM multiplies operands expanded to 4-bit values; when its
      // workspace holds the whole problem the expansion is done straight from
      // the caller's bytes and the reference's pack and transpose steps
      // (src/pipeline/Pipeline.cpp:111-121) with their buffers are not needed.
      rc = ccglib_gemm_create(&p->gemm, B, M, N, K, device, stream, input_type, output_type,
                              kOpt, output_complex_axis_location, c_mem_order, a_mem_order,
                              b_mem_order, alpha_re, alpha_im, beta_re, beta_im);
      if (rc != CCGLIB_OK) break;
      if (p->gemm->int1_direct && !p->gemm->workspace) {
        // room for the 1-bit tiles that the caller's bytes are packed into (the
        // GEMM object owns and frees it)
        const size_t bytes = gemm_int1_tiles_bytes(B, M, N, K);
        DeviceGuard guard(device);
        if (bytes && bytes <= kInt1TilesCap && guard.status() == hipSuccess &&
            hipMalloc(&p->gemm->workspace, bytes) == hipSuccess) {
          p->gemm->workspace_bytes = bytes;
        } else {
          p->gemm->workspace = nullptr;
          (void)hipGetLastError();
        }
      }
      GemmParams probe;
      fill_gemm_params(p->gemm, nullptr, nullptr, nullptr, &probe);
      if (gemm_int1_can_take_bytes(probe)) {
        p->int1_direct = true;
        // (interleaved bytes are de-interleaved while they are packed into tiles)
        p->gemm->input_interleaved = (input_complex_axis_location == kInterleaved);
        break;
      }
      ccglib_gemm_destroy(p->gemm);
      p->gemm = nullptr;
    }
    if (packing) {
      const size_t num_a = B * 2 * M * K, num_b = B * 2 * N * K;  // :57-58
      if ((rc = ccglib_packing_create(&p->pack_a, num_a, kForward, device, stream,
                                      input_complex_axis_location)))
        break;
      if ((rc = ccglib_packing_create(&p->pack_b, num_b, kForward, device, stream,
                                      input_complex_axis_location)))
        break;
      if (input_complex_axis_location == kInterleaved && B > 1) {
        // The reference packs the whole buffer as one (kernels/packing_kernel.cu:15-22:
        // all real bits of all batches, then all imaginary bits), which is the
        // planar layout [B][2][rows][K] that the next steps read only for B = 1.
        // Here every batch is packed on its own; that needs whole words per plane.
        if ((M * K) % 32 != 0 || (N * K) % 32 != 0) {
          rc = fail(CCGLIB_ERROR_UNSUPPORTED,
                    "1-bit interleaved input with several batches needs M*K and N*K to be "
                    "multiples of 32 (got M=%zu N=%zu K=%zu)", M, N, K);
          break;
        }
        p->pack_a->segments = B;
        p->pack_b->segments = B;
      }
      DeviceGuard guard(device);
      hipError_t e = hipMalloc(&p->d_a_packed, ceil_div(num_a, 32) * 4 + 16);
      if (e == hipSuccess) e = hipMalloc(&p->d_b_packed, ceil_div(num_b, 32) * 4 + 16);
      if (e != hipSuccess) {
        rc = fail_hip(e, "hipMalloc(packed scratch)");
        break;
      }
    }
    unsigned mb = 0, nb = 0, kc = 0;
    if ((rc = ccglib_gemm_get_dimensions(input_type, output_type, variant, &mb, &nb, &kc))) break;
    if (transposing) {
      const size_t bits = (size_t)bits_of(input_type);
      if ((rc = ccglib_transpose_create(&p->trans_a, B, M, K, mb, kc, bits, device, stream,
                                        axis_after_packing)))  // :78-84
        break;
      if ((rc = ccglib_transpose_create(&p->trans_b, B, N, K, nb, kc, bits, device, stream,
                                        axis_after_packing)))
        break;
      // padded to whole tiles (:87-96)
      const size_t mp = ceil_div(M, mb) * mb, np = ceil_div(N, nb) * nb, kp = ceil_div(K, kc) * kc;
      DeviceGuard guard(device);
      hipError_t e = hipMalloc(&p->d_a_trans, B * 2 * mp * kp * bits / 8 + 16);
      if (e == hipSuccess) e = hipMalloc(&p->d_b_trans, B * 2 * np * kp * bits / 8 + 16);
      if (e != hipSuccess) {
        rc = fail_hip(e, "hipMalloc(transposed scratch)");
        break;
      }
    }
    rc = ccglib_gemm_create(&p->gemm, B, M, N, K, device, stream, input_type, output_type,
                            (fused || basic_needs_tiles) ? (int)kOpt
                            : planar_in_place            ? (int)kBasic
                                                         : variant,
                            output_complex_axis_location,
                            c_mem_order, a_mem_order, b_mem_order, alpha_re, alpha_im, beta_re,
                            beta_im);  // :102-105
    if (rc == CCGLIB_OK) p->gemm->input_interleaved = fused;
    p->fused = fused || planar_in_place;   // (both need 16-byte aligned rows at Run)
    if (rc == CCGLIB_OK && p->fused && allow_fused &&
        g_options[CCGLIB_AMD_OPTION_EXPECT_UNALIGNED] != 0) {
      // the pipeline with transposes that takes over for unaligned buffers, now
      // rather than at the first Run that meets them
      ccglib_pipeline *stand_by = nullptr;
      rc = pipeline_create(&stand_by, B, M, N, K, device, stream, input_complex_axis_location,
                           output_complex_axis_location, a_mem_order, b_mem_order, c_mem_order,
                           input_type, output_type, variant, alpha_re, alpha_im, beta_re, beta_im,
                           false);
      p->unfused.store(stand_by, std::memory_order_release);
    }
  } while (false);
  if (rc != CCGLIB_OK) {
    const std::string keep = g_last_error;
    ccglib_pipeline_destroy(p);
    g_last_error = keep;
    return rc;
  }
  *pipeline = p;
  return CCGLIB_OK;
}

}  // namespace

extern "C" {

int ccglib_pipeline_reads_in_place(ccglib_pipeline_t p, int *in_place) {
  if (!p || !in_place) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null argument");
  *in_place = p->fused ? 1 : 0;
  return CCGLIB_OK;
}

int ccglib_pipeline_create(ccglib_pipeline_t *pipeline, size_t B, size_t M, size_t N, size_t K,
                           int device, void *stream, int input_complex_axis_location,
                           int output_complex_axis_location, int a_mem_order, int b_mem_order,
                           int c_mem_order, int input_type, int output_type, int variant,
                           float alpha_re, float alpha_im, float beta_re, float beta_im) {
  return pipeline_create(pipeline, B, M, N, K, device, stream, input_complex_axis_location,
                         output_complex_axis_location, a_mem_order, b_mem_order, c_mem_order,
                         input_type, output_type, variant, alpha_re, alpha_im, beta_re, beta_im,
                         true);
}

int ccglib_pipeline_run(ccglib_pipeline_t p, const void *d_a, const void *d_b, void *d_c) {
  if (!p) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null pipeline handle");
  int rc;
  const void *a = d_a, *b = d_b;
  if (p->fused && d_a && d_b && ((uintptr_t)d_a % 16 != 0 || (uintptr_t)d_b % 16 != 0)) {
    // The GEMM's copies to LDS need 16-byte aligned rows; the transposes take any
    // element-aligned address. The pipeline that runs them is created here, once
    // (the one allocation a device Run may make), and kept.
    ccglib_pipeline *stand_by = p->unfused.load(std::memory_order_acquire);
    if (!stand_by) {
      if (stream_is_capturing(p->stream)) {
        return fail(CCGLIB_ERROR_INVALID_ARGUMENT,
                    "pipeline input is not 16-byte aligned: the pipeline with transposes that takes "
                    "such buffers cannot be allocated while the stream is being captured (run once "
                    "before the capture, or create the pipeline with the option EXPECT_UNALIGNED)");
      }
      // (two threads may Run one object: only one of them creates the stand-by)
      std::lock_guard<std::mutex> lock(p->lazy_lock);
      stand_by = p->unfused.load(std::memory_order_acquire);
      if (!stand_by) {
        rc = pipeline_create(&stand_by, p->B, p->M, p->N, p->K, p->device, p->stream, p->in_axis,
                             p->c_axis, p->a_order, p->b_order, p->c_order, p->type_in, p->type_out,
                             p->variant, p->alpha_re, p->alpha_im, p->beta_re, p->beta_im, false);
        if (rc != CCGLIB_OK) return rc;
        p->unfused.store(stand_by, std::memory_order_release);
      }
    }
    return ccglib_pipeline_run(stand_by, d_a, d_b, d_c);
  }
  if (p->int1_direct) {
    ccglib_gemm *g = p->gemm;
    if (!d_a || !d_b || !d_c) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null device pointer");
    GemmParams q;
    fill_gemm_params(g, d_a, d_b, d_c, &q);
    DeviceGuard guard(g->device);
    HIP_TRY(guard.status());
    const hipError_t e = launch_gemm_int1_from_bytes(q, g->stream);
    if (e != hipSuccess) return fail_hip(e, "1-bit pipeline launch");
    return CCGLIB_OK;
  }
  if (p->pack_a) {  // src/pipeline/Pipeline.cpp:111-114
    if ((rc = ccglib_packing_run(p->pack_a, a, p->d_a_packed))) return rc;
    if ((rc = ccglib_packing_run(p->pack_b, b, p->d_b_packed))) return rc;
    a = p->d_a_packed;
    b = p->d_b_packed;
  }
  if (p->trans_a) {  // :116-121
    if ((rc = ccglib_transpose_run_pair(p->trans_a, a, p->d_a_trans, p->trans_b, b, p->d_b_trans))) {
      return rc;
    }
    a = p->d_a_trans;
    b = p->d_b_trans;
  }
  return ccglib_gemm_run(p->gemm, a, b, d_c);  // :123-125
}

}  // extern "C"

namespace {

// Batches per chunk of the overlapped host path, or 0 when the problem is run
// in one piece: a single batch or less than 8 MiB to move. Chunks of about
// 32 MiB keep copies in both directions in flight at once (sizes from 8 to
// 64 MiB measured the same, 128 MiB 7 % slower);
// the option CCGLIB_AMD_OPTION_HOST_CHUNK_BYTES overrides that size.
size_t host_chunk_batches(const ccglib_pipeline *p, size_t bytes_total) {
  if (p->B < 2) return 0;
  size_t target = (size_t)32 << 20;
  if (g_options[CCGLIB_AMD_OPTION_HOST_CHUNK_BYTES]) {
    target = g_options[CCGLIB_AMD_OPTION_HOST_CHUNK_BYTES];
  } else if (bytes_total < ((size_t)8 << 20)) {
    return 0;
  }
  const size_t per_batch = std::max<size_t>(1, bytes_total / p->B);
  const size_t chunk = std::max<size_t>(1, target / per_batch);
  return chunk < p->B ? chunk : ceil_div(p->B, 2);   // the last chunk may hold fewer batches
}

// Creates the lanes of the chunked host path; an object whose chunk size
// changed (the option) gets new ones.
int make_host_lanes(ccglib_pipeline *p, size_t chunk, size_t bytes_a, size_t bytes_b,
                    size_t bytes_c) {
  constexpr int kLanes = ccglib_pipeline::kHostLanes;
  if (p->chunk_B == chunk) return CCGLIB_OK;
  destroy_host_lanes(p);
  const size_t chunks = ceil_div(p->B, chunk), tail = p->B - (chunks - 1) * chunk;
  hipError_t e = hipEventCreateWithFlags(&p->caller_ready, hipEventDisableTiming);
  for (int l = 0; l < kLanes && e == hipSuccess; ++l) {
    e = hipStreamCreateWithFlags(&p->lane_stream[l], hipStreamNonBlocking);
    if (e == hipSuccess) e = hipMalloc(&p->lane_a[l], bytes_a / p->B * chunk + 16);
    if (e == hipSuccess) e = hipMalloc(&p->lane_b[l], bytes_b / p->B * chunk + 16);
    if (e == hipSuccess) e = hipMalloc(&p->lane_c[l], bytes_c / p->B * chunk + 16);
  }
  if (e != hipSuccess) {
    destroy_host_lanes(p);
    return fail_hip(e, "pipeline host lanes");
  }
  for (int l = 0; l <= kLanes; ++l) {
    if (l == kLanes && tail == chunk) break;
    // the last chunk is number chunks - 1 and runs on that lane's stream
    const int rc = ccglib_pipeline_create(
        l < kLanes ? &p->lane[l] : &p->lane_tail, l < kLanes ? chunk : tail, p->M, p->N, p->K,
        p->device, p->lane_stream[l < kLanes ? l : (int)((chunks - 1) % kLanes)], p->in_axis,
        p->c_axis, p->a_order, p->b_order, p->c_order, p->type_in, p->type_out, p->variant,
        p->alpha_re, p->alpha_im, p->beta_re, p->beta_im);
    if (rc != CCGLIB_OK) {
      const std::string keep = g_last_error;
      destroy_host_lanes(p);
      g_last_error = keep;
      return rc;
    }
  }
  p->chunk_B = chunk;
  return CCGLIB_OK;
}

}  // namespace

extern "C" {

int ccglib_pipeline_run_host(ccglib_pipeline_t p, const void *h_a, const void *h_b, void *h_c) {
  if (!p) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null pipeline handle");
  if (!h_a || !h_b || !h_c) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null host pointer");
  // input is one byte per sample when packing happens inside the pipeline
  const size_t in_bits = (p->type_in == kInt1) ? 8 : (size_t)bits_of(p->type_in);
  const size_t bytes_a = p->B * 2 * p->M * p->K * in_bits / 8;
  const size_t bytes_b = p->B * 2 * p->N * p->K * in_bits / 8;
  const size_t bytes_c = p->B * 2 * p->M * p->N * (size_t)bits_of(p->type_out) / 8;
  if (bytes_c == 0) return CCGLIB_OK;
  DeviceGuard guard(p->device);
  HIP_TRY(guard.status());
  int rc = CCGLIB_OK;
  hipError_t e = hipSuccess;

  const size_t chunk = host_chunk_batches(p, bytes_a + bytes_b + bytes_c);
  if (chunk) {
    // Chunks of whole batches go round the lanes; within a lane the
    // stream keeps copy in -> kernels -> copy out of one chunk, and the next use
    // of the lane's buffers, in order. With pinned host memory every call below
    // returns at once and the lanes run against each other (the copies of one
    // with the kernels and the opposite copies of the other); with pageable
    // memory the copies block the host, and the result is the same.
    if ((rc = make_host_lanes(p, chunk, bytes_a, bytes_b, bytes_c))) return rc;
    const size_t chunks = ceil_div(p->B, chunk);
    const size_t batch_a = bytes_a / p->B, batch_b = bytes_b / p->B, batch_c = bytes_c / p->B;
    // work the caller queued on its stream comes first
    e = hipEventRecord(p->caller_ready, p->stream);
    for (int l = 0; l < ccglib_pipeline::kHostLanes && e == hipSuccess; ++l) {
      e = hipStreamWaitEvent(p->lane_stream[l], p->caller_ready, 0);
    }
    for (size_t i = 0; i < chunks && e == hipSuccess && rc == CCGLIB_OK; ++i) {
      const int l = (int)(i % ccglib_pipeline::kHostLanes);
      hipStream_t s = p->lane_stream[l];
      const size_t batches = std::min(chunk, p->B - i * chunk);
      ccglib_pipeline *lane = batches == chunk ? p->lane[l] : p->lane_tail;
      const size_t ca = batches * batch_a, cb = batches * batch_b, cc = batches * batch_c;
      const char *ha = static_cast<const char *>(h_a) + i * chunk * batch_a;
      const char *hb = static_cast<const char *>(h_b) + i * chunk * batch_b;
      char *hc = static_cast<char *>(h_c) + i * chunk * batch_c;
      if (ca) e = hipMemcpyAsync(p->lane_a[l], ha, ca, hipMemcpyHostToDevice, s);
      if (e == hipSuccess && cb) e = hipMemcpyAsync(p->lane_b[l], hb, cb, hipMemcpyHostToDevice, s);
      if (e == hipSuccess && p->need_copyin_c) {
        e = hipMemcpyAsync(p->lane_c[l], hc, cc, hipMemcpyHostToDevice, s);
      }
      if (e != hipSuccess) break;
      rc = ccglib_pipeline_run(lane, p->lane_a[l], p->lane_b[l], p->lane_c[l]);
      if (rc == CCGLIB_OK) e = hipMemcpyAsync(hc, p->lane_c[l], cc, hipMemcpyDeviceToHost, s);
    }
    // the host Run returns with c complete (src/pipeline/Pipeline.cpp:175)
    for (int l = 0; l < ccglib_pipeline::kHostLanes; ++l) {
      const hipError_t es = hipStreamSynchronize(p->lane_stream[l]);
      if (e == hipSuccess) e = es;
    }
    if (rc == CCGLIB_OK && e != hipSuccess) rc = fail_hip(e, "pipeline host run in chunks");
    return rc;
  }

  void *d_a = nullptr, *d_b = nullptr, *d_c = nullptr;
  e = hipMalloc(&d_a, bytes_a ? bytes_a : 16);
  if (e == hipSuccess) e = hipMalloc(&d_b, bytes_b ? bytes_b : 16);
  if (e == hipSuccess) e = hipMalloc(&d_c, bytes_c);
  if (e == hipSuccess && bytes_a) e = hipMemcpyAsync(d_a, h_a, bytes_a, hipMemcpyHostToDevice, p->stream);
  if (e == hipSuccess && bytes_b) e = hipMemcpyAsync(d_b, h_b, bytes_b, hipMemcpyHostToDevice, p->stream);
  if (e == hipSuccess) {
    // src/pipeline/Pipeline.cpp:168-172
    e = p->need_copyin_c ? hipMemcpyAsync(d_c, h_c, bytes_c, hipMemcpyHostToDevice, p->stream)
                         : hipMemsetAsync(d_c, 0, bytes_c, p->stream);
  }
  if (e != hipSuccess) rc = fail_hip(e, "pipeline host staging");
  if (rc == CCGLIB_OK) rc = ccglib_pipeline_run(p, d_a, d_b, d_c);
  if (rc == CCGLIB_OK) {
    e = hipMemcpyAsync(h_c, d_c, bytes_c, hipMemcpyDeviceToHost, p->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(p->stream);
    if (e != hipSuccess) rc = fail_hip(e, "pipeline copy back");
  } else {
    (void)hipStreamSynchronize(p->stream);
  }
  if (d_a) (void)hipFree(d_a);
  if (d_b) (void)hipFree(d_b);
  if (d_c) (void)hipFree(d_c);
  return rc;
}

}  // extern "C"

/* ---------------------- Pipeline without allocations --------------------- */

namespace {

// Scratch of the stateless pipeline call: the tiled (and, for 1-bit
// interleaved input, packed) copies of A and B that a pipeline object keeps in
// memory it allocates. One array per GPU, held from the moment the library's
// code is loaded there until the process ends; every call on that GPU uses it.
constexpr size_t kStaticScratchBytes = CCGLIB_AMD_STATIC_SCRATCH_BYTES;
static_assert(kStaticScratchBytes >= 256 && kStaticScratchBytes % 256 == 0,
              "CCGLIB_AMD_STATIC_SCRATCH_BYTES must be a positive multiple of 256");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on each GPU. In host code the array's name is only
// a handle for hipGetSymbolAddress, never an address a kernel could use.
constexpr int kMaxScratchDevices = 64;
unsigned char *g_scratch_ptr[kMaxScratchDevices] = {};
std::atomic<bool> g_scratch_ready[kMaxScratchDevices];

// First call on a device: checks the device and looks up its copy of the array
// (with that device current).
int static_scratch(int device, unsigned char **ptr) {
  if (device < 0 || device >= kMaxScratchDevices) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "device ordinal %d out of range", device);
  }
  if (!g_scratch_ready[device].load(std::memory_order_acquire)) {
    if (int rc = check_device(device)) return rc;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail_hip(e, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[device] = static_cast<unsigned char *>(p);
    g_scratch_ready[device].store(true, std::memory_order_release);
  }
  *ptr = g_scratch_ptr[device];
  return CCGLIB_OK;
}

size_t round_up_256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

extern "C" {

size_t ccglib_amd_static_scratch_bytes(void) { return kStaticScratchBytes; }

int ccglib_pipeline_run_static(size_t B, size_t M, size_t N, size_t K, int device, void *stream,
                               int input_complex_axis_location,
                               int output_complex_axis_location, int a_mem_order,
                               int b_mem_order, int c_mem_order, int input_type, int output_type,
                               int variant, float alpha_re, float alpha_im, float beta_re,
                               float beta_im, const void *d_a, const void *d_b, void *d_c) {
  if (!is_enum01(input_complex_axis_location)) {
    return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "enum argument out of range");
  }
  if (int rc = validate_gemm(B, M, N, K, input_type, output_type, variant,
                             output_complex_axis_location, c_mem_order, a_mem_order,
                             b_mem_order)) {
    return rc;
  }
  if (B == 0 || M == 0 || N == 0) return CCGLIB_OK;
  if (K == 0) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "K = 0 has no tiled layout");
  if (!d_a || !d_b || !d_c) return fail(CCGLIB_ERROR_INVALID_ARGUMENT, "null device pointer");
  const bool int1 = (input_type == kInt1);
  if (int1 && K % 32 != 0) {
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "1-bit input needs K to be a multiple of 32 here (got %zu)", K);
  }
  DeviceGuard guard(device);
  HIP_TRY(guard.status());
  unsigned char *ws = nullptr;
  if (int rc = static_scratch(device, &ws)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);

  // The GEMM always reads tiled copies here (what the opt variant reads; for the
  // basic variant the same numbers, as the kernels only differ in their loaders).
  ccglib_gemm g;
  init_gemm(&g, B, M, N, K, device, stream, input_type, output_type, kOpt,
            output_complex_axis_location, c_mem_order, alpha_re, alpha_im, beta_re, beta_im);
  size_t tiled_a = 0, tiled_b = 0;
  tiled_bytes(&g, &tiled_a, &tiled_b);
  const bool pack_first = int1 && input_complex_axis_location == kInterleaved;
  if (int1 && tiled_a + tiled_b <= kStaticScratchBytes) {
    // one byte per sample, planar or (re, im) pairs: packed straight into 1-bit
    // tiles (A's and B's back to back), then multiplied
    g.workspace = ws;
    g.workspace_bytes = tiled_a + tiled_b;
    g.input_interleaved = pack_first;
    GemmParams q;
    fill_gemm_params(&g, d_a, d_b, d_c, &q);
    q.int1_direct = 1;
    if (gemm_int1_can_take_bytes(q)) {
      const hipError_t e = launch_gemm_int1_from_bytes(q, s);
      if (e != hipSuccess) return fail_hip(e, "1-bit pipeline launch");
      return CCGLIB_OK;
    }
    if (!pack_first) {
      return fail(CCGLIB_ERROR_UNSUPPORTED, "ccglib_pipeline_run_static: 1-bit problem out of range");
    }
    g.workspace = nullptr;
    g.workspace_bytes = 0;
    g.input_interleaved = false;
  }
  const size_t packed_a = pack_first ? round_up_256(B * 2 * M * K / 8) : 0;
  const size_t packed_b = pack_first ? round_up_256(B * 2 * N * K / 8) : 0;
  const size_t need = round_up_256(tiled_a) + round_up_256(tiled_b) + packed_a + packed_b;
  if (need > kStaticScratchBytes) {
    return fail(CCGLIB_ERROR_UNSUPPORTED,
                "ccglib_pipeline_run_static: the tiled copies of A and B take %zu bytes, the "
                "static scratch holds %zu; use a pipeline object for this size", need,
                kStaticScratchBytes);
  }
  unsigned char *ws_a = ws, *ws_b = ws + round_up_256(tiled_a);
  unsigned char *ws_pa = ws_b + round_up_256(tiled_b), *ws_pb = ws_pa + packed_a;

  const void *src_a = d_a, *src_b = d_b;
  int axis = input_complex_axis_location;
  if (pack_first) {
    // every batch packed on its own: real bits, then imaginary bits (planar)
    if ((M * K) % 32 != 0 || (N * K) % 32 != 0) {
      return fail(CCGLIB_ERROR_UNSUPPORTED, "1-bit interleaved input needs M*K and N*K to be multiples of 32");
    }
    hipError_t e = launch_pack_bits(static_cast<const unsigned char *>(d_a),
                                    reinterpret_cast<unsigned *>(ws_pa), 2 * M * K, 1, s, B);
    if (e == hipSuccess) {
      e = launch_pack_bits(static_cast<const unsigned char *>(d_b),
                           reinterpret_cast<unsigned *>(ws_pb), 2 * N * K, 1, s, B);
    }
    if (e != hipSuccess) return fail_hip(e, "packing kernel launch");
    src_a = ws_pa;
    src_b = ws_pb;
    axis = kPlanar;
  }
  TransposeParams t;
  t.batch = B;
  t.n = int1 ? K / 32 : K;
  t.m_chunk = kTileRows;
  t.n_chunk = int1 ? (size_t)k_per_tile(kInt1) / 32 : (size_t)k_per_tile(input_type);
  t.elem_bytes = int1 ? 4 : bits_of(input_type) / 8;
  t.interleaved = (axis == kInterleaved);
  t.in = src_a;
  t.out = ws_a;
  t.m = M;
  TransposeParams tb = t;
  tb.in = src_b;
  tb.out = ws_b;
  tb.m = N;
  hipError_t e = launch_transpose_pair(t, tb, s);
  if (e != hipSuccess) return fail_hip(e, "transpose kernel launch");
  GemmParams p;
  fill_gemm_params(&g, ws_a, ws_b, d_c, &p);
  e = int1 ? launch_gemm_int1(p, s) : launch_gemm_mfma(p, s);
  if (e != hipSuccess) return fail_hip(e, "GEMM kernel launch");
  return CCGLIB_OK;
}

}  // extern "C"
