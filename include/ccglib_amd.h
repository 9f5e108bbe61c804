/*
 * C ABI of the MI355X (gfx950) complex-GEMM library: plain pointers and sizes,
 * opaque handles, integer status codes. These entry points are what the C++
 * classes of the ccglib API bind to (include/ccglib/...): each section names the
 * reference interface it stands in for, as file:line in the reference tree.
 *
 * Conventions
 *  - Every function returns CCGLIB_OK (0) or a non-zero status; the text of the
 *    last failure on the calling thread is returned by ccglib_last_error().
 *  - `device` is a HIP device ordinal; `stream` is a hipStream_t passed as
 *    void* (NULL = the default stream). All run functions only enqueue work on
 *    that stream and return; they never synchronise, allocate or free, except
 *    the *_run_host variants, which stage the host buffer through a
 *    stream-ordered temporary.
 *  - Pointers given to run functions are device pointers unless the name says
 *    host. The library never owns caller buffers.
 *  - Enum arguments are plain ints holding the values of the reference enums
 *    (repeated below as CCGLIB_* constants).
 *  - Objects are not thread-safe; use one per thread or serialise calls.
 */
#ifndef CCGLIB_AMD_H_
#define CCGLIB_AMD_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CCGLIB_API __attribute__((visibility("default")))

/* status codes */
enum {
  CCGLIB_OK = 0,
  CCGLIB_ERROR_INVALID_ARGUMENT = 1, /* bad handle, null pointer, bad enum   */
  CCGLIB_ERROR_UNSUPPORTED = 2,      /* valid request the library cannot do  */
  CCGLIB_ERROR_RUNTIME = 3           /* a HIP call failed                    */
};

/* ValueType: include/ccglib/common/value_type.h:14-22 */
enum {
  CCGLIB_INT1 = 0,
  CCGLIB_INT32 = 1,
  CCGLIB_BFLOAT16 = 2,
  CCGLIB_FLOAT8E4M3 = 3,
  CCGLIB_FLOAT8E5M2 = 4,
  CCGLIB_FLOAT16 = 5,
  CCGLIB_FLOAT32 = 6
};
/* ComplexAxisLocation: include/ccglib/common/complex_order.h:12 */
enum { CCGLIB_COMPLEX_PLANAR = 0, CCGLIB_COMPLEX_INTERLEAVED = 1 };
/* Direction: include/ccglib/common/direction.h:6 */
enum { CCGLIB_FORWARD = 0, CCGLIB_BACKWARD = 1 };
/* MemOrder: include/ccglib/gemm/mem_order.h:6 */
enum { CCGLIB_ROW_MAJOR = 0, CCGLIB_COL_MAJOR = 1 };
/* Variant: include/ccglib/gemm/variant.h:6 */
enum { CCGLIB_BASIC = 0, CCGLIB_OPT = 1 };

typedef struct ccglib_gemm *ccglib_gemm_t;
typedef struct ccglib_transpose *ccglib_transpose_t;
typedef struct ccglib_packing *ccglib_packing_t;
typedef struct ccglib_pipeline *ccglib_pipeline_t;

/* Text of the last error raised on this thread ("" if none). */
CCGLIB_API const char *ccglib_last_error(void);
/* Library version string. */
CCGLIB_API const char *ccglib_version(void);

/* ------------------------------------------------------------------------
 * Process-wide options. No counterpart in the reference (whose only such
 * channel is its JIT macros, src/mma/GEMM.cpp:140-214): they select code paths
 * that produce the same results, for tests and for tuning. An option is read
 * when an object is created (HOST_CHUNK_BYTES: at every host Run); setting
 * one is not synchronised with other threads.
 *   INT1_POPCOUNT    0 (default): the 1-bit GEMM runs on the matrix cores (fp4
 *                    MFMA on +-1 values, exact); 1: XOR + population count on
 *                    the vector ALUs, which is otherwise only the fallback.
 *   BASIC_RETILE     1 (default): a basic-variant GEMM whose planar rows are not
 *                    whole 16-byte chunks, or whose operands are not 16-byte
 *                    aligned, owns a tiled copy of A and B and re-tiles into it
 *                    at every Run; 0: it reads such rows in place through
 *                    registers (several times slower, no extra memory).
 *   HOST_CHUNK_BYTES 0 (default): ccglib_pipeline_run_host moves jobs of 8 MiB
 *                    or more in chunks of whole batches of about 32 MiB; any
 *                    other value: chunks of about that many bytes, whatever
 *                    the size of the job.
 *   GEMM_BLOCK_TILE  0 (default): GEMMs on tiled or whole-chunk planar
 *                    operands use 256 x 128 block tiles, 128 x 128 ones when
 *                    the larger would leave compute units idle (small
 *                    problems), or 192 x 256 ones (16-bit tiled input, planar C
 *                    without beta, M and N multiples of 64, K of more
 *                    than 32) when those fill the compute units well enough;
 *                    1: always 256 x 128; 2: always 128 x 128; 3: 192 x 256
 *                    wherever that kernel applies, else as 0. The 192 x 256
 *                    block also serves 16-bit interleaved rows read in place
 *                    (the pipeline) when K is a multiple of 32.
 *   EXPECT_UNALIGNED 0 (default): a basic-variant GEMM that meets operands that
 *                    are not 16-byte aligned allocates its tiled copies at that
 *                    Run, and a pipeline that reads rows in place creates the
 *                    pipeline with transposes that takes over for such buffers
 *                    at that Run (never while the stream is being captured
 *                    into a graph: the GEMM then reads the rows through
 *                    registers, the pipeline reports an error); 1: both are
 *                    allocated when the object is created, and no device Run
 *                    allocates.
 *   PIPELINE_ROUTE   0 (default): an opt-variant pipeline whose input rows are
 *                    whole 16-byte chunks lets the GEMM read them in place
 *                    where that is faster than transposing them into tiles
 *                    first (small M N / (M + N); the break-even points are
 *                    measured ones), and transposes otherwise; 1: in place
 *                    wherever the GEMM can; 2: always through the transposes.
 *                    ccglib_pipeline_reads_in_place tells which one an object
 *                    took.
 * ---------------------------------------------------------------------- */
enum {
  CCGLIB_AMD_OPTION_INT1_POPCOUNT = 0,
  CCGLIB_AMD_OPTION_BASIC_RETILE = 1,
  CCGLIB_AMD_OPTION_HOST_CHUNK_BYTES = 2,
  CCGLIB_AMD_OPTION_GEMM_BLOCK_TILE = 3,
  CCGLIB_AMD_OPTION_EXPECT_UNALIGNED = 4,
  CCGLIB_AMD_OPTION_PIPELINE_ROUTE = 5,
  CCGLIB_AMD_OPTION_COUNT = 6
};
CCGLIB_API int ccglib_amd_set_option(int option, size_t value);
CCGLIB_API int ccglib_amd_get_option(int option, size_t *value);

/* ------------------------------------------------------------------------
 * Complex GEMM  C[b] = alpha * A[b] * B[b]^T + beta * C[b]
 * Replaces ccglib::mma::GEMM: constructor include/ccglib/gemm/mma.h:42-49
 * (src/mma/GEMM.cpp:243-254), Run :50 (src/mma/GEMM.cpp:263-268),
 * GetDimensions :39-40 (src/mma/GEMM.cpp:270-275).
 *
 * Layouts (kernels/type_selector.h:224-241, kernels/gemm_kernel_float.cu:28-33):
 *   basic: A [B][2][M][K], B [B][2][N][K] (K in 32-bit words for 1-bit input)
 *   opt:   A [B][Mp/Mb][Kp/Kc][2][Mb][Kc], B likewise with Nb: the output of
 *          the transpose below with the chunk sizes of get_dimensions
 *   C:     planar [B][2][M][N] (row major) / [B][2][N][M] (column major);
 *          interleaved [B][M][N][2] / [B][N][M][2] (opt variant only)
 * Supported (type_in -> type_out): float16->float32|float16,
 * bfloat16->float32|bfloat16, float32->float32|float16|bfloat16,
 * float8e4m3->float32, float8e5m2->float32, int1->int32 (the reference's
 * matrix, kernels/type_selector.h:65-212). Accumulation is float32 (int32 for
 * 1-bit input).
 * a_order must be row major and b_order column major (as in the reference,
 * where anything else fails to compile: kernels/gemm_kernel_float.cu:20-25);
 * the error text keeps the token HIPRTC_ERROR_COMPILATION that the
 * reference's callers match on (test/gemm/mma.cpp:598-627).
 * 1-bit input: K must be a multiple of 32; alpha and beta are truncated to
 * integers (src/reference/GEMM.cpp:202-205).
 * C is read only when beta != 0.
 * K whose interleaved row (2 * K * bits / 8 bytes) does not fit 32 bits is
 * refused. Operands should be 16-byte aligned: basic-variant operands that are
 * not (or whose rows are not whole 16-byte chunks) are re-tiled into a
 * workspace the object owns (allocated at creation for such K, at the first
 * such Run for such pointers; see CCGLIB_AMD_OPTION_BASIC_RETILE); opt-variant
 * operands that are not are refused by Run.
 * ---------------------------------------------------------------------- */
CCGLIB_API int ccglib_gemm_create(ccglib_gemm_t *gemm, size_t B, size_t M,
                                  size_t N, size_t K, int device, void *stream,
                                  int type_in, int type_out, int variant,
                                  int c_complex_axis_location, int c_mem_order,
                                  int a_mem_order, int b_mem_order,
                                  float alpha_re, float alpha_im, float beta_re,
                                  float beta_im);
/* Argument order (a, b, c) as in GEMM::Run. */
CCGLIB_API int ccglib_gemm_run(ccglib_gemm_t gemm, const void *d_a,
                               const void *d_b, void *d_c);
/* Which kernel Run launches for 16-byte aligned buffers, in words (kernel
 * function, block tile, operand layout). No counterpart in the reference, whose
 * one kernel per precision is fixed by its parameter tables (src/mma/Kernel*.cpp);
 * here the choice depends on the problem size, and benchmark output names it. */
CCGLIB_API int ccglib_gemm_kernel_name(ccglib_gemm_t gemm, char *name, size_t size);
CCGLIB_API int ccglib_gemm_destroy(ccglib_gemm_t gemm);
/* (m_per_block, n_per_block, k_chunk): the chunk sizes of the opt layout. */
CCGLIB_API int ccglib_gemm_get_dimensions(int type_in, int type_out,
                                          int variant, unsigned *m_per_block,
                                          unsigned *n_per_block,
                                          unsigned *k_chunk);

/* ------------------------------------------------------------------------
 * Transpose into the tiled layout of the opt GEMM.
 * Replaces ccglib::transpose::Transpose: constructor
 * include/ccglib/transpose/transpose.h:26-29
 * (src/transpose/Transpose.cpp:131-141), Run(device) :31
 * (src/transpose/Transpose.cpp:160-164), Run(host) :30 (a no-op in the
 * reference, src/transpose/Transpose.cpp:147-154; here it does the work).
 *   in  [B][2][M][N] (planar) or [B][M][N][2] (interleaved)
 *   out [B][Mp/Mc][Np/Nc][2][Mc][Nc], zero where m >= M or n >= N
 * nr_bits is 1, 8, 16 or 32; for 1 bit N and N_chunk count samples and must
 * be multiples of 32 (whole 32-bit words move).
 * ---------------------------------------------------------------------- */
CCGLIB_API int ccglib_transpose_create(ccglib_transpose_t *transpose, size_t B,
                                       size_t M, size_t N, size_t M_chunk,
                                       size_t N_chunk, size_t nr_bits,
                                       int device, void *stream,
                                       int input_complex_axis_location);
CCGLIB_API int ccglib_transpose_run(ccglib_transpose_t transpose,
                                    const void *d_input, void *d_output);
CCGLIB_API int ccglib_transpose_run_host(ccglib_transpose_t transpose,
                                         const void *h_input, void *d_output);
/* Both operands of one GEMM: the same as ccglib_transpose_run on each, in one
 * kernel launch where the two have the same batch size, row length N, N_chunk,
 * width and input layout and one has at most a quarter of the other's rows
 * (otherwise in two: operands of similar size measured 1-3 % faster one after
 * the other). No counterpart in the reference,
 * whose pipeline launches one transpose per operand
 * (src/pipeline/Pipeline.cpp:116-121); a small operand no longer pays for a
 * launch, ramp-up and tail of its own. Both objects must have been created
 * for the same device and stream. */
CCGLIB_API int ccglib_transpose_run_pair(ccglib_transpose_t transpose_a,
                                         const void *d_input_a, void *d_output_a,
                                         ccglib_transpose_t transpose_b,
                                         const void *d_input_b, void *d_output_b);
CCGLIB_API int ccglib_transpose_destroy(ccglib_transpose_t transpose);

/* ------------------------------------------------------------------------
 * Bit packing: N one-byte samples <-> N bits, LSB first in 32-bit words.
 * Replaces ccglib::packing::Packing: constructor
 * include/ccglib/packing/packing.h:35-38 (src/packing/Packing.cpp:136-141),
 * Run(device) :40 (src/packing/Packing.cpp:162-166), Run(host) :39
 * (src/packing/Packing.cpp:152-156).
 * forward: byte != 0 -> bit 1; interleaved input (re,im pairs) is packed as all
 * real bits followed by all imaginary bits (kernels/packing_kernel.cu:15-22).
 * backward: bits -> bytes of 0/1, planar only (create fails otherwise, as
 * src/packing/Packing.cpp:49-53). The packed buffer holds ceil(N/32) words.
 * ---------------------------------------------------------------------- */
CCGLIB_API int ccglib_packing_create(ccglib_packing_t *packing, size_t N,
                                     int direction, int device, void *stream,
                                     int input_complex_axis_location);
CCGLIB_API int ccglib_packing_run(ccglib_packing_t packing,
                                  const void *d_input, void *d_output);
CCGLIB_API int ccglib_packing_run_host(ccglib_packing_t packing,
                                       const void *h_input, void *d_output);
CCGLIB_API int ccglib_packing_destroy(ccglib_packing_t packing);

/* ------------------------------------------------------------------------
 * Pipeline: [pack] -> [transpose] -> GEMM with scratch buffers owned by the
 * object. Replaces ccglib::pipeline::Pipeline: constructor
 * include/ccglib/pipeline/pipeline.h:44-53 (src/pipeline/Pipeline.cpp:145-160),
 * Run(device) :54 (src/pipeline/Pipeline.cpp:183-188), Run(host) :41
 * (src/pipeline/Pipeline.cpp:162-176).
 * 1-bit input is one byte per sample and is packed first (interleaved input:
 * every batch on its own, real bits then imaginary bits; the reference packs
 * the whole buffer as one, kernels/packing_kernel.cu:15-22, which is the same
 * for B = 1. With K a multiple of 32 the bytes go straight into the GEMM's
 * 1-bit tiles; otherwise, and with CCGLIB_AMD_OPTION_INT1_POPCOUNT, through a
 * packed buffer, which for interleaved input and B > 1 needs M*K and N*K to be
 * multiples of 32); the
 * opt variant transposes A and B first. 8- and 16-bit interleaved input whose
 * rows are whole 16-byte chunks is read by the GEMM in place instead (no
 * transposes), and so is planar input of the opt variant with such rows when
 * the problem is small enough for the transposes to cost more than they save;
 * if a Run then gets pointers that are not 16-byte aligned, the
 * object builds the pipeline with transposes at that Run and uses it for such
 * calls. Argument order follows the reference constructor.
 * run_host copies a, b (and c when beta != 0) to the device, runs, copies c
 * back and returns when c is complete; sizes are those of the layouts above.
 * Jobs of 8 MiB or more with several batches move in chunks of whole batches
 * over two internal streams (ordered after the work already queued on the
 * object's stream), so that with page-locked host buffers the copies in, the
 * kernels and the copies out overlap; the result is the same either way.
 * ---------------------------------------------------------------------- */
CCGLIB_API int ccglib_pipeline_create(
    ccglib_pipeline_t *pipeline, size_t B, size_t M, size_t N, size_t K,
    int device, void *stream, int input_complex_axis_location,
    int output_complex_axis_location, int a_mem_order, int b_mem_order,
    int c_mem_order, int input_type, int output_type, int variant,
    float alpha_re, float alpha_im, float beta_re, float beta_im);
CCGLIB_API int ccglib_pipeline_run(ccglib_pipeline_t pipeline, const void *d_a,
                                   const void *d_b, void *d_c);
CCGLIB_API int ccglib_pipeline_run_host(ccglib_pipeline_t pipeline,
                                        const void *h_a, const void *h_b,
                                        void *h_c);
/* Whether the object's GEMM reads the caller's rows in place (1) or the tiles
 * that its transposes write (0); see the option PIPELINE_ROUTE. No counterpart
 * in the reference, which always transposes for the opt variant
 * (src/pipeline/Pipeline.cpp:53, :78-93). */
CCGLIB_API int ccglib_pipeline_reads_in_place(ccglib_pipeline_t pipeline, int *in_place);
CCGLIB_API int ccglib_pipeline_destroy(ccglib_pipeline_t pipeline);

/* ------------------------------------------------------------------------
 * The pipeline as one stateless call that allocates nothing.
 * No counterpart in the reference. It is for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc. ccglib_pipeline_create allocates the scratch of its
 * object (the packed and transposed copies of A and B); this call does the
 * work of create + run + destroy with that scratch in a static device array
 * of CCGLIB_AMD_STATIC_SCRATCH_BYTES, which every GPU the library's code is
 * loaded on holds until the process ends. It calls no hipMalloc / hipFree (nor
 * their stream-ordered forms) and creates no host objects. (The HIP runtime
 * loads a code object on a GPU when something in it is first used there: the
 * array comes to exist, and its bytes leave the device's free memory, at the
 * first call on that GPU, which therefore belongs before a graph capture. No
 * later call moves the device's free memory.)
 *   - Arguments as ccglib_pipeline_create followed by those of
 *     ccglib_pipeline_run; only enqueues on `stream`.
 *   - Route: [1-bit interleaved input: pack each batch] -> transpose A and B
 *     into the tiled layout (1-bit planar input: bytes packed straight into
 *     1-bit tiles) -> GEMM on the tiles, whatever the variant. The process-wide
 *     options do not apply.
 *   - The tiled copies (rows padded to 128, K to the chunk of get_dimensions)
 *     plus the packed copies must fit the array; otherwise
 *     CCGLIB_ERROR_UNSUPPORTED and nothing is enqueued. K must be positive
 *     (1-bit input: a multiple of 32).
 *   - All calls on one GPU share the array: calls whose kernels may overlap
 *     (different streams, no dependency) race. Calls on one stream are safe.
 *   - What fits the default of 32 MiB, with M', N' the rows padded to 128 and
 *     K' padded to the chunk: B (M' + N') K' <= 8 Mi (2^23) elements for 16-bit
 *     input, 16 Mi for fp8, 4 Mi for float32, 128 Mi samples for 1-bit planar
 *     input and about 64 Mi for 1-bit interleaved input (whose packed copies live
 *     in the array too). E.g. 16-bit: B = 16 of 256 x 256 x 1024, or one
 *     1024 x 1024 x 4096.
 *   - The size is a build option: compile the library with
 *     -DCCGLIB_AMD_STATIC_SCRATCH_BYTES=<bytes> (a multiple of 256;
 *     ccglib_amd/build.py reads the environment variable of the same name).
 *     ccglib_amd_static_scratch_bytes() returns what the loaded library was
 *     built with, which is the figure that binds - not this header's default.
 * ---------------------------------------------------------------------- */
#ifndef CCGLIB_AMD_STATIC_SCRATCH_BYTES
#define CCGLIB_AMD_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
#endif
CCGLIB_API size_t ccglib_amd_static_scratch_bytes(void);
CCGLIB_API int ccglib_pipeline_run_static(
    size_t B, size_t M, size_t N, size_t K, int device, void *stream,
    int input_complex_axis_location, int output_complex_axis_location,
    int a_mem_order, int b_mem_order, int c_mem_order, int input_type,
    int output_type, int variant, float alpha_re, float alpha_im, float beta_re,
    float beta_im, const void *d_a, const void *d_b, void *d_c);

#ifdef __cplusplus
}
#endif
#endif /* CCGLIB_AMD_H_ */
