/*
 * gern_pipelines.h - C ABI over the fused pipelines of the hot path.
 *
 * Each *_create call does what the `main()` of the corresponding reference
 * application does with Gern's C++ API: declare the data structures, compose
 * the annotated functions with Tile / Reduce / Global, hand the program to a
 * Runner and compile it (here: HIP for gfx950 through hiprtc).  Each *_run
 * call is Runner::evaluate on caller-owned DEVICE buffers; it is asynchronous
 * on the given HIP stream (NULL = default stream).
 *
 * Plain pointers and sizes only.  Every function returns 0 on success; on
 * failure the calling thread's message is read with gern_pipelines_last_error().
 * A failure to find a GPU is an error, never a fallback.
 *
 * Threads: different pipelines may be created and run from different threads;
 * one pipeline handle is for one thread at a time (a run records which of its
 * kernels it used, and sets the stream of its Runner).  The reference's Runner
 * is not thread-safe either (src/codegen/runner.cpp, src/codegen/codegen_printer.cpp:7: static state).
 */
#ifndef GERN_PIPELINES_H
#define GERN_PIPELINES_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gern_pipeline_s *gern_pipeline;

enum {
    /* Generate the source and compile it for gfx950, but do not load it: the
     * pipeline can be inspected (gern_pipeline_source) on a machine without a
     * GPU and cannot be run. */
    GERN_PIPELINE_COMPILE_ONLY = 1,
    /* Launch workgroups in plain blockIdx order (no XCD-aware renumbering). */
    GERN_PIPELINE_NO_XCD_REMAP = 2,
    /* GEMM only: C = A * B (C is written, never read) instead of C += A * B. */
    GERN_PIPELINE_GEMM_OVERWRITE = 4,
    /* GEMM only: build and run only the kernel that takes every shape (fp32:
     * vector-ALU FMAs; bf16: the four-wavefront kernel that stages through
     * registers), also for shapes the direct-to-LDS matrix-core kernels take. */
    GERN_PIPELINE_GEMM_GENERAL_ONLY = 8,
    /* Blur only: every tile stores exactly its own tile_cols columns, also
     * when tile_cols would allow windows moved to whole 128-byte lines. */
    GERN_PIPELINE_BLUR_PLAIN_STORES = 16,
    /* QK^T softmax only: sixteen whole rows of S per workgroup also for head
     * dimensions that the 256 x 256 tile kernel takes (multiples of 64). */
    GERN_PIPELINE_QK_ROW_BLOCKS = 32,
    /* Workgroup order in which the 32 workgroups that run on one XCD at a
     * time take a block of 4 x 8 tiles (grids that are a multiple of 4 x 8
     * workgroups and of 256 in all; others keep the plain order).  The
     * matrix-core GEMM kernels use it unless GERN_PIPELINE_NO_XCD_REMAP asks
     * for the plain order. */
    GERN_PIPELINE_XCD_TILE_BLOCKS = 64
};

/* Device memory through which the workgroups of the QK^T softmax tile kernel
 * exchange row statistics: 256 bytes of state, then 8 bytes per (row, padded
 * to a multiple of 256; block of 256 keys, padded to a multiple of sixteen
 * blocks).  Enough for M = 16384 rows at 4096 keys. */
#define GERN_QK_SCRATCH_BYTES ((size_t)2 * 1024 * 1024 + 256)

/* Fused separable box-blur chain.  `pattern` is a string over {'x','y'},
 * applied left to right ("xy" = horizontal then vertical, "xyx" = the
 * three-stage chain); every stage has `stride` taps of weight 1/stride and
 * produces the valid region only.  One wavefront produces one
 * tile_rows x tile_cols output tile; tile_cols + (#x stages)*(stride-1) must
 * not exceed 256.  waves_per_block wavefronts (side by side along the
 * columns) form a workgroup.  When tile_cols is a multiple of 32 and
 * tile_cols + 28 + (#x stages)*(stride-1) <= 256 (224 for up to two 3-tap x
 * stages), each wavefront moves the columns it stores, row by row, to whole
 * 128-byte lines of the result: the same elements are written, each once, by
 * possibly a neighbouring wavefront, and no partial line reaches memory.
 * Composes what apps/blur/blur.cpp:31-73 composes (there: blur_x, blur_y). */
int gern_blur_chain_create(const char *pattern, int64_t stride, int64_t tile_rows, int64_t tile_cols,
                           int waves_per_block, int flags, gern_pipeline *out);
/* in is rows x cols (row stride ld_in); out is
 * (rows - ny*(stride-1)) x (cols - nx*(stride-1)) (row stride ld_out).
 * Runner::evaluate of the program above, apps/blur/blur.cpp:85-88. */
int gern_blur_chain_run(gern_pipeline p, const float *in, int64_t rows, int64_t cols, int64_t ld_in,
                        float *out, int64_t ld_out, void *stream);

/* Row-wise numerically stable softmax over matrices with exactly `ncol`
 * columns (1 .. GERN_SOFTMAX_MAX_COLS): max, x - max, exp, sum, divide, fused;
 * a workgroup holds rows_per_wave rows in registers, in one wavefront or, for
 * rows of 1024 columns and more that divide into 256-column chunks, spread
 * over 2, 4 or 8 wavefronts; rows wider than 8192 columns, of any width, are
 * spread over 4, 8 or 16 wavefronts (rows_per_wave must then be 1).  The
 * reference's row reductions likewise share a row among `stride` threads and
 * meet in shared memory (apps/common/impl/impl.h:80-188).  The five calls are
 * the reference's softmax gernels, apps/common/annot/functions.h:9-173. */
#define GERN_SOFTMAX_MAX_COLS 65536
int gern_softmax_create(int64_t ncol, int64_t rows_per_wave, int flags, gern_pipeline *out);
int gern_softmax_run(gern_pipeline p, const float *in, float *out, int64_t rows, int64_t ld,
                     void *stream);

/* Dense GEMM C += A * B (or C = A * B with GERN_PIPELINE_GEMM_OVERWRITE),
 * row-major, A is M x K, B is K x N, C is M x N fp32.
 * variant 0: fp32 inputs and fp32 arithmetic.  With a 16-byte aligned A the
 *            product runs on the fp32 matrix instruction
 *            (v_mfma_f32_32x32x2_f32), operands loaded straight into LDS; when
 *            K is not a multiple of 4, the last K % 4 columns of A are added by
 *            a second launch of the vector-ALU kernel, which also takes K < 4
 *            and unaligned A.  Both sum each dot product in fp32; the order of
 *            the additions differs.
 * variant 1: bf16 inputs (bit patterns), fp32 accumulation on MFMA; needs
 *            K % 8 == 0 and N % 2 == 0, A 16-byte and B 4-byte aligned.  All
 *            such shapes take the kernel that loads both operands straight
 *            into LDS (row pitches up to 2^20 elements).
 * Composes Tile(i)(Tile(j)(Reduce(k)(matrix_multiply))) as
 * gernels/mm/kernel_3.cu:61-75 does. */
int gern_gemm_create(int variant, int flags, gern_pipeline *out);
int gern_gemm_run(gern_pipeline p, const void *A, const void *B, float *C, int64_t M, int64_t N,
                  int64_t K, void *stream);

/* S = softmax_rows(scale * Q K^T): Q is M x D and K is N x D in bf16 (bit
 * patterns), S is M x N fp32; MFMA tiles feed an in-register row reduction.
 * Q and K 16-byte aligned.
 * head_dim = D (a multiple of 32, at most 256); max_keys bounds N (a multiple
 * of 256, at most GERN_QK_MAX_KEYS when D is a multiple of 64, else 4096).
 * D a multiple of 64: one workgroup per 256 x 256 tile of S; the workgroups
 * of a row block exchange their row maxima and sums through
 * GERN_QK_SCRATCH_BYTES of device memory that create allocates (the only device
 * memory this library allocates) and the tiles wait in registers meanwhile.
 * M x N must fit that memory (8 bytes per row and 256 keys, keys rounded up
 * to a multiple of 4096: M up to 16384 at 4096 keys, 8192 at 8192 keys, 1024
 * at 65536); runs of ONE pipeline must not overlap in time
 * (launch them on one stream, or order the streams).  A wavefront that waits
 * in vain for the rest of its row block (after a second or so: the launch
 * shares the GPU with something that keeps its partners from starting) stores
 * NaN in its rows, and so does a row whose logits exceed 22 000 in magnitude;
 * the run still returns 0 (it is asynchronous), and gern_pipeline_faults
 * reports both afterwards.  The environment variable GERN_QK_SPIN_LIMIT (a
 * whole number from 0 to 2^31 - 1; anything else makes the run fail) sets the
 * number of polls before a wavefront gives up.
 * Other D (or GERN_PIPELINE_QK_ROW_BLOCKS): sixteen whole rows of S per
 * workgroup, logits in accumulators, no device memory besides Q, K and S.
 * No counterpart in the reference (it has no bf16 and no matrix-core path);
 * the softmax stages are those of apps/common/annot/functions.h:9-173. */
#define GERN_QK_MAX_KEYS 65536
int gern_qk_softmax_create(int64_t head_dim, int64_t max_keys, int flags, gern_pipeline *out);
int gern_qk_softmax_run(gern_pipeline p, const uint16_t *Q, const uint16_t *K, float *S, int64_t M,
                        int64_t N, float scale, void *stream);

/* User-level GEMM schedules, C += A * B on square fp32 matrices of
 * GERN_GEMM_SCHEDULE_SIZE rows (row-major, dense): the compositions of the
 * reference's gernels/mm/kernel_3.cu:61-75 (block tiles staged through LDS one
 * float per lane, 4 x 4 outputs per thread), kernel_6.cu:61-74 (staged 16
 * bytes per lane) and kernel_10.cu:108-131 (block -> wavefront -> lane tiling,
 * operands staged by loads that write LDS directly, register copies per
 * lane), with tile sizes for 64-lane wavefronts, over the scalar
 * matrix_multiply gernel.  They exist to run and time schedules written at
 * the level of Gern's API (gernels/mm/bench.cu:72-89 times such a kernel);
 * the tuned GEMM is gern_gemm_create.  schedule: 3, 6 or 10. */
#define GERN_GEMM_SCHEDULE_SIZE 1024
int gern_gemm_schedule_create(int schedule, int flags, gern_pipeline *out);
int gern_gemm_schedule_run(gern_pipeline p, const float *A, const float *B, float *C, void *stream);

/* gern_qk_softmax_run with the exchange memory taken from a device array of
 * this library (GERN_QK_SCRATCH_BYTES, one copy per GPU, held from the first
 * gern_qk_softmax_create of a tile-kernel pipeline on that GPU until the
 * process ends) instead of the pipeline's own allocation: the call allocates
 * nothing on the device and looks nothing up (gern_qk_softmax_create found the
 * array, which is when the runtime loads this library's device code), for
 * callers that must not allocate (a stream under HIP graph capture, a serving
 * loop that forbids it).
 * Same arguments, same limits (M x N must fit GERN_QK_SCRATCH_BYTES), same
 * results.  All pipelines of a process share the array of a GPU: calls of this
 * function that overlap in time on one GPU race (launch them on one stream,
 * or order the streams); calls of gern_qk_softmax_run do not touch it.  A
 * pipeline built with another launch-tag period than the library's default
 * (an experiment option) is refused: all users of the array must agree on it.
 * No counterpart in the reference. */
int gern_qk_softmax_run_no_alloc(gern_pipeline p, const uint16_t *Q, const uint16_t *K, float *S,
                                 int64_t M, int64_t N, float scale, void *stream);

/* What the kernels of the pipeline could not do and could only signal in
 * their results, since a run returns before they execute.  Waits for the
 * device, then stores in *count, and clears, the sum of
 *   - wavefronts of the QK^T softmax tile kernel that gave up waiting for
 *     the rest of their row block (their rows of S hold NaN),
 *   - (row, block of 256 keys) pairs of that kernel whose largest logit is
 *     beyond +-22 000 or not a number (those rows of S hold NaN),
 *     both over all runs of this pipeline since the last call (runs through
 *     gern_qk_softmax_run_no_alloc count in one place per GPU, shared with
 *     the other pipelines that use it),
 *   - requests that the LDS allocator of a gern_gemm_schedule pipeline could
 *     not meet (not cleared: a count over the life of the pipeline).
 * 0 means every result is what the pipeline computes.  Takes the place of the
 * reference's check after each launch,
 * include/gern/codegen/helpers/check_last_error.h:7-18. */
int gern_pipeline_faults(gern_pipeline p, int64_t *count);

/* The generated device source (owned by the pipeline, valid until destroy).
 * A pipeline that holds more than one kernel (the GEMMs) reports the one its
 * last run used; before any run, the faster one. */
const char *gern_pipeline_source(gern_pipeline p);
/* The name expression of the instantiated kernel, e.g. "function_7<252, 8, 3>". */
const char *gern_pipeline_kernel_name(gern_pipeline p);
/* Waits for the device (a run may still be in flight), unloads the pipeline's
 * code objects and frees the handle. */
int gern_pipeline_destroy(gern_pipeline p);

size_t gern_pipelines_last_error(char *buf, size_t buf_size);

#ifdef __cplusplus
}
#endif
#endif
