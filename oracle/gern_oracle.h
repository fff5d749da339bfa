/*
 * CPU oracle for the fused-kernel hot path (blur chain, row softmax, GEMM,
 * QK^T -> softmax).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the CPU-baseline leg of the benchmark may link or load it.
 * The HIP path never calls into this library.
 *
 * Every function restates, in plain scalar C, the arithmetic that the
 * reference executes on its CPU path; the reference file:line that fixes the
 * operation order is cited next to each definition in gern_oracle.c.
 *
 * Pinning status (what checks each function before it is trusted):
 *   oracle_blur_x / oracle_blur_y / oracle_blur_chain
 *       - closed form of the reference's own blur test (ascending input,
 *         apps/blur/blur.cpp:96-108): X->Y output(i,j) == in(i+1,j+1)
 *       - golden vectors written by the reference library's CPU lowering of
 *         the same composed pipeline (tests/golden/)
 *       - brute force on tiny inputs, constant-image invariant
 *   oracle_softmax_rows
 *       - golden vectors from the reference's CPU gernels
 *         (test/library/matrix/impl/cpu-matrix.h:134-194, with x - max)
 *       - rows sum to 1, shift invariance, constant row == 1/N,
 *         torch.softmax cross-check
 *   oracle_gemm_f32
 *       - reference known-answer tests (test/test-cpu-mm.cpp: ascending 4x4
 *         and 10x10 against impl::matrix_multiply), identity / permutation
 *         matrices, fp64 cross-check
 *   oracle_gemm_bf16_f32acc, oracle_qk_softmax
 *       - nothing in the reference uses bf16; pinned by exact small-integer
 *         products, fp64 cross-check and by composition of the two pinned
 *         pieces above (gemm + softmax)
 *   oracle_mt19937_u32
 *       - the 10000th output of std::mt19937 with the default seed is
 *         4123659995 (ISO C++ [rand.predef]); numpy RandomState raw words
 */
#ifndef GERN_ORACLE_H
#define GERN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- portable seeded inputs ------------------------------------------- */
void oracle_mt19937_u32(uint32_t seed, uint32_t *out, size_t n);
/* u = (word >> 8) * 2^-24 in [0,1); value = lo + (hi - lo) * u (fp32). */
void oracle_fill_uniform(float *out, size_t n, uint32_t seed, float lo, float hi);
/* Box-Muller in fp64 on pairs of words, cast to fp32. */
void oracle_fill_normal(float *out, size_t n, uint32_t seed, double mean, double sigma);
/* value = linear index (row-major), as MatrixCPU::ascending(). */
void oracle_fill_ascending(float *out, int64_t rows, int64_t cols, int64_t lda);

/* ---- bf16 helpers ------------------------------------------------------ */
uint16_t oracle_f32_to_bf16_rne(float x);
float oracle_bf16_to_f32(uint16_t b);
void oracle_round_to_bf16(const float *in, uint16_t *out_bits, float *out_f32, size_t n);

/* ---- blur --------------------------------------------------------------- */
/* out(i,j) = (0 + in(i,j) + ... + in(i,j+stride-1)) / stride, out is
 * rows x (cols_in - stride + 1). */
void oracle_blur_x(const float *in, int64_t rows, int64_t cols_in, int64_t lda_in,
                   float *out, int64_t lda_out, int stride);
/* out(i,j) = (0 + in(i,j) + ... + in(i+stride-1,j)) / stride, out is
 * (rows_in - stride + 1) x cols. */
void oracle_blur_y(const float *in, int64_t rows_in, int64_t cols, int64_t lda_in,
                   float *out, int64_t lda_out, int stride);
/* pattern is a string over {'x','y'}, applied left to right, e.g. "xy",
 * "xyx".  out must hold (rows - ny*(stride-1)) x (cols - nx*(stride-1)).
 * Returns 0, or -1 on a bad pattern / shape. */
int oracle_blur_chain(const float *in, int64_t rows, int64_t cols, const char *pattern,
                      int stride, float *out);
/* Same chain executed the way the fused pipeline executes it: per output
 * tile, intermediates sized by the inferred halos. */
int oracle_blur_chain_tiled(const float *in, int64_t rows, int64_t cols, const char *pattern,
                            int stride, int64_t tile_rows, int64_t tile_cols, float *out);

/* ---- softmax ------------------------------------------------------------ */
void oracle_softmax_rows(const float *in, int64_t rows, int64_t cols, int64_t lda,
                         float *out, int64_t ldo);

/* ---- GEMM --------------------------------------------------------------- */
/* C(i,j) += sum_k A(i,k)*B(k,j), the inner sum accumulated in a local fp32
 * starting from 0, products and sums rounded separately (no FMA). */
void oracle_gemm_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K);
/* Rows [i0,i1) only (for sampled parity at full size). */
void oracle_gemm_f32_rows(const float *A, const float *B, float *C, int64_t M, int64_t N,
                          int64_t K, int64_t i0, int64_t i1);
/* bf16 inputs (bit patterns), fp32 products and accumulation. */
void oracle_gemm_bf16_f32acc(const uint16_t *A, const uint16_t *B, float *C, int64_t M,
                             int64_t N, int64_t K);
void oracle_gemm_bf16_f32acc_rows(const uint16_t *A, const uint16_t *B, float *C, int64_t M,
                                  int64_t N, int64_t K, int64_t i0, int64_t i1);
/* S = softmax_rows(scale * Q K^T), Q is M x D, K is N x D (both bf16 bits,
 * row-major), S is M x N fp32.  Rows [i0,i1) only. */
void oracle_qk_softmax_rows(const uint16_t *Q, const uint16_t *Kmat, float *S, int64_t M,
                            int64_t N, int64_t D, float scale, int64_t i0, int64_t i1);

/* ---- division by a constant ------------------------------------------- */
/* q = x * RN(1/d); r = fma(-d, q, x); q' = fma(r, RN(1/d), q), then the IEEE
 * result for zero / infinite / NaN dividends (what v_div_fixup_f32 does).  The
 * HIP blur gernels divide this way when a tile holds tiny values or zeros;
 * this restates it with libm fmaf. */
float oracle_div_const_fma(float x, float d);
/* Number of fp32 bit patterns in [lo_bits, hi_bits) for which
 * oracle_div_const_fma(x,d) differs bitwise from x / d (NaNs skipped). */
uint64_t oracle_div_const_mismatches(float d, uint32_t lo_bits, uint32_t hi_bits);

/* ---- division of a tap sum by the tap count ---------------------------- */
/* What the HIP blur gernels compute for (0 + taps...) / d from the tap sum s
 * formed WITHOUT the leading zero (gernels/prelude.h, quotient_of_sum): for
 * d == 3 two FMAs with 1/3 split in two floats, for powers of two one FMA.
 * This restates it with libm fmaf so that it can be checked on the host. */
float oracle_quotient_of_sum(float s, float d);
/* Bit patterns in [lo_bits, hi_bits) for which oracle_quotient_of_sum(x, d)
 * differs bitwise from the reference's (0.0f + x) / d (NaNs skipped), the
 * largest difference in ulp, and the range of |x| where they occur. */
uint64_t oracle_quotient_mismatches(float d, uint32_t lo_bits, uint32_t hi_bits, uint32_t *max_ulp,
                                    float *min_abs, float *max_abs);

/* ---- comparison helpers ------------------------------------------------ */
/* Largest ulp distance between two fp32 arrays (both finite). */
uint32_t oracle_max_ulp(const float *a, const float *b, size_t n);

#ifdef __cplusplus
}
#endif
#endif
