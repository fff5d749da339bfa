/*
 * CPU oracle (test infrastructure only; see gern_oracle.h).
 *
 * Compile WITHOUT -ffast-math and without FMA contraction
 * (-ffp-contract=off): the reference's CPU path is built by the host
 * compiler for baseline x86-64, where a*b+c is two roundings.
 */
#include "gern_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* MT19937, the generator the reference seeds its random fills with    */
/* (test/library/matrix/impl/cpu-matrix.h:71-81 uses std::mt19937).    */
/* Only the raw 32-bit words are used, because the mapping of words to */
/* floats by std::uniform_real_distribution is implementation-defined. */
/* ------------------------------------------------------------------ */
typedef struct {
    uint32_t mt[624];
    int idx;
} mt_state;

static void mt_seed(mt_state *s, uint32_t seed) {
    s->mt[0] = seed;
    for (int i = 1; i < 624; i++) {
        s->mt[i] = 1812433253u * (s->mt[i - 1] ^ (s->mt[i - 1] >> 30)) + (uint32_t)i;
    }
    s->idx = 624;
}

static uint32_t mt_next(mt_state *s) {
    if (s->idx >= 624) {
        for (int k = 0; k < 624; k++) {
            uint32_t y = (s->mt[k] & 0x80000000u) | (s->mt[(k + 1) % 624] & 0x7fffffffu);
            uint32_t v = s->mt[(k + 397) % 624] ^ (y >> 1);
            if (y & 1u) v ^= 0x9908b0dfu;
            s->mt[k] = v;
        }
        s->idx = 0;
    }
    uint32_t y = s->mt[s->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}

void oracle_mt19937_u32(uint32_t seed, uint32_t *out, size_t n) {
    mt_state s;
    mt_seed(&s, seed);
    for (size_t i = 0; i < n; i++) out[i] = mt_next(&s);
}

void oracle_fill_uniform(float *out, size_t n, uint32_t seed, float lo, float hi) {
    mt_state s;
    mt_seed(&s, seed);
    const float scale = 1.0f / 16777216.0f; /* 2^-24, exact */
    for (size_t i = 0; i < n; i++) {
        float u = (float)(mt_next(&s) >> 8) * scale; /* exact: 24-bit integer */
        out[i] = lo + (hi - lo) * u;
    }
}

void oracle_fill_normal(float *out, size_t n, uint32_t seed, double mean, double sigma) {
    mt_state s;
    mt_seed(&s, seed);
    const double two_pi = 6.283185307179586476925286766559;
    for (size_t i = 0; i < n; i += 2) {
        /* u1 in (0,1], u2 in [0,1) */
        double u1 = ((double)(mt_next(&s) >> 8) + 1.0) / 16777216.0;
        double u2 = (double)(mt_next(&s) >> 8) / 16777216.0;
        double r = sqrt(-2.0 * log(u1));
        out[i] = (float)(mean + sigma * r * cos(two_pi * u2));
        if (i + 1 < n) out[i + 1] = (float)(mean + sigma * r * sin(two_pi * u2));
    }
}

/* MatrixCPU::ascending(), test/library/matrix/impl/cpu-matrix.h:83-91:
 * data[i*lda + j] = i*col + j. */
void oracle_fill_ascending(float *out, int64_t rows, int64_t cols, int64_t lda) {
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) out[i * lda + j] = (float)(i * cols + j);
}

/* ------------------------------------------------------------------ */
/* bf16 (not present in the reference: round-to-nearest-even on the    */
/* upper 16 bits of the fp32 pattern).                                 */
/* ------------------------------------------------------------------ */
uint16_t oracle_f32_to_bf16_rne(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void oracle_round_to_bf16(const float *in, uint16_t *out_bits, float *out_f32, size_t n) {
    for (size_t i = 0; i < n; i++) {
        uint16_t b = oracle_f32_to_bf16_rne(in[i]);
        if (out_bits) out_bits[i] = b;
        if (out_f32) out_f32[i] = oracle_bf16_to_f32(b);
    }
}

/* ------------------------------------------------------------------ */
/* Blur.  apps/common/impl/impl.h:190-214 (blur_x) and :216-250        */
/* (blur_y): the running sum starts at 0, taps are added left to right */
/* (top to bottom), then ONE true fp32 division by the tap count.      */
/* apps/blur/blur.cpp:11-25 is the same arithmetic without the "0 +".  */
/* ------------------------------------------------------------------ */
void oracle_blur_x(const float *in, int64_t rows, int64_t cols_in, int64_t lda_in, float *out,
                   int64_t lda_out, int stride) {
    const int64_t cols_out = cols_in - stride + 1;
    const float d = (float)stride;
    for (int64_t i = 0; i < rows; i++) {
        const float *r = in + i * lda_in;
        float *o = out + i * lda_out;
        for (int64_t j = 0; j < cols_out; j++) {
            float sum = 0;
            for (int s = 0; s < stride; s++) sum += r[j + s];
            o[j] = sum / d;
        }
    }
}

void oracle_blur_y(const float *in, int64_t rows_in, int64_t cols, int64_t lda_in, float *out,
                   int64_t lda_out, int stride) {
    const int64_t rows_out = rows_in - stride + 1;
    const float d = (float)stride;
    for (int64_t i = 0; i < rows_out; i++) {
        float *o = out + i * lda_out;
        for (int64_t j = 0; j < cols; j++) {
            float sum = 0;
            for (int s = 0; s < stride; s++) sum += in[(i + s) * lda_in + j];
            o[j] = sum / d;
        }
    }
}

static int count_pattern(const char *pattern, int *nx, int *ny) {
    *nx = *ny = 0;
    if (!pattern || !*pattern) return -1;
    for (const char *p = pattern; *p; p++) {
        if (*p == 'x') (*nx)++;
        else if (*p == 'y') (*ny)++;
        else return -1;
    }
    return 0;
}

/* The unfused sequence of whole-image passes, as the reference's own check
 * does it (apps/blur/blur.cpp:96-101). */
int oracle_blur_chain(const float *in, int64_t rows, int64_t cols, const char *pattern,
                      int stride, float *out) {
    int nx, ny;
    if (count_pattern(pattern, &nx, &ny) || stride < 1) return -1;
    if (rows - (int64_t)ny * (stride - 1) <= 0 || cols - (int64_t)nx * (stride - 1) <= 0) return -1;
    size_t nstage = strlen(pattern);
    const float *cur = in;
    float *owned = NULL;
    int64_t r = rows, c = cols;
    for (size_t s = 0; s < nstage; s++) {
        int64_t r2 = r, c2 = c;
        if (pattern[s] == 'x') c2 = c - stride + 1;
        else r2 = r - stride + 1;
        float *dst = (s + 1 == nstage) ? out : (float *)malloc(sizeof(float) * (size_t)r2 * (size_t)c2);
        if (!dst) {
            free(owned);
            return -1;
        }
        if (pattern[s] == 'x') oracle_blur_x(cur, r, c, c, dst, c2, stride);
        else oracle_blur_y(cur, r, c, c, dst, c2, stride);
        free(owned);
        owned = (s + 1 == nstage) ? NULL : dst;
        cur = dst;
        r = r2;
        c = c2;
    }
    return 0;
}

/* The fused schedule: Tile(rows)(Tile(cols)(stage_0, ..., stage_n)).  For one
 * output tile the chain is walked backwards to size each intermediate
 * (rows + (#later y stages)*(stride-1)) x (cols + (#later x stages)*(stride-1)),
 * the halo extents the composed annotations infer, then each stage runs on
 * its temporary (views into the input, a fresh buffer per intermediate, as
 * MatrixCPU::query / ::allocate do, cpu-matrix.h:31-43). */
int oracle_blur_chain_tiled(const float *in, int64_t rows, int64_t cols, const char *pattern,
                            int stride, int64_t tile_rows, int64_t tile_cols, float *out) {
    int nx, ny;
    if (count_pattern(pattern, &nx, &ny) || stride < 1 || tile_rows < 1 || tile_cols < 1) return -1;
    const int64_t h = stride - 1;
    const int64_t out_rows = rows - ny * h, out_cols = cols - nx * h;
    if (out_rows <= 0 || out_cols <= 0) return -1;
    const size_t nstage = strlen(pattern);
    const int64_t max_r = tile_rows + ny * h, max_c = tile_cols + nx * h;
    float *bufA = (float *)malloc(sizeof(float) * (size_t)max_r * (size_t)max_c);
    float *bufB = (float *)malloc(sizeof(float) * (size_t)max_r * (size_t)max_c);
    if (!bufA || !bufB) {
        free(bufA);
        free(bufB);
        return -1;
    }
    for (int64_t x0 = 0; x0 < out_rows; x0 += tile_rows) {
        const int64_t tr = (x0 + tile_rows <= out_rows) ? tile_rows : out_rows - x0;
        for (int64_t y0 = 0; y0 < out_cols; y0 += tile_cols) {
            const int64_t tc = (y0 + tile_cols <= out_cols) ? tile_cols : out_cols - y0;
            /* extents of the input view for this tile */
            int64_t r = tr + ny * h, c = tc + nx * h;
            const float *cur = in + x0 * cols + y0;
            int64_t cur_ld = cols;
            for (size_t s = 0; s < nstage; s++) {
                int64_t r2 = r, c2 = c;
                if (pattern[s] == 'x') c2 = c - h;
                else r2 = r - h;
                float *dst;
                int64_t dst_ld;
                if (s + 1 == nstage) {
                    dst = out + x0 * out_cols + y0;
                    dst_ld = out_cols;
                } else {
                    dst = (cur == bufA) ? bufB : bufA;
                    dst_ld = c2;
                }
                if (pattern[s] == 'x') oracle_blur_x(cur, r, c, cur_ld, dst, dst_ld, stride);
                else oracle_blur_y(cur, r, c, cur_ld, dst, dst_ld, stride);
                cur = dst;
                cur_ld = dst_ld;
                r = r2;
                c = c2;
            }
        }
    }
    free(bufA);
    free(bufB);
    return 0;
}

/* ------------------------------------------------------------------ */
/* Row softmax.  test/library/matrix/impl/cpu-matrix.h:                */
/*   max_row :157-168 (sequential std::max), subtract_vec :170-181,    */
/*   exp_matrix :134-144 (expf), sum_row :146-155 (sequential fp32     */
/*   left-to-right sum from 0.0f), divide_vec :183-194 (true division).*/
/* Two defects of the reference's CPU twins are NOT inherited: the max */
/* is seeded with the row's first element rather than with             */
/* numeric_limits<float>::min() (:161), and the shift is x - max, as   */
/* the GPU twin computes it (apps/common/impl/impl.h:71), not          */
/* max - x (:178).                                                     */
/* ------------------------------------------------------------------ */
void oracle_softmax_rows(const float *in, int64_t rows, int64_t cols, int64_t lda, float *out,
                         int64_t ldo) {
    for (int64_t i = 0; i < rows; i++) {
        const float *a = in + i * lda;
        float *o = out + i * ldo;
        float maximum = a[0];
        for (int64_t j = 1; j < cols; j++) maximum = (maximum < a[j]) ? a[j] : maximum;
        for (int64_t j = 0; j < cols; j++) o[j] = a[j] - maximum;
        for (int64_t j = 0; j < cols; j++) o[j] = expf(o[j]);
        float sum = 0.0f;
        for (int64_t j = 0; j < cols; j++) sum += o[j];
        for (int64_t j = 0; j < cols; j++) o[j] = o[j] / sum;
    }
}

/* ------------------------------------------------------------------ */
/* GEMM.  test/library/matrix/impl/cpu-matrix.h:196-212: per (i,j) a   */
/* local fp32 sum over k from 0.0f, then c += sum.  (The GPU twin,     */
/* gernels/mm/impl/matrix_multiply.h:50-61, accumulates straight into  */
/* C; with C zeroed and one k pass the two orders are identical.)      */
/* ------------------------------------------------------------------ */
void oracle_gemm_f32_rows(const float *A, const float *B, float *C, int64_t M, int64_t N,
                          int64_t K, int64_t i0, int64_t i1) {
    (void)M;
    for (int64_t i = i0; i < i1; i++) {
        const float *a = A + i * K;
        float *c = C + i * N;
        for (int64_t j = 0; j < N; j++) {
            float sum = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                float p = a[k] * B[k * N + j];
                sum = sum + p;
            }
            c[j] += sum;
        }
    }
}

void oracle_gemm_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K) {
    oracle_gemm_f32_rows(A, B, C, M, N, K, 0, M);
}

void oracle_gemm_bf16_f32acc_rows(const uint16_t *A, const uint16_t *B, float *C, int64_t M,
                                  int64_t N, int64_t K, int64_t i0, int64_t i1) {
    (void)M;
    /* expand B once per call: the products are exact in fp32 (8-bit x 8-bit
     * significands), only the accumulation rounds. */
    float *Bf = (float *)malloc(sizeof(float) * (size_t)K * (size_t)N);
    float *arow = (float *)malloc(sizeof(float) * (size_t)K);
    if (!Bf || !arow) {
        free(Bf);
        free(arow);
        return;
    }
    for (int64_t t = 0; t < K * N; t++) Bf[t] = oracle_bf16_to_f32(B[t]);
    for (int64_t i = i0; i < i1; i++) {
        for (int64_t k = 0; k < K; k++) arow[k] = oracle_bf16_to_f32(A[i * K + k]);
        float *c = C + i * N;
        for (int64_t j = 0; j < N; j++) {
            float sum = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                float p = arow[k] * Bf[k * N + j];
                sum = sum + p;
            }
            c[j] += sum;
        }
    }
    free(Bf);
    free(arow);
}

void oracle_gemm_bf16_f32acc(const uint16_t *A, const uint16_t *B, float *C, int64_t M,
                             int64_t N, int64_t K) {
    oracle_gemm_bf16_f32acc_rows(A, B, C, M, N, K, 0, M);
}

/* S = softmax_rows(scale * Q K^T): the GEMM above with B = K^T, the logits
 * scaled by one fp32 multiply, then the row softmax above. */
void oracle_qk_softmax_rows(const uint16_t *Q, const uint16_t *Kmat, float *S, int64_t M,
                            int64_t N, int64_t D, float scale, int64_t i0, int64_t i1) {
    (void)M;
    float *Kf = (float *)malloc(sizeof(float) * (size_t)N * (size_t)D);
    float *q = (float *)malloc(sizeof(float) * (size_t)D);
    float *logits = (float *)malloc(sizeof(float) * (size_t)N);
    if (!Kf || !q || !logits) {
        free(Kf);
        free(q);
        free(logits);
        return;
    }
    for (int64_t t = 0; t < N * D; t++) Kf[t] = oracle_bf16_to_f32(Kmat[t]);
    for (int64_t i = i0; i < i1; i++) {
        for (int64_t k = 0; k < D; k++) q[k] = oracle_bf16_to_f32(Q[i * D + k]);
        for (int64_t j = 0; j < N; j++) {
            float sum = 0.0f;
            const float *kr = Kf + j * D;
            for (int64_t k = 0; k < D; k++) {
                float p = q[k] * kr[k];
                sum = sum + p;
            }
            logits[j] = sum * scale;
        }
        oracle_softmax_rows(logits, 1, N, N, S + i * N, N);
    }
    free(Kf);
    free(q);
    free(logits);
}

/* ------------------------------------------------------------------ */
/* Division by a constant with one FMA correction step: what the blur  */
/* gernels fall back to for tiles that hold tiny values or zeros.      */
/* ------------------------------------------------------------------ */
float oracle_div_const_fma(float x, float d) {
    const float c = 1.0f / d;
    float q = x * c;
    float r = fmaf(-d, q, x);
    q = fmaf(r, c, q);
    /* The device code finishes with v_div_fixup_f32, which returns the IEEE
     * result for zero, infinite and NaN operands (sign of a zero included). */
    if (x == 0.0f || isinf(x) || x != x) return x / d;
    return q;
}

uint64_t oracle_div_const_mismatches(float d, uint32_t lo_bits, uint32_t hi_bits) {
    uint64_t bad = 0;
    for (uint64_t b = lo_bits; b < (uint64_t)hi_bits; b++) {
        uint32_t u = (uint32_t)b;
        float x;
        memcpy(&x, &u, 4);
        if (x != x) continue;
        float want = x / d;
        float got = oracle_div_const_fma(x, d);
        uint32_t wu, gu;
        memcpy(&wu, &want, 4);
        memcpy(&gu, &got, 4);
        if (wu != gu) bad++;
    }
    return bad;
}

/* ------------------------------------------------------------------ */
/* Division of a tap sum by the tap count, as the HIP blur gernels do  */
/* it (gernels/prelude.h, quotient_of_sum): restated with libm fmaf.   */
/* ------------------------------------------------------------------ */
float oracle_quotient_of_sum(float s, float d) {
    if (d == 3.0f) {
        uint32_t hi_bits = 0x3EAAAAAAu, lo_bits = 0x32AAAAABu; /* largest float below 1/3; 1/3 minus it */
        float c_hi, c_lo;
        memcpy(&c_hi, &hi_bits, 4);
        memcpy(&c_lo, &lo_bits, 4);
        float t = fmaf(s, c_lo, 0.0f);
        return fmaf(s, c_hi, t);
    }
    if (d == 2.0f || d == 4.0f || d == 8.0f) {
        return fmaf(s, 1.0f / d, 0.0f);
    }
    return (0.0f + s) / d;
}

/* Compares oracle_quotient_of_sum(x, d) with what the reference computes from
 * the same sum, (0.0f + x) / d, over the bit patterns [lo_bits, hi_bits).
 * NaNs are skipped.  Returns the number of patterns that differ bitwise;
 * *max_ulp receives the largest difference in units in the last place and
 * *min_abs / *max_abs the smallest and largest |x| among the differing ones. */
uint64_t oracle_quotient_mismatches(float d, uint32_t lo_bits, uint32_t hi_bits, uint32_t *max_ulp,
                                    float *min_abs, float *max_abs) {
    uint64_t bad = 0;
    uint32_t worst = 0;
    float lo = INFINITY, hi = 0.0f;
    for (uint64_t b = lo_bits; b < (uint64_t)hi_bits; b++) {
        uint32_t u = (uint32_t)b;
        float x;
        memcpy(&x, &u, 4);
        if (x != x) continue;
        volatile float sum = 0.0f + x;
        float want = sum / d;
        float got = oracle_quotient_of_sum(x, d);
        uint32_t wu, gu;
        memcpy(&wu, &want, 4);
        memcpy(&gu, &got, 4);
        if (wu != gu) {
            bad++;
            /* same sign here (a sign flip would be a difference of ~2^31) */
            uint32_t diff = wu > gu ? wu - gu : gu - wu;
            if (diff > worst) worst = diff;
            float ax = fabsf(x);
            if (ax < lo) lo = ax;
            if (ax > hi) hi = ax;
        }
    }
    if (max_ulp) *max_ulp = worst;
    if (min_abs) *min_abs = lo;
    if (max_abs) *max_abs = hi;
    return bad;
}

/* ------------------------------------------------------------------ */
static int32_t ordered_bits(float f) {
    int32_t i;
    memcpy(&i, &f, 4);
    return (i < 0) ? (int32_t)(0x80000000u - (uint32_t)i) : i;
}

uint32_t oracle_max_ulp(const float *a, const float *b, size_t n) {
    uint32_t worst = 0;
    for (size_t i = 0; i < n; i++) {
        if (a[i] != a[i] || b[i] != b[i]) return 0xffffffffu;
        int64_t d = (int64_t)ordered_bits(a[i]) - (int64_t)ordered_bits(b[i]);
        if (d < 0) d = -d;
        if ((uint64_t)d > worst) worst = (uint32_t)d;
    }
    return worst;
}
