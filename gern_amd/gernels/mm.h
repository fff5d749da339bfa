// Block-cooperative GEMM gernels for gfx950.
//
// One workgroup of 256 threads (four wavefronts, 2 x 2) owns a BM x BN tile of
// C.  The operands are windows onto A and B in HBM; the gernel walks their
// shared K extent in BK-deep steps, staging each step through LDS (double
// buffered, next step's global loads in flight while this step computes) and
// accumulating into registers.  Two flavours:
//
//   bf16 inputs, fp32 accumulation on the matrix cores
//       v_mfma_f32_32x32x16_bf16; each wavefront owns (BM/2) x (BN/2) of C as
//       (BM/64) x (BN/64) MFMA tiles of 16 accumulator registers.  B is
//       row-major (K x N) but the matrix core wants K-contiguous fragments, so
//       B is transposed on its way into LDS (dword loads of column pairs,
//       v_perm to split them).  LDS rows are padded to 144 bytes so that the
//       16-byte fragment reads of eight consecutive lanes hit distinct banks.
//   fp32 inputs, fp32 FMAs on the vector ALU
//       the classic register-tiled scheme: 8 x 8 outputs per thread, A staged
//       K-major so that both operands are read from LDS as float4.
//
// These replace the reference's GEMM gernels and their staging methods
// (gernels/mm/impl/matrix_multiply.h:50-61, matrix-gpu.h:240-374): same role in
// a composed program (query operands, query/insert the C tile, call
// matrix_multiply inside Reduce), different machine mapping.  The reference
// has no matrix-core path and no bf16 type at all.
#pragma once

#include "gernels/wave_tile.h"

namespace gernels {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Dynamic LDS of the kernel; the launch sizes it (Global(..., smem_size)).
extern __shared__ __attribute__((aligned(16))) unsigned char gern_lds[];

// A window onto a row-major matrix in HBM: at most R x C, of which
// rows x cols lie inside the matrix.
template<int64_t R, int64_t C, typename T>
struct GlobalView {
    const T *data;
    int64_t lda;
    int64_t rows;
    int64_t cols;
};

template<int64_t R, int64_t C>
__device__ __forceinline__ GlobalView<R, C, float> MatrixF32::view(int64_t x, int64_t y) const {
    const int64_t r = row - x, c = col - y;
    return GlobalView<R, C, float>{data + x * lda + y, lda, r < R ? (r < 0 ? 0 : r) : R, c < C ? (c < 0 ? 0 : c) : C};
}

// Row-major bf16 matrix in HBM (bit patterns).
struct MatrixBF16 {
    uint16_t *data;
    int64_t row;
    int64_t col;
    int64_t lda;

    template<int64_t R, int64_t C>
    __device__ __forceinline__ GlobalView<R, C, uint16_t> view(int64_t x, int64_t y) const {
        const int64_t r = row - x, c = col - y;
        return GlobalView<R, C, uint16_t>{data + x * lda + y, lda, r < R ? (r < 0 ? 0 : r) : R,
                                          c < C ? (c < 0 ? 0 : c) : C};
    }
};

// ---------------------------------------------------------------------------
// bf16 x bf16 -> fp32 on MFMA
// ---------------------------------------------------------------------------
// Accumulators of a BM x BN tile, spread over the 2 x 2 wavefronts of the
// workgroup.  Wavefront (wm, wn) owns rows [wm*BM/2, ...) and columns
// [wn*BN/2, ...); inside a 32 x 32 MFMA tile lane l, register i holds
// row 8*(i/4) + 4*(l/32) + i%4, column l%32.
template<int64_t BM, int64_t BN>
struct MfmaAcc {
    static_assert(BM % 64 == 0 && BN % 64 == 0, "a wavefront owns whole 32 x 32 MFMA tiles");
    static constexpr int TM = BM / 64;
    static constexpr int TN = BN / 64;
    f32x16_t acc[TM][TN];

    __device__ __forceinline__ void destroy() {
    }
};

namespace detail {

__device__ __forceinline__ int wave_in_block() {
    return (int)(threadIdx.x / kWaveSize);
}

template<int64_t BM, int64_t BN, typename F>
__device__ __forceinline__ void for_each_acc(F &&f) {
    const int lane = lane_id();
    const int w = wave_in_block();
    const int64_t row0 = (int64_t)(w / 2) * (BM / 2) + 4 * (lane / 32);
    const int64_t col0 = (int64_t)(w % 2) * (BN / 2) + (lane % 32);
#pragma unroll
    for (int tm = 0; tm < MfmaAcc<BM, BN>::TM; tm++) {
#pragma unroll
        for (int tn = 0; tn < MfmaAcc<BM, BN>::TN; tn++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                f(tm, tn, i, row0 + tm * 32 + 8 * (i / 4) + (i % 4), col0 + tn * 32);
            }
        }
    }
}

}  // namespace detail

// C tile -> accumulators (C += A * B keeps what C held).
template<int64_t BM, int64_t BN>
__device__ __forceinline__ MfmaAcc<BM, BN> MatrixF32::load_acc_mfma(int64_t x, int64_t y) const {
    MfmaAcc<BM, BN> t;
    detail::for_each_acc<BM, BN>([&](int tm, int tn, int i, int64_t r, int64_t c) {
        const int64_t rr = x + r, cc = y + c;
        t.acc[tm][tn][i] = (rr < row && cc < col) ? data[rr * lda + cc] : 0.f;
    });
    return t;
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::store_acc(int64_t x, int64_t y, const MfmaAcc<BM, BN> &t) const {
    detail::for_each_acc<BM, BN>([&](int tm, int tn, int i, int64_t r, int64_t c) {
        const int64_t rr = x + r, cc = y + c;
        if (rr < row && cc < col) {
            data[rr * lda + cc] = t.acc[tm][tn][i];
        }
    });
}

constexpr int kMfmaBK = 64;                  // K depth of one LDS stage
constexpr int kMfmaRowBytes = 2 * kMfmaBK + 16;  // padded LDS row: 144 bytes

// LDS needed by matrix_multiply on bf16 operands.
template<int64_t BM, int64_t BN>
constexpr int64_t mfma_lds_bytes() {
    return 2 * (BM + BN) * kMfmaRowBytes;
}

template<int64_t BM, int64_t BN, int64_t KC>
__device__ __forceinline__ void matrix_multiply(const GlobalView<BM, KC, uint16_t> &A,
                                                const GlobalView<KC, BN, uint16_t> &B, MfmaAcc<BM, BN> &C) {
    static_assert(BM % 64 == 0 && BN % 64 == 0 && BM <= 256 && BN <= 256, "tile shape");
    constexpr int A_CHUNKS = BM * (kMfmaBK / 8) / 256;   // 16-byte chunks of A per thread per stage
    constexpr int B_TASKS = (BN / 2) * (kMfmaBK / 8) / 256;  // 8-deep column pairs of B per thread per stage
    static_assert(A_CHUNKS >= 1 && B_TASKS >= 1, "tile too small for 256 threads");
    constexpr int STAGE_BYTES = (BM + BN) * kMfmaRowBytes;

    const int tid = (int)threadIdx.x;
    const int lane = lane_id();
    const int w = detail::wave_in_block();
    const int64_t k_total = A.cols < B.rows ? A.cols : B.rows;
    const int nk = (int)((k_total + kMfmaBK - 1) / kMfmaBK);

    uint4 ra[A_CHUNKS];
    uint32_t rb[B_TASKS][8];

    auto fetch = [&](int kt) {
        const int64_t k0 = (int64_t)kt * kMfmaBK;
#pragma unroll
        for (int j = 0; j < A_CHUNKS; j++) {
            const int c = tid + 256 * j;
            const int64_t r = c / 8, kk = k0 + (c % 8) * 8;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (r < A.rows && kk + 7 < k_total) {
                v = *reinterpret_cast<const uint4 *>(A.data + r * A.lda + kk);
            } else if (r < A.rows && kk < k_total) {
                uint16_t e[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int q = 0; q < 8; q++) {
                    if (kk + q < k_total) e[q] = A.data[r * A.lda + kk + q];
                }
                v = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
            }
            ra[j] = v;
        }
#pragma unroll
        for (int j = 0; j < B_TASKS; j++) {
            const int id = tid + 256 * j;
            const int64_t n = 2 * (id % (BN / 2)), kk = k0 + 8 * (id / (BN / 2));
#pragma unroll
            for (int q = 0; q < 8; q++) {
                uint32_t v = 0u;
                if (kk + q < k_total) {
                    const uint16_t *p = B.data + (kk + q) * B.lda + n;
                    if (n + 1 < B.cols) {
                        v = *reinterpret_cast<const uint32_t *>(p);
                    } else if (n < B.cols) {
                        v = p[0];
                    }
                }
                rb[j][q] = v;
            }
        }
    };

    auto stash = [&](int buf) {
        unsigned char *a_lds = gern_lds + buf * STAGE_BYTES;
        unsigned char *b_lds = a_lds + BM * kMfmaRowBytes;
#pragma unroll
        for (int j = 0; j < A_CHUNKS; j++) {
            const int c = tid + 256 * j;
            *reinterpret_cast<uint4 *>(a_lds + (c / 8) * kMfmaRowBytes + (c % 8) * 16) = ra[j];
        }
#pragma unroll
        for (int j = 0; j < B_TASKS; j++) {
            const int id = tid + 256 * j;
            const int n = 2 * (id % (BN / 2)), g = id / (BN / 2);
            // rb[j][q] = {B[k+q][n] (low half), B[k+q][n+1] (high half)}: split
            // into the K-contiguous vectors of column n and column n+1.
            uint4 lo, hi;
            lo.x = __builtin_amdgcn_perm(rb[j][1], rb[j][0], 0x05040100u);
            lo.y = __builtin_amdgcn_perm(rb[j][3], rb[j][2], 0x05040100u);
            lo.z = __builtin_amdgcn_perm(rb[j][5], rb[j][4], 0x05040100u);
            lo.w = __builtin_amdgcn_perm(rb[j][7], rb[j][6], 0x05040100u);
            hi.x = __builtin_amdgcn_perm(rb[j][1], rb[j][0], 0x07060302u);
            hi.y = __builtin_amdgcn_perm(rb[j][3], rb[j][2], 0x07060302u);
            hi.z = __builtin_amdgcn_perm(rb[j][5], rb[j][4], 0x07060302u);
            hi.w = __builtin_amdgcn_perm(rb[j][7], rb[j][6], 0x07060302u);
            *reinterpret_cast<uint4 *>(b_lds + n * kMfmaRowBytes + g * 16) = lo;
            *reinterpret_cast<uint4 *>(b_lds + (n + 1) * kMfmaRowBytes + g * 16) = hi;
        }
    };

    if (nk == 0) {
        return;
    }
    fetch(0);
    stash(0);
    __syncthreads();

    const int a_row0 = (w / 2) * (int)(BM / 2) + (lane % 32);
    const int b_row0 = (w % 2) * (int)(BN / 2) + (lane % 32);
    const int k_off = (lane / 32) * 16;

    for (int kt = 0; kt < nk; kt++) {
        if (kt + 1 < nk) {
            fetch(kt + 1);
        }
        const unsigned char *a_lds = gern_lds + (kt & 1) * STAGE_BYTES;
        const unsigned char *b_lds = a_lds + BM * kMfmaRowBytes;
#pragma unroll
        for (int s = 0; s < kMfmaBK / 16; s++) {
            bf16x8_t af[MfmaAcc<BM, BN>::TM], bfr[MfmaAcc<BM, BN>::TN];
#pragma unroll
            for (int tm = 0; tm < MfmaAcc<BM, BN>::TM; tm++) {
                af[tm] = *reinterpret_cast<const bf16x8_t *>(a_lds + (a_row0 + tm * 32) * kMfmaRowBytes + s * 32 + k_off);
            }
#pragma unroll
            for (int tn = 0; tn < MfmaAcc<BM, BN>::TN; tn++) {
                bfr[tn] = *reinterpret_cast<const bf16x8_t *>(b_lds + (b_row0 + tn * 32) * kMfmaRowBytes + s * 32 + k_off);
            }
#pragma unroll
            for (int tm = 0; tm < MfmaAcc<BM, BN>::TM; tm++) {
#pragma unroll
                for (int tn = 0; tn < MfmaAcc<BM, BN>::TN; tn++) {
                    C.acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[tm], bfr[tn], C.acc[tm][tn], 0, 0, 0);
                }
            }
        }
        if (kt + 1 < nk) {
            stash((kt + 1) & 1);
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// fp32 x fp32 -> fp32 on the vector ALU
// ---------------------------------------------------------------------------
// 128 x 128 tile, 256 threads as 16 x 16; thread (ty, tx) owns rows
// {ty*4 .. ty*4+3} and {64 + ty*4 ..}, columns {tx*4 ..} and {64 + tx*4 ..}.
template<int64_t BM, int64_t BN>
struct FmaAcc {
    static_assert(BM == 128 && BN == 128, "the fp32 gernel is written for 128 x 128 tiles");
    float acc[8][8];

    __device__ __forceinline__ void destroy() {
    }
};

namespace detail {

template<typename F>
__device__ __forceinline__ void for_each_fma_acc(F &&f) {
    const int ty = (int)threadIdx.x / 16, tx = (int)threadIdx.x % 16;
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int j = 0; j < 8; j += 4) {
            f(i, j, (int64_t)(i / 4) * 64 + ty * 4 + (i % 4), (int64_t)(j / 4) * 64 + tx * 4);
        }
    }
}

}  // namespace detail

template<int64_t BM, int64_t BN>
__device__ __forceinline__ FmaAcc<BM, BN> MatrixF32::load_acc_fma(int64_t x, int64_t y) const {
    FmaAcc<BM, BN> t;
    detail::for_each_fma_acc([&](int i, int j, int64_t r, int64_t c) {
        const int64_t rr = x + r, cc = y + c;
        const float *p = data + rr * lda + cc;
        if (rr < row && cc + 3 < col && ((((uint64_t)p) & 15u) == 0)) {
            const float4 v = *reinterpret_cast<const float4 *>(p);
            t.acc[i][j] = v.x;
            t.acc[i][j + 1] = v.y;
            t.acc[i][j + 2] = v.z;
            t.acc[i][j + 3] = v.w;
        } else {
            for (int e = 0; e < 4; e++) {
                t.acc[i][j + e] = (rr < row && cc + e < col) ? p[e] : 0.f;
            }
        }
    });
    return t;
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::store_acc(int64_t x, int64_t y, const FmaAcc<BM, BN> &t) const {
    detail::for_each_fma_acc([&](int i, int j, int64_t r, int64_t c) {
        const int64_t rr = x + r, cc = y + c;
        float *p = data + rr * lda + cc;
        if (rr < row && cc + 3 < col && ((((uint64_t)p) & 15u) == 0)) {
            *reinterpret_cast<float4 *>(p) = make_float4(t.acc[i][j], t.acc[i][j + 1], t.acc[i][j + 2], t.acc[i][j + 3]);
        } else {
            for (int e = 0; e < 4; e++) {
                if (rr < row && cc + e < col) p[e] = t.acc[i][j + e];
            }
        }
    });
}

constexpr int kFmaBK = 16;
constexpr int kFmaLd = 128 + 4;  // padded LDS row, in floats

template<int64_t BM, int64_t BN>
constexpr int64_t fma_lds_bytes() {
    return 2 * 2 * kFmaBK * kFmaLd * 4;
}

template<int64_t BM, int64_t BN, int64_t KC>
__device__ __forceinline__ void matrix_multiply(const GlobalView<BM, KC, float> &A, const GlobalView<KC, BN, float> &B,
                                                FmaAcc<BM, BN> &C) {
    constexpr int STAGE_FLOATS = 2 * kFmaBK * kFmaLd;
    float *lds = reinterpret_cast<float *>(gern_lds);
    const int tid = (int)threadIdx.x;
    const int ty = tid / 16, tx = tid % 16;
    const int64_t k_total = A.cols < B.rows ? A.cols : B.rows;
    const int nk = (int)((k_total + kFmaBK - 1) / kFmaBK);

    // A stage: 128 rows x 16 k = 512 float4 along k, two per thread.
    // B stage: 16 k x 128 n = 512 float4 along n, two per thread.
    float4 ra[2], rb[2];
    const bool a_vec = ((((uint64_t)A.data) & 15u) == 0) && (A.lda % 4 == 0);
    const bool b_vec = ((((uint64_t)B.data) & 15u) == 0) && (B.lda % 4 == 0);

    auto fetch = [&](int kt) {
        const int64_t k0 = (int64_t)kt * kFmaBK;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int c = tid + 256 * j;
            {
                const int64_t r = c / 4, kk = k0 + (c % 4) * 4;
                const float *p = A.data + r * A.lda + kk;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (r < A.rows && kk + 3 < k_total && a_vec) {
                    v = *reinterpret_cast<const float4 *>(p);
                } else if (r < A.rows) {
                    if (kk + 0 < k_total) v.x = p[0];
                    if (kk + 1 < k_total) v.y = p[1];
                    if (kk + 2 < k_total) v.z = p[2];
                    if (kk + 3 < k_total) v.w = p[3];
                }
                ra[j] = v;
            }
            {
                const int64_t kk = k0 + c / 32, n = (c % 32) * 4;
                const float *p = B.data + kk * B.lda + n;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (kk < k_total && n + 3 < B.cols && b_vec) {
                    v = *reinterpret_cast<const float4 *>(p);
                } else if (kk < k_total) {
                    if (n + 0 < B.cols) v.x = p[0];
                    if (n + 1 < B.cols) v.y = p[1];
                    if (n + 2 < B.cols) v.z = p[2];
                    if (n + 3 < B.cols) v.w = p[3];
                }
                rb[j] = v;
            }
        }
    };

    auto stash = [&](int buf) {
        float *a_lds = lds + buf * STAGE_FLOATS;      // [k][m], K-major
        float *b_lds = a_lds + kFmaBK * kFmaLd;       // [k][n]
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int c = tid + 256 * j;
            const int r = c / 4, kk = (c % 4) * 4;
            a_lds[(kk + 0) * kFmaLd + r] = ra[j].x;
            a_lds[(kk + 1) * kFmaLd + r] = ra[j].y;
            a_lds[(kk + 2) * kFmaLd + r] = ra[j].z;
            a_lds[(kk + 3) * kFmaLd + r] = ra[j].w;
            *reinterpret_cast<float4 *>(b_lds + (c / 32) * kFmaLd + (c % 32) * 4) = rb[j];
        }
    };

    if (nk == 0) {
        return;
    }
    fetch(0);
    stash(0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        if (kt + 1 < nk) {
            fetch(kt + 1);
        }
        const float *a_lds = lds + (kt & 1) * STAGE_FLOATS;
        const float *b_lds = a_lds + kFmaBK * kFmaLd;
#pragma unroll
        for (int k = 0; k < kFmaBK; k++) {
            const float4 a0 = *reinterpret_cast<const float4 *>(a_lds + k * kFmaLd + ty * 4);
            const float4 a1 = *reinterpret_cast<const float4 *>(a_lds + k * kFmaLd + 64 + ty * 4);
            const float4 b0 = *reinterpret_cast<const float4 *>(b_lds + k * kFmaLd + tx * 4);
            const float4 b1 = *reinterpret_cast<const float4 *>(b_lds + k * kFmaLd + 64 + tx * 4);
            const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    C.acc[i][j] = __builtin_fmaf(a[i], b[j], C.acc[i][j]);
                }
            }
        }
        if (kt + 1 < nk) {
            stash((kt + 1) & 1);
        }
        __syncthreads();
    }
}

}  // namespace gernels
