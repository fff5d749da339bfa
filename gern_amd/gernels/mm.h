// Block-cooperative GEMM gernels for gfx950.
//
// One workgroup owns a BM x BN tile of C.  The operands are windows onto A and
// B in HBM; the gernel walks their shared K extent in BK-deep steps, staging
// each step through LDS (double buffered, next step's global loads in flight
// while this step computes) and accumulating into registers.  Two flavours:
//
//   bf16 inputs, fp32 accumulation on the matrix cores
//       v_mfma_f32_32x32x16_bf16, MFMA tiles of 16 accumulator registers.
//       Eight wavefronts (2 x 4) with operands loaded straight into LDS
//       (detail::mfma_direct below) when the matrix shapes allow it; otherwise
//       four wavefronts (2 x 2) that stage through registers: B is row-major
//       (K x N) but the matrix core wants K-contiguous fragments, so B is
//       transposed on its way into LDS (dword loads of column pairs, v_perm
//       to split them), and LDS rows are padded to 144 bytes so that the
//       16-byte fragment reads of eight consecutive lanes hit distinct banks.
//   fp32 inputs, fp32 FMAs on the vector ALU
//       256 threads, the classic register-tiled scheme: 8 x 8 outputs per
//       thread, A staged K-major so that both operands are read from LDS as
//       float4.
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
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// Dynamic LDS of the kernel; the launch sizes it (Global(..., smem_size)).
extern __shared__ __attribute__((aligned(16))) unsigned char gern_lds[];

// A window onto a row-major matrix in HBM: at most R x C, of which
// rows x cols lie inside the matrix.  EXACT is a promise about the matrix the
// window was cut from, made by the program that declares the operand: the
// matrix is one dense allocation that ends with its last element, A starts on
// a 16-byte boundary and the part of each of its rows that is multiplied is a
// whole number of 16-byte pieces (the reduction extent is a multiple of 8 for
// bf16, of 4 for fp32; the rows themselves need only 4-byte alignment, their
// pitch may be longer than the reduction extent), B starts on a 4-byte
// boundary, and row pitches stay below kMfmaMaxLd elements.
// Windows on the bottom and right edges may be partial, and so may the last
// stage of the reduction: rows and cols say how much of them exists.
template<int64_t R, int64_t C, typename T, bool EXACT>
struct GlobalView {
    const T *data;
    int64_t lda;
    int64_t rows;
    int64_t cols;
};

template<int64_t R, int64_t C>
__device__ __forceinline__ GlobalView<R, C, float, false> MatrixF32::view(int64_t x, int64_t y) const {
    const int64_t r = row - x, c = col - y;
    return GlobalView<R, C, float, false>{data + x * lda + y, lda, r < R ? (r < 0 ? 0 : r) : R,
                                          c < C ? (c < 0 ? 0 : c) : C};
}

// The same window for a matrix that keeps the EXACT promise of GlobalView.
template<int64_t R, int64_t C>
__device__ __forceinline__ GlobalView<R, C, float, true> MatrixF32::view_exact(int64_t x, int64_t y) const {
    const int64_t r = row - x, c = col - y;
    return GlobalView<R, C, float, true>{data + x * lda + y, lda, r < R ? (r < 0 ? 0 : r) : R,
                                         c < C ? (c < 0 ? 0 : c) : C};
}

// Row-major bf16 matrix in HBM (bit patterns).
struct MatrixBF16 {
    uint16_t *data;
    int64_t row;
    int64_t col;
    int64_t lda;

    template<int64_t R, int64_t C>
    __device__ __forceinline__ GlobalView<R, C, uint16_t, false> view(int64_t x, int64_t y) const {
        const int64_t r = row - x, c = col - y;
        return GlobalView<R, C, uint16_t, false>{data + x * lda + y, lda, r < R ? (r < 0 ? 0 : r) : R,
                                                 c < C ? (c < 0 ? 0 : c) : C};
    }
    // The same window for a matrix that keeps the EXACT promise of GlobalView.
    template<int64_t R, int64_t C>
    __device__ __forceinline__ GlobalView<R, C, uint16_t, true> view_exact(int64_t x, int64_t y) const {
        const int64_t r = row - x, c = col - y;
        return GlobalView<R, C, uint16_t, true>{data + x * lda + y, lda, r < R ? (r < 0 ? 0 : r) : R,
                                                c < C ? (c < 0 ? 0 : c) : C};
    }
};

// ---------------------------------------------------------------------------
// bf16 x bf16 -> fp32 on MFMA
// ---------------------------------------------------------------------------
// Accumulators of a BM x BN tile, spread over the NW wavefronts of the
// workgroup, arranged 2 x (NW/2).  Wavefront (wm, wn) owns rows
// [wm*BM/2, ...) and columns [wn*BN/(NW/2), ...); inside a 32 x 32 MFMA tile
// lane l, register i holds row 8*(i/4) + 4*(l/32) + i%4, column l%32.
//
// NW = 8 (two wavefronts per SIMD) is the fast shape: a single wavefront
// stalls on its own LDS reads, two fill each other's gaps (the SIMD gives the
// matrix pipe to the older of the two whenever both are ready).
template<int64_t BM, int64_t BN, int NW = 4>
struct MfmaAcc {
    static_assert(NW == 4 || NW == 8, "four or eight wavefronts per workgroup");
    static constexpr int WC = NW / 2;           // wavefront columns
    static constexpr int64_t WM = BM / 2;       // rows per wavefront
    static constexpr int64_t WN = BN / WC;      // columns per wavefront
    static_assert(WM % 32 == 0 && WN % 32 == 0, "a wavefront owns whole 32 x 32 MFMA tiles");
    static constexpr int TM = (int)(WM / 32);
    static constexpr int TN = (int)(WN / 32);
    static constexpr int threads = NW * kWaveSize;
    static constexpr int kTile = 32;            // edge of the matrix instruction's result
    f32x16_t acc[TM][TN];

    __device__ __forceinline__ void destroy() {
    }
};

// The accumulators of the fast bf16 path: a 256 x 256 tile on eight wavefronts
// (2 x 4, 128 rows x 64 columns each) as 8 x 4 results of
// v_mfma_f32_16x16x32_bf16, computed TRANSPOSED (B's fragment is the
// instruction's first operand): acc[tm][tn][i] of lane l is row
// 128 wm + 16 tm + l % 16, column 64 wn + 16 tn + 4 (l / 16) + i, four
// consecutive columns of C per lane and tile (16-byte stores).
//
// The 16 x 16 x 32 instruction does the work of the 32 x 32 x 16 one in the
// same number of cycles (a loop of nothing but matrix instructions on random
// operands runs both at 1024 flop per cycle and SIMD) but DRAWS LESS POWER, and
// power is what sets the clock of a kernel like this one: that loop settles at
// 2.05-2.1 GHz with 16 x 16 x 32 and at 1.78-1.85 GHz with 32 x 32 x 16.
template<int64_t BM, int64_t BN>
struct MfmaAcc16 {
    static_assert(BM == 256 && BN == 256, "written for 256 x 256 tiles");
    static constexpr int WC = 4;
    static constexpr int64_t WM = 128;
    static constexpr int64_t WN = 64;
    static constexpr int TM = 8;
    static constexpr int TN = 4;
    static constexpr int threads = 8 * kWaveSize;
    static constexpr int kTile = 16;
    f32x4_t acc[TM][TN];

    __device__ __forceinline__ void destroy() {
    }
};

namespace detail {

__device__ __forceinline__ int wave_in_block() {
    return (int)(threadIdx.x / kWaveSize);
}

template<int64_t BM, int64_t BN, int NW>
__device__ __forceinline__ MfmaAcc<BM, BN, NW> zero_acc() {
    MfmaAcc<BM, BN, NW> t;
#pragma unroll
    for (int tm = 0; tm < MfmaAcc<BM, BN, NW>::TM; tm++) {
#pragma unroll
        for (int tn = 0; tn < MfmaAcc<BM, BN, NW>::TN; tn++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                t.acc[tm][tn][i] = 0.f;
            }
        }
    }
    return t;
}

// ADD: C += tile (read-modify-write); otherwise C = tile.
template<bool ADD, int64_t BM, int64_t BN, int NW>
__device__ __forceinline__ void write_acc(const MatrixF32 &m, int64_t x, int64_t y, const MfmaAcc<BM, BN, NW> &t) {
    using Acc = MfmaAcc<BM, BN, NW>;
    const int lane = lane_id();
    const int w = wave_in_block();
    const int64_t r0 = x + (int64_t)(w / Acc::WC) * Acc::WM + 4 * (lane / 32);
    const int64_t c0 = y + (int64_t)(w % Acc::WC) * Acc::WN + (lane % 32);
    const bool inside = (x + BM <= m.row) && (y + BN <= m.col);  // workgroup-uniform
    const int ld = (int)m.lda;
#pragma unroll
    for (int tm = 0; tm < Acc::TM; tm++) {
#pragma unroll
        for (int tn = 0; tn < Acc::TN; tn++) {
            float *p = m.data + (r0 + tm * 32) * m.lda + (c0 + tn * 32);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int dr = 8 * (i / 4) + (i % 4);
                if (inside || ((r0 + tm * 32 + dr < m.row) && (c0 + tn * 32 < m.col))) {
                    if (ADD) {
                        p[dr * ld] += t.acc[tm][tn][i];
                    } else {
                        // written once, never re-read by this kernel
                        store_result4<kThroughStores>(m.data, (m.row - 1) * m.lda + m.col, (r0 + tm * 32 + dr) * m.lda + (c0 + tn * 32), t.acc[tm][tn][i]);
                    }
                }
            }
        }
    }
}

}  // namespace detail

// The accumulator tile is a DEFERRED update of C: it starts at zero and the
// insert either adds it to what C holds (add_acc: C += A * B, the contract of
// the reference's matrix_multiply) or overwrites C (store_acc: C = A * B,
// which never reads C).  Loading C into the accumulators up front would give
// the same sum, but parks up to 256 live values in VGPRs across the main loop.
template<int64_t BM, int64_t BN>
__device__ __forceinline__ MfmaAcc<BM, BN, 4> MatrixF32::load_acc_mfma(int64_t, int64_t) const {
    return detail::zero_acc<BM, BN, 4>();
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ MfmaAcc<BM, BN, 8> MatrixF32::load_acc_mfma8(int64_t, int64_t) const {
    return detail::zero_acc<BM, BN, 8>();
}

template<int64_t BM, int64_t BN, int NW>
__device__ __forceinline__ void MatrixF32::add_acc(int64_t x, int64_t y, const MfmaAcc<BM, BN, NW> &t) const {
    detail::write_acc<true>(*this, x, y, t);
}

template<int64_t BM, int64_t BN, int NW>
__device__ __forceinline__ void MatrixF32::store_acc(int64_t x, int64_t y, const MfmaAcc<BM, BN, NW> &t) const {
    detail::write_acc<false>(*this, x, y, t);
}

namespace detail {

// ADD: C += tile (read-modify-write); otherwise C = tile.
template<bool ADD, int64_t BM, int64_t BN>
__device__ __forceinline__ void write_acc16(const MatrixF32 &m, int64_t x, int64_t y, const MfmaAcc16<BM, BN> &t) {
    using Acc = MfmaAcc16<BM, BN>;
    const int lane = lane_id();
    const int w = wave_in_block();
    const int64_t r0 = x + (int64_t)(w / Acc::WC) * Acc::WM + (lane % 16);
    const int64_t c0 = y + (int64_t)(w % Acc::WC) * Acc::WN + 4 * (lane / 16);
    // workgroup-uniform: every group of four columns starts on a 16-byte boundary
    const bool aligned = ((((uint64_t)m.data) & 15u) == 0) && (m.lda % 4 == 0) && (y % 4 == 0);
    const int64_t span = (m.row - 1) * m.lda + m.col;
#pragma unroll
    for (int tm = 0; tm < Acc::TM; tm++) {
        const int64_t rr = r0 + tm * 16;
        if (rr >= m.row) {
            continue;
        }
        // the two tiles of a pair of tn fill the same 128-byte lines: back to back
#pragma unroll
        for (int tn = 0; tn < Acc::TN; tn++) {
            const int64_t cc = c0 + tn * 16;
            const f32x4_t a = t.acc[tm][tn];
            float *p = m.data + rr * m.lda + cc;
            if (aligned && cc + 3 < m.col) {
                float4 v = make_float4(a[0], a[1], a[2], a[3]);
                if (ADD) {
                    const float4 o = *reinterpret_cast<const float4 *>(p);
                    v = make_float4(o.x + v.x, o.y + v.y, o.z + v.z, o.w + v.w);
                    *reinterpret_cast<float4 *>(p) = v;
                } else {
                    // written once, never re-read by this kernel
                    store_result16<kThroughStores>(m.data, span, rr * m.lda + cc, v);
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (cc + q < m.col) {
                        if (ADD) {
                            p[q] += a[q];
                        } else {
                            store_result4<kThroughStores>(m.data, span, rr * m.lda + cc + q, a[q]);
                        }
                    }
                }
            }
        }
    }
}

}  // namespace detail

template<int64_t BM, int64_t BN>
__device__ __forceinline__ MfmaAcc16<BM, BN> MatrixF32::load_acc_mfma16(int64_t, int64_t) const {
    MfmaAcc16<BM, BN> t;
#pragma unroll
    for (int tm = 0; tm < MfmaAcc16<BM, BN>::TM; tm++) {
#pragma unroll
        for (int tn = 0; tn < MfmaAcc16<BM, BN>::TN; tn++) {
            t.acc[tm][tn] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
    }
    return t;
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::add_acc(int64_t x, int64_t y, const MfmaAcc16<BM, BN> &t) const {
    detail::write_acc16<true>(*this, x, y, t);
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::store_acc(int64_t x, int64_t y, const MfmaAcc16<BM, BN> &t) const {
    detail::write_acc16<false>(*this, x, y, t);
}

constexpr int kMfmaBK = 64;                      // K depth of one LDS stage
constexpr int64_t kMfmaMaxLd = 1 << 20;          // direct-to-LDS paths: largest row pitch of A and B, in elements
constexpr int kMfmaRowBytes = 2 * kMfmaBK + 16;  // padded LDS row: 144 bytes

// LDS needed by matrix_multiply on bf16 operands.
template<int64_t BM, int64_t BN>
constexpr int64_t mfma_lds_bytes() {
    return 2 * (BM + BN) * kMfmaRowBytes;
}

namespace detail {

// The fast bf16 path: 256 x 256 tile, eight wavefronts, for either accumulator
// type (MfmaAcc16: v_mfma_f32_16x16x32_bf16, the one the pipeline uses;
// MfmaAcc<.., 8>: v_mfma_f32_32x32x16_bf16); tiles at the bottom and right
// edges of C may be partial, and so may the last stage of K.
//
// Both operands go from global memory STRAIGHT INTO LDS (buffer_load ... lds, 16
// bytes per lane, no register round trip, no LDS write instructions), two
// stages of 64 K each; all eight wavefronts issue the loads of stage k+1,
// compute stage k, wait for their loads and meet at one barrier.
//
//  * A stage: 256 rows x 128 bytes.  A load instruction fills 1 KiB of LDS in
//    lane order, so rows cannot be padded; instead the 16-byte chunk c of row
//    m is kept at position c ^ ((m >> 1) & 7), which spreads the sixteen rows
//    that one ds_read_b128 pass touches over all 64 banks.  The permutation
//    is applied on the GLOBAL side (each lane picks the chunk whose home is
//    its LDS slot) and stays inside 64-byte groups, so loads remain coalesced.
//  * B stage: 64 K rows x 512 bytes, kept as it lies in memory (columns
//    contiguous).  The MFMA wants K contiguous per column: ds_read_b64_tr_b16
//    transposes on the way out (inside each group of sixteen lanes, lane i
//    receives, as element j, element i % 4 of the 8 bytes addressed by lane
//    4 j + i / 4).  Chunk c of K row k sits at position c ^ (4 * (k & 3)).
//  * The two stages are two distinct static arrays: a single dynamic array
//    would make the compiler wait for the loads into one stage before any
//    LDS read of the other (it cannot tell them apart), serialising the two.
//
// Measured alternatives at 4096^3 (us): register-staged with one barrier per
// stage 167; two wavefront groups half a stage out of phase (one computing
// while the other moves data) 140; this one, with 64-bit lane addresses, 131;
// on v_mfma_f32_32x32x16_bf16 (MfmaAcc) 116-120; on v_mfma_f32_16x16x32_bf16
// (MfmaAcc16) 104-109, with its order of issue written out 101-106.
//
// THE KERNEL RUNS INTO THE POWER LIMIT: the two instructions need the same
// number of cycles (246 500 and 250 800 per launch and XCD, counted by
// GRBM_GUI_ACTIVE), but the clock settles at 2.05 GHz with the first and at
// 2.28-2.35 GHz with the second, and the time follows the clock.  Close to
// the clock's ceiling cycles count again: with the order of issue inside a
// stage written out (compute(), below) the 16 x 16 x 32 kernel takes 221 100
// cycles at 2.18 GHz, 101.3 us.  What did not help, each measured against the
// kernel as it is in one process: the K loop rotated so that the barrier
// stands before a stage's last sixteen instructions (they cover the wait for
// the next stage's first fragments), with the compiler's order or a written-out
// one (+2 to +3 %); the loads of the next stage spread among the first phase's
// matrix instructions instead of issued in front of them (+1 %); C stored in
// whole 128-byte lines (lanes p and p ^ 8 swapping a piece through DPP)
// instead of 64-byte halves (no difference).
template<int64_t BM, int64_t BN, int64_t KC, typename Acc>
__device__ __forceinline__ void mfma_direct(const GlobalView<BM, KC, uint16_t, true> &A,
                                            const GlobalView<KC, BN, uint16_t, true> &B, Acc &C) {
    static_assert(BM == 256 && BN == 256 && Acc::threads == 512 && Acc::WC == 4, "written for 256 x 256 tiles on eight wavefronts");
    constexpr int TM = Acc::TM, TN = Acc::TN;
    constexpr bool k16 = Acc::kTile == 16;  // v_mfma_f32_16x16x32_bf16 (MfmaAcc16) or v_mfma_f32_32x32x16_bf16 (MfmaAcc)
    constexpr int KSTEPS = kMfmaBK / (k16 ? 32 : 16);
    constexpr int A_BYTES = 256 * 128;
    constexpr int STAGE = A_BYTES + 64 * 512;
    typedef short v4s_t __attribute__((ext_vector_type(4)));
    typedef short v8s_t __attribute__((ext_vector_type(8)));
    __shared__ __attribute__((aligned(16))) unsigned char stage_even[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char stage_odd[STAGE];

    const int lane = lane_id();
    const int w = wave_in_block();
    const int64_t k_total = A.cols < B.rows ? A.cols : B.rows;
    // A last stage may be partial (its depth `tail` a multiple of 8, as rows of
    // A are whole 16-byte pieces): its missing part is ZERO in LDS, see issue().
    const int nk = (int)((k_total + kMfmaBK - 1) / kMfmaBK);
    const int tail = (int)(k_total % kMfmaBK);
    if (nk == 0 || A.rows <= 0 || B.cols <= 0) {  // workgroup-uniform
        return;
    }

    // Wavefront w issues A instructions 4w .. 4w+3 (8 rows each) and B
    // instructions 4w .. 4w+3 (2 K rows each) of every stage, as buffer loads:
    // descriptor and per-instruction byte offset live in scalar registers, the
    // lane's own offset is one of two constants (it depends on the parity of
    // the instruction only), so issuing a stage takes no vector ALU work.  It
    // matters: the SIMD hands its vector-ALU slot to the oldest wavefront, and
    // one that streams MFMAs starves the address arithmetic of the other
    // (64-bit lane addresses made this kernel 10 % slower).
    // Byte offsets are 32 bit: lda and ldb below kMfmaMaxLd elements.
    const int wu = __builtin_amdgcn_readfirstlane(w);
    // A tile at the bottom or right edge of C has fewer than 256 valid rows of
    // A or columns of B.  LDS slots past the edge are filled from the last
    // valid row / 8-column chunk instead (they only feed accumulators that the
    // insert does not write), so no load leaves the matrices.
    const int last_row_a = (int)A.rows - 1;
    const int last_chunk_b = ((int)B.cols - 1) / 8;
    int lane_off_a[4], lane_off_b[2];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        // A slot: row 8 i + lane / 8 (i = 4 w + j), position lane % 8, holds
        // chunk (lane % 8) ^ ((row >> 1) & 7) of that row
        const int row = 8 * (wu * 4 + j) + lane / 8;
        const int chunk_a = (lane % 8) ^ ((row >> 1) & 7);
        const int from_row = row < last_row_a ? row : last_row_a;
        lane_off_a[j] = (from_row * (int)A.lda + chunk_a * 8) * 2;
    }
#pragma unroll
    for (int odd = 0; odd < 2; odd++) {
        // B slot: K row 2 i + lane / 32, position lane % 32, holds chunk
        // (lane % 32) ^ (4 * (K row & 3)); the K row's parity class is that of j
        // (16 x 16 x 32: also ^ 2 where bit 3 of the K row is set, which is the parity of the wavefront:
        // the K row is 8 w + 2 j + lane / 32.  The two groups of sixteen lanes that one pass of a
        // transposing read serves then address K rows 8 apart, and would meet in the same banks.)
        const int chunk_b = (lane % 32) ^ (4 * ((2 * odd + lane / 32) & 3)) ^ (k16 ? 2 * (wu & 1) : 0);
        lane_off_b[odd] = ((lane / 32) * (int)B.lda + (chunk_b < last_chunk_b ? chunk_b : last_chunk_b) * 8) * 2;
    }
    // Raw 32-bit buffer descriptors whose num_records end at the last valid
    // element of the window: the hardware checks vector + scalar offset of
    // every dword against it, and a dword past it reads as ZERO (also into
    // LDS).  That is how K rows of B past the end of a partial last stage, and
    // the few elements past the end of the last row, become zeros without a
    // branch; chunks of A past K lie INSIDE the matrix (in the next row), so
    // the lanes that would fetch them are sent out of range instead.
    constexpr int kRawBuffer = 0x00020000;
    constexpr int kOutOfRange = 0x7FFF0000;
    const __amdgpu_buffer_rsrc_t desc_a =
        __builtin_amdgcn_make_buffer_rsrc((void *)A.data, 0, (int)((((int64_t)A.rows - 1) * A.lda + A.cols) * 2), kRawBuffer);
    const int row_bytes_b = (int)B.lda * 2;
    auto issue_from = [&](int kt, unsigned char *dst, const int (&off_a)[4]) {
        const int k0 = kt * (int)kMfmaBK;
        const int64_t left_b = (((int64_t)B.rows - 1 - k0) * B.lda + B.cols) * 2;  // bytes from this stage's first row to the end
        const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(B.data + (int64_t)k0 * B.lda), 0, (int)(left_b < 0 ? 0 : left_b < 0xFFFFFFFFll ? left_b : 0xFFFFFFFFll), kRawBuffer);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = wu * 4 + j;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_a, (__attribute__((address_space(3))) void *)(dst + (i * 1024)), 16,
                                                     off_a[j], k0 * 2, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = wu * 4 + j;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_b,
                                                     (__attribute__((address_space(3))) void *)(dst + (A_BYTES + i * 1024)),
                                                     16, lane_off_b[j & 1], 2 * i * row_bytes_b, 0, 0);
        }
    };
    auto issue = [&](int kt, unsigned char *dst) {
        if (tail != 0 && kt == nk - 1) {  // workgroup-uniform; at most once per call
            int off_tail[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int row = 8 * (wu * 4 + j) + lane / 8;
                const int chunk_a = (lane % 8) ^ ((row >> 1) & 7);
                off_tail[j] = chunk_a * 8 < tail ? lane_off_a[j] : kOutOfRange;
            }
            issue_from(kt, dst, off_tail);
        } else {
            issue_from(kt, dst, lane_off_a);
        }
    };

    // 32 x 32 x 16.  A fragment of this lane: row lane % 32 of each 32-row tile, K block
    // 2 s + lane / 32 of K step s.
    // 16 x 16 x 32.  Row lane % 16 of each 16-row tile, K block 4 s + lane / 16 of K step s (32 deep).
    constexpr int kRows = k16 ? 16 : 32;  // rows of A (columns of B) per instruction
    const int a_row_off = ((w / Acc::WC) * (int)Acc::WM + (lane % kRows)) * 128;
    const int a_swz = ((lane % kRows) >> 1) & 7;
    const int a_part = lane / kRows;
    // B fragment, 32 x 32 x 16: lane p of 16-lane group g addresses K row 16 s + 8 (g / 2) +
    // 4 q + p / 4, columns 16 (g % 2) + 4 (p % 4) .. + 3 of the 32-column tile;
    // the transposing read hands it K rows 8 (g / 2) + 4 q .. + 3 of column
    // 16 (g % 2) + p, which is what MFMA lane 16 g + p holds.
    // 16 x 16 x 32: K row 32 s + 8 g + 4 q + p / 4, columns 4 (p % 4) .. + 3 of the 16-column tile; the
    // read hands it K rows 8 g + 4 q .. + 3 of column p.
    const int g = lane / 16, p = lane % 16;
    const int b_col0 = (w % Acc::WC) * (int)Acc::WN + (k16 ? 0 : 16 * (g % 2));
    const int b_krow = (k16 ? 8 * g : 8 * (g / 2)) + p / 4;
    const int b_swz = (4 * (p / 4)) ^ (k16 ? 2 * (g & 1) : 0);  // (k & 3) == p / 4: the other terms are multiples of 4
    // Every LDS address below is ONE offset from the stage array: the compiler
    // tells the two stages apart only through short pointer chains.
    // (LDS pointers in their own address space from the array on: every conversion to a generic pointer and
    // back is a step in the chain along which the compiler keeps track of WHICH array an access goes to, and
    // it follows only a few; an access it cannot place waits for all loads into the other stage)
    typedef const __attribute__((address_space(3))) unsigned char *lds_bytes;
    auto load_a = [&](const unsigned char *stage_generic, int tm, int s) {
        lds_bytes stage = (lds_bytes)stage_generic;
        const int pos = ((k16 ? 4 : 2) * s + a_part) ^ a_swz;
        const int at = a_row_off + tm * kRows * 128 + pos * 16;
        return *(const __attribute__((address_space(3))) bf16x8_t *)(stage + at);
    };
    // The lane's own part of a B fragment's address is ONE value per column tile that the compiler may not
    // take apart (it would spread the sum over a chain of pointer steps, and lose track of the array at the
    // end of a long one): array + that value + a constant.
    int b_lane[TN];
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const int chunk = ((b_col0 + tn * kRows) / 8 + (p % 4) / 2) ^ b_swz;
        int v = b_krow * 512 + chunk * 16 + (p % 2) * 8;
        asm volatile("" : "+v"(v));
        b_lane[tn] = v;
    }
    auto load_b = [&](const unsigned char *stage_generic, int tn, int s) {
        lds_bytes lane_base = (lds_bytes)stage_generic + b_lane[tn];
        const int at = A_BYTES + (k16 ? 32 : 16) * s * 512;
        const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t *)(lane_base + at));
        const v4s_t hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t *)(lane_base + (at + 4 * 512)));
        const v8s_t both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        return __builtin_bit_cast(bf16x8_t, both);
    };
    auto compute = [&](const unsigned char *stage) {
        if constexpr (k16) {
            // Four phases per stage: (K step, upper or lower four row tiles).  The fragments of the next
            // phase are read while the sixteen instructions of this one run.
            constexpr int HALF = TM / 2;
            bf16x8_t af[2][HALF], bfr[2][TN];
#pragma unroll
            for (int t = 0; t < HALF; t++) {
                af[0][t] = load_a(stage, t, 0);
            }
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                bfr[0][tn] = load_b(stage, tn, 0);
            }
#pragma unroll
            for (int ph = 0; ph < 2 * KSTEPS; ph++) {
                const int s = ph / 2, h = ph % 2;
                if (ph + 1 < 2 * KSTEPS) {
                    const int ns = (ph + 1) / 2, nh = (ph + 1) % 2;
#pragma unroll
                    for (int t = 0; t < HALF; t++) {
                        af[(ph + 1) & 1][t] = load_a(stage, nh * HALF + t, ns);
                    }
                    if (nh == 0) {
#pragma unroll
                        for (int tn = 0; tn < TN; tn++) {
                            bfr[ns & 1][tn] = load_b(stage, tn, ns);
                        }
                    }
                }
#pragma unroll
                for (int t = 0; t < HALF; t++) {
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        // transposed: B's fragment first, so that a lane ends up with four consecutive columns
                        C.acc[h * HALF + t][tn] =
                            __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[s & 1][tn], af[ph & 1][t], C.acc[h * HALF + t][tn], 0, 0, 0);
                    }
                }
            }
            // THE ORDER OF ISSUE IS WRITTEN OUT (sched_group_barrier: the next n instructions of a kind).
            // Left to itself the compiler reads a fragment just before its first use -- eight matrix
            // instructions, two reads, a wait for them, eight more -- and what a wavefront loses to LDS latency
            // the other wavefront of the SIMD only partly makes up (4096^3: 105.6 -> 101.4 us, 108.1 -> 103.4 us
            // on a slower GPU).  Here: the twelve reads of the first phase; then, phase by phase, the reads of
            // the NEXT phase spread among the sixteen matrix instructions of this one.
            static_assert(HALF == 4 && TN == 4 && KSTEPS == 2, "the order of issue below is written out for these");
#define GERN_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define GERN_READ_THEN(n) GERN_SGB(0x100, 1); GERN_SGB(0x008, n)
            GERN_SGB(0x100, 12);
            GERN_READ_THEN(4); GERN_READ_THEN(4); GERN_READ_THEN(4); GERN_READ_THEN(4);
            GERN_READ_THEN(1); GERN_READ_THEN(1); GERN_READ_THEN(1); GERN_READ_THEN(1);
            GERN_READ_THEN(1); GERN_READ_THEN(1); GERN_READ_THEN(1); GERN_READ_THEN(1);
            GERN_READ_THEN(1); GERN_READ_THEN(1); GERN_READ_THEN(1); GERN_READ_THEN(1);
            GERN_SGB(0x008, 4);
            GERN_READ_THEN(4); GERN_READ_THEN(4); GERN_READ_THEN(4); GERN_READ_THEN(4);
            GERN_SGB(0x008, 16);
#undef GERN_READ_THEN
#undef GERN_SGB
        } else {
            bf16x8_t af[2][TM], bfr[2][TN];
#pragma unroll
            for (int tm = 0; tm < TM; tm++) {
                af[0][tm] = load_a(stage, tm, 0);
            }
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                bfr[0][tn] = load_b(stage, tn, 0);
            }
#pragma unroll
            for (int s = 0; s < KSTEPS; s++) {
                const int cur = s & 1, nxt = cur ^ 1;
                if (s + 1 < KSTEPS) {
#pragma unroll
                    for (int tm = 0; tm < TM; tm++) {
                        af[nxt][tm] = load_a(stage, tm, s + 1);
                    }
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        bfr[nxt][tn] = load_b(stage, tn, s + 1);
                    }
                }
#pragma unroll
                for (int tm = 0; tm < TM; tm++) {
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        C.acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[cur][tm], bfr[cur][tn], C.acc[tm][tn], 0, 0, 0);
                    }
                }
            }
        }
    };
    auto arrive = [&]() {
        // vmcnt(0) lgkmcnt(0): this wavefront's loads have landed in LDS and its
        // LDS reads are done; then everybody's.
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
    };

    issue(0, stage_even);
    arrive();
    for (int kt = 0; kt < nk; kt += 2) {
        if (kt + 1 < nk) {
            issue(kt + 1, stage_odd);
        }
        compute(stage_even);
        arrive();
        if (kt + 1 < nk) {
            if (kt + 2 < nk) {
                issue(kt + 2, stage_even);
            }
            compute(stage_odd);
            arrive();
        }
    }
}

}  // namespace detail

template<int64_t BM, int64_t BN, int64_t KC>
__device__ __forceinline__ void matrix_multiply(const GlobalView<BM, KC, uint16_t, true> &A,
                                                const GlobalView<KC, BN, uint16_t, true> &B, MfmaAcc16<BM, BN> &C) {
    detail::mfma_direct(A, B, C);
}

template<int64_t BM, int64_t BN, int64_t KC, int NW, bool EXACT>
__device__ __forceinline__ void matrix_multiply(const GlobalView<BM, KC, uint16_t, EXACT> &A,
                                                const GlobalView<KC, BN, uint16_t, EXACT> &B, MfmaAcc<BM, BN, NW> &C) {
    if constexpr (NW == 8 && EXACT && BM == 256 && BN == 256) {
        detail::mfma_direct(A, B, C);
        return;
    }
    using Acc = MfmaAcc<BM, BN, NW>;
    constexpr int T = Acc::threads;
    static_assert(BM <= 256 && BN <= 256, "tile shape");
    // Per stage, per thread: A_CHUNKS 16-byte pieces of A rows (8 bf16 along
    // K), B_TASKS 8-deep column pairs of B.
    constexpr int A_CHUNKS = (int)(BM * (kMfmaBK / 8) / T);
    constexpr int B_TASKS = (int)((BN / 2) * (kMfmaBK / 8) / T);
    static_assert(A_CHUNKS >= 1 && B_TASKS >= 1, "tile too small for the workgroup");
    constexpr int A_ROW_STEP = T / (kMfmaBK / 8);  // rows between a thread's consecutive A chunks
    constexpr int B_G_STEP = T / (int)(BN / 2);    // 8-deep K groups between a thread's consecutive B tasks
    static_assert(B_G_STEP >= 1 && B_G_STEP * B_TASKS == kMfmaBK / 8, "B staging covers the stage exactly");
    constexpr int STAGE_BYTES = (int)(BM + BN) * kMfmaRowBytes;
    constexpr int TM = Acc::TM, TN = Acc::TN;

    const int tid = (int)threadIdx.x;
    const int lane = lane_id();
    const int w = detail::wave_in_block();
    const int64_t k_total = A.cols < B.rows ? A.cols : B.rows;
    const int nk = (int)((k_total + kMfmaBK - 1) / kMfmaBK);
    if (nk == 0) {
        return;
    }

    const int a_row = tid / (kMfmaBK / 8), a_kc = tid % (kMfmaBK / 8);
    const int b_pair = tid % (int)(BN / 2), b_g = tid / (int)(BN / 2);
    const uint16_t *a_ptr = A.data + (int64_t)a_row * A.lda + a_kc * 8;
    const uint16_t *b_ptr = B.data + (int64_t)(8 * b_g) * B.lda + 2 * b_pair;
    const int a_step = A_ROW_STEP * (int)A.lda;    // elements between chunks
    const int b_step = 8 * B_G_STEP * (int)B.lda;  // elements between tasks
    const int b_ld = (int)B.lda;

    // Native vector types: selecting between two of HIP's uint4 structs
    // (cond ? a : b) takes their addresses and sends both to scratch memory.
    u32x4_t ra[A_CHUNKS];
    uint32_t rb[B_TASKS][8];

    auto fetch = [&](int kt) {
        const int64_t k0 = (int64_t)kt * kMfmaBK;
        {
            // Every access under a predicate (tiles may be ragged).  A row
            // of A is read in whole 16-byte pieces and a row of B in whole
            // column pairs (the caller guarantees K % 8 == 0 and N % 2 == 0).
#pragma unroll
            for (int j = 0; j < A_CHUNKS; j++) {
                const bool ok = (a_row + j * A_ROW_STEP < A.rows) && (k0 + a_kc * 8 < k_total);
                ra[j] = u32x4_t{0u, 0u, 0u, 0u};
                if (ok) {
                    ra[j] = *reinterpret_cast<const u32x4_t *>(a_ptr + k0 + j * a_step);
                }
            }
            const uint16_t *bp = b_ptr + k0 * B.lda;
            const bool col_ok = 2 * b_pair < B.cols;
#pragma unroll
            for (int j = 0; j < B_TASKS; j++) {
                const int64_t kk = k0 + 8 * (b_g + j * B_G_STEP);
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const bool ok = col_ok && (kk + q < k_total);
                    rb[j][q] = ok ? *reinterpret_cast<const uint32_t *>(bp + j * b_step + q * b_ld) : 0u;
                }
            }
        }
    };

    auto stash = [&](int buf) {
        unsigned char *a_lds = gern_lds + buf * STAGE_BYTES + a_row * kMfmaRowBytes + a_kc * 16;
        unsigned char *b_lds = gern_lds + buf * STAGE_BYTES + (int)BM * kMfmaRowBytes + (2 * b_pair) * kMfmaRowBytes + b_g * 16;
#pragma unroll
        for (int j = 0; j < A_CHUNKS; j++) {
            *reinterpret_cast<u32x4_t *>(a_lds + j * A_ROW_STEP * kMfmaRowBytes) = ra[j];
        }
#pragma unroll
        for (int j = 0; j < B_TASKS; j++) {
            // rb[j][q] = {B[k+q][n] (low half), B[k+q][n+1] (high half)}: split
            // into the K-contiguous vectors of column n and column n+1.
            u32x4_t lo, hi;
            lo.x = __builtin_amdgcn_perm(rb[j][1], rb[j][0], 0x05040100u);
            lo.y = __builtin_amdgcn_perm(rb[j][3], rb[j][2], 0x05040100u);
            lo.z = __builtin_amdgcn_perm(rb[j][5], rb[j][4], 0x05040100u);
            lo.w = __builtin_amdgcn_perm(rb[j][7], rb[j][6], 0x05040100u);
            hi.x = __builtin_amdgcn_perm(rb[j][1], rb[j][0], 0x07060302u);
            hi.y = __builtin_amdgcn_perm(rb[j][3], rb[j][2], 0x07060302u);
            hi.z = __builtin_amdgcn_perm(rb[j][5], rb[j][4], 0x07060302u);
            hi.w = __builtin_amdgcn_perm(rb[j][7], rb[j][6], 0x07060302u);
            // Column n goes to LDS row n, column n+1 to row n+1.  Eight
            // consecutive lanes must hit eight different 16-byte bank groups;
            // rows 2p (p = 0..7) only reach four, so lanes with bit 2 of p set
            // write their odd row first: rows 0,2,4,6,9,11,13,15.
            const bool odd_first = (b_pair & 4) != 0;
            *reinterpret_cast<u32x4_t *>(b_lds + (odd_first ? kMfmaRowBytes : 0) + j * B_G_STEP * 16) = odd_first ? hi : lo;
            *reinterpret_cast<u32x4_t *>(b_lds + (odd_first ? 0 : kMfmaRowBytes) + j * B_G_STEP * 16) = odd_first ? lo : hi;
        }
    };

    // Workgroups of different XCDs start their walk over K at different steps
    // (and wrap around).  With a power-of-two row pitch the rows of one K step
    // all fall into the same memory channel; if every workgroup asked for the
    // same step at once, one channel would serve the whole chip.  The
    // workgroups of ONE XCD (launch number modulo 8) walk in step, so that the
    // panels they share are fetched into that XCD's L2 once: with a start per
    // workgroup the fp32 kernel read its operands 20 times over (4.0 GB per
    // 4096^3 product), with a start per XCD 0.78 GB, and ran 3 % faster.  The
    // sum over K does not depend on where the walk starts.
    const int k_shift = (int)((((blockIdx.x + gridDim.x * blockIdx.y) % 8u) * (unsigned)nk) / 8u);
    auto step_of = [&](int kt) {
        const int s = kt + k_shift;
        return s >= nk ? s - nk : s;
    };

    fetch(step_of(0));
    stash(0);
    __syncthreads();

    // This lane's fragment addresses inside a stage: row (lane % 32) of each
    // 32-row MFMA tile, 16 bytes at K offset 8 * (lane / 32) of each K step.
    const int a_frag = ((w / Acc::WC) * (int)Acc::WM + (lane % 32)) * kMfmaRowBytes + (lane / 32) * 16;
    const int b_frag = (int)BM * kMfmaRowBytes + ((w % Acc::WC) * (int)Acc::WN + (lane % 32)) * kMfmaRowBytes + (lane / 32) * 16;

    for (int kt = 0; kt < nk; kt++) {
        if (kt + 1 < nk) {
            fetch(step_of(kt + 1));
        }
        const unsigned char *stage = gern_lds + (kt & 1) * STAGE_BYTES;
        if constexpr (NW == 4) {
            // One wavefront per SIMD: read the next K step's fragments while
            // this step's MFMAs run.
            bf16x8_t af[2][TM], bfr[2][TN];
#pragma unroll
            for (int tm = 0; tm < TM; tm++) {
                af[0][tm] = *reinterpret_cast<const bf16x8_t *>(stage + a_frag + tm * 32 * kMfmaRowBytes);
            }
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                bfr[0][tn] = *reinterpret_cast<const bf16x8_t *>(stage + b_frag + tn * 32 * kMfmaRowBytes);
            }
#pragma unroll
            for (int s = 0; s < kMfmaBK / 16; s++) {
                const int cur = s & 1, nxt = cur ^ 1;
                if (s + 1 < kMfmaBK / 16) {
#pragma unroll
                    for (int tm = 0; tm < TM; tm++) {
                        af[nxt][tm] = *reinterpret_cast<const bf16x8_t *>(stage + a_frag + tm * 32 * kMfmaRowBytes + (s + 1) * 32);
                    }
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        bfr[nxt][tn] = *reinterpret_cast<const bf16x8_t *>(stage + b_frag + tn * 32 * kMfmaRowBytes + (s + 1) * 32);
                    }
                }
#pragma unroll
                for (int tm = 0; tm < TM; tm++) {
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        C.acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[cur][tm], bfr[cur][tn], C.acc[tm][tn], 0, 0, 0);
                    }
                }
            }
        } else {
            // Two wavefronts per SIMD cover each other's LDS waits; single
            // fragment buffers keep each within half the register file.
#pragma unroll
            for (int s = 0; s < kMfmaBK / 16; s++) {
                bf16x8_t af[TM], bfr[TN];
#pragma unroll
                for (int tm = 0; tm < TM; tm++) {
                    af[tm] = *reinterpret_cast<const bf16x8_t *>(stage + a_frag + tm * 32 * kMfmaRowBytes + s * 32);
                }
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    bfr[tn] = *reinterpret_cast<const bf16x8_t *>(stage + b_frag + tn * 32 * kMfmaRowBytes + s * 32);
                }
#pragma unroll
                for (int tm = 0; tm < TM; tm++) {
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        C.acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[tm], bfr[tn], C.acc[tm][tn], 0, 0, 0);
                    }
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
// fp32 x fp32 -> fp32 on the matrix cores
// ---------------------------------------------------------------------------
// v_mfma_f32_32x32x2_f32 multiplies in fp32 (no reduced-precision inputs) at
// 256 flop per cycle and CU, twice what the vector ALU reaches without packed
// instructions.  256 x 256 tile, eight wavefronts as 4 x 2: wavefront (wr, wc)
// owns rows [64 wr, 64 wr + 64) as two MFMA row tiles and columns
// [128 wc, 128 wc + 128) as four INTERLEAVED column tiles: tile tn, MFMA
// column j is column 4 j + tn.  A lane then gets the B operands of its four
// column tiles with one 16-byte LDS read of four consecutive columns, and
// holds four consecutive columns of C per row: 16-byte stores.
//
// acc[tm][tn][i] of lane l: row 64 wr + 32 tm + 8 (i / 4) + 4 (l / 32) + i % 4,
// column 128 wc + 4 (l % 32) + tn.
template<int64_t BM, int64_t BN>
struct MfmaAccF32 {
    static_assert(BM == 256 && BN == 256, "the fp32 matrix-core gernel is written for 256 x 256 tiles");
    static constexpr int WR = 4, WC = 2;
    static constexpr int TM = 2, TN = 4;
    static constexpr int threads = 8 * kWaveSize;
    f32x16_t acc[TM][TN];

    __device__ __forceinline__ void destroy() {
    }
};

template<int64_t BM, int64_t BN>
__device__ __forceinline__ MfmaAccF32<BM, BN> MatrixF32::load_acc_mfma8_f32(int64_t, int64_t) const {
    MfmaAccF32<BM, BN> t;
#pragma unroll
    for (int tm = 0; tm < MfmaAccF32<BM, BN>::TM; tm++) {
#pragma unroll
        for (int tn = 0; tn < MfmaAccF32<BM, BN>::TN; tn++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                t.acc[tm][tn][i] = 0.f;
            }
        }
    }
    return t;
}

namespace detail {

template<bool ADD, int64_t BM, int64_t BN>
__device__ __forceinline__ void write_acc_f32(const MatrixF32 &m, int64_t x, int64_t y, const MfmaAccF32<BM, BN> &t) {
    using Acc = MfmaAccF32<BM, BN>;
    const int lane = lane_id();
    const int w = wave_in_block();
    const int64_t r0 = x + (int64_t)(w / Acc::WC) * 64 + 4 * (lane / 32);
    const int64_t c0 = y + (int64_t)(w % Acc::WC) * 128 + 4 * (lane % 32);
#pragma unroll
    for (int tm = 0; tm < Acc::TM; tm++) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int64_t rr = r0 + tm * 32 + 8 * (i / 4) + (i % 4);
            if (rr >= m.row) {
                continue;
            }
            float *p = m.data + rr * m.lda + c0;
            float4 v = make_float4(t.acc[tm][0][i], t.acc[tm][1][i], t.acc[tm][2][i], t.acc[tm][3][i]);
            if (c0 + 3 < m.col && ((((uint64_t)p) & 15u) == 0)) {
                if (ADD) {
                    const float4 o = *reinterpret_cast<const float4 *>(p);
                    v = make_float4(o.x + v.x, o.y + v.y, o.z + v.z, o.w + v.w);
                    *reinterpret_cast<float4 *>(p) = v;
                } else {
                    store_result16<kThroughStores>(m.data, (m.row - 1) * m.lda + m.col, rr * m.lda + c0, v);
                }
            } else {
                const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (c0 + q < m.col) {
                        p[q] = ADD ? p[q] + e[q] : e[q];
                    }
                }
            }
        }
    }
}

// Same structure as mfma_direct (the bf16 kernel above): both operands loaded
// straight into LDS with scalar-addressed buffer loads, two static 64 KiB
// stages, one barrier per stage; a stage is 32 deep in K.
//
//  * A stage: 256 rows x 128 bytes (32 floats); 16-byte chunk c of row m at
//    position c ^ ((m >> 1) & 7).  Lane l of an MFMA holds row l % 32 and one
//    of the two K indices of the instruction; lanes 0-31 take chunk 2 b, lanes
//    32-63 chunk 2 b + 1 of K block b (8 deep), and use the chunk's four
//    floats in four consecutive MFMAs: K index 8 b + 4 (l / 32) + j in MFMA j.
//  * B stage: 32 K rows x 1024 bytes as they lie in memory.  For MFMA j a
//    lane reads the four consecutive columns 128 wc + 4 (l % 32) .. + 3 of K
//    row 8 b + 4 (l / 32) + j: one operand for each of its four column tiles.
//  Six 16-byte LDS reads feed 32 MFMAs of 64 cycles each.
template<int64_t BM, int64_t BN, int64_t KC>
__device__ __forceinline__ void mfma_direct_f32(const GlobalView<BM, KC, float, true> &A,
                                                const GlobalView<KC, BN, float, true> &B, MfmaAccF32<BM, BN> &C) {
    using Acc = MfmaAccF32<BM, BN>;
    constexpr int BK = 32;
    constexpr int A_BYTES = 256 * 128;
    constexpr int STAGE = A_BYTES + BK * 1024;
    typedef float f32x4_native __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) unsigned char stage_even_f32[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char stage_odd_f32[STAGE];

    const int lane = lane_id();
    const int w = wave_in_block();
    const int64_t k_total = A.cols < B.rows ? A.cols : B.rows;
    // A partial last stage (depth `tail`, a multiple of 4) is zero-filled, as in mfma_direct.
    const int nk = (int)((k_total + BK - 1) / BK);
    const int tail = (int)(k_total % BK);
    if (nk == 0 || A.rows <= 0 || B.cols <= 0) {  // workgroup-uniform
        return;
    }
    const int wu = __builtin_amdgcn_readfirstlane(w);
    // Slots past the bottom / right edge of a partial tile are filled from the
    // last valid row / 16-byte chunk (they feed only accumulators that the
    // insert does not write), so no load leaves the matrices.
    const int last_row_a = (int)A.rows - 1;
    const int last_chunk_b = ((int)B.cols - 1) / 4;
    int lane_off_a[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = 8 * (wu * 4 + j) + lane / 8;
        const int chunk = (lane % 8) ^ ((row >> 1) & 7);
        lane_off_a[j] = ((row < last_row_a ? row : last_row_a) * (int)A.lda + chunk * 4) * 4;
    }
    const int lane_off_b = (lane < last_chunk_b ? lane : last_chunk_b) * 16;
    // Descriptors that end at the last valid element of each window: dwords
    // past it (K rows of B beyond a partial last stage, the end of the last
    // row) read as zero; lanes of A past K are sent out of range (mfma_direct).
    constexpr int kRawBuffer = 0x00020000;
    constexpr int kOutOfRange = 0x7FFF0000;
    const __amdgpu_buffer_rsrc_t desc_a =
        __builtin_amdgcn_make_buffer_rsrc((void *)A.data, 0, (int)((((int64_t)A.rows - 1) * A.lda + A.cols) * 4), kRawBuffer);
    const int row_bytes_b = (int)B.lda * 4;
    // Wavefront w issues A instructions 4w .. 4w+3 (8 rows each) and B
    // instructions 4w .. 4w+3 (one K row each) of every stage.  What a stage's
    // loads need is computed apart from the loads themselves (Loads), so that
    // the arithmetic can stand before the barrier that the loads follow.
    // The lanes' A offsets for a partial last stage: chunks past K are sent out of range.
    int lane_off_a_tail[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = 8 * (wu * 4 + j) + lane / 8;
        const int chunk = (lane % 8) ^ ((row >> 1) & 7);
        lane_off_a_tail[j] = (tail == 0 || chunk * 4 < tail) ? lane_off_a[j] : kOutOfRange;
    }
    struct Loads {
        __amdgpu_buffer_rsrc_t desc_b;
        int k0_bytes;
        int off_a[4];
    };
    auto prepare = [&](int kt) {
        Loads l;
        const int k0 = kt * BK;
        const int64_t left_b = k0 < (int64_t)B.rows ? (((int64_t)B.rows - 1 - k0) * B.lda + B.cols) * 4 : 0;  // 0: all zeros
        l.desc_b = __builtin_amdgcn_make_buffer_rsrc((void *)(B.data + (int64_t)k0 * B.lda), 0,
                                                     (int)(left_b < 0xFFFFFFFFll ? left_b : 0xFFFFFFFFll), kRawBuffer);
        l.k0_bytes = k0 * 4;
        // workgroup-uniform, and selects rather than branches, so that a stage stays one block of code; a stage
        // past K (the loop below takes stages in pairs) is filled with zeros: every lane out of range
        const bool partial = tail != 0 && kt == nk - 1;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            l.off_a[j] = kt >= nk ? kOutOfRange : partial ? lane_off_a_tail[j] : lane_off_a[j];
        }
        return l;
    };
    auto issue = [&](const Loads &l, unsigned char *dst) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = wu * 4 + j;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_a, (__attribute__((address_space(3))) void *)(dst + (i * 1024)), 16,
                                                     l.off_a[j], l.k0_bytes, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = wu * 4 + j;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l.desc_b,
                                                     (__attribute__((address_space(3))) void *)(dst + (A_BYTES + i * 1024)),
                                                     16, lane_off_b, i * row_bytes_b, 0, 0);
        }
    };

    const int half = lane / 32;
    const int a_row = (w / Acc::WC) * 64 + (lane % 32);
    const int a_swz = ((lane % 32) >> 1) & 7;  // rows 64 wr + 32 tm + lane % 32: the other terms are multiples of 16
    const int b_off = A_BYTES + (4 * half) * 1024 + ((w % Acc::WC) * 128 + 4 * (lane % 32)) * 4;
    // The fragments of K block kb (8 deep) of a stage: two reads for A, four for B.
    auto read_block = [&](const unsigned char *stage, int kb, f32x4_native (&a)[Acc::TM], f32x4_native (&b)[4]) {
#pragma unroll
        for (int tm = 0; tm < Acc::TM; tm++) {
            const int at = (a_row + tm * 32) * 128 + (((2 * kb + half) ^ a_swz) * 16);
            a[tm] = *reinterpret_cast<const f32x4_native *>(stage + at);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int at = b_off + (8 * kb + j) * 1024;
            b[j] = *reinterpret_cast<const f32x4_native *>(stage + at);
        }
    };
    // and their 32 matrix instructions (64 cycles each)
    auto multiply_block = [&](const f32x4_native (&a)[Acc::TM], const f32x4_native (&b)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int tm = 0; tm < Acc::TM; tm++) {
#pragma unroll
                for (int tn = 0; tn < Acc::TN; tn++) {
                    C.acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm][j], b[j][tn], C.acc[tm][tn], 0, 0, 0);
                }
            }
        }
    };
    auto arrive = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
    };

    // A stage is four K blocks, and the fragments of a block are read WHILE THE BLOCK BEFORE IT IS MULTIPLIED
    // (two sets of fragment registers, p and q).  The stage's one barrier stands before its last block: by then
    // every wavefront holds that block's fragments in registers, so the stage's LDS can be given to the loads of
    // the stage after the next, and the first block of the next stage (whose loads were issued a stage ago) is
    // read behind the barrier, under the 32 matrix instructions of the last block.  Left to the compiler's
    // order, every block began with its own reads and a wait for them, four times per stage and on both
    // wavefronts of a SIMD at once (they leave the barrier together): 8.5 % of the launch without a matrix
    // instruction in flight; about 5 % now.  The order is written out with sched_group_barrier (0x008 matrix
    // instruction, 0x100 LDS read, 0x010 memory instruction), one region per side of the barrier; the
    // arithmetic for the loads (prepare) stands in the region before the barrier.  Measured, 4096^3, same
    // process, alternating (us per launch; the order the compiler chose before: 952): a block's six reads one
    // matrix instruction apart, two apart or back to back 921-924, five apart (spread over the block) 930; the
    // eight loads three or two matrix instructions apart 918-919, in pairs 923, back to back 929-936, the
    // four loads of B moved into the next stage's first block 930 against 925.  Without the loads the loop
    // takes 901-909, without the barrier 4 us less: what is left is what the loads and reads cost in issue.
    f32x4_native ap[Acc::TM], bp[4], aq[Acc::TM], bq[4];
#define GERN_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define GERN_SIX_READS_EVERY(n) \
    GERN_SGB(0x100, 1); GERN_SGB(0x008, n); GERN_SGB(0x100, 1); GERN_SGB(0x008, n); GERN_SGB(0x100, 1); GERN_SGB(0x008, n); \
    GERN_SGB(0x100, 1); GERN_SGB(0x008, n); GERN_SGB(0x100, 1); GERN_SGB(0x008, n); GERN_SGB(0x100, 1); GERN_SGB(0x008, n)
#define GERN_EIGHT_LOADS_EVERY(n) \
    GERN_SGB(0x010, 1); GERN_SGB(0x008, n); GERN_SGB(0x010, 1); GERN_SGB(0x008, n); GERN_SGB(0x010, 1); GERN_SGB(0x008, n); \
    GERN_SGB(0x010, 1); GERN_SGB(0x008, n); GERN_SGB(0x010, 1); GERN_SGB(0x008, n); GERN_SGB(0x010, 1); GERN_SGB(0x008, n); \
    GERN_SGB(0x010, 1); GERN_SGB(0x008, n); GERN_SGB(0x010, 1); GERN_SGB(0x008, n)
    // On entry p holds block 0 of `cur`; on exit, block 0 of `nxt`.  Stage kt + 2 is loaded into `cur`.
    auto stage = [&](unsigned char *cur, const unsigned char *nxt, int kt) {
        const Loads after_next = prepare(kt + 2);
        read_block(cur, 1, aq, bq);
        multiply_block(ap, bp);
        read_block(cur, 2, ap, bp);
        multiply_block(aq, bq);
        read_block(cur, 3, aq, bq);
        multiply_block(ap, bp);
        GERN_SGB(0x008, 2); GERN_SIX_READS_EVERY(2); GERN_SGB(0x008, 18);
        GERN_SGB(0x008, 2); GERN_SIX_READS_EVERY(2); GERN_SGB(0x008, 18);
        GERN_SGB(0x008, 2); GERN_SIX_READS_EVERY(2); GERN_SGB(0x008, 18);
        __builtin_amdgcn_sched_barrier(0);
        arrive();
        read_block(nxt, 0, ap, bp);
        issue(after_next, cur);
        multiply_block(aq, bq);
        GERN_SGB(0x008, 1); GERN_SIX_READS_EVERY(1); GERN_EIGHT_LOADS_EVERY(3); GERN_SGB(0x008, 1);
    };
#undef GERN_EIGHT_LOADS_EVERY
#undef GERN_SIX_READS_EVERY
#undef GERN_SGB

    // Stages are taken in pairs, one per LDS array, in a loop without a branch inside: when the number of
    // stages is odd the last pair's second stage is all zeros (its loads are sent out of range, above), and
    // the loads and reads that the last stages issue for stages past K fetch nothing and feed nothing.
    issue(prepare(0), stage_even_f32);
    arrive();
    issue(prepare(1), stage_odd_f32);
    read_block(stage_even_f32, 0, ap, bp);
    for (int kt = 0; kt < nk; kt += 2) {
        stage(stage_even_f32, stage_odd_f32, kt);
        stage(stage_odd_f32, stage_even_f32, kt + 1);
    }
    arrive();  // no load into LDS is in flight when the next call begins
}

}  // namespace detail

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::add_acc(int64_t x, int64_t y, const MfmaAccF32<BM, BN> &t) const {
    detail::write_acc_f32<true>(*this, x, y, t);
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::store_acc(int64_t x, int64_t y, const MfmaAccF32<BM, BN> &t) const {
    detail::write_acc_f32<false>(*this, x, y, t);
}

template<int64_t BM, int64_t BN, int64_t KC>
__device__ __forceinline__ void matrix_multiply(const GlobalView<BM, KC, float, true> &A,
                                                const GlobalView<KC, BN, float, true> &B, MfmaAccF32<BM, BN> &C) {
    detail::mfma_direct_f32(A, B, C);
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

// Like the MFMA tile, a deferred update of C: zero at query, added to
// (add_acc) or written over (store_acc) C at insert.
template<int64_t BM, int64_t BN>
__device__ __forceinline__ FmaAcc<BM, BN> MatrixF32::load_acc_fma(int64_t, int64_t) const {
    FmaAcc<BM, BN> t;
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            t.acc[i][j] = 0.f;
        }
    }
    return t;
}

namespace detail {

template<bool ADD, int64_t BM, int64_t BN>
__device__ __forceinline__ void write_fma_acc(const MatrixF32 &m, int64_t x, int64_t y, const FmaAcc<BM, BN> &t) {
    for_each_fma_acc([&](int i, int j, int64_t r, int64_t c) {
        const int64_t rr = x + r, cc = y + c;
        float *p = m.data + rr * m.lda + cc;
        if (rr < m.row && cc + 3 < m.col && ((((uint64_t)p) & 15u) == 0)) {
            float4 v = make_float4(t.acc[i][j], t.acc[i][j + 1], t.acc[i][j + 2], t.acc[i][j + 3]);
            if (ADD) {
                const float4 o = *reinterpret_cast<const float4 *>(p);
                v = make_float4(o.x + v.x, o.y + v.y, o.z + v.z, o.w + v.w);
            }
            *reinterpret_cast<float4 *>(p) = v;
        } else {
            for (int e = 0; e < 4; e++) {
                if (rr < m.row && cc + e < m.col) {
                    p[e] = ADD ? p[e] + t.acc[i][j + e] : t.acc[i][j + e];
                }
            }
        }
    });
}

}  // namespace detail

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::store_acc(int64_t x, int64_t y, const FmaAcc<BM, BN> &t) const {
    detail::write_fma_acc<false>(*this, x, y, t);
}

template<int64_t BM, int64_t BN>
__device__ __forceinline__ void MatrixF32::add_acc(int64_t x, int64_t y, const FmaAcc<BM, BN> &t) const {
    detail::write_fma_acc<true>(*this, x, y, t);
}

constexpr int kFmaBK = 16;
constexpr int kFmaLd = 128 + 4;  // padded LDS row, in floats

template<int64_t BM, int64_t BN>
constexpr int64_t fma_lds_bytes() {
    return 2 * 2 * kFmaBK * kFmaLd * 4;
}

template<int64_t BM, int64_t BN, int64_t KC>
__device__ __forceinline__ void matrix_multiply(const GlobalView<BM, KC, float, false> &A,
                                                const GlobalView<KC, BN, float, false> &B, FmaAcc<BM, BN> &C) {
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
    // The workgroups of one XCD walk over K in step (see the MFMA gernel above);
    // the eight XCDs start an eighth of K apart.
    const int k_shift = (int)((((blockIdx.x + gridDim.x * blockIdx.y) % 8u) * (unsigned)nk) / 8u);
    auto step_of = [&](int kt) {
        const int s = kt + k_shift;
        return s >= nk ? s - nk : s;
    };
    fetch(step_of(0));
    stash(0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        if (kt + 1 < nk) {
            fetch(step_of(kt + 1));
        }
        const float *a_lds = lds + (kt & 1) * STAGE_FLOATS;
        const float *b_lds = a_lds + kFmaBK * kFmaLd;
        // Four K steps per loop body: enough independent FMAs to cover the
        // LDS reads of the next step.  Unrolling all sixteen makes the compiler
        // hoist every read and spread over 384 registers (measured: 40 instead
        // of 72 TFLOP/s).
#pragma unroll 4
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
