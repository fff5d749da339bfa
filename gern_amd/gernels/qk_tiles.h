// Fused S = softmax_rows(scale * Q K^T) on 256 x 256 tiles of S, one per
// workgroup, for head dimensions that are multiples of 64.
//
// The row-block gernels of gernels/qk_softmax.h give a workgroup sixteen whole
// rows of S, so every workgroup streams ALL of K out of L2 (256 MiB of L2
// traffic at 4096 x 4096 x 128: half of that kernel's time).  Here a
// workgroup owns a 256 x 256 tile, reads 64 KiB of Q and 64 KiB of K once, and
// the workgroups of a row block combine their row statistics through global
// memory while the tiles wait in registers:
//
//   qk_scaled                    MFMA: the tile's logits, kept as raw accumulators plus
//                                the factor that turns them into log2 units
//   softmax_rows_across_tiles    per row of the tile: maximum m, e = 2^(x - m), sum s
//                                of e; publishes (m, s), waits for the same from the
//                                other tiles of the row block, scales e by
//                                2^(m - M) / S with M, S the statistics of the whole
//                                row, and stores
//
// so a softmax over tiled rows is the five stages of the reference's softmax
// gernels (apps/common/impl/impl.h:7-188: max, subtract, exp, sum, divide) with
// the two reductions finished across workgroups, as the reference's
// grid_reduce_total finishes a sum across blocks with a device-scope atomic
// (gernels/cccl/wrappers/reduce_wrappers.cuh:42-61).  The five stages are ONE
// gernel here because they are pipelined over the two 16-row halves of a
// wavefront's rows: the statistics of the first half are on their way to the
// other workgroups while the exponentials of the second are computed, and the
// first half is being stored while the second waits for its statistics (as
// three gernels with one exchange for all rows: 25.1 us at 4096 x 4096 x 128;
// this way 22.2 us, measured in one process).
//
// Eight wavefronts; wavefront w owns rows [32 w, 32 w + 32) of the tile and all
// 256 columns, as 2 x 16 v_mfma_f32_16x16x32_bf16 tiles.  MFMA column j of
// tile tn = 4 g + t stands for key 64 g + 4 j + t, so a lane holds four
// consecutive columns of S per group g and stores them with one 16-byte store.
//
// The exchange.  An entry is one 64-bit word per (row, column block): s in the
// upper half, below it m as a sixteen-bit integer (a row is shifted by
// the floor of its largest logit in log2 units: any shift near the maximum
// serves, and a whole number makes 2^(m - M) an exact power of two), and a
// sixteen-bit tag.  The tag is the launch's number, which is kept in device
// memory next to the entries and advanced by the last wavefront of every
// launch.  An entry says by itself whether it belongs to this launch: nothing
// is cleared between launches, nothing is passed from the host (a captured
// launch can be replayed), and no counter sits between the writes and the
// reads.  When the number wraps around (kRowStatsTagPeriod launches) that last
// wavefront clears all entries, so a tag left behind by an older launch of
// another shape is never mistaken for a new one.  Entries are written and read
// with agent-scope atomic accesses, which go to the memory side past the
// caches that are private to an XCD; no cache is written back or invalidated.
// Such reads run at about 3 TB/s over the whole GPU, and every tile reads the
// entries of its whole row block, so the size of an entry is what the exchange
// costs: 8 MiB and 2.5 us at 4096 x 4096 (entries of 16 bytes that held m as a
// float: twice that).  Each wavefront polls the sixteen entries of its own 32
// rows on its own.  Workgroup ids run along the columns, so the workgroups of
// a row block are dispatched together; a workgroup waits only for workgroups
// of its own row block, and those never wait for a later one.  The wait is
// bounded all the same: after spin_limit polls a wavefront gives up and stores
// NaN in its rows.  Logits beyond +-32767 in log2 units (22 000 in natural
// units) do not fit an entry; their rows come out as NaN.  Neither goes
// unnoticed by the host: state[2] counts the wavefronts that gave up and
// state[3] the (row, column block) pairs whose shift did not fit or whose
// logits were not all numbers, for the host to read and clear after the launch (the reference
// checks for an error after every launch,
// include/gern/codegen/helpers/check_last_error.h:7-18).
//
// Two launches that use the same exchange must not overlap in time.
#pragma once

#include "gernels/mm.h"
#include "gernels/softmax.h"

namespace gernels {

typedef float score_f32x4_t __attribute__((ext_vector_type(4)));

// Launch numbers run from 0 to kRowStatsTagPeriod - 1; a tag is the number + 1,
// and 0 is a word that was never written.
#ifndef GERN_QK_TAG_PERIOD
#define GERN_QK_TAG_PERIOD 65535u
#endif
constexpr unsigned int kRowStatsTagPeriod = GERN_QK_TAG_PERIOD;

// What the launch passes by value (the host fills in a struct of the same
// layout): `entries` holds `capacity` entries of 8 bytes, at least rows x
// pitch for the padded row count of the launch, pitch >= the number of column
// blocks; state[0] is the launch number, state[1] counts the workgroups that
// are done, state[2] the wavefronts that gave up waiting and state[3] the
// (row, column block) pairs whose logits did not fit an entry (the host reads
// and clears these two).  All of it starts as zeros.
struct RowStatsSession {
    unsigned long long *entries;
    unsigned int *state;
    int pitch;
    int spin_limit;
    long long capacity;
    unsigned int tag;
};

struct RowStatsExchange {
    unsigned long long *entries;
    unsigned int *state;
    int pitch;
    int spin_limit;
    long long capacity;

    // Reads the launch number.  The generated kernel calls this before the
    // first load of the tile, so the round trip hides behind those.
    __device__ __forceinline__ RowStatsSession open() const {
        const unsigned int n = __hip_atomic_load(state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return RowStatsSession{entries, state, pitch, spin_limit, capacity, n % kRowStatsTagPeriod + 1u};
    }
};

namespace detail {
// Wavefronts of the workgroup that are done with the exchange.  qk_scaled clears
// it ahead of its first barrier and softmax_rows_across_tiles counts in it, so
// that the exchange needs no barrier of its own: the wavefronts of a workgroup
// finish their exponentials up to a microsecond or two apart (a SIMD serves its older
// wavefront first), and a wavefront exchanges only with its namesakes in the
// other tiles of the row block, so the early ones are storing their rows while
// the late ones still compute.
__shared__ unsigned int row_stats_waves_done;
}  // namespace detail

// A 256 x 256 tile of scores spread over eight wavefronts: acc[tm][4 g + t][i]
// is row 32 w + 16 tm + 4 (lane / 16) + i, column 64 g + 4 (lane % 16) + t,
// in units of `unit` (value = acc * unit) as qk_scaled leaves it, plain afterwards.
// shift / sum: the statistics of the lane's eight rows over the tile's columns.
template<int64_t R, int64_t C>
struct ScoreTile {
    static_assert(R == 256 && C == 256, "score tiles are 256 x 256");
    static constexpr int64_t rows = R;
    static constexpr int64_t cols = C;
    score_f32x4_t acc[2][16];
    float shift[2][4];
    float sum[2][4];
    float unit;
    int valid_cols;  // columns of the tile that exist (keys)
    // A view of a matrix (view_score_tile): the matrix and where the tile's first
    // element lies in it.  A gernel may write its rows through the view as they
    // become final; `stored` then tells store_score_tile that nothing is left.
    MatrixF32 home;
    int row0, col0;
    bool stored;

    __device__ __forceinline__ void destroy() {
    }
};

template<int64_t R, int64_t C>
__device__ __forceinline__ ScoreTile<R, C> allocate_score_tile() {
    ScoreTile<R, C> t;
    t.home = MatrixF32{nullptr, 0, 0, 0};
    t.row0 = t.col0 = 0;
    t.stored = false;
    return t;
}

template<int64_t R, int64_t C>
__device__ __forceinline__ ScoreTile<R, C> MatrixF32::view_score_tile(int64_t x, int64_t y) const {
    ScoreTile<R, C> t;
    t.home = *this;
    t.row0 = (int)x;
    t.col0 = (int)y;
    t.stored = false;
    return t;
}

namespace detail {

// Row 16 tm + i of each lane's rows (32 w + 4 (lane / 16) + that), every value
// times f, 16 bytes per lane and store.
template<int64_t R, int64_t C>
__device__ __forceinline__ void store_score_row(const MatrixF32 &m, int64_t x, int64_t y, const ScoreTile<R, C> &t, int tm, int i, float f) {
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
    const int jl = lane % 16;
    const int64_t rr = x + 32 * w + 16 * tm + 4 * (lane / 16) + i;
    if (rr >= m.row) {
        return;
    }
    float *p = m.data + rr * m.lda;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const int64_t cc = y + 64 * g + 4 * jl;
        const float4 val = make_float4(t.acc[tm][4 * g + 0][i] * f, t.acc[tm][4 * g + 1][i] * f, t.acc[tm][4 * g + 2][i] * f,
                                       t.acc[tm][4 * g + 3][i] * f);
        if (cc + 3 < m.col && ((((uint64_t)(p + cc)) & 15u) == 0)) {
            store_result16<kThroughStores>(m.data, (m.row - 1) * m.lda + m.col, rr * m.lda + cc, val);
        } else {
            if (cc + 0 < m.col) p[cc + 0] = val.x;
            if (cc + 1 < m.col) p[cc + 1] = val.y;
            if (cc + 2 < m.col) p[cc + 2] = val.z;
            if (cc + 3 < m.col) p[cc + 3] = val.w;
        }
    }
}

}  // namespace detail

template<int64_t R, int64_t C>
__device__ __forceinline__ void MatrixF32::store_score_tile(int64_t x, int64_t y, const ScoreTile<R, C> &t) const {
    if (t.stored) {  // its rows went out through the view
        return;
    }
#pragma unroll
    for (int tm = 0; tm < 2; tm++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            detail::store_score_row(*this, x, y, t, tm, i, 1.0f);
        }
    }
}

// The raw products Q K^T of the tile; S.unit = scale * log2(e).
//
// Both operands are loaded straight into LDS (16 bytes per lane, no register
// round trip) in stages of 64 along the head dimension, two stages in flight
// from the start: a stage is 256 rows of Q and 256 keys of K, 128 bytes each,
// with the 16-byte piece c of LDS row r at position c ^ ((r >> 1) & 7), which
// spreads the sixteen rows of one fragment read over all banks.  LDS row
// 64 g + 16 t + j of the K stage holds key 64 g + 4 j + t: the sixteen keys of
// MFMA tile 4 g + t are then sixteen consecutive LDS rows, like the rows of Q.
// Rows of Q and keys past the end of the matrices are read from the last
// valid one (rows past the end are never stored, keys past the end are left
// out of the statistics by softmax_rows_across_tiles).
template<int64_t R, int64_t C, int64_t D>
__device__ __forceinline__ void qk_scaled(const GlobalView<R, D, uint16_t, false> &Q, const GlobalView<C, D, uint16_t, false> &K,
                                          ScoreTile<R, C> &S, float scale) {
    static_assert(D % 64 == 0 && D >= 64, "score tiles stage the head dimension in steps of 64");
    constexpr int NK = (int)(D / 64);
    constexpr int HALF = 256 * 128;  // bytes of one operand's stage
    __shared__ __attribute__((aligned(16))) unsigned char qk_stage_even[2 * HALF];
    __shared__ __attribute__((aligned(16))) unsigned char qk_stage_odd[2 * HALF];
    const int lane = lane_id();
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWaveSize));

    S.unit = scale * 1.4426950408889634f;
    S.valid_cols = (int)K.rows;
#pragma unroll
    for (int tm = 0; tm < 2; tm++) {
#pragma unroll
        for (int tn = 0; tn < 16; tn++) {
            S.acc[tm][tn] = score_f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
    }
    if (threadIdx.x == 0) {
        detail::row_stats_waves_done = 0u;  // seen by all after the first barrier below
    }
    if (Q.rows <= 0 || K.rows <= 0) {  // workgroup-uniform
        __syncthreads();
        return;
    }
    // Wavefront w issues Q instructions 4w .. 4w+3 and K instructions 4w .. 4w+3
    // (eight LDS rows each) of every stage: descriptor and stage offset in
    // scalar registers, one lane offset per instruction.
    constexpr int kRawBuffer = 0x00020000;
    const int64_t q_bytes = ((int64_t)(Q.rows - 1) * Q.lda + D) * 2, k_bytes = ((int64_t)(K.rows - 1) * K.lda + D) * 2;
    const __amdgpu_buffer_rsrc_t desc_q =
        __builtin_amdgcn_make_buffer_rsrc((void *)Q.data, 0, (int)(q_bytes < 0xFFFFFFFFll ? q_bytes : 0xFFFFFFFFll), kRawBuffer);
    const __amdgpu_buffer_rsrc_t desc_k =
        __builtin_amdgcn_make_buffer_rsrc((void *)K.data, 0, (int)(k_bytes < 0xFFFFFFFFll ? k_bytes : 0xFFFFFFFFll), kRawBuffer);
    int off_q[4], off_k[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = 8 * (w * 4 + j) + lane / 8;  // LDS row
        const int piece = (lane % 8) ^ ((r >> 1) & 7);
        const int q_row = r < (int)Q.rows - 1 ? r : (int)Q.rows - 1;
        off_q[j] = (q_row * (int)Q.lda + piece * 8) * 2;
        int key = 64 * (r / 64) + 4 * (r % 16) + (r / 16) % 4;
        key = key < (int)K.rows - 1 ? key : (int)K.rows - 1;
        off_k[j] = (key * (int)K.lda + piece * 8) * 2;
    }
    auto issue = [&](int kt, unsigned char *dst) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_q, (__attribute__((address_space(3))) void *)(dst + (w * 4 + j) * 1024), 16,
                                                     off_q[j], kt * 128, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc_k, (__attribute__((address_space(3))) void *)(dst + HALF + (w * 4 + j) * 1024),
                                                     16, off_k[j], kt * 128, 0, 0);
        }
    };
    // Fragments: lane l holds row / key l % 16 of an MFMA tile and the eight
    // values 8 (l / 16) .. + 7 of a 32-deep step.  Every LDS address is one
    // offset from its stage array (the compiler then orders reads of one stage
    // against the loads into that stage only).
    const int swz = ((lane % 16) >> 1) & 7;
    const int a_off = (32 * w + (lane % 16)) * 128;
    const int b_off = HALF + (lane % 16) * 128;
    auto compute = [&](const unsigned char *stage) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const int pos = ((4 * s + lane / 16) ^ swz) * 16;
            const bf16x8_t a0 = *reinterpret_cast<const bf16x8_t *>(stage + (a_off + pos));
            const bf16x8_t a1 = *reinterpret_cast<const bf16x8_t *>(stage + (a_off + 16 * 128 + pos));
#pragma unroll
            for (int tn = 0; tn < 16; tn++) {
                const bf16x8_t b = *reinterpret_cast<const bf16x8_t *>(stage + (b_off + tn * 16 * 128 + pos));
                S.acc[0][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b, S.acc[0][tn], 0, 0, 0);
                S.acc[1][tn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b, S.acc[1][tn], 0, 0, 0);
            }
        }
    };
    issue(0, qk_stage_even);
    if (NK > 1) {
        issue(1, qk_stage_odd);
    }
#pragma unroll
    for (int kt = 0; kt < NK; kt++) {
        // this wavefront's loads of stage kt have landed (those of stage kt + 1,
        // eight instructions, may still be in flight), then everybody's
        if (kt + 1 < NK) {
            __builtin_amdgcn_s_waitcnt(0x0078);  // vmcnt(8) lgkmcnt(0)
        } else {
            __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
        }
        __builtin_amdgcn_s_barrier();
        compute((kt & 1) ? qk_stage_odd : qk_stage_even);
        if (kt + 2 < NK) {
            // every wavefront is done reading the stage before it is refilled
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
            __builtin_amdgcn_s_barrier();
            issue(kt + 2, (kt & 1) ? qk_stage_odd : qk_stage_even);
        }
    }
}

namespace detail {

// The last workgroup of a launch advances the launch number and clears the
// count; when the number wraps around it first clears every entry (tag 0: never
// written).  Every wavefront calls this once it no longer reads entries;
// `waves_done` is a zeroed counter in LDS.  Only the last wavefront of a
// workgroup goes on to the device-wide count (and waits for its answer), so the
// others start storing their rows at once.
__device__ __forceinline__ void close_row_stats(const RowStatsSession &ex, unsigned int *waves_done) {
    const int lane = lane_id();
    unsigned int seen = 0;
    if (lane == 0) {
        seen = __hip_atomic_fetch_add(waves_done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    seen = (unsigned int)__builtin_amdgcn_readfirstlane((int)seen);
    if (seen + 1u != blockDim.x / kWaveSize) {  // wave-uniform
        return;
    }
    const unsigned int total = gridDim.x * gridDim.y * gridDim.z;
    const unsigned int next = ex.tag;  // launch number + 1
    unsigned int before = 0;
    if (lane == 0) {
        before = __hip_atomic_fetch_add(ex.state + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    before = (unsigned int)__builtin_amdgcn_readfirstlane((int)before);
    if (before + 1u != total) {
        return;
    }
    if (next == kRowStatsTagPeriod) {  // once in kRowStatsTagPeriod launches: every other wavefront of the launch is done with the entries
        for (long long i = lane; i < ex.capacity; i += kWaveSize) {
            __hip_atomic_store(ex.entries + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
    }
    if (lane == 0) {
        __hip_atomic_store(ex.state + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(ex.state, next == kRowStatsTagPeriod ? 0u : next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace detail

// out = softmax over the WHOLE rows of S that the tile `in` of scaled products
// (value = acc * in.unit, in log2 units) is a 256-column piece of; `out` is a
// view of S and its rows are stored through it.  Per 16-row half of a
// wavefront's rows, in this order:
//
//   half 0: m = floor(max), e = 2^(x - m), s = sum e; publish (m, s) per row
//   half 1: the same
//   half 0: wait for the sixteen column blocks' (m, s) of its rows, combine to
//           (M, S), store e * 2^(m - M) / S
//   half 1: the same
//
// so the entries of half 0 travel while half 1 is computed, and half 0 is
// stored while half 1 waits.  An entry is published by lanes j < 4 of each
// 16-lane row (row slot i = j of the half).
template<int64_t R, int64_t C>
__device__ __forceinline__ void softmax_rows_across_tiles(const ScoreTile<R, C> &in, const RowStatsSession &ex, ScoreTile<R, C> &out) {
    typedef unsigned long long u64;
    // Rows per lane and pipeline step (slot r = 4 tm + i is row 16 tm + i of the lane's eight rows).  Measured
    // at 4096 x 4096 x 128 in one process: 8 (one exchange for all rows) 24.3 us, 4 (the two halves) 21.7 us,
    // 1 (row by row) 23.6 us.
    constexpr int G = 4;
    static_assert(G == 1 || G == 2 || G == 4 || G == 8, "group size");
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
    const int jl = lane % 16;
    const float unit = in.unit;
    const bool partial = in.valid_cols < (int)C;  // workgroup-uniform: the last column block only
    const bool flip = unit < 0.f;                 // a negative scale turns the largest product into the smallest logit
    const int bj = out.col0 / (int)C, nbj = (int)gridDim.x;  // one workgroup per column block along x
    const int64_t row0 = (int64_t)out.row0 + 32 * w + 4 * (lane / 16);
    const u64 tag = ex.tag;
    out.unit = 1.0f;
    out.valid_cols = in.valid_cols;
    unsigned int unfit = 0;  // rows of this lane whose shift does not fit an entry (the same in all sixteen lanes of a row)
#pragma unroll
    for (int grp = 0; grp < 8 / G; grp++) {
#pragma unroll
        for (int r = grp * G; r < grp * G + G; r++) {
            const int tm = r / 4, i = r % 4;
            float x[16];
#pragma unroll
            for (int tn = 0; tn < 16; tn++) {
                x[tn] = in.acc[tm][tn][i];
            }
            if (flip) {
#pragma unroll
                for (int tn = 0; tn < 16; tn++) {
                    x[tn] = -x[tn];
                }
            }
            if (partial) {
#pragma unroll
                for (int tn = 0; tn < 16; tn++) {
                    const int key = 64 * (tn / 4) + 4 * jl + (tn % 4);
                    x[tn] = key < in.valid_cols ? x[tn] : -__builtin_huge_valf();
                }
            }
            float m = x[0];
#pragma unroll
            for (int tn = 1; tn < 16; tn++) {
                m = __builtin_fmaxf(m, x[tn]);
            }
            m = __builtin_fmaxf(m, dpp_move<0xB1>(m));
            m = __builtin_fmaxf(m, dpp_move<0x4E>(m));
            m = __builtin_fmaxf(m, dpp_move<0x141>(m));
            m = __builtin_fmaxf(m, dpp_move<0x140>(m));
            const float a = flip ? -unit : unit;
            // The floor of the row's largest logit in log2 units (a >= 0), within what an entry of
            // the exchange holds: the largest e is then in [1, 2) and no e that matters underflows.
            const float whole = __builtin_floorf(m * a);
            const float shift = __builtin_fminf(__builtin_fmaxf(whole, -32768.0f), 32767.0f);
            float s = 0.f;
#pragma unroll
            for (int tn = 0; tn < 16; tn++) {
                // a masked column is -inf: 2^-inf = 0 unless a == 0 (0 * inf), which the test below catches
                float e = __builtin_amdgcn_exp2f(__builtin_fmaf(x[tn], a, -shift));
                if (partial) {
                    const int key = 64 * (tn / 4) + 4 * jl + (tn % 4);
                    e = key < in.valid_cols ? e : 0.f;
                }
                out.acc[tm][tn][i] = e;
                s += e;
            }
            s += dpp_move<0xB1>(s);
            s += dpp_move<0x4E>(s);
            s += dpp_move<0x141>(s);
            s += dpp_move<0x140>(s);
            out.shift[tm][i] = shift;
            out.sum[tm][i] = s;
            // the largest logit beyond an entry's range or not a number, or a logit that is not a number
            unfit += (whole != shift || s != s) ? 1u : 0u;
        }
        {
            // lane j < G of each 16-lane row publishes slot grp * G + j
            float m = out.shift[(grp * G) / 4][(grp * G) % 4], s = out.sum[(grp * G) / 4][(grp * G) % 4];
#pragma unroll
            for (int q = 1; q < G; q++) {
                m = jl == q ? out.shift[(grp * G + q) / 4][(grp * G + q) % 4] : m;
                s = jl == q ? out.sum[(grp * G + q) / 4][(grp * G + q) % 4] : s;
            }
            if (jl < G) {
                const int r = grp * G + jl;
                u64 *e = ex.entries + ((row0 + 16 * (r / 4) + (r % 4)) * ex.pitch + bj);
                const u64 word = ((u64)(unsigned int)as_int(s) << 32) | ((u64)((unsigned int)(int)m & 0xFFFFu) << 16) | tag;
                __hip_atomic_store(e, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if (unfit != 0u && jl == 0) {  // never, for logits that fit: one lane per 16-lane row reports its rows
        __hip_atomic_fetch_add(ex.state + 3, unfit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    bool gave_up = false;
#pragma unroll
    for (int grp = 0; grp < 8 / G; grp++) {
        // Lane j collects column block j (j + 16, ...) for the G rows it holds of this group.
        float big_m[G], big_s[G];
#pragma unroll
        for (int q = 0; q < G; q++) {
            big_m[q] = -__builtin_huge_valf();
            big_s[q] = 0.f;
        }
        bool failed = false;
        for (int b0 = 0; b0 < nbj; b0 += 16) {  // one pass for up to 4096 keys
            const int b = b0 + jl;
            u64 got[G];
            int spins = 0;
            for (;;) {
                bool mine = true;
                if (b < nbj) {
#pragma unroll
                    for (int q = 0; q < G; q++) {
                        const int r = grp * G + q;
                        const u64 *e = ex.entries + ((row0 + 16 * (r / 4) + (r % 4)) * ex.pitch + b);
                        got[q] = __hip_atomic_load(e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int q = 0; q < G; q++) {
                        mine = mine && (got[q] & 0xFFFFull) == tag;
                    }
                }
                if (__builtin_amdgcn_ballot_w64(!mine) == 0) {
                    break;
                }
                if (++spins > ex.spin_limit) {  // wave-uniform
                    failed = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(2);  // 0 to 32 measure the same
            }
            if (b < nbj) {
#pragma unroll
                for (int q = 0; q < G; q++) {
                    const float m = (float)(short)(unsigned short)((got[q] >> 16) & 0xFFFFull), s = as_float((int)(unsigned int)(got[q] >> 32));
                    const float top = __builtin_fmaxf(big_m[q], m);
                    big_s[q] = big_s[q] * __builtin_amdgcn_exp2f(big_m[q] - top) + s * __builtin_amdgcn_exp2f(m - top);
                    big_m[q] = top;
                }
            }
        }
        gave_up = gave_up || failed;
        if (grp == 8 / G - 1) {
            if (gave_up && lane == 0) {  // wave-uniform condition
                __hip_atomic_fetch_add(ex.state + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            detail::close_row_stats(ex, &detail::row_stats_waves_done);  // this wavefront reads no entry from here on
        }
#pragma unroll
        for (int q = 0; q < G; q++) {
            const int r = grp * G + q, tm = r / 4, i = r % 4;
            const float m = big_m[q];
            float top = m;
            top = __builtin_fmaxf(top, dpp_move<0xB1>(top));
            top = __builtin_fmaxf(top, dpp_move<0x4E>(top));
            top = __builtin_fmaxf(top, dpp_move<0x141>(top));
            top = __builtin_fmaxf(top, dpp_move<0x140>(top));
            // a lane with no column block holds (-inf, 0) and adds 0 * 2^-inf = 0
            float s = big_s[q] * __builtin_amdgcn_exp2f(m - top);
            s += dpp_move<0xB1>(s);
            s += dpp_move<0x4E>(s);
            s += dpp_move<0x141>(s);
            s += dpp_move<0x140>(s);
            float f = __builtin_amdgcn_exp2f(out.shift[tm][i] - top) * (1.0f / s);
            f = failed ? __builtin_nanf("") : f;
            detail::store_score_row(out.home, out.row0, out.col0, out, tm, i, f);
        }
    }
    out.stored = true;
}

}  // namespace gernels
