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
// (gernels/cccl/wrappers/reduce_wrappers.cuh:42-61).
//
// Eight wavefronts; wavefront w owns rows [32 w, 32 w + 32) of the tile and all
// 256 columns, as eight v_mfma_f32_32x32x16_bf16 tiles that are computed
// TRANSPOSED: the keys are the rows of the matrix instruction and the queries
// its columns, so lane l holds, of query row 32 w + l % 32, the 128 scores of
// keys 32 t + 8 a + 4 (l / 32) + b (tile t < 8, a < 4, b < 4).  A row of S is
// thus spread over just two lanes (l and l + 32): its maximum and its sum are
// 128 operations inside a lane and ONE exchange between the two, no DPP
// butterflies, and the four scores b = 0 .. 3 are consecutive columns of S, one
// 16-byte store.  (With the 16 x 16 x 32 instruction, whose accumulators put a
// row on sixteen lanes with four columns each, the butterflies over sixteen
// lanes were a third of the vector-ALU work of the softmax.  The two
// instructions do the same work per cycle; the products of this kernel wait
// for their operands, not for the matrix pipe, with either.)
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
// Each wavefront polls the sixteen entries of its own 32 rows on its own (lane
// l the column blocks 8 (l / 32) .. + 7 of row l % 32).  Workgroup ids run
// along the columns, so the workgroups of a row block are dispatched together;
// a workgroup waits only for workgroups of its own row block, and those never
// wait for a later one.  The wait is bounded all the same: after spin_limit
// polls a wavefront gives up and stores NaN in its rows.  Logits beyond
// +-32767 in log2 units (22 000 in natural units) do not fit an entry; their
// rows come out as NaN.  Neither goes unnoticed by the host: state[2] counts
// the wavefronts that gave up and state[3] the (row, column block) pairs whose
// shift did not fit or whose logits were not all numbers, for the host to read
// and clear after the launch (the reference checks for an error after every
// launch, include/gern/codegen/helpers/check_last_error.h:7-18).
//
// Two launches that use the same exchange must not overlap in time.
#pragma once

#include "gernels/mm.h"
#include "gernels/softmax.h"

namespace gernels {

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
// that the exchange needs no barrier of its own: a wavefront exchanges only with
// its namesakes in the other tiles of the row block, and the wavefronts of a
// workgroup reach the exchange a microsecond or two apart (a SIMD serves its
// older wavefront first), so the early ones are storing their rows while the
// late ones still compute.
__shared__ unsigned int row_stats_waves_done;

// The two LDS stages of qk_scaled (64 KiB each: 256 rows of Q, then 256 keys of K, 128 bytes per row).
// Once every wavefront of the workgroup has read its last fragment (qk_waves_done_reading counts them),
// softmax_rows_across_tiles turns its rows around through the first one on their way to memory.
constexpr int kQkStageHalf = 256 * 128;  // bytes of one operand's stage
__shared__ __attribute__((aligned(16))) unsigned char qk_stage_even[2 * kQkStageHalf];
__shared__ __attribute__((aligned(16))) unsigned char qk_stage_odd[2 * kQkStageHalf];
__shared__ unsigned int qk_waves_done_reading;

// Where the entry of (row, column block) lies: the 256 rows of a row block side by side per column block, so
// that the 32 lanes that publish or read one column block for 32 consecutive rows touch 256 consecutive
// bytes (with the rows of a column block apart, every 8-byte entry was a memory access of its own, and a
// round of polls over all tiles took microseconds).  `pitch` entries per row, at least the number of column blocks.
__device__ __forceinline__ long long row_stats_entry(long long row, int block, int pitch) {
    return ((row >> 8) * pitch + block) * 256 + (row & 255);
}

// The value that lane l ^ 32 holds (the other half of a row of scores).
__device__ __forceinline__ float other_half(float x) {
    return as_float(__builtin_amdgcn_ds_bpermute((lane_id() ^ 32) * 4, as_int(x)));
}
}  // namespace detail

// A 256 x 256 tile of scores spread over eight wavefronts: acc[t][4 a + b] of lane l
// is row 32 w + l % 32, column 32 t + 8 a + 4 (l / 32) + b, in units of `unit`
// (value = acc * unit) as qk_scaled leaves it, plain afterwards.
// shift / sum: the statistics of the lane's row over the tile's columns.
template<int64_t R, int64_t C>
struct ScoreTile {
    static_assert(R == 256 && C == 256, "score tiles are 256 x 256");
    static constexpr int64_t rows = R;
    static constexpr int64_t cols = C;
    f32x16_t acc[8];
    float shift;
    float sum;
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

// The wavefront's 32 rows of the tile at (x, y) of m, every value times f.  A lane holds ONE row
// (32 bytes of it per group of four accumulators, side by side with lane l ^ 32), so stored from the
// registers as they are an instruction would write 32 bytes of each of 32 rows: measured, such stores take
// three times as long as whole lines (36.5 against about 11 us for the 64 MiB of a 4096 x 4096 result).
// Each 32 x 32 tile is therefore turned around through LDS: written as the lanes hold it (row l % 32,
// 16-byte piece 2 a + l / 32 at position piece ^ ((row >> 1) & 7), which keeps both directions free of
// bank conflicts), read back with eight lanes per row, and stored: an instruction then writes eight whole
// 128-byte lines.  `lds` is 8 KiB that belong to this wavefront (two tiles: the next one is written while
// the last one is read).
template<int POLICY, int64_t R, int64_t C>
__device__ __forceinline__ void store_score_rows(const MatrixF32 &m, int64_t x, int64_t y, const ScoreTile<R, C> &t, float f,
                                                 unsigned char *lds) {
    typedef float f32x4_native __attribute__((ext_vector_type(4)));
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
    const int n = lane % 32, h = lane / 32;
    const int put = n * 128, put_swz = (n >> 1) & 7;
    const int64_t span = (m.row - 1) * m.lda + m.col;
#pragma unroll
    for (int tn = 0; tn < 8; tn++) {
        unsigned char *tile = lds + (tn & 1) * 4096;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const f32x4_native val = {t.acc[tn][4 * a + 0] * f, t.acc[tn][4 * a + 1] * f, t.acc[tn][4 * a + 2] * f, t.acc[tn][4 * a + 3] * f};
            *reinterpret_cast<f32x4_native *>(tile + put + (((2 * a + h) ^ put_swz) * 16)) = val;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int r = 8 * j + lane / 8, piece = lane % 8;
            const f32x4_native q = *reinterpret_cast<const f32x4_native *>(tile + r * 128 + ((piece ^ ((r >> 1) & 7)) * 16));
            const int64_t rr = x + 32 * w + r, cc = y + 32 * tn + 4 * piece;
            if (rr >= m.row) {
                continue;
            }
            float *p = m.data + rr * m.lda;
            const float4 val = make_float4(q[0], q[1], q[2], q[3]);
            if (cc + 3 < m.col && ((((uint64_t)(p + cc)) & 15u) == 0)) {
                store_result16<POLICY>(m.data, span, rr * m.lda + cc, val);
            } else {
                if (cc + 0 < m.col) p[cc + 0] = val.x;
                if (cc + 1 < m.col) p[cc + 1] = val.y;
                if (cc + 2 < m.col) p[cc + 2] = val.z;
                if (cc + 3 < m.col) p[cc + 3] = val.w;
            }
        }
    }
}

// The 8 KiB of the first stage that wavefront w may use once no wavefront reads the stages any more; waits
// for that (normally it has long been so: the products end microseconds before the first row is final).
__device__ __forceinline__ unsigned char *own_lds_after_products() {
    const unsigned int waves = blockDim.x / kWaveSize;
    while (__hip_atomic_load(&qk_waves_done_reading, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < waves) {
        __builtin_amdgcn_s_sleep(1);
    }
    return qk_stage_even + (threadIdx.x / kWaveSize) * 8192;
}

}  // namespace detail

template<int64_t R, int64_t C>
__device__ __forceinline__ void MatrixF32::store_score_tile(int64_t x, int64_t y, const ScoreTile<R, C> &t) const {
    if (t.stored) {  // its rows went out through the view
        return;
    }
    detail::store_score_rows<kThroughStores>(*this, x, y, t, 1.0f, detail::own_lds_after_products());
}

// The raw products Q K^T of the tile; S.unit = scale * log2(e).
//
// Both operands are loaded straight into LDS (16 bytes per lane, no register
// round trip) in stages of 64 along the head dimension, two stages in flight
// from the start: a stage is 256 rows of Q and 256 keys of K, 128 bytes each,
// with the 16-byte piece c of LDS row r at position c ^ ((r >> 1) & 7), which
// spreads the sixteen rows of one pass of a fragment read over all banks.
// The loads (128 KiB per workgroup, 32 MiB out of L2 over all of them at
// 4096 x 4096 x 128) are what this gernel waits for: its products end about
// 4 us after the launch with either matrix instruction.  Stages of 32 (whose
// products could start earlier) fetch half a cache line per row and
// instruction and end a microsecond LATER.
// Rows of Q and keys past the end of the matrices are read from the last
// valid one (rows past the end are never stored, keys past the end are left
// out of the statistics by softmax_rows_across_tiles).
template<int64_t R, int64_t C, int64_t D>
__device__ __forceinline__ void qk_scaled(const GlobalView<R, D, uint16_t, false> &Q, const GlobalView<C, D, uint16_t, false> &K,
                                          ScoreTile<R, C> &S, float scale) {
    static_assert(D % 64 == 0 && D >= 64, "score tiles stage the head dimension in steps of 64");
    constexpr int NK = (int)(D / 64);
    constexpr int HALF = detail::kQkStageHalf;
    unsigned char *const qk_stage_even = detail::qk_stage_even;
    unsigned char *const qk_stage_odd = detail::qk_stage_odd;
    const int lane = lane_id();
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWaveSize));

    S.unit = scale * 1.4426950408889634f;
    S.valid_cols = (int)K.rows;
#pragma unroll
    for (int tn = 0; tn < 8; tn++) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            S.acc[tn][i] = 0.f;
        }
    }
    if (threadIdx.x == 0) {
        detail::row_stats_waves_done = 0u;  // seen by all after the first barrier below
        detail::qk_waves_done_reading = 0u;
    }
    if (Q.rows <= 0 || K.rows <= 0) {  // workgroup-uniform
        __syncthreads();
        if (lane == 0) {
            __hip_atomic_fetch_add(&detail::qk_waves_done_reading, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
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
        const int r = 8 * (w * 4 + j) + lane / 8;  // LDS row = row of Q, key of K
        const int piece = (lane % 8) ^ ((r >> 1) & 7);
        const int q_row = r < (int)Q.rows - 1 ? r : (int)Q.rows - 1;
        off_q[j] = (q_row * (int)Q.lda + piece * 8) * 2;
        const int key = r < (int)K.rows - 1 ? r : (int)K.rows - 1;
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
    // Fragments of a 16-deep step: lane l holds row l % 32 (a key of a K tile,
    // a query of this wavefront's rows of Q) and the eight values
    // 8 (l / 32) .. + 7 of the step.  Every LDS address is one offset from its
    // stage array (the compiler then orders reads of one stage against the
    // loads into that stage only).
    const int swz = ((lane % 32) >> 1) & 7;  // rows 32 t + l % 32: the other terms are multiples of 16
    const int q_off = (32 * w + (lane % 32)) * 128;
    const int k_off = HALF + (lane % 32) * 128;
    auto compute = [&](const unsigned char *stage) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const int pos = ((2 * s + lane / 32) ^ swz) * 16;
            const bf16x8_t q = *reinterpret_cast<const bf16x8_t *>(stage + (q_off + pos));
#pragma unroll
            for (int tn = 0; tn < 8; tn++) {
                const bf16x8_t k = *reinterpret_cast<const bf16x8_t *>(stage + (k_off + tn * 32 * 128 + pos));
                // keys are the rows of the product, queries its columns
                S.acc[tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k, q, S.acc[tn], 0, 0, 0);
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
    // this wavefront reads the stages no more
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    if (lane == 0) {
        __hip_atomic_fetch_add(&detail::qk_waves_done_reading, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
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
// view of S and its rows are stored through it.  Per wavefront (32 rows, one
// per pair of lanes):
//
//   m = floor(max), e = 2^(x - m), s = sum e; publish (m, s) per row
//   wait for the sixteen column blocks' (m, s) of the rows, combine to (M, S)
//   store e * 2^(m - M) / S
//
// The two wavefronts of a SIMD do not run side by side: the SIMD serves the
// older one first, so one is at its exponentials while the other multiplies,
// and one waits for the exchange or stores while the other is at its
// exponentials.
template<int64_t R, int64_t C>
__device__ __forceinline__ void softmax_rows_across_tiles(const ScoreTile<R, C> &in, const RowStatsSession &ex, ScoreTile<R, C> &out) {
    typedef unsigned long long u64;
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
    const int half = lane / 32;
    const float unit = in.unit;
    const bool partial = in.valid_cols < (int)C;  // workgroup-uniform: the last column block only
    const bool flip = unit < 0.f;                 // a negative scale turns the largest product into the smallest logit
    const int bj = out.col0 / (int)C, nbj = (int)gridDim.x;  // one workgroup per column block along x
    const int64_t row = (int64_t)out.row0 + 32 * w + lane % 32;
    const u64 tag = ex.tag;
    out.unit = 1.0f;
    out.valid_cols = in.valid_cols;

    // ---- the tile's own statistics of the row ----
#pragma unroll
    for (int tn = 0; tn < 8; tn++) {
        out.acc[tn] = in.acc[tn];
    }
    if (flip) {  // uniform
#pragma unroll
        for (int tn = 0; tn < 8; tn++) {
            out.acc[tn] = -out.acc[tn];
        }
    }
    if (partial) {  // uniform
#pragma unroll
        for (int tn = 0; tn < 8; tn++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int key = 32 * tn + 8 * (i / 4) + 4 * half + (i % 4);
                out.acc[tn][i] = key < in.valid_cols ? out.acc[tn][i] : -__builtin_huge_valf();
            }
        }
    }
    float m4[4] = {-__builtin_huge_valf(), -__builtin_huge_valf(), -__builtin_huge_valf(), -__builtin_huge_valf()};
#pragma unroll
    for (int tn = 0; tn < 8; tn++) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            m4[i % 4] = __builtin_fmaxf(m4[i % 4], out.acc[tn][i]);
        }
    }
    float m = __builtin_fmaxf(__builtin_fmaxf(m4[0], m4[1]), __builtin_fmaxf(m4[2], m4[3]));
    m = __builtin_fmaxf(m, detail::other_half(m));
    const float a = flip ? -unit : unit;
    // The floor of the row's largest logit in log2 units (a >= 0), within what an entry of
    // the exchange holds: the largest e is then in [1, 2) and no e that matters underflows.
    const float whole = __builtin_floorf(m * a);
    const float shift = __builtin_fminf(__builtin_fmaxf(whole, -32768.0f), 32767.0f);
    // a masked column is -inf: 2^-inf = 0 unless a == 0 (0 * inf = NaN), which the masking after the loop catches
    float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tn = 0; tn < 8; tn++) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            out.acc[tn][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(out.acc[tn][i], a, -shift));
        }
    }
    if (partial) {  // uniform
#pragma unroll
        for (int tn = 0; tn < 8; tn++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int key = 32 * tn + 8 * (i / 4) + 4 * half + (i % 4);
                out.acc[tn][i] = key < in.valid_cols ? out.acc[tn][i] : 0.f;
            }
        }
    }
#pragma unroll
    for (int tn = 0; tn < 8; tn++) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            s4[i % 4] += out.acc[tn][i];
        }
    }
    float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    s += detail::other_half(s);
    // The largest logit beyond an entry's range or not a number, or a logit that is not a number: the sum
    // travels as NaN, which makes the whole row NaN in every tile.
    const bool bad = whole != shift || s != s;
    s = bad ? __builtin_nanf("") : s;
    out.shift = shift;
    out.sum = s;
    if (half == 0) {
        u64 *e = ex.entries + detail::row_stats_entry(row, bj, ex.pitch);
        const u64 word = ((u64)(unsigned int)as_int(s) << 32) | ((u64)((unsigned int)(int)shift & 0xFFFFu) << 16) | tag;
        __hip_atomic_store(e, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (bad && row < out.home.row) {  // never, for logits that fit (rows past the end repeat the last one)
            __hip_atomic_fetch_add(ex.state + 3, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    // ---- the statistics of the whole row: lane l collects column blocks 8 (l / 32) .. + 7 (+ 16, ...) ----
    float big_m = -__builtin_huge_valf(), big_s = 0.f;
    bool failed = false;
    for (int b0 = 0; b0 < nbj; b0 += 16) {  // one pass for up to 4096 keys
        u64 got[8];
        int spins = 0;
        for (;;) {
            bool mine = true;
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const int b = b0 + 8 * half + q;
                if (b < nbj) {
                    got[q] = __hip_atomic_load(ex.entries + detail::row_stats_entry(row, b, ex.pitch), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
#pragma unroll
            for (int q = 0; q < 8; q++) {
                mine = mine && (b0 + 8 * half + q >= nbj || (got[q] & 0xFFFFull) == tag);
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
#pragma unroll
        for (int q = 0; q < 8; q++) {
            if (b0 + 8 * half + q < nbj) {
                const float em = (float)(short)(unsigned short)((got[q] >> 16) & 0xFFFFull), es = as_float((int)(unsigned int)(got[q] >> 32));
                const float top = __builtin_fmaxf(big_m, em);
                big_s = big_s * __builtin_amdgcn_exp2f(big_m - top) + es * __builtin_amdgcn_exp2f(em - top);
                big_m = top;
            }
        }
    }
    if (failed && lane == 0) {  // wave-uniform condition
        __hip_atomic_fetch_add(ex.state + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    detail::close_row_stats(ex, &detail::row_stats_waves_done);  // this wavefront reads no entry from here on
    {
        // a lane with no column block holds (-inf, 0) and adds 0 * 2^-inf = 0
        const float top = __builtin_fmaxf(big_m, detail::other_half(big_m));
        float sum = big_s * __builtin_amdgcn_exp2f(big_m - top);
        sum += detail::other_half(sum);
        float f = __builtin_amdgcn_exp2f(shift - top) * (1.0f / sum);
        f = failed ? __builtin_nanf("") : f;
        detail::store_score_rows<kThroughStores>(out.home, out.row0, out.col0, out, f, detail::own_lds_after_products());
    }
    out.stored = true;
}

}  // namespace gernels
