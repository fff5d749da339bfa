// Row-softmax building blocks on wave-distributed register tiles: row maximum,
// row sum, x - v[row], exp, x / v[row].
//
// They are the wavefront-level twins of the reference's softmax gernels
// (apps/common/impl/impl.h:7-24 exp_matrix, :26-51 divide_vec, :53-78
// subtract_vec, :80-133 sum_row, :135-188 max_shuffle).  The reference reduces
// a row with 32-lane shuffles plus a shared-memory hop between warps; here a
// whole row lives in one 64-lane wavefront, so the reduction is a lane-local
// scan followed by a DPP / ds_swizzle butterfly that never leaves the wave.
#pragma once

#include "gernels/wave_tile.h"

namespace gernels {

struct MaxOp {
    static __device__ __forceinline__ float identity() {
        return -__builtin_huge_valf();
    }
    static __device__ __forceinline__ float apply(float a, float b) {
        return __builtin_fmaxf(a, b);
    }
};

struct SumOp {
    static __device__ __forceinline__ float identity() {
        return 0.f;
    }
    static __device__ __forceinline__ float apply(float a, float b) {
        return a + b;
    }
};

template<int kCtrl>
__device__ __forceinline__ float dpp_move(float x) {
    return as_float(__builtin_amdgcn_update_dpp(as_int(x), as_int(x), kCtrl, 0xf, 0xf, false));
}

// All-lanes reduction over one wavefront.  Steps 1-4 stay inside a 16-lane DPP
// row (quad permutes, then half-mirror and mirror); step 5 swaps the two rows
// of each 32-lane half through ds_swizzle; step 6 combines the two halves by
// reading one lane of each into scalars, which also leaves the result uniform.
template<typename Op>
__device__ __forceinline__ float wave_all_reduce(float x) {
    x = Op::apply(x, dpp_move<0xB1>(x));   // quad_perm [1,0,3,2]
    x = Op::apply(x, dpp_move<0x4E>(x));   // quad_perm [2,3,0,1]
    x = Op::apply(x, dpp_move<0x141>(x));  // row_half_mirror
    x = Op::apply(x, dpp_move<0x140>(x));  // row_mirror
    // bit-mode swizzle: and_mask 0x1f, or_mask 0, xor_mask 0x10 -> lane ^ 16
    x = Op::apply(x, as_float(__builtin_amdgcn_ds_swizzle(as_int(x), 0x401F)));
    const float lo = as_float(__builtin_amdgcn_readlane(as_int(x), 0));
    const float hi = as_float(__builtin_amdgcn_readlane(as_int(x), 32));
    return Op::apply(lo, hi);
}

template<typename Op, typename TV, typename TI>
__device__ __forceinline__ void reduce_rows(TV &out, const TI &in) {
    static_assert(TV::size == TI::rows, "one scalar per tile row");
    const int lane = lane_id();
#pragma unroll
    for (int64_t r = 0; r < TI::rows; r++) {
        float acc = Op::identity();
#pragma unroll
        for (int64_t k = 0; k < TI::chunks; k++) {
            const float4 t = in.v[r][k];
            const int64_t lc = k * kWaveCols + 4 * lane;
            // columns past the tile's logical width do not take part
            if (lc + 0 < TI::cols) acc = Op::apply(acc, t.x);
            if (lc + 1 < TI::cols) acc = Op::apply(acc, t.y);
            if (lc + 2 < TI::cols) acc = Op::apply(acc, t.z);
            if (lc + 3 < TI::cols) acc = Op::apply(acc, t.w);
        }
        out.val[r] = wave_all_reduce<Op>(acc);
    }
}

// `stride` (the number of threads sharing a row in the reference's signature)
// is accepted for source compatibility and ignored: a row is always one wave.
template<int64_t stride = 64, typename TV, typename TI>
__device__ __forceinline__ void max_row(TV &out, const TI &in) {
    reduce_rows<MaxOp>(out, in);
}

template<int64_t stride = 64, typename TV, typename TI>
__device__ __forceinline__ void sum_row(TV &out, const TI &in) {
    reduce_rows<SumOp>(out, in);
}

template<typename TV, typename T>
__device__ __forceinline__ void subtract_vec(const TV &vec, const T &in, T &out) {
    static_assert(TV::size == T::rows, "one scalar per tile row");
#pragma unroll
    for (int64_t r = 0; r < T::rows; r++) {
        const float s = vec.val[r];
#pragma unroll
        for (int64_t k = 0; k < T::chunks; k++) {
            const float4 t = in.v[r][k];
            out.v[r][k] = make_float4(t.x - s, t.y - s, t.z - s, t.w - s);
        }
    }
}

// exp(x) as one multiply and one v_exp_f32 (2^y).  For x in [-87, 0] -- what a
// max-subtracted row holds -- the product x * log2(e) is off by at most half
// an ulp of 126, i.e. the result by 2.6e-6 relative, plus the instruction's own
// 1 ulp.  The raw instruction flushes results below 2^-126 to zero, and large
// positive arguments lose more, so a chunk in which ANY lane is outside
// [-87, 87] takes the library expf instead (a wave-uniform branch, never taken
// for the rows a softmax sees in practice).
__device__ __forceinline__ float4 exp4(const float4 &t) {
    const float lo = __builtin_fminf(__builtin_fminf(t.x, t.y), __builtin_fminf(t.z, t.w));
    const float hi = __builtin_fmaxf(__builtin_fmaxf(t.x, t.y), __builtin_fmaxf(t.z, t.w));
    // NaN compares false on both sides of the range test: written so that it
    // takes the library path too.
    if (__builtin_amdgcn_ballot_w64(!(lo >= -87.0f && hi <= 87.0f)) != 0) {
        return make_float4(expf(t.x), expf(t.y), expf(t.z), expf(t.w));
    }
    const float l2e = 1.4426950408889634f;
    return make_float4(__builtin_amdgcn_exp2f(t.x * l2e), __builtin_amdgcn_exp2f(t.y * l2e),
                       __builtin_amdgcn_exp2f(t.z * l2e), __builtin_amdgcn_exp2f(t.w * l2e));
}

template<typename T>
__device__ __forceinline__ void exp_matrix(const T &in, T &out) {
#pragma unroll
    for (int64_t r = 0; r < T::rows; r++) {
#pragma unroll
        for (int64_t k = 0; k < T::chunks; k++) {
            out.v[r][k] = exp4(in.v[r][k]);
        }
    }
}

template<typename TV, typename T>
__device__ __forceinline__ void divide_vec(const TV &vec, const T &in, T &out) {
    static_assert(TV::size == T::rows, "one scalar per tile row");
#pragma unroll
    for (int64_t r = 0; r < T::rows; r++) {
        // One IEEE division per row, then a multiply per element: within
        // 1 ulp of the true quotient (the softmax bar is 1e-5 relative).
        const float rcp = 1.0f / vec.val[r];
#pragma unroll
        for (int64_t k = 0; k < T::chunks; k++) {
            const float4 t = in.v[r][k];
            out.v[r][k] = make_float4(t.x * rcp, t.y * rcp, t.z * rcp, t.w * rcp);
        }
    }
}

// ---------------------------------------------------------------------------
// Rows spread over the wavefronts of a workgroup
// ---------------------------------------------------------------------------
// R full rows of C columns held by the NW wavefronts of a workgroup:
// wavefront w keeps columns [w * C / NW, (w + 1) * C / NW) as a WaveTile.  The
// reference's row reductions work the same way (apps/common/impl/impl.h:80-188:
// `stride` threads share a row, partial results meet in shared memory).  A
// wide row cut into several short wavefronts finishes in many small pieces
// that start and end at different times, so loads and stores of different
// rows overlap; one wavefront per 4096-column row keeps 64 values per lane,
// leaves room for three wavefronts per SIMD, and measures 20 % slower.
//
// A width that does not divide into NW whole 16-byte pieces is cut into pieces
// of wave_cols = ceil(C / NW) rounded up to whole 256-column chunks; the last
// wavefronts then use only part of their piece, or none of it.
template<int64_t R, int64_t C, int NW>
struct BlockTile {
    static_assert(NW >= 1 && C >= 1, "at least one wavefront and one column");
    static constexpr int64_t rows = R;
    static constexpr int64_t cols = C;
    static constexpr int waves = NW;
    static constexpr int64_t wave_cols = C % (4 * NW) == 0 ? C / NW : ((C + NW - 1) / NW + kWaveCols - 1) / kWaveCols * kWaveCols;
    static constexpr bool even = wave_cols * NW == C;
    WaveTile<R, wave_cols> part;

    // Wavefronts 0 .. full - 1 use their whole piece, wavefront `full` the first `rest` columns of its piece
    // (if any), the wavefronts after it nothing.
    static constexpr int full = (int)(C / wave_cols);
    static constexpr int64_t rest = C - full * wave_cols;
    static __device__ __forceinline__ int64_t used_by(int w) {
        return even || w < full ? wave_cols : (w == full ? rest : 0);
    }

    __device__ __forceinline__ void destroy() {
    }
};

#define GERN_BLOCK_ALLOCATOR(NW)                                              \
    template<int64_t R, int64_t C>                                            \
    __device__ __forceinline__ BlockTile<R, C, NW> allocate_block_tile##NW() { \
        return BlockTile<R, C, NW>();                                         \
    }
GERN_BLOCK_ALLOCATOR(2)
GERN_BLOCK_ALLOCATOR(4)
GERN_BLOCK_ALLOCATOR(8)
GERN_BLOCK_ALLOCATOR(16)
#undef GERN_BLOCK_ALLOCATOR

template<int NW, int64_t R, int64_t C>
__device__ __forceinline__ BlockTile<R, C, NW> MatrixF32::load_block(int64_t x, int64_t y) const {
    using T = BlockTile<R, C, NW>;
    T t;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWaveSize));
    t.part = load_wave<R, T::wave_cols>(x, y + w * T::wave_cols);
    if constexpr (!T::even) {
        // The columns of a piece that are not in use (whatever the matrix holds there) become -infinity: no
        // row maximum takes it, and its exponential adds nothing to a row sum, so that every later stage runs
        // the same code on every wavefront; only the store needs the width again.  One code path on purpose:
        // separate instances per wavefront for the reductions keep a second copy of the tile alive where the
        // paths meet (16 chunks per lane: 282 registers spilled).
        const int left0 = (int)T::used_by(w) - 4 * lane_id();
        const float none = -__builtin_huge_valf();
#pragma unroll
        for (int64_t r = 0; r < R; r++) {
#pragma unroll
            for (int64_t k = 0; k < WaveTile<R, T::wave_cols>::chunks; k++) {
                const int left = left0 - (int)(k * kWaveCols);
                float4 v = t.part.v[r][k];
                v.x = 0 < left ? v.x : none;
                v.y = 1 < left ? v.y : none;
                v.z = 2 < left ? v.z : none;
                v.w = 3 < left ? v.w : none;
                t.part.v[r][k] = v;
            }
        }
    }
    return t;
}

template<int NW, int64_t R, int64_t C>
__device__ __forceinline__ BlockTile<R, C, NW> MatrixF32::view_block(int64_t, int64_t) const {
    return BlockTile<R, C, NW>();
}

template<int64_t R, int64_t C, int NW>
__device__ __forceinline__ void MatrixF32::store_block(int64_t x, int64_t y, const BlockTile<R, C, NW> &t) const {
    using T = BlockTile<R, C, NW>;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWaveSize));
    if constexpr (T::even) {
        store_wave(x, y + w * T::wave_cols, t.part);
    } else {
        // The tile ends at column y + C: stored through a copy of the matrix that ends there too, so that the
        // one bounds test every store has anyway does the clipping (a width passed to store_wave as a run-time
        // value costs the kernel 85 registers).
        MatrixF32 clipped = *this;
        clipped.col = y + C < col ? y + C : col;
        clipped.store_wave(x, y + w * T::wave_cols, t.part);
    }
}

namespace detail {

// Row reduction of a block tile: each wavefront reduces its columns, lane 0
// leaves the R partial results in `scratch` (R x NW floats of LDS), and after
// one barrier every lane combines the NW partials of each row in wavefront
// order.  The two reductions of a softmax use different scratch arrays, so a
// wavefront may start the second while another still reads the first.
template<typename Op, typename TV, int64_t R, int64_t C, int NW>
__device__ __forceinline__ void reduce_block_rows(TV &out, const BlockTile<R, C, NW> &in, float *scratch) {
    // (columns of a piece that are not in use hold -infinity, then 0 after the exponential: see load_block)
    reduce_rows<Op>(out, in.part);
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWaveSize));
    if (lane_id() == 0) {
#pragma unroll
        for (int64_t r = 0; r < R; r++) {
            scratch[r * NW + w] = out.val[r];
        }
    }
    __syncthreads();
#pragma unroll
    for (int64_t r = 0; r < R; r++) {
        float acc = scratch[r * NW];
#pragma unroll
        for (int q = 1; q < NW; q++) {
            acc = Op::apply(acc, scratch[r * NW + q]);
        }
        out.val[r] = acc;
    }
}

}  // namespace detail

template<int64_t stride = 64, typename TV, int64_t R, int64_t C, int NW>
__device__ __forceinline__ void max_row(TV &out, const BlockTile<R, C, NW> &in) {
    __shared__ float block_max_scratch[R * NW];
    detail::reduce_block_rows<MaxOp>(out, in, block_max_scratch);
}

template<int64_t stride = 64, typename TV, int64_t R, int64_t C, int NW>
__device__ __forceinline__ void sum_row(TV &out, const BlockTile<R, C, NW> &in) {
    __shared__ float block_sum_scratch[R * NW];
    detail::reduce_block_rows<SumOp>(out, in, block_sum_scratch);
}

template<typename TV, int64_t R, int64_t C, int NW>
__device__ __forceinline__ void subtract_vec(const TV &vec, const BlockTile<R, C, NW> &in, BlockTile<R, C, NW> &out) {
    subtract_vec(vec, in.part, out.part);
}

template<int64_t R, int64_t C, int NW>
__device__ __forceinline__ void exp_matrix(const BlockTile<R, C, NW> &in, BlockTile<R, C, NW> &out) {
    exp_matrix(in.part, out.part);
}

template<typename TV, int64_t R, int64_t C, int NW>
__device__ __forceinline__ void divide_vec(const TV &vec, const BlockTile<R, C, NW> &in, BlockTile<R, C, NW> &out) {
    divide_vec(vec, in.part, out.part);
}

}  // namespace gernels
