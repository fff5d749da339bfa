// Wave-distributed register tiles and the global fp32 matrix they are cut from.
//
// A WaveTile<R, C> is an R x C fp32 tile owned by ONE 64-lane wavefront and
// held entirely in VGPRs: lane l keeps, for every row and every 256-column
// chunk k, the float4 covering columns 256*k + 4*l .. 256*k + 4*l + 3.  One
// row of a chunk is therefore one fully coalesced 1 KiB access (64 lanes x
// 16 B), which is how MatrixF32 loads and stores it.
//
// This is the gfx950 counterpart of the per-thread StaticMatrix register tile
// of the reference (apps/common/impl/gpu-matrix-const.h:29-38, query :131-150,
// insert :152-170, allocate_static :251-254): the same query / allocate /
// insert contract that generated code calls, re-laid-out so that the unit that
// owns a tile is a wavefront rather than a thread and neighbouring columns
// live in neighbouring lanes (one DPP move away) rather than in a halo that
// every thread re-reads from memory.
#pragma once

#include "gernels/prelude.h"

namespace gernels {

template<int64_t R, int64_t C>
struct WaveTile {
    static constexpr int64_t rows = R;
    static constexpr int64_t cols = C;
    static constexpr int64_t chunks = (C + kWaveCols - 1) / kWaveCols;
    float4 v[R][chunks];

    __device__ __forceinline__ void destroy() {
    }
};

// Per-row scalars (row maxima, row sums), replicated in every lane.
template<int64_t R>
struct WaveVec {
    static constexpr int64_t size = R;
    float val[R];

    __device__ __forceinline__ void destroy() {
    }
};

// 16-byte streaming store (the nontemporal builtin wants a native vector).
__device__ __forceinline__ void store_streaming(float *p, const float4 &v) {
    typedef float f32x4_native __attribute__((ext_vector_type(4)));
    const f32x4_native q = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(q, reinterpret_cast<f32x4_native *>(p));
}

// Stores of RESULTS, which the kernel does not read again: base[elem .. elem + 3]
// (base[elem]) of a matrix that spans `span` elements from base.  They go out as
// buffer stores that are written through to memory at once (agent scope): the
// lines are then clean when the kernel ends, where ordinary and nontemporal
// stores leave them for the write-back that closes every kernel.  POLICY is the
// cache policy of the buffer instruction (1 = sc0, 2 = nt, 16 = sc1):
//   kThroughStores           written through; for kernels that re-read nothing
//                            from L2 (64 MiB of results, us per launch: write-only
//                            kernel 11.1 -> 10.1, QK^T softmax tiles 22.4 -> 21.2,
//                            row blocks 27.4 -> 24.6; the GEMMs: no difference)
//   kThroughStreamingStores  written through and nontemporal; for kernels whose
//                            inputs must stay in L2 for a neighbouring tile (blur
//                            8192^2 over rotating buffers 91.2 -> 90.0 us, softmax
//                            45.0 -> 44.5 us; written through only: 91.4 and 45.4,
//                            and the blur on the same buffers 90 instead of 81 us)
// Buffer addressing takes 32-bit byte offsets, so a matrix of 4 GiB or more
// keeps nontemporal stores.
constexpr int kThroughStores = 16;
constexpr int kThroughStreamingStores = 18;

template<int POLICY>
__device__ __forceinline__ void store_result16(float *base, int64_t span, int64_t elem, const float4 &v) {
    typedef unsigned int u32x4_native __attribute__((ext_vector_type(4)));
    if ((uint64_t)span * 4u < 0xFFFFFFF0ull) {  // uniform
        const __amdgpu_buffer_rsrc_t desc = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(span * 4), 0x00020000);
        const u32x4_native bits = {__builtin_bit_cast(unsigned int, v.x), __builtin_bit_cast(unsigned int, v.y),
                                   __builtin_bit_cast(unsigned int, v.z), __builtin_bit_cast(unsigned int, v.w)};
        __builtin_amdgcn_raw_buffer_store_b128(bits, desc, (int)(elem * 4), 0, POLICY);
    } else {
        store_streaming(base + elem, v);
    }
}

template<int POLICY>
__device__ __forceinline__ void store_result4(float *base, int64_t span, int64_t elem, float v) {
    if ((uint64_t)span * 4u < 0xFFFFFFF0ull) {  // uniform
        const __amdgpu_buffer_rsrc_t desc = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, (int)(span * 4), 0x00020000);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), desc, (int)(elem * 4), 0, POLICY);
    } else {
        __builtin_nontemporal_store(v, base + elem);
    }
}

template<int64_t R, int64_t C>
__device__ __forceinline__ WaveTile<R, C> allocate_wave_tile() {
    return WaveTile<R, C>();
}

template<int64_t R>
__device__ __forceinline__ WaveVec<R> allocate_wave_vec() {
    return WaveVec<R>();
}

// Defined in gernels/mm.h: a window onto a matrix in HBM (no data movement) and
// the two block-distributed accumulator tiles of the GEMM gernels.
template<int64_t R, int64_t C, typename T, bool EXACT>
struct GlobalView;
template<int64_t BM, int64_t BN, int NW>
struct MfmaAcc;
template<int64_t BM, int64_t BN>
struct MfmaAcc16;
template<int64_t BM, int64_t BN>
struct FmaAcc;
template<int64_t BM, int64_t BN>
struct MfmaAccF32;
// Defined in gernels/qk_softmax.h: sixteen full rows of logits in registers.
template<int64_t R, int64_t N>
struct RowBlock;
// Defined in gernels/qk_tiles.h: a 256 x 256 tile of scores spread over a workgroup.
template<int64_t R, int64_t C>
struct ScoreTile;
// Defined in gernels/softmax.h: R full rows spread over the NW wavefronts of a
// workgroup.
template<int64_t R, int64_t C, int NW>
struct BlockTile;

// Row-major fp32 matrix in HBM.  Plain aggregate: the host fills one in and
// the launch passes it by value, so host and device layouts must agree
// (pointer, then three 64-bit integers).
struct MatrixF32 {
    float *data;
    int64_t row;
    int64_t col;
    int64_t lda;

    // GEMM operand / result access (gernels/mm.h).
    template<int64_t R, int64_t C>
    __device__ __forceinline__ GlobalView<R, C, float, false> view(int64_t x, int64_t y) const;
    template<int64_t R, int64_t C>
    __device__ __forceinline__ GlobalView<R, C, float, true> view_exact(int64_t x, int64_t y) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ MfmaAccF32<BM, BN> load_acc_mfma8_f32(int64_t x, int64_t y) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ void add_acc(int64_t x, int64_t y, const MfmaAccF32<BM, BN> &t) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ void store_acc(int64_t x, int64_t y, const MfmaAccF32<BM, BN> &t) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ MfmaAcc<BM, BN, 4> load_acc_mfma(int64_t x, int64_t y) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ MfmaAcc<BM, BN, 8> load_acc_mfma8(int64_t x, int64_t y) const;
    template<int64_t BM, int64_t BN, int NW>
    __device__ __forceinline__ void add_acc(int64_t x, int64_t y, const MfmaAcc<BM, BN, NW> &t) const;
    template<int64_t BM, int64_t BN, int NW>
    __device__ __forceinline__ void store_acc(int64_t x, int64_t y, const MfmaAcc<BM, BN, NW> &t) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ MfmaAcc16<BM, BN> load_acc_mfma16(int64_t x, int64_t y) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ void add_acc(int64_t x, int64_t y, const MfmaAcc16<BM, BN> &t) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ void store_acc(int64_t x, int64_t y, const MfmaAcc16<BM, BN> &t) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ FmaAcc<BM, BN> load_acc_fma(int64_t x, int64_t y) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ void store_acc(int64_t x, int64_t y, const FmaAcc<BM, BN> &t) const;
    template<int64_t BM, int64_t BN>
    __device__ __forceinline__ void add_acc(int64_t x, int64_t y, const FmaAcc<BM, BN> &t) const;
    // Fused QK^T -> softmax result access (gernels/qk_softmax.h).
    template<int64_t R, int64_t N>
    __device__ __forceinline__ RowBlock<R, N> view_row_block(int64_t x, int64_t y) const;
    template<int64_t R, int64_t N>
    __device__ __forceinline__ void store_row_block(int64_t x, int64_t y, const RowBlock<R, N> &t) const;
    // The same on 256 x 256 tiles (gernels/qk_tiles.h).
    template<int64_t R, int64_t C>
    __device__ __forceinline__ ScoreTile<R, C> view_score_tile(int64_t x, int64_t y) const;
    template<int64_t R, int64_t C>
    __device__ __forceinline__ void store_score_tile(int64_t x, int64_t y, const ScoreTile<R, C> &t) const;

    // Rows spread over the wavefronts of a workgroup (gernels/softmax.h).  The
    // wavefront count is part of the name because the code generator pastes
    // names and appends <rows, cols> only.
    template<int NW, int64_t R, int64_t C>
    __device__ __forceinline__ BlockTile<R, C, NW> load_block(int64_t x, int64_t y) const;
    template<int NW, int64_t R, int64_t C>
    __device__ __forceinline__ BlockTile<R, C, NW> view_block(int64_t x, int64_t y) const;
    template<int64_t R, int64_t C, int NW>
    __device__ __forceinline__ void store_block(int64_t x, int64_t y, const BlockTile<R, C, NW> &t) const;
#define GERN_BLOCK_ACCESSORS(NW)                                                                     \
    template<int64_t R, int64_t C>                                                                   \
    __device__ __forceinline__ BlockTile<R, C, NW> load_block##NW(int64_t x, int64_t y) const {      \
        return load_block<NW, R, C>(x, y);                                                           \
    }                                                                                                \
    template<int64_t R, int64_t C>                                                                   \
    __device__ __forceinline__ BlockTile<R, C, NW> view_block##NW(int64_t x, int64_t y) const {      \
        return view_block<NW, R, C>(x, y);                                                           \
    }
    GERN_BLOCK_ACCESSORS(2)
    GERN_BLOCK_ACCESSORS(4)
    GERN_BLOCK_ACCESSORS(8)
    GERN_BLOCK_ACCESSORS(16)
#undef GERN_BLOCK_ACCESSORS

    // Loads the R x C tile whose top-left element is (x, y).  Elements outside
    // the matrix read as 0; a tile may therefore hang over the right or bottom
    // edge (ragged last tile of a grid).
    template<int64_t R, int64_t C>
    __device__ __forceinline__ WaveTile<R, C> load_wave(int64_t x, int64_t y) const {
        WaveTile<R, C> t;
        const int lane = lane_id();
#pragma unroll
        for (int64_t r = 0; r < R; r++) {
            const int64_t rr = x + r;
            const bool row_ok = rr < row;
            const float *p = data + rr * lda + y;
            // A row can use 16-byte accesses when its first element is 16-byte
            // aligned; the test is wave-uniform.
            const bool vec_ok = (((uint64_t)p) & 15u) == 0;
#pragma unroll
            for (int64_t k = 0; k < WaveTile<R, C>::chunks; k++) {
                const int64_t lc = k * kWaveCols + 4 * lane;  // column inside the tile
                const int64_t cc = y + lc;                    // column inside the matrix
                float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
                if (row_ok && lc < C) {
                    if (vec_ok && cc + 3 < col) {
                        val = *reinterpret_cast<const float4 *>(p + lc);
                    } else {
                        if (cc + 0 < col) val.x = p[lc + 0];
                        if (cc + 1 < col) val.y = p[lc + 1];
                        if (cc + 2 < col) val.z = p[lc + 2];
                        if (cc + 3 < col) val.w = p[lc + 3];
                    }
                }
                t.v[r][k] = val;
            }
        }
        return t;
    }

    // The same tile with EVERY column of its 256-column chunks that lies
    // inside the matrix, also those past the tile's logical width C.  A chain
    // of lane-wise stages then produces valid results in those lanes too, which
    // is what store_wave_lines needs to move its window to cache-line boundaries.
    template<int64_t R, int64_t C>
    __device__ __forceinline__ WaveTile<R, C> load_wave_wide(int64_t x, int64_t y) const {
        constexpr int64_t W = WaveTile<R, C>::chunks * kWaveCols;
        const WaveTile<R, W> t = load_wave<R, W>(x, y);
        WaveTile<R, C> out;
#pragma unroll
        for (int64_t r = 0; r < R; r++) {
#pragma unroll
            for (int64_t k = 0; k < WaveTile<R, C>::chunks; k++) {
                out.v[r][k] = t.v[r][k];
            }
        }
        return out;
    }

    // An output tile: nothing is read, the producer overwrites every element.
    template<int64_t R, int64_t C>
    __device__ __forceinline__ WaveTile<R, C> view_wave(int64_t, int64_t) const {
        return WaveTile<R, C>();
    }

    // Stores the tile at (x, y), clipped to the tile's logical width C and to
    // the matrix bounds.
    template<int64_t R, int64_t C>
    __device__ __forceinline__ void store_wave(int64_t x, int64_t y, const WaveTile<R, C> &t) const {
        const int lane = lane_id();
#pragma unroll
        for (int64_t r = 0; r < R; r++) {
            const int64_t rr = x + r;
            if (rr >= row) {
                continue;
            }
            float *p = data + rr * lda + y;
            const bool vec_ok = (((uint64_t)p) & 15u) == 0;
#pragma unroll
            for (int64_t k = 0; k < WaveTile<R, C>::chunks; k++) {
                const int64_t lc = k * kWaveCols + 4 * lane;
                const int64_t cc = y + lc;
                const float4 val = t.v[r][k];
                if (vec_ok && lc + 3 < C && cc + 3 < col) {
                    // A result tile is written once and never read back by
                    // the kernel: a streaming (nontemporal) store keeps it
                    // from displacing the input rows that neighbouring tiles
                    // are about to re-read from L2 (and it is written through).
                    store_result16<kThroughStreamingStores>(data, (row - 1) * lda + col, rr * lda + y + lc, val);
                } else {
                    if (lc + 0 < C && cc + 0 < col) p[lc + 0] = val.x;
                    if (lc + 1 < C && cc + 1 < col) p[lc + 1] = val.y;
                    if (lc + 2 < C && cc + 2 < col) p[lc + 2] = val.z;
                    if (lc + 3 < C && cc + 3 < col) p[lc + 3] = val.w;
                }
            }
        }
    }

    // store_wave for a row of tiles that are C columns apart (C a multiple of
    // 32, one chunk), with every tile's window moved to whole 128-byte lines:
    // in row r the tile at column y writes from the first line boundary at or
    // after y (from column 0 when y == 0) up to the first line boundary at or
    // after y + C (up to the end of the row for the last tile).  Neighbouring
    // tiles agree on each boundary, so every element is still written exactly
    // once, and no line is shared between two wavefronts except the one that
    // holds the end of one row and the start of the next.  A window starts up
    // to 28 columns past y, so the lanes past C must hold valid results
    // (load_wave_wide, and C + 28 + the halo of the chain <= 256).  Partial
    // lines cost a read-modify-write at the memory side: on an 8192 x 8192
    // image whose result rows are 8188 floats apart, line-aligned windows take
    // the x,y,x chain from 101 to 95 us when its buffers come from HBM.
    // Rows that do not start on a 16-byte boundary keep the plain window.
    template<int64_t R, int64_t C>
    __device__ __forceinline__ void store_wave_lines(int64_t x, int64_t y, const WaveTile<R, C> &t) const {
        static_assert(WaveTile<R, C>::chunks == 1 && C % 32 == 0, "line-aligned windows: one chunk, whole lines per tile");
        const int lane = lane_id();
        const int64_t cc = y + 4 * lane;
#pragma unroll
        for (int64_t r = 0; r < R; r++) {
            const int64_t rr = x + r;
            if (rr >= row) {
                continue;
            }
            float *p = data + rr * lda;
            const uint64_t a0 = (uint64_t)(p + y), a1 = (uint64_t)(p + y + C);
            const bool vec_ok = (a0 & 15u) == 0;  // wave-uniform
            int64_t lo = y, hi = y + C;
            if (vec_ok) {
                lo = y == 0 ? 0 : y + (int64_t)(((128 - (a0 & 127u)) & 127u) / 4);
                hi = y + C + (int64_t)(((128 - (a1 & 127u)) & 127u) / 4);
            }
            hi = hi < col ? hi : col;
            const float4 val = t.v[r][0];
            if (vec_ok && cc >= lo && cc + 3 < hi) {
                store_result16<kThroughStreamingStores>(data, (row - 1) * lda + col, rr * lda + cc, val);
            } else {
                if (cc + 0 >= lo && cc + 0 < hi) p[cc + 0] = val.x;
                if (cc + 1 >= lo && cc + 1 < hi) p[cc + 1] = val.y;
                if (cc + 2 >= lo && cc + 2 < hi) p[cc + 2] = val.z;
                if (cc + 3 >= lo && cc + 3 < hi) p[cc + 3] = val.w;
            }
        }
    }
};

}  // namespace gernels
