// The reference's blur gernels (apps/common/impl/impl.h:190-250: `stride` taps
// added left to right, then one division by `stride`) on the tile types of
// gernels/lds_matrix.h: anything with constant extents row / col and element
// access (i, j) -- a window of a tile that the workgroup staged into LDS, a
// thread's register tile, a window of a matrix in global memory.  With them a
// user-level schedule can stage a block's input tile, HALO INCLUDED, into LDS
// once and let every thread take its own window of it: the halo extents are
// the ones the composed annotations infer (annot/blur.h), nobody writes them
// down.
//
// These are one-thread-per-tile functions for schedules written at the level
// of the API; the tuned blur (one wavefront per tile, register halos, DPP) is
// gernels/blur.h.
#pragma once

#include "gernels/lds_matrix.h"

namespace gernels {

// out(i, j) = (in(i, j) + ... + in(i, j + stride - 1)) / stride
template<int64_t stride, typename In, typename Out>
__device__ __forceinline__ void blur_x_per_thread(const In &in, Out &out) {
    static_assert(In::row >= Out::row && In::col >= Out::col + stride - 1, "the input tile holds the halo columns");
#pragma unroll
    for (int64_t i = 0; i < Out::row; i++) {
#pragma unroll
        for (int64_t j = 0; j < Out::col; j++) {
            float sum = 0.0f;
#pragma unroll
            for (int64_t s = 0; s < stride; s++) {
                sum += in(i, j + s);
            }
            out(i, j) = sum / (float)stride;
        }
    }
}

// out(i, j) = (in(i, j) + ... + in(i + stride - 1, j)) / stride
template<int64_t stride, typename In, typename Out>
__device__ __forceinline__ void blur_y_per_thread(const In &in, Out &out) {
    static_assert(In::row >= Out::row + stride - 1 && In::col >= Out::col, "the input tile holds the halo rows");
#pragma unroll
    for (int64_t i = 0; i < Out::row; i++) {
#pragma unroll
        for (int64_t j = 0; j < Out::col; j++) {
            float sum = 0.0f;
#pragma unroll
            for (int64_t s = 0; s < stride; s++) {
                sum += in(i + s, j);
            }
            out(i, j) = sum / (float)stride;
        }
    }
}

}  // namespace gernels
