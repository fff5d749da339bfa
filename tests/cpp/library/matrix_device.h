// Device-side matrix for the GPU lowering tests: a view type over global
// memory, and a variant whose query stages the tile into LDS through the
// workgroup allocator.
//
// Interface as in the reference's device test library
// (test/library/matrix/impl/gpu-matrix.h:19-110).
#pragma once

#include "gernels/lds_alloc.h"

namespace gern {
namespace impl {

struct MatrixGPU {
    float *data;
    int64_t row, col, lda;

    __device__ MatrixGPU query(int64_t x, int64_t y, int64_t l_x, int64_t l_y) const {
        return MatrixGPU{data + x * lda + y, l_x, l_y, lda};
    }
    // Collective over the workgroup: copies the l_x x l_y tile at (x, y) into
    // freshly allocated LDS (row pitch l_y).
    __device__ MatrixGPU stage_into_smem(int64_t x, int64_t y, int64_t l_x, int64_t l_y) const {
        float *tile = static_cast<float *>(gernels::lds_alloc(l_x * l_y * (int64_t)sizeof(float)));
        const int64_t nthreads = (int64_t)blockDim.x * blockDim.y * blockDim.z;
        const int64_t tid = threadIdx.x + (int64_t)blockDim.x * (threadIdx.y + (int64_t)blockDim.y * threadIdx.z);
        for (int64_t e = tid; e < l_x * l_y; e += nthreads) {
            tile[e] = data[(x + e / l_y) * lda + (y + e % l_y)];
        }
        __syncthreads();
        return MatrixGPU{tile, l_x, l_y, l_y};
    }
    // Collective: writes a tile back (no-op for a view of the same storage).
    __device__ void insert(int64_t x, int64_t y, int64_t l_x, int64_t l_y, const MatrixGPU &part) const {
        if (part.data == data + x * lda + y) {
            return;
        }
        __syncthreads();
        const int64_t nthreads = (int64_t)blockDim.x * blockDim.y * blockDim.z;
        const int64_t tid = threadIdx.x + (int64_t)blockDim.x * (threadIdx.y + (int64_t)blockDim.y * threadIdx.z);
        for (int64_t e = tid; e < l_x * l_y; e += nthreads) {
            data[(x + e / l_y) * lda + (y + e % l_y)] = part.data[(e / l_y) * part.lda + e % l_y];
        }
    }
    __device__ void destroy() const {
    }
};

// One thread does the whole tile.
__device__ inline void add(MatrixGPU in, MatrixGPU out) {
    for (int64_t i = 0; i < in.row; i++) {
        for (int64_t j = 0; j < in.col; j++) {
            out.data[i * out.lda + j] = in.data[i * in.lda + j] + 1.0f;
        }
    }
}

// The threads of the workgroup share the tile.
__device__ inline void add_smem(MatrixGPU in, MatrixGPU out) {
    for (int64_t i = threadIdx.x; i < in.row; i += blockDim.x) {
        for (int64_t j = threadIdx.y; j < in.col; j += blockDim.y) {
            out.data[i * out.lda + j] = in.data[i * in.lda + j] + 1.0f;
        }
    }
    __syncthreads();
}

}  // namespace impl
}  // namespace gern
