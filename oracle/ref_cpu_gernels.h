// Host functions on the reference's CPU matrix view that the reference tree
// does not provide itself, used ONLY when the reference library is built into
// oracle/_ref/ to lower the composed pipelines on the CPU (test
// infrastructure; never part of the product).
//
// blur_x / blur_y restate apps/common/impl/impl.h:190-250 (GPU register tiles)
// for impl::MatrixCPU views: running sum from 0, taps left to right (top to
// bottom), one division by the tap count.  subtract_vec_fixed is the
// reference's subtract_vec (test/library/matrix/impl/cpu-matrix.h:170-181)
// with the operands in the order its GPU twin uses (x - v, impl.h:71).
#pragma once

#include "cpu-matrix.h"

namespace gern {
namespace impl {

template<int64_t stride>
inline void blur_x(MatrixCPU in, MatrixCPU out) {
    for (int64_t i = 0; i < out.row; i++) {
        for (int64_t j = 0; j < out.col; j++) {
            float sum = 0;
            for (int64_t s = 0; s < stride; s++) {
                sum += in.data[i * in.lda + j + s];
            }
            out.data[i * out.lda + j] = sum / stride;
        }
    }
}

template<int64_t stride>
inline void blur_y(MatrixCPU in, MatrixCPU out) {
    for (int64_t i = 0; i < out.row; i++) {
        for (int64_t j = 0; j < out.col; j++) {
            float sum = 0;
            for (int64_t s = 0; s < stride; s++) {
                sum += in.data[(i + s) * in.lda + j];
            }
            out.data[i * out.lda + j] = sum / stride;
        }
    }
}

inline void subtract_vec_fixed(ArrayCPU b, MatrixCPU a, MatrixCPU out) {
    for (int64_t i = 0; i < a.row; i++) {
        float v = b.data[i];
        for (int64_t j = 0; j < a.col; j++) {
            out.data[i * out.lda + j] = a.data[i * a.lda + j] - v;
        }
    }
}

}  // namespace impl
}  // namespace gern
