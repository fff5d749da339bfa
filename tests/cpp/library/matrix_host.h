// Host-side dense row-major matrix with a row pitch, and the functions the
// host lowering tests compose.
//
// Same interface and semantics as the reference's test library
// (test/library/matrix/impl/cpu-matrix.h:21-212): query is a view that shares
// the parent's pitch, allocate is a fresh matrix with pitch = its width, insert
// copies rows back (nothing to do for a view of the same storage).
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>

namespace gern {
namespace impl {

struct MatrixCPU {
    float *data = nullptr;
    int64_t row = 0, col = 0, lda = 0;

    MatrixCPU(float *data, int64_t row, int64_t col, int64_t lda)
        : data(data), row(row), col(col), lda(lda) {
    }
    MatrixCPU(int64_t row, int64_t col, int64_t lda)
        : data(static_cast<float *>(std::malloc(sizeof(float) * (row * lda > 0 ? row * lda : 1)))), row(row), col(col), lda(lda) {
    }
    static MatrixCPU allocate(int64_t, int64_t, int64_t l_x, int64_t l_y) {
        return MatrixCPU(l_x, l_y, l_y);
    }
    static MatrixCPU allocate_zero(int64_t, int64_t, int64_t l_x, int64_t l_y) {
        MatrixCPU m(l_x, l_y, l_y);
        m.fill(0.0f);
        return m;
    }
    MatrixCPU query(int64_t x, int64_t y, int64_t l_x, int64_t l_y) const {
        return MatrixCPU(data + x * lda + y, l_x, l_y, lda);
    }
    void insert(int64_t x, int64_t y, int64_t l_x, int64_t l_y, const MatrixCPU &part) {
        for (int64_t i = 0; i < l_x; i++) {
            float *dst = data + (x + i) * lda + y;
            const float *src = part.data + i * part.lda;
            if (dst != src) {
                std::memmove(dst, src, sizeof(float) * l_y);
            }
        }
    }
    void destroy() {
        std::free(data);
        data = nullptr;
    }
    float &at(int64_t i, int64_t j) {
        return data[i * lda + j];
    }
    const float &at(int64_t i, int64_t j) const {
        return data[i * lda + j];
    }
    void fill(float v) {
        for (int64_t i = 0; i < row; i++) {
            for (int64_t j = 0; j < col; j++) {
                at(i, j) = v;
            }
        }
    }
    void ascending() {
        for (int64_t i = 0; i < row; i++) {
            for (int64_t j = 0; j < col; j++) {
                at(i, j) = static_cast<float>(i * col + j);
            }
        }
    }
};

inline void add(MatrixCPU in, MatrixCPU out) {
    for (int64_t i = 0; i < in.row; i++) {
        for (int64_t j = 0; j < in.col; j++) {
            out.at(i, j) = in.at(i, j) + 1.0f;
        }
    }
}

// c(i,j) += sum over k of a(i,k) * b(k,j), the sum formed in a local first.
inline void matrix_multiply(MatrixCPU a, MatrixCPU b, MatrixCPU c, int64_t k_dim) {
    for (int64_t i = 0; i < c.row; i++) {
        for (int64_t j = 0; j < c.col; j++) {
            float sum = 0.0f;
            for (int64_t k = 0; k < k_dim; k++) {
                sum += a.at(i, k) * b.at(k, j);
            }
            c.at(i, j) += sum;
        }
    }
}

}  // namespace impl
}  // namespace gern
