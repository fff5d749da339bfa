// Host-side handles of the device test data structures: same layout as the
// structs in array_device.h / matrix_device.h (they are passed to the kernel
// by value), with upload / download helpers over the C ABI runtime.
#pragma once

#include "gern_hip.h"

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace gern {
namespace impl {

inline void hipCheck(int rc) {
    if (rc != 0) {
        std::string msg(gern_hip_last_error(nullptr, 0) + 1, '\0');
        gern_hip_last_error(msg.data(), msg.size());
        throw std::runtime_error(msg);
    }
}

struct ArrayGPU {
    float *data = nullptr;
    int64_t size = 0;

    explicit ArrayGPU(int64_t n)
        : size(n) {
        hipCheck(gern_hip_malloc(reinterpret_cast<void **>(&data), sizeof(float) * n));
        hipCheck(gern_hip_memset(data, 0, sizeof(float) * n));
    }
    void upload(const std::vector<float> &v) {
        hipCheck(gern_hip_memcpy_h2d(data, v.data(), sizeof(float) * size));
    }
    void ascending() {
        std::vector<float> v(size);
        for (int64_t i = 0; i < size; i++) {
            v[i] = static_cast<float>(i);
        }
        upload(v);
    }
    std::vector<float> get() const {
        hipCheck(gern_hip_sync());
        std::vector<float> v(size);
        hipCheck(gern_hip_memcpy_d2h(v.data(), data, sizeof(float) * size));
        return v;
    }
    void destroy() {
        gern_hip_free(data);
        data = nullptr;
    }
};

struct MatrixGPU {
    float *data = nullptr;
    int64_t row = 0, col = 0, lda = 0;

    MatrixGPU(int64_t row, int64_t col, int64_t lda)
        : row(row), col(col), lda(lda) {
        hipCheck(gern_hip_malloc(reinterpret_cast<void **>(&data), sizeof(float) * row * lda));
        hipCheck(gern_hip_memset(data, 0, sizeof(float) * row * lda));
    }
    void fill(float value) {
        std::vector<float> v(row * lda, value);
        hipCheck(gern_hip_memcpy_h2d(data, v.data(), sizeof(float) * v.size()));
    }
    void ascending() {
        std::vector<float> v(row * lda, 0.0f);
        for (int64_t i = 0; i < row; i++) {
            for (int64_t j = 0; j < col; j++) {
                v[i * lda + j] = static_cast<float>(i * col + j);
            }
        }
        hipCheck(gern_hip_memcpy_h2d(data, v.data(), sizeof(float) * v.size()));
    }
    std::vector<float> get() const {
        hipCheck(gern_hip_sync());
        std::vector<float> v(row * lda);
        hipCheck(gern_hip_memcpy_d2h(v.data(), data, sizeof(float) * v.size()));
        return v;
    }
    void destroy() {
        gern_hip_free(data);
        data = nullptr;
    }
};

}  // namespace impl
}  // namespace gern
