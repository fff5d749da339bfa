// Host-side float array and the element-wise functions the CPU lowering
// tests compose.  Included both by the test programs and by the code the
// Runner generates for them.
//
// Same interface and semantics as the reference's test library
// (test/library/array/impl/cpu-array.h:16-118): query is a pointer view,
// allocate is a zeroed fresh array, insert copies a sub-range back.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <cstring>

namespace gern {
namespace impl {

struct ArrayCPU {
    float *data = nullptr;
    int64_t size = 0;

    ArrayCPU(float *data, int64_t size)
        : data(data), size(size) {
    }
    explicit ArrayCPU(int64_t size)
        : data(static_cast<float *>(std::calloc(size > 0 ? size : 1, sizeof(float)))), size(size) {
    }
    static ArrayCPU allocate(int64_t, int64_t len) {
        return ArrayCPU(len);
    }
    ArrayCPU query(int64_t start, int64_t len) const {
        return ArrayCPU(data + start, len);
    }
    ArrayCPU new_stage(int64_t start, int64_t len) const {
        return query(start, len);
    }
    void insert(int64_t start, int64_t len, const ArrayCPU &part) {
        if (part.data != data + start) {
            std::memmove(data + start, part.data, sizeof(float) * len);
        }
    }
    void new_insert(int64_t start, int64_t len, const ArrayCPU &part) {
        insert(start, len, part);
    }
    void destroy() {
        std::free(data);
        data = nullptr;
    }
    void fill(float v) {
        for (int64_t i = 0; i < size; i++) {
            data[i] = v;
        }
    }
    void ascending() {
        for (int64_t i = 0; i < size; i++) {
            data[i] = static_cast<float>(i);
        }
    }
};

inline void add_1(ArrayCPU in, ArrayCPU out) {
    for (int64_t i = 0; i < in.size; i++) {
        out.data[i] = in.data[i] + 1.0f;
    }
}

template<int64_t Len>
inline void add1Template(ArrayCPU in, ArrayCPU out) {
    for (int64_t i = 0; i < Len; i++) {
        out.data[i] = in.data[i] + 1.0f;
    }
}

inline void add_1_float(ArrayCPU in, ArrayCPU out, float f) {
    for (int64_t i = 0; i < in.size; i++) {
        out.data[i] = in.data[i] + f;
    }
}

// out[i] += sum of the first k entries of `in`, for every i of `out`.
inline void reduction(ArrayCPU in, ArrayCPU out, int64_t k) {
    for (int64_t i = 0; i < out.size; i++) {
        for (int64_t j = 0; j < k; j++) {
            out.data[i] += in.data[j];
        }
    }
}

}  // namespace impl
}  // namespace gern
