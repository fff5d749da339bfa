// Host-side float array and the element-wise functions the CPU lowering
// tests compose.  Included both by the test programs and by the code the
// Runner generates for them.
//
// Same interface and semantics as the reference's test library
// (test/library/array/impl/cpu-array.h:16-118): query is a pointer view,
// allocate is a zeroed fresh array, insert copies a sub-range back.
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <numeric>

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
        std::fill_n(data, size, v);
    }
    void ascending() {
        std::iota(data, data + size, 0.0f);
    }
};

namespace detail {
// out[i] = in[i] + delta for the first n elements
inline void add_constant(const ArrayCPU &in, ArrayCPU &out, int64_t n, float delta) {
    std::transform(in.data, in.data + n, out.data, [delta](float v) { return v + delta; });
}
}  // namespace detail

inline void add_1(ArrayCPU in, ArrayCPU out) {
    detail::add_constant(in, out, in.size, 1.0f);
}

template<int64_t Len>
inline void add1Template(ArrayCPU in, ArrayCPU out) {
    detail::add_constant(in, out, Len, 1.0f);
}

inline void add_1_float(ArrayCPU in, ArrayCPU out, float f) {
    detail::add_constant(in, out, in.size, f);
}

// Every element of `out` grows by in[0] + ... + in[k - 1], added one term at a
// time (left to right, in fp32) to the element itself.
inline void reduction(ArrayCPU in, ArrayCPU out, int64_t k) {
    for (float *o = out.data; o != out.data + out.size; ++o) {
        *o = std::accumulate(in.data, in.data + k, *o);
    }
}

// One float that a program computes once and every tile reads: a data
// structure without index fields (its query, open(), takes nothing).
struct ScalarCPU {
    float *value = nullptr;
    static ScalarCPU allocate() {
        ScalarCPU s;
        s.value = static_cast<float *>(std::calloc(1, sizeof(float)));
        return s;
    }
    ScalarCPU open() const {
        return *this;
    }
    void destroy() {
        std::free(value);
        value = nullptr;
    }
};

// *out = in[0] (what the array starts with)
inline void first_element(ArrayCPU in, ScalarCPU out) {
    *out.value = in.data[0];
}

// out[i] = in[i] + *s
inline void add_scalar(ArrayCPU in, ScalarCPU s, ArrayCPU out) {
    detail::add_constant(in, out, in.size, *s.value);
}

}  // namespace impl
}  // namespace gern
