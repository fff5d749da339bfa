// Host arrays of a compile-time length: subsets are copies held by value, so a
// query copies in and an insert copies back (no heap temporaries).
//
// Same interface as the reference's test library
// (test/library/array/impl/cpu-array-template.h).
#pragma once

#include <algorithm>
#include <cstdint>
#include <numeric>

namespace gern {
namespace impl {

template<int64_t Size>
struct ArrayCPUTemplate {
    static constexpr int64_t size = Size;
    float data[Size] = {0};

    // elements [start, start + Len) as a value
    template<int64_t Len>
    ArrayCPUTemplate<Len> query(int64_t start) const {
        ArrayCPUTemplate<Len> part;
        std::copy_n(data + start, Len, part.data);
        return part;
    }
    // ... and back
    template<int64_t Len>
    void insert(int64_t start, const ArrayCPUTemplate<Len> &part) {
        std::copy_n(part.data, Len, data + start);
    }
    void destroy() {
    }
    // 0, 1, 2, ...
    void ascending() {
        std::iota(data, data + Size, 0.0f);
    }
};

template<int64_t Len>
inline ArrayCPUTemplate<Len> temp_allocate() {
    return {};
}

template<int64_t Len, typename In, typename Out>
inline void add(const In &in, Out &out) {
    std::transform(in.data, in.data + Len, out.data, [](float v) { return v + 1.0f; });
}

}  // namespace impl
}  // namespace gern
