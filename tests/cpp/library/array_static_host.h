// Host arrays of a compile-time length: subsets are copies held by value, so a
// query copies in and an insert copies back (no heap temporaries).
//
// Same interface as the reference's test library
// (test/library/array/impl/cpu-array-template.h).
#pragma once

#include <cstdint>

namespace gern {
namespace impl {

template<int64_t Size>
struct ArrayCPUTemplate {
    float data[Size] = {0};
    static constexpr int64_t size = Size;

    template<int64_t Len>
    ArrayCPUTemplate<Len> query(int64_t start) const {
        ArrayCPUTemplate<Len> part;
        for (int64_t i = 0; i < Len; i++) {
            part.data[i] = data[start + i];
        }
        return part;
    }
    template<int64_t Len>
    void insert(int64_t start, const ArrayCPUTemplate<Len> &part) {
        for (int64_t i = 0; i < Len; i++) {
            data[start + i] = part.data[i];
        }
    }
    void destroy() {
    }
    void ascending() {
        for (int64_t i = 0; i < Size; i++) {
            data[i] = static_cast<float>(i);
        }
    }
};

template<int64_t Len>
inline ArrayCPUTemplate<Len> temp_allocate() {
    return ArrayCPUTemplate<Len>();
}

template<int64_t Len, typename In, typename Out>
inline void add(const In &in, Out &out) {
    for (int64_t i = 0; i < Len; i++) {
        out.data[i] = in.data[i] + 1.0f;
    }
}

}  // namespace impl
}  // namespace gern
