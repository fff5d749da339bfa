// Device-side float array for the GPU lowering tests; included by the code
// the Runner generates and compiles with hiprtc (no host code, no C library).
//
// Same interface as the reference's device test library
// (test/library/array/impl/gpu-array.h:23-102, gpu-array.cu).
#pragma once

#include "gernels/prelude.h"

namespace gern {
namespace impl {

template<int64_t Size>
struct ArrayStaticGPU {
    float data[Size];
    static constexpr int64_t size = Size;
    __device__ void dummy() const {
    }
};

struct ArrayGPU {
    float *data;
    int64_t size;

    __device__ ArrayGPU query(int64_t start, int64_t len) const {
        return ArrayGPU{data + start, len};
    }
    // A queried ArrayGPU is a view: nothing to copy back.
    __device__ void insert(int64_t, int64_t, const ArrayGPU &) const {
    }
    template<int64_t Size>
    __device__ ArrayStaticGPU<Size> query(int64_t start) const {
        ArrayStaticGPU<Size> part;
        for (int64_t i = 0; i < Size; i++) {
            part.data[i] = data[start + i];
        }
        return part;
    }
    template<int64_t Size>
    __device__ void insert_array(int64_t start, const ArrayStaticGPU<Size> &part) const {
        for (int64_t i = 0; i < Size; i++) {
            data[start + i] = part.data[i];
        }
    }
    __device__ void destroy() const {
    }
    __device__ void dummy() const {
    }
};

template<int64_t Size>
__device__ ArrayStaticGPU<Size> allocate_local() {
    ArrayStaticGPU<Size> a;
    for (int64_t i = 0; i < Size; i++) {
        a.data[i] = 0.0f;
    }
    return a;
}

__device__ inline void add_1(ArrayGPU in, ArrayGPU out) {
    for (int64_t i = 0; i < in.size; i++) {
        out.data[i] = in.data[i] + 1.0f;
    }
}

template<int64_t Len, typename In, typename Out>
__device__ inline void add_1(const In &in, Out &out) {
    for (int64_t i = 0; i < Len; i++) {
        out.data[i] = in.data[i] + 1.0f;
    }
}

// out[i] += sum of the first k entries of `in`.
__device__ inline void reduction(ArrayGPU in, ArrayGPU out, int64_t k) {
    for (int64_t i = 0; i < out.size; i++) {
        for (int64_t j = 0; j < k; j++) {
            out.data[i] += in.data[j];
        }
    }
}

}  // namespace impl
}  // namespace gern
