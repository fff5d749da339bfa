// Workgroup and device-wide sum reductions, as gernels.
//
// Same names, template parameters and argument order as the reference's
// wrappers around cub::BlockReduce and cuda::atomic_ref
// (gernels/cccl/wrappers/reduce_wrappers.cuh:11-73), so that its annotations
// (gernels/cccl/gern_annot/functions.h) compose them unchanged.  The block
// reduction is a DPP / ds_swizzle butterfly inside each 64-lane wavefront and
// one LDS hop between wavefronts; the device-wide step is one relaxed
// agent-scope atomic add per workgroup (a vector-memory atomic).
#pragma once

#include "gernels/softmax.h"

namespace gernels {

// Register array of a compile-time length (what a query of ArrayF32 returns).
template<int64_t Size>
struct StaticArrayF32 {
    float data[Size];
    static constexpr int64_t size = Size;
    __device__ __forceinline__ void dummy() const {
    }
};

// float array in HBM; passed to kernels by value (pointer, length).
struct ArrayF32 {
    float *data;
    int64_t size;

    __device__ __forceinline__ ArrayF32 query(int64_t start, int64_t len) const {
        return ArrayF32{data + start, len};
    }
    template<int64_t Size>
    __device__ __forceinline__ StaticArrayF32<Size> query(int64_t start) const {
        StaticArrayF32<Size> part;
#pragma unroll
        for (int64_t i = 0; i < Size; i++) {
            part.data[i] = data[start + i];
        }
        return part;
    }
    template<int64_t Size>
    __device__ __forceinline__ void insert_array(int64_t start, const StaticArrayF32<Size> &part) const {
#pragma unroll
        for (int64_t i = 0; i < Size; i++) {
            data[start + i] = part.data[i];
        }
    }
    __device__ __forceinline__ void dummy() const {
    }
};

template<int64_t Size>
__device__ __forceinline__ StaticArrayF32<Size> allocate_local() {
    StaticArrayF32<Size> a;
#pragma unroll
    for (int64_t i = 0; i < Size; i++) {
        a.data[i] = 0.0f;
    }
    return a;
}

// Sum of `v` over the first block_size threads of the workgroup (threads are
// numbered along x); every thread gets the result.  Collective: all threads
// of the workgroup must call it.
template<int block_size>
__device__ __forceinline__ float block_sum(float v) {
    static_assert(block_size >= 1 && block_size <= 1024, "workgroup size");
    const int tid = (int)threadIdx.x;
    if constexpr (block_size % kWaveSize == 0) {
        // Whole wavefronts: butterfly inside each, one LDS hop between them.
        constexpr int kWaves = block_size / kWaveSize;
        __shared__ float partial[kWaves];
        const float x = wave_all_reduce<SumOp>(v);
        if constexpr (kWaves == 1) {
            return x;
        }
        if (lane_id() == 0) {
            partial[tid / kWaveSize] = x;
        }
        __syncthreads();
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            total += partial[w];
        }
        __syncthreads();  // partial[] may be reused by the next call
        return total;
    } else {
        // A partly filled wavefront: the cross-lane moves of the butterfly
        // would read lanes that do not exist, so the tree goes through LDS.
        __shared__ float vals[block_size];
        if (tid < block_size) {
            vals[tid] = v;
        }
        __syncthreads();
        int span = 1;
        while (span < block_size) {
            span *= 2;
        }
        for (int s = span / 2; s > 0; s /= 2) {
            if (tid < s && tid + s < block_size) {
                vals[tid] += vals[tid + s];
            }
            __syncthreads();
        }
        const float total = vals[0];
        __syncthreads();
        return total;
    }
}

// output[i] = sum of input[i * block_size .. (i + 1) * block_size); one input
// element per thread.
template<int block_size, typename T1, typename T2>
__device__ __forceinline__ void block_reduce(T1 &output, const T2 &input) {
    static_assert(T2::size == T1::size * block_size, "one input element per thread and output element");
#pragma unroll
    for (int64_t i = 0; i < T1::size; i++) {
        const int tid = (int)threadIdx.x;
        const float sum = block_sum<block_size>(tid < block_size ? input.data[i * block_size + tid] : 0.0f);
        output.data[i] = sum;  // every thread keeps the sum; thread 0's copy is the one the reference defines
    }
}

// One relaxed device-scope add per workgroup.
__device__ __forceinline__ void global_sum_single(float *total_sum, float input) {
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(total_sum, input, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// *total_sum += sum of the workgroup's block_size inputs (k is the full
// reduction length; the composed Reduce hands each workgroup its slice).
template<int k, int block_size, typename T2>
__device__ __forceinline__ void grid_reduce_total(float *total_sum, const T2 &input) {
    const int tid = (int)threadIdx.x;
    const float sum = block_sum<block_size>(tid < block_size ? input.data[tid] : 0.0f);
    global_sum_single(total_sum, sum);
}

// *total_sum += input[0] + ... + input[k - 1], added one by one by thread 0.
template<int k, typename T>
__device__ __forceinline__ void global_sum(float *total_sum, const T &input) {
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < k; i++) {
            __hip_atomic_fetch_add(total_sum, input.data[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace gernels
