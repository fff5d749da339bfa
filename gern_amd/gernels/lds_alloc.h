// A workgroup-level allocator over the kernel's dynamic LDS, for data
// structures that stage tiles into LDS (Stage(...) with an LDS query function)
// and for Global(..., smem_size, SharedMemoryManager).
//
// The reference's allocator (test/library/smem_allocator/sh_malloc.h:12-56)
// is a bump pointer kept in the first words of shared memory and is called by
// thread 0 only.  This one is collective: every thread of the workgroup calls
// lds_alloc and every thread gets the same address, so the callers need no
// extra __shared__ pointer and no second barrier.  Allocation is a bump with
// LIFO release (lds_release back to a mark), which is what nested Stage scopes
// need; the 160 KB of a gfx950 CU are the hard limit (checked at launch).
#pragma once

#include "gernels/prelude.h"

namespace gernels {

extern __shared__ __attribute__((aligned(16))) unsigned char gern_lds[];

// Header at the start of dynamic LDS: capacity and current top, in bytes.
struct LdsHeader {
    uint32_t capacity;
    uint32_t top;
    uint32_t pad[2];
};

// Called once at the top of the kernel (SharedMemoryManager's init call).
__device__ __forceinline__ void lds_init(int64_t bytes) {
    if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
        LdsHeader *h = reinterpret_cast<LdsHeader *>(gern_lds);
        h->capacity = (uint32_t)bytes;
        h->top = (uint32_t)sizeof(LdsHeader);
    }
    __syncthreads();
}

// Collective: all threads of the workgroup call with the same size and get
// the same 16-byte aligned block, or nullptr when the region is exhausted.
__device__ __forceinline__ void *lds_alloc(int64_t bytes) {
    LdsHeader *h = reinterpret_cast<LdsHeader *>(gern_lds);
    const uint32_t need = ((uint32_t)bytes + 15u) & ~15u;
    const uint32_t at = h->top;  // every thread reads the same value
    __syncthreads();             // ... before anyone moves it
    if (at + need > h->capacity) {
        return nullptr;
    }
    if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
        h->top = at + need;
    }
    __syncthreads();
    return gern_lds + at;
}

// Current top, to release everything allocated after it.
__device__ __forceinline__ uint32_t lds_mark() {
    return reinterpret_cast<LdsHeader *>(gern_lds)->top;
}

__device__ __forceinline__ void lds_release(uint32_t mark) {
    __syncthreads();  // all readers of the released blocks are done
    if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
        reinterpret_cast<LdsHeader *>(gern_lds)->top = mark;
    }
    __syncthreads();
}

}  // namespace gernels
