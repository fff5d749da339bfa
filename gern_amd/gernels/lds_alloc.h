// A workgroup-level allocator over the kernel's dynamic LDS, for data
// structures that stage tiles into LDS (Stage(...) with an LDS query function)
// and for Global(..., smem_size, SharedMemoryManager).
//
// The reference's allocator (test/library/smem_allocator/sh_malloc.h:12-56,
// gernels/mm/impl/sh_malloc.h) is a bump pointer that never frees and
// overwrites live data once it wraps.  This one keeps a first-fit free list
// in a small table at the start of LDS, so that the staged tiles of a loop
// body are returned on every iteration and nested Stage scopes may release
// their blocks in any order; the 160 KB of a gfx950 CU are the hard limit
// (checked at launch).
//
// Every entry point is COLLECTIVE: all threads of the workgroup call it with
// the same arguments and get the same answer; thread 0 edits the table.
#pragma once

#include "gernels/prelude.h"

namespace gernels {

extern __shared__ __attribute__((aligned(16))) unsigned char gern_lds[];

constexpr int kLdsMaxBlocks = 14;

}  // namespace gernels

// Requests the allocator could not meet since the code was loaded, over all
// launches and workgroups.  A word in device memory with an unmangled name, so
// that the host can find it in the loaded code (Runner::ldsOverflows()).
extern "C" __device__ unsigned int gern_lds_overflows = 0;

namespace gernels {

// Table at the start of dynamic LDS (128 bytes).  Blocks are kept sorted by
// offset and cover [first, capacity) without gaps; a block is free or in use.
struct LdsTable {
    uint32_t capacity;
    uint32_t count;
    uint32_t answer;    // the last allocation's offset, read by every thread
    uint32_t overflow;  // set once a request could not be met
    uint32_t offset[kLdsMaxBlocks];
    uint32_t size_used[kLdsMaxBlocks];  // size in bytes, bit 0 = in use
};

__device__ __forceinline__ bool lds_first_thread() {
    return threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0;
}

// Called once at the top of the kernel (SharedMemoryManager's init call).
__device__ __forceinline__ void lds_init(int64_t bytes) {
    if (lds_first_thread()) {
        LdsTable *t = reinterpret_cast<LdsTable *>(gern_lds);
        const uint32_t first = (uint32_t)sizeof(LdsTable);
        t->capacity = (uint32_t)bytes;
        t->count = 1;
        t->answer = 0;
        t->overflow = 0;
        t->offset[0] = first;
        t->size_used[0] = (bytes > first ? ((uint32_t)bytes - first) & ~15u : 0u);
    }
    __syncthreads();
}

// A 16-byte aligned block of at least `bytes`.  When nothing fits (or the table
// is full) the request cannot fail loudly from inside a kernel: the table's
// overflow flag is set and the START of the heap is returned, so that the
// caller's accesses stay inside LDS (results are then wrong, as with the
// reference's allocator once it wraps, but nothing faults).  lds_overflowed()
// tells the kernel, the count in gern_lds_overflows tells the host.
__device__ __forceinline__ void *lds_alloc(int64_t bytes) {
    LdsTable *t = reinterpret_cast<LdsTable *>(gern_lds);
    __syncthreads();  // earlier readers of `answer` are done
    if (lds_first_thread()) {
        const uint32_t need = (((uint32_t)bytes + 15u) & ~15u);
        uint32_t got = 0;
        for (uint32_t b = 0; b < t->count; b++) {
            const uint32_t sz = t->size_used[b] & ~1u;
            if ((t->size_used[b] & 1u) || sz < need) {
                continue;
            }
            if (sz > need && t->count < (uint32_t)kLdsMaxBlocks) {
                // split: the tail stays free
                for (uint32_t m = t->count; m > b + 1; m--) {
                    t->offset[m] = t->offset[m - 1];
                    t->size_used[m] = t->size_used[m - 1];
                }
                t->offset[b + 1] = t->offset[b] + need;
                t->size_used[b + 1] = sz - need;
                t->count++;
                t->size_used[b] = need | 1u;
            } else {
                t->size_used[b] = sz | 1u;
            }
            got = t->offset[b];
            break;
        }
        if (got == 0) {
            t->overflow = 1;
            got = (uint32_t)sizeof(LdsTable);
            atomicAdd(&gern_lds_overflows, 1u);
        }
        t->answer = got;
    }
    __syncthreads();
    return gern_lds + t->answer;
}

__device__ __forceinline__ bool lds_overflowed() {
    return reinterpret_cast<const LdsTable *>(gern_lds)->overflow != 0;
}

// Returns a block; neighbouring free blocks are merged.
__device__ __forceinline__ void lds_free(const void *ptr) {
    LdsTable *t = reinterpret_cast<LdsTable *>(gern_lds);
    __syncthreads();  // all readers of the block are done
    if (lds_first_thread() && ptr != nullptr && !t->overflow) {
        const uint32_t at = (uint32_t)(static_cast<const unsigned char *>(ptr) - gern_lds);
        for (uint32_t b = 0; b < t->count; b++) {
            if (t->offset[b] != at) {
                continue;
            }
            t->size_used[b] &= ~1u;
            // merge with the next block, then with the previous one
            for (int pass = 0; pass < 2; pass++) {
                const uint32_t lo = pass == 0 ? b : (b > 0 ? b - 1 : t->count);
                if (lo + 1 < t->count && !(t->size_used[lo] & 1u) && !(t->size_used[lo + 1] & 1u)) {
                    t->size_used[lo] += t->size_used[lo + 1];
                    for (uint32_t m = lo + 1; m + 1 < t->count; m++) {
                        t->offset[m] = t->offset[m + 1];
                        t->size_used[m] = t->size_used[m + 1];
                    }
                    t->count--;
                }
            }
            break;
        }
    }
    __syncthreads();
}

// Bytes currently handed out (for tests and reports).
__device__ __forceinline__ uint32_t lds_in_use() {
    const LdsTable *t = reinterpret_cast<const LdsTable *>(gern_lds);
    uint32_t total = 0;
    for (uint32_t b = 0; b < t->count; b++) {
        if (t->size_used[b] & 1u) {
            total += t->size_used[b] & ~1u;
        }
    }
    return total;
}

}  // namespace gernels
