// A workgroup-level allocator over the kernel's dynamic LDS, for data
// structures that stage tiles into LDS (Stage(...) with an LDS query function)
// and for Global(..., smem_size, SharedMemoryManager).
//
// The reference's allocator (test/library/smem_allocator/sh_malloc.h:12-56,
// gernels/mm/impl/sh_malloc.h) is a bump pointer that never frees and
// overwrites live data once it wraps.  This one is a stack with a small table
// at the start of LDS: a request takes the space above the highest block, a
// block may be given back in any order, and the stack shrinks past every
// block that has been given back once nothing in use lies above it.  The
// staged tiles of a loop body are thus returned on every iteration, nested
// Stage scopes may release their blocks in any order, and the space of a
// block released out of order comes back when the blocks above it do.  The
// 160 KB of a gfx950 CU are the hard limit (checked at launch).
//
// Every entry point is COLLECTIVE: all threads of the workgroup call it with
// the same arguments and get the same answer.  An allocation costs two
// barriers and one LDS read per thread (every thread reads the top of the
// stack itself; the first thread records the block), a release one barrier.
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

// Table at the start of dynamic LDS (128 bytes): a stack of blocks in address
// order, [sizeof(LdsTable), top) in all.
struct LdsTable {
    uint32_t capacity;  // bytes of dynamic LDS
    uint32_t top;       // first byte above the highest block
    uint32_t count;     // blocks on the stack
    uint32_t overflow;  // set once a request could not be met
    struct Block {
        uint32_t offset;
        uint32_t size_used;  // size in bytes, bit 0 = in use
    } block[kLdsMaxBlocks];
};
static_assert(sizeof(LdsTable) == 128, "the table is 128 bytes");

__device__ __forceinline__ bool lds_first_thread() {
    return threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0;
}

// Called once at the top of the kernel (SharedMemoryManager's init call).
__device__ __forceinline__ void lds_init(int64_t bytes) {
    if (lds_first_thread()) {
        LdsTable *t = reinterpret_cast<LdsTable *>(gern_lds);
        t->capacity = (uint32_t)bytes;
        t->top = (uint32_t)sizeof(LdsTable);
        t->count = 0;
        t->overflow = 0;
    }
    __syncthreads();
}

// A 16-byte aligned block of at least `bytes`.  When it does not fit (or the
// table is full) the request cannot fail loudly from inside a kernel: the
// table's overflow flag is set and the START of the heap is returned, so that
// the caller's accesses stay inside LDS (results are then wrong, as with the
// reference's allocator once it wraps, but nothing faults).  lds_overflowed()
// tells the kernel, the count in gern_lds_overflows tells the host.
__device__ __forceinline__ void *lds_alloc(int64_t bytes) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    LdsTable *t = reinterpret_cast<LdsTable *>(gern_lds);
    __syncthreads();  // the table is as the last call left it, and readers of released blocks are done
    const u32x4 head = *reinterpret_cast<const u32x4 *>(gern_lds);  // capacity, top, count, overflow
    const uint32_t need = (((uint32_t)bytes + 15u) & ~15u);
    const bool fits = head[2] < (uint32_t)kLdsMaxBlocks && (uint64_t)head[1] + need <= (uint64_t)head[0] &&
                      head[0] >= (uint32_t)sizeof(LdsTable);
    const uint32_t got = fits ? head[1] : (uint32_t)sizeof(LdsTable);
    __syncthreads();  // every thread has read the top of the stack
    if (lds_first_thread()) {
        if (fits) {
            t->block[head[2]].offset = got;
            t->block[head[2]].size_used = need | 1u;
            t->top = got + need;
            t->count = head[2] + 1u;
        } else {
            t->overflow = 1;
            atomicAdd(&gern_lds_overflows, 1u);
        }
    }
    return gern_lds + got;
}

__device__ __forceinline__ bool lds_overflowed() {
    return reinterpret_cast<const LdsTable *>(gern_lds)->overflow != 0;
}

// Returns a block.  The stack shrinks past every released block that has
// nothing in use above it.
__device__ __forceinline__ void lds_free(const void *ptr) {
    LdsTable *t = reinterpret_cast<LdsTable *>(gern_lds);
    __syncthreads();  // all readers of the block are done; the table is as the last call left it
    if (lds_first_thread() && ptr != nullptr && !t->overflow) {
        const uint32_t at = (uint32_t)(static_cast<const unsigned char *>(ptr) - gern_lds);
        uint32_t count = t->count;
        for (uint32_t b = count; b-- > 0;) {  // the block is usually the highest one or the one below
            if (t->block[b].offset == at) {
                t->block[b].size_used &= ~1u;
                break;
            }
        }
        while (count > 0 && !(t->block[count - 1].size_used & 1u)) {
            count--;
        }
        t->top = count > 0 ? t->block[count - 1].offset + (t->block[count - 1].size_used & ~1u) : (uint32_t)sizeof(LdsTable);
        t->count = count;
    }
    // no barrier here: every entry point starts with one
}

// Bytes currently handed out (for tests and reports).
__device__ __forceinline__ uint32_t lds_in_use() {
    const LdsTable *t = reinterpret_cast<const LdsTable *>(gern_lds);
    uint32_t total = 0;
    for (uint32_t b = 0; b < t->count; b++) {
        if (t->block[b].size_used & 1u) {
            total += t->block[b].size_used & ~1u;
        }
    }
    return total;
}

}  // namespace gernels
