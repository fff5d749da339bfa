// Matrices for USER-WRITTEN schedules: a global matrix whose tiles can be
// viewed in place, copied into registers, or staged into LDS by the whole
// workgroup, and the scalar matrix_multiply that works on any of them.
//
// This is the gfx950 counterpart of the reference's gernels/mm/impl/
// matrix-gpu.h:182-508 and matrix_multiply.h:18-76, with the same method names
// (the reference's annotations name them in generated code), except that
// "smem" stays in the names only for that compatibility.  What differs:
//  * the three staging methods are three ways of filling an LDS tile with ALL
//    threads of the workgroup, whatever the block shape (the reference
//    indexes by threadIdx.x / .y and silently assumes the block shape matches
//    the tile): stage_into_smem copies one float per lane and step,
//    stage_into_smem_vec 16 bytes per lane and step through registers, and
//    stage_into_smem_flat has the memory pipeline write into LDS directly
//    (buffer_load_dwordx4 ... lds, no register round trip, no LDS write
//    instruction), which fixes the LDS layout to the dense one;
//  * LDS rows are padded by one 16-byte slot when their pitch would be a
//    multiple of 128 bytes (every row on the same banks);
//  * LDS comes from the stack allocator in lds_alloc.h and is given back
//    by free_smem().
#pragma once

#include "gernels/lds_alloc.h"

namespace gernels {

template<int64_t H, int64_t W>
struct RegTile {
    static constexpr int64_t row = H;
    static constexpr int64_t col = W;
    float v[H * W];

    __device__ __forceinline__ float &operator()(int64_t i, int64_t j) {
        return v[i * W + j];
    }
    __device__ __forceinline__ float operator()(int64_t i, int64_t j) const {
        return v[i * W + j];
    }
    // A window of the tile, as a copy (registers cannot be pointed into; the
    // reference's get_view on register tiles, gernels/mm/impl/matrix-gpu.h:200-210).
    template<int64_t h, int64_t w>
    __device__ __forceinline__ RegTile<h, w> get_view(int64_t x, int64_t y) const {
        RegTile<h, w> t;
#pragma unroll
        for (int64_t i = 0; i < h; i++) {
#pragma unroll
            for (int64_t j = 0; j < w; j++) {
                t.v[i * w + j] = v[(x + i) * W + (y + j)];
            }
        }
        return t;
    }
    __device__ __forceinline__ void free_smem() const {
    }
};

template<int64_t H, int64_t W>
__device__ __forceinline__ RegTile<H, W> allocate_static() {
    RegTile<H, W> t;
#pragma unroll
    for (int64_t e = 0; e < H * W; e++) {
        t.v[e] = 0.0f;
    }
    return t;
}

// A per-thread tile of float4: H rows of W / 4 vectors (the reference's
// StaticMatrix<float4>, gernels/mm/impl/matrix-gpu.h:29-72).
template<int64_t H, int64_t W>
struct RegTile4 {
    static_assert(W % 4 == 0, "rows are whole float4");
    static constexpr int64_t rows = H;
    static constexpr int64_t cols_by_4 = W / 4;
    static constexpr int64_t row = H;
    static constexpr int64_t col = W;
    float4 array[H * (W / 4)];

    __device__ __forceinline__ void free_smem() const {
    }
};

template<int64_t H, int64_t W>
__device__ __forceinline__ RegTile4<H, W> allocate_static_vec() {
    RegTile4<H, W> t;
#pragma unroll
    for (int64_t e = 0; e < H * (W / 4); e++) {
        t.array[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    return t;
}

// Pitch (in floats) of an LDS tile with W columns: rows that are a multiple of 16 floats long are padded by
// four, so that rows 1, 2 or 4 apart (what the threads of a wavefront read when each holds a few rows of C)
// do not start in the same bank, and 16-byte accesses stay aligned.
constexpr int64_t lds_pitch(int64_t w) {
    return (w % 16 == 0) ? w + 4 : w;
}

// An H x W tile in LDS (or a window of one): `owner` is the allocation to give
// back, null for windows.
template<int64_t H, int64_t W, int64_t LDA>
struct LdsTile {
    static constexpr int64_t row = H;
    static constexpr int64_t col = W;
    static constexpr int64_t lda = LDA;
    float *data;
    float *owner;

    __device__ __forceinline__ float &operator()(int64_t i, int64_t j) {
        return data[i * LDA + j];
    }
    __device__ __forceinline__ float operator()(int64_t i, int64_t j) const {
        return data[i * LDA + j];
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, LDA> get_view(int64_t x, int64_t y) const {
        return LdsTile<h, w, LDA>{data + x * LDA + y, nullptr};
    }
    // The same window under the reference's other name (there: a window whose
    // users read float4; here a window has no access width of its own).
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, LDA> get_view_vec(int64_t x, int64_t y) const {
        return get_view<h, w>(x, y);
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ RegTile<h, w> query_2_reg_no_vector(int64_t x, int64_t y) const {
        RegTile<h, w> t;
#pragma unroll
        for (int64_t i = 0; i < h; i++) {
#pragma unroll
            for (int64_t j = 0; j < w; j++) {
                t(i, j) = data[(x + i) * LDA + (y + j)];
            }
        }
        return t;
    }
    // Collective.
    __device__ __forceinline__ void free_smem() const {
        if (owner != nullptr) {
            lds_free(owner);
        }
    }
};

namespace detail {

__device__ __forceinline__ int flat_thread() {
    return (int)(threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z));
}

__device__ __forceinline__ int flat_block_size() {
    return (int)(blockDim.x * blockDim.y * blockDim.z);
}

}  // namespace detail

// Row-major fp32 matrix in HBM with compile-time extents.  The object is a
// single pointer: that is what the host passes to the kernel.
template<int64_t Row, int64_t Col, int64_t LDA>
struct GlobalMatrix {
    static constexpr int64_t row = Row;
    static constexpr int64_t col = Col;
    static constexpr int64_t lda = LDA;
    float *data;

    __device__ __forceinline__ float &operator()(int64_t i, int64_t j) {
        return data[i * LDA + j];
    }
    __device__ __forceinline__ float operator()(int64_t i, int64_t j) const {
        return data[i * LDA + j];
    }

    // A window in place.
    template<int64_t h, int64_t w>
    __device__ __forceinline__ GlobalMatrix<h, w, LDA> query_global_2_global(int64_t x, int64_t y) const {
        return GlobalMatrix<h, w, LDA>{data + x * LDA + y};
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ void insert_global_2_global(int64_t, int64_t, const GlobalMatrix<h, w, LDA> &) const {
    }

    // A private copy in registers (per thread).
    template<int64_t h, int64_t w>
    __device__ __forceinline__ RegTile<h, w> query_2_reg_no_vector(int64_t x, int64_t y) const {
        RegTile<h, w> t;
#pragma unroll
        for (int64_t i = 0; i < h; i++) {
#pragma unroll
            for (int64_t j = 0; j < w; j++) {
                t(i, j) = data[(x + i) * LDA + (y + j)];
            }
        }
        return t;
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ void insert_2_reg_no_vector(int64_t x, int64_t y, const RegTile<h, w> &t) const {
#pragma unroll
        for (int64_t i = 0; i < h; i++) {
#pragma unroll
            for (int64_t j = 0; j < w; j++) {
                data[(x + i) * LDA + (y + j)] = t(i, j);
            }
        }
    }

    // A private copy in registers as float4 (per thread; 16-byte loads and
    // stores when the window allows, gernels/mm/impl/matrix-gpu.h:404-440).
    template<int64_t h, int64_t w>
    __device__ __forceinline__ RegTile4<h, w> query(int64_t x, int64_t y) const {
        RegTile4<h, w> t;
        const float *src = data + x * LDA + y;
        const bool vec = (LDA % 4 == 0) && ((((uint64_t)src) & 15u) == 0);
#pragma unroll
        for (int64_t i = 0; i < h; i++) {
#pragma unroll
            for (int64_t j = 0; j < w / 4; j++) {
                const float *p = src + i * LDA + 4 * j;
                t.array[i * (w / 4) + j] = vec ? *reinterpret_cast<const float4 *>(p) : make_float4(p[0], p[1], p[2], p[3]);
            }
        }
        return t;
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ void insert(int64_t x, int64_t y, const RegTile4<h, w> &t) const {
        float *dst = data + x * LDA + y;
        const bool vec = (LDA % 4 == 0) && ((((uint64_t)dst) & 15u) == 0);
#pragma unroll
        for (int64_t i = 0; i < h; i++) {
#pragma unroll
            for (int64_t j = 0; j < w / 4; j++) {
                float *p = dst + i * LDA + 4 * j;
                const float4 v = t.array[i * (w / 4) + j];
                if (vec) {
                    *reinterpret_cast<float4 *>(p) = v;
                } else {
                    p[0] = v.x;
                    p[1] = v.y;
                    p[2] = v.z;
                    p[3] = v.w;
                }
            }
        }
    }

    // Collective: the h x w tile at (x, y), copied into freshly allocated LDS,
    // one float per lane and step (consecutive lanes on consecutive floats).
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, lds_pitch(w)> stage_into_smem(int64_t x, int64_t y) const {
        constexpr int64_t P = lds_pitch(w);
        float *tile = static_cast<float *>(lds_alloc(h * P * (int64_t)sizeof(float)));
        const int tid = detail::flat_thread(), nt = detail::flat_block_size();
        const float *src = data + x * LDA + y;
        for (int64_t e = tid; e < h * w; e += nt) {
            const int64_t i = e / w, j = e % w;
            tile[i * P + j] = src[i * LDA + j];
        }
        __syncthreads();
        return LdsTile<h, w, P>{tile, tile};
    }
    // The same with 16 bytes per lane and step (through registers); tiles whose
    // rows are not whole, aligned float4 take the scalar copy.
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, lds_pitch(w)> stage_into_smem_vec(int64_t x, int64_t y) const {
        const float *src = data + x * LDA + y;
        if constexpr (w % 4 != 0 || LDA % 4 != 0) {
            return stage_into_smem<h, w>(x, y);
        } else {
            if ((((uint64_t)src) & 15u) != 0) {  // workgroup-uniform
                return stage_into_smem<h, w>(x, y);
            }
            constexpr int64_t P = lds_pitch(w);
            constexpr int64_t W4 = w / 4;
            float *tile = static_cast<float *>(lds_alloc(h * P * (int64_t)sizeof(float)));
            const int tid = detail::flat_thread(), nt = detail::flat_block_size();
            for (int64_t e = tid; e < h * W4; e += nt) {
                const int64_t i = e / W4, j = (e % W4) * 4;
                *reinterpret_cast<float4 *>(tile + i * P + j) = *reinterpret_cast<const float4 *>(src + i * LDA + j);
            }
            __syncthreads();
            return LdsTile<h, w, P>{tile, tile};
        }
    }
    // The same with loads that write LDS directly: a load instruction of a
    // wavefront fills 1 KiB of LDS in lane order (lane l the 16 bytes at
    // 16 l), so the tile is DENSE in LDS (pitch w, no padding) and lane l of
    // step s fetches flat elements 256 s' + 4 l .. + 3 of the tile, s'
    // numbering the 1 KiB pieces over all wavefronts.  Lanes past the end of
    // the tile are sent out of the buffer's range (they write zeros into the
    // slack that the allocation leaves behind the tile).  Tiles whose rows are
    // not whole float4 take the scalar copy into a dense tile.
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, w> stage_into_smem_flat(int64_t x, int64_t y) const {
        constexpr int64_t PIECES = (h * w + 255) / 256;  // 1 KiB each
        float *tile = static_cast<float *>(lds_alloc(PIECES * 1024));
        const float *src = data + x * LDA + y;
        const int tid = detail::flat_thread(), nt = detail::flat_block_size();
        if constexpr (w % 4 != 0) {
            for (int64_t e = tid; e < h * w; e += nt) {
                tile[e] = src[(e / w) * LDA + e % w];
            }
        } else {
            const int lane = tid % kWaveSize;
            const int wave = __builtin_amdgcn_readfirstlane(tid / kWaveSize), waves = (nt + kWaveSize - 1) / kWaveSize;
            constexpr int kRawBuffer = 0x00020000;
            constexpr int kOutOfRange = 0x7FFF0000;
            // the window, from its first element to the end of its last row
            const __amdgpu_buffer_rsrc_t desc =
                __builtin_amdgcn_make_buffer_rsrc((void *)src, 0, (int)(((h - 1) * LDA + w) * 4), kRawBuffer);
            for (int64_t piece = wave; piece < PIECES; piece += waves) {
                const int64_t e = piece * 256 + 4 * lane;
                const int off = e < h * w ? (int)(((e / w) * LDA + e % w) * 4) : kOutOfRange;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(desc, (__attribute__((address_space(3))) void *)(tile + piece * 256), 16, off,
                                                         0, 0, 0);
            }
            __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): this wavefront's pieces are in LDS
        }
        __syncthreads();
        return LdsTile<h, w, w>{tile, tile};
    }
    // Collective: writes an LDS tile back to (x, y).
    template<int64_t h, int64_t w, int64_t q_lda>
    __device__ __forceinline__ void insert_from_smem(int64_t x, int64_t y, const LdsTile<h, w, q_lda> &m) const {
        __syncthreads();
        const int tid = detail::flat_thread(), nt = detail::flat_block_size();
        float *dst = data + x * LDA + y;
        for (int64_t e = tid; e < h * w; e += nt) {
            const int64_t i = e / w, j = e % w;
            dst[i * LDA + j] = m.data[i * q_lda + j];
        }
    }
    __device__ __forceinline__ void free_smem() const {
    }
};

// C(i, j) += sum_k A(i, k) * B(k, j), term by term in k order, on any of the
// tile types above (gernels/mm/impl/matrix_multiply.h:63-76 of the reference).
// The thread's elements of C are read once, updated in registers and written once per call: added to in
// place, a C that lives in global memory would have to be stored after every term and the operands read
// again after every store, because the compiler cannot rule out that the operands (generic pointers into
// LDS) alias it.  (How much of that a compiler removes by itself differed between two versions of the
// same compiler by a factor of 1.5 on the kernel_3 schedule.)
template<int64_t k_dim, typename AT, typename BT, typename CT>
__device__ __forceinline__ void matrix_multiply(const AT &A, const BT &B, CT &C) {
    if constexpr (AT::row * BT::col <= 64) {
        float c[AT::row][BT::col];
#pragma unroll
        for (int64_t i = 0; i < AT::row; i++) {
#pragma unroll
            for (int64_t j = 0; j < BT::col; j++) {
                c[i][j] = C(i, j);
            }
        }
#pragma unroll
        for (int64_t i = 0; i < AT::row; i++) {
#pragma unroll
            for (int64_t j = 0; j < BT::col; j++) {
                for (int64_t k = 0; k < k_dim; k++) {
                    c[i][j] += A(i, k) * B(k, j);
                }
            }
        }
#pragma unroll
        for (int64_t i = 0; i < AT::row; i++) {
#pragma unroll
            for (int64_t j = 0; j < BT::col; j++) {
                C(i, j) = c[i][j];
            }
        }
    } else {
        for (int64_t i = 0; i < AT::row; i++) {
            for (int64_t j = 0; j < BT::col; j++) {
                float c = C(i, j);
                for (int64_t k = 0; k < k_dim; k++) {
                    c += A(i, k) * B(k, j);
                }
                C(i, j) = c;
            }
        }
    }
}

// The same product, term by term in the same k order per element of C, for operands that are tiles (or
// windows of tiles) in LDS and a tile of C in the thread's registers: four steps of k at a time, the thread
// reads its H rows of A (16 bytes each) and the four rows of B (W consecutive floats each, 16 bytes at a
// time) once and does 4 H W multiply-adds on them.  This is the overload a schedule reaches when it stages C
// into registers (Stage(C, query_2_reg_no_vector, ...)) around operands staged into LDS; windows that are
// not 16-byte aligned take the scalar loop.
template<int64_t k_dim, int64_t HA, int64_t WA, int64_t LA, int64_t HB, int64_t WB, int64_t LB, int64_t H, int64_t W>
__device__ __forceinline__ void matrix_multiply(const LdsTile<HA, WA, LA> &A, const LdsTile<HB, WB, LB> &B, RegTile<H, W> &C) {
    static_assert(HA == H && WB == W && WA >= k_dim && HB >= k_dim, "tile shapes of C = A B");
    constexpr bool vec = (k_dim % 4 == 0) && (W % 4 == 0) && (LA % 4 == 0) && (LB % 4 == 0);
    if (vec && ((((uint64_t)A.data) | ((uint64_t)B.data)) & 15u) == 0) {
        typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int64_t k = 0; k < (vec ? k_dim : 0); k += 4) {
            f4 a[H], b[4][W / 4 > 0 ? W / 4 : 1];
#pragma unroll
            for (int64_t i = 0; i < H; i++) {
                a[i] = *reinterpret_cast<const f4 *>(A.data + i * LA + k);
            }
#pragma unroll
            for (int64_t kk = 0; kk < 4; kk++) {
#pragma unroll
                for (int64_t j = 0; j < W / 4; j++) {
                    b[kk][j] = *reinterpret_cast<const f4 *>(B.data + (k + kk) * LB + 4 * j);
                }
            }
#pragma unroll
            for (int64_t kk = 0; kk < 4; kk++) {
#pragma unroll
                for (int64_t i = 0; i < H; i++) {
#pragma unroll
                    for (int64_t j = 0; j < W; j++) {
                        C(i, j) += a[i][kk] * b[kk][j / 4][j % 4];
                    }
                }
            }
        }
        return;
    }
    for (int64_t i = 0; i < H; i++) {
        for (int64_t j = 0; j < W; j++) {
            for (int64_t k = 0; k < k_dim; k++) {
                C(i, j) += A(i, k) * B(k, j);
            }
        }
    }
}

// The same product on float4 register tiles (RegTile4), four columns of C at
// a time (gernels/mm/impl/matrix_multiply.h:18-48 of the reference, including
// its order of additions: per group of four k, x y z w in turn, into a local
// sum that is added to C at the end).
template<int64_t k_dim, typename AT, typename BT, typename CT>
__device__ __forceinline__ void matrix_multiply_reg(const AT &A, const BT &B, CT &C) {
    const float *b_flat = reinterpret_cast<const float *>(B.array);
    constexpr int64_t B_cols = BT::cols_by_4 * 4;
#pragma unroll
    for (int64_t i = 0; i < CT::rows; i++) {
#pragma unroll
        for (int64_t j = 0; j < CT::cols_by_4; j++) {
            float tmp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int64_t k = 0; k < AT::cols_by_4; k++) {
                const float4 a = A.array[i * AT::cols_by_4 + k];
#pragma unroll
                for (int64_t l = 0; l < 4; l++) {
                    tmp[l] += a.x * b_flat[(4 * k + 0) * B_cols + 4 * j + l];
                    tmp[l] += a.y * b_flat[(4 * k + 1) * B_cols + 4 * j + l];
                    tmp[l] += a.z * b_flat[(4 * k + 2) * B_cols + 4 * j + l];
                    tmp[l] += a.w * b_flat[(4 * k + 3) * B_cols + 4 * j + l];
                }
            }
            float4 &c = C.array[i * CT::cols_by_4 + j];
            c.x += tmp[0];
            c.y += tmp[1];
            c.z += tmp[2];
            c.w += tmp[3];
        }
    }
}

}  // namespace gernels
