// Matrices for USER-WRITTEN schedules: a global matrix whose tiles can be
// viewed in place, copied into registers, or staged into LDS by the whole
// workgroup, and the scalar matrix_multiply that works on any of them.
//
// This is the gfx950 counterpart of the reference's gernels/mm/impl/
// matrix-gpu.h:182-508 and matrix_multiply.h:18-76, with the same method names
// (the reference's annotations name them in generated code), except that
// "smem" stays in the names only for that compatibility.  What differs:
//  * staging is one flat, fully coalesced sweep of the tile by ALL threads of
//    the workgroup, 16 bytes per lane where the tile allows, whatever the
//    block shape (the reference indexes by threadIdx.x / .y and silently
//    assumes the block shape matches the tile);
//  * LDS rows are padded by one 16-byte slot when their pitch would be a
//    multiple of 128 bytes (every row on the same banks);
//  * LDS comes from the free-list allocator in lds_alloc.h and is given back
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

// Pitch (in floats) of an LDS tile with W columns.
constexpr int64_t lds_pitch(int64_t w) {
    return (w % 32 == 0) ? w + 4 : w;
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

    // Collective: the h x w tile at (x, y), copied into freshly allocated LDS.
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, lds_pitch(w)> stage_into_smem(int64_t x, int64_t y) const {
        constexpr int64_t P = lds_pitch(w);
        float *tile = static_cast<float *>(lds_alloc(h * P * (int64_t)sizeof(float)));
        const int tid = detail::flat_thread(), nt = detail::flat_block_size();
        const float *src = data + x * LDA + y;
        const bool vec = (w % 4 == 0) && (LDA % 4 == 0) && ((((uint64_t)src) & 15u) == 0);
        if (vec) {
            constexpr int64_t W4 = w / 4 > 0 ? w / 4 : 1;
            for (int64_t e = tid; e < h * W4; e += nt) {
                const int64_t i = e / W4, j = (e % W4) * 4;
                *reinterpret_cast<float4 *>(tile + i * P + j) = *reinterpret_cast<const float4 *>(src + i * LDA + j);
            }
        } else {
            for (int64_t e = tid; e < h * w; e += nt) {
                const int64_t i = e / w, j = e % w;
                tile[i * P + j] = src[i * LDA + j];
            }
        }
        __syncthreads();
        return LdsTile<h, w, P>{tile, tile};
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, lds_pitch(w)> stage_into_smem_vec(int64_t x, int64_t y) const {
        return stage_into_smem<h, w>(x, y);
    }
    template<int64_t h, int64_t w>
    __device__ __forceinline__ LdsTile<h, w, lds_pitch(w)> stage_into_smem_flat(int64_t x, int64_t y) const {
        return stage_into_smem<h, w>(x, y);
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
template<int64_t k_dim, typename AT, typename BT, typename CT>
__device__ __forceinline__ void matrix_multiply(const AT &A, const BT &B, CT &C) {
    for (int64_t i = 0; i < AT::row; i++) {
        for (int64_t j = 0; j < BT::col; j++) {
            for (int64_t k = 0; k < k_dim; k++) {
                C(i, j) += A(i, k) * B(k, j);
            }
        }
    }
}

}  // namespace gernels
