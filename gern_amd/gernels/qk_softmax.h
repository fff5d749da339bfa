// Fused S = softmax_rows(scale * Q K^T) for bf16 Q (M x D) and K (N x D).
//
// One workgroup of NW wavefronts owns 16 rows of S and ALL N <= 4096 columns,
// held as MFMA accumulators: wavefront w owns columns [w*N/NW, (w+1)*N/NW), as
// groups of 64 columns, each group four v_mfma_f32_16x16x32_bf16 tiles.
// Inside a group, tile t / lane column j stands for key 4*j + t, so that the
// four tiles of a group give every lane FOUR CONSECUTIVE columns of S and a row
// of the block is stored with 16-byte stores, 256 contiguous bytes per sixteen
// lanes.  The logits never leave registers: row maximum and row sum are reduced
// inside the 16-lane DPP rows that share an S row, then across the wavefronts
// through a few hundred bytes of LDS (one barrier per reduction).  S is
// written once, with streaming stores; Q and K (1 MiB each, L2-resident) are
// the only reads.
//
// NW grows with N (8 wavefronts from 2048 keys on): S has only M/16 row
// blocks, so the columns of a block are spread over several wavefronts for the
// chip to be busy; 128 accumulators per lane leave room for two wavefronts per
// SIMD (16 wavefronts with 64 accumulators each measured slower: the
// compiler spills at 128 registers).
//
// The reference has nothing like this (no bf16, no matrix-core path, no fused
// GEMM -> softmax); the softmax stages reuse the names and argument order of
// its softmax gernels (apps/common/impl/impl.h:7-188) so that the same
// annotations compose them.
#pragma once

#include "gernels/mm.h"
#include "gernels/softmax.h"

namespace gernels {

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Wavefronts per workgroup for a row block of N columns; the host sizes the
// launch with the same rule (threads = 64 * qk_waves(N)).
#ifndef GERN_QK_WAVES
constexpr int qk_waves(int64_t n) {
    return (n >= 2048 && n % 512 == 0) ? 8 : 4;
}
#else
constexpr int qk_waves(int64_t) {
    return GERN_QK_WAVES;
}
#endif

// 16 x N logits / probabilities, distributed over the workgroup as described
// above: acc[g][t][i] is row 4*(lane/16) + i, column
// wave*(N/NW) + 64*g + 4*(lane%16) + t.
template<int64_t R, int64_t N>
struct RowBlock {
    static_assert(R == 16, "a row block is one MFMA tile high");
    static constexpr int NW = qk_waves(N);
    static_assert(N % (64 * NW) == 0 && N <= 4096, "wavefronts x 64-column groups, at most 4096 columns");
    static constexpr int64_t rows = R;
    static constexpr int64_t cols = N;
    static constexpr int64_t wave_cols = N / NW;
    static constexpr int G = (int)(N / (64 * NW));
    f32x4_t acc[G][4];

    __device__ __forceinline__ void destroy() {
    }
};

// Per-row scalars of a row block: lane l keeps rows 4*(l/16) .. +3.
template<int64_t R>
struct RowStat {
    static constexpr int64_t size = R;
    float v[4];

    __device__ __forceinline__ void destroy() {
    }
};

template<int64_t R, int64_t N>
__device__ __forceinline__ RowBlock<R, N> allocate_row_block() {
    return RowBlock<R, N>();
}

template<int64_t R>
__device__ __forceinline__ RowStat<R> allocate_row_stat() {
    return RowStat<R>();
}

// The output window of a row block (nothing is read).
template<int64_t R, int64_t N>
__device__ __forceinline__ RowBlock<R, N> MatrixF32::view_row_block(int64_t, int64_t) const {
    return RowBlock<R, N>();
}

template<int64_t R, int64_t N>
__device__ __forceinline__ void MatrixF32::store_row_block(int64_t x, int64_t y, const RowBlock<R, N> &t) const {
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
    const int64_t c0 = y + (int64_t)w * RowBlock<R, N>::wave_cols + 4 * (lane % 16);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int64_t rr = x + 4 * (lane / 16) + i;
        if (rr >= row) {
            continue;
        }
        float *p = data + rr * lda;
        const bool vec_ok = ((((uint64_t)(p + y)) & 15u) == 0);
#pragma unroll
        for (int g = 0; g < RowBlock<R, N>::G; g++) {
            const int64_t cc = c0 + 64 * g;
            const float4 val = make_float4(t.acc[g][0][i], t.acc[g][1][i], t.acc[g][2][i], t.acc[g][3][i]);
            if (vec_ok && cc + 3 < col) {
                store_result16<kThroughStores>(data, (row - 1) * lda + col, rr * lda + cc, val);
            } else {
                if (cc + 0 < col) p[cc + 0] = val.x;
                if (cc + 1 < col) p[cc + 1] = val.y;
                if (cc + 2 < col) p[cc + 2] = val.z;
                if (cc + 3 < col) p[cc + 3] = val.w;
            }
        }
    }
}

namespace detail {

// Q K^T of one wavefront's columns with K streamed through LDS, for head
// dimensions whose rows fill whole load instructions (D = 32, 64, 128, 256).
//
// A tile is the 16 keys of one MFMA (keys 4 j + t of a 64-key group, see
// RowBlock) x D: 32 D bytes.  It is fetched with loads that write straight
// into LDS (16 bytes per lane, lanes in LDS order): sixteen-byte piece `slot`
// of key j lands at j * 2 D + slot * 16, and holds piece slot ^ swz(j) of the
// key, so that the sixteen lanes of one LDS read pass (sixteen keys, the same
// piece) fall into sixteen different 16-byte bank groups.  Consecutive lanes
// read consecutive bytes of one key: whole cache lines per lane group, and no
// cross-lane shuffle afterwards (loading in the MFMA's own lane order costs
// four ds_bpermute per load).  Each wavefront owns its keys, so the pipeline
// is private to the wavefront (P tiles in flight, no workgroup barrier); the
// P slots are separate arrays for the compiler to order loads and reads per
// slot instead of waiting for every outstanding load.
template<int64_t R, int64_t N, int64_t D>
__device__ __forceinline__ void qk_through_lds(const bf16x8_t (&q)[D / 32], const GlobalView<N, D, uint16_t, false> &K,
                                               RowBlock<R, N> &S, float to_log2) {
    using Block = RowBlock<R, N>;
    constexpr int NW = Block::NW;
    constexpr int KS = (int)(D / 32);
    constexpr int PR = (int)(D / 8);            // 16-byte pieces per key
    constexpr int TILE = 32 * (int)D;           // bytes of a tile
    constexpr int LOADS = TILE / 1024;          // load instructions per tile
    constexpr int KEYS_PER_LOAD = 16 / LOADS;
    constexpr int P = TILE >= 8192 ? 2 : 4;     // tiles in flight (at most 16 KiB per wavefront)
    constexpr int TILES = Block::G * 4;
    static_assert(TILE % 1024 == 0 && 64 % PR == 0 || PR == 32, "rows fill whole load instructions");
    __shared__ __attribute__((aligned(16))) unsigned char k_slot0[NW * TILE];
    __shared__ __attribute__((aligned(16))) unsigned char k_slot1[NW * TILE];
    __shared__ __attribute__((aligned(16))) unsigned char k_slot2[P == 4 ? NW * TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char k_slot3[P == 4 ? NW * TILE : 16];

    const int lane = lane_id();
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWaveSize));
    // swz(j): what the piece index of key j is XORed with
    auto swz = [](int j) { return PR >= 16 ? j % 16 : (j / (16 / PR)) % PR; };
    const int last_key = (int)K.rows - 1;
    const int row_bytes = (int)K.lda * 2;
    constexpr int kRawBuffer = 0x00020000;
    // no key at all: a descriptor of zero bytes makes every load return zeros without touching memory
    const __amdgpu_buffer_rsrc_t desc = __builtin_amdgcn_make_buffer_rsrc((void *)K.data, 0, last_key >= 0 ? -1 : 0, kRawBuffer);
    const int wave_key0 = w * (int)Block::wave_cols;

    auto slot_of = [&](int tile) -> unsigned char * {
        switch (tile % P) {
        case 0: return k_slot0;
        case 1: return k_slot1;
        case 2: return k_slot2;
        default: return k_slot3;
        }
    };
    auto issue = [&](int tile) {
        const int g = tile / 4, t = tile % 4;
        unsigned char *dst = slot_of(tile);
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
            const int j = i * KEYS_PER_LOAD + lane / PR;
            const int piece = (lane % PR) ^ swz(j);
            int key = wave_key0 + 64 * g + 4 * j + t;
            key = key < last_key ? key : last_key;  // keys past the end are masked below; read a valid one
            __builtin_amdgcn_raw_ptr_buffer_load_lds(desc, (__attribute__((address_space(3))) void *)(dst + (w * TILE + i * 1024)),
                                                     16, key * row_bytes + piece * 16, 0, 0, 0);
        }
    };
    const int j_mine = lane % 16;
    const int frag_base = w * TILE + j_mine * 2 * (int)D;
#pragma unroll
    for (int tile = 0; tile < P - 1 && tile < TILES; tile++) {
        issue(tile);
    }
#pragma unroll
    for (int tile = 0; tile < TILES; tile++) {
        if (tile + P - 1 < TILES) {
            issue(tile + P - 1);
        }
        const unsigned char *src = slot_of(tile);
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const int slot = (4 * s + lane / 16) ^ swz(j_mine);
            const bf16x8_t k = *reinterpret_cast<const bf16x8_t *>(src + (frag_base + slot * 16));
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(q[s], k, acc, 0, 0, 0);
        }
        S.acc[tile / 4][tile % 4] = acc * to_log2;
    }
}

}  // namespace detail

// S = log2(e) * scale * Q K^T for the 16 rows of Q in view (log2 units, see
// exp_matrix below); columns past the last key get -inf so that they vanish
// from the softmax.
template<int64_t R, int64_t N, int64_t D>
__device__ __forceinline__ void qk_scaled(const GlobalView<R, D, uint16_t, false> &Q, const GlobalView<N, D, uint16_t, false> &K,
                                          RowBlock<R, N> &S, float scale) {
    static_assert(D % 32 == 0 && D <= 256, "head dimension in MFMA K steps of 32");
    constexpr int KS = (int)(D / 32);
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
    const int k_off = 8 * (lane / 16);

    bf16x8_t q[KS];
    {
        const int64_t r = lane % 16;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (r < Q.rows) {
                v = *reinterpret_cast<const uint4 *>(Q.data + r * Q.lda + s * 32 + k_off);
            }
            q[s] = __builtin_bit_cast(bf16x8_t, v);
        }
    }
    // The logits are kept in log2 units (scale * log2(e) folded into one
    // multiply), so that the exp stage is a bare v_exp_f32.
    const float to_log2 = scale * 1.4426950408889634f;
    if constexpr (D == 32 || D == 64 || D == 128 || D == 256) {
        detail::qk_through_lds<R, N, D>(q, K, S, to_log2);
    } else {
    // Other head dimensions: K goes through registers.
    // K is read with lanes 4j .. 4j+3 on the four 16-byte pieces of ONE key's
    // 64 bytes (sixteen keys per load), so that each group of four lanes
    // touches a single cache line: the vector cache looks up one line per
    // cycle, and the layout the MFMA wants (lane l: key l%16, piece l/16) would
    // make every lane of a quad hit a different line, a quarter of the rate.
    // The pieces then move to the lanes that feed the MFMA with ds_bpermute
    // (lane l takes from lane 4*(l%16) + l/16), which costs no LDS space.
    const int take_from = 4 * (4 * (lane % 16) + lane / 16);
#pragma unroll
    for (int g = 0; g < RowBlock<R, N>::G; g++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int64_t load_key = (int64_t)w * RowBlock<R, N>::wave_cols + 64 * g + 4 * (lane / 4) + t;
            const bool ok = load_key < K.rows;
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                uint4 v = make_uint4(0u, 0u, 0u, 0u);
                if (ok) {
                    v = *reinterpret_cast<const uint4 *>(K.data + load_key * K.lda + s * 32 + 8 * (lane % 4));
                }
                v.x = (uint32_t)__builtin_amdgcn_ds_bpermute(take_from, (int)v.x);
                v.y = (uint32_t)__builtin_amdgcn_ds_bpermute(take_from, (int)v.y);
                v.z = (uint32_t)__builtin_amdgcn_ds_bpermute(take_from, (int)v.z);
                v.w = (uint32_t)__builtin_amdgcn_ds_bpermute(take_from, (int)v.w);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(q[s], __builtin_bit_cast(bf16x8_t, v), acc, 0, 0, 0);
            }
            S.acc[g][t] = acc * to_log2;
        }
    }
    }
    // The column a lane holds in tile t is its own key, so validity is a
    // per-lane, per-tile property.
#pragma unroll
    for (int g = 0; g < RowBlock<R, N>::G; g++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int64_t key = (int64_t)w * RowBlock<R, N>::wave_cols + 64 * g + 4 * (lane % 16) + t;
            if (key >= K.rows) {
                S.acc[g][t] = f32x4_t{-__builtin_huge_valf(), -__builtin_huge_valf(), -__builtin_huge_valf(),
                                      -__builtin_huge_valf()};
            }
        }
    }
}

namespace detail {

// Reduces the four row values of a lane over the 16 lanes of a DPP row (the
// lanes that share S rows), then over the NW wavefronts through `lds`
// (16 rows x NW floats; the two reductions of a softmax use different buffers,
// so one barrier each is enough).
template<typename Op, int NW>
__device__ __forceinline__ void row_block_reduce(float (&x)[4], float *lds) {
    const int lane = lane_id();
    const int w = (int)(threadIdx.x / kWaveSize);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float v = x[i];
        v = Op::apply(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
        v = Op::apply(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
        v = Op::apply(v, dpp_move<0x141>(v));  // row_half_mirror
        v = Op::apply(v, dpp_move<0x140>(v));  // row_mirror
        x[i] = v;
    }
    if (lane % 16 == 0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lds[(4 * (lane / 16) + i) * NW + w] = x[i];
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const f32x4_t *row = reinterpret_cast<const f32x4_t *>(lds + (4 * (lane / 16) + i) * NW);
        float r = Op::identity();
#pragma unroll
        for (int q = 0; q < NW / 4; q++) {
            const f32x4_t part = row[q];
            r = Op::apply(Op::apply(r, part[0]), Op::apply(part[1], Op::apply(part[2], part[3])));
        }
        x[i] = r;
    }
}

template<typename Op, int64_t R, int64_t N>
__device__ __forceinline__ void reduce_row_block(RowStat<R> &out, const RowBlock<R, N> &in, float *lds) {
    float acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        acc[i] = Op::identity();
#pragma unroll
        for (int g = 0; g < RowBlock<R, N>::G; g++) {
#pragma unroll
            for (int t = 0; t < 4; t++) {
                acc[i] = Op::apply(acc[i], in.acc[g][t][i]);
            }
        }
    }
    row_block_reduce<Op, RowBlock<R, N>::NW>(acc, lds);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        out.v[i] = acc[i];
    }
}

}  // namespace detail

template<int64_t stride = 64, int64_t R, int64_t N>
__device__ __forceinline__ void max_row(RowStat<R> &out, const RowBlock<R, N> &in) {
    __shared__ __attribute__((aligned(16))) float max_scratch[16 * RowBlock<R, N>::NW];
    detail::reduce_row_block<MaxOp>(out, in, max_scratch);
}

template<int64_t stride = 64, int64_t R, int64_t N>
__device__ __forceinline__ void sum_row(RowStat<R> &out, const RowBlock<R, N> &in) {
    __shared__ __attribute__((aligned(16))) float sum_scratch[16 * RowBlock<R, N>::NW];
    detail::reduce_row_block<SumOp>(out, in, sum_scratch);
}

template<int64_t R, int64_t N>
__device__ __forceinline__ void subtract_vec(const RowStat<R> &vec, const RowBlock<R, N> &in, RowBlock<R, N> &out) {
#pragma unroll
    for (int g = 0; g < RowBlock<R, N>::G; g++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                out.acc[g][t][i] = in.acc[g][t][i] - vec.v[i];
            }
        }
    }
}

// A row block holds logits in log2 units, so exp is 2^x: one v_exp_f32 per
// element.  Its arguments are <= 0 here (a row maximum has been subtracted);
// results below 2^-126 come out as 0, i.e. probabilities that fp32 could only
// hold as denormals are flushed to zero.
template<int64_t R, int64_t N>
__device__ __forceinline__ void exp_matrix(const RowBlock<R, N> &in, RowBlock<R, N> &out) {
#pragma unroll
    for (int g = 0; g < RowBlock<R, N>::G; g++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const f32x4_t a = in.acc[g][t];
            out.acc[g][t] = f32x4_t{__builtin_amdgcn_exp2f(a[0]), __builtin_amdgcn_exp2f(a[1]),
                                    __builtin_amdgcn_exp2f(a[2]), __builtin_amdgcn_exp2f(a[3])};
        }
    }
}

template<int64_t R, int64_t N>
__device__ __forceinline__ void divide_vec(const RowStat<R> &vec, const RowBlock<R, N> &in, RowBlock<R, N> &out) {
    float rcp[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        rcp[i] = 1.0f / vec.v[i];
    }
#pragma unroll
    for (int g = 0; g < RowBlock<R, N>::G; g++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                out.acc[g][t][i] = in.acc[g][t][i] * rcp[i];
            }
        }
    }
}

}  // namespace gernels
