// Ahead-of-time instantiation of every gernel for gfx950: the build check.
// The kernels that run are instantiated by hiprtc from generated code; this
// file only proves that the library compiles with hipcc as well.
#include "gernels/blur.h"
#include "gernels/softmax.h"

template<int64_t col, int64_t row, int64_t stride>
__global__ void __launch_bounds__(64) check_blur_xyx(gernels::MatrixF32 input, gernels::MatrixF32 output) {
    const int64_t y = blockIdx.x * col;
    const int64_t x = blockIdx.y * row;
    auto out_tile = output.template view_wave<row, col>(x, y);
    auto t2 = gernels::allocate_wave_tile<row, col + stride - 1>();
    auto t1 = gernels::allocate_wave_tile<row + stride - 1, col + stride - 1>();
    auto in_tile = input.template load_wave<row + stride - 1, col + 2 * (stride - 1)>(x, y);
    gernels::blur_x<stride>(in_tile, t1);
    gernels::blur_y<stride>(t1, t2);
    gernels::blur_x<stride>(t2, out_tile);
    output.store_wave(x, y, out_tile);
}
template __global__ void check_blur_xyx<252, 8, 3>(gernels::MatrixF32, gernels::MatrixF32);
template __global__ void check_blur_xyx<248, 4, 5>(gernels::MatrixF32, gernels::MatrixF32);

template<int64_t ncol, int64_t row>
__global__ void __launch_bounds__(64) check_softmax(gernels::MatrixF32 input, gernels::MatrixF32 output) {
    const int64_t x = blockIdx.x * row;
    auto in_tile = input.template load_wave<row, ncol>(x, 0);
    auto vec = gernels::allocate_wave_vec<row>();
    gernels::max_row(vec, in_tile);
    auto t = gernels::allocate_wave_tile<row, ncol>();
    gernels::subtract_vec(vec, in_tile, t);
    auto e = gernels::allocate_wave_tile<row, ncol>();
    gernels::exp_matrix(t, e);
    gernels::sum_row(vec, e);
    auto out_tile = output.template view_wave<row, ncol>(x, 0);
    gernels::divide_vec(vec, e, out_tile);
    output.store_wave(x, 0, out_tile);
}
template __global__ void check_softmax<4096, 1>(gernels::MatrixF32, gernels::MatrixF32);
template __global__ void check_softmax<1000, 2>(gernels::MatrixF32, gernels::MatrixF32);

#include "gernels/mm.h"

template<int64_t BM, int64_t BN, int64_t KC>
__global__ void __launch_bounds__(256) check_gemm_bf16(gernels::MatrixBF16 A, gernels::MatrixBF16 B, gernels::MatrixF32 C) {
    const int64_t i = blockIdx.y * BM, j = blockIdx.x * BN;
    auto acc = C.template load_acc_mfma<BM, BN>(i, j);
    for (int64_t k = 0; k < A.col; k += KC) {
        auto a = A.template view<BM, KC>(i, k);
        auto b = B.template view<KC, BN>(k, j);
        gernels::matrix_multiply(a, b, acc);
    }
    C.add_acc(i, j, acc);
}
template __global__ void check_gemm_bf16<256, 256, 4096>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32);
template __global__ void check_gemm_bf16<128, 128, 4096>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32);

template<int64_t BM, int64_t BN, int64_t KC>
__global__ void __launch_bounds__(512) check_gemm_bf16_8waves(gernels::MatrixBF16 A, gernels::MatrixBF16 B, gernels::MatrixF32 C) {
    const int64_t i = blockIdx.y * BM, j = blockIdx.x * BN;
    auto acc = C.template load_acc_mfma8<BM, BN>(i, j);
    for (int64_t k = 0; k < A.col; k += KC) {
        auto a = A.template view_exact<BM, KC>(i, k);
        auto b = B.template view_exact<KC, BN>(k, j);
        gernels::matrix_multiply(a, b, acc);
    }
    C.store_acc(i, j, acc);
}
template __global__ void check_gemm_bf16_8waves<256, 256, 4096>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32);

template<int64_t BM, int64_t BN, int64_t KC, bool ADD>
__global__ void __launch_bounds__(512) check_gemm_bf16_16x16x32(gernels::MatrixBF16 A, gernels::MatrixBF16 B, gernels::MatrixF32 C) {
    const int64_t i = blockIdx.y * BM, j = blockIdx.x * BN;
    auto acc = C.template load_acc_mfma16<BM, BN>(i, j);
    for (int64_t k = 0; k < A.col; k += KC) {
        auto a = A.template view_exact<BM, KC>(i, k);
        auto b = B.template view_exact<KC, BN>(k, j);
        gernels::matrix_multiply(a, b, acc);
    }
    if (ADD) {
        C.add_acc(i, j, acc);
    } else {
        C.store_acc(i, j, acc);
    }
}
template __global__ void check_gemm_bf16_16x16x32<256, 256, 4096, false>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32);
template __global__ void check_gemm_bf16_16x16x32<256, 256, 4096, true>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32);

template<int64_t BM, int64_t BN, int64_t KC>
__global__ void __launch_bounds__(256) check_gemm_f32(gernels::MatrixF32 A, gernels::MatrixF32 B, gernels::MatrixF32 C) {
    const int64_t i = blockIdx.y * BM, j = blockIdx.x * BN;
    auto acc = C.template load_acc_fma<BM, BN>(i, j);
    for (int64_t k = 0; k < A.col; k += KC) {
        auto a = A.template view<BM, KC>(i, k);
        auto b = B.template view<KC, BN>(k, j);
        gernels::matrix_multiply(a, b, acc);
    }
    C.store_acc(i, j, acc);
}
template __global__ void check_gemm_f32<128, 128, 4096>(gernels::MatrixF32, gernels::MatrixF32, gernels::MatrixF32);

template<int64_t BM, int64_t BN, int64_t KC>
__global__ void __launch_bounds__(512) check_gemm_f32_mfma(gernels::MatrixF32 A, gernels::MatrixF32 B, gernels::MatrixF32 C) {
    const int64_t i = blockIdx.y * BM, j = blockIdx.x * BN;
    auto acc = C.template load_acc_mfma8_f32<BM, BN>(i, j);
    for (int64_t k = 0; k < A.col; k += KC) {
        auto a = A.template view_exact<BM, KC>(i, k);
        auto b = B.template view_exact<KC, BN>(k, j);
        gernels::matrix_multiply(a, b, acc);
    }
    C.add_acc(i, j, acc);
}
template __global__ void check_gemm_f32_mfma<256, 256, 4096>(gernels::MatrixF32, gernels::MatrixF32, gernels::MatrixF32);

#include "gernels/qk_softmax.h"

template<int64_t N, int64_t D>
__global__ void __launch_bounds__(64 * gernels::qk_waves(N)) check_qk_softmax(gernels::MatrixBF16 Q, gernels::MatrixBF16 K, gernels::MatrixF32 S,
                                                        float scale) {
    const int64_t x = blockIdx.x * 16;
    auto q = Q.template view<16, D>(x, 0);
    auto k = K.template view<N, D>(0, 0);
    auto logits = gernels::allocate_row_block<16, N>();
    gernels::qk_scaled(q, k, logits, scale);
    auto stat = gernels::allocate_row_stat<16>();
    gernels::max_row(stat, logits);
    auto shifted = gernels::allocate_row_block<16, N>();
    gernels::subtract_vec(stat, logits, shifted);
    auto expd = gernels::allocate_row_block<16, N>();
    gernels::exp_matrix(shifted, expd);
    gernels::sum_row(stat, expd);
    auto out = S.template view_row_block<16, N>(x, 0);
    gernels::divide_vec(stat, expd, out);
    S.store_row_block(x, 0, out);
}
template __global__ void check_qk_softmax<4096, 128>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32, float);
template __global__ void check_qk_softmax<1024, 64>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32, float);

#include "gernels/qk_tiles.h"

// The tile program of the fused QK^T softmax: one workgroup per 256 x 256 tile of S.
template<int64_t D>
__global__ void __launch_bounds__(512) check_qk_softmax_tiles(gernels::MatrixBF16 Q, gernels::MatrixBF16 K, gernels::MatrixF32 S,
                                                             gernels::RowStatsExchange exchange, float scale) {
    const int64_t x = (int64_t)blockIdx.y * 256, y = (int64_t)blockIdx.x * 256;
    auto session = exchange.open();
    auto out = S.template view_score_tile<256, 256>(x, y);
    auto logits = gernels::allocate_score_tile<256, 256>();
    auto q = Q.template view<256, D>(x, 0);
    auto k = K.template view<256, D>(y, 0);
    gernels::qk_scaled(q, k, logits, scale);
    gernels::softmax_rows_across_tiles(logits, session, out);
    S.store_score_tile(x, y, out);
}
template __global__ void check_qk_softmax_tiles<128>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32, gernels::RowStatsExchange, float);
template __global__ void check_qk_softmax_tiles<192>(gernels::MatrixBF16, gernels::MatrixBF16, gernels::MatrixF32, gernels::RowStatsExchange, float);
