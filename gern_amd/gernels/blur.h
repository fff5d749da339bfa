// Separable box-blur stages on wave-distributed register tiles.
//
// Arithmetic follows the reference gernels (apps/common/impl/impl.h:190-214
// blur_x, :216-250 blur_y): a running fp32 sum that starts at 0, taps added
// left to right (top to bottom), then a division by the tap count.  The sum
// is formed without its leading +0 and divided by quotient_of_sum<>
// (gernels/prelude.h), which accounts for it.  For three taps that is two FMAs,
// identical to the IEEE quotient except for sums in [2^-126, 2^-122); a stage
// first rules such sums out for its whole tile and otherwise divides with the
// slower form that is exact everywhere, so the results match the reference's bit for bit for every input.
//
// blur_x needs, for the float4 a lane owns, the first (stride - 1) values of
// the lane to its right; they arrive by DPP wave shifts, so a fused chain of
// stages never touches LDS or memory between its first load and last store.
// The rightmost (stride - 1) columns of a blur_x result therefore hold
// garbage in lane 63; they lie outside the logical width of the output tile
// (in.cols >= out.cols + stride - 1) and are never stored.
#pragma once

#include "gernels/wave_tile.h"

namespace gernels {

namespace detail {

// The two-FMA quotient of three taps (quotient_of_sum<3>) is the IEEE quotient
// unless the tap sum lies in [2^-126, 2^-122).  A sum of values that are all
// at least 2^-60 in magnitude is either zero or a multiple of 2^-83, so a tile
// whose values pass this test cannot produce such a sum.  The test is one
// v_min3 per two values and one wave-wide vote per stage; tiles that fail it
// (values that small, or zeros, e.g. the zero fill past the edge of the image)
// take the four-instruction division that is exact everywhere.  NaNs do not
// take part (min ignores them).
template<typename TI>
__device__ __forceinline__ bool no_tiny_values(const TI &in) {
    float m = __builtin_huge_valf();
#pragma unroll
    for (int64_t r = 0; r < TI::rows; r++) {
#pragma unroll
        for (int64_t k = 0; k < TI::chunks; k++) {
            const float4 t = in.v[r][k];
            m = __builtin_fminf(m, __builtin_fminf(__builtin_fabsf(t.x), __builtin_fabsf(t.y)));
            m = __builtin_fminf(m, __builtin_fminf(__builtin_fabsf(t.z), __builtin_fabsf(t.w)));
        }
    }
    return __builtin_amdgcn_ballot_w64(m < 0x1p-60f) == 0;
}

// (0 + sum) / D for a sum formed without its leading zero.  FAST: the caller
// has ruled tiny sums out (or D needs no such care); otherwise the
// four-instruction form that is exact for every operand (gernels/prelude.h).
template<int64_t D, bool FAST>
__device__ __forceinline__ float blur_quotient(float sum) {
    if constexpr (FAST || D != 3) {
        return quotient_of_sum<D>(sum);
    } else {
        return div_by(0.0f + sum, 3.0f, 1.0f / 3.0f);
    }
}

template<int64_t stride, bool FAST, typename TI, typename TO>
__device__ __forceinline__ void blur_x_rows(const TI &in, TO &out) {
#pragma unroll
    for (int64_t r = 0; r < TO::rows; r++) {
        const float4 a = in.v[r][0];
        float w[8] = {a.x, a.y, a.z, a.w, 0.f, 0.f, 0.f, 0.f};
        if constexpr (stride > 1) w[4] = from_next_lane(a.x);
        if constexpr (stride > 2) w[5] = from_next_lane(a.y);
        if constexpr (stride > 3) w[6] = from_next_lane(a.z);
        if constexpr (stride > 4) w[7] = from_next_lane(a.w);
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float sum = w[e];
#pragma unroll
            for (int s = 1; s < stride; s++) {
                sum += w[e + s];
            }
            o[e] = blur_quotient<stride, FAST>(sum);
        }
        out.v[r][0] = make_float4(o[0], o[1], o[2], o[3]);
    }
}

template<int64_t stride, bool FAST, typename TI, typename TO>
__device__ __forceinline__ void blur_y_rows(const TI &in, TO &out) {
#pragma unroll
    for (int64_t r = 0; r < TO::rows; r++) {
#pragma unroll
        for (int64_t k = 0; k < TO::chunks; k++) {
            float4 sum = in.v[r][k];
#pragma unroll
            for (int64_t s = 1; s < stride; s++) {
                const float4 t = in.v[r + s][k];
                sum.x += t.x;
                sum.y += t.y;
                sum.z += t.z;
                sum.w += t.w;
            }
            out.v[r][k] = make_float4(blur_quotient<stride, FAST>(sum.x), blur_quotient<stride, FAST>(sum.y),
                                      blur_quotient<stride, FAST>(sum.z), blur_quotient<stride, FAST>(sum.w));
        }
    }
}

}  // namespace detail

// The choice between the two forms of the division is made once per stage
// and tile (a wave-uniform branch): chosen per row of outputs instead, the
// many short branches cost more than the test saves (85.7 us against 83.7 at
// the benchmark shape; with no test at all, and a sliver of inexact results,
// 81.1).
template<int64_t stride, typename TI, typename TO>
__device__ __forceinline__ void blur_x(const TI &in, TO &out) {
    static_assert(TI::chunks == 1 && TO::chunks == 1, "blur_x works on tiles at most 256 columns wide");
    static_assert(stride >= 1 && stride <= 5, "the right-hand halo must fit in the neighbouring lane");
    static_assert(TI::cols >= TO::cols + stride - 1, "input tile narrower than output + halo");
    static_assert(TI::rows >= TO::rows, "input tile shorter than output");
    if constexpr (stride == 3) {
        if (detail::no_tiny_values(in)) {
            detail::blur_x_rows<stride, true>(in, out);
        } else {
            detail::blur_x_rows<stride, false>(in, out);
        }
    } else {
        detail::blur_x_rows<stride, true>(in, out);
    }
}

template<int64_t stride, typename TI, typename TO>
__device__ __forceinline__ void blur_y(const TI &in, TO &out) {
    static_assert(TI::chunks == TO::chunks, "blur_y keeps the column layout");
    static_assert(TI::rows >= TO::rows + stride - 1, "input tile shorter than output + halo");
    if constexpr (stride == 3) {
        if (detail::no_tiny_values(in)) {
            detail::blur_y_rows<stride, true>(in, out);
        } else {
            detail::blur_y_rows<stride, false>(in, out);
        }
    } else {
        detail::blur_y_rows<stride, true>(in, out);
    }
}

}  // namespace gernels
