// Separable box-blur stages on wave-distributed register tiles.
//
// Arithmetic follows the reference gernels (apps/common/impl/impl.h:190-214
// blur_x, :216-250 blur_y): a running fp32 sum that starts at 0, taps added
// left to right (top to bottom), then a division by the tap count.  The
// division is done by div_const<>, which is bit-identical to the IEEE
// quotient for the tap counts it accelerates.
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

template<int64_t stride, typename TI, typename TO>
__device__ __forceinline__ void blur_x(const TI &in, TO &out) {
    static_assert(TI::chunks == 1 && TO::chunks == 1, "blur_x works on tiles at most 256 columns wide");
    static_assert(stride >= 1 && stride <= 5, "the right-hand halo must fit in the neighbouring lane");
    static_assert(TI::cols >= TO::cols + stride - 1, "input tile narrower than output + halo");
    static_assert(TI::rows >= TO::rows, "input tile shorter than output");
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
            float sum = 0;
#pragma unroll
            for (int s = 0; s < stride; s++) {
                sum += w[e + s];
            }
            o[e] = div_const<stride>(sum);
        }
        out.v[r][0] = make_float4(o[0], o[1], o[2], o[3]);
    }
}

template<int64_t stride, typename TI, typename TO>
__device__ __forceinline__ void blur_y(const TI &in, TO &out) {
    static_assert(TI::chunks == TO::chunks, "blur_y keeps the column layout");
    static_assert(TI::rows >= TO::rows + stride - 1, "input tile shorter than output + halo");
#pragma unroll
    for (int64_t r = 0; r < TO::rows; r++) {
#pragma unroll
        for (int64_t k = 0; k < TO::chunks; k++) {
            float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int64_t s = 0; s < stride; s++) {
                const float4 t = in.v[r + s][k];
                sum.x += t.x;
                sum.y += t.y;
                sum.z += t.z;
                sum.w += t.w;
            }
            out.v[r][k] = make_float4(div_const<stride>(sum.x), div_const<stride>(sum.y),
                                      div_const<stride>(sum.z), div_const<stride>(sum.w));
        }
    }
}

}  // namespace gernels
