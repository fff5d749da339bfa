// Common definitions for the gfx950 gernel library.
//
// Every header in this directory is device code that the generated kernel
// #includes; it is compiled either by hiprtc at run time (the Runner's path)
// or by hipcc ahead of time (the build check).  hiprtc ships no C library
// headers, so the fixed-width integer names come from its built-in runtime
// header there and from <cstdint> under hipcc.
#pragma once

#if defined(__HIPCC_RTC__)
using __hip_internal::int32_t;
using __hip_internal::int64_t;
using __hip_internal::uint16_t;
using __hip_internal::uint32_t;
using __hip_internal::uint64_t;
#else
#include <cstdint>
#include <hip/hip_runtime.h>
#endif

namespace gernels {

// CDNA4 executes 64-lane wavefronts; every wave-cooperative gernel below is
// written against this width.
constexpr int kWaveSize = 64;
// Lanes of one wave cover this many consecutive fp32 columns per 16-byte
// access (64 lanes x float4).
constexpr int kWaveCols = 4 * kWaveSize;

__device__ __forceinline__ int lane_id() {
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

__device__ __forceinline__ float as_float(int x) {
    return __builtin_bit_cast(float, x);
}
__device__ __forceinline__ int as_int(float x) {
    return __builtin_bit_cast(int, x);
}

// Value held by lane+1 (lane 63 receives 0).  One DPP move, no LDS traffic.
__device__ __forceinline__ float from_next_lane(float x) {
    return as_float(__builtin_amdgcn_update_dpp(0, as_int(x), 0x130 /* wave_shl:1 */, 0xf, 0xf, true));
}

// x / d for a divisor that is the same for many dividends: multiply by the
// rounded reciprocal, then one FMA residual correction.  For d == 3 this
// equals the IEEE quotient for every finite fp32 x (checked exhaustively on
// the host); v_div_fixup restores the IEEE result for infinities, NaNs and
// zero operands.
__device__ __forceinline__ float div_by(float x, float d, float rcp_d) {
    float q = x * rcp_d;
    float r = __builtin_fmaf(-d, q, x);
    q = __builtin_fmaf(r, rcp_d, q);
    return __builtin_amdgcn_div_fixupf(q, d, x);
}

// Divisors for which div_by() is bit-exact against IEEE division over all
// finite fp32 dividends: 3 by exhaustive check on the host; powers of two
// because x * 2^-k is already the correctly rounded quotient and the residual
// step then rounds the exact quotient once more.  Any other divisor takes the
// full IEEE division.
template<int64_t D>
struct ExactReciprocal {
    static constexpr bool value = (D == 2 || D == 3 || D == 4 || D == 8);
};

template<int64_t D>
__device__ __forceinline__ float div_const(float x) {
    if constexpr (D == 1) {
        return x;
    } else if constexpr (ExactReciprocal<D>::value) {
        return div_by(x, (float)D, 1.0f / (float)D);
    } else {
        return x / (float)D;
    }
}

}  // namespace gernels
