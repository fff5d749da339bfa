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

// Division of a tap sum by the tap count.
//
// The reference's blur sums start at +0 (apps/common/impl/impl.h:190-250), so
// a sum is never -0 unless it underflowed; "sum" below is that sum with the
// leading +0 left out, which differs only when every tap is -0 (then it is -0
// instead of +0).  quotient_of_sum<D>() returns what the reference's
// (0 + taps...) / D gives, bit for bit:
//
//  * D == 3: 1/3 = c_hi + c_lo with c_hi rounded DOWN, so that c_lo > 0;
//    t = fma(s, c_lo, +0) is the correction term, with -0 turned into +0 on
//    the way; q = fma(s, c_hi, t) rounds the (nearly) exact quotient once.
//    Infinities, NaNs and zeros come out as IEEE division gives them without
//    a fix-up (inf * c_hi + inf * c_lo = inf).  Checked on the host against
//    x / 3.0f for all 2^32 operands: identical except for dividends with
//    2^-126 <= |x| < 2^-122, where t underflows and the quotient (a subnormal
//    number below 4e-38) can be one unit in the last place off: callers rule
//    that range out first (gernels/blur.h).  The previous form -- multiply,
//    two FMAs and v_div_fixup, exact everywhere -- cost four instructions per
//    output instead of two, and the blur chain is limited by vector-ALU issue
//    as much as by memory.
//  * D a power of two: s * 2^-k is exact; the FMA with +0 only turns -0 into +0.
//  * other D: IEEE division of (0 + s).
template<int64_t D>
struct ExactReciprocal {
    static constexpr bool value = (D == 2 || D == 3 || D == 4 || D == 8);
};

template<int64_t D>
__device__ __forceinline__ float quotient_of_sum(float s) {
    if constexpr (D == 3) {
        const float c_hi = as_float(0x3EAAAAAA);  // largest float below 1/3
        const float c_lo = as_float(0x32AAAAAB);  // 1/3 - c_hi, rounded to nearest
        const float t = __builtin_fmaf(s, c_lo, 0.0f);
        return __builtin_fmaf(s, c_hi, t);
    } else if constexpr (D == 2 || D == 4 || D == 8) {
        return __builtin_fmaf(s, 1.0f / (float)D, 0.0f);
    } else {
        return (0.0f + s) / (float)D;
    }
}

}  // namespace gernels
