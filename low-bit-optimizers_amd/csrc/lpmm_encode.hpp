// Fast code assignment for the two standard 4-bit maps, written so that the same source
// compiles for the device (HIP) and for the host (exhaustive check in tests/).
//
// Both return exactly what the reference search returns for every non-NaN x: the number of
// fp32 midpoints of the map that are < x
// (lpmm/cpp_extension/fused_adamw_kernel.cu:27-49).  NaN is the caller's business.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define LPMM_HD __host__ __device__ __forceinline__
#else
#define LPMM_HD static inline
#endif
#if !defined(__HIP_DEVICE_COMPILE__)
#include <cmath>
#include <cstring>
#endif

namespace lpmm {

#include "std_tables.inc"

// The first-moment encode table lives in LDS at byte (bucket index * 16) for x >= 0 and
// kEncSignStride bytes further for x < 0; bucket indices run from kEncLo to kEncHi, so the
// bytes below kEncLo*16 are free for other use.
static constexpr uint32_t kEncLdsBegin = (uint32_t)kEncLo * 16;
static constexpr uint32_t kEncLdsEnd = (uint32_t)(kEncHi + 1) * 16 + kEncSignStride;
static_assert((uint32_t)(kEncHi + 1) * 16 <= kEncSignStride, "sign bit collides with the bucket offset");
static_assert(kEncMantBits == 2, "shifts below assume 21 dropped mantissa bits");

LPMM_HD uint32_t f32_bits(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(x);
#else
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
#endif
}

LPMM_HD float bits_f32(uint32_t u)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(u);
#else
    float x;
    memcpy(&x, &u, 4);
    return x;
#endif
}

// LDS byte offset of x's table entry {thr, code_le, code_gt}.
LPMM_HD uint32_t enc_m_lds_offset(float x)
{
    const float lo = bits_f32(kEncClampLoBits), hi = bits_f32(kEncClampHiBits);
#if defined(__HIP_DEVICE_COMPILE__)
    const float a = __builtin_amdgcn_fmed3f(__builtin_fabsf(x), lo, hi);
#else
    const float a = std::fmin(std::fmax(std::fabs(x), lo), hi);
#endif
    // (bits(a) >> 21) * 16, plus kEncSignStride when the sign bit of x is set
    return ((f32_bits(a) >> 17) & 0x3FF0u) | ((f32_bits(x) >> 18) & kEncSignStride);
}

// thr is compared as a float: magnitudes order like their bit patterns, and the "no
// midpoint in this bucket" pattern 0xffffffff is a NaN, which never compares below.
LPMM_HD uint32_t enc_m_pick(float x, uint32_t thr, uint32_t code_le, uint32_t code_gt)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return (__builtin_fabsf(x) > bits_f32(thr)) ? code_gt : code_le;
#else
    return (std::fabs(x) > bits_f32(thr)) ? code_gt : code_le;
#endif
}

// Second-moment map q[k] = (k+1)/16, midpoints (2k+1)/32 for k = 1..15:
// code = #{k : (2k+1)/32 < x} = clamp(ceil(16x - 1.5), 0, 15); 16x - 1.5 is computed with one
// rounding (fma) and is exact wherever its value decides the code.
LPMM_HD uint32_t enc_v_linear(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const int c = (int)__builtin_ceilf(__builtin_fmaf(x, 16.0f, -1.5f));  // v_cvt_i32_f32 saturates
    return (uint32_t)(c < 0 ? 0 : (c > 15 ? 15 : c));  // v_med3_i32
#else
    const float t = std::ceil(std::fmaf(x, 16.0f, -1.5f));
    return (uint32_t)((t < 0.0f) ? 0 : ((t > 15.0f) ? 15 : (int)t));
#endif
}

}  // namespace lpmm
