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

// The first-moment encode table lives in LDS at kEncLdsBegin + 16 * (bucket byte); the bytes
// between the two maps and the table are free for other use.
static constexpr uint32_t kEncLdsBegin = 4224;
static constexpr uint32_t kEncLdsEnd = kEncLdsBegin + (uint32_t)kEncEntries * 16;

// Where bucket `idx` (0..255) sits in the stored table, and whether it is the NaN bucket,
// whose entry is patched to code 15 on both sides.
LPMM_HD uint32_t enc_m_stored_index(uint32_t idx)
{
    uint32_t m = idx & 127u;
    m = m < kEncCompactLo ? kEncCompactLo : (m > kEncCompactHi ? kEncCompactHi : m);
    return (idx >> 7) * kEncCompactPerSign + m - kEncCompactLo;
}
static constexpr uint32_t kEncNanBucket = 0xfeu;

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

// The bucket byte of x: x converted to an 8-bit float with 5 exponent and 2 mantissa bits, round
// to nearest even, overflow to infinity (0x7c), every NaN to 0xfe.  On the device this is one
// v_cvt_pk_bf8_f32 for two values (encode8_std_m in lpmm_codec.hpp); this host twin restates the
// conversion for the exhaustive check of the table.
#if !defined(__HIP_DEVICE_COMPILE__)
static inline uint32_t enc_m_bucket_host(float x)
{
    const uint32_t b = f32_bits(x), sign = (b >> 31) << 7, mag = b & 0x7fffffffu;
    if (mag > 0x7f800000u)
        return 0xfeu;
    if ((mag >> 23) >= 113u) {
        const uint32_t r = (mag + 0xfffffu + ((mag >> 21) & 1u)) >> 21;
        return sign | (r - 448u < 0x7cu ? r - 448u : 0x7cu);
    }
    const double q = (double)bits_f32(mag) * 65536.0;  // multiples of 2^-16 below 2^-14
    uint32_t n = (uint32_t)q;
    const double frac = q - (double)n;
    if (frac > 0.5 || (frac == 0.5 && (n & 1u)))
        ++n;
    return sign | n;
}
#endif

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
