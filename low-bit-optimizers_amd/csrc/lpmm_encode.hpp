// Fast code assignment for the two standard 4-bit maps, written so that the same source
// compiles for the device (HIP) and for the host (exhaustive checks in tests/).
//
// Both functions return exactly what the reference search returns for every non-NaN x:
// the number of fp32 midpoints of the map that are < x
// (lpmm/cpp_extension/fused_adamw_kernel.cu:27-49).  NaN is the caller's business.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define LPMM_HD __host__ __device__ __forceinline__
#else
#define LPMM_HD static inline
#include <cmath>
#include <cstring>
#endif

namespace lpmm {

#include "std_tables.inc"

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

// Byte offset of x's entry in the first-moment encode table (16 bytes per entry, negative
// half after kEncBuckets entries).
LPMM_HD uint32_t enc_m_offset(uint32_t xb)
{
    int32_t idx = (int32_t)((xb & 0x7fffffffu) >> (23 - kEncMantBits));
    idx = idx < kEncLo ? kEncLo : (idx > kEncHi ? kEncHi : idx);
    return ((uint32_t)(idx - kEncLo) << 4) + ((xb >> 31) * (uint32_t)(kEncBuckets * 16));
}

// entry = {thr, code_le, code_gt, 0}
LPMM_HD uint32_t enc_m_select(uint32_t xb, uint32_t thr, uint32_t code_le, uint32_t code_gt)
{
    return ((xb & 0x7fffffffu) > thr) ? code_gt : code_le;
}

// Second-moment map q[k] = (k+1)/16, midpoints (2k+1)/32 for k = 1..15:
// code = #{k : (2k+1)/32 < x} = clamp(ceil(16x - 1.5), 0, 15); 16x - 1.5 is computed with one
// rounding (fma) and is exact wherever its value matters.
LPMM_HD uint32_t enc_v_linear(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const float t = __builtin_ceilf(__builtin_fmaf(x, 16.0f, -1.5f));
#else
    const float t = std::ceil(std::fmaf(x, 16.0f, -1.5f));
#endif
    int32_t c = (t < 0.0f) ? 0 : ((t > 15.0f) ? 15 : (int32_t)t);  // also maps NaN to 15? no: NaN -> 15 below
    return (uint32_t)c;
}

}  // namespace lpmm
