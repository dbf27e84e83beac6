// Device-side building blocks shared by the gfx950 kernels: streaming (nontemporal) memory
// access, near-exact sqrt/division from the hardware approximations, the LDS-resident
// quantisation maps and first-moment encode table, and 4-bit code assignment.
#pragma once

#include "lpmm_common.hpp"
#include "lpmm_encode.hpp"

namespace lpmm {

// ---------------------------------------------------------------------------------------
// Streaming access.  Every large operand of these kernels is touched exactly once per
// launch, so loads and stores carry the nontemporal hint: on MI355X the same access pattern
// runs at 5.9 TB/s with it and 4.8 TB/s without.
// ---------------------------------------------------------------------------------------
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float4 load4(const float *p)
{
    const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void store4(float *p, float4 v)
{
    const v4f t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(p));
}
__device__ __forceinline__ uint32_t load_u16(const uint16_t *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_u16(uint16_t *p, uint32_t v) { __builtin_nontemporal_store((uint16_t)v, p); }
__device__ __forceinline__ uint32_t load_u32(const uint32_t *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_u32(uint32_t *p, uint32_t v) { __builtin_nontemporal_store(v, p); }

// ---------------------------------------------------------------------------------------
// Near-exact arithmetic: hardware approximation + one fma correction of the exact residual.
// ---------------------------------------------------------------------------------------

// sqrt(x) for x >= 0: correctly rounded for x >= 2^-100 (no difference from sqrtf on every
// 16th float on the device); below that the residual underflows and the result may be 1 ulp
// off, and inputs below the smallest normal are treated as that value -- the square root of
// such a second moment is far below any eps it is added to.
__device__ __forceinline__ float sqrt_fast(float x)
{
    // max(x, 2^-126) on the bit patterns: the same as on the values for x >= +0 (a second moment is
    // never negative and never -0), one instruction instead of a canonicalising float max
    const uint32_t xb = __float_as_uint(x);
    const float y = __builtin_amdgcn_rsqf(__uint_as_float(xb > 0x00800000u ? xb : 0x00800000u));
    const float s = x * y;
    const float h = 0.5f * y;
    const float r = __builtin_fmaf(-s, s, x);
    return __builtin_fmaf(r, h, s);
}

// x / d: no difference from the correctly rounded quotient on 2^30 random pairs on the device.
__device__ __forceinline__ float div_fast(float x, float d)
{
    const float rc = __builtin_amdgcn_rcpf(d);
    const float q = x * rc;
    const float r = __builtin_fmaf(-q, d, x);
    return __builtin_fmaf(r, rc, q);
}

// x / y given rc = RN(1/y): one multiply and two fmas give the correctly rounded quotient
// when y lies in [2^-60, 2^60] and |x| <= y (no intermediate underflow where a code depends
// on it).
__device__ __forceinline__ float div_by_rc(float x, float y, float rc)
{
    const float q = x * rc;
    const float r = __builtin_fmaf(-q, y, x);
    return __builtin_fmaf(r, rc, q);
}

__device__ __forceinline__ bool rc_safe(float y) { return y >= 0x1p-60f && y <= 0x1p60f; }

// 1 / y for y in [2^-60, 2^60]: the hardware approximation and one Newton step.  Equal to the
// correctly rounded reciprocal for every float of that range on gfx950 (all 1 006 632 961 of
// them are compared by the device self-test), at 3 instructions instead of the 10 of the IEEE
// division sequence.
__device__ __forceinline__ float rcp_exact(float y)
{
    const float r = __builtin_amdgcn_rcpf(y);
    return __builtin_fmaf(__builtin_fmaf(-y, r, 1.0f), r, r);
}

// ---------------------------------------------------------------------------------------
// Which map is this?  Decided on the device from the 16 values themselves (scalar loads,
// xor/or, no branches, no host round trip).
// ---------------------------------------------------------------------------------------
enum MapKind : int { kMapGeneric = 0, kMapStdM = 1, kMapStdV = 2 };

__device__ __forceinline__ int classify_map(const float *__restrict__ qmap)
{
    uint32_t dm = 0, dv = 0;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        const uint32_t b = __float_as_uint(qmap[k]);
        dm |= b ^ kStdQmapMBits[k];
        dv |= b ^ kStdQmapVBits[k];
    }
    return dm == 0 ? kMapStdM : (dv == 0 ? kMapStdV : kMapGeneric);
}

// ---------------------------------------------------------------------------------------
// LDS map (bytes): [0,64) first map, [64,128) second map, then the first-moment encode
// table at the offsets lpmm_encode.hpp computes (the bytes in between stay unused).
// ---------------------------------------------------------------------------------------
constexpr uint32_t kLdsBytes = kEncLdsEnd;
constexpr uint32_t kLdsQ0 = 0, kLdsQ1 = 64;
static_assert(kLdsQ1 + 64 <= kEncLdsBegin, "maps overlap the encode table");

// Workgroup barrier that orders LDS accesses only: the waves wait for their own LDS
// operations, not for global loads that are still in flight.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <typename T>
__device__ __forceinline__ T lds_read(const uint32_t *lds, uint32_t byte_off)
{
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(lds) + byte_off);
}

// The encode-table entry of bucket idx (0..255), from the stored table: 80 entries of global
// memory serve all 256 buckets, so a workgroup's table costs 10 cache lines, not 32.
__device__ __forceinline__ uint4 enc_entry(uint32_t idx)
{
    uint4 e = *reinterpret_cast<const uint4 *>(kEncTableM[enc_m_stored_index(idx)]);
    if (idx == kEncNanBucket)
        e.y = e.z = 15u;
    return e;
}

// Threads [0,16) copy map 0, [16,32) map 1 (if given), all threads the encode table (one
// 16-byte entry each, in rounds of the workgroup's size).  The caller synchronises the
// workgroup afterwards.
__device__ __forceinline__ void lds_fill(uint32_t *lds, const float *__restrict__ q0, const float *__restrict__ q1)
{
    if (threadIdx.x < 16)
        lds[kLdsQ0 / 4 + threadIdx.x] = __float_as_uint(q0[threadIdx.x]);
    else if (threadIdx.x < 32 && q1 != nullptr)
        lds[kLdsQ1 / 4 + threadIdx.x - 16] = __float_as_uint(q1[threadIdx.x - 16]);
    for (uint32_t i = threadIdx.x; i < (uint32_t)kEncEntries; i += blockDim.x)
        *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(lds) + kEncLdsBegin + 16 * i) = enc_entry(i);
}

// The same in two halves for workgroups of exactly kEncEntries threads, so that a kernel can
// issue these small loads first, start its streaming loads, and write LDS once the small ones
// have arrived (loads return in order).  Every thread loads and every thread stores (threads
// past the maps repeat a map entry, so some addresses are written several times with the same
// value): no branch surrounds either half, and the wait before the stores counts exactly the
// loads issued in between.
struct LdsFill {
    uint32_t q;
    uint4 e;
};

__device__ __forceinline__ LdsFill lds_fill_load(const float *__restrict__ q0, const float *__restrict__ q1)
{
    LdsFill f;
    const uint32_t t = threadIdx.x;
    const float *qp = ((t & 16) == 0) ? q0 + (t & 15) : q1 + (t & 15);
    f.q = __float_as_uint(*qp);
    f.e = enc_entry(t);
    return f;
}

__device__ __forceinline__ void lds_fill_store(uint32_t *lds, const LdsFill &f)
{
    lds[threadIdx.x & 31] = f.q;  // kLdsQ0 = 0, kLdsQ1 = 64: the two maps are adjacent
    *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(lds) + kEncLdsBegin + 16 * threadIdx.x) = f.e;
}
static_assert(kLdsQ0 == 0 && kLdsQ1 == 64, "lds_fill_store writes the maps back to back");

// Codes of 8 values with the standard first-moment map: nibble k = code of x[k].  The bucket of
// a value is its conversion to an 8-bit float (two values per instruction, the four bytes of a
// word are the buckets of four values); the bucket's table entry {thr, code_le, code_gt} decides
// with one compare.  Any float is a legal input; a NaN gives 15.
__device__ __forceinline__ uint32_t encode8_std_m(const uint32_t *lds, const float (&x)[8])
{
    uint32_t w = 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        int b = __builtin_amdgcn_cvt_pk_bf8_f32(x[4 * h], x[4 * h + 1], 0, false);
        b = __builtin_amdgcn_cvt_pk_bf8_f32(x[4 * h + 2], x[4 * h + 3], b, true);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t off = (((uint32_t)b >> (8 * k)) & 0xffu) << 4;
            const uint4 e = lds_read<uint4>(lds, kEncLdsBegin + off);
            w |= enc_m_pick(x[4 * h + k], e.x, e.y, e.z) << (4 * (4 * h + k));
        }
    }
    return w;
}

// The same for the standard second-moment map; requires 0 <= x[k] <= 1 (so the code never
// exceeds 15) -- the clamp at 0 is done by the saturating byte conversion.
__device__ __forceinline__ uint32_t encode8_std_v(const float (&x)[8])
{
    uint32_t b[2] = {0u, 0u};  // codes of elements 0..3 / 4..7, one per byte
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float t = __builtin_ceilf(__builtin_fmaf(x[k], 16.0f, -1.5f));
        b[k >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(t, k & 3, b[k >> 2]);
    }
    // bytes {c0,c1,c2,c3} -> byte 0 = c0|c1<<4, byte 2 = c2|c3<<4; gather bytes 0, 2 of both words
    const uint32_t t0 = b[0] | (b[0] >> 4), t1 = b[1] | (b[1] >> 4);
    return __builtin_amdgcn_perm(t1, t0, 0x06040200u);
}

// Any ascending map: count of midpoints below x; NaN -> 15.
__device__ __forceinline__ uint32_t encode8_generic(const Mids &mids, const float (&x)[8])
{
    uint32_t w = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k)
        w |= ((x[k] != x[k]) ? 15u : encode_count(mids, x[k])) << (4 * k);
    return w;
}

// Codes of v[k] / amax for the 8 values of a lane (amax uniform over the lanes that share a
// scale).  `kind` says which map sits at LDS offset `lds_map`; an all-zero group (0/0 -> NaN)
// gives code 15 throughout, as in the reference.  For kMapStdV the values must be >= 0.
__device__ __forceinline__ uint32_t encode8_scaled(const uint32_t *lds, uint32_t lds_map, int kind,
                                                   const float (&v)[8], float amax)
{
    float x[8];
    if (kind != kMapGeneric && rc_safe(amax)) {
        const float rc = rcp_exact(amax);
#pragma unroll
        for (int k = 0; k < 8; ++k)
            x[k] = div_by_rc(v[k], amax, rc);
        return kind == kMapStdM ? encode8_std_m(lds, x) : encode8_std_v(x);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
        x[k] = v[k] / amax;
    // the map is read back from LDS so that it occupies registers only on this path
    const Mids mids = make_mids(reinterpret_cast<const float *>(lds) + lds_map / 4);
    return encode8_generic(mids, x);
}

// Codes of 8 values that are already normalised (no division); `kind` says which map sits at
// LDS offset `lds_map`.  NaN -> 15 like the reference.
__device__ __forceinline__ uint32_t encode8_plain(const uint32_t *lds, uint32_t lds_map, int kind, const float (&x)[8])
{
    if (kind == kMapGeneric)
        return encode8_generic(make_mids(reinterpret_cast<const float *>(lds) + lds_map / 4), x);
    uint32_t w;
    if (kind == kMapStdM) {
        w = encode8_std_m(lds, x);
    } else {
        // the closed form needs x <= 1 for the upper clamp; larger inputs are legal here
        float y[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            y[k] = fminf(x[k], 1.0f);
        w = encode8_std_v(y);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k)
        if (x[k] != x[k])
            w |= 15u << (4 * k);
    return w;
}

// Packed codes of a 128-value group in the row layout: lane l of the DPP row works on the 16-bit
// halves l (elements 4l .. 4l+3) and 16 + l (elements 64+4l .. 64+4l+3) of the group's 64 bytes, as
// the word  half l | half (16 + l) << 16.  In memory the group is 16 dwords, dword d = halves 2d, 2d+1.
// Lane 2i accesses dword i (the first halves of lanes 2i and 2i+1), lane 2i+1 dword 8 + i (their second
// halves); one exchange between the two lanes turns the memory form into the lane form and back
// (it is its own inverse): even lane {own.lo, neighbour.lo}, odd lane {neighbour.hi, own.hi}.
__device__ __forceinline__ uint32_t code_dword_of_lane(int lane16)
{
    return (lane16 & 1) ? 8u + ((uint32_t)lane16 >> 1) : (uint32_t)lane16 >> 1;
}
__device__ __forceinline__ uint32_t code_swap_selector(int lane16)
{
    return (lane16 & 1) ? 0x03020706u : 0x05040100u;  // v_perm_b32 byte selectors, {neighbour, own}
}
__device__ __forceinline__ uint32_t swap_code_halves(uint32_t w, uint32_t selector)
{
    const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xB1 /* quad_perm:[1,0,3,2] */, 0xF, 0xF, false);
    return __builtin_amdgcn_perm(nb, w, selector);
}

// Decode offsets: byte j of `even` / `odd` holds 4 * nibble (2j) / (2j+1) of the code word.
struct Nibbles {
    uint32_t even, odd;
};

__device__ __forceinline__ Nibbles split_nibbles(uint32_t w)
{
    Nibbles n;
    n.even = (w << 2) & 0x3C3C3C3Cu;
    n.odd = (w >> 2) & 0x3C3C3C3Cu;
    // keep the masked words as they are, so that each offset below is one bit-field extract
    asm volatile("" : "+v"(n.even), "+v"(n.odd));
    return n;
}

// qmap[nibble k] from the map at LDS offset lds_map
__device__ __forceinline__ float decode_nibble(const uint32_t *lds, uint32_t lds_map, const Nibbles &n, int k)
{
    const uint32_t off = __builtin_amdgcn_ubfe((k & 1) ? n.odd : n.even, 8 * (k >> 1), 8);
    return lds_read<float>(lds, lds_map + off);
}

}  // namespace lpmm
