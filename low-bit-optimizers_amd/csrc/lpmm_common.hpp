// Shared host/device helpers of the gfx950 kernels.  Wave size is 64; a DPP row is 16 lanes.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "lpmm_hip.h"

namespace lpmm {

constexpr int kWave = 64;
constexpr int kGroup = LPMM_GROUP;

// ---------------------------------------------------------------------------------------
// host-side argument checks
// ---------------------------------------------------------------------------------------
inline bool aligned_to(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

#define LPMM_REQUIRE_PTR(p)       \
    do {                          \
        if ((p) == nullptr)       \
            return LPMM_ERR_NULL; \
    } while (0)

#define LPMM_REQUIRE_ALIGN(p, a)   \
    do {                           \
        if (!lpmm::aligned_to(p, a)) \
            return LPMM_ERR_ALIGN; \
    } while (0)

inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? LPMM_OK : LPMM_ERR_LAUNCH;
}

// ---------------------------------------------------------------------------------------
// Tile order of the one-shot streaming kernels.  The hardware hands consecutive workgroup indices to
// the 8 XCDs of an MI355X in turn, so with "workgroup i takes tile i" every XCD touches every
// neighbouring tile of every operand.  The memory system gives 3-5 % more to a streaming kernel when
// each XCD instead works through runs of 128 KB of address space whose position within the enclosing
// 1 MB block is the same for all of its runs (measured on copies, in-place updates and the seven streams of the
// fused step; 96, 160 or 256 KB runs, or 128 KB runs that start 64 KB off a 128 KB boundary, lose the
// gain again; which XCD takes which of the eight positions does not matter).  xcd_run_order maps the index a
// workgroup has within its tensor to the tile it works on: within every whole, 1 MB-aligned block of
// tiles the 8 << LOG2 consecutive indices go to the 8 runs in turn, so the 8 XCDs advance through their
// runs side by side and the tiles in flight still form one compact window.  Blocks cut by either end of
// the tensor keep the plain order.  `phase` is the position of the tensor's first tile within its 1 MB
// block of address space, in tiles (run_phase).
// ---------------------------------------------------------------------------------------
constexpr uint32_t kXcds = 8;
constexpr uint32_t kXcdRunBytes = 128 * 1024;

template <int LOG2>
__device__ __forceinline__ uint32_t xcd_run_order(uint32_t index, uint32_t tiles, uint32_t phase)
{
    constexpr uint32_t kBlock = kXcds << LOG2, kMask = kBlock - 1u;
    const uint32_t v = index + phase, block0 = v & ~kMask;
    if (block0 < phase || block0 + kBlock > phase + tiles)
        return index;
    return (block0 | ((v & (kXcds - 1u)) << LOG2) | ((v >> 3) & ((1u << LOG2) - 1u))) - phase;
}

// tile_bytes: bytes of the dominant operand per tile (a power of two); 8 << LOG2 tiles make 1 MB
template <int LOG2>
__device__ __forceinline__ uint32_t run_phase(const void *base, uint32_t tile_bytes)
{
    return (uint32_t)(reinterpret_cast<uintptr_t>(base) / tile_bytes) & ((kXcds << LOG2) - 1u);
}

// ---------------------------------------------------------------------------------------
// DPP lane exchange inside a 16-lane row.  The four steps quad xor 1, quad xor 2,
// half-row mirror and row mirror leave the row-wide result in every lane.
// ---------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}

// One step: v = max(v, v of the lane the DPP control names).  The exchange is an operand
// modifier of the max itself (one instruction per step).  A DPP operand may be read two wait
// states after the instruction that wrote it at the earliest; inline assembly is outside the
// compiler's hazard handling, so the s_nop in front supplies them.
#define LPMM_DPP_MAX(ctrl) "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 " ctrl " row_mask:0xf bank_mask:0xf\n\t"
#define LPMM_DPP_MAX2(ctrl)                                              \
    "s_nop 0\n\tv_max_f32_dpp %0, %0, %0 " ctrl " row_mask:0xf bank_mask:0xf\n\t" \
    "v_max_f32_dpp %1, %1, %1 " ctrl " row_mask:0xf bank_mask:0xf\n\t"

__device__ __forceinline__ float row16_max(float v)
{
    asm(LPMM_DPP_MAX("quad_perm:[1,0,3,2]") LPMM_DPP_MAX("quad_perm:[2,3,0,1]")
            LPMM_DPP_MAX("row_half_mirror") LPMM_DPP_MAX("row_mirror")
        : "+v"(v));
    return v;
}

// Two row maxima at once: the second value's instruction fills one of the wait states of the first.
__device__ __forceinline__ void row16_max2(float &a, float &b)
{
    asm("s_nop 1\n\t" LPMM_DPP_MAX2("quad_perm:[1,0,3,2]") LPMM_DPP_MAX2("quad_perm:[2,3,0,1]")
            LPMM_DPP_MAX2("row_half_mirror") LPMM_DPP_MAX2("row_mirror")
        : "+v"(a), "+v"(b));
}

// Row layout: the 16 lanes of a DPP row own one 128-element group, lane l the elements
// [4l, 4l+4) and [64+4l, 64+4l+4); element k (0..7) of a lane sits at this offset in the group.
__device__ __forceinline__ int elt_offset(int lane16, int k) { return lane16 * 4 + (k & 3) + (k >> 2) * 64; }

// max of non-negative floats == max of their bit patterns as unsigned integers
__device__ __forceinline__ void atomic_max_nonneg(float *addr, float v)
{
    atomicMax(reinterpret_cast<unsigned int *>(addr), __float_as_uint(v));
}

__device__ __forceinline__ float wave_max(float v)
{
    v = row16_max(v);
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

__device__ __forceinline__ double wave_sum_f64(double v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// Eight wave-wide sums at once.  Three halving exchanges (lane ^ 32, ^ 16, ^ 8) in each of
// which a lane keeps half of its values and hands the other half over, then three steps on
// the one value left: lane 8j (and the seven lanes after it) holds the sum of v[j] over the
// wave.  7 value exchanges through the LDS crossbar instead of 48, the order of the additions
// is fixed.
template <int CTRL>
__device__ __forceinline__ double dpp_f64(double v)
{
    const uint64_t u = (uint64_t)__double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)u, CTRL, 0xF, 0xF, false);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(u >> 32), CTRL, 0xF, 0xF, false);
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}

__device__ __forceinline__ double wave_sum8_f64(const double (&v)[8], int lane)
{
    double a[4], b[2], c;
    const bool h32 = (lane & 32) != 0, h16 = (lane & 16) != 0, h8 = (lane & 8) != 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const double keep = h32 ? v[4 + i] : v[i], give = h32 ? v[i] : v[4 + i];
        a[i] = keep + __shfl_xor(give, 32, 64);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const double keep = h16 ? a[2 + i] : a[i], give = h16 ? a[i] : a[2 + i];
        b[i] = keep + __shfl_xor(give, 16, 64);
    }
    {
        const double keep = h8 ? b[1] : b[0], give = h8 ? b[0] : b[1];
        c = keep + __shfl_xor(give, 8, 64);
    }
    c += dpp_f64<0xB1>(c);   // quad_perm [1,0,3,2]
    c += dpp_f64<0x4E>(c);   // quad_perm [2,3,0,1]
    c += dpp_f64<0x141>(c);  // row_half_mirror: the other quad of the same eight lanes
    return c;
}

// The same for eight wave-wide maxima of floats: lane 8j (and the seven lanes after it) ends
// up with the maximum of v[j] over the wave.
__device__ __forceinline__ float wave_max8(const float (&v)[8], int lane)
{
    float a[4], b[2], c;
    const bool h32 = (lane & 32) != 0, h16 = (lane & 16) != 0, h8 = (lane & 8) != 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float keep = h32 ? v[4 + i] : v[i], give = h32 ? v[i] : v[4 + i];
        a[i] = fmaxf(keep, __shfl_xor(give, 32, 64));
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const float keep = h16 ? a[2 + i] : a[i], give = h16 ? a[i] : a[2 + i];
        b[i] = fmaxf(keep, __shfl_xor(give, 16, 64));
    }
    {
        const float keep = h8 ? b[1] : b[0], give = h8 ? b[0] : b[1];
        c = fmaxf(keep, __shfl_xor(give, 8, 64));
    }
    c = fmaxf(c, dpp_f32<0xB1>(c));   // quad_perm [1,0,3,2]
    c = fmaxf(c, dpp_f32<0x4E>(c));   // quad_perm [2,3,0,1]
    c = fmaxf(c, dpp_f32<0x141>(c));  // row_half_mirror: the other quad of the same eight lanes
    return c;
}

// ---------------------------------------------------------------------------------------
// Code assignment for an ascending 16-entry map given its 15 fp32 midpoints:
// code = number of midpoints strictly below x.  Identical to the reference's upper-bound
// search followed by the midpoint test, including "exact tie -> lower code".  NaN compares
// false everywhere and yields 0 here; callers map NaN to 15 themselves (a NaN arises only
// from 0/0, i.e. a group whose maximum is 0, which is uniform over the group).
// ---------------------------------------------------------------------------------------
struct Mids {
    float v[15];
};

__device__ __forceinline__ Mids make_mids(const float *__restrict__ qmap)
{
    Mids m;
    float prev = qmap[0];
#pragma unroll
    for (int k = 1; k < 16; ++k) {
        const float cur = qmap[k];
        m.v[k - 1] = (prev + cur) * 0.5f;
        prev = cur;
    }
    return m;
}

__device__ __forceinline__ uint32_t encode_count(const Mids &m, float x)
{
    uint32_t c = 0;
#pragma unroll
    for (int k = 0; k < 15; ++k)
        c += (m.v[k] < x) ? 1u : 0u;
    return c;
}

}  // namespace lpmm
