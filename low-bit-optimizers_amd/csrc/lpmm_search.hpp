// Code search for maps of 2^bits entries (1..8 bits) in LDS, shared by the stand-alone quantisers
// and the optimizer-step kernels for code widths other than 4.
#pragma once
#include "lpmm_codec.hpp"

namespace lpmm {

__host__ __device__ __forceinline__ int codes_per_byte(int bits) { return (bits == 1 || bits == 2 || bits == 4) ? 8 / bits : 1; }

// the map, 2^bits floats, into LDS; the caller synchronises
__device__ __forceinline__ void fill_map(float *lds_map, const float *__restrict__ qmap, int bits)
{
    for (int j = threadIdx.x; j < (1 << bits); j += blockDim.x)
        lds_map[j] = qmap[j];
}

// quantize_bsearch<false> (quantization_kernel.cu:397-427) as the stored code, without a data
// dependent branch.  The reference returns 0 for x <= q[0] and N-1 for q[N-1] <= x; otherwise it
// finds lo = the first entry above x (upper bound) and answers lo or lo-1 by the midpoint test
// mid = (q[lo-1] + q[lo]) * 0.5f < x.  For NaN its search ends at lo = 0 and returns -1, which it
// casts to uint8_t (one code per byte: 255) or masks (packed: the all-ones code).
//
// Here the upper bound among the first N-1 entries of the non-decreasing map (repeated entries
// included) comes from a descent through the entries in breadth-first order: node i of the
// perfect tree over q[0..N-2] holds its in-order entry, i = 2i + (node <= x) for `bits` levels,
// and i - N is the number of entries <= x.  A binary search over the sorted array would read, at
// every level, entries that are a power of two apart -- all in the same LDS bank; in
// breadth-first order the nodes of a level are neighbours, so up to 32 of them sit in 32
// different banks (and lanes that read the same node share one access).  The midpoints are
// formed once per workgroup with the reference's expression.
//
// The evenly spaced map without zero, q[k] = (k + 1) / N (create_pow_map(b, False, 1),
// lpmm/functional.py:303-315: the second moment's map of every shipped configuration), needs no
// search: its midpoints are (2j + 1) / 2N, and the number of them below x is
// ceil(x * N - 1.5) clamped to [0, N - 1] -- exact in float arithmetic (x * N is a scaling by a
// power of two, and the fused subtraction rounds once).  The stored code depends on the map only
// through its first and last entry and its midpoints (the entries themselves only select which
// midpoint decides), so the closed form applies whenever those have the values of that map, which
// is checked while the tables are filled: every wave records whether its entries match.
struct SearchLds {
    float tree[256];  // [1, N): breadth-first; [0]: q[0]
    float mid[256];   // [1, N): (q[lo-1] + q[lo]) * 0.5f; [0]: q[N-1]
    uint32_t even[16];  // per wave of the workgroup: do the entries it filled match the evenly spaced map
};

// does entry j (as stored: tree[0] = q[0], mid[0] = q[N-1], mid[j] for j >= 1) match the evenly spaced map
__device__ __forceinline__ bool matches_even_map(uint32_t j, float tree, float mid, int bits)
{
    const float step = __uint_as_float((127u - (uint32_t)bits) << 23);  // 1 / N
    return j == 0 ? (tree == step && mid == 1.0f) : mid == (float)(2u * j + 1u) * (0.5f * step);
}

// all waves' records (after the barrier that follows the fill); uniform over the workgroup, in a scalar register
__device__ __forceinline__ bool map_is_even(const SearchLds &t)
{
    uint32_t ok = 1u;
    for (uint32_t w = 0; w < (blockDim.x + kWave - 1) / kWave; ++w)
        ok &= t.even[w];
    return __builtin_amdgcn_readfirstlane((int)ok) != 0;
}

// the caller synchronises
__device__ __forceinline__ void fill_search(SearchLds &t, const float *__restrict__ qmap, int bits)
{
    const uint32_t n = 1u << bits;
    bool even = true;
    for (uint32_t j = threadIdx.x; j < n; j += blockDim.x) {
        float tree, mid;
        if (j == 0) {
            tree = qmap[0];
            mid = qmap[n - 1];
        } else {
            const uint32_t level = 31u - (uint32_t)__clz((int)j);
            const uint32_t k = j - (1u << level);
            tree = qmap[(((2u * k + 1u) << (bits - 1 - level))) - 1u];
            mid = (qmap[j - 1] + qmap[j]) * 0.5f;
        }
        t.tree[j] = tree;
        t.mid[j] = mid;
        even = even && matches_even_map(j, tree, mid, bits);
    }
    const bool wave_even = __all(even);
    if ((threadIdx.x & (kWave - 1)) == 0)
        t.even[threadIdx.x / kWave] = wave_even;
}

// The same in two halves for workgroups of at least 2^bits threads (one entry per thread), so that a
// kernel can issue these small loads first, start its streaming loads, and write LDS once the small
// ones have arrived (loads return in order).
struct SearchFill {
    float tree, mid;
};

__device__ __forceinline__ SearchFill fill_search_load(const float *__restrict__ qmap, int bits)
{
    SearchFill f;
    const uint32_t n = 1u << bits, j = threadIdx.x;
    f.tree = f.mid = 0.0f;
    if (j == 0) {
        f.tree = qmap[0];
        f.mid = qmap[n - 1];
    } else if (j < n) {
        const uint32_t level = 31u - (uint32_t)__clz((int)j);
        const uint32_t k = j - (1u << level);
        f.tree = qmap[(((2u * k + 1u) << (bits - 1 - level))) - 1u];
        f.mid = (qmap[j - 1] + qmap[j]) * 0.5f;
    }
    return f;
}

__device__ __forceinline__ void fill_search_store(SearchLds &t, const SearchFill &f, int bits)
{
    const bool mine = threadIdx.x < (1u << bits);
    if (mine) {
        t.tree[threadIdx.x] = f.tree;
        t.mid[threadIdx.x] = f.mid;
    }
    const bool wave_even = __all(!mine || matches_even_map(threadIdx.x, f.tree, f.mid, bits));
    if ((threadIdx.x & (kWave - 1)) == 0)
        t.even[threadIdx.x / kWave] = wave_even;
}

__device__ __forceinline__ uint32_t search_code(const SearchLds &t, int bits, float x)
{
    const uint32_t n = 1u << bits;
    uint32_t i = 1;
    for (int l = 0; l < bits; ++l)
        i = 2u * i + ((t.tree[i] <= x) ? 1u : 0u);
    const uint32_t pos = i - n;  // entries among the first n-1 that are <= x
    // Inside the map's range the upper bound is pos (q[n-1] > x there), at least 1
    const uint32_t lo = pos > 0 ? pos : 1u;
    uint32_t code = (t.mid[lo] < x) ? lo : lo - 1u;
    code = (t.mid[0] <= x) ? n - 1u : code;
    code = (x <= t.tree[0]) ? 0u : code;
    const uint32_t nan_code = codes_per_byte(bits) == 1 ? 255u : n - 1u;
    return (x != x) ? nan_code : code;
}

// The same for a lane's 8 values at once (even: map_is_even(t), read once per kernel after the
// barrier that follows the fill): the levels are the outer loop, so that the 8 reads of
// a level are in flight together instead of 8 x `bits` dependent ones in a row.
__device__ __forceinline__ void search_codes8(const SearchLds &t, int bits, bool even, const float (&x)[8],
                                              uint32_t (&code)[8])
{
    const uint32_t n = 1u << bits;
    if (even) {
        const float scale = (float)n, top = (float)(n - 1u);
        const uint32_t nan = codes_per_byte(bits) == 1 ? 255u : n - 1u;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float c = fminf(fmaxf(__builtin_ceilf(__builtin_fmaf(x[k], scale, -1.5f)), 0.0f), top);
            code[k] = (x[k] != x[k]) ? nan : (uint32_t)c;
        }
        return;
    }
    // a = byte offset of the node (4 i): one shift-or per level, no separate address computation
    uint32_t a[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
        a[k] = 4;
    const char *tree = reinterpret_cast<const char *>(t.tree);
    for (int l = 0; l < bits; ++l) {
        // The eight compares write eight different scalar register pairs and the eight selects
        // follow them: a select may read a mask two wait states after the compare that wrote it
        // at the earliest, which the seven instructions in between supply (the compiler's own
        // code goes through VCC and pays a pause per value and level).
        float node[8];
        uint64_t le[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            node[k] = *reinterpret_cast<const float *>(tree + a[k]);
#pragma unroll
        for (int k = 0; k < 8; ++k)
            asm volatile("v_cmp_le_f32_e64 %0, %1, %2" : "=s"(le[k]) : "v"(node[k]), "v"(x[k]));
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            uint32_t step;
            asm volatile("v_cndmask_b32_e64 %0, 0, 4, %1" : "=v"(step) : "s"(le[k]));
            a[k] = (a[k] << 1) | step;
        }
    }
    uint32_t i[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
        i[k] = a[k] >> 2;
    const float first = t.tree[0], last = t.mid[0];
    const uint32_t nan_code = codes_per_byte(bits) == 1 ? 255u : n - 1u;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t pos = i[k] - n;
        const uint32_t lo = pos > 0 ? pos : 1u;
        uint32_t c = (t.mid[lo] < x[k]) ? lo : lo - 1u;
        c = (last <= x[k]) ? n - 1u : c;
        c = (x[k] <= first) ? 0u : c;
        code[k] = (x[k] != x[k]) ? nan_code : c;
    }
}

}  // namespace lpmm
