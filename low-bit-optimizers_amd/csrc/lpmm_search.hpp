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
    float below, above;  // q[j-1], q[j] of thread j (j >= 1)
};

__device__ __forceinline__ SearchFill fill_search_load(const float *__restrict__ qmap, int bits)
{
    SearchFill f;
    const uint32_t n = 1u << bits, j = threadIdx.x;
    f.tree = f.mid = f.below = f.above = 0.0f;
    if (j == 0) {
        f.tree = qmap[0];
        f.mid = qmap[n - 1];
    } else if (j < n) {
        const uint32_t level = 31u - (uint32_t)__clz((int)j);
        const uint32_t k = j - (1u << level);
        f.tree = qmap[(((2u * k + 1u) << (bits - 1 - level))) - 1u];
        f.below = qmap[j - 1];
        f.above = qmap[j];
        f.mid = (f.below + f.above) * 0.5f;
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

// ---------------------------------------------------------------------------------------
// The same codes from one table look-up instead of `bits` dependent ones.
//
// With a strictly increasing map whose midpoints lie strictly between their entries, the code
// the search returns is the number of midpoints below x (for x <= q[0] none is, for
// q[N-1] <= x all are).  That is a step function of x, so a table over buckets of x that hold
// at most one step each answers with one read: entry = (steps below the bucket, position of the
// bucket's own step), code = steps + (x lies above the step).
//
// Buckets are cut from the float itself: sign, exponent and the leading M = bits - 2 mantissa
// bits for magnitudes from 2^-23 up to 1, one bucket per sign for everything smaller (zero
// included) and one for everything from 1 up.  In the order-preserving integer image of a float
// (positive: bits | 2^31, negative: ~bits) every bucket is an aligned interval of 2^(23-M)
// integers, on either side of zero, so "above the step" is one unsigned compare of the low
// 23 - M bits of that image with the step's.  create_dynamic_map(True, b - 1, b)
// (lpmm/functional.py:272-300: per decade 2^k evenly spaced values, at most 64 between 0.1 and 1
// for 8 bits) never puts two midpoints closer than a bucket is wide; whether a map qualifies --
// increasing, midpoints inside, none below 2^-23 or from 1 up in magnitude, none sharing a bucket --
// is checked while the table is filled, and a map that does not qualify is searched.
//
// The table is filled by the workgroup itself, without a search: thread j writes midpoint j (its
// rank j - 1 and its low bits) into its slot, then every thread completes a run of consecutive
// slots with the number of steps below each.
// ---------------------------------------------------------------------------------------
constexpr int kBucketOctaves = 23;
constexpr int kBucketMaxMantissa = 6;  // 8 bits
constexpr int kBucketMaxSide = kBucketOctaves * (1 << kBucketMaxMantissa) + 2;
constexpr int kBucketEntries = (2 * kBucketMaxSide + 255) / 256 * 256;  // whole runs of four per thread
constexpr uint32_t kBucketNever = 0xFFFFFFu;  // no step in the bucket: the low bits never exceed it

// entry[side + bucket] for x >= 0 and entry[side - 1 - bucket] for x < 0 (ascending in x):
// steps below the bucket << 24 | low bits of the bucket's step in the order image
struct BucketLds {
    __align__(16) uint32_t entry[kBucketEntries];
    uint32_t wave_last[16];
    uint32_t bad[16];  // per wave: something it saw disqualifies the map
};

__host__ __device__ __forceinline__ bool bucket_bits_ok(int bits) { return bits >= 3 && bits <= 8; }

struct BucketShape {
    uint32_t shift, side, key0;  // 23 - M; buckets per sign; key of the first bucket above the smallest one, less 1
};

__device__ __forceinline__ BucketShape bucket_shape(int bits)
{
    BucketShape s;
    const uint32_t m = (uint32_t)bits - 2u;
    s.shift = 23u - m;
    s.side = ((uint32_t)kBucketOctaves << m) + 2u;
    s.key0 = ((127u - (uint32_t)kBucketOctaves) << m) - 1u;
    return s;
}

// table slot of x and the low bits that are compared with the slot's step
__device__ __forceinline__ uint32_t bucket_slot(const BucketShape &s, uint32_t u, uint32_t sign)
{
    uint32_t key = (u & 0x7fffffffu) >> s.shift;
    key = min(max(key, s.key0), s.key0 + s.side - 1u) - s.key0;
    return s.side + (key ^ sign);
}

__device__ __forceinline__ uint32_t bucket_low(const BucketShape &s, uint32_t u, uint32_t sign)
{
    return (u ^ sign) & ((1u << s.shift) - 1u);
}

template <int CTRL, int ROWS>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v)
{
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROWS, 0xF, false);
    return v > o ? v : o;
}

// What thread j (1 <= j < 2^bits) contributes: the table slot of midpoint j and its entry.
struct BucketFill {
    uint32_t slot, value;
    bool mine, bad;
};

// First part (no LDS of other threads needed): the thread's midpoint from the loads of
// fill_search_load, and the thread's run of table entries set to "no step".  A barrier follows.
__device__ __forceinline__ BucketFill fill_buckets_init(BucketLds &b, const SearchFill &f, int bits)
{
    const BucketShape s = bucket_shape(bits);
    const uint32_t n = 1u << bits, j = threadIdx.x;
    BucketFill w;
    w.mine = j >= 1 && j < n;
    const float mag = fabsf(f.mid);
    // negated comparisons: a NaN anywhere disqualifies
    w.bad = w.mine && (!(f.below < f.mid) || !(f.mid < f.above) || !(mag >= __uint_as_float((127u - kBucketOctaves) << 23)) ||
                       !(mag < 1.0f));
    const uint32_t u = __float_as_uint(f.mid), sign = (uint32_t)((int32_t)u >> 31);
    w.slot = bucket_slot(s, u, sign);
    w.value = ((j - 1u) << 24) | bucket_low(s, u, sign);
    const uint32_t total = 2u * s.side;
    const uint32_t vecs = (total + 4u * blockDim.x - 1u) / (4u * blockDim.x);  // runs of four entries per thread
    const uint4 none = make_uint4(kBucketNever, kBucketNever, kBucketNever, kBucketNever);
    for (uint32_t i = 0; i < vecs; ++i) {
        const uint32_t e = (threadIdx.x * vecs + i) * 4u;
        if (e < total)
            *reinterpret_cast<uint4 *>(b.entry + e) = none;
    }
    return w;
}

// Second part: the midpoints go to their slots; a barrier follows.
__device__ __forceinline__ void fill_buckets_scatter(BucketLds &b, const BucketFill &w)
{
    if (w.mine)
        b.entry[w.slot] = w.value;
}

// Third part (contains one barrier; another one follows before buckets_ok / bucket_codes8): every
// slot without a step gets the number of steps below it -- the steps of a thread's run of slots
// are counted on the way through it, those of the runs before it come from a maximum scan over
// the workgroup (a step's entry holds its own rank, and ranks ascend with the slots).
__device__ __forceinline__ void fill_buckets_counts(BucketLds &b, BucketFill w, int bits)
{
    const BucketShape s = bucket_shape(bits);
    const uint32_t total = 2u * s.side;
    const uint32_t vecs = (total + 4u * blockDim.x - 1u) / (4u * blockDim.x);
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    // two midpoints in one slot: one of them finds the other's entry
    if (w.mine && b.entry[w.slot] != w.value)
        w.bad = true;
    constexpr int kMaxVecs = kBucketEntries / 256 / 4;
    uint4 r[kMaxVecs];
    uint32_t last = 0;  // rank + 1 of the last step in the thread's run, 0: none
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
        const uint32_t e = (threadIdx.x * vecs + i) * 4u;
        const bool live = (uint32_t)i < vecs && e < total;
        r[i] = live ? *reinterpret_cast<const uint4 *>(b.entry + e) : make_uint4(kBucketNever, kBucketNever, kBucketNever, kBucketNever);
        const uint32_t q[4] = {r[i].x, r[i].y, r[i].z, r[i].w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            last = (q[k] & 0xFFFFFFu) != kBucketNever ? (q[k] >> 24) + 1u : last;
    }
    // inclusive maximum scan over the wave: within rows of 16 lanes, then across the rows
    uint32_t inc = last;
    inc = dpp_max_u32<0x111, 0xF>(inc);  // row_shr:1
    inc = dpp_max_u32<0x112, 0xF>(inc);  // row_shr:2
    inc = dpp_max_u32<0x114, 0xF>(inc);  // row_shr:4
    inc = dpp_max_u32<0x118, 0xF>(inc);  // row_shr:8
    inc = dpp_max_u32<0x142, 0xA>(inc);  // row_bcast:15 into rows 1 and 3
    inc = dpp_max_u32<0x143, 0xC>(inc);  // row_bcast:31 into rows 2 and 3
    if (lane == kWave - 1)
        b.wave_last[wave] = inc;
    const bool wave_bad = __any(w.bad);
    if (lane == 0)
        b.bad[wave] = wave_bad;
    lds_barrier();
    // steps below the thread's run: the lane before it, and the waves before this one
    uint32_t below = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)inc, 0x138, 0xF, 0xF, false);  // wave_shr:1
    for (uint32_t v = 0; v < wave; ++v)
        below = max(below, b.wave_last[v]);
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
        const uint32_t e = (threadIdx.x * vecs + i) * 4u;
        uint32_t q[4] = {r[i].x, r[i].y, r[i].z, r[i].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const bool step = (q[k] & 0xFFFFFFu) != kBucketNever;
            q[k] = step ? q[k] : (below << 24) | kBucketNever;
            below = step ? (q[k] >> 24) + 1u : below;
        }
        if ((uint32_t)i < vecs && e < total)
            *reinterpret_cast<uint4 *>(b.entry + e) = make_uint4(q[0], q[1], q[2], q[3]);
    }
}

__device__ __forceinline__ bool buckets_ok(const BucketLds &b)
{
    uint32_t bad = 0u;
    for (uint32_t w = 0; w < (blockDim.x + kWave - 1) / kWave; ++w)
        bad |= b.bad[w];
    return __builtin_amdgcn_readfirstlane((int)bad) == 0;
}

// ---------------------------------------------------------------------------------------
// A map's table is built once (lpmm_code_table_build: one workgroup) and handed to the kernels,
// which copy it from L2 into LDS with three 16-byte loads per thread: kBucketEntries words, the
// last of which (never a slot: the table proper is shorter) tells what the builder found:
// bits << 8 | mode.
// ---------------------------------------------------------------------------------------
static_assert(2 * kBucketMaxSide < kBucketEntries, "the last word of the table is the tag");
constexpr int kCodeTableTag = kBucketEntries - 1;
enum CodeMode : uint32_t {
    kCodeSearch = 0,  // no table given, or the map does not qualify: the search
    kCodeEven = 1,    // the evenly spaced map without zero: closed form, no LDS tables at all
    kCodeTable = 2    // one table read per value
};

// The tag is read first thing in a kernel (a scalar load: uniform address) and decoded after the
// kernel's streaming loads are issued, so that they do not wait for it; a table built for another
// width counts as none.
__device__ __forceinline__ uint32_t code_table_tag(const uint32_t *__restrict__ table)
{
    return table != nullptr ? table[kCodeTableTag] : 0u;
}

__device__ __forceinline__ uint32_t code_table_mode(uint32_t tag, int bits)
{
    return (tag >> 8) == (uint32_t)bits ? (tag & 0xFFu) : (uint32_t)kCodeSearch;
}

constexpr int kCodeTableVecs = kBucketEntries / 4 / 256;  // per thread of a 256-thread workgroup

struct CodeTableRegs {
    uint4 v[kCodeTableVecs];
};

__device__ __forceinline__ CodeTableRegs code_table_load(const uint32_t *__restrict__ table)
{
    CodeTableRegs r;
#pragma unroll
    for (int i = 0; i < kCodeTableVecs; ++i)
        r.v[i] = reinterpret_cast<const uint4 *>(table)[threadIdx.x + i * 256];
    return r;
}

// the caller synchronises
__device__ __forceinline__ void code_table_store(BucketLds &b, const CodeTableRegs &r)
{
#pragma unroll
    for (int i = 0; i < kCodeTableVecs; ++i)
        reinterpret_cast<uint4 *>(b.entry)[threadIdx.x + i * 256] = r.v[i];
}

__device__ __forceinline__ uint32_t bucket_code(const BucketLds &b, const BucketShape &s, uint32_t nan_code, float x)
{
    const uint32_t u = __float_as_uint(x);
    const uint32_t sign = (uint32_t)((int32_t)u >> 31);
    const uint32_t e = b.entry[bucket_slot(s, u, sign)];
    const uint32_t code = (e >> 24) + (bucket_low(s, u, sign) > (e & 0xFFFFFFu) ? 1u : 0u);
    return (x != x) ? nan_code : code;
}

__device__ __forceinline__ void bucket_codes8(const BucketLds &b, int bits, const float (&x)[8], uint32_t (&code)[8])
{
    const BucketShape s = bucket_shape(bits);
    const uint32_t nan_code = codes_per_byte(bits) == 1 ? 255u : (1u << bits) - 1u;
#pragma unroll
    for (int k = 0; k < 8; ++k)
        code[k] = bucket_code(b, s, nan_code, x[k]);
}

// a lane's eight codes by the mode of the launch (uniform)
__device__ __forceinline__ void codes8_by_mode(uint32_t mode, const SearchLds &t, const BucketLds &b, int bits,
                                               bool even, const float (&x)[8], uint32_t (&code)[8])
{
    if (mode == kCodeTable)
        bucket_codes8(b, bits, x, code);
    else
        search_codes8(t, bits, even, x, code);
}

// one value (the code of a plain zero for the padding)
__device__ __forceinline__ uint32_t code1_by_mode(uint32_t mode, const SearchLds &t, const BucketLds &b, int bits, float x)
{
    const uint32_t n = 1u << bits;
    const uint32_t nan_code = codes_per_byte(bits) == 1 ? 255u : n - 1u;
    if (mode == kCodeTable)
        return bucket_code(b, bucket_shape(bits), nan_code, x);
    if (mode == kCodeEven) {
        const float c = fminf(fmaxf(__builtin_ceilf(__builtin_fmaf(x, (float)n, -1.5f)), 0.0f), (float)(n - 1u));
        return (x != x) ? nan_code : (uint32_t)c;
    }
    return search_code(t, bits, x);
}

}  // namespace lpmm
