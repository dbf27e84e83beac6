// Quantise / dequantise for every code width the reference's operators accept (1..8 bits),
// non-stochastic.  lpmm/cpp_extension/quantization_kernel.cu:592-601, :695-705 choose the
// storage: widths that divide 8 and are below 8 (1, 2, 4) pack 8/bits codes per byte, code j
// of a byte at bit j*bits (:430-459, :604-628); every other width (3, 5, 6, 7, 8) stores one
// code per byte (:516-533, :656-669).  Either way the packed array has one extra last byte
// (:476, :550), written as 0 here.
//
// The 4-bit kernels of quantize.hip stay the fast path for the width the optimizers use by
// default; these kernels serve the other widths (lpmm/configs/default_{5,6,7,8}b.yml).  The
// flat kernels let a lane own 8 consecutive values, a 256-thread workgroup one 2048-value pack
// group; the widths with one code per byte also have kernels in the row layout of the 4-bit
// path (further down) for whole tiles.  The map (2^bits entries) sits in LDS and the code is
// found by the reference's own search (upper bound, then the midpoint test, :397-427), so maps
// with repeated entries behave as there.
#include "lpmm_search.hpp"

namespace lpmm {

constexpr int kBThreads = 256;
constexpr int kBElts = 8;
constexpr int kBTile = kBThreads * kBElts;  // 2048

static_assert(kBThreads >= 256, "fill_search_load: one map entry per thread for up to 8 bits");

// codes of the lane's 8 values (base = index of the first, a multiple of 8) into the array
__device__ __forceinline__ void store_codes(uint8_t *__restrict__ codes, int64_t base, int bits,
                                            const uint32_t (&c)[kBElts])
{
    const int per = codes_per_byte(bits);
    if (per == 1) {
        uint2 w;
        w.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
        w.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
        *reinterpret_cast<uint2 *>(codes + base) = w;
    } else {
        uint32_t w = 0;
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            w |= c[k] << (k * bits);  // 8, 16 or 32 bits in all
        if (per == 8)
            codes[base >> 3] = (uint8_t)w;
        else if (per == 4)
            *reinterpret_cast<uint16_t *>(codes + (base >> 2)) = (uint16_t)w;
        else
            *reinterpret_cast<uint32_t *>(codes + (base >> 1)) = w;
    }
}

// map entries of the lane's 8 codes.  One code per byte: the reference indexes the map with
// the whole byte (quantization_kernel.cu:666-667), which for a 255 stored for NaN reads past a
// map of fewer than 256 entries; here the index is reduced to the map's range.
__device__ __forceinline__ void load_decode(const uint8_t *__restrict__ codes, int64_t base, int bits,
                                            const float *lds_map, float (&v)[kBElts])
{
    const int per = codes_per_byte(bits);
    const uint32_t mask = (1u << bits) - 1u;
    if (per == 1) {
        const uint2 w = *reinterpret_cast<const uint2 *>(codes + base);
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            v[k] = lds_map[(((k < 4 ? w.x : w.y) >> (8 * (k & 3))) & 0xFFu) & mask];
    } else {
        uint32_t w;
        if (per == 8)
            w = codes[base >> 3];
        else if (per == 4)
            w = *reinterpret_cast<const uint16_t *>(codes + (base >> 2));
        else
            w = *reinterpret_cast<const uint32_t *>(codes + (base >> 1));
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            v[k] = lds_map[(w >> (k * bits)) & mask];
    }
}

__device__ __forceinline__ void load_values(const float *__restrict__ x, int64_t base, int64_t n, bool vec,
                                            float (&v)[kBElts])
{
    if (vec && base + kBElts <= n) {
        const float4 a = load4(x + base), b = load4(x + base + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            v[k] = (base + k < n) ? x[base + k] : 0.0f;
    }
}

__device__ __forceinline__ void store_values(float *__restrict__ out, int64_t base, int64_t n, bool vec,
                                             const float (&v)[kBElts])
{
    if (vec && base + kBElts <= n) {
        store4(out + base, make_float4(v[0], v[1], v[2], v[3]));
        store4(out + base + 4, make_float4(v[4], v[5], v[6], v[7]));
    } else {
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            if (base + k < n)
                out[base + k] = v[k];
    }
}

// index of the extra last byte of an array of n_padded codes
__device__ __forceinline__ int64_t last_byte(int64_t n_padded, int bits) { return n_padded / codes_per_byte(bits); }

// pack_nonlinear: x holds n_padded values that are already normalised.
__global__ __launch_bounds__(kBThreads) void pack_bits_kernel(const float *__restrict__ x,
                                                              const float *__restrict__ qmap, int bits,
                                                              int64_t n_padded, uint8_t *__restrict__ out, bool vec)
{
    __shared__ SearchLds lds_map;
    fill_search(lds_map, qmap, bits);
    __syncthreads();
    const bool map_even = map_is_even(lds_map);
    const int64_t base = ((int64_t)blockIdx.x * kBThreads + threadIdx.x) * kBElts;
    if (base == 0)
        out[last_byte(n_padded, bits)] = 0;
    if (base >= n_padded)
        return;
    float v[kBElts];
    load_values(x, base, n_padded, vec, v);
    uint32_t c[kBElts];
    search_codes8(lds_map, bits, map_even, v, c);
    store_codes(out, base, bits, c);
}

// ---------------------------------------------------------------------------------------
// Stochastic rounding: pack_nonlinear(..., stochastic=True) of the reference
// (quantization_kernel.cu:418-421 for the rounding, :443-451 and :526-531 for the random
// stream).  The reference draws one curand_uniform per value from a Philox4x32-10 state that
// curand_init(seed, thread id, offset) sets up per thread, a thread handling
// work_per_thread = 4 * codes_per_byte consecutive values.  Philox is counter-based, so value i
// gets its number directly: subsequence i / work_per_thread, output number
// offset + i % work_per_thread of it -- counter {block lo, block hi, subsequence lo,
// subsequence hi} with block = output number / 4, key = the two halves of the seed, the four
// outputs of a block taken in the order x, y, z, w.
// ---------------------------------------------------------------------------------------
struct Philox4 {
    uint32_t v[4];
};

__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                 uint32_t k1)
{
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        c0 = hi1 ^ c1 ^ k0;
        c1 = lo1;
        c2 = hi0 ^ c3 ^ k1;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    Philox4 o;
    o.v[0] = c0; o.v[1] = c1; o.v[2] = c2; o.v[3] = c3;
    return o;
}

// curand_uniform: (0, 1]
__device__ __forceinline__ float philox_uniform(uint32_t u) { return (float)u * 0x1p-32f + 0x1p-33f; }

// quantize_bsearch<true>: the code as stored (NaN -> all ones, as in search_code)
__device__ __forceinline__ uint32_t search_code_sr(const float *lds_map, int bits, float x, float noise)
{
    int lo = 0, hi = 1 << bits;
    if (x <= lds_map[0])
        return 0u;
    if (lds_map[hi - 1] <= x)
        return (uint32_t)(hi - 1);
    while (lo < hi) {
        const int mi = (lo + hi) >> 1;
        if (lds_map[mi] <= x)
            lo = mi + 1;
        else
            hi = mi;
    }
    if (lo == 0)
        return codes_per_byte(bits) == 1 ? 255u : (1u << bits) - 1u;
    const float proba = (x - lds_map[lo - 1]) / (lds_map[lo] - lds_map[lo - 1]);
    const float t = (proba + noise) - 0.5f;
    const int flag = (int)__builtin_rintf(t);  // __float2int_rn
    return (uint32_t)(flag ? lo : lo - 1);
}

__global__ __launch_bounds__(kBThreads) void pack_bits_sr_kernel(const float *__restrict__ x,
                                                                 const float *__restrict__ qmap, int bits,
                                                                 int64_t n_padded, uint64_t seed, uint64_t offset,
                                                                 uint8_t *__restrict__ out, bool vec)
{
    __shared__ float lds_map[256];
    fill_map(lds_map, qmap, bits);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kBThreads + threadIdx.x) * kBElts;
    if (base == 0)
        out[last_byte(n_padded, bits)] = 0;
    if (base >= n_padded)
        return;
    float v[kBElts];
    load_values(x, base, n_padded, vec, v);
    // the lane's 8 values are two runs of 4 consecutive outputs: work_per_thread is 4, 8, 16 or
    // 32 and base a multiple of 8, so a run of 4 never straddles reference threads; it
    // straddles Philox blocks only when offset is not a multiple of 4
    const int wpt = 4 * codes_per_byte(bits);
    uint32_t c[kBElts];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint64_t i = (uint64_t)base + 4 * h;
        const uint64_t sub = i / wpt;
        const uint64_t pos = offset + (i - sub * wpt);  // output number of the run's first value
        const uint64_t blk = pos >> 2;
        const int ph = (int)(pos & 3);
        const Philox4 a = philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)sub, (uint32_t)(sub >> 32),
                                        (uint32_t)seed, (uint32_t)(seed >> 32));
        uint32_t u[4] = {a.v[0], a.v[1], a.v[2], a.v[3]};
        if (ph != 0) {  // uniform over the launch
            const uint64_t nb = blk + 1;
            const Philox4 b = philox4x32_10((uint32_t)nb, (uint32_t)(nb >> 32), (uint32_t)sub, (uint32_t)(sub >> 32),
                                            (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
            for (int k = 0; k < 4; ++k)
                u[k] = (k + ph < 4) ? a.v[(k + ph) & 3] : b.v[(k + ph) & 3];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            c[4 * h + k] = search_code_sr(lds_map, bits, v[4 * h + k], philox_uniform(u[k]));
    }
    store_codes(out, base, bits, c);
}

// unpack_nonlinear: out[i] = qmap[code_i] for i < n (n a multiple of 8).
__global__ __launch_bounds__(kBThreads) void unpack_bits_kernel(const uint8_t *__restrict__ codes,
                                                                const float *__restrict__ qmap, int bits, int64_t n,
                                                                float *__restrict__ out, bool vec)
{
    __shared__ float lds_map[256];
    fill_map(lds_map, qmap, bits);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kBThreads + threadIdx.x) * kBElts;
    if (base >= n)
        return;
    float v[kBElts];
    load_decode(codes, base, bits, lds_map, v);
    store_values(out, base, n, vec, v);
}

// 'group' scaling in one pass, any width.  THREADS as in quantize.hip's 4-bit kernel.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void quant_group_bits_kernel(const float *__restrict__ x, int64_t n,
                                                                   int rows_per_group,
                                                                   const float *__restrict__ qmap, int bits,
                                                                   uint8_t *__restrict__ codes,
                                                                   float *__restrict__ max1, int64_t n_groups,
                                                                   int64_t n_padded, bool vec)
{
    __shared__ SearchLds lds_map;
    __shared__ float s_row[THREADS / 16];
    fill_search(lds_map, qmap, bits);
    const int64_t base = ((int64_t)blockIdx.x * THREADS + threadIdx.x) * kBElts;
    if (base == 0)
        codes[last_byte(n_padded, bits)] = 0;
    float v[kBElts];
    load_values(x, base, n, vec, v);  // zero beyond n: the reference's zero padding
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kBElts; ++k)
        amax = fmaxf(amax, fabsf(v[k]));
    amax = row16_max(amax);
    if ((threadIdx.x & 15) == 0)
        s_row[threadIdx.x >> 4] = amax;
    __syncthreads();
    const bool map_even = map_is_even(lds_map);
    if (rows_per_group > 1) {
        const int first = (threadIdx.x >> 4) & ~(rows_per_group - 1);
        amax = s_row[first];
        for (int r = 1; r < rows_per_group; ++r)
            amax = fmaxf(amax, s_row[first + r]);
    }
    if (base >= n_padded)
        return;
    const int64_t gp_sz = (int64_t)rows_per_group * kGroup;
    const int64_t grp = base / gp_sz;
    uint32_t c[kBElts];
    if (grp < n_groups) {
        if ((base % gp_sz) == 0)
            max1[grp] = amax;
        // |v| <= amax: with the correctly rounded reciprocal one multiply and two fmas give the
        // correctly rounded quotient; group maxima outside the reciprocal's exact range (0 included:
        // 0/0 must give NaN) take the plain division
        float xs[kBElts];
        if (__all(rc_safe(amax))) {
            const float rc = rcp_exact(amax);
#pragma unroll
            for (int k = 0; k < kBElts; ++k)
                xs[k] = div_by_rc(v[k], amax, rc);
        } else {
#pragma unroll
            for (int k = 0; k < kBElts; ++k)
                xs[k] = v[k] / amax;
        }
        search_codes8(lds_map, bits, map_even, xs, c);
    } else {
        // padding added by the re-grouping to 2048: plain zeros, not divided by anything
        const uint32_t z = search_code(lds_map, bits, 0.0f);
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            c[k] = z;
    }
    store_codes(codes, base, bits, c);
}

__global__ __launch_bounds__(kBThreads) void dequant_group_bits_kernel(const uint8_t *__restrict__ codes,
                                                                       const float *__restrict__ max1,
                                                                       const float *__restrict__ qmap, int bits,
                                                                       int64_t n, int64_t gp_sz,
                                                                       float *__restrict__ out, bool vec)
{
    __shared__ float lds_map[256];
    fill_map(lds_map, qmap, bits);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kBThreads + threadIdx.x) * kBElts;
    if (base >= n)
        return;
    float v[kBElts];
    load_decode(codes, base, bits, lds_map, v);  // the array is padded: a whole word is always there
    const float s = max1[base / gp_sz];          // gp_sz is a multiple of 128, so uniform over the lane's 8
#pragma unroll
    for (int k = 0; k < kBElts; ++k)
        v[k] *= s;
    store_values(out, base, n, vec, v);
}

// 'rank1' scaling of a row-major R x C tensor: normalise by min(rowmax[r], colmax[c]), search,
// store.  A lane's 8 values may straddle rows.
__global__ __launch_bounds__(kBThreads) void quant_rank1_bits_kernel(const float *__restrict__ x, int64_t n,
                                                                     int64_t C, const float *__restrict__ rowmax,
                                                                     const float *__restrict__ colmax,
                                                                     const float *__restrict__ qmap, int bits,
                                                                     uint8_t *__restrict__ codes, int64_t n_padded,
                                                                     bool vec)
{
    __shared__ SearchLds lds_map;
    fill_search(lds_map, qmap, bits);
    __syncthreads();
    const bool map_even = map_is_even(lds_map);
    const int64_t base = ((int64_t)blockIdx.x * kBThreads + threadIdx.x) * kBElts;
    if (base == 0)
        codes[last_byte(n_padded, bits)] = 0;
    if (base >= n_padded)
        return;
    float v[kBElts];
    load_values(x, base, n, vec, v);
    int64_t r = base / C;
    int64_t c = base - r * C;
    float rm = (base < n) ? rowmax[r] : 0.0f;
    uint32_t code[kBElts];
    float xs[kBElts];
#pragma unroll
    for (int k = 0; k < kBElts; ++k) {
        xs[k] = 0.0f;  // padding added by the re-grouping to 2048
        if (base + k < n) {
            const float cmx = colmax[c];
            xs[k] = v[k] / ((cmx < rm) ? cmx : rm);
            if (++c == C) {
                c = 0;
                ++r;
                rm = (base + k + 1 < n) ? rowmax[r] : 0.0f;
            }
        }
    }
    search_codes8(lds_map, bits, map_even, xs, code);
    store_codes(codes, base, bits, code);
}

__global__ __launch_bounds__(kBThreads) void dequant_rank1_bits_kernel(const uint8_t *__restrict__ codes,
                                                                       const float *__restrict__ rowmax,
                                                                       const float *__restrict__ colmax,
                                                                       const float *__restrict__ qmap, int bits,
                                                                       int64_t n, int64_t C, float *__restrict__ out,
                                                                       bool vec)
{
    __shared__ float lds_map[256];
    fill_map(lds_map, qmap, bits);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kBThreads + threadIdx.x) * kBElts;
    if (base >= n)
        return;
    float v[kBElts];
    load_decode(codes, base, bits, lds_map, v);
    int64_t r = base / C;
    int64_t c = base - r * C;
    float rm = rowmax[r];
#pragma unroll
    for (int k = 0; k < kBElts; ++k) {
        if (base + k < n) {
            const float cmx = colmax[c];
            v[k] *= (cmx < rm) ? cmx : rm;
            if (++c == C) {
                c = 0;
                ++r;
                rm = (base + k + 1 < n) ? rowmax[r] : 0.0f;
            }
        }
    }
    store_values(out, base, n, vec, v);
}

// ---------------------------------------------------------------------------------------
// Row layout for the widths that store one code per byte (3, 5, 6, 7, 8 bits): as in the 4-bit
// kernels of quantize.hip, 16 lanes (one DPP row) own 128 consecutive values, lane l the values
// [4l, 4l+4) and [64+4l, 64+4l+4), so that every 16-byte access of a row covers whole cache
// lines and a lane's codes are two aligned 4-byte words.  These kernels take the part of a
// tensor that consists of whole 2048-value tiles (whole 128-value groups for the dequantiser);
// the flat kernels above take the rest and every packed width.
// ---------------------------------------------------------------------------------------
#ifndef LPMM_BROWS_T
#define LPMM_BROWS_T 2
#endif
constexpr int kBRowsT = LPMM_BROWS_T;       // tiles (passes of 16 groups) per workgroup: loads first, map afterwards
constexpr int kBRank1Rows = 4;   // rows of one 2048-column chunk per workgroup of the rank-1 kernels

__device__ __forceinline__ uint32_t bytes4(uint32_t a, uint32_t b, uint32_t c, uint32_t d)
{
    return a | (b << 8) | (c << 16) | (d << 24);
}

__device__ __forceinline__ void unpack8(const float4 &a, const float4 &b, float (&o)[kBElts])
{
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}

__device__ __forceinline__ void decode_bytes(uint32_t w0, uint32_t w1, uint32_t mask, const float *lds_map,
                                             float (&v)[kBElts])
{
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        v[k] = lds_map[((w0 >> (8 * k)) & 0xFFu) & mask];
        v[4 + k] = lds_map[((w1 >> (8 * k)) & 0xFFu) & mask];
    }
}

// Builds the code table of a map (lpmm_search.hpp): one workgroup of 256 threads.
__global__ __launch_bounds__(256) void code_table_kernel(const float *__restrict__ qmap, int bits,
                                                         uint32_t *__restrict__ table)
{
    __shared__ SearchLds tree;
    __shared__ BucketLds bucket;
    const SearchFill fill = fill_search_load(qmap, bits);
    fill_search_store(tree, fill, bits);
    uint32_t mode = kCodeSearch, total = 0;
    if (bucket_bits_ok(bits)) {  // uniform
        const BucketFill bucket_fill = fill_buckets_init(bucket, fill, bits);
        __syncthreads();
        fill_buckets_scatter(bucket, bucket_fill);
        __syncthreads();
        fill_buckets_counts(bucket, bucket_fill, bits);
        __syncthreads();
        total = 2u * bucket_shape(bits).side;
        mode = buckets_ok(bucket) ? kCodeTable : kCodeSearch;
    } else {
        __syncthreads();
    }
    if (map_is_even(tree))
        mode = kCodeEven;
    for (uint32_t i = threadIdx.x; i < (uint32_t)kBucketEntries; i += blockDim.x)
        table[i] = i == (uint32_t)kCodeTableTag ? ((uint32_t)bits << 8) | mode : (mode == kCodeTable && i < total ? bucket.entry[i] : 0u);
}

template <int T>
__global__ __launch_bounds__(kBThreads) void quant_group_bits_rows_kernel(const float *__restrict__ x,
                                                                          int64_t full_tiles, int rows_per_group,
                                                                          const float *__restrict__ qmap, int bits,
                                                                          const uint32_t *__restrict__ table,
                                                                          uint8_t *__restrict__ codes,
                                                                          float *__restrict__ max1, int64_t trailing)
{
    __shared__ SearchLds lds_map;
    __shared__ BucketLds lds_bucket;
    __shared__ float s_row[T][kBThreads / 16];
    const int lane16 = threadIdx.x & 15, wrow = threadIdx.x >> 4;
    const int64_t tile0 = (int64_t)blockIdx.x * T;
    // the small loads that feed LDS first (they return first), then the tiles' loads
    const uint32_t tag = code_table_tag(table);
    SearchFill fill;
    if (table == nullptr)
        fill = fill_search_load(qmap, bits);
    float v[T][kBElts];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f), b = a;
        if (tile0 + t < full_tiles) {  // uniform over the workgroup
            const float *p = x + (tile0 + t) * kBTile + wrow * kGroup + lane16 * 4;
            a = load4(p);
            b = load4(p + 64);
        }
        unpack8(a, b, v[t]);
    }
    const uint32_t mode = code_table_mode(tag, bits);
    if (mode == kCodeTable) {
        code_table_store(lds_bucket, code_table_load(table));
    } else if (mode == kCodeSearch) {
        if (table != nullptr)  // a table that says "search"
            fill = fill_search_load(qmap, bits);
        fill_search_store(lds_map, fill, bits);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0)
        codes[trailing] = 0;
    float amax[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        float m = 0.0f;
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            m = fmaxf(m, fabsf(v[t][k]));
        amax[t] = row16_max(m);
        if (lane16 == 0)
            s_row[t][wrow] = amax[t];
    }
    lds_barrier();
    const bool map_even = mode == kCodeEven || (mode == kCodeSearch && map_is_even(lds_map));
    const int first = wrow & ~(rows_per_group - 1);
    const int64_t gp_sz = (int64_t)rows_per_group * kGroup;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (tile0 + t >= full_tiles)
            break;
        if (rows_per_group > 1) {
            amax[t] = s_row[t][first];
            for (int r = 1; r < rows_per_group; ++r)
                amax[t] = fmaxf(amax[t], s_row[t][first + r]);
        }
        const int64_t base = (tile0 + t) * kBTile + wrow * kGroup;
        if ((base % gp_sz) == 0 && lane16 == 0)
            max1[base / gp_sz] = amax[t];
        float xs[kBElts];
        if (__all(rc_safe(amax[t]))) {
            const float rc = rcp_exact(amax[t]);
#pragma unroll
            for (int k = 0; k < kBElts; ++k)
                xs[k] = div_by_rc(v[t][k], amax[t], rc);
        } else {
#pragma unroll
            for (int k = 0; k < kBElts; ++k)
                xs[k] = v[t][k] / amax[t];
        }
        uint32_t c[kBElts];
        codes8_by_mode(mode, lds_map, lds_bucket, bits, map_even, xs, c);
        uint32_t *cp = reinterpret_cast<uint32_t *>(codes + base) + lane16;
        store_u32(cp, bytes4(c[0], c[1], c[2], c[3]));
        store_u32(cp + 16, bytes4(c[4], c[5], c[6], c[7]));
    }
}

template <int T>
__global__ __launch_bounds__(kBThreads) void dequant_group_bits_rows_kernel(const uint8_t *__restrict__ codes,
                                                                            const float *__restrict__ max1,
                                                                            const float *__restrict__ qmap, int bits,
                                                                            int64_t full_groups, int64_t rows_per_group,
                                                                            float *__restrict__ out)
{
    __shared__ float lds_map[256];
    const int lane16 = threadIdx.x & 15;
    const int64_t row0 = (int64_t)blockIdx.x * T * (kBThreads / 16) + (threadIdx.x >> 4);
    uint32_t w0[T], w1[T];
    float s[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int64_t row = row0 + t * (kBThreads / 16);
        w0[t] = w1[t] = 0;
        s[t] = 0.0f;
        if (row < full_groups) {
            const uint32_t *cp = reinterpret_cast<const uint32_t *>(codes + row * kGroup) + lane16;
            w0[t] = load_u32(cp);
            w1[t] = load_u32(cp + 16);
            s[t] = max1[row / rows_per_group];
        }
    }
    fill_map(lds_map, qmap, bits);
    lds_barrier();
    const uint32_t mask = (1u << bits) - 1u;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int64_t row = row0 + t * (kBThreads / 16);
        if (row >= full_groups)
            continue;
        float v[kBElts];
        decode_bytes(w0[t], w1[t], mask, lds_map, v);
        float *o = out + row * kGroup + lane16 * 4;
        store4(o, make_float4(v[0] * s[t], v[1] * s[t], v[2] * s[t], v[3] * s[t]));
        store4(o + 64, make_float4(v[4] * s[t], v[5] * s[t], v[6] * s[t], v[7] * s[t]));
    }
}

// 'rank1' scaling, columns a multiple of 128: grid (2048-column chunks, groups of kBRank1Rows
// rows).  A lane keeps the maxima of its 8 columns, and their correctly rounded reciprocals,
// over the rows of its workgroup; x / min(rowmax, colmax) is then one multiply and two fmas that
// give the correctly rounded quotient (|x| <= scale by construction) wherever all the scales of
// the wave lie in the range in which the reciprocal is exact, and the plain division otherwise.
__global__ __launch_bounds__(kBThreads) void quant_rank1_bits_rows128_kernel(const float *__restrict__ x, int64_t R,
                                                                             int64_t C,
                                                                             const float *__restrict__ rowmax,
                                                                             const float *__restrict__ colmax,
                                                                             const float *__restrict__ qmap, int bits,
                                                                             const uint32_t *__restrict__ table,
                                                                             uint8_t *__restrict__ codes,
                                                                             int64_t n_padded)
{
    constexpr int T = kBRank1Rows;
    __shared__ SearchLds lds_map;
    __shared__ BucketLds lds_bucket;
    const uint32_t tag = code_table_tag(table);
    const int64_t n = R * C;
    const int lane16 = threadIdx.x & 15;
    const int64_t r0 = (int64_t)blockIdx.y * T;
    const int64_t c0 = (int64_t)blockIdx.x * kBTile + (int64_t)(threadIdx.x >> 4) * kGroup;
    const bool live = c0 < C;  // uniform over the 16 lanes of a group
    // the small loads that feed LDS first (they return first), then the rows' loads
    SearchFill fill;
    if (table == nullptr)
        fill = fill_search_load(qmap, bits);
    float4 a[T], b[T], ca, cb;
    float rm[T];
    if (live) {
        const float *cmp = colmax + c0 + lane16 * 4;
        ca = *reinterpret_cast<const float4 *>(cmp);
        cb = *reinterpret_cast<const float4 *>(cmp + 64);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            if (r0 + t < R) {
                const float *p = x + (r0 + t) * C + c0 + lane16 * 4;
                a[t] = load4(p);
                b[t] = load4(p + 64);
                rm[t] = rowmax[r0 + t];
            }
        }
    }
    const uint32_t mode = code_table_mode(tag, bits);
    if (mode == kCodeTable) {
        code_table_store(lds_bucket, code_table_load(table));
    } else if (mode == kCodeSearch) {
        if (table != nullptr)  // a table that says "search"
            fill = fill_search_load(qmap, bits);
        fill_search_store(lds_map, fill, bits);
    }
    lds_barrier();
    const bool map_even = mode == kCodeEven || (mode == kCodeSearch && map_is_even(lds_map));
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        // the padding added by the re-grouping to 2048: plain zeros, not divided by anything
        const uint32_t z = code1_by_mode(mode, lds_map, lds_bucket, bits, 0.0f);
        const uint32_t wz = bytes4(z, z, z, z);
        for (int64_t i = n + (int64_t)threadIdx.x * 4; i < n_padded; i += kBThreads * 4)
            *reinterpret_cast<uint32_t *>(codes + i) = wz;
        if (threadIdx.x == 0)
            codes[n_padded] = 0;
    }
    if (!live)
        return;
    float cmx[kBElts], crc[kBElts];
    unpack8(ca, cb, cmx);
    bool cols_safe = true;
#pragma unroll
    for (int k = 0; k < kBElts; ++k) {
        crc[k] = rcp_exact(cmx[k]);
        cols_safe = cols_safe && rc_safe(cmx[k]);
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (r0 + t >= R)
            break;
        float v[kBElts], xs[kBElts];
        unpack8(a[t], b[t], v);
        if (__all(cols_safe && rc_safe(rm[t]))) {
            const float rr = rcp_exact(rm[t]);
#pragma unroll
            for (int k = 0; k < kBElts; ++k) {
                const bool by_col = cmx[k] < rm[t];
                xs[k] = div_by_rc(v[k], by_col ? cmx[k] : rm[t], by_col ? crc[k] : rr);
            }
        } else {
#pragma unroll
            for (int k = 0; k < kBElts; ++k)
                xs[k] = v[k] / ((cmx[k] < rm[t]) ? cmx[k] : rm[t]);
        }
        uint32_t c[kBElts];
        codes8_by_mode(mode, lds_map, lds_bucket, bits, map_even, xs, c);
        uint32_t *cp = reinterpret_cast<uint32_t *>(codes + (r0 + t) * C + c0) + lane16;
        store_u32(cp, bytes4(c[0], c[1], c[2], c[3]));
        store_u32(cp + 16, bytes4(c[4], c[5], c[6], c[7]));
    }
}

__global__ __launch_bounds__(kBThreads) void dequant_rank1_bits_rows128_kernel(const uint8_t *__restrict__ codes,
                                                                               const float *__restrict__ rowmax,
                                                                               const float *__restrict__ colmax,
                                                                               const float *__restrict__ qmap, int bits,
                                                                               int64_t R, int64_t C,
                                                                               float *__restrict__ out)
{
    constexpr int T = kBRank1Rows;
    __shared__ float lds_map[256];
    const int lane16 = threadIdx.x & 15;
    const int64_t r0 = (int64_t)blockIdx.y * T;
    const int64_t c0 = (int64_t)blockIdx.x * kBTile + (int64_t)(threadIdx.x >> 4) * kGroup;
    const bool live = c0 < C;
    uint32_t w0[T], w1[T];
    float rm[T];
    float4 ca, cb;
    if (live) {
        const float *cmp = colmax + c0 + lane16 * 4;
        ca = *reinterpret_cast<const float4 *>(cmp);
        cb = *reinterpret_cast<const float4 *>(cmp + 64);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            if (r0 + t < R) {
                const uint32_t *cp = reinterpret_cast<const uint32_t *>(codes + (r0 + t) * C + c0) + lane16;
                w0[t] = load_u32(cp);
                w1[t] = load_u32(cp + 16);
                rm[t] = rowmax[r0 + t];
            }
        }
    }
    fill_map(lds_map, qmap, bits);
    lds_barrier();
    if (!live)
        return;
    float cmx[kBElts];
    unpack8(ca, cb, cmx);
    const uint32_t mask = (1u << bits) - 1u;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (r0 + t >= R)
            break;
        float v[kBElts];
        decode_bytes(w0[t], w1[t], mask, lds_map, v);
#pragma unroll
        for (int k = 0; k < kBElts; ++k)
            v[k] *= (cmx[k] < rm[t]) ? cmx[k] : rm[t];
        float *o = out + (r0 + t) * C + c0 + lane16 * 4;
        store4(o, make_float4(v[0], v[1], v[2], v[3]));
        store4(o + 64, make_float4(v[4], v[5], v[6], v[7]));
    }
}

// rank-1 row kernels: one code per byte, columns a multiple of 128, aligned operands, rows fit grid.y
inline bool rank1_bits_rows_ok(int bits, const void *x, const void *colmax, const void *codes, int64_t rows,
                               int64_t cols)
{
    return codes_per_byte(bits) == 1 && (cols % kGroup) == 0 && rows <= 65535LL * kBRank1Rows &&
           (cols + kBTile - 1) / kBTile <= 0x7fffffffLL && aligned_to(x, 16) && aligned_to(colmax, 16) &&
           aligned_to(codes, 4);
}

inline bool bits_ok(int bits) { return bits >= 1 && bits <= 8; }

inline bool tiles_for(int64_t n, uint32_t *tiles)
{
    const int64_t t = (n + kBTile - 1) / kBTile;
    if (t > 0x7fffffffLL)
        return false;
    *tiles = (uint32_t)t;
    return true;
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_pack_nonlinear(const float *x, const float *qmap, int bits, int64_t n_padded, uint8_t *out,
                                   void *stream)
{
    if (!bits_ok(bits) || n_padded <= 0 || (n_padded % 8) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 8);
    uint32_t tiles;
    if (!tiles_for(n_padded, &tiles))
        return LPMM_ERR_SIZE;
    hipLaunchKernelGGL(pack_bits_kernel, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream, x, qmap, bits,
                       n_padded, out, aligned_to(x, 16));
    return launch_status();
}

extern "C" int lpmm_pack_nonlinear_sr(const float *x, const float *qmap, int bits, int64_t n_padded,
                                      uint64_t seed, uint64_t offset, uint8_t *out, void *stream)
{
    // a reference thread handles up to 32 values (1-bit codes): whole threads only
    if (!bits_ok(bits) || n_padded <= 0 || (n_padded % 32) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 8);
    uint32_t tiles;
    if (!tiles_for(n_padded, &tiles))
        return LPMM_ERR_SIZE;
    hipLaunchKernelGGL(pack_bits_sr_kernel, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream, x, qmap, bits,
                       n_padded, seed, offset, out, aligned_to(x, 16));
    return launch_status();
}

extern "C" int lpmm_unpack_nonlinear(const uint8_t *codes, const float *qmap, int bits, int64_t n, float *out,
                                     void *stream)
{
    if (!bits_ok(bits) || n <= 0 || (n % 8) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(codes, 8);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 4);
    uint32_t tiles;
    if (!tiles_for(n, &tiles))
        return LPMM_ERR_SIZE;
    hipLaunchKernelGGL(unpack_bits_kernel, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream, codes, qmap, bits,
                       n, out, aligned_to(out, 16));
    return launch_status();
}

extern "C" int lpmm_code_table_build(const float *qmap, int bits, void *table, void *stream)
{
    if (!bits_ok(bits))
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(table);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(table, 16);
    static_assert(LPMM_CODE_TABLE_BYTES == kBucketEntries * 4, "the header's size of a code table");
    hipLaunchKernelGGL(code_table_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, qmap, bits,
                       static_cast<uint32_t *>(table));
    return launch_status();
}

extern "C" int lpmm_quant_group_bits(const float *x, int64_t n, int64_t gp_sz, const float *qmap, int bits,
                                     uint8_t *codes, float *max1, void *stream)
{
    return lpmm_quant_group_bits_table(x, n, gp_sz, qmap, bits, nullptr, codes, max1, stream);
}

extern "C" int lpmm_quant_group_bits_table(const float *x, int64_t n, int64_t gp_sz, const float *qmap, int bits,
                                           const void *table, uint8_t *codes, float *max1, void *stream)
{
    if (!bits_ok(bits) || n <= 0)
        return LPMM_ERR_SIZE;
    if (table != nullptr)
        LPMM_REQUIRE_ALIGN(table, 16);
    if (gp_sz < kGroup || gp_sz > 2 * kBTile || (gp_sz & (gp_sz - 1)) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(max1);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(max1, 4);
    LPMM_REQUIRE_ALIGN(codes, 8);
    const int64_t n_groups = (n + gp_sz - 1) / gp_sz;
    uint32_t tiles;
    if (!tiles_for(n_groups * gp_sz, &tiles))
        return LPMM_ERR_SIZE;
    const int64_t n_padded = (int64_t)tiles * kBTile;
    hipStream_t s = (hipStream_t)stream;
    const int64_t full_tiles = n / kBTile;
    if (codes_per_byte(bits) == 1 && gp_sz <= kBTile && full_tiles > 0 && aligned_to(x, 16)) {
        // whole tiles in the row layout, the ragged end and the padding by the flat kernel
        const uint32_t wgs = (uint32_t)((full_tiles + kBRowsT - 1) / kBRowsT);
        hipLaunchKernelGGL(quant_group_bits_rows_kernel<kBRowsT>, dim3(wgs), dim3(kBThreads), 0, s, x, full_tiles,
                           (int)(gp_sz / kGroup), qmap, bits, static_cast<const uint32_t *>(table), codes, max1,
                           n_padded);
        const int64_t done = full_tiles * kBTile;
        if (done < n_padded)
            hipLaunchKernelGGL(quant_group_bits_kernel<kBThreads>, dim3((uint32_t)((n_padded - done) / kBTile)),
                               dim3(kBThreads), 0, s, x + done, n - done, (int)(gp_sz / kGroup), qmap, bits,
                               codes + done, max1 + done / gp_sz, n_groups - done / gp_sz, n_padded - done, true);
        return launch_status();
    }
    if (gp_sz > kBTile)
        hipLaunchKernelGGL(quant_group_bits_kernel<2 * kBThreads>, dim3((tiles + 1) / 2), dim3(2 * kBThreads), 0,
                           (hipStream_t)stream, x, n, (int)(gp_sz / kGroup), qmap, bits, codes, max1, n_groups,
                           n_padded, aligned_to(x, 16));
    else
        hipLaunchKernelGGL(quant_group_bits_kernel<kBThreads>, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream,
                           x, n, (int)(gp_sz / kGroup), qmap, bits, codes, max1, n_groups, n_padded,
                           aligned_to(x, 16));
    return launch_status();
}

extern "C" int lpmm_dequant_group_bits(const uint8_t *codes, const float *max1, const float *qmap, int bits,
                                       int64_t n, int64_t gp_sz, float *out, void *stream)
{
    if (!bits_ok(bits) || n <= 0 || gp_sz < kGroup || (gp_sz % kGroup) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(max1);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(codes, 8);
    LPMM_REQUIRE_ALIGN(max1, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 4);
    uint32_t tiles;
    if (!tiles_for(n, &tiles))
        return LPMM_ERR_SIZE;
    const int64_t full_groups = n / kGroup;
    if (codes_per_byte(bits) == 1 && full_groups > 0 && aligned_to(out, 16)) {
        constexpr int64_t per_wg = (int64_t)kBRowsT * (kBThreads / 16);
        hipLaunchKernelGGL(dequant_group_bits_rows_kernel<kBRowsT>, dim3((uint32_t)((full_groups + per_wg - 1) / per_wg)),
                           dim3(kBThreads), 0, (hipStream_t)stream, codes, max1, qmap, bits, full_groups,
                           gp_sz / kGroup, out);
        const int64_t done = full_groups * kGroup;
        if (done < n)  // fewer than 128 values, all in the group of value `done`
            hipLaunchKernelGGL(dequant_group_bits_kernel, dim3(1), dim3(kBThreads), 0, (hipStream_t)stream,
                               codes + done, max1 + done / gp_sz, qmap, bits, n - done, gp_sz, out + done, false);
        return launch_status();
    }
    hipLaunchKernelGGL(dequant_group_bits_kernel, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream, codes, max1,
                       qmap, bits, n, gp_sz, out, aligned_to(out, 16));
    return launch_status();
}

extern "C" int lpmm_quant_rank1_bits(const float *x, int64_t rows, int64_t cols, const float *rowmax,
                                     const float *colmax, const float *qmap, int bits, uint8_t *codes,
                                     void *stream)
{
    return lpmm_quant_rank1_bits_table(x, rows, cols, rowmax, colmax, qmap, bits, nullptr, codes, stream);
}

extern "C" int lpmm_quant_rank1_bits_table(const float *x, int64_t rows, int64_t cols, const float *rowmax,
                                           const float *colmax, const float *qmap, int bits, const void *table,
                                           uint8_t *codes, void *stream)
{
    if (!bits_ok(bits) || rows <= 0 || cols <= 0 || rows > INT64_MAX / cols)
        return LPMM_ERR_SIZE;
    if (table != nullptr)
        LPMM_REQUIRE_ALIGN(table, 16);
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(rowmax);
    LPMM_REQUIRE_PTR(colmax);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(rowmax, 4);
    LPMM_REQUIRE_ALIGN(colmax, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(codes, 8);
    const int64_t n = rows * cols;
    uint32_t tiles;
    if (!tiles_for(n, &tiles))
        return LPMM_ERR_SIZE;
    if (rank1_bits_rows_ok(bits, x, colmax, codes, rows, cols)) {
        const dim3 grid((uint32_t)((cols + kBTile - 1) / kBTile), (uint32_t)((rows + kBRank1Rows - 1) / kBRank1Rows));
        hipLaunchKernelGGL(quant_rank1_bits_rows128_kernel, grid, dim3(kBThreads), 0, (hipStream_t)stream, x, rows, cols,
                           rowmax, colmax, qmap, bits, static_cast<const uint32_t *>(table), codes,
                           (int64_t)tiles * kBTile);
        return launch_status();
    }
    hipLaunchKernelGGL(quant_rank1_bits_kernel, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream, x, n, cols,
                       rowmax, colmax, qmap, bits, codes, (int64_t)tiles * kBTile, aligned_to(x, 16));
    return launch_status();
}

extern "C" int lpmm_dequant_rank1_bits(const uint8_t *codes, const float *rowmax, const float *colmax,
                                       const float *qmap, int bits, int64_t rows, int64_t cols, float *out,
                                       void *stream)
{
    if (!bits_ok(bits) || rows <= 0 || cols <= 0 || rows > INT64_MAX / cols)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(rowmax);
    LPMM_REQUIRE_PTR(colmax);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(codes, 8);
    LPMM_REQUIRE_ALIGN(rowmax, 4);
    LPMM_REQUIRE_ALIGN(colmax, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 4);
    const int64_t n = rows * cols;
    uint32_t tiles;
    if (!tiles_for(n, &tiles))
        return LPMM_ERR_SIZE;
    if (rank1_bits_rows_ok(bits, out, colmax, codes, rows, cols)) {
        const dim3 grid((uint32_t)((cols + kBTile - 1) / kBTile), (uint32_t)((rows + kBRank1Rows - 1) / kBRank1Rows));
        hipLaunchKernelGGL(dequant_rank1_bits_rows128_kernel, grid, dim3(kBThreads), 0, (hipStream_t)stream, codes,
                           rowmax, colmax, qmap, bits, rows, cols, out);
        return launch_status();
    }
    hipLaunchKernelGGL(dequant_rank1_bits_kernel, dim3(tiles), dim3(kBThreads), 0, (hipStream_t)stream, codes, rowmax,
                       colmax, qmap, bits, n, cols, out, aligned_to(out, 16));
    return launch_status();
}
