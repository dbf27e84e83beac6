// Device self-test of the near-exact arithmetic in lpmm_codec.hpp against the compiler's
// correctly rounded sqrt and division.  Diagnostic only: no counterpart in the reference.
#include "lpmm_search.hpp"

namespace lpmm {

// counts[0] sqrt inputs, [1] sqrt results that differ from sqrtf, [2] of those, more than 1 ulp apart,
// [3] of those, with an input of at least 2^-100 (below that the residual underflows),
// counts[4] div pairs, [5] div_fast != x/d, [6] of those, more than 1 ulp apart,
// counts[7] div_by_rc pairs, [8] div_by_rc != x/y,
// counts[9] reciprocal inputs (every float in [2^-60, 2^60]), [10] rcp_exact != 1/y
__global__ __launch_bounds__(256) void selftest_kernel(unsigned long long *counts, uint32_t sqrt_stride,
                                                       uint64_t pairs_per_thread, uint32_t seed)
{
    unsigned long long c[11] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nthreads = (uint64_t)gridDim.x * blockDim.x;
    // every sqrt_stride-th positive normal float (stride 1: all of them)
    for (uint64_t b = 0x00800000ull + tid * sqrt_stride; b < 0x7f800000ull; b += nthreads * sqrt_stride) {
        const float x = __uint_as_float((uint32_t)b);
        const float want = sqrtf(x), got = sqrt_fast(x);
        ++c[0];
        if (got != want) {
            ++c[1];
            const int d = (int)__float_as_uint(got) - (int)__float_as_uint(want);
            if (d > 1 || d < -1)
                ++c[2];
            if (x >= 0x1p-100f)
                ++c[3];
        }
    }
    // pseudo-random pairs: divisor in [2^-40, 2^40], |quotient| in [2^-30, 2^30] for div_fast;
    // 0 <= x <= y in [2^-60, 2^60] for div_by_rc
    uint64_t s = (tid + 1) * 0x9E3779B97F4A7C15ull ^ seed;
    for (uint64_t i = 0; i < pairs_per_thread; ++i) {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        const uint32_t ym = (uint32_t)s & 0x7fffffu, xm = (uint32_t)(s >> 23) & 0x7fffffu;
        const uint32_t ye = 87u + (uint32_t)((s >> 46) % 80u), de = (uint32_t)((s >> 54) % 60u);
        const float y = __uint_as_float((ye << 23) | ym);
        const float x = __uint_as_float(((ye + 30u - de) << 23) | xm);
        ++c[4];
        const float q = div_fast(x, y), qw = x / y;
        if (q != qw) {
            ++c[5];
            const int d = (int)__float_as_uint(q) - (int)__float_as_uint(qw);
            if (d > 1 || d < -1)
                ++c[6];
        }
        const uint32_t ye2 = 67u + (uint32_t)((s >> 40) % 120u), de2 = (uint32_t)((s >> 50) % 13u);
        float y2 = __uint_as_float((ye2 << 23) | ym), x2 = __uint_as_float(((ye2 - de2) << 23) | xm);
        if (x2 > y2) {
            const float t = x2;
            x2 = y2;
            y2 = t;
        }
        ++c[7];
        if (div_by_rc(x2, y2, rcp_exact(y2)) != x2 / y2)
            ++c[8];
    }
    // the reciprocal of the group maximum: every float it is used for
    for (uint64_t b = 0x21800000ull + tid; b <= 0x5d800000ull; b += nthreads) {
        const float y = __uint_as_float((uint32_t)b);
        ++c[9];
        if (rcp_exact(y) != 1.0f / y)
            ++c[10];
    }
#pragma unroll
    for (int k = 0; k < 11; ++k)
        if (c[k])
            atomicAdd(counts + k, c[k]);
}

// ---------------------------------------------------------------------------------------
// The code assignment of the kernels, as they run it (LDS tables, saturating byte conversion,
// byte permute, median-of-three clamp), against the count of midpoints on the same device.
// counts: [0] values through encode8_plain with the standard first-moment map (every one of the
// 2^32 bit patterns, NaNs included: they must give 15), [1] wrong codes; [2], [3] the same for
// the standard second-moment map; [4] values <= 1 through the bare closed form encode8_std_v,
// [5] wrong codes; [6] values through encode8_scaled with the first-moment map, [7] wrong codes;
// [8], [9] the same with the second-moment map.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t ref_code(const Mids &mids, float x)
{
    return (x != x) ? 15u : encode_count(mids, x);
}

__device__ __forceinline__ void selftest_lds_setup(uint32_t *lds)
{
    for (uint32_t i = threadIdx.x; i < 16; i += blockDim.x) {
        lds[kLdsQ0 / 4 + i] = kStdQmapMBits[i];
        lds[kLdsQ1 / 4 + i] = kStdQmapVBits[i];
    }
    for (uint32_t i = threadIdx.x; i < (uint32_t)kEncEntries; i += blockDim.x)
        *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(lds) + kEncLdsBegin + 16 * i) = enc_entry(i);
    __syncthreads();
}

__global__ __launch_bounds__(256) void encoder_sweep_kernel(unsigned long long *counts)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    selftest_lds_setup(lds);
    const Mids mm = make_mids(reinterpret_cast<const float *>(lds) + kLdsQ0 / 4);
    const Mids mv = make_mids(reinterpret_cast<const float *>(lds) + kLdsQ1 / 4);
    unsigned long long c[6] = {0, 0, 0, 0, 0, 0};
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nthreads = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t grp = tid; grp < (1ull << 29); grp += nthreads) {  // 8 consecutive bit patterns each
        float x[8];
        bool le1 = true;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            x[k] = __uint_as_float((uint32_t)(grp * 8 + k));
            le1 = le1 && (x[k] <= 1.0f);  // false for NaN
        }
        const uint32_t wm = encode8_plain(lds, kLdsQ0, kMapStdM, x);
        const uint32_t wv = encode8_plain(lds, kLdsQ1, kMapStdV, x);
        const uint32_t wr = le1 ? encode8_std_v(x) : 0u;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            c[1] += ((wm >> (4 * k)) & 15u) != ref_code(mm, x[k]);
            c[3] += ((wv >> (4 * k)) & 15u) != ref_code(mv, x[k]);
            if (le1)
                c[5] += ((wr >> (4 * k)) & 15u) != ref_code(mv, x[k]);
        }
        c[0] += 8;
        c[2] += 8;
        if (le1)
            c[4] += 8;
    }
#pragma unroll
    for (int k = 0; k < 6; ++k)
        if (c[k])
            atomicAdd(counts + k, c[k]);
}

// Group maxima the scaled encoder is tried with: both ends of the range in which it divides by
// the corrected reciprocal (2^-60 and 2^60) with their neighbours, the cases outside it (zero,
// subnormal, huge, infinite), and pseudo-random maxima in between.
__device__ __forceinline__ float selftest_amax(uint32_t i)
{
    const uint32_t fixed[16] = {0x21800000u, 0x217fffffu, 0x21800001u, 0x5d800000u, 0x5d7fffffu, 0x5d800001u,
                                0x00000000u, 0x00000001u, 0x00800000u, 0x3f800000u, 0x7f7fffffu, 0x7f800000u,
                                0x3a83126fu, 0x358637bdu, 0x1e3ce508u, 0x60ad78ecu};
    if (i < 16)
        return __uint_as_float(fixed[i]);
    uint32_t h = i * 0x9E3779B9u;
    h ^= h >> 15; h *= 0x85EBCA6Bu; h ^= h >> 13;
    // exponent 2^-70 .. 2^70, random mantissa
    return __uint_as_float(((57u + h % 141u) << 23) | ((h >> 8) & 0x7fffffu));
}

__global__ __launch_bounds__(256) void encoder_scaled_kernel(unsigned long long *counts, uint32_t chunks)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    selftest_lds_setup(lds);
    const Mids mm = make_mids(reinterpret_cast<const float *>(lds) + kLdsQ0 / 4);
    const Mids mv = make_mids(reinterpret_cast<const float *>(lds) + kLdsQ1 / 4);
    unsigned long long c[4] = {0, 0, 0, 0};
    const float amax = selftest_amax(blockIdx.y);  // uniform over the workgroup, as over a group's lanes
    for (uint32_t chunk = blockIdx.x * blockDim.x + threadIdx.x; chunk < chunks; chunk += gridDim.x * blockDim.x) {
        float vm[8], vv[8];
        if (chunk < 15 * 32) {
            // 256 neighbouring floats around midpoint * amax, for both maps and both signs
            const uint32_t k15 = chunk / 32, sub = chunk % 32;
            const float cm = fabsf(mm.v[k15]) * amax, cv = mv.v[k15] * amax;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int off = (int)(sub % 16) * 8 + k - 64;
                float a = __uint_as_float((uint32_t)max(0, (int)__float_as_uint(cm) + off));
                float b = __uint_as_float((uint32_t)max(0, (int)__float_as_uint(cv) + off));
                a = (a <= amax) ? a : amax;  // also turns a NaN pattern into amax
                b = (b <= amax) ? b : amax;
                vm[k] = (sub >= 16) ? -a : a;
                vv[k] = b;
            }
        } else {
            uint64_t s = ((uint64_t)chunk << 20 | blockIdx.y) * 0x9E3779B97F4A7C15ull + 1;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                s ^= s << 13; s ^= s >> 7; s ^= s << 17;
                const float u = (float)(uint32_t)(s >> 40) * 0x1p-24f;  // [0, 1)
                float a = amax * u;
                a = (a <= amax) ? a : amax;
                vm[k] = (s & 1) ? -a : a;
                vv[k] = a;
            }
        }
        const uint32_t wm = encode8_scaled(lds, kLdsQ0, kMapStdM, vm, amax);
        const uint32_t wv = encode8_scaled(lds, kLdsQ1, kMapStdV, vv, amax);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            c[1] += ((wm >> (4 * k)) & 15u) != ref_code(mm, vm[k] / amax);
            c[3] += ((wv >> (4 * k)) & 15u) != ref_code(mv, vv[k] / amax);
        }
        c[0] += 8;
        c[2] += 8;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (c[k])
            atomicAdd(counts + 6 + k, c[k]);
}

// counts[0] bit patterns tried, [1] codes of the table that differ from the search's,
// [2] 1 if the map qualifies for the table (otherwise nothing is tried).  The table is built in
// LDS by the steps of the builder kernel and read back through the kernels' own look-up.
__global__ __launch_bounds__(256) void bucket_sweep_kernel(const float *__restrict__ qmap, int bits,
                                                           unsigned long long *counts)
{
    __shared__ SearchLds tree;
    __shared__ BucketLds bucket;
    const SearchFill fill = fill_search_load(qmap, bits);
    fill_search_store(tree, fill, bits);
    const BucketFill bucket_fill = fill_buckets_init(bucket, fill, bits);
    __syncthreads();
    fill_buckets_scatter(bucket, bucket_fill);
    __syncthreads();
    fill_buckets_counts(bucket, bucket_fill, bits);
    __syncthreads();
    const bool ok = buckets_ok(bucket);
    if (blockIdx.x == 0 && threadIdx.x == 0)
        counts[2] = ok ? 1ull : 0ull;
    if (!ok)
        return;
    const BucketShape s = bucket_shape(bits);
    const uint32_t nan_code = codes_per_byte(bits) == 1 ? 255u : (1u << bits) - 1u;
    unsigned long long tried = 0, wrong = 0;
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nthreads = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = tid; i < (1ull << 32); i += nthreads) {
        const float x = __uint_as_float((uint32_t)i);
        wrong += bucket_code(bucket, s, nan_code, x) != search_code(tree, bits, x);
        ++tried;
    }
    atomicAdd(counts, tried);
    if (wrong)
        atomicAdd(counts + 1, wrong);
}

}  // namespace lpmm

extern "C" int lpmm_selftest_bucket_encoder(const float *qmap, int bits, unsigned long long *counts, void *stream)
{
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(counts);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(counts, 8);
    if (!lpmm::bucket_bits_ok(bits))
        return LPMM_ERR_SIZE;
    hipLaunchKernelGGL(lpmm::bucket_sweep_kernel, dim3(8192), dim3(256), 0, (hipStream_t)stream, qmap, bits, counts);
    return lpmm::launch_status();
}

extern "C" int lpmm_selftest_encoders(unsigned long long *counts, void *stream)
{
    LPMM_REQUIRE_PTR(counts);
    LPMM_REQUIRE_ALIGN(counts, 8);
    hipLaunchKernelGGL(lpmm::encoder_sweep_kernel, dim3(8192), dim3(256), 0, (hipStream_t)stream, counts);
    int st = lpmm::launch_status();
    if (st != LPMM_OK)
        return st;
    // 256 group maxima x 2^16 chunks of 8 values
    hipLaunchKernelGGL(lpmm::encoder_scaled_kernel, dim3(64, 256), dim3(256), 0, (hipStream_t)stream, counts,
                       1u << 16);
    return lpmm::launch_status();
}

extern "C" int lpmm_selftest_arithmetic(unsigned long long *counts, uint32_t sqrt_stride, uint64_t pairs,
                                        uint32_t seed, void *stream)
{
    LPMM_REQUIRE_PTR(counts);
    LPMM_REQUIRE_ALIGN(counts, 8);
    if (sqrt_stride == 0)
        return LPMM_ERR_SIZE;
    const uint32_t blocks = 4096, threads = 256;
    const uint64_t per_thread = (pairs + (uint64_t)blocks * threads - 1) / ((uint64_t)blocks * threads);
    hipLaunchKernelGGL(lpmm::selftest_kernel, dim3(blocks), dim3(threads), 0, (hipStream_t)stream, counts, sqrt_stride,
                       per_thread, seed);
    return lpmm::launch_status();
}
