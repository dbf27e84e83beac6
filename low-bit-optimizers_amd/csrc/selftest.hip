// Device self-test of the near-exact arithmetic in lpmm_codec.hpp against the compiler's
// correctly rounded sqrt and division.  Diagnostic only: no counterpart in the reference.
#include "lpmm_codec.hpp"

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

}  // namespace lpmm

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
