// 'rank1' scaling of tensors with more than two dimensions (lpmm/functional.py:190-203 with
// get_sm3_statistics :512-531 and _compute_sm3_scale_tensor :503-509 of the reference).
//
// For a contiguous tensor of shape (d_0, ..., d_{k}) the statistics are, for every dimension i,
// stat_i[j] = max |x| over all elements whose i-th index is j, and an element is scaled by the
// smallest of its k+1 statistics.  The reference gets them from k * (k+1) PyTorch reductions of
// |x| and a chain of broadcast minima.  Here:
//
//   * rank1_fold_nd_kernel reads its input once.  A workgroup takes 2048 consecutive elements.
//     Along dimension i (stride s_i) those elements touch at most min(d_i, 2047 / s_i + 2)
//     consecutive (cyclically) indices, so a workgroup keeps one LDS slot per touched index and
//     dimension (fewer than 4096 in all for up to 8 dimensions), takes maxima there with LDS
//     atomics and afterwards sends every non-zero slot to the global statistics with one
//     atomic each.  Maxima of non-negative floats are maxima of their bit patterns, so integer
//     atomics do; a NaN has the largest pattern and survives, as it does in torch.max.  A wave
//     whose 256 values share one index (every dimension whose stride is 256 or more, for
//     most waves) reduces across its lanes first and issues one LDS atomic.
//   * When the last dimension is long, the 2-D kernel of quantize.hip computes its statistics
//     and the maxima of the rows of the (d_0 * ... * d_{k-1}) x d_k view at its own streaming
//     rate, and the fold kernel only runs over those row maxima with the leading dimensions.
//   * rank1_row_scale_nd_kernel writes, for every row of that 2-D view, the minimum of the
//     leading dimensions' statistics.  With that array as `rowmax` and stat_k as `colmax` the
//     2-D quantise / dequantise kernels (any code width) serve the N-D tensor unchanged:
//     min(min(leading statistics), stat_k) is the reference's scale.
#include "lpmm_common.hpp"

namespace lpmm {

constexpr int kNdMax = LPMM_RANK1_ND_MAX;
constexpr int kNdThreads = 256;
constexpr int kNdTile = 2048;
constexpr int kNdSlots = 4096;

struct NdDims {
    int64_t n;  // elements = product of dim[0..ndim)
    int64_t dim[kNdMax];
    int64_t stride[kNdMax];  // contiguous strides in elements
    float *stat[kNdMax];
    int32_t ndim;
};

__global__ __launch_bounds__(256) void nd_zero_kernel(NdDims sh)
{
    const int i = blockIdx.y;
    const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (j < sh.dim[i])
        sh.stat[i][j] = 0.0f;
}

__device__ __forceinline__ uint32_t wave_umax(uint32_t v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t w = (uint32_t)__shfl_xor((int)v, o, 64);
        v = w > v ? w : v;
    }
    return v;
}

__device__ __forceinline__ uint32_t abs_bits(float v) { return __float_as_uint(v) & 0x7fffffffu; }

__global__ __launch_bounds__(kNdThreads) void rank1_fold_nd_kernel(const float *__restrict__ x, NdDims sh, bool vec)
{
    __shared__ uint32_t s_slot[kNdSlots];
    __shared__ int64_t s_rem0[kNdMax];   // (first element of the tile) mod stride
    __shared__ int64_t s_first[kNdMax];  // index along the dimension of the tile's first element
    __shared__ uint32_t s_cnt[kNdMax];   // slots of the dimension
    __shared__ uint32_t s_base[kNdMax + 1];
    __shared__ uint32_t s_wrap[kNdMax];  // the tile touches every index of the dimension: slot = index
    const int64_t start = (int64_t)blockIdx.x * kNdTile;
    const int64_t stop = (start + kNdTile < sh.n) ? start + kNdTile : sh.n;
    if (threadIdx.x == 0) {
        uint32_t base = 0;
        for (int i = 0; i < sh.ndim; ++i) {
            const int64_t s = sh.stride[i], d = sh.dim[i];
            const int64_t q0 = start / s, q1 = (stop - 1) / s;
            const int64_t span = q1 - q0 + 1;
            const bool wrap = span >= d;
            s_rem0[i] = start - q0 * s;
            s_first[i] = q0 % d;
            s_cnt[i] = (uint32_t)(wrap ? d : span);
            s_wrap[i] = wrap ? 1u : 0u;
            s_base[i] = base;
            base += s_cnt[i];
        }
        s_base[sh.ndim] = base;
    }
    __syncthreads();
    const uint32_t used = s_base[sh.ndim];  // <= kNdSlots: checked on the host
    for (uint32_t j = threadIdx.x; j < used; j += kNdThreads)
        s_slot[j] = 0;
    __syncthreads();

    const uint32_t lane = threadIdx.x & 63u;
#pragma unroll 1
    for (int h = 0; h < 2; ++h) {
        const uint32_t r = h * (kNdTile / 2) + threadIdx.x * 4;
        const int64_t e = start + r;
        const bool full = e + 4 <= stop;
        uint32_t u[4];
        if (full && vec) {
            const float4 a = *reinterpret_cast<const float4 *>(x + e);
            u[0] = abs_bits(a.x); u[1] = abs_bits(a.y); u[2] = abs_bits(a.z); u[3] = abs_bits(a.w);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                u[k] = (e + k < stop) ? abs_bits(x[e + k]) : 0u;
        }
        uint32_t um = u[0] > u[1] ? u[0] : u[1];
        um = u[2] > um ? u[2] : um;
        um = u[3] > um ? u[3] : um;
#pragma unroll 1
        for (int i = 0; i < sh.ndim; ++i) {
            const int64_t s = sh.stride[i];
            const bool wide = s > 0x7fffffffLL;  // then at most one index change inside the tile
            const uint32_t s32 = (uint32_t)s;
            const int64_t t = s_rem0[i] + r;     // < s + 2048
            const bool wrap = s_wrap[i] != 0;
            const uint32_t d32 = (uint32_t)sh.dim[i], first32 = (uint32_t)s_first[i];  // used when wrap: d <= 2049
            const uint32_t base = s_base[i];
            uint32_t dqa, dqb;  // index steps since the tile's first element, of the lane's first and last value
            if (wide) {
                dqa = t >= s ? 1u : 0u;
                dqb = t + 3 >= s ? 1u : 0u;
            } else if (s32 == 1u) {
                dqa = (uint32_t)t;
                dqb = (uint32_t)t + 3u;
            } else {
                dqa = (uint32_t)t / s32;
                dqb = ((uint32_t)t + 3u) / s32;
            }
            const bool same = full && dqa == dqb;
            const uint32_t lead = (uint32_t)__builtin_amdgcn_readfirstlane((int)dqa);
            if (__all(same && dqa == lead)) {
                const uint32_t w = wave_umax(um);
                if (lane == 0)
                    atomicMax(&s_slot[base + (wrap ? (first32 + lead) % d32 : lead)], w);
            } else if (same) {
                atomicMax(&s_slot[base + (wrap ? (first32 + dqa) % d32 : dqa)], um);
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (e + k < stop) {
                        uint32_t dq;
                        if (wide)
                            dq = t + k >= s ? 1u : 0u;
                        else if (s32 == 1u)
                            dq = (uint32_t)t + k;
                        else
                            dq = ((uint32_t)t + k) / s32;
                        atomicMax(&s_slot[base + (wrap ? (first32 + dq) % d32 : dq)], u[k]);
                    }
                }
            }
        }
    }
    __syncthreads();
#pragma unroll 1
    for (int i = 0; i < sh.ndim; ++i) {
        const uint32_t cnt = s_cnt[i], base = s_base[i];
        const bool wrap = s_wrap[i] != 0;
        const int64_t first = s_first[i], d = sh.dim[i];
        unsigned int *out = reinterpret_cast<unsigned int *>(sh.stat[i]);
        for (uint32_t j = threadIdx.x; j < cnt; j += kNdThreads) {
            const uint32_t v = s_slot[base + j];
            if (v != 0u) {
                int64_t idx = wrap ? (int64_t)j : first + j;
                idx = idx >= d ? idx - d : idx;
                atomicMax(out + idx, v);
            }
        }
    }
}

// torch.min of two statistics: the smaller one, NaN if either is
__device__ __forceinline__ float min_nan(float a, float b)
{
    const float m = (b < a) ? b : a;
    return (b != b) ? b : m;
}

__global__ __launch_bounds__(256) void rank1_row_scale_nd_kernel(NdDims lead, float *__restrict__ out)
{
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= lead.n)
        return;
    int64_t rem = row;
    float scale = 0.0f;
#pragma unroll 1
    for (int i = lead.ndim - 1; i >= 0; --i) {
        const int64_t d = lead.dim[i];
        const int64_t q = rem / d;
        const float s = lead.stat[i][rem - q * d];
        rem = q;
        scale = (i == lead.ndim - 1) ? s : min_nan(scale, s);
    }
    out[row] = scale;
}

// ---------------------------------------------------------------------------------------
// Statistics and scale of a short vector, many vectors per launch.  Between the two passes of the
// optimizer step on a tensor of more than two dimensions (viewed as shape[0] x rest) the column
// maxima of the new second moment -- a vector of `rest` values with the tensor's trailing
// dimensions -- are folded into those dimensions' statistics, and the vector of their minima is
// what the second pass divides by.  For a convolution weight that vector has a few thousand
// entries and the statistics a few hundred: one workgroup per tensor keeps the statistics in LDS
// (maxima by LDS atomics on the bit patterns), writes them out and derives the scale from the LDS
// copy, in one launch for up to 32 tensors instead of three launches per tensor.
// ---------------------------------------------------------------------------------------
constexpr int kNdSmallMax = 32;      // vectors per launch
constexpr int kNdSmallSlots = 8192;  // statistics entries of one vector (sum of its dimensions)

struct NdSmall {
    const float *x;   // the vector: product of dim[] values
    float *scale;     // out: min over the dimensions' statistics, per element of the vector
    float *stat[kNdMax - 1];
    uint32_t dim[kNdMax - 1];
    uint32_t ndim;
    uint32_t n;
};

struct NdSmallArgs {
    NdSmall t[kNdSmallMax];
};
static_assert(sizeof(NdSmallArgs) <= 4096, "kernel arguments exceed 4 KB");

__global__ __launch_bounds__(256) void rank1_small_fold_scale_kernel(const NdSmallArgs args)
{
    __shared__ uint32_t slots[kNdSmallSlots];
    const NdSmall &t = args.t[blockIdx.x];
    uint32_t base[kNdMax - 1], total = 0;
    for (uint32_t i = 0; i < t.ndim; ++i) {
        base[i] = total;
        total += t.dim[i];
    }
    for (uint32_t j = threadIdx.x; j < total; j += blockDim.x)
        slots[j] = 0u;
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < t.n; e += blockDim.x) {
        const uint32_t v = abs_bits(t.x[e]);
        uint32_t rem = e;
        for (int i = (int)t.ndim - 1; i >= 0; --i) {
            const uint32_t q = rem / t.dim[i];
            atomicMax(slots + base[i] + (rem - q * t.dim[i]), v);
            rem = q;
        }
    }
    __syncthreads();
    for (uint32_t i = 0; i < t.ndim; ++i)
        for (uint32_t j = threadIdx.x; j < t.dim[i]; j += blockDim.x)
            t.stat[i][j] = __uint_as_float(slots[base[i] + j]);
    for (uint32_t e = threadIdx.x; e < t.n; e += blockDim.x) {
        uint32_t rem = e;
        float scale = 0.0f;
        for (int i = (int)t.ndim - 1; i >= 0; --i) {
            const uint32_t q = rem / t.dim[i];
            const float s = __uint_as_float(slots[base[i] + (rem - q * t.dim[i])]);
            rem = q;
            scale = (i == (int)t.ndim - 1) ? s : min_nan(scale, s);
        }
        t.scale[e] = scale;
    }
}

// shape -> NdDims for the first `ndim` dimensions; false when a size is not positive, the element
// count overflows or the tile count does not fit a grid
static bool nd_dims(int ndim, const int64_t *shape, float *const *stats, NdDims *out)
{
    out->ndim = ndim;
    int64_t n = 1;
    for (int i = ndim - 1; i >= 0; --i) {
        if (shape[i] <= 0 || n > INT64_MAX / shape[i])
            return false;
        out->dim[i] = shape[i];
        out->stride[i] = n;
        out->stat[i] = stats[i];
        n *= shape[i];
    }
    for (int i = ndim; i < kNdMax; ++i) {
        out->dim[i] = 1;
        out->stride[i] = 1;
        out->stat[i] = nullptr;
    }
    out->n = n;
    return (n + kNdTile - 1) / kNdTile <= 0x7fffffffLL;
}

// LDS slots a workgroup of the fold kernel can need
static int64_t nd_slots(const NdDims &sh)
{
    int64_t total = 0;
    for (int i = 0; i < sh.ndim; ++i) {
        const int64_t by_stride = (kNdTile - 1) / sh.stride[i] + 2;
        total += sh.dim[i] < by_stride ? sh.dim[i] : by_stride;
    }
    return total;
}

static int launch_fold(const float *x, const NdDims &sh, hipStream_t stream)
{
    if (nd_slots(sh) > kNdSlots)
        return LPMM_ERR_SIZE;
    const uint32_t tiles = (uint32_t)((sh.n + kNdTile - 1) / kNdTile);
    hipLaunchKernelGGL(rank1_fold_nd_kernel, dim3(tiles), dim3(kNdThreads), 0, stream, x, sh, aligned_to(x, 16));
    return launch_status();
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_rank1_stats_nd(const float *x, int ndim, const int64_t *shape, float *const *stats, float *work,
                                   void *stream)
{
    if (ndim < 1 || ndim > kNdMax)
        return LPMM_ERR_ARG;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(shape);
    LPMM_REQUIRE_PTR(stats);
    LPMM_REQUIRE_ALIGN(x, 4);
    for (int i = 0; i < ndim; ++i) {
        LPMM_REQUIRE_PTR(stats[i]);
        LPMM_REQUIRE_ALIGN(stats[i], 4);
    }
    NdDims all;
    if (!nd_dims(ndim, shape, stats, &all))
        return LPMM_ERR_SIZE;
    hipStream_t s = (hipStream_t)stream;
    int64_t longest = 1;
    for (int i = 0; i < ndim; ++i)
        longest = shape[i] > longest ? shape[i] : longest;
    if ((longest + 255) / 256 > 0x7fffffffLL)
        return LPMM_ERR_SIZE;
    hipLaunchKernelGGL(nd_zero_kernel, dim3((uint32_t)((longest + 255) / 256), (uint32_t)ndim), dim3(256), 0, s, all);
    const int64_t cols = shape[ndim - 1];
    if (work != nullptr && ndim >= 2 && cols >= 32) {
        LPMM_REQUIRE_ALIGN(work, 4);
        // last dimension and row maxima by the 2-D kernel, leading dimensions from the row maxima
        const int st = lpmm_rank1_stats(x, all.n / cols, cols, work, stats[ndim - 1], stream);
        if (st == LPMM_OK) {
            NdDims lead;
            if (!nd_dims(ndim - 1, shape, stats, &lead))
                return LPMM_ERR_SIZE;
            return launch_fold(work, lead, s);
        }
        if (st != LPMM_ERR_SIZE)
            return st;
        // more rows than the 2-D kernel's grid takes: the one-pass kernel below
    }
    return launch_fold(x, all, s);
}

extern "C" int lpmm_rank1_row_scale_nd(const float *const *stats, int ndim, const int64_t *shape, float *row_scale,
                                       void *stream)
{
    if (ndim < 2 || ndim > kNdMax)
        return LPMM_ERR_ARG;
    LPMM_REQUIRE_PTR(stats);
    LPMM_REQUIRE_PTR(shape);
    LPMM_REQUIRE_PTR(row_scale);
    LPMM_REQUIRE_ALIGN(row_scale, 4);
    for (int i = 0; i < ndim - 1; ++i) {
        LPMM_REQUIRE_PTR(stats[i]);
        LPMM_REQUIRE_ALIGN(stats[i], 4);
    }
    if (shape[ndim - 1] <= 0)
        return LPMM_ERR_SIZE;
    NdDims lead;
    if (!nd_dims(ndim - 1, shape, const_cast<float *const *>(stats), &lead) || (lead.n + 255) / 256 > 0x7fffffffLL)
        return LPMM_ERR_SIZE;
    hipLaunchKernelGGL(rank1_row_scale_nd_kernel, dim3((uint32_t)((lead.n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, lead, row_scale);
    return launch_status();
}

extern "C" int lpmm_rank1_small_fold_scale_multi(const lpmm_rank1_small_vector *vectors, int64_t count, void *stream)
{
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(vectors);
    for (int64_t i = 0; i < count; ++i) {
        const lpmm_rank1_small_vector &v = vectors[i];
        if (v.ndim < 1 || v.ndim > kNdMax - 1)
            return LPMM_ERR_ARG;
        LPMM_REQUIRE_PTR(v.x);
        LPMM_REQUIRE_PTR(v.scale);
        LPMM_REQUIRE_ALIGN(v.x, 4);
        LPMM_REQUIRE_ALIGN(v.scale, 4);
        int64_t n = 1, slots = 0;
        for (int k = 0; k < v.ndim; ++k) {
            LPMM_REQUIRE_PTR(v.stats[k]);
            LPMM_REQUIRE_ALIGN(v.stats[k], 4);
            if (v.shape[k] <= 0 || v.shape[k] > kNdSmallSlots || n > (int64_t)0x7fffffff / v.shape[k])
                return LPMM_ERR_SIZE;
            n *= v.shape[k];
            slots += v.shape[k];
        }
        if (slots > kNdSmallSlots)
            return LPMM_ERR_SIZE;
    }
    for (int64_t i = 0; i < count; i += kNdSmallMax) {
        NdSmallArgs args;
        const int k = (int)(count - i < kNdSmallMax ? count - i : kNdSmallMax);
        for (int j = 0; j < k; ++j) {
            const lpmm_rank1_small_vector &v = vectors[i + j];
            NdSmall &t = args.t[j];
            t.x = v.x;
            t.scale = v.scale;
            t.ndim = (uint32_t)v.ndim;
            uint32_t n = 1;
            for (int a = 0; a < kNdMax - 1; ++a) {
                t.stat[a] = a < v.ndim ? v.stats[a] : nullptr;
                t.dim[a] = a < v.ndim ? (uint32_t)v.shape[a] : 1u;
                n *= t.dim[a];
            }
            t.n = n;
        }
        hipLaunchKernelGGL(rank1_small_fold_scale_kernel, dim3((uint32_t)k), dim3(256), 0, (hipStream_t)stream, args);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}
