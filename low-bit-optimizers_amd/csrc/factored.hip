// Non-fused elementwise AdamW update and the factored second-moment step for gfx950.
//
// Roundings follow the PyTorch CPU kernels that the reference's op sequence runs
// (lpmm/optim/adamw.py:367-369, :412-422, :579-627): multiply by the float-cast Python
// scalar, lerp as fma(w, g - m, m) for w < 0.5, addcmul as v + (value*g)*g, true division
// by the float-cast sqrt(bias_correction2), addcdiv as p + (value*m)/denom.
// Row/column means of g*g are summed in double in a fixed order and rounded once.
#include "lpmm_common.hpp"

#include <math.h>

namespace lpmm {

constexpr int kFThreads = 256;
constexpr int kFElts = 8;
constexpr int kFTile = kFThreads * kFElts;  // 2048

struct NfHyper {
    float decay, w1, b2, w2, neg_step_size, bc2_sqrt, eps;
};

inline NfHyper make_nf_hyper(double beta1, double beta2, double lr, double wd, double eps, double step)
{
    NfHyper h;
    h.decay = (float)(1.0 - lr * wd);
    h.w1 = (float)(1.0 - beta1);
    h.b2 = (float)beta2;
    h.w2 = (float)(1.0 - beta2);
    const double bc1 = 1.0 - pow(beta1, step);
    const double bc2 = 1.0 - pow(beta2, step);
    h.neg_step_size = (float)(-(lr / bc1));
    h.bc2_sqrt = (float)sqrt(bc2);
    h.eps = (float)eps;
    return h;
}

__device__ __forceinline__ float lerp_w(float a, float b, float w)
{
    return (fabsf(w) < 0.5f) ? __builtin_fmaf(w, b - a, a) : __builtin_fmaf(w - 1.0f, b - a, b);
}

__global__ __launch_bounds__(kFThreads) void nonfused_update_kernel(float *__restrict__ p,
                                                                    const float *__restrict__ g,
                                                                    float *__restrict__ m, float *__restrict__ v,
                                                                    int64_t n, NfHyper h)
{
    const int64_t stride = (int64_t)gridDim.x * kFThreads;
    for (int64_t i = (int64_t)blockIdx.x * kFThreads + threadIdx.x; i < n; i += stride) {
        const float gi = g[i];
        const float pi = p[i] * h.decay;
        const float mi = lerp_w(m[i], gi, h.w1);
        float vi = v[i] * h.b2;
        vi = vi + (h.w2 * gi) * gi;
        const float denom = sqrtf(vi) / h.bc2_sqrt + h.eps;
        p[i] = pi + (h.neg_step_size * mi) / denom;
        m[i] = mi;
        v[i] = vi;
    }
}

// ---------------------------------------------------------------------------------------
// Factored statistics, pass A: partial row/column sums of g*g over tiles of
// kSRows x kSCols, accumulated in double.  Partials go to the workspace:
//   colpart[ty][c]  (ty = row-tile index)   rowpart[tx*4 + wave][r]  (tx = column-tile index)
// ---------------------------------------------------------------------------------------
constexpr int kSRows = 128;
constexpr int kSCols = 1024;  // 256 threads x 4 columns

__global__ __launch_bounds__(kFThreads) void factored_partial_kernel(const float *__restrict__ g, int64_t R,
                                                                     int64_t C, double *__restrict__ colpart,
                                                                     double *__restrict__ rowpart, bool vec)
{
    const int64_t c0 = (int64_t)blockIdx.x * kSCols + (int64_t)threadIdx.x * 4;
    const int64_t r0 = (int64_t)blockIdx.y * kSRows;
    const int64_t r1 = (r0 + kSRows < R) ? r0 + kSRows : R;
    // one row partial per wave: rowpart[(column tile * 4 + wave)][r]
    double *rp = rowpart + ((int64_t)blockIdx.x * (kFThreads / kWave) + (threadIdx.x >> 6)) * R;
    double cs[4] = {0.0, 0.0, 0.0, 0.0};
    for (int64_t r = r0; r < r1; ++r) {
        float u[4];
        const float *row = g + r * C;
        if (vec && c0 + 4 <= C) {
            const float4 t = *reinterpret_cast<const float4 *>(row + c0);
            u[0] = t.x * t.x; u[1] = t.y * t.y; u[2] = t.z * t.z; u[3] = t.w * t.w;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float t = (c0 + k < C) ? row[c0 + k] : 0.0f;
                u[k] = t * t;
            }
        }
        double rs = ((double)u[0] + (double)u[1]) + ((double)u[2] + (double)u[3]);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            cs[k] += (double)u[k];
        rs = wave_sum_f64(rs);
        if ((threadIdx.x & 63) == 0)
            rp[r] = rs;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (c0 + k < C)
            colpart[(int64_t)blockIdx.y * C + c0 + k] = cs[k];
}

// Pass B: fold the partials in a fixed order, update the EMAs
// (row.mul_(beta2).add_(mean, alpha=1-beta2): fma(mean, 1-beta2, row*beta2)).
// Workgroups 1.. handle columns; workgroup 0 handles all rows and mean(row).
__global__ __launch_bounds__(kFThreads) void factored_finalize_kernel(const double *__restrict__ colpart,
                                                                      const double *__restrict__ rowpart,
                                                                      int64_t R, int64_t C, int tiles_y,
                                                                      int tiles_x, float *__restrict__ row,
                                                                      float *__restrict__ col,
                                                                      float *__restrict__ row_mean_all, float b2,
                                                                      float w2)
{
    if (blockIdx.x > 0) {
        const int64_t c = (int64_t)(blockIdx.x - 1) * kFThreads + threadIdx.x;
        if (c < C) {
            double s = 0.0;
            for (int t = 0; t < tiles_y; ++t)
                s += colpart[(int64_t)t * C + c];
            const float mean = (float)(s / (double)R);
            col[c] = __builtin_fmaf(mean, w2, col[c] * b2);
        }
        return;
    }
    __shared__ double s_sum[kFThreads];
    double acc = 0.0;
    for (int64_t r = threadIdx.x; r < R; r += kFThreads) {
        double s = 0.0;
        for (int t = 0; t < tiles_x; ++t)
            s += rowpart[(int64_t)t * R + r];
        const float mean = (float)(s / (double)C);
        const float nr = __builtin_fmaf(mean, w2, row[r] * b2);
        row[r] = nr;
        acc += (double)nr;
    }
    s_sum[threadIdx.x] = acc;
    __syncthreads();
    for (int o = kFThreads / 2; o > 0; o >>= 1) {
        if (threadIdx.x < o)
            s_sum[threadIdx.x] += s_sum[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        *row_mean_all = (float)(s_sum[0] / (double)R);
}

// ---------------------------------------------------------------------------------------
// Factored update, one pass: decay p, decode m (group-128 codes of the non-fused layout),
// lerp, v = row/mean(row) * col, update p, re-quantise m and write its pad codes.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kFThreads) void factored_update_kernel(
    float *__restrict__ p, const float *__restrict__ g, uint8_t *__restrict__ m_codes,
    float *__restrict__ m_max1, const float *__restrict__ qmap_m, const float *__restrict__ row,
    const float *__restrict__ col, const float *__restrict__ row_mean_all, int64_t n, int64_t C,
    int64_t n_groups, int64_t n_padded, NfHyper h, bool first_step, bool vec)
{
    __shared__ float s_q[16];
    if (threadIdx.x < 16)
        s_q[threadIdx.x] = qmap_m[threadIdx.x];
    const Mids mids = make_mids(qmap_m);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kFThreads + threadIdx.x) * kFElts;
    if (base == 0)
        m_codes[n_padded / 2] = 0;
    const int64_t grp = base / kGroup;
    const bool any = base < n;
    const bool full = vec && (base + kFElts <= n);
    float pv[kFElts], gv[kFElts], m[kFElts];
    uint32_t wm = 0;
    float sm = 0.0f;
    if (full) {
        const float4 a0 = *reinterpret_cast<const float4 *>(p + base);
        const float4 a1 = *reinterpret_cast<const float4 *>(p + base + 4);
        const float4 b0 = *reinterpret_cast<const float4 *>(g + base);
        const float4 b1 = *reinterpret_cast<const float4 *>(g + base + 4);
        pv[0] = a0.x; pv[1] = a0.y; pv[2] = a0.z; pv[3] = a0.w;
        pv[4] = a1.x; pv[5] = a1.y; pv[6] = a1.z; pv[7] = a1.w;
        gv[0] = b0.x; gv[1] = b0.y; gv[2] = b0.z; gv[3] = b0.w;
        gv[4] = b1.x; gv[5] = b1.y; gv[6] = b1.z; gv[7] = b1.w;
    } else {
#pragma unroll
        for (int k = 0; k < kFElts; ++k) {
            pv[k] = (base + k < n) ? p[base + k] : 0.0f;
            gv[k] = (base + k < n) ? g[base + k] : 0.0f;
        }
    }
    if (any && !first_step) {
        wm = *reinterpret_cast<const uint32_t *>(m_codes + (base >> 1));  // padded buffer: always inside
        sm = m_max1[grp];
    }
    const float mean_all = *row_mean_all;
    int64_t r = any ? base / C : 0;
    int64_t c = any ? base - r * C : 0;
    float rf = any ? row[r] / mean_all : 0.0f;
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kFElts; ++k) {
        m[k] = 0.0f;
        if (base + k < n) {
            const float m_old = first_step ? 0.0f : s_q[(wm >> (4 * k)) & 0xF] * sm;
            const float pi = pv[k] * h.decay;
            const float mi = lerp_w(m_old, gv[k], h.w1);
            const float vi = rf * col[c];
            const float denom = sqrtf(vi) / h.bc2_sqrt + h.eps;
            pv[k] = pi + (h.neg_step_size * mi) / denom;
            m[k] = mi;
            amax = fmaxf(amax, fabsf(mi));
            if (++c == C) {
                c = 0;
                ++r;
                rf = (base + k + 1 < n) ? row[r] / mean_all : 0.0f;
            }
        }
    }
    amax = row16_max(amax);
    const bool in_scaled = grp < n_groups;
    if (in_scaled && (threadIdx.x & 15) == 0)
        m_max1[grp] = amax;
    uint32_t om = 0;
#pragma unroll
    for (int k = 0; k < kFElts; ++k) {
        const float val = in_scaled ? m[k] / amax : 0.0f;
        om |= ((val != val) ? 15u : encode_count(mids, val)) << (4 * k);
    }
    *reinterpret_cast<uint32_t *>(m_codes + (base >> 1)) = om;
    if (full) {
        *reinterpret_cast<float4 *>(p + base) = make_float4(pv[0], pv[1], pv[2], pv[3]);
        *reinterpret_cast<float4 *>(p + base + 4) = make_float4(pv[4], pv[5], pv[6], pv[7]);
    } else {
#pragma unroll
        for (int k = 0; k < kFElts; ++k)
            if (base + k < n)
                p[base + k] = pv[k];
    }
}

// The same update with an fp32 first moment (tensors at or under the quantisation threshold,
// or first-moment quantisation disabled): m is read and written as floats.
__global__ __launch_bounds__(kFThreads) void factored_update_fp32m_kernel(
    float *__restrict__ p, const float *__restrict__ g, float *__restrict__ m, const float *__restrict__ row,
    const float *__restrict__ col, const float *__restrict__ row_mean_all, int64_t n, int64_t C, NfHyper h)
{
    const float mean_all = *row_mean_all;
    const int64_t stride = (int64_t)gridDim.x * kFThreads;
    for (int64_t i = (int64_t)blockIdx.x * kFThreads + threadIdx.x; i < n; i += stride) {
        const int64_t r = i / C, c = i - r * C;
        const float pi = p[i] * h.decay;
        const float mi = lerp_w(m[i], g[i], h.w1);
        const float vi = (row[r] / mean_all) * col[c];
        const float denom = sqrtf(vi) / h.bc2_sqrt + h.eps;
        p[i] = pi + (h.neg_step_size * mi) / denom;
        m[i] = mi;
    }
}

inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_nonfused_update(float *p, const float *g, float *m, float *v, int64_t n, double beta1,
                                    double beta2, double lr, double weight_decay, double eps, double step,
                                    void *stream)
{
    if (n < 0)
        return LPMM_ERR_SIZE;
    if (n == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(p);
    LPMM_REQUIRE_PTR(g);
    LPMM_REQUIRE_PTR(m);
    LPMM_REQUIRE_PTR(v);
    LPMM_REQUIRE_ALIGN(p, 4);
    LPMM_REQUIRE_ALIGN(g, 4);
    LPMM_REQUIRE_ALIGN(m, 4);
    LPMM_REQUIRE_ALIGN(v, 4);
    int64_t blocks = (n + kFThreads - 1) / kFThreads;
    if (blocks > 256 * 64)
        blocks = 256 * 64;
    hipLaunchKernelGGL(nonfused_update_kernel, dim3((uint32_t)blocks), dim3(kFThreads), 0,
                       (hipStream_t)stream, p, g, m, v, n,
                       make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step));
    return launch_status();
}

extern "C" int64_t lpmm_factored_workspace_bytes(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0)
        return 0;
    const int64_t ty = (rows + kSRows - 1) / kSRows, tx = (cols + kSCols - 1) / kSCols;
    return (ty * cols + tx * (kFThreads / kWave) * rows) * (int64_t)sizeof(double);
}

extern "C" int lpmm_factored_stats(const float *g, int64_t rows, int64_t cols, float *row, float *col,
                                   float *row_mean_all, double beta2, void *workspace, void *stream)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(g);
    LPMM_REQUIRE_PTR(row);
    LPMM_REQUIRE_PTR(col);
    LPMM_REQUIRE_PTR(row_mean_all);
    LPMM_REQUIRE_PTR(workspace);
    LPMM_REQUIRE_ALIGN(g, 4);
    LPMM_REQUIRE_ALIGN(row, 4);
    LPMM_REQUIRE_ALIGN(col, 4);
    LPMM_REQUIRE_ALIGN(row_mean_all, 4);
    LPMM_REQUIRE_ALIGN(workspace, 8);
    const int64_t ty = (rows + kSRows - 1) / kSRows, tx = (cols + kSCols - 1) / kSCols;
    if (ty > 65535 || tx > 0x7fffffffLL)
        return LPMM_ERR_SIZE;
    double *colpart = static_cast<double *>(workspace);
    double *rowpart = colpart + ty * cols;
    const bool vec = aligned_to(g, 16) && (cols % 4) == 0;
    hipLaunchKernelGGL(factored_partial_kernel, dim3((uint32_t)tx, (uint32_t)ty), dim3(kFThreads), 0,
                       (hipStream_t)stream, g, rows, cols, colpart, rowpart, vec);
    int st = launch_status();
    if (st != LPMM_OK)
        return st;
    const int64_t col_blocks = (cols + kFThreads - 1) / kFThreads;
    hipLaunchKernelGGL(factored_finalize_kernel, dim3((uint32_t)(col_blocks + 1)), dim3(kFThreads), 0,
                       (hipStream_t)stream, colpart, rowpart, rows, cols, (int)ty, (int)tx * (kFThreads / kWave), row, col,
                       row_mean_all, (float)beta2, (float)(1.0 - beta2));
    return launch_status();
}

extern "C" int lpmm_factored_update(float *p, const float *g, uint8_t *m_codes, float *m_max1,
                                    const float *qmap_m, const float *row, const float *col,
                                    const float *row_mean_all, int64_t rows, int64_t cols, double beta1,
                                    double beta2, double lr, double weight_decay, double eps, double step,
                                    int first_step, void *stream)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(p);
    LPMM_REQUIRE_PTR(g);
    LPMM_REQUIRE_PTR(m_codes);
    LPMM_REQUIRE_PTR(m_max1);
    LPMM_REQUIRE_PTR(qmap_m);
    LPMM_REQUIRE_PTR(row);
    LPMM_REQUIRE_PTR(col);
    LPMM_REQUIRE_PTR(row_mean_all);
    LPMM_REQUIRE_ALIGN(p, 4);
    LPMM_REQUIRE_ALIGN(g, 4);
    LPMM_REQUIRE_ALIGN(m_codes, 4);
    LPMM_REQUIRE_ALIGN(m_max1, 4);
    LPMM_REQUIRE_ALIGN(qmap_m, 4);
    LPMM_REQUIRE_ALIGN(row, 4);
    LPMM_REQUIRE_ALIGN(col, 4);
    LPMM_REQUIRE_ALIGN(row_mean_all, 4);
    const int64_t n = rows * cols;
    const int64_t n_groups = (n + kGroup - 1) / kGroup;
    const int64_t n_padded = round_up(n_groups * kGroup, kFTile);
    const int64_t tiles = n_padded / kFTile;
    if (tiles > 0x7fffffffLL)
        return LPMM_ERR_SIZE;
    const bool vec = aligned_to(p, 16) && aligned_to(g, 16);
    hipLaunchKernelGGL(factored_update_kernel, dim3((uint32_t)tiles), dim3(kFThreads), 0,
                       (hipStream_t)stream, p, g, m_codes, m_max1, qmap_m, row, col, row_mean_all, n, cols,
                       n_groups, n_padded, make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step),
                       first_step != 0, vec);
    return launch_status();
}

extern "C" int lpmm_factored_update_fp32m(float *p, const float *g, float *m, const float *row,
                                          const float *col, const float *row_mean_all, int64_t rows,
                                          int64_t cols, double beta1, double beta2, double lr,
                                          double weight_decay, double eps, double step, void *stream)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(p);
    LPMM_REQUIRE_PTR(g);
    LPMM_REQUIRE_PTR(m);
    LPMM_REQUIRE_PTR(row);
    LPMM_REQUIRE_PTR(col);
    LPMM_REQUIRE_PTR(row_mean_all);
    LPMM_REQUIRE_ALIGN(p, 4);
    LPMM_REQUIRE_ALIGN(g, 4);
    LPMM_REQUIRE_ALIGN(m, 4);
    LPMM_REQUIRE_ALIGN(row, 4);
    LPMM_REQUIRE_ALIGN(col, 4);
    LPMM_REQUIRE_ALIGN(row_mean_all, 4);
    const int64_t n = rows * cols;
    int64_t blocks = (n + kFThreads - 1) / kFThreads;
    if (blocks > 256 * 64)
        blocks = 256 * 64;
    hipLaunchKernelGGL(factored_update_fp32m_kernel, dim3((uint32_t)blocks), dim3(kFThreads), 0,
                       (hipStream_t)stream, p, g, m, row, col, row_mean_all, n, cols,
                       make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step));
    return launch_status();
}
