// Non-fused elementwise AdamW update and the factored second-moment step for gfx950.
//
// Roundings follow the PyTorch CPU kernels that the reference's op sequence runs
// (lpmm/optim/adamw.py:367-369, :412-422, :579-627): multiply by the float-cast Python
// scalar, lerp as fma(w, g - m, m) for w < 0.5, addcmul as v + (value*g)*g, true division
// by the float-cast sqrt(bias_correction2), addcdiv as p + (value*m)/denom.  m and v are
// computed exactly so; the square root and the two divisions of the parameter update use
// the hardware approximations with one fma correction of the residual (correctly rounded
// except for a vanishing fraction of inputs; the parameter never feeds back into a state).
// Row/column means of g*g are summed in double in a fixed order and rounded once.
#include "lpmm_update.hpp"

#include <mutex>

namespace lpmm {

constexpr int kFThreads = 256;
constexpr int kFElts = 8;
constexpr int kFTile = kFThreads * kFElts;  // 2048

__global__ __launch_bounds__(kFThreads) void nonfused_update_kernel(float *__restrict__ p,
                                                                    const float *__restrict__ g,
                                                                    float *__restrict__ m, float *__restrict__ v,
                                                                    int64_t n, NfHyper h, bool vec)
{
    const int64_t base = ((int64_t)blockIdx.x * kFThreads + threadIdx.x) * 4;
    if (base >= n)
        return;
    if (vec && base + 4 <= n) {
        float4 pp = load4(p + base), mm = load4(m + base), vv = load4(v + base);
        const float4 gg = load4(g + base);
        nonfused_elt(pp.x, gg.x, mm.x, vv.x, h);
        nonfused_elt(pp.y, gg.y, mm.y, vv.y, h);
        nonfused_elt(pp.z, gg.z, mm.z, vv.z, h);
        nonfused_elt(pp.w, gg.w, mm.w, vv.w, h);
        store4(p + base, pp);
        store4(m + base, mm);
        store4(v + base, vv);
    } else {
        for (int64_t i = base; i < base + 4 && i < n; ++i) {
            float pi = p[i], mi = m[i], vi = v[i];
            nonfused_elt(pi, g[i], mi, vi, h);
            p[i] = pi;
            m[i] = mi;
            v[i] = vi;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Factored statistics, pass A: partial row/column sums of g*g over tiles of
// kSRows x kSCols, accumulated in double.  Partials go to the workspace:
//   colpart[ty][c]  (ty = row-tile index)   rowpart[tx][r]  (tx = column-tile index)
// One-shot: a wave takes 16 rows x 256 columns of the tile (a lane: 4 columns of each row) and
// issues all 16 loads at once; there is no loop, so the grid's many small workgroups keep the
// memory system as busy as a plain streaming read does.  The wave owns its rows (their sums go
// straight to rowpart); the column sums of the four waves meet in LDS in a fixed order.
// ---------------------------------------------------------------------------------------
constexpr int kSRows = 64;
constexpr int kSCols = 256;   // 64 lanes x 4 columns
constexpr int kSWaveRows = kSRows / (kFThreads / kWave);  // 16
static_assert(kSWaveRows == 16, "two wave_sum8_f64 reductions per wave");

__device__ __forceinline__ void partial_body(const float *__restrict__ g, int64_t R, int64_t C,
                                             double *__restrict__ colpart, double *__restrict__ rowpart, bool vec,
                                             uint32_t bx, uint32_t by)
{
    __shared__ double s_col[kFThreads / kWave][kSCols];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t c0 = (int64_t)bx * kSCols + lane * 4;
    const int64_t r0 = (int64_t)by * kSRows + wave * kSWaveRows;
    float4 t[kSWaveRows];
    if (vec && c0 + 4 <= C && r0 + kSWaveRows <= R) {
        const float *base = g + r0 * C + c0;
#pragma unroll
        for (int u = 0; u < kSWaveRows; ++u)
            t[u] = load4(base + (int64_t)u * C);
    } else {
#pragma unroll
        for (int u = 0; u < kSWaveRows; ++u) {
            const int64_t r = r0 + u;
            float e[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
                e[k] = (r < R && c0 + k < C) ? g[r * C + c0 + k] : 0.0f;
            t[u] = make_float4(e[0], e[1], e[2], e[3]);
        }
    }
    double cs[4] = {0.0, 0.0, 0.0, 0.0};
    double *rp = rowpart + (int64_t)bx * R;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        double rs[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float4 &x = t[half * 8 + j];
            const float u[4] = {x.x * x.x, x.y * x.y, x.z * x.z, x.w * x.w};
            rs[j] = ((double)u[0] + (double)u[1]) + ((double)u[2] + (double)u[3]);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                cs[k] += (double)u[k];
        }
        // the wave's 8 row sums at once: lane 8j ends up with the sum of row j of this half
        const double tot = wave_sum8_f64(rs, lane);
        const int64_t r = r0 + half * 8 + (lane >> 3);
        if ((lane & 7) == 0 && r < R)
            rp[r] = tot;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
        s_col[wave][lane * 4 + k] = cs[k];
    __syncthreads();
    const int64_t c = (int64_t)bx * kSCols + threadIdx.x;
    if (threadIdx.x < kSCols && c < C)
        colpart[(int64_t)by * C + c] = (s_col[0][threadIdx.x] + s_col[1][threadIdx.x]) +
                                       (s_col[2][threadIdx.x] + s_col[3][threadIdx.x]);
}

__global__ __launch_bounds__(kFThreads) void factored_partial_kernel(const float *__restrict__ g, int64_t R,
                                                                     int64_t C, double *__restrict__ colpart,
                                                                     double *__restrict__ rowpart, bool vec)
{
    partial_body(g, R, C, colpart, rowpart, vec, blockIdx.x, blockIdx.y);
}

// Pass B: fold the partials in a fixed order and update the EMAs
// (row.mul_(beta2).add_(mean, alpha=1-beta2): fma(mean, 1-beta2, row*beta2)).
// Workgroups [0, row_blocks) take 256 rows each and leave the sum of their new row values in
// rowblock[b]; the remaining workgroups take 64 columns each.
__device__ __forceinline__ void finalize_body(const double *__restrict__ colpart, const double *__restrict__ rowpart,
                                              double *__restrict__ rowblock, int64_t R, int64_t C, int tiles_y,
                                              int tiles_x, int row_blocks, float *__restrict__ row,
                                              float *__restrict__ col, float b2, float w2, uint32_t bx)
{
    if ((int)bx >= row_blocks) {
        // 64 columns per workgroup; the partials of a column are split over 4 threads, each
        // summing its contiguous quarter 8 loads at a time, and folded in a fixed order
        __shared__ double s_col[kFThreads];
        const int64_t c = (int64_t)(bx - row_blocks) * 64 + (threadIdx.x & 63);
        const int quarter = threadIdx.x >> 6;
        const int per = (tiles_y + 3) / 4;
        const int t0 = quarter * per, t1 = (t0 + per < tiles_y) ? t0 + per : tiles_y;
        double s = 0.0;
        if (c < C) {
            int t = t0;
            for (; t + 8 <= t1; t += 8) {
                double a[8];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    a[k] = colpart[(int64_t)(t + k) * C + c];
                s += ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
            }
            for (; t < t1; ++t)
                s += colpart[(int64_t)t * C + c];
        }
        s_col[threadIdx.x] = s;
        __syncthreads();
        if (quarter == 0 && c < C) {
            const double tot = (s_col[threadIdx.x] + s_col[threadIdx.x + 64]) +
                               (s_col[threadIdx.x + 128] + s_col[threadIdx.x + 192]);
            const float mean = (float)(tot / (double)R);
            col[c] = __builtin_fmaf(mean, w2, col[c] * b2);
        }
        return;
    }
    __shared__ double s_sum[kFThreads];
    const int64_t r = (int64_t)bx * kFThreads + threadIdx.x;
    double mine = 0.0;
    if (r < R) {
        double s = 0.0;
        for (int t = 0; t < tiles_x; ++t)
            s += rowpart[(int64_t)t * R + r];
        const float mean = (float)(s / (double)C);
        const float nr = __builtin_fmaf(mean, w2, row[r] * b2);
        row[r] = nr;
        mine = (double)nr;
    }
    s_sum[threadIdx.x] = mine;
    __syncthreads();
    for (int o = kFThreads / 2; o > 0; o >>= 1) {
        if (threadIdx.x < o)
            s_sum[threadIdx.x] += s_sum[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        rowblock[bx] = s_sum[0];
}

__global__ __launch_bounds__(kFThreads) void factored_finalize_kernel(const double *__restrict__ colpart,
                                                                      const double *__restrict__ rowpart,
                                                                      double *__restrict__ rowblock, int64_t R,
                                                                      int64_t C, int tiles_y, int tiles_x,
                                                                      int row_blocks, float *__restrict__ row,
                                                                      float *__restrict__ col, float b2, float w2)
{
    finalize_body(colpart, rowpart, rowblock, R, C, tiles_y, tiles_x, row_blocks, row, col, b2, w2, blockIdx.x);
}

// Pass C: mean(row) from the per-workgroup sums, in order.
__global__ void factored_mean_kernel(const double *__restrict__ rowblock, int row_blocks, int64_t R,
                                     float *__restrict__ row_mean_all)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        double s = 0.0;
        for (int b = 0; b < row_blocks; ++b)
            s += rowblock[b];
        *row_mean_all = (float)(s / (double)R);
    }
}

// ---------------------------------------------------------------------------------------
// Factored update, one pass: decay p, decode m (group-128 codes of the non-fused layout),
// lerp, v = row/mean(row) * col, update p, re-quantise m and write its pad codes.
// ROWS: the column count is a multiple of 8, so a lane's 8 elements lie in one row and the
// row index comes from one division per lane; otherwise every element tracks its own
// (row, column).
// ---------------------------------------------------------------------------------------
template <bool ROWS>
__global__ __launch_bounds__(kFThreads) void factored_update_kernel(
    float *__restrict__ p, const float *__restrict__ g, uint8_t *__restrict__ m_codes,
    float *__restrict__ m_max1, const float *__restrict__ qmap_m, const float *__restrict__ row,
    const float *__restrict__ col, const float *__restrict__ row_mean_all, int64_t n, int64_t C,
    int64_t n_groups, int64_t n_padded, NfHyper h, bool first_step, bool vec)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    lds_fill(lds, qmap_m, nullptr);
    const int kind = classify_map(qmap_m);
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
        const float4 a0 = load4(p + base), a1 = load4(p + base + 4);
        const float4 b0 = load4(g + base), b1 = load4(g + base + 4);
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
        wm = load_u32(reinterpret_cast<const uint32_t *>(m_codes + (base >> 1)));  // padded buffer: always inside
        sm = m_max1[grp];
    }
    const Nibbles nm = split_nibbles(wm);
    const float mean_all = *row_mean_all;
    int64_t r = any ? base / C : 0;
    int64_t c = any ? base - r * C : 0;
    float rf = any ? row[r] / mean_all : 0.0f;
    float cv[kFElts];
    if (ROWS && any) {
        const float4 c0 = *reinterpret_cast<const float4 *>(col + c), c1 = *reinterpret_cast<const float4 *>(col + c + 4);
        cv[0] = c0.x; cv[1] = c0.y; cv[2] = c0.z; cv[3] = c0.w;
        cv[4] = c1.x; cv[5] = c1.y; cv[6] = c1.z; cv[7] = c1.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kFElts; ++k) {
        m[k] = 0.0f;
        if (base + k < n) {
            const float m_old = first_step ? 0.0f : decode_nibble(lds, kLdsQ0, nm, k) * sm;
            const float pi = pv[k] * h.decay;
            const float mi = lerp_w(m_old, gv[k], h.w1);
            const float vi = rf * (ROWS ? cv[k] : col[c]);
            const float denom = div_by_rc(sqrt_fast(vi), h.bc2_sqrt, h.rbc2_sqrt) + h.eps;
            pv[k] = pi + div_fast(h.neg_step_size * mi, denom);
            m[k] = mi;
            amax = fmaxf(amax, fabsf(mi));
            if (!ROWS && ++c == C) {
                c = 0;
                ++r;
                rf = (base + k + 1 < n) ? row[r] / mean_all : 0.0f;
            }
        }
    }
    amax = row16_max(amax);
    uint32_t om;
    if (grp < n_groups) {
        if ((threadIdx.x & 15) == 0)
            m_max1[grp] = amax;
        om = encode8_scaled(lds, kLdsQ0, kind, m, amax);
    } else {
        // padding added by the re-grouping to 2048: the code of a plain 0.0
        const float z[kFElts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        om = kind == kMapStdM ? encode8_std_m(lds, z)
                              : encode8_generic(make_mids(reinterpret_cast<const float *>(lds) + kLdsQ0 / 4), z);
    }
    store_u32(reinterpret_cast<uint32_t *>(m_codes + (base >> 1)), om);
    if (full) {
        store4(p + base, make_float4(pv[0], pv[1], pv[2], pv[3]));
        store4(p + base + 4, make_float4(pv[4], pv[5], pv[6], pv[7]));
    } else {
#pragma unroll
        for (int k = 0; k < kFElts; ++k)
            if (base + k < n)
                p[base + k] = pv[k];
    }
}

// The same pass when the column count is a multiple of 128: every 128-element group of the
// flattened tensor is a 128-column piece of one row.  A workgroup takes a tile of 8 rows by 2
// adjacent groups (2048 elements in runs of 1 KB), the 16 lanes of a DPP row own one group in
// the row layout of the fused step (lane l: columns [4l, 4l+4) and [64+4l, 64+4l+4) of the
// piece; whole cache lines per store).  The 8 rows of a tile read the same column statistics,
// which a tile of 16 consecutive groups of one row does not: 1970 -> 1880 us per launch of
// 8.6e8 elements on the LLaMA-7B MLP shapes (4 rows by 4 groups 1905 us, 16 rows by 1 group
// 2060 us: its 512-byte runs cost more than the shared statistics save).  Tile 0 also writes
// the pad codes past the tensor.
#ifndef LPMM_FA_UPD_LDS_KB
#define LPMM_FA_UPD_LDS_KB 0
#endif
#ifndef LPMM_FA_TILE_ROWS
#define LPMM_FA_TILE_ROWS 8
#endif
constexpr uint32_t kFaTileRows = LPMM_FA_TILE_ROWS;
static_assert((kFTile / kGroup) % LPMM_FA_TILE_ROWS == 0, "a tile is a whole number of groups per row");
constexpr uint32_t kFaUpdLds = LPMM_FA_UPD_LDS_KB * 1024u > kLdsBytes ? LPMM_FA_UPD_LDS_KB * 1024u : kLdsBytes;

__device__ __forceinline__ void update_rows128_body(
    float *__restrict__ p, const float *__restrict__ g, uint8_t *__restrict__ m_codes,
    float *__restrict__ m_max1, const float *__restrict__ qmap_m, const float *__restrict__ row,
    const float *__restrict__ col, const float *__restrict__ row_mean_all, int64_t R, int64_t C,
    int64_t n_padded, const NfHyper &h, bool first_step, uint32_t tile)
{
    __shared__ __align__(16) uint32_t lds[kFaUpdLds / 4];
    const int64_t n = R * C;
    const int lane16 = threadIdx.x & 15;
    const uint32_t col_blocks = (uint32_t)(C / kGroup);
    // tile = kFaTileRows rows by 16 / kFaTileRows adjacent groups
    constexpr uint32_t kGPS = (kFTile / kGroup) / kFaTileRows;
    const uint32_t col_tiles = (col_blocks + kGPS - 1) / kGPS;
#ifndef LPMM_FA_RUN_ORDER
#define LPMM_FA_RUN_ORDER 1
#endif
    // Where 16 consecutive tiles (column tile fastest) are 128 KB of contiguous parameters -- 256, 512, ...
    // 4096 columns -- the tiles are handed out in the order of xcd_run_order: an XCD streams whole runs.
    if (LPMM_FA_RUN_ORDER && kFaTileRows == 8 && (16u % col_tiles) == 0u)
        tile = xcd_run_order<4>(tile, (uint32_t)((R + kFaTileRows - 1) / kFaTileRows) * col_tiles,
                                run_phase<4>(p, kFTile * sizeof(float)));
    const uint32_t rb = tile / col_tiles, ct = tile - rb * col_tiles;
    const uint32_t drow = threadIdx.x >> 4;
    const int64_t r = (int64_t)rb * kFaTileRows + drow / kGPS;
    const uint32_t cb = ct * kGPS + drow % kGPS;
    const bool live = r < R && cb < col_blocks;  // uniform over the 16 lanes of the group
    const int64_t grp = r * col_blocks + cb;
    const int64_t gbase = grp * kGroup;
    float *pp = p + gbase + lane16 * 4;
    uint16_t *mcp = reinterpret_cast<uint16_t *>(m_codes + (gbase >> 1)) + lane16;
    // the small loads that feed LDS first (they return first), then the group's loads
    const LdsFill fill = lds_fill_load(qmap_m, qmap_m);
    float4 a0, a1, b0, b1, c_lo, c_hi;
    uint32_t w0 = 0, w1 = 0;
    float sm = 0.0f, row_r = 0.0f, mean_all = 1.0f;
    if (live) {
        const float *gp = g + gbase + lane16 * 4;
        const float *cp = col + (int64_t)cb * kGroup + lane16 * 4;
        a0 = load4(pp);
        a1 = load4(pp + 64);
        b0 = load4(gp);
        b1 = load4(gp + 64);
        c_lo = *reinterpret_cast<const float4 *>(cp);
        c_hi = *reinterpret_cast<const float4 *>(cp + 64);
        if (!first_step) {
            w0 = load_u16(mcp);
            w1 = load_u16(mcp + 16);
            sm = m_max1[grp];
        }
        row_r = row[r];
        mean_all = *row_mean_all;
    }
    lds_fill_store(lds, fill);
    const int kind = classify_map(qmap_m);
    lds_barrier();
    if (tile == 0) {
        const float z[kFElts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t wz = kind == kMapStdM ? encode8_std_m(lds, z)
                                             : encode8_generic(make_mids(reinterpret_cast<const float *>(lds) + kLdsQ0 / 4), z);
        for (int64_t i = n + (int64_t)threadIdx.x * kFElts; i < n_padded; i += kFTile)
            *reinterpret_cast<uint32_t *>(m_codes + (i >> 1)) = wz;
        if (threadIdx.x == 0)
            m_codes[n_padded / 2] = 0;
    }
    if (!live)
        return;
    const uint32_t wm = w0 | (w1 << 16);
    const Nibbles nm = split_nibbles(wm);
    const float rf = row_r / mean_all;
    float pv[kFElts] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const float gv[kFElts] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
    const float cv[kFElts] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
    float m[kFElts];
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kFElts; ++k) {
        const float m_old = first_step ? 0.0f : decode_nibble(lds, kLdsQ0, nm, k) * sm;
        const float pi = pv[k] * h.decay;
        m[k] = lerp_w(m_old, gv[k], h.w1);
        const float vi = rf * cv[k];
        const float denom = div_by_rc(sqrt_fast(vi), h.bc2_sqrt, h.rbc2_sqrt) + h.eps;
        pv[k] = pi + div_fast(h.neg_step_size * m[k], denom);
        amax = fmaxf(amax, fabsf(m[k]));
    }
    amax = row16_max(amax);
    const uint32_t om = encode8_scaled(lds, kLdsQ0, kind, m, amax);
    store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
    store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
    store_u16(mcp, om & 0xFFFFu);
    store_u16(mcp + 16, om >> 16);
    if (lane16 == 0)
        m_max1[grp] = amax;
}

__global__ __launch_bounds__(kFThreads) void factored_update_rows128_kernel(
    float *__restrict__ p, const float *__restrict__ g, uint8_t *__restrict__ m_codes,
    float *__restrict__ m_max1, const float *__restrict__ qmap_m, const float *__restrict__ row,
    const float *__restrict__ col, const float *__restrict__ row_mean_all, int64_t R, int64_t C,
    int64_t n_padded, NfHyper h, bool first_step)
{
    update_rows128_body(p, g, m_codes, m_max1, qmap_m, row, col, row_mean_all, R, C, n_padded, h, first_step,
                        blockIdx.x);
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
        const float denom = div_by_rc(sqrt_fast(vi), h.bc2_sqrt, h.rbc2_sqrt) + h.eps;
        p[i] = pi + div_fast(h.neg_step_size * mi, denom);
        m[i] = mi;
    }
}

// ---------------------------------------------------------------------------------------
// The whole factored step for a list of tensors: the three statistics kernels and the update
// run once per launch group instead of once per tensor.  Each workgroup finds its tensor in
// a prefix sum of workgroup counts kept in the kernel arguments and then does exactly what
// the single-tensor kernels above do.
// ---------------------------------------------------------------------------------------
constexpr int kFaMax = 24;  // tensors per launch group

struct TensorFa {
    float *p;
    const float *g;
    uint8_t *mc;
    float *ms;
    float *row;
    float *col;
    double *colpart;
    double *rowpart;
    double *rowblock;
    float *mean;
    int64_t R, C;
    int64_t n_padded;
    uint32_t tiles_x, tiles_y;  // statistics tiles
    uint32_t row_blocks;        // finalize: workgroups that take rows; the rest take 64 columns each
    uint32_t upd_x;             // update: 2048-element tiles of the tensor
    uint32_t first_step;
    float neg_step_size, bc2_sqrt, rbc2_sqrt;
};

// Launch groups are bounded by the tensor count alone.  Both passes stream the gradient from HBM
// (nontemporal loads): batches small enough for the statistics pass to leave the gradient in the
// 256 MB memory-side cache for the update were measured too (384 MB per batch: 10.6 ms per step on
// LLaMA-7B MLP shapes against 10.4 with groups bounded by the tensor count alone and streaming
// loads in the statistics pass).

struct MultiFa {
    TensorFa t[kFaMax];
    // prefix sums of workgroups per tensor for the three big kernels; unused slots hold the total
    uint32_t start_stats[kFaMax + 1], start_fin[kFaMax + 1], start_upd[kFaMax + 1];
    int count;
    float decay, w1, b2, w2, eps;
};

static_assert(sizeof(MultiFa) + sizeof(void *) <= 4096, "kernel arguments exceed 4 KB");
static_assert(kFaMax <= kWave, "one prefix-sum entry per lane");

__device__ __forceinline__ int find_slot(const uint32_t (&start)[kFaMax + 1], uint32_t block)
{
    const int lane = threadIdx.x & (kWave - 1);
    const bool started = lane + 1 < kFaMax && start[lane + 1] <= block;
    return __popcll(__ballot(started));
}

__global__ __launch_bounds__(kFThreads) void factored_partial_multi_kernel(const MultiFa args)
{
    const int i = find_slot(args.start_stats, blockIdx.x);
    const TensorFa &t = args.t[i];
    const uint32_t local = blockIdx.x - args.start_stats[i];
    const uint32_t by = local / t.tiles_x, bx = local - by * t.tiles_x;
    partial_body(t.g, t.R, t.C, t.colpart, t.rowpart, true, bx, by);
}

__global__ __launch_bounds__(kFThreads) void factored_finalize_multi_kernel(const MultiFa args)
{
    const int i = find_slot(args.start_fin, blockIdx.x);
    const TensorFa &t = args.t[i];
    finalize_body(t.colpart, t.rowpart, t.rowblock, t.R, t.C, (int)t.tiles_y, (int)t.tiles_x, (int)t.row_blocks,
                  t.row, t.col, args.b2, args.w2, blockIdx.x - args.start_fin[i]);
}

__global__ void factored_mean_multi_kernel(const MultiFa args)
{
    const TensorFa &t = args.t[blockIdx.x];
    if (threadIdx.x == 0) {
        double s = 0.0;
        for (uint32_t b = 0; b < t.row_blocks; ++b)
            s += t.rowblock[b];
        *t.mean = (float)(s / (double)t.R);
    }
}

__global__ __launch_bounds__(kFThreads) void factored_update_multi_kernel(const MultiFa args,
                                                                          const float *__restrict__ qmap_m)
{
    const uint32_t block = blockIdx.x;
    const int i = find_slot(args.start_upd, block);
    const TensorFa &t = args.t[i];
    const uint32_t local = block - args.start_upd[i];
    NfHyper h;
    h.decay = args.decay;
    h.w1 = args.w1;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.eps = args.eps;
    h.neg_step_size = t.neg_step_size;
    h.bc2_sqrt = t.bc2_sqrt;
    h.rbc2_sqrt = t.rbc2_sqrt;
    update_rows128_body(t.p, t.g, t.mc, t.ms, qmap_m, t.row, t.col, t.mean, t.R, t.C, t.n_padded, h,
                        t.first_step != 0, local);
}

inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

// update tiles of a rows x cols tensor (cols a multiple of 128)
inline uint64_t update_tiles(int64_t rows, int64_t cols)
{
    constexpr int64_t kTR = kFaTileRows, kGPS = (kFTile / kGroup) / kTR;
    return (uint64_t)(((rows + kTR - 1) / kTR) * ((cols / kGroup + kGPS - 1) / kGPS));
}

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
    const int64_t blocks = (n + kFThreads * 4 - 1) / (kFThreads * 4);
    if (blocks > 0x7fffffffLL)
        return LPMM_ERR_SIZE;
    const bool vec = aligned_to(p, 16) && aligned_to(g, 16) && aligned_to(m, 16) && aligned_to(v, 16);
    hipLaunchKernelGGL(nonfused_update_kernel, dim3((uint32_t)blocks), dim3(kFThreads), 0,
                       (hipStream_t)stream, p, g, m, v, n,
                       make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step), vec);
    return launch_status();
}

extern "C" int64_t lpmm_factored_workspace_bytes(int64_t rows, int64_t cols)
{
    if (rows <= 0 || cols <= 0)
        return 0;
    const int64_t ty = (rows + kSRows - 1) / kSRows, tx = (cols + kSCols - 1) / kSCols;
    const int64_t row_blocks = (rows + kFThreads - 1) / kFThreads;
    // column partials, row partials, per-workgroup sums of the new row statistics, and (used by
    // the multi-tensor step only) mean(row)
    return (ty * cols + tx * rows + row_blocks + 1) * (int64_t)sizeof(double);
}

// argument checks shared by the two forms of the statistics pass
static int factored_stats_check(const float *g, int64_t rows, int64_t cols, const float *row, const float *col,
                                const float *row_mean_all)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(g);
    LPMM_REQUIRE_PTR(row);
    LPMM_REQUIRE_PTR(col);
    LPMM_REQUIRE_PTR(row_mean_all);
    LPMM_REQUIRE_ALIGN(g, 4);
    LPMM_REQUIRE_ALIGN(row, 4);
    LPMM_REQUIRE_ALIGN(col, 4);
    LPMM_REQUIRE_ALIGN(row_mean_all, 4);
    const int64_t ty = (rows + kSRows - 1) / kSRows, tx = (cols + kSCols - 1) / kSCols;
    const int64_t row_blocks = (rows + kFThreads - 1) / kFThreads;
    const int64_t col_blocks = (cols + 63) / 64;
    if (ty > 65535 || tx > 0x7fffffffLL || row_blocks + col_blocks > 0x7fffffffLL)
        return LPMM_ERR_SIZE;
    return LPMM_OK;
}

// the three launches of the statistics pass; `workspace` is a device address of at least
// lpmm_factored_workspace_bytes(rows, cols) bytes, 8-byte aligned
static int factored_stats_launch(const float *g, int64_t rows, int64_t cols, float *row, float *col,
                                 float *row_mean_all, double beta2, void *workspace, void *stream)
{
    const int64_t ty = (rows + kSRows - 1) / kSRows, tx = (cols + kSCols - 1) / kSCols;
    double *colpart = static_cast<double *>(workspace);
    double *rowpart = colpart + ty * cols;
    double *rowblock = rowpart + tx * rows;
    const int64_t row_blocks = (rows + kFThreads - 1) / kFThreads;
    const int64_t col_blocks = (cols + 63) / 64;
    const bool vec = aligned_to(g, 16) && (cols % 4) == 0;
    hipLaunchKernelGGL(factored_partial_kernel, dim3((uint32_t)tx, (uint32_t)ty), dim3(kFThreads), 0,
                       (hipStream_t)stream, g, rows, cols, colpart, rowpart, vec);
    int st = launch_status();
    if (st != LPMM_OK)
        return st;
    hipLaunchKernelGGL(factored_finalize_kernel, dim3((uint32_t)(row_blocks + col_blocks)), dim3(kFThreads), 0,
                       (hipStream_t)stream, colpart, rowpart, rowblock, rows, cols, (int)ty, (int)tx,
                       (int)row_blocks, row, col, (float)beta2, (float)(1.0 - beta2));
    st = launch_status();
    if (st != LPMM_OK)
        return st;
    hipLaunchKernelGGL(factored_mean_kernel, dim3(1), dim3(kWave), 0, (hipStream_t)stream, rowblock,
                       (int)row_blocks, rows, row_mean_all);
    return launch_status();
}

extern "C" int lpmm_factored_stats(const float *g, int64_t rows, int64_t cols, float *row, float *col,
                                   float *row_mean_all, double beta2, void *workspace, void *stream)
{
    const int st = factored_stats_check(g, rows, cols, row, col, row_mean_all);
    if (st != LPMM_OK)
        return st;
    LPMM_REQUIRE_PTR(workspace);
    LPMM_REQUIRE_ALIGN(workspace, 8);
    return factored_stats_launch(g, rows, cols, row, col, row_mean_all, beta2, workspace, stream);
}

// The workspace of lpmm_factored_stats_static: one array per GPU, held by the library's code
// object until the process ends.  In host code the name below is only a handle for
// hipGetSymbolAddress; kernels receive the device address that call returns.
static __device__ __align__(256) unsigned char scratch[LPMM_FACTORED_STATIC_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices];  // the current device's copy of `scratch`, looked up once per device
}  // namespace

extern "C" int lpmm_factored_stats_static(const float *g, int64_t rows, int64_t cols, float *row, float *col,
                                          float *row_mean_all, double beta2, void *stream)
{
    const int st = factored_stats_check(g, rows, cols, row, col, row_mean_all);
    if (st != LPMM_OK)
        return st;
    if (lpmm_factored_workspace_bytes(rows, cols) > (int64_t)LPMM_FACTORED_STATIC_BYTES)
        return LPMM_ERR_SIZE;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return LPMM_ERR_LAUNCH;
    // The address is looked up on the first call on each GPU (callers make that call outside stream
    // capture); afterwards this block only reads the cached pointer.
    void *ws = nullptr;
    {
        std::lock_guard<std::mutex> hold(g_scratch_lock);
        if (g_scratch_ptr[dev] == nullptr) {
            void *ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
                (void)hipGetLastError();
                return LPMM_ERR_LAUNCH;
            }
            g_scratch_ptr[dev] = ptr;
        }
        ws = g_scratch_ptr[dev];
    }
    // every partial the finalize kernels read is written by the partial kernel of the same call:
    // nothing in the array has to start at zero
    return factored_stats_launch(g, rows, cols, row, col, row_mean_all, beta2, ws, stream);
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
    const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step);
    if ((cols % kGroup) == 0 && vec && aligned_to(col, 16) && aligned_to(m_codes, 4)) {
        const uint64_t row_tiles = update_tiles(rows, cols);
        if (row_tiles > 0x7fffffffULL)
            return LPMM_ERR_SIZE;
        hipLaunchKernelGGL(factored_update_rows128_kernel, dim3((uint32_t)row_tiles), dim3(kFThreads), 0,
                           (hipStream_t)stream, p, g, m_codes, m_max1, qmap_m, row, col, row_mean_all, rows, cols,
                           n_padded, h, first_step != 0);
    } else if ((cols % 8) == 0 && aligned_to(col, 16))
        hipLaunchKernelGGL(factored_update_kernel<true>, dim3((uint32_t)tiles), dim3(kFThreads), 0,
                           (hipStream_t)stream, p, g, m_codes, m_max1, qmap_m, row, col, row_mean_all, n, cols,
                           n_groups, n_padded, h, first_step != 0, vec);
    else
        hipLaunchKernelGGL(factored_update_kernel<false>, dim3((uint32_t)tiles), dim3(kFThreads), 0,
                           (hipStream_t)stream, p, g, m_codes, m_max1, qmap_m, row, col, row_mean_all, n, cols,
                           n_groups, n_padded, h, first_step != 0, vec);
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

extern "C" int lpmm_factored_step_multi(const lpmm_factored_tensor *tensors, int64_t count, const float *qmap_m,
                                        double beta1, double beta2, double lr, double weight_decay, double eps,
                                        void *stream)
{
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(tensors);
    LPMM_REQUIRE_PTR(qmap_m);
    LPMM_REQUIRE_ALIGN(qmap_m, 4);
    for (int64_t i = 0; i < count; ++i) {
        const lpmm_factored_tensor &t = tensors[i];
        if (t.rows <= 0 || t.cols <= 0 || t.cols % kGroup != 0 || t.rows > INT64_MAX / t.cols)
            return LPMM_ERR_SIZE;
        const int64_t ty = (t.rows + kSRows - 1) / kSRows, tx = (t.cols + kSCols - 1) / kSCols;
        const int64_t ux = (t.cols + kFTile - 1) / kFTile + 1;  // per row: an upper bound for any tile shape
        if (tx > 0x7fffffffLL / ty || ux > 0x7fffffffLL / t.rows ||
            (t.rows + kFThreads - 1) / kFThreads + (t.cols + 63) / 64 > 0x7fffffffLL)
            return LPMM_ERR_SIZE;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(t.m_codes);
        LPMM_REQUIRE_PTR(t.m_max1);
        LPMM_REQUIRE_PTR(t.row);
        LPMM_REQUIRE_PTR(t.col);
        LPMM_REQUIRE_PTR(t.workspace);
        LPMM_REQUIRE_ALIGN(t.p, 16);
        LPMM_REQUIRE_ALIGN(t.g, 16);
        LPMM_REQUIRE_ALIGN(t.m_codes, 4);
        LPMM_REQUIRE_ALIGN(t.m_max1, 4);
        LPMM_REQUIRE_ALIGN(t.row, 4);
        LPMM_REQUIRE_ALIGN(t.col, 16);
        LPMM_REQUIRE_ALIGN(t.workspace, 8);
    }

    const NfHyper c = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, 1.0);
    MultiFa args;
    args.decay = c.decay;
    args.w1 = c.w1;
    args.b2 = c.b2;
    args.w2 = c.w2;
    args.eps = c.eps;
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t n_stats = 0, n_fin = 0, n_upd = 0;
        args.start_stats[0] = args.start_fin[0] = args.start_upd[0] = 0;
        while (i < count && k < kFaMax) {
            const lpmm_factored_tensor &t = tensors[i];
            const uint64_t ty = (uint64_t)((t.rows + kSRows - 1) / kSRows), tx = (uint64_t)((t.cols + kSCols - 1) / kSCols);
            const uint64_t row_blocks = (uint64_t)((t.rows + kFThreads - 1) / kFThreads);
            const uint64_t fin = row_blocks + (uint64_t)((t.cols + 63) / 64);
            const uint64_t ux = update_tiles(t.rows, t.cols);
            if (n_stats + tx * ty > 0x7fffffffULL || n_fin + fin > 0x7fffffffULL ||
                n_upd + ux > 0x7fffffffULL) {
                if (k == 0)
                    return LPMM_ERR_SIZE;  // cannot happen after the checks above
                break;
            }
            TensorFa &d = args.t[k];
            d.p = t.p;
            d.g = t.g;
            d.mc = t.m_codes;
            d.ms = t.m_max1;
            d.row = t.row;
            d.col = t.col;
            d.colpart = static_cast<double *>(t.workspace);
            d.rowpart = d.colpart + ty * (uint64_t)t.cols;
            d.rowblock = d.rowpart + tx * (uint64_t)t.rows;
            d.mean = reinterpret_cast<float *>(d.rowblock + row_blocks);
            d.R = t.rows;
            d.C = t.cols;
            d.n_padded = round_up(t.rows * t.cols, kFTile);
            d.tiles_x = (uint32_t)tx;
            d.tiles_y = (uint32_t)ty;
            d.row_blocks = (uint32_t)row_blocks;
            d.upd_x = (uint32_t)ux;
            d.first_step = t.first_step != 0;
            const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, t.step);
            d.neg_step_size = h.neg_step_size;
            d.bc2_sqrt = h.bc2_sqrt;
            d.rbc2_sqrt = h.rbc2_sqrt;
            n_stats += tx * ty;
            n_fin += fin;
            n_upd += ux;
            ++k;
            args.start_stats[k] = (uint32_t)n_stats;
            args.start_fin[k] = (uint32_t)n_fin;
            args.start_upd[k] = (uint32_t)n_upd;
            ++i;
        }
        args.count = k;
        for (int j = k + 1; j <= kFaMax; ++j) {
            args.start_stats[j] = (uint32_t)n_stats;
            args.start_fin[j] = (uint32_t)n_fin;
            args.start_upd[j] = (uint32_t)n_upd;
        }
        hipStream_t s = (hipStream_t)stream;
        hipLaunchKernelGGL(factored_partial_multi_kernel, dim3((uint32_t)n_stats), dim3(kFThreads), 0, s, args);
        hipLaunchKernelGGL(factored_finalize_multi_kernel, dim3((uint32_t)n_fin), dim3(kFThreads), 0, s, args);
        hipLaunchKernelGGL(factored_mean_multi_kernel, dim3((uint32_t)k), dim3(kWave), 0, s, args);
        hipLaunchKernelGGL(factored_update_multi_kernel, dim3((uint32_t)n_upd), dim3(kFThreads), 0, s, args, qmap_m);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}
