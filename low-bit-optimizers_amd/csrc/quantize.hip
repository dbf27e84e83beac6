// Stand-alone 4-bit quantise / dequantise kernels for gfx950 in the non-fused packed layout
// of lpmm: codes of the flattened, zero-padded tensor, two per byte (low nibble = even
// index), padded to a multiple of 2048 values, plus one trailing byte
// (lpmm/functional.py:359-369, lpmm/cpp_extension/quantization_kernel.cu:430-477).
//
// A lane owns 8 consecutive values = one 32-bit word of codes; a 256-thread workgroup
// covers one 2048-value pack group.  Group maxima use DPP row reductions (128 values =
// 16 lanes) and, for larger groups, 16 floats of LDS per workgroup.  Code assignment uses
// the table / closed-form encoders of lpmm_codec.hpp when the map is one of the two
// standard ones and the count-of-midpoints search otherwise.
#include "lpmm_codec.hpp"

namespace lpmm {

constexpr int kQThreads = 256;
static_assert(kQThreads == kEncEntries, "lds_fill_load / lds_fill_store: one encode-table entry per thread");
constexpr int kQElts = 8;
constexpr int kQTile = kQThreads * kQElts;  // 2048

__device__ __forceinline__ void load8(const float *__restrict__ x, int64_t base, int64_t n, bool vec,
                                      float (&v)[kQElts])
{
    if (vec && base + kQElts <= n) {
        const float4 a = load4(x + base), b = load4(x + base + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
        for (int k = 0; k < kQElts; ++k)
            v[k] = (base + k < n) ? x[base + k] : 0.0f;
    }
}

__device__ __forceinline__ void store8(float *__restrict__ out, int64_t base, int64_t n, bool vec,
                                       const float (&v)[kQElts])
{
    if (vec && base + kQElts <= n) {
        store4(out + base, make_float4(v[0], v[1], v[2], v[3]));
        store4(out + base + 4, make_float4(v[4], v[5], v[6], v[7]));
    } else {
#pragma unroll
        for (int k = 0; k < kQElts; ++k)
            if (base + k < n)
                out[base + k] = v[k];
    }
}

// codes hold at least ceil(n/2) bytes; whole words are read only where they lie inside.
__device__ __forceinline__ uint32_t load_codes8(const uint8_t *__restrict__ codes, int64_t base, int64_t n,
                                                bool vec)
{
    if (vec && base + kQElts <= n)
        return load_u32(reinterpret_cast<const uint32_t *>(codes + (base >> 1)));
    uint32_t w = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (base + 2 * k < n)
            w |= (uint32_t)codes[(base >> 1) + k] << (8 * k);
    return w;
}

// ---------------------------------------------------------------------------------------
// pack_nonlinear / unpack_nonlinear (values already normalised)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kQThreads) void pack4_kernel(const float *__restrict__ x,
                                                          const float *__restrict__ qmap,
                                                          int64_t n_padded, uint8_t *__restrict__ out,
                                                          bool vec)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    lds_fill(lds, qmap, nullptr);
    const int kind = classify_map(qmap);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) * kQElts;
    if (base == 0)
        out[n_padded / 2] = 0;
    if (base >= n_padded)
        return;
    float v[kQElts];
    load8(x, base, n_padded, vec, v);
    const uint32_t w = encode8_plain(lds, kLdsQ0, kind, v);
    if (vec) {
        store_u32(reinterpret_cast<uint32_t *>(out + (base >> 1)), w);
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            out[(base >> 1) + k] = (uint8_t)(w >> (8 * k));
    }
}

__global__ __launch_bounds__(kQThreads) void unpack4_kernel(const uint8_t *__restrict__ codes,
                                                            const float *__restrict__ qmap, int64_t n,
                                                            float *__restrict__ out, bool vec)
{
    __shared__ __align__(16) uint32_t lds[32];
    if (threadIdx.x < 16)
        lds[threadIdx.x] = __float_as_uint(qmap[threadIdx.x]);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) * kQElts;
    if (base >= n)
        return;
    const Nibbles nb = split_nibbles(load_codes8(codes, base, n, vec));
    float v[kQElts];
#pragma unroll
    for (int k = 0; k < kQElts; ++k)
        v[k] = decode_nibble(lds, kLdsQ0, nb, k);
    store8(out, base, n, vec, v);
}

// ---------------------------------------------------------------------------------------
// 'group' scaling: max|x| per gp_sz values, x / max, search, pack -- one pass.
// rows_per_group = gp_sz / 128 in {1, 2, 4, 8, 16, 32}.
// ---------------------------------------------------------------------------------------
// THREADS: 256 (a tile is one 2048-value pack group) or, for gp_sz 4096, 512; a workgroup
// handles T consecutive tiles, so that the set-up of the LDS tables is paid once per T tiles.
// A workgroup whose values all lie inside the tensor (and whose operands allow vector access)
// works in the row layout of the fused step: 16 lanes own 128 consecutive values, lane l the
// values [4l, 4l+4) and [64+4l, 64+4l+4), so every 16-byte load of a row covers whole cache
// lines; the loads of all its tiles are issued before the LDS tables are set up.  Other
// workgroups (the ragged end, the padding) let every lane own 8 consecutive values and guard
// each access.
template <int THREADS, int T>
__global__ __launch_bounds__(THREADS) void quant_group_kernel(const float *__restrict__ x, int64_t n,
                                                              int rows_per_group,
                                                              const float *__restrict__ qmap,
                                                              uint8_t *__restrict__ codes,
                                                              float *__restrict__ max1, int64_t n_groups,
                                                              int64_t n_padded, bool vec)
{
    constexpr int kTileElts = THREADS * kQElts;
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    __shared__ float s_row[T][THREADS / 16];
    // the workgroup's span of T tiles, in the launch order that lets an XCD stream 128 KB runs of x
    constexpr int kSpanLog2 = (T * kTileElts * sizeof(float) == 16384) ? 3 : ((T * kTileElts * sizeof(float) == 8192) ? 4 : -1);
    uint32_t span = blockIdx.x;
    if constexpr (kSpanLog2 > 0)
        span = xcd_run_order<kSpanLog2>(span, gridDim.x, run_phase<kSpanLog2>(x, T * kTileElts * sizeof(float)));
    const int64_t tile0 = (int64_t)span * T * kTileElts;
    const int lane16 = threadIdx.x & 15;
    const int wrow = threadIdx.x >> 4;
    const int64_t gp_sz = (int64_t)rows_per_group * kGroup;
    const int first = wrow & ~(rows_per_group - 1);

    if (vec && tile0 + (int64_t)T * kTileElts <= n) {  // uniform over the workgroup
        float v[T][kQElts];
        // the small loads that feed LDS first (they return first), then the tiles' loads (workgroups
        // of one thread per encode-table entry; larger ones fill the tables after their loads)
        LdsFill fill;
        if (THREADS == kEncEntries)
            fill = lds_fill_load(qmap, qmap);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float *p = x + tile0 + (int64_t)t * kTileElts + wrow * kGroup + lane16 * 4;
            const float4 a = load4(p), b = load4(p + 64);
            v[t][0] = a.x; v[t][1] = a.y; v[t][2] = a.z; v[t][3] = a.w;
            v[t][4] = b.x; v[t][5] = b.y; v[t][6] = b.z; v[t][7] = b.w;
        }
        if (THREADS == kEncEntries)
            lds_fill_store(lds, fill);
        else
            lds_fill(lds, qmap, nullptr);
        const int kind = classify_map(qmap);
        if (tile0 == 0 && threadIdx.x == 0)
            codes[n_padded / 2] = 0;
        float amax[T];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            float m = 0.0f;
#pragma unroll
            for (int k = 0; k < kQElts; ++k)
                m = fmaxf(m, fabsf(v[t][k]));
            amax[t] = row16_max(m);
            if (lane16 == 0)
                s_row[t][wrow] = amax[t];
        }
        lds_barrier();
#pragma unroll
        for (int t = 0; t < T; ++t) {
            if (rows_per_group > 1) {
                amax[t] = s_row[t][first];
                for (int r = 1; r < rows_per_group; ++r)
                    amax[t] = fmaxf(amax[t], s_row[t][first + r]);
            }
            const int64_t base = tile0 + (int64_t)t * kTileElts + wrow * kGroup;
            if ((base % gp_sz) == 0 && lane16 == 0)
                max1[base / gp_sz] = amax[t];
            const uint32_t w = encode8_scaled(lds, kLdsQ0, kind, v[t], amax[t]);
            uint16_t *cp = reinterpret_cast<uint16_t *>(codes + (base >> 1)) + lane16;
            store_u16(cp, w & 0xFFFFu);
            store_u16(cp + 16, w >> 16);
        }
        return;
    }

    lds_fill(lds, qmap, nullptr);
    const int kind = classify_map(qmap);
    if (tile0 == 0 && threadIdx.x == 0)
        codes[n_padded / 2] = 0;
    for (int t = 0; t < T; ++t) {  // uniform trip count: the barriers below are reached by all
        const int64_t base = tile0 + (int64_t)t * kTileElts + (int64_t)threadIdx.x * kQElts;
        float v[kQElts];
        load8(x, base, n, vec, v);  // zero beyond n: the reference's zero padding
        float amax = 0.0f;
#pragma unroll
        for (int k = 0; k < kQElts; ++k)
            amax = fmaxf(amax, fabsf(v[k]));
        amax = row16_max(amax);
        __syncthreads();  // the previous tile's readers are done (and, first, the tables are in)
        if (lane16 == 0)
            s_row[0][wrow] = amax;
        __syncthreads();
        if (rows_per_group > 1) {
            amax = s_row[0][first];
            for (int r = 1; r < rows_per_group; ++r)
                amax = fmaxf(amax, s_row[0][first + r]);
        }
        const int64_t grp = base / gp_sz;
        uint32_t w;
        if (grp < n_groups) {
            if ((base % gp_sz) == 0)
                max1[grp] = amax;
            w = encode8_scaled(lds, kLdsQ0, kind, v, amax);
        } else {
            // padding added by the re-grouping to 2048: plain zeros, not divided by anything
            const float z[kQElts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            w = encode8_plain(lds, kLdsQ0, kind, z);
        }
        if (base < n_padded)  // the last workgroup may reach past the last pack group
            store_u32(reinterpret_cast<uint32_t *>(codes + (base >> 1)), w);
    }
}

__global__ __launch_bounds__(kQThreads) void dequant_group_kernel(const uint8_t *__restrict__ codes,
                                                                  const float *__restrict__ max1,
                                                                  const float *__restrict__ qmap, int64_t n,
                                                                  int64_t gp_sz, float *__restrict__ out,
                                                                  bool vec)
{
    __shared__ __align__(16) uint32_t lds[32];
    if (threadIdx.x < 16)
        lds[threadIdx.x] = __float_as_uint(qmap[threadIdx.x]);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) * kQElts;
    if (base >= n)
        return;
    const Nibbles nb = split_nibbles(load_codes8(codes, base, n, vec));
    const float s = max1[base / gp_sz];  // gp_sz is a multiple of 128, so uniform over the lane's 8
    float v[kQElts];
#pragma unroll
    for (int k = 0; k < kQElts; ++k)
        v[k] = decode_nibble(lds, kLdsQ0, nb, k) * s;
    store8(out, base, n, vec, v);
}

// Row layout (as in the fused step): 16 lanes own one 128-value group, lane l owns values
// [4l, 4l+4) and [64+4l, 64+4l+4), so that every 16-byte store of a row covers whole cache
// lines.  Handles the groups that lie fully inside the tensor; n must be >= 128.
#ifndef LPMM_DQ_LDS_KB
#define LPMM_DQ_LDS_KB 0
#endif
// the map needs 16 words (32 allocated); more caps the workgroups resident per CU
constexpr int kDequantLdsWords = LPMM_DQ_LDS_KB > 0 ? LPMM_DQ_LDS_KB * 256 : 32;
template <int T>
__global__ __launch_bounds__(kQThreads) void dequant_group_rows_kernel(const uint8_t *__restrict__ codes,
                                                                       const float *__restrict__ max1,
                                                                       const float *__restrict__ qmap,
                                                                       int64_t full_groups, int rows_per_group,
                                                                       float *__restrict__ out)
{
    __shared__ __align__(16) uint32_t lds[kDequantLdsWords];
    const int lane16 = threadIdx.x & 15;
    // T passes of 16 rows each; the loads of all passes first, the map afterwards
    // the workgroup's span of T x 16 rows, in the launch order that lets an XCD stream 128 KB runs of the output
    constexpr int kSpanLog2 = (T * 2048 * sizeof(float) == 16384) ? 3 : ((T * 2048 * sizeof(float) == 8192) ? 4 : -1);
    uint32_t span = blockIdx.x;
    if constexpr (kSpanLog2 > 0)
        span = xcd_run_order<kSpanLog2>(span, gridDim.x, run_phase<kSpanLog2>(out, T * 2048 * sizeof(float)));
    const int64_t row0 = (int64_t)span * T * (kQThreads / 16) + (threadIdx.x >> 4);
    uint32_t c0[T], c1[T];
    float s[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int64_t row = row0 + t * (kQThreads / 16);
        c0[t] = c1[t] = 0;
        s[t] = 0.0f;
        if (row < full_groups) {
            const uint16_t *cp = reinterpret_cast<const uint16_t *>(codes + row * 64) + lane16;
            c0[t] = load_u16(cp);
            c1[t] = load_u16(cp + 16);
            s[t] = max1[row / rows_per_group];
        }
    }
    if (threadIdx.x < 16)
        lds[threadIdx.x] = __float_as_uint(qmap[threadIdx.x]);
    lds_barrier();
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int64_t row = row0 + t * (kQThreads / 16);
        if (row >= full_groups)
            continue;
        const Nibbles nb = split_nibbles(c0[t] | (c1[t] << 16));
        float v[kQElts];
#pragma unroll
        for (int k = 0; k < kQElts; ++k)
            v[k] = decode_nibble(lds, kLdsQ0, nb, k) * s[t];
        float *o = out + row * kGroup + lane16 * 4;
        store4(o, make_float4(v[0], v[1], v[2], v[3]));
        store4(o + 64, make_float4(v[4], v[5], v[6], v[7]));
    }
}

// ---------------------------------------------------------------------------------------
// 'rank1' scaling of a row-major R x C tensor.
// ---------------------------------------------------------------------------------------
__global__ void fill_zero_kernel(float *__restrict__ a, int64_t na, float *__restrict__ b, int64_t nb)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < na)
        a[i] = 0.0f;
    if (i < nb)
        b[i] = 0.0f;
}

constexpr int kStatRows = 64;
constexpr int kStatCols = 1024;  // 256 threads x 4 columns
constexpr int kStatUnroll = 8;   // rows in flight per lane

// Tile of kStatRows x kStatCols; a lane keeps 4 column maxima in registers, row maxima are
// reduced over the wave and merged with atomics (max is exact and order-independent).
__global__ __launch_bounds__(kQThreads) void rank1_stats_kernel(const float *__restrict__ x, int64_t R,
                                                                int64_t C, float *__restrict__ rowmax,
                                                                float *__restrict__ colmax, bool vec)
{
    const int64_t c0 = (int64_t)blockIdx.x * kStatCols + (int64_t)threadIdx.x * 4;
    const int64_t r0 = (int64_t)blockIdx.y * kStatRows;
    const int64_t r1 = (r0 + kStatRows < R) ? r0 + kStatRows : R;
    const bool lane_vec = vec && c0 + 4 <= C;
    float cm[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int64_t rb = r0; rb < r1; rb += kStatUnroll) {
        float a[kStatUnroll][4];
        if (lane_vec && rb + kStatUnroll <= r1) {
            // straight-line: all loads of the batch are in flight before the first use
            float4 t[kStatUnroll];
#pragma unroll
            for (int u = 0; u < kStatUnroll; ++u)
                t[u] = load4(x + (rb + u) * C + c0);
#pragma unroll
            for (int u = 0; u < kStatUnroll; ++u) {
                a[u][0] = fabsf(t[u].x); a[u][1] = fabsf(t[u].y); a[u][2] = fabsf(t[u].z); a[u][3] = fabsf(t[u].w);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kStatUnroll; ++u) {
                const int64_t r = rb + u;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    a[u][k] = (r < r1 && c0 + k < C) ? fabsf(x[r * C + c0 + k]) : 0.0f;
            }
        }
        float rm[kStatUnroll];
#pragma unroll
        for (int u = 0; u < kStatUnroll; ++u) {
            rm[u] = fmaxf(fmaxf(a[u][0], a[u][1]), fmaxf(a[u][2], a[u][3]));
#pragma unroll
            for (int k = 0; k < 4; ++k)
                cm[k] = fmaxf(cm[k], a[u][k]);
        }
        // the wave's 8 row maxima at once: lane 8u holds the maximum of row rb + u
        static_assert(kStatUnroll == 8, "wave_max8 reduces eight rows");
        const int lane = threadIdx.x & 63;
        const float m = wave_max8(rm, lane);
        if ((lane & 7) == 0 && rb + (lane >> 3) < r1)
            atomic_max_nonneg(rowmax + rb + (lane >> 3), m);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (c0 + k < C)
            atomic_max_nonneg(colmax + c0 + k, cm[k]);
}

// The same statistics, one-shot: a workgroup takes a tile of 32 rows x 256 columns, a wave 8 of
// those rows (a lane: 4 columns of each), and issues all its loads at once -- no loop, so the
// grid's many small workgroups keep the memory system busy the way a plain streaming read does.
// Column maxima of the four waves meet in LDS: one atomic per column and tile.  Requires whole
// tiles' worth of vector access: 16-byte aligned x, columns a multiple of 4.
constexpr int kStat2Rows = 32, kStat2Cols = 256;
#ifndef LPMM_STAT2_LDS_KB
#define LPMM_STAT2_LDS_KB 4
#endif

__global__ __launch_bounds__(kQThreads) void rank1_stats_tile_kernel(const float *__restrict__ x, int64_t R, int64_t C,
                                                                     uint32_t tiles_x, float *__restrict__ rowmax,
                                                                     float *__restrict__ colmax)
{
    __shared__ float s_col[LPMM_STAT2_LDS_KB * 256];  // [4 waves][256 columns] used; the rest caps residency
    const uint32_t ty = blockIdx.x / tiles_x, tx = blockIdx.x - ty * tiles_x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t c0 = (int64_t)tx * kStat2Cols + lane * 4;
    const int64_t r0 = (int64_t)ty * kStat2Rows + wave * 8;
    const bool cols_in = c0 + 4 <= C;
    float4 t[8];
    if (cols_in && r0 + 8 <= R) {
        const float *base = x + r0 * C + c0;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            t[u] = load4(base + (int64_t)u * C);
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            t[u] = (cols_in && r0 + u < R) ? load4(x + (r0 + u) * C + c0) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    float rm[8], cm[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const float a0 = fabsf(t[u].x), a1 = fabsf(t[u].y), a2 = fabsf(t[u].z), a3 = fabsf(t[u].w);
        rm[u] = fmaxf(fmaxf(a0, a1), fmaxf(a2, a3));
        cm[0] = fmaxf(cm[0], a0);
        cm[1] = fmaxf(cm[1], a1);
        cm[2] = fmaxf(cm[2], a2);
        cm[3] = fmaxf(cm[3], a3);
    }
    const float m = wave_max8(rm, lane);  // lane 8u: maximum of row r0 + u over the wave's 256 columns
    if ((lane & 7) == 0 && r0 + (lane >> 3) < R)
        atomic_max_nonneg(rowmax + r0 + (lane >> 3), m);
    *reinterpret_cast<float4 *>(s_col + wave * kStat2Cols + lane * 4) = make_float4(cm[0], cm[1], cm[2], cm[3]);
    __syncthreads();
    const int64_t c = (int64_t)tx * kStat2Cols + threadIdx.x;
    if (c < C) {
        const float v = fmaxf(fmaxf(s_col[threadIdx.x], s_col[kStat2Cols + threadIdx.x]),
                              fmaxf(s_col[2 * kStat2Cols + threadIdx.x], s_col[3 * kStat2Cols + threadIdx.x]));
        atomic_max_nonneg(colmax + c, v);
    }
}

// Normalise by min(rowmax[r], colmax[c]), search, pack.  Flattened indexing: a lane's 8
// values may straddle rows (any C).
__global__ __launch_bounds__(kQThreads) void quant_rank1_kernel(const float *__restrict__ x, int64_t n,
                                                                int64_t C, const float *__restrict__ rowmax,
                                                                const float *__restrict__ colmax,
                                                                const float *__restrict__ qmap,
                                                                uint8_t *__restrict__ codes, int64_t n_padded,
                                                                bool vec)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    lds_fill(lds, qmap, nullptr);
    const int kind = classify_map(qmap);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) * kQElts;
    if (base == 0)
        codes[n_padded / 2] = 0;
    float v[kQElts], xs[kQElts];
    load8(x, base, n, vec, v);
    int64_t r = base / C;
    int64_t c = base - r * C;
    float rm = (base < n) ? rowmax[r] : 0.0f;
#pragma unroll
    for (int k = 0; k < kQElts; ++k) {
        xs[k] = 0.0f;  // padding added by the re-grouping to 2048
        if (base + k < n) {
            const float cmx = colmax[c];
            const float st = (cmx < rm) ? cmx : rm;
            xs[k] = v[k] / st;
            if (++c == C) {
                c = 0;
                ++r;
                rm = (base + k + 1 < n) ? rowmax[r] : 0.0f;
            }
        }
    }
    store_u32(reinterpret_cast<uint32_t *>(codes + (base >> 1)), encode8_plain(lds, kLdsQ0, kind, xs));
}

// Codes of v[k] / min(cmx[k], rm) for a lane's 8 values of one row.  The column maxima stay the
// same for every row a lane handles, so their correctly rounded reciprocals are formed once
// (col_rcp); with the row's reciprocal that turns every division into one multiply and two fmas
// that give the correctly rounded quotient (|v| <= scale by construction).  Scales outside the
// range in which the reciprocal is exact, and maps other than the two standard ones, take the
// plain division and the generic search.
struct ColRcp {
    float rc[kQElts];
    bool safe;
};

__device__ __forceinline__ ColRcp col_rcp(const float (&cmx)[kQElts])
{
    ColRcp c;
    c.safe = true;
#pragma unroll
    for (int k = 0; k < kQElts; ++k) {
        c.rc[k] = rcp_exact(cmx[k]);
        c.safe = c.safe && rc_safe(cmx[k]);
    }
    return c;
}

__device__ __forceinline__ uint32_t encode8_rank1(const uint32_t *lds, int kind, const float (&v)[kQElts],
                                                  const float (&cmx)[kQElts], const ColRcp &cr, float rm)
{
    float xs[kQElts];
    if (kind != kMapGeneric && __all(cr.safe && rc_safe(rm))) {
        const float rr = rcp_exact(rm);
#pragma unroll
        for (int k = 0; k < kQElts; ++k) {
            const bool by_col = cmx[k] < rm;
            xs[k] = div_by_rc(v[k], by_col ? cmx[k] : rm, by_col ? cr.rc[k] : rr);
        }
        // the closed form of the second-moment code needs 0 <= x <= 1; values below 0 are legal here
        return kind == kMapStdM ? encode8_std_m(lds, xs) : encode8_plain(lds, kLdsQ0, kind, xs);
    }
#pragma unroll
    for (int k = 0; k < kQElts; ++k)
        xs[k] = v[k] / ((cmx[k] < rm) ? cmx[k] : rm);
    return encode8_plain(lds, kLdsQ0, kind, xs);
}

// The same when C is a multiple of 8: a lane's 8 values lie in one row, the grid is
// (column chunks, rows) and no index division is needed.  Workgroup (0,0) also writes the
// pad codes past the tensor.
constexpr int kR1Cols = kQThreads * kQElts;  // columns per workgroup

#ifndef LPMM_R1_ROWS_PER_WG
#define LPMM_R1_ROWS_PER_WG 4
#endif
constexpr int kR1RowsPerWg = LPMM_R1_ROWS_PER_WG;  // rows of one column chunk per workgroup: the column maxima are loaded once

__global__ __launch_bounds__(kQThreads) void quant_rank1_rows_kernel(const float *__restrict__ x, int64_t R,
                                                                     int64_t C, const float *__restrict__ rowmax,
                                                                     const float *__restrict__ colmax,
                                                                     const float *__restrict__ qmap,
                                                                     uint8_t *__restrict__ codes, int64_t n_padded)
{
    constexpr int T = kR1RowsPerWg;
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    const int64_t n = R * C;
    const int64_t r0 = (int64_t)blockIdx.y * T;
    const int64_t c = (int64_t)blockIdx.x * kR1Cols + (int64_t)threadIdx.x * kQElts;
    const bool live = c < C;
    // the lane's loads first, the LDS tables afterwards
    float4 a[T], b[T], ca, cb;
    float rm[T];
    if (live) {
        ca = *reinterpret_cast<const float4 *>(colmax + c);
        cb = *reinterpret_cast<const float4 *>(colmax + c + 4);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            if (r0 + t < R) {
                const float *p = x + (r0 + t) * C + c;
                a[t] = load4(p);
                b[t] = load4(p + 4);
                rm[t] = rowmax[r0 + t];
            }
        }
    }
    lds_fill(lds, qmap, nullptr);
    const int kind = classify_map(qmap);
    lds_barrier();
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        const float z[kQElts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t wz = encode8_plain(lds, kLdsQ0, kind, z);
        for (int64_t i = n + (int64_t)threadIdx.x * kQElts; i < n_padded; i += kR1Cols)
            *reinterpret_cast<uint32_t *>(codes + (i >> 1)) = wz;
        if (threadIdx.x == 0)
            codes[n_padded / 2] = 0;
    }
    if (!live)
        return;
    const float cmx[kQElts] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
    const ColRcp cr = col_rcp(cmx);
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (r0 + t >= R)
            break;
        const float v[kQElts] = {a[t].x, a[t].y, a[t].z, a[t].w, b[t].x, b[t].y, b[t].z, b[t].w};
        store_u32(reinterpret_cast<uint32_t *>(codes + (((r0 + t) * C + c) >> 1)),
                  encode8_rank1(lds, kind, v, cmx, cr, rm[t]));
    }
}

// The same in the row layout of the fused step for column counts that are a multiple of 128:
// 16 lanes own 128 consecutive columns of one row, lane l the columns [4l, 4l+4) and
// [64+4l, 64+4l+4), so that every 16-byte load covers whole cache lines.
__global__ __launch_bounds__(kQThreads) void quant_rank1_rows128_kernel(const float *__restrict__ x, int64_t R,
                                                                        int64_t C, const float *__restrict__ rowmax,
                                                                        const float *__restrict__ colmax,
                                                                        const float *__restrict__ qmap,
                                                                        uint8_t *__restrict__ codes, int64_t n_padded)
{
    constexpr int T = kR1RowsPerWg;
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    const int64_t n = R * C;
    const int lane16 = threadIdx.x & 15;
    const int64_t r0 = (int64_t)blockIdx.y * T;
    const int64_t c0 = (int64_t)blockIdx.x * kR1Cols + (int64_t)(threadIdx.x >> 4) * kGroup;
    const bool live = c0 < C;  // uniform over the 16 lanes of a group
    // the small loads that feed LDS first (they return first), then the rows' loads
    const LdsFill fill = lds_fill_load(qmap, qmap);
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
    lds_fill_store(lds, fill);
    const int kind = classify_map(qmap);
    lds_barrier();
    if (blockIdx.x == 0 && blockIdx.y == 0) {
        const float z[kQElts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t wz = encode8_plain(lds, kLdsQ0, kind, z);
        for (int64_t i = n + (int64_t)threadIdx.x * kQElts; i < n_padded; i += kR1Cols)
            *reinterpret_cast<uint32_t *>(codes + (i >> 1)) = wz;
        if (threadIdx.x == 0)
            codes[n_padded / 2] = 0;
    }
    if (!live)
        return;
    const float cmx[kQElts] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
    const ColRcp cr = col_rcp(cmx);
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (r0 + t >= R)
            break;
        const float v[kQElts] = {a[t].x, a[t].y, a[t].z, a[t].w, b[t].x, b[t].y, b[t].z, b[t].w};
        const uint32_t w = encode8_rank1(lds, kind, v, cmx, cr, rm[t]);
        uint16_t *cp = reinterpret_cast<uint16_t *>(codes + (((r0 + t) * C + c0) >> 1)) + lane16;
        store_u16(cp, w & 0xFFFFu);
        store_u16(cp + 16, w >> 16);
    }
}

__global__ __launch_bounds__(kQThreads) void dequant_rank1_kernel(const uint8_t *__restrict__ codes,
                                                                  const float *__restrict__ rowmax,
                                                                  const float *__restrict__ colmax,
                                                                  const float *__restrict__ qmap, int64_t n,
                                                                  int64_t C, float *__restrict__ out, bool vec)
{
    __shared__ __align__(16) uint32_t lds[32];
    if (threadIdx.x < 16)
        lds[threadIdx.x] = __float_as_uint(qmap[threadIdx.x]);
    __syncthreads();
    const int64_t base = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) * kQElts;
    if (base >= n)
        return;
    const Nibbles nb = split_nibbles(load_codes8(codes, base, n, vec));
    int64_t r = base / C;
    int64_t c = base - r * C;
    float rm = rowmax[r];
    float v[kQElts];
#pragma unroll
    for (int k = 0; k < kQElts; ++k) {
        v[k] = 0.0f;
        if (base + k < n) {
            const float cmx = colmax[c];
            const float st = (cmx < rm) ? cmx : rm;
            v[k] = decode_nibble(lds, kLdsQ0, nb, k) * st;
            if (++c == C) {
                c = 0;
                ++r;
                rm = (base + k + 1 < n) ? rowmax[r] : 0.0f;
            }
        }
    }
    store8(out, base, n, vec, v);
}

__global__ __launch_bounds__(kQThreads) void dequant_rank1_rows_kernel(const uint8_t *__restrict__ codes,
                                                                       const float *__restrict__ rowmax,
                                                                       const float *__restrict__ colmax,
                                                                       const float *__restrict__ qmap, int64_t R,
                                                                       int64_t C, float *__restrict__ out)
{
    constexpr int T = kR1RowsPerWg;
    __shared__ __align__(16) uint32_t lds[32];
    const int64_t r0 = (int64_t)blockIdx.y * T;
    const int64_t c = (int64_t)blockIdx.x * kR1Cols + (int64_t)threadIdx.x * kQElts;
    const bool live = c < C;
    uint32_t w[T];
    float rm[T];
    float4 ca, cb;
    if (live) {
        ca = *reinterpret_cast<const float4 *>(colmax + c);
        cb = *reinterpret_cast<const float4 *>(colmax + c + 4);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            if (r0 + t < R) {
                w[t] = load_u32(reinterpret_cast<const uint32_t *>(codes + (((r0 + t) * C + c) >> 1)));
                rm[t] = rowmax[r0 + t];
            }
        }
    }
    if (threadIdx.x < 16)
        lds[threadIdx.x] = __float_as_uint(qmap[threadIdx.x]);
    lds_barrier();
    if (!live)
        return;
    const float cmx[kQElts] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (r0 + t >= R)
            break;
        const Nibbles nb = split_nibbles(w[t]);
        float v[kQElts];
#pragma unroll
        for (int k = 0; k < kQElts; ++k)
            v[k] = decode_nibble(lds, kLdsQ0, nb, k) * ((cmx[k] < rm[t]) ? cmx[k] : rm[t]);
        float *o = out + (r0 + t) * C + c;
        store4(o, make_float4(v[0], v[1], v[2], v[3]));
        store4(o + 4, make_float4(v[4], v[5], v[6], v[7]));
    }
}

// Row layout variant for column counts that are a multiple of 128: 16 lanes own 128
// consecutive columns of one row, lane l the columns [4l, 4l+4) and [64+4l, 64+4l+4), so that
// every 16-byte store covers whole cache lines.
__global__ __launch_bounds__(kQThreads) void dequant_rank1_rows128_kernel(const uint8_t *__restrict__ codes,
                                                                          const float *__restrict__ rowmax,
                                                                          const float *__restrict__ colmax,
                                                                          const float *__restrict__ qmap, int64_t R,
                                                                          int64_t C, float *__restrict__ out)
{
    constexpr int T = kR1RowsPerWg;
    __shared__ __align__(16) uint32_t lds[kDequantLdsWords];
    const int lane16 = threadIdx.x & 15;
    const int64_t r0 = (int64_t)blockIdx.y * T;
    const int64_t c0 = (int64_t)blockIdx.x * kR1Cols + (int64_t)(threadIdx.x >> 4) * kGroup;
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
                const uint16_t *cp = reinterpret_cast<const uint16_t *>(codes + (((r0 + t) * C + c0) >> 1)) + lane16;
                w0[t] = load_u16(cp);
                w1[t] = load_u16(cp + 16);
                rm[t] = rowmax[r0 + t];
            }
        }
    }
    if (threadIdx.x < 16)
        lds[threadIdx.x] = __float_as_uint(qmap[threadIdx.x]);
    lds_barrier();
    if (!live)
        return;
    const float cmx[kQElts] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (r0 + t >= R)
            break;
        const Nibbles nb = split_nibbles(w0[t] | (w1[t] << 16));
        float v[kQElts];
#pragma unroll
        for (int k = 0; k < kQElts; ++k)
            v[k] = decode_nibble(lds, kLdsQ0, nb, k) * ((cmx[k] < rm[t]) ? cmx[k] : rm[t]);
        float *o = out + (r0 + t) * C + c0 + lane16 * 4;
        store4(o, make_float4(v[0], v[1], v[2], v[3]));
        store4(o + 64, make_float4(v[4], v[5], v[6], v[7]));
    }
}

inline bool tiles_ok(int64_t n, int64_t tile, uint32_t *tiles)
{
    const int64_t t = (n + tile - 1) / tile;
    if (t > 0x7fffffffLL)
        return false;
    *tiles = (uint32_t)t;
    return true;
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_pack_nonlinear_4bit(const float *x, const float *qmap, int64_t n_padded,
                                        uint8_t *out, void *stream)
{
    if (n_padded < 0 || (n_padded % 8) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    if (n_padded > 0) {
        LPMM_REQUIRE_PTR(x);
        LPMM_REQUIRE_ALIGN(x, 4);
    }
    uint32_t tiles;
    if (!tiles_ok(n_padded > 0 ? n_padded : 1, kQTile, &tiles))
        return LPMM_ERR_SIZE;
    const bool vec = aligned_to(x, 16) && aligned_to(out, 4);
    hipLaunchKernelGGL(pack4_kernel, dim3(tiles), dim3(kQThreads), 0, (hipStream_t)stream, x, qmap,
                       n_padded, out, vec);
    return launch_status();
}

extern "C" int lpmm_unpack_nonlinear_4bit(const uint8_t *codes, const float *qmap, int64_t n,
                                          float *out, void *stream)
{
    if (n < 0)
        return LPMM_ERR_SIZE;
    if (n == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 4);
    uint32_t tiles;
    if (!tiles_ok(n, kQTile, &tiles))
        return LPMM_ERR_SIZE;
    const bool vec = aligned_to(out, 16) && aligned_to(codes, 4);
    hipLaunchKernelGGL(unpack4_kernel, dim3(tiles), dim3(kQThreads), 0, (hipStream_t)stream, codes, qmap,
                       n, out, vec);
    return launch_status();
}

extern "C" int lpmm_quant_group(const float *x, int64_t n, int64_t gp_sz, const float *qmap,
                                uint8_t *codes, float *max1, void *stream)
{
    if (n <= 0)
        return LPMM_ERR_SIZE;
    if (gp_sz < kGroup || gp_sz > 2 * kQTile || (gp_sz & (gp_sz - 1)) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(max1);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(max1, 4);
    LPMM_REQUIRE_ALIGN(codes, 4);
    const int64_t n_groups = (n + gp_sz - 1) / gp_sz;
    uint32_t tiles;
    if (!tiles_ok(n_groups * gp_sz, kQTile, &tiles))
        return LPMM_ERR_SIZE;
    const int64_t n_padded = (int64_t)tiles * kQTile;
#ifndef LPMM_QG_T
#define LPMM_QG_T 2
#endif
    constexpr int kT = LPMM_QG_T;  // tiles per workgroup
    if (gp_sz > kQTile)
        hipLaunchKernelGGL((quant_group_kernel<2 * kQThreads, 1>), dim3((tiles + 1) / 2), dim3(2 * kQThreads), 0,
                           (hipStream_t)stream, x, n, (int)(gp_sz / kGroup), qmap, codes, max1, n_groups, n_padded,
                           aligned_to(x, 16));
    else
        hipLaunchKernelGGL((quant_group_kernel<kQThreads, kT>), dim3((tiles + kT - 1) / kT), dim3(kQThreads), 0,
                           (hipStream_t)stream, x, n, (int)(gp_sz / kGroup), qmap, codes, max1, n_groups, n_padded,
                           aligned_to(x, 16));
    return launch_status();
}

extern "C" int lpmm_dequant_group(const uint8_t *codes, const float *max1, const float *qmap, int64_t n,
                                  int64_t gp_sz, float *out, void *stream)
{
    if (n <= 0 || gp_sz < kGroup || (gp_sz % kGroup) != 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(max1);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(max1, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 4);
    uint32_t tiles;
    if (!tiles_ok(n, kQTile, &tiles))
        return LPMM_ERR_SIZE;
    const bool vec = aligned_to(out, 16) && aligned_to(codes, 4);
    const int64_t full_groups = n / kGroup;
    if (vec && full_groups > 0 && full_groups <= 0x7fffffffLL * 16) {
        // whole 128-value rows in the row layout, the ragged tail (< 128 values) element-wise
#ifndef LPMM_DQ_T
#define LPMM_DQ_T 2
#endif
        constexpr int kT = LPMM_DQ_T;  // passes of 16 rows per workgroup
        hipLaunchKernelGGL(dequant_group_rows_kernel<kT>, dim3((uint32_t)((full_groups + 16 * kT - 1) / (16 * kT))),
                           dim3(kQThreads), 0, (hipStream_t)stream, codes, max1, qmap, full_groups,
                           (int)(gp_sz / kGroup), out);
        const int64_t done = full_groups * kGroup;
        if (done < n)
            hipLaunchKernelGGL(dequant_group_kernel, dim3(1), dim3(kQThreads), 0, (hipStream_t)stream,
                               codes + done / 2, max1 + done / gp_sz, qmap, n - done, gp_sz, out + done, false);
        return launch_status();
    }
    hipLaunchKernelGGL(dequant_group_kernel, dim3(tiles), dim3(kQThreads), 0, (hipStream_t)stream, codes,
                       max1, qmap, n, gp_sz, out, vec);
    return launch_status();
}

extern "C" int lpmm_rank1_stats(const float *x, int64_t rows, int64_t cols, float *rowmax, float *colmax,
                                void *stream)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(rowmax);
    LPMM_REQUIRE_PTR(colmax);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(rowmax, 4);
    LPMM_REQUIRE_ALIGN(colmax, 4);
    const int64_t gx = (cols + kStatCols - 1) / kStatCols, gy = (rows + kStatRows - 1) / kStatRows;
    if (gx > 0x7fffffffLL || gy > 65535)
        return LPMM_ERR_SIZE;
    const int64_t mx = rows > cols ? rows : cols;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((uint32_t)((mx + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, rowmax, rows, colmax, cols);
    const bool vec = aligned_to(x, 16) && (cols % 4) == 0;
    const int64_t tx = (cols + kStat2Cols - 1) / kStat2Cols, ty = (rows + kStat2Rows - 1) / kStat2Rows;
    if (vec && tx * ty <= 0x7fffffffLL)
        hipLaunchKernelGGL(rank1_stats_tile_kernel, dim3((uint32_t)(tx * ty)), dim3(kQThreads), 0, (hipStream_t)stream,
                           x, rows, cols, (uint32_t)tx, rowmax, colmax);
    else
        hipLaunchKernelGGL(rank1_stats_kernel, dim3((uint32_t)gx, (uint32_t)gy), dim3(kQThreads), 0,
                           (hipStream_t)stream, x, rows, cols, rowmax, colmax, vec);
    return launch_status();
}

// row-wise kernels: columns a multiple of 8, 16-byte aligned operands, rows fit grid.y
static bool rank1_rows_ok(const void *x, const void *colmax, const void *codes, int64_t rows, int64_t cols)
{
    return (cols % 8) == 0 && rows <= 65535LL * kR1RowsPerWg && aligned_to(x, 16) && aligned_to(colmax, 16) && aligned_to(codes, 4);
}

extern "C" int lpmm_quant_rank1(const float *x, int64_t rows, int64_t cols, const float *rowmax,
                                const float *colmax, const float *qmap, uint8_t *codes, void *stream)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(x);
    LPMM_REQUIRE_PTR(rowmax);
    LPMM_REQUIRE_PTR(colmax);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_ALIGN(x, 4);
    LPMM_REQUIRE_ALIGN(rowmax, 4);
    LPMM_REQUIRE_ALIGN(colmax, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(codes, 4);
    const int64_t n = rows * cols;
    uint32_t tiles;
    if (!tiles_ok(n, kQTile, &tiles))
        return LPMM_ERR_SIZE;
    const int64_t n_padded = (int64_t)tiles * kQTile;
    if (rank1_rows_ok(x, colmax, codes, rows, cols)) {
        const uint32_t gx = (uint32_t)((cols + kR1Cols - 1) / kR1Cols);
        const uint32_t gy = (uint32_t)((rows + kR1RowsPerWg - 1) / kR1RowsPerWg);
        if ((cols % kGroup) == 0)
            hipLaunchKernelGGL(quant_rank1_rows128_kernel, dim3(gx, gy), dim3(kQThreads), 0,
                               (hipStream_t)stream, x, rows, cols, rowmax, colmax, qmap, codes, n_padded);
        else
            hipLaunchKernelGGL(quant_rank1_rows_kernel, dim3(gx, gy), dim3(kQThreads), 0,
                               (hipStream_t)stream, x, rows, cols, rowmax, colmax, qmap, codes, n_padded);
    } else {
        hipLaunchKernelGGL(quant_rank1_kernel, dim3(tiles), dim3(kQThreads), 0, (hipStream_t)stream, x, n, cols,
                           rowmax, colmax, qmap, codes, n_padded, aligned_to(x, 16));
    }
    return launch_status();
}

extern "C" int lpmm_dequant_rank1(const uint8_t *codes, const float *rowmax, const float *colmax,
                                  const float *qmap, int64_t rows, int64_t cols, float *out, void *stream)
{
    if (rows <= 0 || cols <= 0)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(codes);
    LPMM_REQUIRE_PTR(rowmax);
    LPMM_REQUIRE_PTR(colmax);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_PTR(out);
    LPMM_REQUIRE_ALIGN(rowmax, 4);
    LPMM_REQUIRE_ALIGN(colmax, 4);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    LPMM_REQUIRE_ALIGN(out, 4);
    const int64_t n = rows * cols;
    uint32_t tiles;
    if (!tiles_ok(n, kQTile, &tiles))
        return LPMM_ERR_SIZE;
    if (rank1_rows_ok(out, colmax, codes, rows, cols) && (cols % kGroup) == 0) {
        const uint32_t gx = (uint32_t)((cols + kR1Cols - 1) / kR1Cols);
        const uint32_t gy = (uint32_t)((rows + kR1RowsPerWg - 1) / kR1RowsPerWg);
        hipLaunchKernelGGL(dequant_rank1_rows128_kernel, dim3(gx, gy), dim3(kQThreads), 0,
                           (hipStream_t)stream, codes, rowmax, colmax, qmap, rows, cols, out);
    } else if (rank1_rows_ok(out, colmax, codes, rows, cols)) {
        const uint32_t gx = (uint32_t)((cols + kR1Cols - 1) / kR1Cols);
        const uint32_t gy = (uint32_t)((rows + kR1RowsPerWg - 1) / kR1RowsPerWg);
        hipLaunchKernelGGL(dequant_rank1_rows_kernel, dim3(gx, gy), dim3(kQThreads), 0,
                           (hipStream_t)stream, codes, rowmax, colmax, qmap, rows, cols, out);
    } else {
        const bool vec = aligned_to(out, 16) && aligned_to(codes, 4);
        hipLaunchKernelGGL(dequant_rank1_kernel, dim3(tiles), dim3(kQThreads), 0, (hipStream_t)stream, codes,
                           rowmax, colmax, qmap, n, cols, out, vec);
    }
    return launch_status();
}
