// The non-fused AdamW step on 4-bit states with the reference's default scalings -- first
// moment block-wise over 128 values, second moment rank-1 (scale[r, c] = min(rowmax[r],
// colmax[c])) -- in two passes over HBM instead of the seven of the staged path
// (lpmm/optim/adamw.py:394-436: two dequantisations, the update, the statistics of the new
// second moment, two quantisations).
//
// The second moment cannot be re-quantised where it is computed, because its scales are
// maxima over whole rows and columns of the new values.  So:
//
//   pass 1 (update):   reads p, g, both code arrays and the current statistics; updates p,
//                      re-quantises m, and merges the row/column maxima of the new v into the
//                      next statistics (atomic max on the bit patterns: exact, order-free);
//   pass 2 (requant):  reads g, the old v codes and both sets of statistics, recomputes the
//                      new v with the same operations (bit-identical), normalises by the next
//                      statistics and overwrites the v codes in place.
//
// 18.5 bytes per parameter cross HBM instead of 50.  The column count must be a multiple of
// 128, so that the 128-value groups of m never straddle rows: 16 lanes (one DPP row) own 128
// consecutive columns of one tensor row.  A 256-thread workgroup covers tile_rows rows by
// 128 << lg_wide columns, per pass (16 >> lg_wide) rows of (1 << lg_wide) adjacent groups, so
// that its accesses to a row are contiguous runs of 512 << lg_wide bytes.
//
// Both kernels run at the rate the memory system gives to their access structure, not at that
// of their arithmetic (with the arithmetic taken out they take the same time).  Measured on the
// LLaMA-7B shapes: a workgroup that walks through many passes is slower than the same accesses
// made by short-lived workgroups in dispatch order (tiles of 1 or 2 passes run at the rate of
// the one-shot fused step, 8 passes over 16 rows by 1024 columns 13 % below it), but short
// tiles mean more column atomics and more tile set-up.  Tiles of 64 rows by 256 columns
// (8 passes of 8 rows) are the best compromise for both kernels.  The row blocks that are
// resident together interleave their passes (block k of a group of `comb` blocks takes the rows
// of pass i at (i * comb + k) * pass_rows), so that at any time a group works on one contiguous
// band of the tensor instead of on `comb` bands a tile apart.  Together 2130 -> 1990 us (first
// pass) and 770 -> 705 us (second pass) per launch of 8.4e8 elements.
#include "lpmm_search.hpp"
#include "lpmm_update.hpp"

namespace lpmm {

constexpr int kThreads = 256;
constexpr int kEltsPerLane = 8;
constexpr int kDppRows = kThreads / 16;  // 128-column groups a workgroup handles per pass
constexpr int kR1Max = 32;               // tensors per launch
// Tile policy: widest tile (lg of 128-column groups), tensor rows per workgroup (more where one pass
// of a narrow tile covers more), workgroups taken to be resident together.
#ifndef LPMM_R1_LG
#define LPMM_R1_LG 1
#endif
#ifndef LPMM_R1_ROWS
#define LPMM_R1_ROWS 64
#endif
#ifndef LPMM_R1_RESIDENT
#define LPMM_R1_RESIDENT 256
#endif
constexpr int kPolicyLgWide = LPMM_R1_LG;
constexpr uint32_t kPolicyRows = LPMM_R1_ROWS, kPolicyResident = LPMM_R1_RESIDENT;
static_assert(LPMM_R1_LG >= 1 && LPMM_R1_LG <= 3, "a tile is 256 to 1024 columns wide at most");
constexpr int kMaxLgWide = kPolicyLgWide;   // the LDS column arrays hold 128 << kMaxLgWide columns
constexpr int kMaxWide = 1 << kMaxLgWide;
// Per-column data of a tile lives in LDS, not in registers (occupancy): the current column
// statistics in the unused bytes between the maps and the encode table, further arrays after
// the table.
constexpr uint32_t kColBytes = kMaxWide * kGroup * 4;
constexpr uint32_t kColOld = kLdsQ1 + 64;
static_assert(kColOld + kColBytes <= kEncLdsBegin, "column statistics overlap the encode table");
constexpr uint32_t kColExtra = (kLdsBytes + 15) / 16 * 16;  // first byte after the table
// Column maxima of the tile, one slot of 8 x 16 words (+16 words of skew, so that the DPP rows
// of a wave hit different banks) per column group: word k * 16 + lane16 of a slot is element k
// of lane lane16.
constexpr uint32_t kRedSlotWords = kGroup + 16;

// A workgroup covers tile_rows rows x (128 << lg_wide) columns: per pass, (16 >> lg_wide) rows of
// (1 << lg_wide) adjacent groups each.
struct TileShape {
    uint32_t lg_wide : 8;
    uint32_t tile_rows : 24;  // max(the policy's rows, rows of one pass)
    uint32_t comb;            // row blocks whose passes interleave
};

struct TensorR1 {
    float *p;
    const float *g;
    uint8_t *mc;  // fp32 first moment: the moment itself (float[rows * cols]), ms unused
    float *ms;
    float *ms_new;  // first-moment groups wider than 128 values: the scales of the new first moment
    uint8_t *vc;
    const float *row_old;
    const float *col_old;
    float *row_new;
    float *col_new;
    int64_t rows;
    uint32_t col_blocks;  // columns / 128
    float neg_step_size, bc2_sqrt, rbc2_sqrt;
    uint32_t m_lg;  // the first moment's group holds 128 << m_lg values
    uint32_t col_tail;  // columns in the last 128-column block (128 unless the column count is ragged)
    TileShape tile;
};

// How the first moment is kept: 4-bit codes in groups of 128 values (re-quantised where it is
// updated), fp32 (read and written as floats), or 4-bit codes in wider groups (256 .. 4096
// values of the flattened tensor: a group spans several DPP rows, tiles and, where the column
// count is not a multiple of the group size, tensor rows.  The update pass only merges the
// groups' maxima into the next scales, the second pass recomputes the moment from g and the old
// codes, bit-identically, and writes its codes -- what both passes do for the second moment).
enum MomentMode { kMCodes128 = 0, kMFloat = 1, kMCodesWide = 2 };

struct MultiR1 {
    TensorR1 t[kR1Max];
    uint32_t tile_start[kR1Max + 1];  // prefix sum of tiles per tensor; unused slots hold the total
    int count;
    float decay, w1, b2, w2, eps;
};

static_assert(sizeof(MultiR1) + 2 * sizeof(void *) <= 4096, "kernel arguments exceed 4 KB");
static_assert(kR1Max <= kWave, "one tile_start entry per lane");

// tensor of this workgroup (uniform): the number of later tensors whose first tile is not
// after this one
__device__ __forceinline__ int find_tensor(const MultiR1 &args)
{
    const int lane = threadIdx.x & (kWave - 1);
    const bool started = lane + 1 < kR1Max && args.tile_start[lane + 1] <= blockIdx.x;
    return __popcll(__ballot(started));
}

__device__ __forceinline__ void unpack8(const float4 &a, const float4 &b, float (&o)[kEltsPerLane])
{
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}

// Where a DPP row of this workgroup works: column group `cg` (fixed), rows row0, row0 + step, ...
struct Geometry {
    int64_t row0;
    uint32_t cg, col_tile;
    int step, passes, wide;
};

__device__ __forceinline__ Geometry geometry(const TensorR1 &t, uint32_t tile, int drow)
{
    Geometry q;
    const TileShape &ts = t.tile;
    q.wide = 1 << ts.lg_wide;
    const uint32_t col_tiles = (t.col_blocks + q.wide - 1) >> ts.lg_wide;
    const uint32_t rb = tile / col_tiles;
    q.col_tile = tile - rb * col_tiles;
    q.cg = q.col_tile * q.wide + (drow & (q.wide - 1));
    const int pass_rows = kDppRows >> ts.lg_wide;
    q.passes = (int)ts.tile_rows / pass_rows;
    // block k of group grp: pass i covers the rows from (grp * passes * comb + i * comb + k) * pass_rows on
    const uint32_t grp = rb / ts.comb, k = rb - grp * ts.comb;
    q.row0 = (int64_t)grp * ts.tile_rows * ts.comb + (int64_t)k * pass_rows + (drow >> ts.lg_wide);
    q.step = pass_rows * (int)ts.comb;
    return q;
}

// Codes of a plain 0.0 into the padding [n, n_padded) of a packed array and 0 into the extra
// last byte; one workgroup.  n and n_padded are multiples of 8, the array is 4-byte aligned.
__device__ __forceinline__ void write_padding(uint8_t *codes, int64_t n, int64_t n_padded, uint32_t zero_word)
{
    for (int64_t i = n + (int64_t)threadIdx.x * kEltsPerLane; i < n_padded; i += kThreads * kEltsPerLane)
        *reinterpret_cast<uint32_t *>(codes + (i >> 1)) = zero_word;
    if (threadIdx.x == 0)
        codes[n_padded / 2] = 0;
}

__global__ __launch_bounds__(kThreads) void rank1_clear_kernel(const MultiR1 args)
{
    const TensorR1 &t = args.t[blockIdx.y];
    const int64_t cols = (int64_t)(t.col_blocks - 1) * kGroup + t.col_tail;
    // first-moment groups that are wider than 128 values or straddle rows: their next scales are
    // merged with atomic maxima as well
    const int64_t group = (int64_t)kGroup << t.m_lg;
    const int64_t m_groups = t.ms_new != nullptr ? (t.rows * cols + group - 1) / group : 0;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < t.rows + cols + m_groups;
         i += (int64_t)gridDim.x * kThreads) {
        if (i < t.rows)
            t.row_new[i] = 0.0f;
        else if (i < t.rows + cols)
            t.col_new[i - t.rows] = 0.0f;
        else
            t.ms_new[i - t.rows - cols] = 0.0f;
    }
}

// operands of one pass of a DPP row, as loaded
struct PassRegs {
    float4 a0, a1, b0, b1;
    float4 c0, c1;  // fp32 first moment only
    uint32_t m0, m1, v0, v1;
    float sm, ro;
};

template <int MODE>
__device__ __forceinline__ void pass_fetch(const TensorR1 &t, uint32_t cg, int lane16, int64_t r, PassRegs &x)
{
    const int64_t grp = r * t.col_blocks + cg;
    const int64_t gbase = grp * kGroup;
    const float *pp = t.p + gbase + lane16 * 4;
    const float *gp = t.g + gbase + lane16 * 4;
    x.a0 = load4(pp);
    x.a1 = load4(pp + 64);
    x.b0 = load4(gp);
    x.b1 = load4(gp + 64);
    const uint16_t *vcp = reinterpret_cast<const uint16_t *>(t.vc + (gbase >> 1)) + lane16;
    if (MODE == kMFloat) {
        const float *mp = reinterpret_cast<const float *>(t.mc) + gbase + lane16 * 4;
        x.c0 = load4(mp);
        x.c1 = load4(mp + 64);
    } else {
        const uint16_t *mcp = reinterpret_cast<const uint16_t *>(t.mc + (gbase >> 1)) + lane16;
        x.m0 = load_u16(mcp);
        x.m1 = load_u16(mcp + 16);
        x.sm = t.ms[MODE == kMCodesWide ? grp >> t.m_lg : grp];
    }
    x.v0 = load_u16(vcp);
    x.v1 = load_u16(vcp + 16);
    x.ro = t.row_old[r];
}

#ifndef LPMM_R1_WAVES
#define LPMM_R1_WAVES 4
#endif
// 4 waves per SIMD, up to 128 registers: the first pass's operands stay live across the prologue and
// the lane's column statistics across the passes (with 5 or 6 the compiler spills or re-reads)
template <int MODE>
__global__ __launch_bounds__(kThreads, LPMM_R1_WAVES) void rank1_update_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[(kColExtra + kMaxWide * kRedSlotWords * 4) / 4];
    uint32_t *colred = lds + kColExtra / 4;
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;

    // Order of the prologue: the small loads that feed LDS (maps, encode table, the tile's current
    // column statistics), then the streaming loads of the first pass, then the LDS writes (the
    // small loads were issued first and return first) and a barrier that orders LDS only -- the
    // first pass's operands are on their way while the tables are set up.
    const LdsFill fill = lds_fill_load(qmap_m, qmap_v);
    constexpr int kColPerThread = kMaxWide * kGroup / kThreads;
    uint32_t co_in[kColPerThread];
#pragma unroll
    for (int i = 0; i < kColPerThread; ++i) {
        const int j = threadIdx.x + i * kThreads;
        co_in[i] = (j < q.wide * kGroup && tile_c0 + j < cols) ? __float_as_uint(t.col_old[tile_c0 + j]) : 0u;
    }
    const bool row_live = q.cg < t.col_blocks;  // the whole DPP row
    PassRegs x;
    if (row_live && q.row0 < t.rows)
        pass_fetch<MODE>(t, q.cg, lane16, q.row0, x);
    lds_fill_store(lds, fill);
    for (int j = threadIdx.x; j < kMaxWide * (int)kRedSlotWords; j += kThreads)
        colred[j] = 0u;
#pragma unroll
    for (int i = 0; i < kColPerThread; ++i)
        lds[kColOld / 4 + threadIdx.x + i * kThreads] = co_in[i];
    const int kind_m = classify_map(qmap_m);
    NfHyper h;
    h.decay = args.decay;
    h.w1 = args.w1;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.eps = args.eps;
    h.neg_step_size = t.neg_step_size;
    h.bc2_sqrt = t.bc2_sqrt;
    h.rbc2_sqrt = t.rbc2_sqrt;
    lds_barrier();

    if (MODE == kMCodes128 && tl == 0) {
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t n = t.rows * cols;
        write_padding(t.mc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                      encode8_plain(lds, kLdsQ0, kind_m, z));
    }

    const int slot = drow & (q.wide - 1);
    if (row_live) {
        const uint32_t co_off = kColOld + (slot * kGroup + lane16 * 4) * 4;
        uint32_t *red = colred + slot * kRedSlotWords + lane16;
        // a lane keeps its eight columns through all passes: their statistics come out of LDS once
        float co[kEltsPerLane];
        unpack8(lds_read<float4>(lds, co_off), lds_read<float4>(lds, co_off + 256), co);
#pragma unroll 1
        for (int it = 0; it < q.passes; ++it) {
            const int64_t r = q.row0 + it * q.step;
            if (r >= t.rows)
                break;
            if (it > 0)
                pass_fetch<MODE>(t, q.cg, lane16, r, x);
            const int64_t grp = r * t.col_blocks + q.cg;
            const int64_t gbase = grp * kGroup;
            float *pp = t.p + gbase + lane16 * 4;
            const uint32_t wv = x.v0 | (x.v1 << 16);
            const float ro = x.ro;
            float pv[kEltsPerLane], gv[kEltsPerLane], m[kEltsPerLane], v[kEltsPerLane];
            unpack8(x.a0, x.a1, pv);
            unpack8(x.b0, x.b1, gv);
            constexpr bool M32 = MODE == kMFloat;
            const Nibbles nm = split_nibbles(M32 ? 0u : (x.m0 | (x.m1 << 16)));
            const float sm = M32 ? 0.0f : x.sm;
            if (M32)
                unpack8(x.c0, x.c1, m);

            const Nibbles nv = split_nibbles(wv);
            float amax_m = 0.0f, vmax = 0.0f;
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                if (!M32)
                    m[k] = decode_nibble(lds, kLdsQ0, nm, k) * sm;
                v[k] = decode_nibble(lds, kLdsQ1, nv, k) * ((co[k] < ro) ? co[k] : ro);
                nonfused_elt(pv[k], gv[k], m[k], v[k], h);
                amax_m = fmaxf(amax_m, fabsf(m[k]));
                vmax = fmaxf(vmax, v[k]);
                atomicMax(red + k * 16, __float_as_uint(v[k]));
            }
            uint32_t cm = 0;
            if (M32) {
                vmax = row16_max(vmax);
            } else {
                row16_max2(amax_m, vmax);
                if (MODE == kMCodes128)
                    cm = encode8_scaled(lds, kLdsQ0, kind_m, m, amax_m);
            }

            store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
            store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
            if (M32) {
                float *mp = reinterpret_cast<float *>(t.mc) + gbase + lane16 * 4;
                store4(mp, make_float4(m[0], m[1], m[2], m[3]));
                store4(mp + 64, make_float4(m[4], m[5], m[6], m[7]));
            } else if (MODE == kMCodes128) {
                uint16_t *mcp = reinterpret_cast<uint16_t *>(t.mc + (gbase >> 1)) + lane16;
                store_u16(mcp, cm & 0xFFFFu);
                store_u16(mcp + 16, cm >> 16);
                if (lane16 == 0)
                    t.ms[grp] = amax_m;
            } else if (lane16 == 0) {
                atomic_max_nonneg(t.ms_new + (grp >> t.m_lg), amax_m);
            }
            if (lane16 == 0)
                atomic_max_nonneg(t.row_new + r, vmax);
        }
    }
    // the column maxima meet in LDS: nothing below depends on the global stores still in flight
    lds_barrier();
    // column j of the tile = element k of lane l of slot s
    for (int j = threadIdx.x; j < q.wide * kGroup; j += kThreads) {
        const int w = j & (kGroup - 1);
        const int k = ((w >> 6) << 2) | (w & 3), l = (w >> 2) & 15;
        if (tile_c0 + j < cols)
            atomic_max_nonneg(t.col_new + tile_c0 + j, __uint_as_float(colred[(j >> 7) * kRedSlotWords + k * 16 + l]));
    }
}

// MWIDE: the first moment's groups are wider than 128 values; its codes are written here too.
template <bool MWIDE>
__global__ __launch_bounds__(kThreads) void rank1_requant_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                 const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[(kColExtra + 2 * kColBytes) / 4];
    constexpr uint32_t kColNew = kColExtra, kColRcp = kColExtra + kColBytes;
    constexpr uint32_t kVMap = MWIDE ? kLdsQ1 : kLdsQ0;  // where the second moment's map sits in LDS
    if (MWIDE)
        lds_fill(lds, qmap_m, qmap_v);
    else
        lds_fill(lds, qmap_v, nullptr);
    const int kind = classify_map(qmap_v);
    const int kind_m = MWIDE ? classify_map(qmap_m) : kMapGeneric;
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    for (int j = threadIdx.x; j < q.wide * kGroup; j += kThreads) {
        const bool in = tile_c0 + j < cols;
        const float cn = in ? t.col_new[tile_c0 + j] : 0.0f;
        lds[kColOld / 4 + j] = in ? __float_as_uint(t.col_old[tile_c0 + j]) : 0u;
        lds[kColNew / 4 + j] = __float_as_uint(cn);
        lds[kColRcp / 4 + j] = __float_as_uint(1.0f / cn);
    }
    NfHyper h;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.w1 = args.w1;
    __syncthreads();

    if (tl == 0) {
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t n = t.rows * cols;
        const int64_t n_pack = (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP;
        write_padding(t.vc, n, n_pack, encode8_plain(lds, kVMap, kind, z));
        if (MWIDE) {
            // The quantiser pads the flattened tensor with zeros to whole groups (functional.py:404-422),
            // the packing pads to whole pack groups of 2048 values.  The zeros that fill up the last
            // group are divided by its scale like its other values (0/0 -> NaN -> code 15 when the
            // group is all zero), those behind it are plain zeros.
            const int64_t group = (int64_t)kGroup << t.m_lg;
            const int64_t n_grp = (n + group - 1) / group * group;
            const int64_t n_all = (n_grp + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP;
            const uint32_t zero_word = encode8_plain(lds, kLdsQ0, kind_m, z);
            uint32_t last_word = zero_word;
            if (n_grp > n) {
                const float last = t.ms_new[(n - 1) >> (7 + t.m_lg)];
                const float zs[kEltsPerLane] = {0.0f / last, 0.0f / last, 0.0f / last, 0.0f / last,
                                                0.0f / last, 0.0f / last, 0.0f / last, 0.0f / last};
                last_word = encode8_plain(lds, kLdsQ0, kind_m, zs);
            }
            for (int64_t i = n + (int64_t)threadIdx.x * kEltsPerLane; i < n_all; i += kThreads * kEltsPerLane)
                *reinterpret_cast<uint32_t *>(t.mc + (i >> 1)) = i < n_grp ? last_word : zero_word;
            if (threadIdx.x == 0)
                t.mc[n_all / 2] = 0;
        }
    }
    if (q.cg >= t.col_blocks)
        return;

    // a lane keeps its eight columns through all passes: their old and new statistics and the
    // reciprocals of the new ones come out of LDS once
    const uint32_t col_off = ((drow & (q.wide - 1)) * kGroup + lane16 * 4) * 4;
    float co[kEltsPerLane], cn[kEltsPerLane], rcn[kEltsPerLane];
    unpack8(lds_read<float4>(lds, kColOld + col_off), lds_read<float4>(lds, kColOld + col_off + 256), co);
    unpack8(lds_read<float4>(lds, kColNew + col_off), lds_read<float4>(lds, kColNew + col_off + 256), cn);
    unpack8(lds_read<float4>(lds, kColRcp + col_off), lds_read<float4>(lds, kColRcp + col_off + 256), rcn);
    bool cols_safe = true;
#pragma unroll
    for (int k = 0; k < kEltsPerLane; ++k)
        cols_safe = cols_safe && rc_safe(cn[k]);
    // the group's 64 code bytes move as one dword per lane (whole lines per access; with the
    // arithmetic taken out this pass is 11 % faster than with two 16-bit accesses per lane)
    const uint32_t code_dword = code_dword_of_lane(lane16), code_sel = code_swap_selector(lane16);
#pragma unroll 1
    for (int it = 0; it < q.passes; ++it) {
        const int64_t r = q.row0 + it * q.step;
        if (r >= t.rows)
            break;
        const int64_t gbase = (r * t.col_blocks + q.cg) * kGroup;
        const float *gp = t.g + gbase + lane16 * 4;
        const float4 b0 = load4(gp), b1 = load4(gp + 64);
        uint32_t *vcp = reinterpret_cast<uint32_t *>(t.vc + (gbase >> 1)) + code_dword;
        const uint32_t wv = swap_code_halves(load_u32(vcp), code_sel);
        uint32_t *mcp = nullptr;
        uint32_t wm = 0;
        float ms_old = 0.0f, ms_new = 0.0f;
        if (MWIDE) {
            mcp = reinterpret_cast<uint32_t *>(t.mc + (gbase >> 1)) + code_dword;
            wm = swap_code_halves(load_u32(mcp), code_sel);
            const int64_t mg = gbase >> (7 + t.m_lg);
            ms_old = t.ms[mg];
            ms_new = t.ms_new[mg];
        }
        const float ro = t.row_old[r], rn = t.row_new[r];
        float gv[kEltsPerLane], v[kEltsPerLane], x[kEltsPerLane];
        unpack8(b0, b1, gv);
        const Nibbles nv = split_nibbles(wv);
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            v[k] = decode_nibble(lds, kVMap, nv, k) * ((co[k] < ro) ? co[k] : ro);
            nonfused_second_moment(v[k], gv[k], h);
        }
        if (MWIDE) {
            // the first moment as the update pass computed it, with the scale of its whole group
            const Nibbles nm = split_nibbles(wm);
            float m[kEltsPerLane];
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                m[k] = lerp_w(decode_nibble(lds, kLdsQ0, nm, k) * ms_old, gv[k], h.w1);
            store_u32(mcp, swap_code_halves(encode8_scaled(lds, kLdsQ0, kind_m, m, ms_new), code_sel));
        }
        uint32_t w;
        // every scale the wave divides by is a column or the row statistic: all in the range in
        // which the reciprocal is exact?
        if (kind == kMapStdV && __all(cols_safe && rc_safe(rn))) {
            // the correctly rounded reciprocal of whichever statistic is the scale, then one
            // multiply and two fmas: the correctly rounded quotient (v <= scale by construction)
            const float rcr = rcp_exact(rn);
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const bool by_col = cn[k] < rn;
                x[k] = div_by_rc(v[k], by_col ? cn[k] : rn, by_col ? rcn[k] : rcr);
            }
            w = encode8_std_v(x);
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                x[k] = v[k] / ((cn[k] < rn) ? cn[k] : rn);
            w = encode8_plain(lds, kVMap, kind, x);
        }
        store_u32(vcp, swap_code_halves(w, code_sel));
    }
}

// ---------------------------------------------------------------------------------------
// The same two passes for code widths of 5 to 8 bits (lpmm/configs/default_{5,6,7,8}b.yml): one
// code per byte (lpmm/cpp_extension/quantization_kernel.cu:516-533, :656-669), maps of 2^bits
// entries in LDS, decoded by indexing and encoded by the reference's search (:397-427) as the
// stand-alone quantisers of these widths do it.  Same tiles and statistics as above; a lane's
// eight codes are two dwords.  21.06 bytes per parameter cross HBM (p 8, g 4 + 4, m codes 2,
// v codes 1 + 2, scales).  LLaMA-7B-shaped set: 25.1 ms per step with 5 bits, 25.3 ms with 8
// (the staged path 67.6 ms); the second moment's evenly spaced map takes the closed form of
// lpmm_search.hpp, so only the first moment is searched.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t byte_of(uint32_t w0, uint32_t w1, int k)
{
    return ((k < 4 ? w0 : w1) >> (8 * (k & 3))) & 0xFFu;
}

__device__ __forceinline__ uint32_t pack4(const uint32_t (&c)[kEltsPerLane], int h)
{
    return c[4 * h] | (c[4 * h + 1] << 8) | (c[4 * h + 2] << 16) | (c[4 * h + 3] << 24);
}

// Code `zero` into the padding [n, n_padded) of an array of one code per byte and 0 into the extra
// last byte; one workgroup.  n and n_padded are multiples of 4, the array is 4-byte aligned.
__device__ __forceinline__ void write_padding_bytes(uint8_t *codes, int64_t n, int64_t n_padded, uint32_t zero)
{
    for (int64_t i = n + (int64_t)threadIdx.x * 4; i < n_padded; i += kThreads * 4)
        *reinterpret_cast<uint32_t *>(codes + i) = zero * 0x01010101u;
    if (threadIdx.x == 0)
        codes[n_padded] = 0;
}

__global__ __launch_bounds__(kThreads) void rank1_update_bits_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                    const float *__restrict__ qmap_v, int bits_m,
                                                                    int bits_v)
{
    __shared__ float map_m[256], map_v[256];
    __shared__ SearchLds search_m;
    __shared__ __align__(16) float col_old[kMaxWide * kGroup];
    __shared__ uint32_t colred[kMaxWide * kRedSlotWords];
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    fill_map(map_m, qmap_m, bits_m);
    fill_map(map_v, qmap_v, bits_v);
    fill_search(search_m, qmap_m, bits_m);
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads)
        col_old[j] = (j < q.wide * kGroup && tile_c0 + j < cols) ? t.col_old[tile_c0 + j] : 0.0f;
    for (int j = threadIdx.x; j < kMaxWide * (int)kRedSlotWords; j += kThreads)
        colred[j] = 0u;
    NfHyper h;
    h.decay = args.decay;
    h.w1 = args.w1;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.eps = args.eps;
    h.neg_step_size = t.neg_step_size;
    h.bc2_sqrt = t.bc2_sqrt;
    h.rbc2_sqrt = t.rbc2_sqrt;
    __syncthreads();
    const bool map_even = map_is_even(search_m);

    if (tl == 0) {
        const int64_t n = t.rows * cols;
        write_padding_bytes(t.mc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                            search_code(search_m, bits_m, 0.0f));
    }
    const uint32_t mask_m = (1u << bits_m) - 1u, mask_v = (1u << bits_v) - 1u;
    const int slot = drow & (q.wide - 1);
    if (q.cg < t.col_blocks) {
        const float *cop = col_old + slot * kGroup + lane16 * 4;
        uint32_t *red = colred + slot * kRedSlotWords + lane16;
        float co[kEltsPerLane];
        unpack8(*reinterpret_cast<const float4 *>(cop), *reinterpret_cast<const float4 *>(cop + 64), co);
#pragma unroll 1
        for (int it = 0; it < q.passes; ++it) {
            const int64_t r = q.row0 + it * q.step;
            if (r >= t.rows)
                break;
            const int64_t grp = r * t.col_blocks + q.cg;
            const int64_t gbase = grp * kGroup;
            float *pp = t.p + gbase + lane16 * 4;
            const float *gp = t.g + gbase + lane16 * 4;
            uint32_t *mcp = reinterpret_cast<uint32_t *>(t.mc + gbase) + lane16;
            const uint32_t *vcp = reinterpret_cast<const uint32_t *>(t.vc + gbase) + lane16;
            const float4 a0 = load4(pp), a1 = load4(pp + 64), b0 = load4(gp), b1 = load4(gp + 64);
            const uint32_t wm0 = load_u32(mcp), wm1 = load_u32(mcp + 16);
            const uint32_t wv0 = load_u32(vcp), wv1 = load_u32(vcp + 16);
            const float sm = t.ms[grp], ro = t.row_old[r];
            float pv[kEltsPerLane], gv[kEltsPerLane], m[kEltsPerLane], v[kEltsPerLane];
            unpack8(a0, a1, pv);
            unpack8(b0, b1, gv);
            float amax_m = 0.0f, vmax = 0.0f;
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                m[k] = map_m[byte_of(wm0, wm1, k) & mask_m] * sm;
                v[k] = map_v[byte_of(wv0, wv1, k) & mask_v] * ((co[k] < ro) ? co[k] : ro);
                nonfused_elt(pv[k], gv[k], m[k], v[k], h);
                amax_m = fmaxf(amax_m, fabsf(m[k]));
                vmax = fmaxf(vmax, v[k]);
                atomicMax(red + k * 16, __float_as_uint(v[k]));
            }
            row16_max2(amax_m, vmax);
            // |m| <= amax: with the correctly rounded reciprocal one multiply and two fmas give the
            // correctly rounded quotient; maxima outside the reciprocal's exact range (0 included:
            // 0/0 must give NaN) take the plain division
            float xs[kEltsPerLane];
            if (__all(rc_safe(amax_m))) {
                const float rc = rcp_exact(amax_m);
#pragma unroll
                for (int k = 0; k < kEltsPerLane; ++k)
                    xs[k] = div_by_rc(m[k], amax_m, rc);
            } else {
#pragma unroll
                for (int k = 0; k < kEltsPerLane; ++k)
                    xs[k] = m[k] / amax_m;
            }
            uint32_t c[kEltsPerLane];
            search_codes8(search_m, bits_m, map_even, xs, c);
            store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
            store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
            store_u32(mcp, pack4(c, 0));
            store_u32(mcp + 16, pack4(c, 1));
            if (lane16 == 0) {
                t.ms[grp] = amax_m;
                atomic_max_nonneg(t.row_new + r, vmax);
            }
        }
    }
    __syncthreads();
    // column j of the tile = element k of lane l of slot s
    for (int j = threadIdx.x; j < q.wide * kGroup; j += kThreads) {
        const int w = j & (kGroup - 1);
        const int k = ((w >> 6) << 2) | (w & 3), l = (w >> 2) & 15;
        if (tile_c0 + j < cols)
            atomic_max_nonneg(t.col_new + tile_c0 + j, __uint_as_float(colred[(j >> 7) * kRedSlotWords + k * 16 + l]));
    }
}

__global__ __launch_bounds__(kThreads) void rank1_requant_bits_kernel(const MultiR1 args, const float *__restrict__ qmap_v,
                                                                     int bits_v)
{
    __shared__ float map_v[256];
    __shared__ SearchLds search_v;
    __shared__ __align__(16) float col_old[kMaxWide * kGroup], col_new[kMaxWide * kGroup];
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    fill_map(map_v, qmap_v, bits_v);
    fill_search(search_v, qmap_v, bits_v);
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads) {
        const bool in = j < q.wide * kGroup && tile_c0 + j < cols;
        col_old[j] = in ? t.col_old[tile_c0 + j] : 0.0f;
        col_new[j] = in ? t.col_new[tile_c0 + j] : 0.0f;
    }
    NfHyper h;
    h.b2 = args.b2;
    h.w2 = args.w2;
    __syncthreads();
    const bool map_even = map_is_even(search_v);

    if (tl == 0) {
        const int64_t n = t.rows * cols;
        write_padding_bytes(t.vc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                            search_code(search_v, bits_v, 0.0f));
    }
    if (q.cg >= t.col_blocks)
        return;
    const uint32_t mask_v = (1u << bits_v) - 1u;
    const int col_off = (drow & (q.wide - 1)) * kGroup + lane16 * 4;
    float co[kEltsPerLane], cn[kEltsPerLane];
    unpack8(*reinterpret_cast<const float4 *>(col_old + col_off), *reinterpret_cast<const float4 *>(col_old + col_off + 64), co);
    unpack8(*reinterpret_cast<const float4 *>(col_new + col_off), *reinterpret_cast<const float4 *>(col_new + col_off + 64), cn);
#pragma unroll 1
    for (int it = 0; it < q.passes; ++it) {
        const int64_t r = q.row0 + it * q.step;
        if (r >= t.rows)
            break;
        const int64_t gbase = (r * t.col_blocks + q.cg) * kGroup;
        const float *gp = t.g + gbase + lane16 * 4;
        const float4 b0 = load4(gp), b1 = load4(gp + 64);
        uint32_t *vcp = reinterpret_cast<uint32_t *>(t.vc + gbase) + lane16;
        const uint32_t wv0 = load_u32(vcp), wv1 = load_u32(vcp + 16);
        const float ro = t.row_old[r], rn = t.row_new[r];
        float gv[kEltsPerLane], x[kEltsPerLane];
        unpack8(b0, b1, gv);
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            float v = map_v[byte_of(wv0, wv1, k) & mask_v] * ((co[k] < ro) ? co[k] : ro);
            nonfused_second_moment(v, gv[k], h);
            x[k] = v / ((cn[k] < rn) ? cn[k] : rn);
        }
        uint32_t c[kEltsPerLane];
        search_codes8(search_v, bits_v, map_even, x, c);
        store_u32(vcp, pack4(c, 0));
        store_u32(vcp + 16, pack4(c, 1));
    }
}

// ---------------------------------------------------------------------------------------
// The two passes for a column count that is no multiple of 128 (a multiple of 8: GPT-2-XL's
// d = 1600, a 1000-class head).  The 128-value groups of the first moment are cut from the
// flattened tensor (group_tensor, lpmm/functional.py:404-422), so here they straddle tensor rows
// and the 128 columns a DPP row works on lie in up to two of them.  The first moment therefore
// takes the route of the wide groups above: the update pass merges the maxima of the new first
// moment into the next scales (one masked row maximum per group a DPP row touches) and the second
// pass recomputes it and writes its codes; any group size from 128 to 4096 is served.  The last
// 128-column block of a row is cut: its lanes beyond the row load nothing, store nothing and
// contribute zeros to every maximum.  A lane's two runs of four values stay whole (the column
// count is a multiple of 4), their codes are one 16-bit access each.
// ---------------------------------------------------------------------------------------
struct RaggedRow {
    int64_t flat;  // index of the DPP row's first value in the flattened tensor
    bool in0, in1;  // does the lane's first / second run of four lie inside the tensor row
};

__device__ __forceinline__ RaggedRow ragged_row(const TensorR1 &t, int64_t cols, uint32_t cg, int lane16, int64_t r)
{
    RaggedRow w;
    const int64_t c0 = (int64_t)cg * kGroup;
    w.flat = r * cols + c0;
    w.in0 = c0 + lane16 * 4 < cols;
    w.in1 = c0 + 64 + lane16 * 4 < cols;
    return w;
}

__global__ __launch_bounds__(kThreads) void rank1_update_ragged_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                      const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[(kColExtra + kMaxWide * kRedSlotWords * 4) / 4];
    uint32_t *colred = lds + kColExtra / 4;
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)(t.col_blocks - 1) * kGroup + t.col_tail;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    lds_fill(lds, qmap_m, qmap_v);
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads)
        lds[kColOld / 4 + j] = (j < q.wide * kGroup && tile_c0 + j < cols) ? __float_as_uint(t.col_old[tile_c0 + j]) : 0u;
    for (int j = threadIdx.x; j < kMaxWide * (int)kRedSlotWords; j += kThreads)
        colred[j] = 0u;
    NfHyper h;
    h.decay = args.decay;
    h.w1 = args.w1;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.eps = args.eps;
    h.neg_step_size = t.neg_step_size;
    h.bc2_sqrt = t.bc2_sqrt;
    h.rbc2_sqrt = t.rbc2_sqrt;
    __syncthreads();

    const int slot = drow & (q.wide - 1);
    const int lg_group = 7 + (int)t.m_lg;
    if (q.cg < t.col_blocks) {
        const uint32_t co_off = kColOld + (slot * kGroup + lane16 * 4) * 4;
        uint32_t *red = colred + slot * kRedSlotWords + lane16;
        float co[kEltsPerLane];
        unpack8(lds_read<float4>(lds, co_off), lds_read<float4>(lds, co_off + 256), co);
#pragma unroll 1
        for (int it = 0; it < q.passes; ++it) {
            const int64_t r = q.row0 + it * q.step;
            if (r >= t.rows)
                break;
            const RaggedRow w = ragged_row(t, cols, q.cg, lane16, r);
            const int64_t f0 = w.flat + lane16 * 4, f1 = f0 + 64;
            const float4 zero4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            const float4 a0 = w.in0 ? load4(t.p + f0) : zero4, a1 = w.in1 ? load4(t.p + f1) : zero4;
            const float4 b0 = w.in0 ? load4(t.g + f0) : zero4, b1 = w.in1 ? load4(t.g + f1) : zero4;
            const int64_t g0 = f0 >> lg_group, g1 = f1 >> lg_group;
            uint32_t wm = 0, wv = 0;
            float sm0 = 0.0f, sm1 = 0.0f;
            if (w.in0) {
                wm = load_u16(reinterpret_cast<const uint16_t *>(t.mc + (f0 >> 1)));
                wv = load_u16(reinterpret_cast<const uint16_t *>(t.vc + (f0 >> 1)));
                sm0 = t.ms[g0];
            }
            if (w.in1) {
                wm |= (uint32_t)load_u16(reinterpret_cast<const uint16_t *>(t.mc + (f1 >> 1))) << 16;
                wv |= (uint32_t)load_u16(reinterpret_cast<const uint16_t *>(t.vc + (f1 >> 1))) << 16;
                sm1 = t.ms[g1];
            }
            const float ro = t.row_old[r];
            float pv[kEltsPerLane], gv[kEltsPerLane], m[kEltsPerLane], v[kEltsPerLane];
            unpack8(a0, a1, pv);
            unpack8(b0, b1, gv);
            const Nibbles nm = split_nibbles(wm), nv = split_nibbles(wv);
            float max0 = 0.0f, max1 = 0.0f, vmax = 0.0f;
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                // outside the row: p = g = 0 and zero scales, so m = v = 0 and nothing below sees them
                m[k] = decode_nibble(lds, kLdsQ0, nm, k) * (k < 4 ? sm0 : sm1);
                const float sc = (co[k] < ro) ? co[k] : ro;
                v[k] = decode_nibble(lds, kLdsQ1, nv, k) * ((k < 4 ? w.in0 : w.in1) ? sc : 0.0f);
                nonfused_elt(pv[k], gv[k], m[k], v[k], h);
                if (k < 4)
                    max0 = fmaxf(max0, fabsf(m[k]));
                else
                    max1 = fmaxf(max1, fabsf(m[k]));
                vmax = fmaxf(vmax, v[k]);
                atomicMax(red + k * 16, __float_as_uint(v[k]));
            }
            // the DPP row's 128 values lie in the group of its first value or in the next one
            const int64_t glo = w.flat >> lg_group;
            float mlo = fmaxf(g0 == glo ? max0 : 0.0f, g1 == glo ? max1 : 0.0f);
            float mhi = fmaxf(g0 == glo ? 0.0f : max0, g1 == glo ? 0.0f : max1);
            row16_max2(mlo, mhi);
            vmax = row16_max(vmax);
            if (w.in0)
                store4(t.p + f0, make_float4(pv[0], pv[1], pv[2], pv[3]));
            if (w.in1)
                store4(t.p + f1, make_float4(pv[4], pv[5], pv[6], pv[7]));
            if (lane16 == 0) {
                // a maximum of zero changes nothing (the next scales start at zero), and only then
                // can the group lie past the end of the tensor
                if (mlo != 0.0f)
                    atomic_max_nonneg(t.ms_new + glo, mlo);
                if (mhi != 0.0f)
                    atomic_max_nonneg(t.ms_new + glo + 1, mhi);
                atomic_max_nonneg(t.row_new + r, vmax);
            }
        }
    }
    __syncthreads();
    // column j of the tile = element k of lane l of slot s
    for (int j = threadIdx.x; j < q.wide * kGroup; j += kThreads) {
        const int w = j & (kGroup - 1);
        const int k = ((w >> 6) << 2) | (w & 3), l = (w >> 2) & 15;
        if (tile_c0 + j < cols)
            atomic_max_nonneg(t.col_new + tile_c0 + j, __uint_as_float(colred[(j >> 7) * kRedSlotWords + k * 16 + l]));
    }
}

__global__ __launch_bounds__(kThreads) void rank1_requant_ragged_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                       const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[(kColExtra + 2 * kColBytes) / 4];
    constexpr uint32_t kColNew = kColExtra, kColRcp = kColExtra + kColBytes;
    lds_fill(lds, qmap_m, qmap_v);
    const int kind_m = classify_map(qmap_m), kind_v = classify_map(qmap_v);
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)(t.col_blocks - 1) * kGroup + t.col_tail;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads) {
        const bool in = j < q.wide * kGroup && tile_c0 + j < cols;
        // columns outside the tensor: statistics of 1, so that they do not keep a wave off the fast division
        const float cn = in ? t.col_new[tile_c0 + j] : 1.0f;
        lds[kColOld / 4 + j] = in ? __float_as_uint(t.col_old[tile_c0 + j]) : 0u;
        lds[kColNew / 4 + j] = __float_as_uint(cn);
        lds[kColRcp / 4 + j] = __float_as_uint(1.0f / cn);
    }
    NfHyper h;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.w1 = args.w1;
    __syncthreads();

    const int lg_group = 7 + (int)t.m_lg;
    if (tl == 0) {
        // Padding.  Second moment: plain zeros from the end of the tensor to whole pack groups of 2048
        // values.  First moment: the quantiser pads the flattened tensor with zeros to whole groups,
        // which are divided by the last group's scale like its other values (0/0 -> NaN -> code 15
        // when the group is all zero); the packing pads with plain zeros behind that.
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t n = t.rows * cols;
        write_padding(t.vc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                      encode8_plain(lds, kLdsQ1, kind_v, z));
        const int64_t group = (int64_t)1 << lg_group;
        const int64_t n_grp = (n + group - 1) / group * group;
        const int64_t n_all = (n_grp + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP;
        const uint32_t zero_word = encode8_plain(lds, kLdsQ0, kind_m, z);
        uint32_t last_word = zero_word;
        if (n_grp > n) {
            const float last = t.ms_new[(n - 1) >> lg_group];
            const float zs[kEltsPerLane] = {0.0f / last, 0.0f / last, 0.0f / last, 0.0f / last,
                                            0.0f / last, 0.0f / last, 0.0f / last, 0.0f / last};
            last_word = encode8_plain(lds, kLdsQ0, kind_m, zs);
        }
        for (int64_t i = n + (int64_t)threadIdx.x * kEltsPerLane; i < n_all; i += kThreads * kEltsPerLane)
            *reinterpret_cast<uint32_t *>(t.mc + (i >> 1)) = i < n_grp ? last_word : zero_word;
        if (threadIdx.x == 0)
            t.mc[n_all / 2] = 0;
    }
    if (q.cg >= t.col_blocks)
        return;

    const uint32_t col_off = ((drow & (q.wide - 1)) * kGroup + lane16 * 4) * 4;
    float co[kEltsPerLane], cn[kEltsPerLane], rcn[kEltsPerLane];
    unpack8(lds_read<float4>(lds, kColOld + col_off), lds_read<float4>(lds, kColOld + col_off + 256), co);
    unpack8(lds_read<float4>(lds, kColNew + col_off), lds_read<float4>(lds, kColNew + col_off + 256), cn);
    unpack8(lds_read<float4>(lds, kColRcp + col_off), lds_read<float4>(lds, kColRcp + col_off + 256), rcn);
    bool cols_safe = true;
#pragma unroll
    for (int k = 0; k < kEltsPerLane; ++k)
        cols_safe = cols_safe && rc_safe(cn[k]);
#pragma unroll 1
    for (int it = 0; it < q.passes; ++it) {
        const int64_t r = q.row0 + it * q.step;
        if (r >= t.rows)
            break;
        const RaggedRow w = ragged_row(t, cols, q.cg, lane16, r);
        const int64_t f0 = w.flat + lane16 * 4, f1 = f0 + 64;
        const float4 zero4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        const float4 b0 = w.in0 ? load4(t.g + f0) : zero4, b1 = w.in1 ? load4(t.g + f1) : zero4;
        uint16_t *mc0 = reinterpret_cast<uint16_t *>(t.mc + (f0 >> 1)), *mc1 = reinterpret_cast<uint16_t *>(t.mc + (f1 >> 1));
        uint16_t *vc0 = reinterpret_cast<uint16_t *>(t.vc + (f0 >> 1)), *vc1 = reinterpret_cast<uint16_t *>(t.vc + (f1 >> 1));
        uint32_t wm = 0, wv = 0;
        float so0 = 0.0f, so1 = 0.0f, sn0 = 1.0f, sn1 = 1.0f;  // outside the row: 0 / 1
        if (w.in0) {
            wm = load_u16(mc0);
            wv = load_u16(vc0);
            so0 = t.ms[f0 >> lg_group];
            sn0 = t.ms_new[f0 >> lg_group];
        }
        if (w.in1) {
            wm |= (uint32_t)load_u16(mc1) << 16;
            wv |= (uint32_t)load_u16(vc1) << 16;
            so1 = t.ms[f1 >> lg_group];
            sn1 = t.ms_new[f1 >> lg_group];
        }
        const float ro = t.row_old[r], rn = t.row_new[r];
        float gv[kEltsPerLane], v[kEltsPerLane], m[kEltsPerLane], x[kEltsPerLane];
        unpack8(b0, b1, gv);
        const Nibbles nm = split_nibbles(wm), nv = split_nibbles(wv);
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            v[k] = decode_nibble(lds, kLdsQ1, nv, k) * ((co[k] < ro) ? co[k] : ro);
            nonfused_second_moment(v[k], gv[k], h);
            m[k] = lerp_w(decode_nibble(lds, kLdsQ0, nm, k) * (k < 4 ? so0 : so1), gv[k], h.w1);
        }
        // Every divisor is a maximum over the values it divides (|x| <= y): where all of a wave's
        // divisors lie in the range in which the reciprocal is exact, the correctly rounded
        // reciprocal, one multiply and two fmas give the correctly rounded quotient.
        uint32_t cm, cv;
        if (kind_m == kMapStdM && __all(rc_safe(sn0) && rc_safe(sn1))) {
            const float rc0 = rcp_exact(sn0), rc1 = rcp_exact(sn1);
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                x[k] = div_by_rc(m[k], k < 4 ? sn0 : sn1, k < 4 ? rc0 : rc1);
            cm = encode8_std_m(lds, x);
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                x[k] = m[k] / (k < 4 ? sn0 : sn1);
            cm = encode8_plain(lds, kLdsQ0, kind_m, x);
        }
        if (kind_v == kMapStdV && __all(cols_safe && rc_safe(rn))) {
            const float rcr = rcp_exact(rn);
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const bool by_col = cn[k] < rn;
                x[k] = div_by_rc(v[k], by_col ? cn[k] : rn, by_col ? rcn[k] : rcr);
            }
            cv = encode8_std_v(x);
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                x[k] = v[k] / ((cn[k] < rn) ? cn[k] : rn);
            cv = encode8_plain(lds, kLdsQ1, kind_v, x);
        }
        if (w.in0) {
            store_u16(mc0, cm & 0xFFFFu);
            store_u16(vc0, cv & 0xFFFFu);
        }
        if (w.in1) {
            store_u16(mc1, cm >> 16);
            store_u16(vc1, cv >> 16);
        }
    }
}

}  // namespace lpmm

using namespace lpmm;

// The widest tile the policy allows (longest contiguous runs) that leaves at most 10 % of the DPP
// rows of a tensor's tiles without a column group; otherwise the width that wastes least.  (13
// column groups, 1600 columns: tiles of two groups with one DPP row in 14 idle run 4 % faster than
// tiles of one group.)
static uint32_t choose_lg_wide(uint32_t col_blocks)
{
    uint32_t best = 0;
    double best_use = 0.0;
    for (int lg = kPolicyLgWide; lg >= 0; --lg) {
        const uint32_t wide = 1u << lg;
        const double use = (double)col_blocks / (double)((col_blocks + wide - 1) / wide * wide);
        if (use >= 0.90)
            return (uint32_t)lg;
        if (use > best_use) {
            best_use = use;
            best = (uint32_t)lg;
        }
    }
    return best;
}

// Tile shape of a rows x (128 * col_blocks) tensor, and its tile count.
static uint64_t shape_tiles(int64_t rows, uint32_t col_blocks, TileShape &ts)
{
    const uint32_t lg_wide = choose_lg_wide(col_blocks);
    const uint32_t col_tiles = (col_blocks + (1u << lg_wide) - 1) >> lg_wide;
    const uint32_t pass_rows = (uint32_t)kDppRows >> lg_wide;
    const uint32_t tile_rows = pass_rows > kPolicyRows ? pass_rows : kPolicyRows;
    const uint64_t row_blocks = (uint64_t)((rows + tile_rows - 1) / tile_rows);
    uint64_t comb = kPolicyResident / col_tiles;
    comb = comb < 1 ? 1 : comb;
    comb = comb > row_blocks ? row_blocks : comb;
    ts.lg_wide = lg_wide;
    ts.tile_rows = tile_rows;
    ts.comb = (uint32_t)comb;
    return (row_blocks + comb - 1) / comb * comb * col_tiles;  // whole groups: the last may hold empty blocks
}

// The first moment of a record: its codes and scales, or the fp32 moment itself.
static uint8_t *first_moment(const lpmm_nonfused_rank1_tensor &t) { return t.m_codes; }
static float *first_moment_scales(const lpmm_nonfused_rank1_tensor &t) { return t.m_max1; }
static uint8_t *first_moment(const lpmm_rank1_v4bit_tensor &t) { return reinterpret_cast<uint8_t *>(t.m); }
static float *first_moment_scales(const lpmm_rank1_v4bit_tensor &) { return nullptr; }
static uint8_t *first_moment(const lpmm_rank1_mgroup_tensor &t) { return t.m_codes; }
static float *first_moment_scales(const lpmm_rank1_mgroup_tensor &t) { return const_cast<float *>(t.m_max1); }
static float *next_scales(const lpmm_nonfused_rank1_tensor &) { return nullptr; }
static float *next_scales(const lpmm_rank1_v4bit_tensor &) { return nullptr; }
static float *next_scales(const lpmm_rank1_mgroup_tensor &t) { return t.m_max1_next; }

// Validation, batching into launches of at most kR1Max tensors, and the three launches.
// m_lg: the first moment's group holds 128 << m_lg values (MODE kMCodesWide only).
template <int MODE, class Record>
static int rank1_step_multi(const Record *tensors, int64_t count, const float *qmap_m, const float *qmap_v,
                            uint32_t m_lg, double beta1, double beta2, double lr, double weight_decay, double eps,
                            void *stream, int bits_m = 4, int bits_v = 4)
{
    constexpr bool M32 = MODE == kMFloat;
    // column counts that are no multiple of 128 (wide-group records only): every tensor of the call
    // then takes the kernels for ragged rows
    bool ragged = false;
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(tensors);
    LPMM_REQUIRE_PTR(qmap_m);
    LPMM_REQUIRE_PTR(qmap_v);
    LPMM_REQUIRE_ALIGN(qmap_m, 4);
    LPMM_REQUIRE_ALIGN(qmap_v, 4);
    for (int64_t i = 0; i < count; ++i) {
        const Record &t = tensors[i];
        if (t.rows < 0 || t.cols < 0 || t.cols % (MODE == kMCodesWide ? 8 : kGroup) != 0)
            return LPMM_ERR_SIZE;
        ragged = ragged || t.cols % kGroup != 0;
        if (t.rows == 0 || t.cols == 0)
            continue;
        const int64_t col_blocks = (t.cols + kGroup - 1) / kGroup;
        // an upper bound: tiles hold at least 16 rows, the last group adds fewer than `resident` blocks
        const int64_t row_blocks = (t.rows + kDppRows - 1) / kDppRows + kPolicyResident;
        if (col_blocks > 0x7fffffffLL / 2 || row_blocks > 0x7fffffffLL / col_blocks ||
            t.rows > INT64_MAX / t.cols)
            return LPMM_ERR_SIZE;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(first_moment(t));
        if (!M32)
            LPMM_REQUIRE_PTR(first_moment_scales(t));
        LPMM_REQUIRE_PTR(t.v_codes);
        LPMM_REQUIRE_PTR(t.v_rowmax);
        LPMM_REQUIRE_PTR(t.v_colmax);
        LPMM_REQUIRE_PTR(t.v_rowmax_next);
        LPMM_REQUIRE_PTR(t.v_colmax_next);
        LPMM_REQUIRE_ALIGN(t.p, 16);
        LPMM_REQUIRE_ALIGN(t.g, 16);
        LPMM_REQUIRE_ALIGN(first_moment(t), M32 ? 16 : 4);
        LPMM_REQUIRE_ALIGN(t.v_codes, 4);
        LPMM_REQUIRE_ALIGN(first_moment_scales(t), 4);
        if (MODE == kMCodesWide) {
            LPMM_REQUIRE_PTR(next_scales(t));
            LPMM_REQUIRE_ALIGN(next_scales(t), 4);
            if (next_scales(t) == first_moment_scales(t))
                return LPMM_ERR_ARG;
        }
        LPMM_REQUIRE_ALIGN(t.v_rowmax, 4);
        LPMM_REQUIRE_ALIGN(t.v_colmax, 16);
        LPMM_REQUIRE_ALIGN(t.v_rowmax_next, 4);
        LPMM_REQUIRE_ALIGN(t.v_colmax_next, 16);
        if (t.v_rowmax == t.v_rowmax_next || t.v_colmax == t.v_colmax_next)
            return LPMM_ERR_ARG;
    }

    const NfHyper c = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, 1.0);
    MultiR1 args;
    args.decay = c.decay;
    args.w1 = c.w1;
    args.b2 = c.b2;
    args.w2 = c.w2;
    args.eps = c.eps;
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t tiles = 0;
        int64_t longest = 0;
        args.tile_start[0] = 0;
        while (i < count && k < kR1Max) {
            const Record &t = tensors[i];
            if (t.rows == 0 || t.cols == 0) {
                ++i;
                continue;
            }
            const uint32_t col_blocks = (uint32_t)((t.cols + kGroup - 1) / kGroup);
            TensorR1 &d = args.t[k];
            const uint64_t nt = shape_tiles(t.rows, col_blocks, d.tile);
            if (tiles + nt > 0x7fffffffULL)
                break;
            d.p = t.p;
            d.g = t.g;
            d.mc = first_moment(t);
            d.ms = first_moment_scales(t);
            d.ms_new = next_scales(t);
            d.m_lg = m_lg;
            d.vc = t.v_codes;
            d.row_old = t.v_rowmax;
            d.col_old = t.v_colmax;
            d.row_new = t.v_rowmax_next;
            d.col_new = t.v_colmax_next;
            d.rows = t.rows;
            d.col_blocks = col_blocks;
            d.col_tail = (uint32_t)(t.cols - (int64_t)(col_blocks - 1) * kGroup);
            const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, t.step);
            d.neg_step_size = h.neg_step_size;
            d.bc2_sqrt = h.bc2_sqrt;
            d.rbc2_sqrt = h.rbc2_sqrt;
            longest = t.rows + t.cols > longest ? t.rows + t.cols : longest;
            tiles += nt;
            args.tile_start[++k] = (uint32_t)tiles;
            ++i;
        }
        if (k == 0) {
            if (i < count)
                return LPMM_ERR_SIZE;  // a single tensor with more tiles than a grid holds
            continue;
        }
        args.count = k;
        for (int j = k + 1; j <= kR1Max; ++j)
            args.tile_start[j] = (uint32_t)tiles;
        int64_t clear_blocks = (longest + kThreads - 1) / kThreads;
        clear_blocks = clear_blocks > 64 ? 64 : clear_blocks;
        hipLaunchKernelGGL(rank1_clear_kernel, dim3((uint32_t)clear_blocks, (uint32_t)k), dim3(kThreads), 0,
                           (hipStream_t)stream, args);
        if (ragged || (MODE == kMCodesWide && m_lg == 0)) {
            hipLaunchKernelGGL(rank1_update_ragged_kernel, dim3((uint32_t)tiles), dim3(kThreads), 0,
                               (hipStream_t)stream, args, qmap_m, qmap_v);
            hipLaunchKernelGGL(rank1_requant_ragged_kernel, dim3((uint32_t)tiles), dim3(kThreads), 0,
                               (hipStream_t)stream, args, qmap_m, qmap_v);
        } else if (bits_m != 4) {
            hipLaunchKernelGGL(rank1_update_bits_kernel, dim3((uint32_t)tiles), dim3(kThreads), 0, (hipStream_t)stream,
                               args, qmap_m, qmap_v, bits_m, bits_v);
            hipLaunchKernelGGL(rank1_requant_bits_kernel, dim3((uint32_t)tiles), dim3(kThreads), 0,
                               (hipStream_t)stream, args, qmap_v, bits_v);
        } else {
            hipLaunchKernelGGL(rank1_update_kernel<MODE>, dim3((uint32_t)tiles), dim3(kThreads), 0,
                               (hipStream_t)stream, args, qmap_m, qmap_v);
            hipLaunchKernelGGL(rank1_requant_kernel<MODE == kMCodesWide>, dim3((uint32_t)tiles), dim3(kThreads), 0,
                               (hipStream_t)stream, args, qmap_m, qmap_v);
        }
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}

extern "C" int lpmm_nonfused_adamw4bit_rank1_step_multi(const lpmm_nonfused_rank1_tensor *tensors, int64_t count,
                                                        const float *qmap_m, const float *qmap_v, double beta1,
                                                        double beta2, double lr, double weight_decay,
                                                        double eps, void *stream)
{
    return rank1_step_multi<kMCodes128>(tensors, count, qmap_m, qmap_v, 0, beta1, beta2, lr, weight_decay, eps, stream);
}

extern "C" int lpmm_nonfused_adamw_v4bit_rank1_step_multi(const lpmm_rank1_v4bit_tensor *tensors, int64_t count,
                                                          const float *qmap_v, double beta1, double beta2,
                                                          double lr, double weight_decay, double eps,
                                                          void *stream)
{
    // the update kernel keeps the second moment's map in both map slots; only the second is read
    return rank1_step_multi<kMFloat>(tensors, count, qmap_v, qmap_v, 0, beta1, beta2, lr, weight_decay, eps, stream);
}

extern "C" int lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi(const lpmm_rank1_mgroup_tensor *tensors, int64_t count,
                                                               const float *qmap_m, const float *qmap_v,
                                                               int64_t m_group_size, double beta1, double beta2,
                                                               double lr, double weight_decay, double eps,
                                                               void *stream)
{
    uint32_t m_lg = 0;
    while (m_lg < 5 && ((int64_t)kGroup << m_lg) < m_group_size)
        ++m_lg;
    if (((int64_t)kGroup << m_lg) != m_group_size)
        return LPMM_ERR_SIZE;  // 128, 256, 512, 1024, 2048 or 4096
    return rank1_step_multi<kMCodesWide>(tensors, count, qmap_m, qmap_v, m_lg, beta1, beta2, lr, weight_decay, eps,
                                         stream);
}

extern "C" int lpmm_nonfused_adamw_bits_rank1_step_multi(const lpmm_nonfused_rank1_tensor *tensors, int64_t count,
                                                         const float *qmap_m, int bits_m, const float *qmap_v,
                                                         int bits_v, double beta1, double beta2, double lr,
                                                         double weight_decay, double eps, void *stream)
{
    if (bits_m < 5 || bits_m > 8 || bits_v < 5 || bits_v > 8)
        return LPMM_ERR_ARG;  // the widths that store one code per byte
    return rank1_step_multi<kMCodes128>(tensors, count, qmap_m, qmap_v, 0, beta1, beta2, lr, weight_decay, eps, stream,
                                        bits_m, bits_v);
}
