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
#include "rank1_tiles.hpp"

namespace lpmm {

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
    float sm, ro, ro1;  // ro1: the second half's row statistic (folded rows; otherwise ro)
};

template <int MODE, bool FOLD>
__device__ __forceinline__ void pass_fetch(const TensorR1 &t, const Fold &f, uint32_t cg, int lane16, int64_t r, PassRegs &x)
{
    const int64_t grp = r * f.col_blocks + cg;
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
    if (FOLD) {
        int64_t r0, r1;
        fold_rows(f, r, cg, r0, r1);
        x.ro = t.row_old[r0];
        x.ro1 = t.row_old[r1];
    } else {
        x.ro = x.ro1 = t.row_old[r];
    }
}

#ifndef LPMM_R1_WAVES
#define LPMM_R1_WAVES 4
#endif
// 4 waves per SIMD, up to 128 registers: the first pass's operands stay live across the prologue and
// the lane's column statistics across the passes (with 5 or 6 the compiler spills or re-reads)
template <int MODE, bool FOLD>
__global__ __launch_bounds__(kThreads, LPMM_R1_WAVES) void rank1_update_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[(kColExtra + kMaxWide * kRedSlotWords * 4) / 4 + kRowSlots];
    uint32_t *colred = lds + kColExtra / 4;
    uint32_t *rowred = colred + kMaxWide * kRedSlotWords;
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Fold f = fold_of<FOLD>(t);
    const Geometry q = geometry(t.tile, f.col_blocks, tl, drow);
    const int64_t cols = (int64_t)f.col_blocks * kGroup;
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
        co_in[i] = (j < q.wide * kGroup && tile_c0 + j < cols)
                       ? __float_as_uint(t.col_old[FOLD ? fold_col(f, (uint32_t)(tile_c0 + j)) : tile_c0 + j])
                       : 0u;
    }
    const bool row_live = q.cg < f.col_blocks;  // the whole DPP row
    PassRegs x;
    if (row_live && q.row0 < f.rows)
        pass_fetch<MODE, FOLD>(t, f, q.cg, lane16, q.row0, x);
    lds_fill_store(lds, fill);
    for (int j = threadIdx.x; j < kMaxWide * (int)kRedSlotWords; j += kThreads)
        colred[j] = 0u;
    if (threadIdx.x < kRowSlots)
        rowred[threadIdx.x] = 0u;
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
        const int64_t n = f.rows * cols;
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
            if (r >= f.rows)
                break;
            if (it > 0)
                pass_fetch<MODE, FOLD>(t, f, q.cg, lane16, r, x);
            const int64_t grp = r * f.col_blocks + q.cg;
            const int64_t gbase = grp * kGroup;
            float *pp = t.p + gbase + lane16 * 4;
            const uint32_t wv = x.v0 | (x.v1 << 16);
            const float ro = x.ro, ro1 = FOLD ? x.ro1 : x.ro;
            float pv[kEltsPerLane], gv[kEltsPerLane], m[kEltsPerLane], v[kEltsPerLane];
            unpack8(x.a0, x.a1, pv);
            unpack8(x.b0, x.b1, gv);
            constexpr bool M32 = MODE == kMFloat;
            const Nibbles nm = split_nibbles(M32 ? 0u : (x.m0 | (x.m1 << 16)));
            const float sm = M32 ? 0.0f : x.sm;
            if (M32)
                unpack8(x.c0, x.c1, m);

            const Nibbles nv = split_nibbles(wv);
            float amax_m = 0.0f, vmax = 0.0f, vmax1 = 0.0f;  // vmax1: the second half's (folded rows)
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                if (!M32)
                    m[k] = decode_nibble(lds, kLdsQ0, nm, k) * sm;
                const float rk = (FOLD && k >= 4) ? ro1 : ro;
                v[k] = decode_nibble(lds, kLdsQ1, nv, k) * ((co[k] < rk) ? co[k] : rk);
                nonfused_elt(pv[k], gv[k], m[k], v[k], h);
                amax_m = fmaxf(amax_m, fabsf(m[k]));
                if (FOLD && k >= 4)
                    vmax1 = fmaxf(vmax1, v[k]);
                else
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
            if (FOLD)
                vmax1 = row16_max(vmax1);

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
            if (lane16 == 0) {
                // the maxima of a tensor row meet in LDS (rank1_tiles.hpp); folded rows: a half goes to the
                // tensor row it lies in
                uint32_t *slot = rowred + row_slot(t.tile, it, drow);
                if (FOLD) {
                    const bool h0 = f.on && q.cg * kGroup >= f.real_cols, h1 = f.on && q.cg * kGroup + 64 >= f.real_cols;
                    atomicMax(slot + (h0 ? 1 : 0), __float_as_uint(vmax));
                    atomicMax(slot + (h1 ? 1 : 0), __float_as_uint(vmax1));
                } else {
                    atomicMax(slot, __float_as_uint(vmax));
                }
            }
        }
    }
    // the column maxima meet in LDS: nothing below depends on the global stores still in flight
    lds_barrier();
    flush_row_maxima(rowred, t.tile, q, drow, f.rows, FOLD && f.on, t.row_new);
    // column j of the tile = element k of lane l of slot s
    for (int j = threadIdx.x; j < q.wide * kGroup; j += kThreads) {
        const int w = j & (kGroup - 1);
        const int k = ((w >> 6) << 2) | (w & 3), l = (w >> 2) & 15;
        if (tile_c0 + j < cols) {
            float *dst = t.col_new + (FOLD ? fold_col(f, (uint32_t)(tile_c0 + j)) : tile_c0 + j);
            const uint32_t mine = colred[(j >> 7) * kRedSlotWords + k * 16 + l];
            atomic_max_nonneg(dst, __uint_as_float(mine));
        }
    }
}

// MWIDE: the first moment's groups are wider than 128 values; its codes are written here too.
template <bool MWIDE, bool FOLD>
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
    const Fold f = fold_of<FOLD>(t);
    const Geometry q = geometry(t.tile, f.col_blocks, tl, drow);
    const int64_t cols = (int64_t)f.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    for (int j = threadIdx.x; j < q.wide * kGroup; j += kThreads) {
        const bool in = tile_c0 + j < cols;
        const int64_t c = FOLD ? fold_col(f, (uint32_t)(tile_c0 + j)) : tile_c0 + j;
        const float cn = in ? t.col_new[c] : 0.0f;
        lds[kColOld / 4 + j] = in ? __float_as_uint(t.col_old[c]) : 0u;
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
        const int64_t n = f.rows * cols;
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
    if (q.cg >= f.col_blocks)
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
        cols_safe = cols_safe && rc_safe(cn[k]) && co[k] == co[k];
    // the group's 64 code bytes move as one dword per lane (whole lines per access; with the
    // arithmetic taken out this pass is 11 % faster than with two 16-bit accesses per lane)
    const uint32_t code_dword = code_dword_of_lane(lane16), code_sel = code_swap_selector(lane16);
#pragma unroll 1
    for (int it = 0; it < q.passes; ++it) {
        const int64_t r = q.row0 + it * q.step;
        if (r >= f.rows)
            break;
        const int64_t gbase = (r * f.col_blocks + q.cg) * kGroup;
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
        int64_t r0 = r, r1 = r;  // the tensor rows of the DPP row's two halves
        if (FOLD)
            fold_rows(f, r, q.cg, r0, r1);
        const float ro = t.row_old[r0], rn = t.row_new[r0];
        const float ro1 = FOLD ? t.row_old[r1] : ro, rn1 = FOLD ? t.row_new[r1] : rn;
        float gv[kEltsPerLane], v[kEltsPerLane], x[kEltsPerLane];
        unpack8(b0, b1, gv);
        const Nibbles nv = split_nibbles(wv);
        // Every statistic the wave touches is a number, and the new ones lie in the range in which the
        // reciprocal is exact?  Then minima and maxima of these non-negative values can be taken on their
        // bit patterns (one instruction each), and the reciprocal of the smaller statistic is the larger
        // of the two reciprocals (rounding is monotonic).
        // (Where that saves registers as well -- double rows, wide first-moment groups -- it is 0.4-3 %
        // of the step; the plain variant would go from 74 to 82 registers and lose a wave per SIMD.)
        constexpr bool kBitMin = FOLD || MWIDE;
        const bool fast = kind == kMapStdV && __all(cols_safe && rc_safe(rn) && rc_safe(rn1) && ro == ro && ro1 == ro1);
        if (kBitMin && fast) {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const float rk = (FOLD && k >= 4) ? ro1 : ro;
                v[k] = decode_nibble(lds, kVMap, nv, k) * __uint_as_float(min(__float_as_uint(co[k]), __float_as_uint(rk)));
                nonfused_second_moment(v[k], gv[k], h);
            }
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const float rk = (FOLD && k >= 4) ? ro1 : ro;
                v[k] = decode_nibble(lds, kVMap, nv, k) * ((co[k] < rk) ? co[k] : rk);
                nonfused_second_moment(v[k], gv[k], h);
            }
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
        if (fast) {
            // the correctly rounded reciprocal of whichever statistic is the scale, then one
            // multiply and two fmas: the correctly rounded quotient (v <= scale by construction)
            const float rcr = rcp_exact(rn), rcr1 = FOLD ? rcp_exact(rn1) : rcr;
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const float rnk = (FOLD && k >= 4) ? rn1 : rn, rck = (FOLD && k >= 4) ? rcr1 : rcr;
                if (kBitMin) {
                    const float sk = __uint_as_float(min(__float_as_uint(cn[k]), __float_as_uint(rnk)));
                    const float rk = __uint_as_float(max(__float_as_uint(rcn[k]), __float_as_uint(rck)));
                    x[k] = div_by_rc(v[k], sk, rk);
                } else {
                    const bool by_col = cn[k] < rnk;
                    x[k] = div_by_rc(v[k], by_col ? cn[k] : rnk, by_col ? rcn[k] : rck);
                }
            }
            w = encode8_std_v(x);
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const float rnk = (FOLD && k >= 4) ? rn1 : rn;
                x[k] = v[k] / ((cn[k] < rnk) ? cn[k] : rnk);
            }
            w = encode8_plain(lds, kVMap, kind, x);
        }
        store_u32(vcp, swap_code_halves(w, code_sel));
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
static uint64_t shape_tiles(int64_t rows, uint32_t col_blocks, TileShape &ts, uint32_t policy_rows)
{
    const uint32_t lg_wide = choose_lg_wide(col_blocks);
    const uint32_t col_tiles = (col_blocks + (1u << lg_wide) - 1) >> lg_wide;
    const uint32_t pass_rows = (uint32_t)kDppRows >> lg_wide;
    const uint32_t tile_rows = pass_rows > policy_rows ? pass_rows : policy_rows;
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

// a tensor that the kernels take as double rows
static bool folds(int64_t rows, int64_t cols) { return cols % kGroup == 64 && rows % 2 == 0; }

// Validation, batching into launches of at most kR1Max tensors, and the three launches.
// m_lg: the first moment's group holds 128 << m_lg values (MODE kMCodesWide only).
template <int MODE, class Record>
static int rank1_step_multi(const Record *tensors, int64_t count, const float *qmap_m, const float *qmap_v,
                            uint32_t m_lg, double beta1, double beta2, double lr, double weight_decay, double eps,
                            void *stream, int bits_m = 4, int bits_v = 4, const void *table_m = nullptr,
                            const void *table_v = nullptr, int passes = 3, bool half_io = false)
{
    // passes: 1 = the first pass alone (with the clearing of the next statistics), 2 = the second alone,
    // 3 = both; one at a time only where the launches below are this file's own
    if (passes < 1 || passes > 3 || (passes != 3 && (MODE != kMCodes128 || bits_m != 4 || half_io)))
        return LPMM_ERR_ARG;
    constexpr bool M32 = MODE == kMFloat;
    // 4-bit codes in 128-value groups: a column count of 64 modulo 128 with an even row count is
    // served as double rows (rank1_tiles.hpp)
    const bool can_fold = MODE == kMCodes128 && bits_m == 4 && !half_io;
    // rows per tile: with an fp32 first moment a pass moves 24.5 instead of 13.5 bytes per element, and
    // tiles of half the rows do better (LLaMA-7B-shaped set 29.3 -> 28.6 ms per step)
    const uint32_t policy_rows = M32 ? kPolicyRowsM32 : kPolicyRows;
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
        if (t.rows < 0 || t.cols < 0)
            return LPMM_ERR_SIZE;
        if (t.cols % (MODE == kMCodesWide ? 8 : kGroup) != 0 && !(can_fold && folds(t.rows, t.cols)))
            return LPMM_ERR_SIZE;
        ragged = ragged || (MODE == kMCodesWide && t.cols % kGroup != 0);
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
        bool folded = false;  // does a tensor of this launch have folded rows
        args.tile_start[0] = 0;
        while (i < count && k < kR1Max) {
            const Record &t = tensors[i];
            if (t.rows == 0 || t.cols == 0) {
                ++i;
                continue;
            }
            const uint32_t col_blocks = (uint32_t)((t.cols + kGroup - 1) / kGroup);
            TensorR1 &d = args.t[k];
            const bool fold = t.cols % kGroup != 0 && can_fold;  // validated above: 64 modulo 128, even rows
            const uint64_t nt = fold ? shape_tiles(t.rows / 2, 2 * col_blocks - 1, d.tile, policy_rows)
                                     : shape_tiles(t.rows, col_blocks, d.tile, policy_rows);
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
            folded = folded || fold;
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
        hipStream_t s = (hipStream_t)stream;
        int64_t clear_blocks = (longest + kThreads - 1) / kThreads;
        clear_blocks = clear_blocks > 64 ? 64 : clear_blocks;
        if (passes & 1)
            hipLaunchKernelGGL(rank1_clear_kernel, dim3((uint32_t)clear_blocks, (uint32_t)k), dim3(kThreads), 0,
                               s, args);
        if (half_io) {
            launch_rank1_half(args, (uint32_t)tiles, qmap_m, qmap_v, s);
        } else if (ragged || (MODE == kMCodesWide && m_lg == 0)) {
            launch_rank1_ragged(args, (uint32_t)tiles, qmap_m, qmap_v, s);
        } else if (bits_m != 4) {
            launch_rank1_bits(args, (uint32_t)tiles, qmap_m, qmap_v, bits_m, bits_v,
                              static_cast<const uint32_t *>(table_m), static_cast<const uint32_t *>(table_v),
                              s);
        } else if (MODE == kMCodes128 && folded) {
            if (passes & 1)
                hipLaunchKernelGGL((rank1_update_kernel<kMCodes128, true>), dim3((uint32_t)tiles), dim3(kThreads), 0,
                                   s, args, qmap_m, qmap_v);
            if (passes & 2)
                hipLaunchKernelGGL((rank1_requant_kernel<false, true>), dim3((uint32_t)tiles), dim3(kThreads), 0,
                                   s, args, qmap_m, qmap_v);
        } else {
            if (passes & 1)
                hipLaunchKernelGGL((rank1_update_kernel<MODE, false>), dim3((uint32_t)tiles), dim3(kThreads), 0,
                                   s, args, qmap_m, qmap_v);
            if (passes & 2)
                hipLaunchKernelGGL((rank1_requant_kernel<MODE == kMCodesWide, false>), dim3((uint32_t)tiles),
                                   dim3(kThreads), 0, s, args, qmap_m, qmap_v);
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

int lpmm::rank1_step_multi_half(const lpmm_nonfused_rank1_tensor *tensors, int64_t count, const float *qmap_m,
                                const float *qmap_v, double beta1, double beta2, double lr, double weight_decay,
                                double eps, void *stream)
{
    return rank1_step_multi<kMCodes128>(tensors, count, qmap_m, qmap_v, 0, beta1, beta2, lr, weight_decay, eps, stream,
                                        4, 4, nullptr, nullptr, 3, true);
}

extern "C" int lpmm_nonfused_adamw4bit_rank1_pass_multi(const lpmm_nonfused_rank1_tensor *tensors, int64_t count,
                                                        const float *qmap_m, const float *qmap_v, double beta1,
                                                        double beta2, double lr, double weight_decay,
                                                        double eps, int pass, void *stream)
{
    if (pass != 1 && pass != 2)
        return LPMM_ERR_ARG;
    return rank1_step_multi<kMCodes128>(tensors, count, qmap_m, qmap_v, 0, beta1, beta2, lr, weight_decay, eps, stream,
                                        4, 4, nullptr, nullptr, pass);
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
    return lpmm_nonfused_adamw_bits_rank1_step_multi_table(tensors, count, qmap_m, bits_m, nullptr, qmap_v, bits_v,
                                                           nullptr, beta1, beta2, lr, weight_decay, eps, stream);
}

extern "C" int lpmm_nonfused_adamw_bits_rank1_step_multi_table(const lpmm_nonfused_rank1_tensor *tensors, int64_t count,
                                                               const float *qmap_m, int bits_m, const void *table_m,
                                                               const float *qmap_v, int bits_v, const void *table_v,
                                                               double beta1, double beta2, double lr,
                                                               double weight_decay, double eps, void *stream)
{
    if (bits_m < 5 || bits_m > 8 || bits_v < 5 || bits_v > 8)
        return LPMM_ERR_ARG;  // the widths that store one code per byte
    if (table_m != nullptr)
        LPMM_REQUIRE_ALIGN(table_m, 16);
    if (table_v != nullptr)
        LPMM_REQUIRE_ALIGN(table_v, 16);
    return rank1_step_multi<kMCodes128>(tensors, count, qmap_m, qmap_v, 0, beta1, beta2, lr, weight_decay, eps, stream,
                                        bits_m, bits_v, table_m, table_v);
}
