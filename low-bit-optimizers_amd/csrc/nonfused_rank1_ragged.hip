// The two passes of the non-fused AdamW step with a rank-1 second moment for column counts that
// are a multiple of 8 but not of 128.  Tiles, records and statistics as in nonfused_rank1.hip.
#include "rank1_tiles.hpp"

namespace lpmm {

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
    __shared__ __align__(16) uint32_t lds[(kColExtra + kMaxWide * kRedSlotWords * 4) / 4 + kRowSlots];
    uint32_t *colred = lds + kColExtra / 4;
    uint32_t *rowred = colred + kMaxWide * kRedSlotWords;
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
    if (threadIdx.x < kRowSlots)
        rowred[threadIdx.x] = 0u;
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
                atomicMax(rowred + row_slot(t.tile, it, drow), __float_as_uint(vmax));  // rank1_tiles.hpp
            }
        }
    }
    __syncthreads();
    flush_row_maxima(rowred, t.tile, q, drow, t.rows, false, t.row_new);
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

void launch_rank1_ragged(const MultiR1 &args, uint32_t tiles, const float *qmap_m, const float *qmap_v,
                         hipStream_t stream)
{
    hipLaunchKernelGGL(rank1_update_ragged_kernel, dim3(tiles), dim3(kThreads), 0, stream, args, qmap_m, qmap_v);
    hipLaunchKernelGGL(rank1_requant_ragged_kernel, dim3(tiles), dim3(kThreads), 0, stream, args, qmap_m, qmap_v);
}

}  // namespace lpmm
