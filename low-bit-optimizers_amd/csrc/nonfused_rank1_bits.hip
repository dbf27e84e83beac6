// The two passes of the non-fused AdamW step with a rank-1 second moment for code widths of 5 to 8
// bits.  Tiles, records and statistics as in nonfused_rank1.hip.
#include "lpmm_search.hpp"
#include "rank1_tiles.hpp"

namespace lpmm {

// ---------------------------------------------------------------------------------------
// The same two passes for code widths of 5 to 8 bits (lpmm/configs/default_{5,6,7,8}b.yml): one
// code per byte (lpmm/cpp_extension/quantization_kernel.cu:516-533, :656-669), maps of 2^bits
// entries in LDS, decoded by indexing and encoded as the stand-alone quantisers of these widths
// do it: by the reference's search (:397-427), by one read of the map's code table where the
// caller passes one, or by the closed form of the evenly spaced map (the second moment's in every
// shipped configuration; lpmm_search.hpp).  Same tiles and statistics as above; a lane's eight
// codes are two dwords.  21.06 bytes per parameter cross HBM (p 8, g 4 + 4, m codes 2, v codes
// 1 + 2, scales).  LLaMA-7B-shaped set: 24.2 ms per step with 5 bits, 24.4 ms with 8 (the staged
// path 67.6 ms).  Both passes run within 5 % of the rate of their 4-bit counterparts per byte:
// with the arithmetic taken out, with the table instead of the search and with 8-byte instead of
// 4-byte code accesses they take the same time -- the tile structure sets it, not the codes.
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
                                                                    int bits_v, const uint32_t *__restrict__ table_m)
{
    __shared__ float map_m[256], map_v[256];
    __shared__ SearchLds search_m;
    __shared__ BucketLds bucket_m;
    const uint32_t mode = code_table_mode(code_table_tag(table_m), bits_m);
    __shared__ __align__(16) float col_old[kMaxWide * kGroup];
    __shared__ uint32_t colred[kMaxWide * kRedSlotWords];
    __shared__ uint32_t rowred[kRowSlots];
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    fill_map(map_m, qmap_m, bits_m);
    fill_map(map_v, qmap_v, bits_v);
    if (mode == kCodeTable)
        code_table_store(bucket_m, code_table_load(table_m));
    else if (mode == kCodeSearch)
        fill_search(search_m, qmap_m, bits_m);
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads)
        col_old[j] = (j < q.wide * kGroup && tile_c0 + j < cols) ? t.col_old[tile_c0 + j] : 0.0f;
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
    const bool map_even = mode == kCodeEven || (mode == kCodeSearch && map_is_even(search_m));

    if (tl == 0) {
        const int64_t n = t.rows * cols;
        write_padding_bytes(t.mc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                            code1_by_mode(mode, search_m, bucket_m, bits_m, 0.0f));
    }
    const uint32_t mask_m = (1u << bits_m) - 1u, mask_v = (1u << bits_v) - 1u;
    const int slot = drow & (q.wide - 1);
    if (q.cg < t.col_blocks) {
        const float *cop = col_old + slot * kGroup + lane16 * 4;
        uint32_t *red = colred + slot * kRedSlotWords + lane16;
        float co[kEltsPerLane];
        unpack8(*reinterpret_cast<const float4 *>(cop), *reinterpret_cast<const float4 *>(cop + 64), co);
        // the operands of a pass are requested one pass ahead, so that a wave has two passes' loads in
        // flight (LLaMA-7B-shaped set, 8 bits: 24.9-25.1 -> 24.5-24.6 ms per step)
        struct Fetch {
            float4 a0, a1, b0, b1;
            uint32_t wm0, wm1, wv0, wv1;
            float sm, ro;
        };
        auto fetch = [&](int it) {
            Fetch x;
            const int64_t r = q.row0 + it * q.step;
            const int64_t grp = r * t.col_blocks + q.cg;
            const int64_t gbase = grp * kGroup;
            const float *pp = t.p + gbase + lane16 * 4;
            const float *gp = t.g + gbase + lane16 * 4;
            const uint32_t *mcp = reinterpret_cast<const uint32_t *>(t.mc + gbase) + lane16;
            const uint32_t *vcp = reinterpret_cast<const uint32_t *>(t.vc + gbase) + lane16;
            x.a0 = load4(pp);
            x.a1 = load4(pp + 64);
            x.b0 = load4(gp);
            x.b1 = load4(gp + 64);
            x.wm0 = load_u32(mcp);
            x.wm1 = load_u32(mcp + 16);
            x.wv0 = load_u32(vcp);
            x.wv1 = load_u32(vcp + 16);
            x.sm = t.ms[grp];
            x.ro = t.row_old[r];
            return x;
        };
        Fetch nxt;
        if (q.row0 < t.rows)
            nxt = fetch(0);
#pragma unroll 1
        for (int it = 0; it < q.passes; ++it) {
            const int64_t r = q.row0 + it * q.step;
            if (r >= t.rows)
                break;
            const Fetch cur = nxt;
            if (it + 1 < q.passes && r + q.step < t.rows)
                nxt = fetch(it + 1);
            const int64_t grp = r * t.col_blocks + q.cg;
            const int64_t gbase = grp * kGroup;
            float *pp = t.p + gbase + lane16 * 4;
            uint32_t *mcp = reinterpret_cast<uint32_t *>(t.mc + gbase) + lane16;
            const float4 a0 = cur.a0, a1 = cur.a1, b0 = cur.b0, b1 = cur.b1;
            const uint32_t wm0 = cur.wm0, wm1 = cur.wm1, wv0 = cur.wv0, wv1 = cur.wv1;
            const float sm = cur.sm, ro = cur.ro;
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
            codes8_by_mode(mode, search_m, bucket_m, bits_m, map_even, xs, c);
            store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
            store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
            store_u32(mcp, pack4(c, 0));
            store_u32(mcp + 16, pack4(c, 1));
            if (lane16 == 0) {
                t.ms[grp] = amax_m;
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

__global__ __launch_bounds__(kThreads) void rank1_requant_bits_kernel(const MultiR1 args, const float *__restrict__ qmap_v,
                                                                     int bits_v, const uint32_t *__restrict__ table_v)
{
    __shared__ float map_v[256];
    __shared__ SearchLds search_v;
    __shared__ BucketLds bucket_v;
    const uint32_t mode = code_table_mode(code_table_tag(table_v), bits_v);
    __shared__ __align__(16) float col_old[kMaxWide * kGroup], col_new[kMaxWide * kGroup];
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    fill_map(map_v, qmap_v, bits_v);
    if (mode == kCodeTable)
        code_table_store(bucket_v, code_table_load(table_v));
    else if (mode == kCodeSearch)
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
    const bool map_even = mode == kCodeEven || (mode == kCodeSearch && map_is_even(search_v));

    if (tl == 0) {
        const int64_t n = t.rows * cols;
        write_padding_bytes(t.vc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                            code1_by_mode(mode, search_v, bucket_v, bits_v, 0.0f));
    }
    if (q.cg >= t.col_blocks)
        return;
    const uint32_t mask_v = (1u << bits_v) - 1u;
    const int col_off = (drow & (q.wide - 1)) * kGroup + lane16 * 4;
    float co[kEltsPerLane], cn[kEltsPerLane];
    unpack8(*reinterpret_cast<const float4 *>(col_old + col_off), *reinterpret_cast<const float4 *>(col_old + col_off + 64), co);
    unpack8(*reinterpret_cast<const float4 *>(col_new + col_off), *reinterpret_cast<const float4 *>(col_new + col_off + 64), cn);
    // the lane's columns through all passes: the correctly rounded reciprocals of their statistics once
    float rcn[kEltsPerLane];
    bool cols_safe = true;
#pragma unroll
    for (int k = 0; k < kEltsPerLane; ++k) {
        rcn[k] = rcp_exact(cn[k]);
        cols_safe = cols_safe && rc_safe(cn[k]);
    }
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
        float gv[kEltsPerLane], v[kEltsPerLane], x[kEltsPerLane];
        unpack8(b0, b1, gv);
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            v[k] = map_v[byte_of(wv0, wv1, k) & mask_v] * ((co[k] < ro) ? co[k] : ro);
            nonfused_second_moment(v[k], gv[k], h);
        }
        // every scale is a maximum over the values it divides (v <= scale): where all of the wave's
        // scales lie in the range in which the reciprocal is exact, the correctly rounded reciprocal,
        // one multiply and two fmas give the correctly rounded quotient
        if (__all(cols_safe && rc_safe(rn))) {
            const float rcr = rcp_exact(rn);
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const bool by_col = cn[k] < rn;
                x[k] = div_by_rc(v[k], by_col ? cn[k] : rn, by_col ? rcn[k] : rcr);
            }
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                x[k] = v[k] / ((cn[k] < rn) ? cn[k] : rn);
        }
        uint32_t c[kEltsPerLane];
        codes8_by_mode(mode, search_v, bucket_v, bits_v, map_even, x, c);
        store_u32(vcp, pack4(c, 0));
        store_u32(vcp + 16, pack4(c, 1));
    }
}

void launch_rank1_bits(const MultiR1 &args, uint32_t tiles, const float *qmap_m, const float *qmap_v, int bits_m,
                       int bits_v, const uint32_t *table_m, const uint32_t *table_v, hipStream_t stream)
{
    hipLaunchKernelGGL(rank1_update_bits_kernel, dim3(tiles), dim3(kThreads), 0, stream, args, qmap_m, qmap_v, bits_m,
                       bits_v, table_m);
    hipLaunchKernelGGL(rank1_requant_bits_kernel, dim3(tiles), dim3(kThreads), 0, stream, args, qmap_v, bits_v, table_v);
}

}  // namespace lpmm
