// AdamW steps on float16 parameters with 4-bit states: the non-fused step as one pass (block-wise second
// moment) and as two passes (rank-1 second moment), and the fused operator's half instantiation (the
// one-pass kernel with that operator's arithmetic and layout, adamw4bit_half_kernel<true>).
//
// With fused=False the reference runs its chain of PyTorch ops in the parameters' type
// (lpmm/optim/adamw.py:367-369, :394-434): every op converts its half operands to float, computes as
// the float kernel does and rounds the result to half once; Python scalars enter as floats.  States,
// scales and statistics are half tensors (lpmm/functional.py:184-203); the normalised values are
// rounded to half by the division and widened to float again by the pack kernel before the search
// (lpmm/cpp_extension/quantization_kernel.cu:450); the unpacked map value (float) times the half scale
// is a float product that takes the state's type last (lpmm/functional.py:97-118, :150).  The kernels
// below do that arithmetic in registers, with a rounding to half wherever an op of the chain ends,
// and move 8.06 bytes per parameter (block-wise second moment: p 2 + 2, g 2, codes 1 + 1, scales
// 4 * 2 / 128) or 7.52 + 3 bytes (rank-1 second moment) instead of the chain's 50.
//
// Layouts, tiles and statistics are those of the float kernels (nonfused_m32.hip, nonfused_rank1_bits.hip).
// The maxima of the new second moment over rows and columns are taken with integer atomics on the
// float images of the half values in a float work array (a maximum of half values is a half value);
// a last small kernel writes them out as halfs.
#include "rank1_tiles.hpp"

namespace lpmm {

typedef _Float16 h16;
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4h load_h4(const h16 *p) { return __builtin_nontemporal_load(reinterpret_cast<const v4h *>(p)); }
__device__ __forceinline__ void store_h4(h16 *p, v4h v) { __builtin_nontemporal_store(v, reinterpret_cast<v4h *>(p)); }

// One rounding to half (nearest even, subnormals kept), as at the end of every op of the chain.  The
// float result is pinned in a register first: otherwise the compiler merges the producing operation
// with the conversion into one mixed-precision instruction (v_fma_mixlo_f16), whose result is rounded
// once, from the exact value, where PyTorch's kernels round the float result a second time -- one
// value in a few thousand then differs in the last place of the half.
__device__ __forceinline__ float rh(float x)
{
    asm("" : "+v"(x));
    return (float)(h16)x;
}

__device__ __forceinline__ void widen8(const v4h &a, const v4h &b, float (&o)[kEltsPerLane])
{
    o[0] = (float)a.x; o[1] = (float)a.y; o[2] = (float)a.z; o[3] = (float)a.w;
    o[4] = (float)b.x; o[5] = (float)b.y; o[6] = (float)b.z; o[7] = (float)b.w;
}

__device__ __forceinline__ v4h narrow4(const float (&x)[kEltsPerLane], int h)
{
    const v4h r = {(h16)x[4 * h], (h16)x[4 * h + 1], (h16)x[4 * h + 2], (h16)x[4 * h + 3]};
    return r;
}

// v.mul_(beta2).addcmul_(g, g, value=1 - beta2) on half tensors
__device__ __forceinline__ void half_second_moment(float &v, float g, const NfHyper &h)
{
    v = rh(v * h.b2);
    v = rh(v + (h.w2 * g) * g);
}

// x / d for a denominator that may be zero: float16 rounds the default eps of 1e-8 to zero, so the
// denominator of an element whose second moment is zero is zero and the parameter becomes infinite or
// NaN, as in the reference.  The quotient of the approximate reciprocal is already the IEEE result then
// (x * inf); elsewhere the residual correction makes it the correctly rounded quotient (div_fast).
__device__ __forceinline__ float div_maybe_zero(float x, float d)
{
    const float rc = __builtin_amdgcn_rcpf(d);
    const float q = x * rc;
    const float r = __builtin_fmaf(-q, d, x);
    const float c = __builtin_fmaf(r, rc, q);
    return d == 0.0f ? q : c;
}

// One element of the chain; p, m and v (halfs held as floats) are updated in place.
__device__ __forceinline__ void half_elt(float &p, float g, float &m, float &v, const NfHyper &h)
{
    const float pi = rh(p * h.decay);
    m = rh(lerp_w(m, g, h.w1));
    half_second_moment(v, g, h);
    float d = rh(sqrt_fast(v));
    d = rh(div_by_rc(d, h.bc2_sqrt, h.rbc2_sqrt));
    d = rh(d + h.eps);
    p = rh(pi + div_maybe_zero(h.neg_step_size * m, d));
}

// Codes of rh(v[k] / scale) for a lane's 8 values; |v[k]| <= scale wherever the scale is finite and
// positive (it is a maximum over the values it divides).
__device__ __forceinline__ uint32_t encode8_scaled_h(const uint32_t *lds, uint32_t lds_map, int kind,
                                                     const float (&v)[kEltsPerLane], float scale)
{
    float x[kEltsPerLane];
    if (kind != kMapGeneric && rc_safe(scale)) {
        // quotients in [-1, 1], no NaN: the closed forms of the standard maps apply as they are
        const float rc = rcp_exact(scale);
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k)
            x[k] = rh(div_by_rc(v[k], scale, rc));
        return kind == kMapStdM ? encode8_std_m(lds, x) : encode8_std_v(x);
    }
#pragma unroll
    for (int k = 0; k < kEltsPerLane; ++k)
        x[k] = rh(v[k] / scale);
    return encode8_plain(lds, lds_map, kind, x);
}

// ---------------------------------------------------------------------------------------
// One pass: both moments block-wise over 128 values.
// ---------------------------------------------------------------------------------------
constexpr int kHTile = kThreads * kEltsPerLane;  // 2048 = one pack group
constexpr int kHMax = 48;                        // tensors per launch
static_assert(kHTile == LPMM_PACK_GROUP, "a tile is a pack group of the non-fused layout");

struct TensorH {
    h16 *p;
    const h16 *g;
    uint8_t *mc, *vc;
    h16 *ms, *vs;
    int64_t n;
    float neg_step_size, bc2_sqrt, rbc2_sqrt;
    uint32_t vec;  // p and g allow 8-byte accesses
};

struct MultiH {
    TensorH t[kHMax];
    uint32_t tile_start[kHMax + 1];
    float decay, w1, b2, w2, eps;
};
static_assert(sizeof(MultiH) + sizeof(Hyper) + 2 * sizeof(void *) <= 4096, "kernel arguments exceed 4 KB");
static_assert(kHMax <= kWave, "one tile_start entry per lane");

// The lane's four code bytes of a group that the end of the tensor cuts, in the layout without padding
// (bytes whose first element lies past the end do not exist): byte j = elements 2 (j & 1) + 64 (j >> 1)
// + 4 lane16 and the one after it.
__device__ __forceinline__ uint32_t load_codes_guarded(const uint8_t *codes, int64_t gbase, int lane16, int64_t n)
{
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t e = gbase + lane16 * 4 + (j & 1) * 2 + (j >> 1) * 64;
        if (e < n)
            w |= (uint32_t)codes[e >> 1] << (8 * j);
    }
    return w;
}

__device__ __forceinline__ void store_codes_guarded(uint8_t *codes, int64_t gbase, int lane16, int64_t n, uint32_t w)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t e = gbase + lane16 * 4 + (j & 1) * 2 + (j >> 1) * 64;
        // an element past the end leaves its nibble 0 (lpmm/cpp_extension/fused_adamw_kernel.cu:148-167)
        const uint32_t byte = (w >> (8 * j)) & (e + 1 < n ? 0xFFu : 0x0Fu);
        if (e < n)
            codes[e >> 1] = (uint8_t)byte;
    }
}

// FUSED: the half instantiation of the reference's fused 4-bit operator
// (lpmm/cpp_extension/fused_adamw_kernel.cu:80-174 with T = at::Half) instead of the chain of PyTorch
// ops: codes and scales without padding, the map entry rounded to half before it meets the scale
// ((T)qmap[idx] * scale, a product of halfs), moments and parameter rounded to half where the kernel
// assigns them to T, everything else in float -- the normalised values included.
template <bool FUSED>
__global__ __launch_bounds__(kThreads) void adamw4bit_half_kernel(const MultiH args, const Hyper fh,
                                                                 const float *__restrict__ qmap_m,
                                                                 const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    const int lane = threadIdx.x & (kWave - 1);
    const bool started = lane + 1 < kHMax && args.tile_start[lane + 1] <= blockIdx.x;
    const int lo = __popcll(__ballot(started));
    const TensorH &t = args.t[lo];
    const uint32_t tiles_in_tensor = args.tile_start[lo + 1] - args.tile_start[lo];
    // 4 KB of parameters per tile: 32 tiles make a 128 KB run of an XCD
    const uint32_t tile = xcd_run_order<5>(blockIdx.x - args.tile_start[lo], tiles_in_tensor,
                                           run_phase<5>(t.p, kHTile * sizeof(h16)));
    const int lane16 = threadIdx.x & 15;
    const int64_t n = t.n;
    const int64_t n_groups = (n + kGroup - 1) / kGroup;
    const int64_t grp = (int64_t)tile * (kHTile / kGroup) + (threadIdx.x >> 4);
    const int64_t gbase = grp * kGroup;
    const bool live = grp < n_groups;  // else: a group the padding to whole pack groups added
    const bool full = live && t.vec != 0 && gbase + kGroup <= n;

    h16 *pp = t.p + gbase + lane16 * 4;
    uint16_t *mcp = reinterpret_cast<uint16_t *>(t.mc + (gbase >> 1)) + lane16;
    uint16_t *vcp = reinterpret_cast<uint16_t *>(t.vc + (gbase >> 1)) + lane16;
    const LdsFill fill = lds_fill_load(qmap_m, qmap_v);
    float pv[kEltsPerLane], gv[kEltsPerLane];
    uint32_t wm = 0, wv = 0;
    float sm = 0.0f, sv = 0.0f;
    if (full) {
        const h16 *gp = t.g + gbase + lane16 * 4;
        const v4h a0 = load_h4(pp), a1 = load_h4(pp + 64), b0 = load_h4(gp), b1 = load_h4(gp + 64);
        widen8(a0, a1, pv);
        widen8(b0, b1, gv);
    } else if (live) {
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            pv[k] = i < n ? (float)t.p[i] : 0.0f;
            gv[k] = i < n ? (float)t.g[i] : 0.0f;
        }
    }
    if (live) {
        if (!FUSED || full) {
            // padded to whole pack groups (the chain's layout), or a whole group: always inside
            wm = load_u16(mcp) | (load_u16(mcp + 16) << 16);
            wv = load_u16(vcp) | (load_u16(vcp + 16) << 16);
        } else {
            wm = load_codes_guarded(t.mc, gbase, lane16, n);
            wv = load_codes_guarded(t.vc, gbase, lane16, n);
        }
        sm = (float)t.ms[grp];
        sv = (float)t.vs[grp];
    }
    lds_fill_store(lds, fill);
    const int kind_m = classify_map(qmap_m), kind_v = classify_map(qmap_v);
    lds_barrier();

    if (!FUSED && threadIdx.x == 0 && tile + 1 == tiles_in_tensor) {
        // the tensor's last tile also owns the extra byte at the end of the code buffers
        t.mc[(int64_t)tiles_in_tensor * (kHTile / 2)] = 0;
        t.vc[(int64_t)tiles_in_tensor * (kHTile / 2)] = 0;
    }
    if (FUSED && !live)
        return;
    if (!live) {
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t zm = encode8_plain(lds, kLdsQ0, kind_m, z), zv = encode8_plain(lds, kLdsQ1, kind_v, z);
        store_u16(mcp, zm & 0xFFFFu);
        store_u16(mcp + 16, zm >> 16);
        store_u16(vcp, zv & 0xFFFFu);
        store_u16(vcp + 16, zv >> 16);
        return;
    }

    NfHyper h;
    h.decay = args.decay;
    h.w1 = args.w1;
    h.b2 = args.b2;
    h.w2 = args.w2;
    h.eps = args.eps;
    h.neg_step_size = t.neg_step_size;
    h.bc2_sqrt = t.bc2_sqrt;
    h.rbc2_sqrt = t.rbc2_sqrt;
    const Nibbles nm = split_nibbles(wm), nv = split_nibbles(wv);
    float m[kEltsPerLane], v[kEltsPerLane];
    float amax_m = 0.0f, amax_v = 0.0f;
#pragma unroll
    for (int k = 0; k < kEltsPerLane; ++k) {
        if (FUSED) {
            m[k] = rh(rh(decode_nibble(lds, kLdsQ0, nm, k)) * sm);
            v[k] = rh(rh(decode_nibble(lds, kLdsQ1, nv, k)) * sv);
            adamw_moments(gv[k], m[k], v[k], fh);
            m[k] = rh(m[k]);
            v[k] = rh(v[k]);
            pv[k] = rh(adamw_param(pv[k], m[k], v[k], fh));
        } else {
            m[k] = rh(decode_nibble(lds, kLdsQ0, nm, k) * sm);
            v[k] = rh(decode_nibble(lds, kLdsQ1, nv, k) * sv);
            half_elt(pv[k], gv[k], m[k], v[k], h);
        }
        // elements past the end of the tensor: the zero padding of the chain's quantiser; threads that
        // the fused operator does not have
        if (!full && gbase + elt_offset(lane16, k) >= n)
            m[k] = v[k] = 0.0f;
        amax_m = fmaxf(amax_m, fabsf(m[k]));
        amax_v = fmaxf(amax_v, fabsf(v[k]));
    }
    row16_max2(amax_m, amax_v);
    // the chain normalises in half (x.div(max1) on half tensors), the fused operator in float
    const uint32_t om = FUSED ? encode8_scaled(lds, kLdsQ0, kind_m, m, amax_m) : encode8_scaled_h(lds, kLdsQ0, kind_m, m, amax_m);
    const uint32_t ov = FUSED ? encode8_scaled(lds, kLdsQ1, kind_v, v, amax_v) : encode8_scaled_h(lds, kLdsQ1, kind_v, v, amax_v);
    if (full) {
        store_h4(pp, narrow4(pv, 0));
        store_h4(pp + 64, narrow4(pv, 1));
    } else {
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            if (i < n)
                t.p[i] = (h16)pv[k];
        }
    }
    if (!FUSED || full) {
        store_u16(mcp, om & 0xFFFFu);
        store_u16(mcp + 16, om >> 16);
        store_u16(vcp, ov & 0xFFFFu);
        store_u16(vcp + 16, ov >> 16);
    } else {
        store_codes_guarded(t.mc, gbase, lane16, n, om);
        store_codes_guarded(t.vc, gbase, lane16, n, ov);
    }
    if (lane16 == 0) {
        t.ms[grp] = (h16)amax_m;
        t.vs[grp] = (h16)amax_v;
    }
}

// ---------------------------------------------------------------------------------------
// Two passes: rank-1 second moment on matrices whose column count is a multiple of 128.  The records
// are MultiR1 with p, g, ms, row_old and col_old pointing at halfs; row_new and col_new are the float
// work arrays.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void rank1_update_half_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                    const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    __shared__ __align__(16) float col_old[kMaxWide * kGroup];
    __shared__ uint32_t colred[kMaxWide * kRedSlotWords];
    __shared__ uint32_t rowred[kRowSlots];
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    h16 *const P = reinterpret_cast<h16 *>(t.p);
    const h16 *const G = reinterpret_cast<const h16 *>(t.g);
    h16 *const MS = reinterpret_cast<h16 *>(t.ms);
    const h16 *const ROW_OLD = reinterpret_cast<const h16 *>(t.row_old);
    const h16 *const COL_OLD = reinterpret_cast<const h16 *>(t.col_old);
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    lds_fill(lds, qmap_m, qmap_v);
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads)
        col_old[j] = (j < q.wide * kGroup && tile_c0 + j < cols) ? (float)COL_OLD[tile_c0 + j] : 0.0f;
    for (int j = threadIdx.x; j < kMaxWide * (int)kRedSlotWords; j += kThreads)
        colred[j] = 0u;
    if (threadIdx.x < kRowSlots)
        rowred[threadIdx.x] = 0u;
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
    __syncthreads();

    if (tl == 0) {
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t n = t.rows * cols;
        write_padding(t.mc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                      encode8_plain(lds, kLdsQ0, kind_m, z));
    }
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
            h16 *pp = P + gbase + lane16 * 4;
            const h16 *gp = G + gbase + lane16 * 4;
            uint16_t *mcp = reinterpret_cast<uint16_t *>(t.mc + (gbase >> 1)) + lane16;
            const uint16_t *vcp = reinterpret_cast<const uint16_t *>(t.vc + (gbase >> 1)) + lane16;
            const v4h a0 = load_h4(pp), a1 = load_h4(pp + 64), b0 = load_h4(gp), b1 = load_h4(gp + 64);
            const uint32_t wm = load_u16(mcp) | (load_u16(mcp + 16) << 16);
            const uint32_t wv = load_u16(vcp) | (load_u16(vcp + 16) << 16);
            const float sm = (float)MS[grp], ro = (float)ROW_OLD[r];
            float pv[kEltsPerLane], gv[kEltsPerLane], m[kEltsPerLane], v[kEltsPerLane];
            widen8(a0, a1, pv);
            widen8(b0, b1, gv);
            const Nibbles nm = split_nibbles(wm), nv = split_nibbles(wv);
            float amax_m = 0.0f, vmax = 0.0f;
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                m[k] = rh(decode_nibble(lds, kLdsQ0, nm, k) * sm);
                v[k] = rh(decode_nibble(lds, kLdsQ1, nv, k) * ((co[k] < ro) ? co[k] : ro));
                half_elt(pv[k], gv[k], m[k], v[k], h);
                amax_m = fmaxf(amax_m, fabsf(m[k]));
                vmax = fmaxf(vmax, v[k]);
                atomicMax(red + k * 16, __float_as_uint(v[k]));
            }
            row16_max2(amax_m, vmax);
            const uint32_t om = encode8_scaled_h(lds, kLdsQ0, kind_m, m, amax_m);
            store_h4(pp, narrow4(pv, 0));
            store_h4(pp + 64, narrow4(pv, 1));
            store_u16(mcp, om & 0xFFFFu);
            store_u16(mcp + 16, om >> 16);
            if (lane16 == 0) {
                MS[grp] = (h16)amax_m;
                atomicMax(rowred + row_slot(t.tile, it, drow), __float_as_uint(vmax));
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

__global__ __launch_bounds__(kThreads) void rank1_requant_half_kernel(const MultiR1 args, const float *__restrict__ qmap_m,
                                                                     const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    __shared__ __align__(16) float col_old[kMaxWide * kGroup], col_new[kMaxWide * kGroup];
    const int lo = find_tensor(args);
    const TensorR1 &t = args.t[lo];
    const h16 *const G = reinterpret_cast<const h16 *>(t.g);
    const h16 *const ROW_OLD = reinterpret_cast<const h16 *>(t.row_old);
    const h16 *const COL_OLD = reinterpret_cast<const h16 *>(t.col_old);
    const uint32_t tl = blockIdx.x - args.tile_start[lo];
    const int lane16 = threadIdx.x & 15, drow = threadIdx.x >> 4;
    const Geometry q = geometry(t, tl, drow);
    const int64_t cols = (int64_t)t.col_blocks * kGroup;
    const int64_t tile_c0 = (int64_t)q.col_tile * q.wide * kGroup;
    lds_fill(lds, qmap_m, qmap_v);
    for (int j = threadIdx.x; j < kMaxWide * kGroup; j += kThreads) {
        const bool in = j < q.wide * kGroup && tile_c0 + j < cols;
        col_old[j] = in ? (float)COL_OLD[tile_c0 + j] : 0.0f;
        col_new[j] = in ? t.col_new[tile_c0 + j] : 0.0f;
    }
    const int kind_v = classify_map(qmap_v);
    NfHyper h;
    h.b2 = args.b2;
    h.w2 = args.w2;
    __syncthreads();

    if (tl == 0) {
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t n = t.rows * cols;
        write_padding(t.vc, n, (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP * LPMM_PACK_GROUP,
                      encode8_plain(lds, kLdsQ1, kind_v, z));
    }
    if (q.cg >= t.col_blocks)
        return;
    const int col_off = (drow & (q.wide - 1)) * kGroup + lane16 * 4;
    float co[kEltsPerLane], cn[kEltsPerLane];
    unpack8(*reinterpret_cast<const float4 *>(col_old + col_off), *reinterpret_cast<const float4 *>(col_old + col_off + 64), co);
    unpack8(*reinterpret_cast<const float4 *>(col_new + col_off), *reinterpret_cast<const float4 *>(col_new + col_off + 64), cn);
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
        const h16 *gp = G + gbase + lane16 * 4;
        const v4h b0 = load_h4(gp), b1 = load_h4(gp + 64);
        uint16_t *vcp = reinterpret_cast<uint16_t *>(t.vc + (gbase >> 1)) + lane16;
        const uint32_t wv = load_u16(vcp) | (load_u16(vcp + 16) << 16);
        const float ro = (float)ROW_OLD[r], rn = t.row_new[r];
        float gv[kEltsPerLane], v[kEltsPerLane], x[kEltsPerLane];
        widen8(b0, b1, gv);
        const Nibbles nv = split_nibbles(wv);
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            v[k] = rh(decode_nibble(lds, kLdsQ1, nv, k) * ((co[k] < ro) ? co[k] : ro));
            half_second_moment(v[k], gv[k], h);
        }
        // every scale is a maximum over the values it divides: where all of the wave's scales lie in the
        // range in which the reciprocal is exact, one multiply and two fmas give the correctly rounded quotient
        uint32_t ov;
        if (__all(cols_safe && rc_safe(rn))) {
            const float rcr = rcp_exact(rn);
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k) {
                const bool by_col = cn[k] < rn;
                x[k] = rh(div_by_rc(v[k], by_col ? cn[k] : rn, by_col ? rcn[k] : rcr));
            }
            // quotients in [0, 1]: the closed form of the standard map applies as it is
            ov = kind_v == kMapStdV ? encode8_std_v(x) : encode8_plain(lds, kLdsQ1, kind_v, x);
        } else {
#pragma unroll
            for (int k = 0; k < kEltsPerLane; ++k)
                x[k] = rh(v[k] / ((cn[k] < rn) ? cn[k] : rn));
            ov = encode8_plain(lds, kLdsQ1, kind_v, x);
        }
        store_u16(vcp, ov & 0xFFFFu);
        store_u16(vcp + 16, ov >> 16);
    }
}

void launch_rank1_half(const MultiR1 &args, uint32_t tiles, const float *qmap_m, const float *qmap_v, hipStream_t stream)
{
    hipLaunchKernelGGL(rank1_update_half_kernel, dim3(tiles), dim3(kThreads), 0, stream, args, qmap_m, qmap_v);
    hipLaunchKernelGGL(rank1_requant_half_kernel, dim3(tiles), dim3(kThreads), 0, stream, args, qmap_m, qmap_v);
}

// The maxima in the float work arrays, written out as the half statistics of the state.
constexpr int kNarrowMax = 64;  // arrays per launch (two per tensor)

struct NarrowArgs {
    const float *src[kNarrowMax];
    h16 *dst[kNarrowMax];
    int64_t n[kNarrowMax];
};
static_assert(sizeof(NarrowArgs) <= 4096, "kernel arguments exceed 4 KB");

__global__ __launch_bounds__(kThreads) void narrow_stats_kernel(const NarrowArgs args)
{
    const float *src = args.src[blockIdx.y];
    h16 *dst = args.dst[blockIdx.y];
    const int64_t n = args.n[blockIdx.y];
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads)
        dst[i] = (h16)src[i];
}

}  // namespace lpmm

using namespace lpmm;

// FUSED: the operator's arithmetic and layout on one tensor (float hyperparameters, as its signature has them)
template <bool FUSED>
static int half_step_multi(const lpmm_adamw4bit_f16_tensor *tensors, int64_t count, const float *qmap_m,
                           const float *qmap_v, double beta1, double beta2, double lr, double weight_decay, double eps,
                           void *stream)
{
    if (FUSED && count != 1)
        return LPMM_ERR_ARG;
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
        const lpmm_adamw4bit_f16_tensor &t = tensors[i];
        if (t.n < 0 || (t.n + kHTile - 1) / kHTile > 0x7fffffffLL)
            return LPMM_ERR_SIZE;
        if (t.n == 0)
            continue;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(t.m_codes);
        LPMM_REQUIRE_PTR(t.m_max1);
        LPMM_REQUIRE_PTR(t.v_codes);
        LPMM_REQUIRE_PTR(t.v_max1);
        LPMM_REQUIRE_ALIGN(t.p, 2);
        LPMM_REQUIRE_ALIGN(t.g, 2);
        LPMM_REQUIRE_ALIGN(t.m_codes, 2);
        LPMM_REQUIRE_ALIGN(t.v_codes, 2);
        LPMM_REQUIRE_ALIGN(t.m_max1, 2);
        LPMM_REQUIRE_ALIGN(t.v_max1, 2);
    }
    const NfHyper c = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, 1.0);
    MultiH args;
    args.decay = c.decay;
    args.w1 = c.w1;
    args.b2 = c.b2;
    args.w2 = c.w2;
    args.eps = c.eps;
    Hyper fh;
    fh.beta1 = (float)beta1;
    fh.beta2 = (float)beta2;
    fh.omb1 = 1 - fh.beta1;  // formed in float, as the operator does
    fh.omb2 = 1 - fh.beta2;
    fh.lr = (float)lr;
    fh.wd = (float)weight_decay;
    fh.eps = (float)eps;
    // bias corrections as the operator computes them per thread, in float
    bias_corrections(fh.beta1, fh.beta2, FUSED ? tensors[0].step : 1.0f, &fh.c1, &fh.c2s);
    fh.rc2s = 1.0f / fh.c2s;
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t tiles = 0;
        args.tile_start[0] = 0;
        while (i < count && k < kHMax) {
            const lpmm_adamw4bit_f16_tensor &t = tensors[i];
            if (t.n == 0) {
                ++i;
                continue;
            }
            const uint64_t nt = (uint64_t)((t.n + kHTile - 1) / kHTile);
            if (tiles + nt > 0x7fffffffULL)
                break;
            TensorH &d = args.t[k];
            d.p = static_cast<h16 *>(t.p);
            d.g = static_cast<const h16 *>(t.g);
            d.mc = t.m_codes;
            d.vc = t.v_codes;
            d.ms = static_cast<h16 *>(t.m_max1);
            d.vs = static_cast<h16 *>(t.v_max1);
            d.n = t.n;
            const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, t.step);
            d.neg_step_size = h.neg_step_size;
            d.bc2_sqrt = h.bc2_sqrt;
            d.rbc2_sqrt = h.rbc2_sqrt;
            d.vec = aligned_to(t.p, 8) && aligned_to(t.g, 8);
            tiles += nt;
            args.tile_start[++k] = (uint32_t)tiles;
            ++i;
        }
        if (k == 0)
            continue;
        for (int j = k + 1; j <= kHMax; ++j)
            args.tile_start[j] = (uint32_t)tiles;
        hipLaunchKernelGGL(adamw4bit_half_kernel<FUSED>, dim3((uint32_t)tiles), dim3(kThreads), 0, (hipStream_t)stream,
                           args, fh, qmap_m, qmap_v);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}

extern "C" int lpmm_nonfused_adamw4bit_f16_step_multi(const lpmm_adamw4bit_f16_tensor *tensors, int64_t count,
                                                      const float *qmap_m, const float *qmap_v, double beta1,
                                                      double beta2, double lr, double weight_decay, double eps,
                                                      void *stream)
{
    return half_step_multi<false>(tensors, count, qmap_m, qmap_v, beta1, beta2, lr, weight_decay, eps, stream);
}

extern "C" int lpmm_adamw4bit_f16_step(void *p, const void *g, uint8_t *m_codes, uint8_t *v_codes, void *m_scale,
                                       void *v_scale, const float *qmap_m, const float *qmap_v, int64_t n, float beta1,
                                       float beta2, float lr, float weight_decay, float eps, float step, void *stream)
{
    lpmm_adamw4bit_f16_tensor t;
    t.p = p;
    t.g = g;
    t.m_codes = m_codes;
    t.v_codes = v_codes;
    t.m_max1 = m_scale;
    t.v_max1 = v_scale;
    t.n = n;
    t.step = step;
    t.reserved = 0.0f;
    return half_step_multi<true>(&t, 1, qmap_m, qmap_v, beta1, beta2, lr, weight_decay, eps, stream);
}

extern "C" int lpmm_nonfused_adamw4bit_rank1_f16_step_multi(const lpmm_nonfused_rank1_f16_tensor *tensors, int64_t count,
                                                            const float *qmap_m, const float *qmap_v, double beta1,
                                                            double beta2, double lr, double weight_decay, double eps,
                                                            void *stream)
{
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(tensors);
    // the float kernels' records, with the work arrays as the next statistics: one launch group at a time
    for (int64_t i = 0; i < count; ++i) {
        const lpmm_nonfused_rank1_f16_tensor &t = tensors[i];
        if (t.rows < 0 || t.cols < 0 || t.cols % kGroup != 0)
            return LPMM_ERR_SIZE;
        if (t.rows == 0 || t.cols == 0)
            continue;
        LPMM_REQUIRE_PTR(t.v_rowmax_next);
        LPMM_REQUIRE_PTR(t.v_colmax_next);
        LPMM_REQUIRE_PTR(t.work);
        LPMM_REQUIRE_ALIGN(t.v_rowmax_next, 2);
        LPMM_REQUIRE_ALIGN(t.v_colmax_next, 2);
        LPMM_REQUIRE_ALIGN(t.work, 16);
        if (t.v_rowmax == t.v_rowmax_next || t.v_colmax == t.v_colmax_next)
            return LPMM_ERR_ARG;
    }
    for (int64_t i0 = 0; i0 < count; i0 += kR1Max) {
        const int k = (int)(count - i0 < kR1Max ? count - i0 : kR1Max);
        lpmm_nonfused_rank1_tensor rec[kR1Max];
        NarrowArgs narrow;
        int arrays = 0;
        int64_t longest = 0;
        for (int j = 0; j < k; ++j) {
            const lpmm_nonfused_rank1_f16_tensor &t = tensors[i0 + j];
            lpmm_nonfused_rank1_tensor &d = rec[j];
            // rows floats, then (from the next multiple of four floats on) cols floats
            float *row_work = t.work, *col_work = t.work == nullptr ? nullptr : t.work + (t.rows + 3) / 4 * 4;
            d.p = static_cast<float *>(t.p);
            d.g = static_cast<const float *>(t.g);
            d.m_codes = t.m_codes;
            d.m_max1 = static_cast<float *>(t.m_max1);
            d.v_codes = t.v_codes;
            d.v_rowmax = static_cast<const float *>(t.v_rowmax);
            d.v_colmax = static_cast<const float *>(t.v_colmax);
            d.v_rowmax_next = row_work;
            d.v_colmax_next = col_work;
            d.rows = t.rows;
            d.cols = t.cols;
            d.step = t.step;
            d.reserved = 0.0f;
            if (t.rows == 0 || t.cols == 0)
                continue;
            narrow.src[arrays] = row_work;
            narrow.dst[arrays] = static_cast<h16 *>(t.v_rowmax_next);
            narrow.n[arrays++] = t.rows;
            narrow.src[arrays] = col_work;
            narrow.dst[arrays] = static_cast<h16 *>(t.v_colmax_next);
            narrow.n[arrays++] = t.cols;
            longest = t.rows > longest ? t.rows : longest;
            longest = t.cols > longest ? t.cols : longest;
        }
        const int st = rank1_step_multi_half(rec, k, qmap_m, qmap_v, beta1, beta2, lr, weight_decay, eps, stream);
        if (st != LPMM_OK)
            return st;
        if (arrays == 0)
            continue;
        int64_t blocks = (longest + kThreads - 1) / kThreads;
        blocks = blocks > 64 ? 64 : blocks;
        hipLaunchKernelGGL(narrow_stats_kernel, dim3((uint32_t)blocks, (uint32_t)arrays), dim3(kThreads), 0,
                           (hipStream_t)stream, narrow);
        const int st2 = launch_status();
        if (st2 != LPMM_OK)
            return st2;
    }
    return LPMM_OK;
}
