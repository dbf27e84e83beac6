// Non-fused AdamW step with an fp32 first moment and a 4-bit second moment ('group' scaling over
// 128 values) in one pass over HBM, for a list of tensors per launch.
//
// This is the reference's _single_tensor_adamw4bit (lpmm/optim/adamw.py:332-436) under a
// configuration that quantises the second moment only (QUANT.M.ENABLE False,
// lpmm/configs/2nd_moment_only_group_128.yml): exp_avg is the state tensor itself and is updated
// in place (:397-399, :412), exp_avg_sq is dequantised, updated and quantised again (:402-409,
// :430-434).  As a chain of PyTorch ops the second moment crosses HBM three times as floats; here
// a tile of 2048 elements is read once (p, g, m, codes, scales: 21.0625 bytes per element with the
// writes), updated in registers and written back.  The codes keep the packed layout of
// vectorwise_quant (codes of the zero-padded flattened tensor in pack groups of 2048 values plus
// one byte, lpmm/functional.py:404-422, :359-369), so states interchange with the staged path.
//
// Layout: the 16 lanes of a DPP row own one 128-value group, lane l the elements [4l, 4l+4) and
// [64+4l, 64+4l+4) of it, so that every 16-byte access covers whole cache lines.  A group that is
// cut by the end of its tensor, or whose pointers are not 16-byte aligned, takes guarded
// element-wise accesses.  97 registers: 4 workgroups per CU.  LLaMA-7B-shaped set: 23-24 ms per
// step (the staged path 40 ms); bounded to 102 registers (5 per CU) the same, to 85 or fewer the
// compiler spills (35 ms and worse).
#include "lpmm_update.hpp"

namespace lpmm {

constexpr int kV4Threads = 256;
constexpr int kV4Elts = 8;
constexpr int kV4Tile = kV4Threads * kV4Elts;  // 2048 = one pack group
constexpr int kV4Max = 48;                     // tensors per launch
static_assert(kV4Tile == LPMM_PACK_GROUP, "a tile is a pack group of the non-fused layout");
static_assert((kV4Tile * sizeof(float)) << 4 == kXcdRunBytes, "16 tiles per run");

struct TensorV4 {
    float *p;
    const float *g;
    float *m;
    uint8_t *vc;
    float *vs;
    int64_t n;
    float neg_step_size, bc2_sqrt, rbc2_sqrt;
    uint32_t vec;  // p, g and m allow 16-byte accesses
};

struct MultiV4 {
    TensorV4 t[kV4Max];
    uint32_t tile_start[kV4Max + 1];  // prefix sum of tiles per tensor; unused slots hold the total
    float decay, w1, b2, w2, eps;
};

static_assert(sizeof(MultiV4) + sizeof(void *) <= 4096, "kernel arguments exceed 4 KB");
static_assert(kV4Max <= kWave, "one tile_start entry per lane");

__device__ __forceinline__ void unpack8(const float4 &a, const float4 &b, float (&o)[kV4Elts])
{
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}

__global__ __launch_bounds__(kV4Threads) void adamw_v4bit_kernel(const MultiV4 args, const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    // tensor of this workgroup (uniform): the number of later tensors whose first tile is not after this one
    const int lane = threadIdx.x & (kWave - 1);
    const bool started = lane + 1 < kV4Max && args.tile_start[lane + 1] <= blockIdx.x;
    const int lo = __popcll(__ballot(started));
    const TensorV4 &t = args.t[lo];
    // which tile of the tensor: launch order rearranged so that an XCD streams 128 KB runs of the parameters
    const uint32_t tiles_in_tensor = args.tile_start[lo + 1] - args.tile_start[lo];
    const uint32_t tile = xcd_run_order<4>(blockIdx.x - args.tile_start[lo], tiles_in_tensor,
                                           run_phase<4>(t.p, kV4Tile * sizeof(float)));
    const int lane16 = threadIdx.x & 15;
    const int64_t n = t.n;
    const int64_t n_groups = (n + kGroup - 1) / kGroup;
    const int64_t grp = (int64_t)tile * (kV4Tile / kGroup) + (threadIdx.x >> 4);
    const int64_t gbase = grp * kGroup;
    const bool live = grp < n_groups;                             // else: a group the padding to whole pack groups added
    const bool full = live && t.vec != 0 && gbase + kGroup <= n;  // uniform over the 16 lanes of the group

    float *pp = t.p + gbase + lane16 * 4;
    float *mp = t.m + gbase + lane16 * 4;
    uint16_t *vcp = reinterpret_cast<uint16_t *>(t.vc + (gbase >> 1)) + lane16;
    // the small loads that feed LDS first (they return first), then the group's streaming loads
    const LdsFill fill = lds_fill_load(qmap_v, qmap_v);
    float pv[kV4Elts], gv[kV4Elts], m[kV4Elts];
    uint32_t w0 = 0, w1 = 0;
    float sv = 0.0f;
    if (full) {
        const float *gp = t.g + gbase + lane16 * 4;
        const float4 a0 = load4(pp), a1 = load4(pp + 64), b0 = load4(gp), b1 = load4(gp + 64);
        const float4 c0 = load4(mp), c1 = load4(mp + 64);
        unpack8(a0, a1, pv);
        unpack8(b0, b1, gv);
        unpack8(c0, c1, m);
    } else if (live) {
#pragma unroll
        for (int k = 0; k < kV4Elts; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            pv[k] = i < n ? t.p[i] : 0.0f;
            gv[k] = i < n ? t.g[i] : 0.0f;
            m[k] = i < n ? t.m[i] : 0.0f;
        }
    }
    if (live) {
        w0 = load_u16(vcp);  // the code buffer is padded to whole pack groups: always inside
        w1 = load_u16(vcp + 16);
        sv = t.vs[grp];
    }
    lds_fill_store(lds, fill);
    const int kind = classify_map(qmap_v);
    lds_barrier();

    if (threadIdx.x == 0 && tile + 1 == tiles_in_tensor) {
        // the tensor's last tile also owns the extra byte at the end of the code buffer
        t.vc[(int64_t)tiles_in_tensor * (kV4Tile / 2)] = 0;
    }
    if (!live) {
        // codes of a plain 0.0
        const float z[kV4Elts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t wz = encode8_plain(lds, kLdsQ0, kind, z);
        store_u16(vcp, wz & 0xFFFFu);
        store_u16(vcp + 16, wz >> 16);
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
    const Nibbles nv = split_nibbles(w0 | (w1 << 16));
    float v[kV4Elts];
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kV4Elts; ++k) {
        v[k] = decode_nibble(lds, kLdsQ0, nv, k) * sv;
        nonfused_elt(pv[k], gv[k], m[k], v[k], h);
        // elements past the end of the tensor are the zero padding of the quantiser
        if (!full && gbase + elt_offset(lane16, k) >= n)
            v[k] = 0.0f;
        amax = fmaxf(amax, fabsf(v[k]));
    }
    amax = row16_max(amax);
    const uint32_t ov = encode8_scaled(lds, kLdsQ0, kind, v, amax);
    if (full) {
        store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
        store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
        store4(mp, make_float4(m[0], m[1], m[2], m[3]));
        store4(mp + 64, make_float4(m[4], m[5], m[6], m[7]));
    } else {
#pragma unroll
        for (int k = 0; k < kV4Elts; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            if (i < n) {
                t.p[i] = pv[k];
                t.m[i] = m[k];
            }
        }
    }
    store_u16(vcp, ov & 0xFFFFu);
    store_u16(vcp + 16, ov >> 16);
    if (lane16 == 0)
        t.vs[grp] = amax;
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_nonfused_adamw_v4bit_step_multi(const lpmm_adamw_v4bit_tensor *tensors, int64_t count,
                                                    const float *qmap_v, double beta1, double beta2, double lr,
                                                    double weight_decay, double eps, void *stream)
{
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(tensors);
    LPMM_REQUIRE_PTR(qmap_v);
    LPMM_REQUIRE_ALIGN(qmap_v, 4);
    for (int64_t i = 0; i < count; ++i) {
        const lpmm_adamw_v4bit_tensor &t = tensors[i];
        if (t.n < 0 || (t.n + kV4Tile - 1) / kV4Tile > 0x7fffffffLL)
            return LPMM_ERR_SIZE;
        if (t.n == 0)
            continue;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(t.m);
        LPMM_REQUIRE_PTR(t.v_codes);
        LPMM_REQUIRE_PTR(t.v_max1);
        LPMM_REQUIRE_ALIGN(t.p, 4);
        LPMM_REQUIRE_ALIGN(t.g, 4);
        LPMM_REQUIRE_ALIGN(t.m, 4);
        LPMM_REQUIRE_ALIGN(t.v_codes, 2);
        LPMM_REQUIRE_ALIGN(t.v_max1, 4);
    }
    const NfHyper c = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, 1.0);
    MultiV4 args;
    args.decay = c.decay;
    args.w1 = c.w1;
    args.b2 = c.b2;
    args.w2 = c.w2;
    args.eps = c.eps;
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t tiles = 0;
        args.tile_start[0] = 0;
        while (i < count && k < kV4Max) {
            const lpmm_adamw_v4bit_tensor &t = tensors[i];
            if (t.n == 0) {
                ++i;
                continue;
            }
            const uint64_t nt = (uint64_t)((t.n + kV4Tile - 1) / kV4Tile);
            if (tiles + nt > 0x7fffffffULL)
                break;
            TensorV4 &d = args.t[k];
            d.p = t.p;
            d.g = t.g;
            d.m = t.m;
            d.vc = t.v_codes;
            d.vs = t.v_max1;
            d.n = t.n;
            const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, t.step);
            d.neg_step_size = h.neg_step_size;
            d.bc2_sqrt = h.bc2_sqrt;
            d.rbc2_sqrt = h.rbc2_sqrt;
            d.vec = aligned_to(t.p, 16) && aligned_to(t.g, 16) && aligned_to(t.m, 16);
            tiles += nt;
            args.tile_start[++k] = (uint32_t)tiles;
            ++i;
        }
        if (k == 0)
            continue;
        for (int j = k + 1; j <= kV4Max; ++j)
            args.tile_start[j] = (uint32_t)tiles;
        hipLaunchKernelGGL(adamw_v4bit_kernel, dim3((uint32_t)tiles), dim3(kV4Threads), 0, (hipStream_t)stream, args,
                           qmap_v);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}
