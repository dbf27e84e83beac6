// SGD with a 4-bit momentum buffer in one pass over HBM, for a list of tensors per launch.
//
// The reference's step (lpmm/optim/sgd.py:133-187, _single_tensor_sgd4bit) is a chain of PyTorch
// ops per tensor: dequantise the buffer, buf.mul_(momentum).add_(d_p, alpha=1-dampening),
// param.add_(d_p, alpha=-lr), quantise the buffer again -- the buffer crosses HBM four times as
// floats.  Here a tile of 2048 elements is read once (p, g, codes, scales: 13.0625 bytes per
// element with the writes), updated in registers and written back.  The buffer is quantised
// block-wise over 128 values into the packed layout of vectorwise_quant (codes of the
// zero-padded flattened tensor in pack groups of 2048 values plus one byte, functional.py:404-422,
// :359-369), so states interchange with the staged path.
//
// Arithmetic: every Tensor.add(other, alpha=s) of the chain is one fused multiply-add with the
// float-cast scalar and mul_ one multiply, which is what PyTorch's kernels compute; the CPU
// oracle restates the same and is checked against the library ops bit for bit.
//
// Layout: the row layout of the fused AdamW step.  The 16 lanes of a DPP row own one 128-value
// group, lane l the elements [4l, 4l+4) and [64+4l, 64+4l+4) of it, so that every 16-byte access
// covers whole cache lines; the group maximum is 7 max operations in registers and 4 DPP steps.
// A group that is cut by the end of its tensor, or whose pointers are not 16-byte aligned, takes
// guarded element-wise accesses.  Unlike the fused AdamW step this kernel runs best with as many
// workgroups per CU as fit (LLaMA-7B-shaped set: 14.8 ms per step; capped at 6, 5, 4 or 3 per CU
// 15.3, 16.6, 16.6, 20.7 ms), and a straight-line variant for launches of whole tiles gains nothing.
#include "lpmm_update.hpp"

namespace lpmm {

constexpr int kSgdThreads = 256;
constexpr int kSgdElts = 8;
constexpr int kSgdTile = kSgdThreads * kSgdElts;  // 2048 = one pack group
constexpr int kSgdMax = 64;                       // tensors per launch
static_assert(kSgdTile == LPMM_PACK_GROUP, "a tile is a pack group of the non-fused layout");
static_assert((kSgdTile * sizeof(float)) << 4 == kXcdRunBytes, "16 tiles per run");

struct TensorSgd {
    float *p;
    const float *g;
    uint8_t *mc;
    float *ms;
    int64_t n;
    uint32_t first_step;  // the buffer does not exist yet: it becomes the (decayed) gradient
    uint32_t vec;         // p and g allow 16-byte accesses
};

struct MultiSgd {
    TensorSgd t[kSgdMax];
    uint32_t tile_start[kSgdMax + 1];  // prefix sum of tiles per tensor; unused slots hold the total
    float mom, w, wd, neg_lr;          // momentum, 1 - dampening, weight decay, -lr, each cast from double
    uint32_t nesterov, maximize, has_wd;
};

static_assert(sizeof(MultiSgd) + sizeof(void *) <= 4096, "kernel arguments exceed 4 KB");
static_assert(kSgdMax <= kWave, "one tile_start entry per lane");

// One element of the chain (sgd.py:152-181); b is the buffer (in: old value, out: new value),
// returns the new parameter.
__device__ __forceinline__ float sgd_elt(float p, float g, float &b, const MultiSgd &a, bool first)
{
    float d = a.maximize ? -g : g;
    if (a.has_wd)
        d = __builtin_fmaf(a.wd, p, d);
    if (first) {
        b = d;
    } else {
        b = b * a.mom;
        b = __builtin_fmaf(a.w, d, b);
    }
    const float u = a.nesterov ? __builtin_fmaf(a.mom, b, d) : b;
    return __builtin_fmaf(a.neg_lr, u, p);
}

__global__ __launch_bounds__(kSgdThreads) void sgd4bit_kernel(const MultiSgd args, const float *__restrict__ qmap)
{
    __shared__ __align__(16) uint32_t lds[kLdsBytes / 4];
    // tensor of this workgroup (uniform): the number of later tensors whose first tile is not after this one
    const int lane = threadIdx.x & (kWave - 1);
    const bool started = lane + 1 < kSgdMax && args.tile_start[lane + 1] <= blockIdx.x;
    const int lo = __popcll(__ballot(started));
    const TensorSgd &t = args.t[lo];
    // which tile of the tensor: launch order rearranged so that an XCD streams 128 KB runs of the parameters
    const uint32_t tiles_in_tensor = args.tile_start[lo + 1] - args.tile_start[lo];
    const uint32_t tile = xcd_run_order<4>(blockIdx.x - args.tile_start[lo], tiles_in_tensor,
                                           run_phase<4>(t.p, kSgdTile * sizeof(float)));
    const int lane16 = threadIdx.x & 15;
    const int64_t n = t.n;
    const int64_t n_groups = (n + kGroup - 1) / kGroup;
    const int64_t grp = (int64_t)tile * (kSgdTile / kGroup) + (threadIdx.x >> 4);
    const int64_t gbase = grp * kGroup;
    const bool first = t.first_step != 0;
    const bool live = grp < n_groups;                        // else: a group the padding to whole pack groups added
    const bool full = live && t.vec != 0 && gbase + kGroup <= n;  // uniform over the 16 lanes of the group

    float *pp = t.p + gbase + lane16 * 4;
    uint16_t *mcp = reinterpret_cast<uint16_t *>(t.mc + (gbase >> 1)) + lane16;
    // the small loads that feed LDS first (they return first), then the group's streaming loads
    const LdsFill fill = lds_fill_load(qmap, qmap);
    float pv[kSgdElts], gv[kSgdElts];
    uint32_t w0 = 0, w1 = 0;
    float sm = 0.0f;
    if (full) {
        const float *gp = t.g + gbase + lane16 * 4;
        const float4 a0 = load4(pp), a1 = load4(pp + 64), b0 = load4(gp), b1 = load4(gp + 64);
        pv[0] = a0.x; pv[1] = a0.y; pv[2] = a0.z; pv[3] = a0.w;
        pv[4] = a1.x; pv[5] = a1.y; pv[6] = a1.z; pv[7] = a1.w;
        gv[0] = b0.x; gv[1] = b0.y; gv[2] = b0.z; gv[3] = b0.w;
        gv[4] = b1.x; gv[5] = b1.y; gv[6] = b1.z; gv[7] = b1.w;
    } else if (live) {
#pragma unroll
        for (int k = 0; k < kSgdElts; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            pv[k] = i < n ? t.p[i] : 0.0f;
            gv[k] = i < n ? t.g[i] : 0.0f;
        }
    }
    if (live && !first) {
        w0 = load_u16(mcp);  // the code buffer is padded to whole pack groups: always inside
        w1 = load_u16(mcp + 16);
        sm = t.ms[grp];
    }
    lds_fill_store(lds, fill);
    const int kind = classify_map(qmap);
    lds_barrier();

    if (threadIdx.x == 0 && tile + 1 == tiles_in_tensor) {
        // the tensor's last tile also owns the extra byte at the end of the code buffer
        t.mc[(int64_t)tiles_in_tensor * (kSgdTile / 2)] = 0;
    }
    if (!live) {
        // codes of a plain 0.0
        const float z[kSgdElts] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t wz = encode8_plain(lds, kLdsQ0, kind, z);
        store_u16(mcp, wz & 0xFFFFu);
        store_u16(mcp + 16, wz >> 16);
        return;
    }

    const Nibbles nm = split_nibbles(w0 | (w1 << 16));
    float b[kSgdElts];
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kSgdElts; ++k) {
        b[k] = first ? 0.0f : decode_nibble(lds, kLdsQ0, nm, k) * sm;
        pv[k] = sgd_elt(pv[k], gv[k], b[k], args, first);
        // elements past the end of the tensor are the zero padding of the quantiser
        if (!full && gbase + elt_offset(lane16, k) >= n)
            b[k] = 0.0f;
        amax = fmaxf(amax, fabsf(b[k]));
    }
    amax = row16_max(amax);
    const uint32_t om = encode8_scaled(lds, kLdsQ0, kind, b, amax);
    if (full) {
        store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
        store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
    } else {
#pragma unroll
        for (int k = 0; k < kSgdElts; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            if (i < n)
                t.p[i] = pv[k];
        }
    }
    store_u16(mcp, om & 0xFFFFu);
    store_u16(mcp + 16, om >> 16);
    if (lane16 == 0)
        t.ms[grp] = amax;
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_sgd4bit_step_multi(const lpmm_sgd4bit_tensor *tensors, int64_t count, const float *qmap,
                                       double momentum, double dampening, double lr, double weight_decay,
                                       int nesterov, int maximize, void *stream)
{
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(tensors);
    LPMM_REQUIRE_PTR(qmap);
    LPMM_REQUIRE_ALIGN(qmap, 4);
    for (int64_t i = 0; i < count; ++i) {
        const lpmm_sgd4bit_tensor &t = tensors[i];
        if (t.n < 0 || (t.n + kSgdTile - 1) / kSgdTile > 0x7fffffffLL)
            return LPMM_ERR_SIZE;
        if (t.n == 0)
            continue;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(t.m_codes);
        LPMM_REQUIRE_PTR(t.m_max1);
        LPMM_REQUIRE_ALIGN(t.p, 4);
        LPMM_REQUIRE_ALIGN(t.g, 4);
        LPMM_REQUIRE_ALIGN(t.m_codes, 2);
        LPMM_REQUIRE_ALIGN(t.m_max1, 4);
    }
    MultiSgd args;
    args.mom = (float)momentum;
    args.w = (float)(1.0 - dampening);
    args.wd = (float)weight_decay;
    args.neg_lr = (float)(-lr);
    args.nesterov = nesterov != 0;
    args.maximize = maximize != 0;
    args.has_wd = weight_decay != 0.0;
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t tiles = 0;
        args.tile_start[0] = 0;
        while (i < count && k < kSgdMax) {
            const lpmm_sgd4bit_tensor &t = tensors[i];
            if (t.n == 0) {
                ++i;
                continue;
            }
            const uint64_t nt = (uint64_t)((t.n + kSgdTile - 1) / kSgdTile);
            if (tiles + nt > 0x7fffffffULL)
                break;
            TensorSgd &d = args.t[k];
            d.p = t.p;
            d.g = t.g;
            d.mc = t.m_codes;
            d.ms = t.m_max1;
            d.n = t.n;
            d.first_step = t.first_step != 0;
            d.vec = aligned_to(t.p, 16) && aligned_to(t.g, 16);
            tiles += nt;
            args.tile_start[++k] = (uint32_t)tiles;
            ++i;
        }
        if (k == 0)
            continue;
        for (int j = k + 1; j <= kSgdMax; ++j)
            args.tile_start[j] = (uint32_t)tiles;
        hipLaunchKernelGGL(sgd4bit_kernel, dim3((uint32_t)tiles), dim3(kSgdThreads), 0, (hipStream_t)stream, args,
                           qmap);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}
