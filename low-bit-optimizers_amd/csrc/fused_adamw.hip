// Fused AdamW steps for gfx950: the 4-bit-state step (decode -> AdamW -> group absmax ->
// re-quantise -> pack, one pass over HBM) and the fp32-state step for small tensors.
//
// Arithmetic follows lpmm/cpp_extension/fused_adamw_kernel.cu:103-172 of the reference
// operation by operation, each operation rounded once (the file is compiled with
// -ffp-contract=off, division and sqrt are the correctly rounded ones).
//
// Work layout of the 4-bit step: 16 lanes (one DPP row) own one 128-element group, a lane
// owns elements [4l, 4l+4) and [64+4l, 64+4l+4) of its group (l = lane within the row), so
// every 16-byte load of a row covers 256 contiguous bytes and the group maxima are 7
// in-register max + 4 DPP steps: no LDS traffic and no atomics for the reduction.  A
// 256-thread workgroup covers a tile of 2048 elements = 16 groups.  LDS holds the two
// 16-entry maps (decode) and the 4 KB first-moment encode table (one entry per bucket byte).
//
// When the maps passed in are the standard ones (dynamic-exponent signed map for m,
// (k+1)/16 for v; checked on the device, no host round trip), the codes are assigned by
// lpmm_encode.hpp and lpmm_codec.hpp (bucket table for m, closed form for v) and the divisions by the group maximum
// use the correctly rounded reciprocal plus one fma correction step; both give the same
// results as the generic search and the plain division, which remain as the fallback for
// any other map.
#include "lpmm_update.hpp"

#include <hip/hip_fp16.h>
#include <math.h>

namespace lpmm {

constexpr int kThreads = 256;
constexpr int kEltsPerLane = 8;
constexpr int kTile = kThreads * kEltsPerLane;  // 2048 elements = 16 groups
// tiles per run of xcd_run_order: 16 tiles x 8 KB of parameters = 128 KB
constexpr int kRunLog2 = 4;
static_assert((kTile * sizeof(float)) << kRunLog2 == kXcdRunBytes, "run length");

// LDS per workgroup.  The tables need kLdsBytes; the allocation is larger on purpose: it caps
// the workgroups resident on a CU (160 KB of LDS).  With the 7 that the registers would allow,
// the waves that are not computing all sit in the memory queues, and the HBM system of MI355X
// sustains less with deeper queues: streaming kernels with this kernel's access pattern and no
// arithmetic peak at 3-5 resident workgroups per CU and lose 8 % at 8.  The kernel itself does
// best with 5 per CU (32 KB; 4 per CU is within 0.3 %, 6 per CU loses 1 %, 3 per CU 20 %: too few
// waves to cover the arithmetic).
#ifndef LPMM_FUSED_LDS_KB_WHOLE
#define LPMM_FUSED_LDS_KB_WHOLE 32
#endif
#ifndef LPMM_FUSED_LDS_KB_RAGGED
#define LPMM_FUSED_LDS_KB_RAGGED 30
#endif
template <bool ALLFULL>
constexpr uint32_t fused_lds_bytes()
{
    return (ALLFULL ? LPMM_FUSED_LDS_KB_WHOLE : LPMM_FUSED_LDS_KB_RAGGED) * 1024u;
}
static_assert(fused_lds_bytes<true>() >= kLdsBytes && fused_lds_bytes<false>() >= kLdsBytes, "tables do not fit");
static_assert(kThreads == kEncEntries, "lds_fill_load / lds_fill_store: one encode-table entry per thread");
// Optional pause (units of 64 cycles) of every wave of the straight-line variant before its first load.
// It paid 0.8 % while consecutive tiles went to different XCDs (6 units); with the tile order below it
// gains nothing and is off.
#ifndef LPMM_FUSED_START_DELAY
#define LPMM_FUSED_START_DELAY 0
#endif
constexpr int kStartDelay = LPMM_FUSED_START_DELAY;

// The parameter update of the 4-bit step uses adamw_param_folded (lpmm_update.hpp); building with
// -DLPMM_FUSED_EXACT_P=1 keeps the reference's operation order with correctly rounded sqrt and divisions
// (bit-identical parameters, 13 more vector instructions per element).
#ifndef LPMM_FUSED_EXACT_P
#define LPMM_FUSED_EXACT_P 0
#endif

struct Tensor4 {
    float *p;
    const float *g;
    uint8_t *mc;
    uint8_t *vc;
    float *ms;
    float *vs;
    int64_t n;
    float k[4];  // per-tensor scalars; which ones, the arithmetic says (FusedArith4, FusedArith, NonFusedArith)
};

constexpr int kStartSlots = LPMM_MULTI_MAX + 8;   // tile_start is read 8 entries at a time
constexpr int kCoarseSlots = LPMM_MULTI_MAX / 8;  // every eighth entry of tile_start

struct Multi4 {
    Tensor4 t[LPMM_MULTI_MAX];
    uint32_t tile_start[kStartSlots];  // prefix sum of tiles per tensor; unused slots hold the total
    uint32_t coarse[kCoarseSlots];     // tile_start[8], tile_start[16], ...
    int count;
    float s[7];  // scalars shared by all tensors, in the order the arithmetic below reads them
};
static_assert(LPMM_MULTI_MAX % 8 == 0, "coarse table");

// The arithmetics the kernels are instantiated with.  They read the shared scalars from
// Multi4::s / MultiF::s and the per-tensor ones from Tensor4::k / TensorF::k.
struct FusedArith {
    // code buffers hold exactly ceil(n/2) bytes; a last odd element leaves its high nibble 0
    static constexpr bool kPadded = false;
    Hyper h;
    template <class M, class T>
    __device__ __forceinline__ FusedArith(const M &a, const T &t)
    {
        h.beta1 = a.s[0];
        h.beta2 = a.s[1];
        h.omb1 = a.s[2];
        h.omb2 = a.s[3];
        h.lr = a.s[4];
        h.wd = a.s[5];
        h.eps = a.s[6];
        h.c1 = t.k[0];   // 1 - beta1^step
        h.c2s = t.k[1];  // sqrt(1 - beta2^step)
        h.rc2s = t.k[2]; // 1 / c2s, correctly rounded (host division)
    }
    __device__ __forceinline__ void elt(float &p, float g, float &m, float &v) const { p = adamw_elt(p, g, m, v, h); }
    // per-tensor scalars of a tensor at step `step`, as the reference computes them per thread
    static void per_tensor(float beta1, float beta2, float eps, float step, float (&k)[4])
    {
        bias_corrections(beta1, beta2, step, &k[0], &k[1]);
        k[2] = 1.0f / k[1];
        k[3] = 0.0f;
    }
};

// The 4-bit step: the moments as FusedArith computes them, the parameter with the folded update.
struct FusedArith4 {
    static constexpr bool kPadded = false;
    Hyper h;
    float fa, fb;
    template <class M, class T>
    __device__ __forceinline__ FusedArith4(const M &a, const T &t)
    {
        h.beta1 = a.s[0];
        h.beta2 = a.s[1];
        h.omb1 = a.s[2];
        h.omb2 = a.s[3];
        h.lr = a.s[4];
        h.wd = a.s[5];
        fa = t.k[0];  // c1 / c2s
        fb = t.k[1];  // eps * c1
    }
    __device__ __forceinline__ void elt(float &p, float g, float &m, float &v) const
    {
        adamw_moments(g, m, v, h);
        p = adamw_param_folded(p, m, v, h.lr, h.wd, fa, fb);
    }
    static void per_tensor(float beta1, float beta2, float eps, float step, float (&k)[4])
    {
        float c1, c2s;
        bias_corrections(beta1, beta2, step, &c1, &c2s);
        k[0] = (float)((double)c1 / (double)c2s);
        k[1] = (float)((double)eps * (double)c1);
        k[2] = k[3] = 0.0f;
    }
};
#if LPMM_FUSED_EXACT_P
using FusedStep4 = FusedArith;
#else
using FusedStep4 = FusedArith4;
#endif

struct NonFusedArith {
    // code buffers are padded to whole tiles plus one byte, as the reference's packing
    // operator lays them out: every nibble of an existing group is written, groups past the
    // tensor hold the code of 0.0
    static constexpr bool kPadded = true;
    NfHyper h;
    template <class M, class T>
    __device__ __forceinline__ NonFusedArith(const M &a, const T &t)
    {
        h.decay = a.s[0];
        h.w1 = a.s[1];
        h.b2 = a.s[2];
        h.w2 = a.s[3];
        h.eps = a.s[4];
        h.neg_step_size = t.k[0];
        h.bc2_sqrt = t.k[1];
        h.rbc2_sqrt = t.k[2];
    }
    __device__ __forceinline__ void elt(float &p, float g, float &m, float &v) const { nonfused_elt(p, g, m, v, h); }
};

static_assert(sizeof(Multi4) + 2 * sizeof(void *) <= 4096, "kernel arguments exceed 4 KB");

// One 128-element group, handled by the 16 lanes of a DPP row.  FULL: the whole group lies
// inside the tensor and the pointers allow vector access; otherwise every access is
// guarded per element.  All 16 lanes take the same instantiation.
// The operands of a lane whose group lies wholly inside the tensor, as loaded from HBM.  The
// loads are issued at the top of the kernel, before the LDS tables are set up, so that their
// latency overlaps the prologue.
struct GroupRegs {
    float4 a0, a1, b0, b1;   // p, g
    uint32_t m0, m1, v0, v1; // code half-words
    float sm, sv;
};

// Where a lane's operands of a whole group live: the tile's base addresses (uniform over the
// workgroup, so they stay in scalar registers) plus 32-bit lane offsets.
struct TileView {
    float *p;
    const float *g;
    uint8_t *mc, *vc;
    float *ms, *vs;
    uint32_t eoff;  // element offset of the lane's first four values in the tile
    uint32_t coff;  // byte offset of its first code half-word
    uint32_t soff;  // its group within the tile
};

__device__ __forceinline__ TileView tile_view(const Tensor4 &t, uint32_t tile_in_tensor)
{
    TileView w;
    const int64_t e0 = (int64_t)tile_in_tensor * kTile;
    w.p = t.p + e0;
    w.g = t.g + e0;
    w.mc = t.mc + (e0 >> 1);
    w.vc = t.vc + (e0 >> 1);
    w.ms = t.ms + e0 / kGroup;
    w.vs = t.vs + e0 / kGroup;
    const uint32_t row = threadIdx.x >> 4, lane16 = threadIdx.x & 15;
    w.eoff = row * kGroup + lane16 * 4;
    w.coff = row * (kGroup / 2) + lane16 * 2;
    w.soff = row;
    return w;
}

__device__ __forceinline__ void group_load(const TileView &w, GroupRegs &r)
{
    const float *pp = w.p + w.eoff;
    const float *gp = w.g + w.eoff;
    r.a0 = load4(pp);
    r.a1 = load4(pp + 64);
    r.b0 = load4(gp);
    r.b1 = load4(gp + 64);
    const uint16_t *mcp = reinterpret_cast<const uint16_t *>(w.mc + w.coff);
    const uint16_t *vcp = reinterpret_cast<const uint16_t *>(w.vc + w.coff);
    r.m0 = load_u16(mcp);
    r.m1 = load_u16(mcp + 16);
    r.v0 = load_u16(vcp);
    r.v1 = load_u16(vcp + 16);
    r.sm = w.ms[w.soff];
    r.sv = w.vs[w.soff];
}

template <bool FULL, class Arith>
__device__ __forceinline__ void group_step(const Tensor4 &t, const TileView &w, const Arith &h, const uint32_t *lds,
                                           bool std_maps, int64_t grp, int lane16, const GroupRegs &r)
{
    const int64_t n = t.n;
    const int64_t gbase = grp * kGroup;
    float pv[kEltsPerLane], gv[kEltsPerLane], m[kEltsPerLane], v[kEltsPerLane];
    uint32_t wm = 0, wv = 0;  // 8 nibbles each: elements 0..3 in the low half-word, 4..7 in the high
    float sm = 0.0f, sv = 0.0f;
    // does the lane store anything: its first element exists, or the buffers are padded
    const bool any = FULL || Arith::kPadded || (gbase + lane16 * 4 < n);

    if (FULL) {
        wm = r.m0 | (r.m1 << 16);
        wv = r.v0 | (r.v1 << 16);
        sm = r.sm;
        sv = r.sv;
        pv[0] = r.a0.x; pv[1] = r.a0.y; pv[2] = r.a0.z; pv[3] = r.a0.w;
        pv[4] = r.a1.x; pv[5] = r.a1.y; pv[6] = r.a1.z; pv[7] = r.a1.w;
        gv[0] = r.b0.x; gv[1] = r.b0.y; gv[2] = r.b0.z; gv[3] = r.b0.w;
        gv[4] = r.b1.x; gv[5] = r.b1.y; gv[6] = r.b1.z; gv[7] = r.b1.w;
    } else if (any) {
        sm = t.ms[grp];
        sv = t.vs[grp];
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            pv[k] = (i < n) ? t.p[i] : 0.0f;
            gv[k] = (i < n) ? t.g[i] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < kEltsPerLane; k += 2) {
            const int64_t i = gbase + elt_offset(lane16, k);
            if (i < n) {
                wm |= (uint32_t)t.mc[i >> 1] << (4 * k);
                wv |= (uint32_t)t.vc[i >> 1] << (4 * k);
            }
        }
    }

    const Nibbles nm = split_nibbles(wm), nv = split_nibbles(wv);
    float amax_m = 0.0f, amax_v = 0.0f;
#pragma unroll
    for (int k = 0; k < kEltsPerLane; ++k) {
        m[k] = decode_nibble(lds, kLdsQ0, nm, k) * sm;
        v[k] = decode_nibble(lds, kLdsQ1, nv, k) * sv;
        if (FULL || (gbase + elt_offset(lane16, k) < n)) {
            h.elt(pv[k], gv[k], m[k], v[k]);
            amax_m = fmaxf(amax_m, fabsf(m[k]));
            amax_v = fmaxf(amax_v, v[k]);
        } else {
            m[k] = 0.0f;
            v[k] = 0.0f;
        }
    }
    // every lane of the row takes part, also those past the end of the tensor
    row16_max2(amax_m, amax_v);
    if (!any)
        return;

    const uint32_t cm = encode8_scaled(lds, kLdsQ0, std_maps ? kMapStdM : kMapGeneric, m, amax_m);
    const uint32_t cv = encode8_scaled(lds, kLdsQ1, std_maps ? kMapStdV : kMapGeneric, v, amax_v);

    if (FULL) {
        float *pp = w.p + w.eoff;
        store4(pp, make_float4(pv[0], pv[1], pv[2], pv[3]));
        store4(pp + 64, make_float4(pv[4], pv[5], pv[6], pv[7]));
        uint16_t *mcp = reinterpret_cast<uint16_t *>(w.mc + w.coff);
        uint16_t *vcp = reinterpret_cast<uint16_t *>(w.vc + w.coff);
        store_u16(mcp, cm & 0xFFFFu);
        store_u16(mcp + 16, cm >> 16);
        store_u16(vcp, cv & 0xFFFFu);
        store_u16(vcp + 16, cv >> 16);
        if (lane16 == 0) {
            w.ms[w.soff] = amax_m;
            w.vs[w.soff] = amax_v;
        }
        return;
    } else {
#pragma unroll
        for (int k = 0; k < kEltsPerLane; ++k) {
            const int64_t i = gbase + elt_offset(lane16, k);
            if (i < n)
                t.p[i] = pv[k];
        }
#pragma unroll
        for (int k = 0; k < kEltsPerLane; k += 2) {
            const int64_t i = gbase + elt_offset(lane16, k);
            if (Arith::kPadded || i < n) {
                // unpadded buffers: a last odd element leaves the high nibble of its byte 0
                const uint32_t keep = (Arith::kPadded || i + 1 < n) ? 0xFFu : 0x0Fu;
                t.mc[i >> 1] = (uint8_t)((cm >> (4 * k)) & keep);
                t.vc[i >> 1] = (uint8_t)((cv >> (4 * k)) & keep);
            }
        }
    }
    if (lane16 == 0) {
        t.ms[grp] = amax_m;
        t.vs[grp] = amax_v;
    }
}

// ALIGNED: every pointer allows vector access.  ALLFULL (implies ALIGNED): every tensor of the
// launch is a whole number of tiles, so no access needs a guard and the loads are straight-line
// code.
template <bool ALIGNED, bool ALLFULL, class Arith>
__global__ __launch_bounds__(kThreads) void adamw4bit_kernel(const Multi4 args,
                                                             const float *__restrict__ qmap_m,
                                                             const float *__restrict__ qmap_v)
{
    __shared__ __align__(16) uint32_t lds[fused_lds_bytes<ALLFULL>() / 4];
    // a short pause before the first load: see kStartDelay
    if (ALLFULL && !Arith::kPadded && kStartDelay > 0)
        __builtin_amdgcn_s_sleep(kStartDelay);
    // the small loads first: maps and encode table for LDS
    const LdsFill fill = lds_fill_load(qmap_m, qmap_v);

    // Which tensor does this tile belong to (uniform over the workgroup): the number of later
    // tensors whose first tile is not after this one; unused slots hold the total, which no
    // block index reaches.  Two rounds of scalar loads from the kernel arguments (every eighth
    // entry, then the seven in between) and scalar compares: nothing here queues behind the
    // streaming traffic of the vector memory path.
    // (start <= bid) as the sign bit of start - 1 - bid (tile counts stay below 2^31): plain
    // scalar arithmetic, no compare masks
    const uint32_t bid = blockIdx.x;
    uint32_t base = 0;
#pragma unroll
    for (int j = 0; j < kCoarseSlots; ++j)
        base += ((args.coarse[j] - 1u - bid) >> 31) * 8u;
    uint32_t lo = base;
#pragma unroll
    for (int i = 1; i < 8; ++i)
        lo += (args.tile_start[base + i] - 1u - bid) >> 31;
    const Tensor4 &t = args.t[lo];
    const int lane16 = threadIdx.x & 15;
    // which tile of the tensor: launch order rearranged so that an XCD streams 128 KB runs of the parameters
    const uint32_t tiles_in_tensor = args.tile_start[lo + 1] - args.tile_start[lo];
    const uint32_t tile_in_tensor = xcd_run_order<kRunLog2>(bid - args.tile_start[lo], tiles_in_tensor,
                                                            run_phase<kRunLog2>(t.p, kTile * sizeof(float)));
    const int64_t grp = (int64_t)tile_in_tensor * (kTile / kGroup) + (threadIdx.x >> 4);
    const TileView view = tile_view(t, tile_in_tensor);

    // a group that lies wholly inside its tensor starts its loads now; the small loads were
    // issued before them and return first
    const bool full = ALLFULL || (ALIGNED && (grp + 1) * kGroup <= t.n);
    GroupRegs regs;
    if (!ALLFULL)
        regs.m0 = regs.m1 = regs.v0 = regs.v1 = 0;
    if (full)
        group_load(view, regs);
    lds_fill_store(lds, fill);
    const bool std_maps = classify_map(qmap_m) == kMapStdM && classify_map(qmap_v) == kMapStdV;
    const Arith h(args, t);
    // the waves wait only for their LDS writes at the barrier (no global access is ordered by it)
    lds_barrier();
    // the loaded words stay as they are until here, so that nothing above waits for them
    asm volatile("" : "+v"(regs.m0), "+v"(regs.m1), "+v"(regs.v0), "+v"(regs.v1));

    if (Arith::kPadded && threadIdx.x == 0 && tile_in_tensor + 1 == tiles_in_tensor) {
        // the tensor's last tile also owns the extra byte at the end of each code buffer
        const int64_t end = (int64_t)tiles_in_tensor * (kTile / 2);
        t.mc[end] = 0;
        t.vc[end] = 0;
    }
    if (!ALLFULL && Arith::kPadded && grp * kGroup >= t.n) {
        // a group the padding to whole tiles added: codes of a plain 0.0
        const float z[kEltsPerLane] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t zm = encode8_plain(lds, kLdsQ0, std_maps ? kMapStdM : kMapGeneric, z);
        const uint32_t zv = encode8_plain(lds, kLdsQ1, std_maps ? kMapStdV : kMapGeneric, z);
        const int64_t b = (grp * kGroup >> 1) + lane16 * 4;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            t.mc[b + k] = (uint8_t)zm;  // all eight codes are the same
            t.vc[b + k] = (uint8_t)zv;
        }
        return;
    }
    if (full)
        group_step<true>(t, view, h, lds, std_maps, grp, lane16, regs);
    else
        group_step<false>(t, view, h, lds, std_maps, grp, lane16, regs);
}

// ---------------------------------------------------------------------------------------
// fp32-state step (lpmm/cpp_extension/fused_adamw_kernel.cu:52-78).
// ---------------------------------------------------------------------------------------
struct TensorF {
    float *p;
    const float *g;
    float *m;
    float *v;
    int64_t n;
    float k[4];  // per-tensor scalars, as in Tensor4
};

constexpr int kMultiFMax = 64;
constexpr int kTileF = 1024;  // 256 threads x 4 elements

struct MultiF {
    TensorF t[kMultiFMax];
    uint32_t tile_start[kMultiFMax + 1];
    int count;
    float s[7];
};

static_assert(sizeof(MultiF) <= 4096, "kernel arguments exceed 4 KB");

// fp32 states, either arithmetic (the FusedArith / NonFusedArith constructors only read the
// scalars, which Multi4 and MultiF name alike)
template <class Arith>
__global__ __launch_bounds__(kThreads) void adamw_fp32_kernel(const MultiF args)
{
    int lo = 0, hi = args.count;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (args.tile_start[mid] <= blockIdx.x)
            lo = mid;
        else
            hi = mid;
    }
    const TensorF &t = args.t[lo];
    const Arith h(args, t);
    const int64_t tile0 = (int64_t)(blockIdx.x - args.tile_start[lo]) * kTileF;
#pragma unroll
    for (int k = 0; k < kTileF / kThreads; ++k) {
        const int64_t i = tile0 + k * kThreads + threadIdx.x;
        if (i < t.n) {
            float p = t.p[i], m = t.m[i], v = t.v[i];
            h.elt(p, t.g[i], m, v);
            t.p[i] = p;
            t.m[i] = m;
            t.v[i] = v;
        }
    }
}

// The fp32-state step on half-precision tensors: p, g, m and v are stored as IEEE half, every
// operation runs in float.  The reference's kernel is instantiated for at::Half by its dispatch
// macro (fused_adamw_kernel.cu:52-78, :188); there every read of a tensor element converts it to
// float and every write rounds the float result to half, so the parameter update sees the moments
// *after* their rounding to half (it reads exp_avg and exp_avg_sq back from memory).
__global__ __launch_bounds__(kThreads) void adamw_fp16_kernel(const MultiF args)
{
    int lo = 0, hi = args.count;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (args.tile_start[mid] <= blockIdx.x)
            lo = mid;
        else
            hi = mid;
    }
    const TensorF &t = args.t[lo];
    const FusedArith a(args, t);
    const Hyper &h = a.h;
    __half *p = reinterpret_cast<__half *>(t.p), *m = reinterpret_cast<__half *>(t.m), *v = reinterpret_cast<__half *>(t.v);
    const __half *g = reinterpret_cast<const __half *>(t.g);
    const int64_t tile0 = (int64_t)(blockIdx.x - args.tile_start[lo]) * kTileF;
#pragma unroll
    for (int k = 0; k < kTileF / kThreads; ++k) {
        const int64_t i = tile0 + k * kThreads + threadIdx.x;
        if (i < t.n) {
            const float gf = __half2float(g[i]), pf = __half2float(p[i]);
            const __half mh = __float2half_rn(h.beta1 * __half2float(m[i]) + h.omb1 * gf);
            const __half vh = __float2half_rn(h.beta2 * __half2float(v[i]) + h.omb2 * gf * gf);
            m[i] = mh;
            v[i] = vh;
            const float denom = (div_by_rc(sqrt_fast(__half2float(vh)), h.c2s, h.rc2s) + h.eps) * h.c1;
            const float update = div_fast(__half2float(mh), denom) + (h.wd * pf);
            p[i] = __float2half_rn(pf - (h.lr * update));
        }
    }
}

}  // namespace lpmm

using namespace lpmm;

// Validation, batching into launches of at most LPMM_MULTI_MAX tensors, and launch, shared
// by the arithmetics.  per_tensor(step, k) fills the per-tensor scalars.
template <class Arith, class PerTensor>
static int step_multi4(const lpmm_adamw4bit_tensor *tensors, int64_t count, const float *qmap_m,
                       const float *qmap_v, const float (&scalars)[7], PerTensor per_tensor, void *stream)
{
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
        const lpmm_adamw4bit_tensor &t = tensors[i];
        if (t.n < 0)
            return LPMM_ERR_SIZE;
        if (t.n == 0)
            continue;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(t.m_codes);
        LPMM_REQUIRE_PTR(t.v_codes);
        LPMM_REQUIRE_PTR(t.m_scale);
        LPMM_REQUIRE_PTR(t.v_scale);
        LPMM_REQUIRE_ALIGN(t.p, 4);
        LPMM_REQUIRE_ALIGN(t.g, 4);
        LPMM_REQUIRE_ALIGN(t.m_scale, 4);
        LPMM_REQUIRE_ALIGN(t.v_scale, 4);
        if ((t.n + kTile - 1) / kTile > 0x7fffffffLL)
            return LPMM_ERR_SIZE;
    }

    Multi4 args;
    for (int j = 0; j < 7; ++j)
        args.s[j] = scalars[j];
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t tiles = 0;
        // per launch: do all pointers allow vector access, is every tensor a whole number of tiles
        bool aligned = true, allfull = true;
        args.tile_start[0] = 0;
        while (i < count && k < LPMM_MULTI_MAX) {
            const lpmm_adamw4bit_tensor &t = tensors[i];
            if (t.n == 0) {
                ++i;
                continue;
            }
            const uint64_t nt = (uint64_t)((t.n + kTile - 1) / kTile);
            if (tiles + nt > 0x7fffffffULL)
                break;
            allfull = allfull && (t.n % kTile) == 0;
            aligned = aligned && aligned_to(t.p, 16) && aligned_to(t.g, 16) && aligned_to(t.m_codes, 2) &&
                      aligned_to(t.v_codes, 2);
            Tensor4 &d = args.t[k];
            d.p = t.p;
            d.g = t.g;
            d.mc = t.m_codes;
            d.vc = t.v_codes;
            d.ms = t.m_scale;
            d.vs = t.v_scale;
            d.n = t.n;
            per_tensor(t.step, d.k);
            tiles += nt;
            args.tile_start[++k] = (uint32_t)tiles;
            ++i;
        }
        if (k == 0)
            continue;
        args.count = k;
        for (int j = k + 1; j < kStartSlots; ++j)
            args.tile_start[j] = (uint32_t)tiles;
        for (int j = 0; j < kCoarseSlots; ++j)
            args.coarse[j] = args.tile_start[8 * (j + 1)];
        const dim3 grid((uint32_t)tiles), block(kThreads);
        if (aligned && allfull)
            hipLaunchKernelGGL((adamw4bit_kernel<true, true, Arith>), grid, block, 0, (hipStream_t)stream, args,
                               qmap_m, qmap_v);
        else if (aligned)
            hipLaunchKernelGGL((adamw4bit_kernel<true, false, Arith>), grid, block, 0, (hipStream_t)stream, args,
                               qmap_m, qmap_v);
        else
            hipLaunchKernelGGL((adamw4bit_kernel<false, false, Arith>), grid, block, 0, (hipStream_t)stream, args,
                               qmap_m, qmap_v);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}

extern "C" int lpmm_adamw4bit_step_multi(const lpmm_adamw4bit_tensor *tensors, int64_t count,
                                         const float *qmap_m, const float *qmap_v, float beta1,
                                         float beta2, float lr, float weight_decay, float eps,
                                         void *stream)
{
    // 1 - beta is formed in float, as the reference kernel does
    const float scalars[7] = {beta1, beta2, 1 - beta1, 1 - beta2, lr, weight_decay, eps};
    return step_multi4<FusedStep4>(tensors, count, qmap_m, qmap_v, scalars,
                                   [=](float step, float (&k)[4]) { FusedStep4::per_tensor(beta1, beta2, eps, step, k); },
                                   stream);
}

extern "C" int lpmm_nonfused_adamw4bit_step_multi(const lpmm_adamw4bit_tensor *tensors, int64_t count,
                                                  const float *qmap_m, const float *qmap_v, double beta1,
                                                  double beta2, double lr, double weight_decay,
                                                  double eps, void *stream)
{
    const NfHyper c = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, 1.0);
    const float scalars[7] = {c.decay, c.w1, c.b2, c.w2, c.eps, 0.0f, 0.0f};
    return step_multi4<NonFusedArith>(tensors, count, qmap_m, qmap_v, scalars,
                                      [=](float step, float (&k)[4]) {
                                          const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step);
                                          k[0] = h.neg_step_size;
                                          k[1] = h.bc2_sqrt;
                                          k[2] = h.rbc2_sqrt;
                                          k[3] = 0.0f;
                                      },
                                      stream);
}

extern "C" int lpmm_adamw4bit_step(float *p, const float *g, uint8_t *m_codes, uint8_t *v_codes,
                                   float *m_scale, float *v_scale, const float *qmap_m,
                                   const float *qmap_v, int64_t n, float beta1, float beta2, float lr,
                                   float weight_decay, float eps, float step, void *stream)
{
    lpmm_adamw4bit_tensor t;
    t.p = p;
    t.g = g;
    t.m_codes = m_codes;
    t.v_codes = v_codes;
    t.m_scale = m_scale;
    t.v_scale = v_scale;
    t.n = n;
    t.step = step;
    t.reserved = 0.0f;
    return lpmm_adamw4bit_step_multi(&t, 1, qmap_m, qmap_v, beta1, beta2, lr, weight_decay, eps, stream);
}

template <class Arith, bool HALF = false, class PerTensor>
static int step_multi_fp32(const lpmm_adamw_fp32_tensor *tensors, int64_t count, const float (&scalars)[7],
                           PerTensor per_tensor, void *stream)
{
    constexpr uintptr_t kEltAlign = HALF ? 2 : 4;
    if (count < 0)
        return LPMM_ERR_SIZE;
    if (count == 0)
        return LPMM_OK;
    LPMM_REQUIRE_PTR(tensors);
    for (int64_t i = 0; i < count; ++i) {
        const lpmm_adamw_fp32_tensor &t = tensors[i];
        if (t.n < 0 || (t.n + kTileF - 1) / kTileF > 0x7fffffffLL)
            return LPMM_ERR_SIZE;
        if (t.n == 0)
            continue;
        LPMM_REQUIRE_PTR(t.p);
        LPMM_REQUIRE_PTR(t.g);
        LPMM_REQUIRE_PTR(t.m);
        LPMM_REQUIRE_PTR(t.v);
        LPMM_REQUIRE_ALIGN(t.p, kEltAlign);
        LPMM_REQUIRE_ALIGN(t.g, kEltAlign);
        LPMM_REQUIRE_ALIGN(t.m, kEltAlign);
        LPMM_REQUIRE_ALIGN(t.v, kEltAlign);
    }
    MultiF args;
    for (int j = 0; j < 7; ++j)
        args.s[j] = scalars[j];
    int64_t i = 0;
    while (i < count) {
        int k = 0;
        uint64_t tiles = 0;
        args.tile_start[0] = 0;
        while (i < count && k < kMultiFMax) {
            const lpmm_adamw_fp32_tensor &t = tensors[i];
            if (t.n == 0) {
                ++i;
                continue;
            }
            const uint64_t nt = (uint64_t)((t.n + kTileF - 1) / kTileF);
            if (tiles + nt > 0x7fffffffULL)
                break;
            TensorF &d = args.t[k];
            d.p = t.p;
            d.g = t.g;
            d.m = t.m;
            d.v = t.v;
            d.n = t.n;
            per_tensor(t.step, d.k);
            tiles += nt;
            args.tile_start[++k] = (uint32_t)tiles;
            ++i;
        }
        if (k == 0)
            continue;
        args.count = k;
        for (int j = k + 1; j <= kMultiFMax; ++j)
            args.tile_start[j] = (uint32_t)tiles;
        if (HALF)
            hipLaunchKernelGGL(adamw_fp16_kernel, dim3((uint32_t)tiles), dim3(kThreads), 0, (hipStream_t)stream, args);
        else
            hipLaunchKernelGGL(adamw_fp32_kernel<Arith>, dim3((uint32_t)tiles), dim3(kThreads), 0,
                               (hipStream_t)stream, args);
        const int st = launch_status();
        if (st != LPMM_OK)
            return st;
    }
    return LPMM_OK;
}

extern "C" int lpmm_adamw_fp32_step_multi(const lpmm_adamw_fp32_tensor *tensors, int64_t count,
                                          float beta1, float beta2, float lr, float weight_decay,
                                          float eps, void *stream)
{
    const float scalars[7] = {beta1, beta2, 1 - beta1, 1 - beta2, lr, weight_decay, eps};
    return step_multi_fp32<FusedArith>(tensors, count, scalars,
                                       [=](float step, float (&k)[4]) { FusedArith::per_tensor(beta1, beta2, eps, step, k); },
                                       stream);
}

extern "C" int lpmm_adamw_fp16_step_multi(const lpmm_adamw_fp32_tensor *tensors, int64_t count, float beta1,
                                          float beta2, float lr, float weight_decay, float eps, void *stream)
{
    const float scalars[7] = {beta1, beta2, 1 - beta1, 1 - beta2, lr, weight_decay, eps};
    return step_multi_fp32<FusedArith, true>(tensors, count, scalars,
                                             [=](float step, float (&k)[4]) { FusedArith::per_tensor(beta1, beta2, eps, step, k); },
                                             stream);
}

extern "C" int lpmm_nonfused_update_multi(const lpmm_adamw_fp32_tensor *tensors, int64_t count, double beta1,
                                          double beta2, double lr, double weight_decay, double eps,
                                          void *stream)
{
    const NfHyper c = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, 1.0);
    const float scalars[7] = {c.decay, c.w1, c.b2, c.w2, c.eps, 0.0f, 0.0f};
    return step_multi_fp32<NonFusedArith>(tensors, count, scalars,
                                          [=](float step, float (&k)[4]) {
                                              const NfHyper h = make_nf_hyper(beta1, beta2, lr, weight_decay, eps, step);
                                              k[0] = h.neg_step_size;
                                              k[1] = h.bc2_sqrt;
                                              k[2] = h.rbc2_sqrt;
                                              k[3] = 0.0f;
                                          },
                                          stream);
}

extern "C" int lpmm_adamw_fp32_step(float *p, const float *g, float *m, float *v, int64_t n,
                                    float beta1, float beta2, float lr, float weight_decay, float eps,
                                    float step, void *stream)
{
    lpmm_adamw_fp32_tensor t;
    t.p = p;
    t.g = g;
    t.m = m;
    t.v = v;
    t.n = n;
    t.step = step;
    t.reserved = 0.0f;
    return lpmm_adamw_fp32_step_multi(&t, 1, beta1, beta2, lr, weight_decay, eps, stream);
}
