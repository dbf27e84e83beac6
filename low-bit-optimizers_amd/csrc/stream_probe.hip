// Streaming-rate calibration kernels for gfx950.  Diagnostic only: no counterpart in the
// reference.  They move bytes the way the fused 4-bit AdamW step moves them (a lane owns the
// 16-byte pieces [4l, 4l+4) and [64+4l, 64+4l+4) of its 128-element group, 16 lanes per group,
// nontemporal accesses, one-shot grid) and do no arithmetic worth the name, so that their rate is
// what the memory system gives to that access pattern: read only, write only, copy, the in-place
// update p += g (two reads per write), and the seven streams of the fused step (p and g read, p
// written, two code arrays and two scale arrays read and written: 9.0625 bytes read and 5.0625
// written per element).  A dynamic LDS allocation the kernels never touch caps the number of
// workgroups resident on a CU.
//
// Workgroup shapes (LPMM_PROBE_SHAPE_*): 256 threads on one 2048-element tile (the fused step's own
// shape), 512 threads on two adjacent tiles, 128 threads on half a tile, and 256 threads that load
// two adjacent tiles before they store either.  With LPMM_PROBE_RUN_ORDER the workgroups take their
// spans of the operands in the order of xcd_run_order (lpmm_common.hpp: every XCD streams 128 KB
// runs of a), otherwise workgroup i takes span i.
#include "lpmm_codec.hpp"

namespace lpmm {

extern __shared__ uint32_t probe_unused_lds[];

struct ProbeArgs {
    float *a;
    const float *b;
    uint8_t *c0, *c1;
    float *s0, *s1;
    uint32_t spans;  // workgroups of the launch
};

struct ProbeLane {
    int64_t elt;   // first element of the lane's first piece
    int64_t code;  // byte offset of its first code half-word
    int64_t grp;   // its group
    bool first;    // lane 0 of its group's 16 lanes
};

// T threads work on a span of T * 8 * TILES elements; `part` selects the T * 8 elements a thread
// handles in its part-th round.
template <int T, int TILES, bool RUN>
__device__ __forceinline__ ProbeLane probe_lane(const ProbeArgs &g, int part)
{
    constexpr uint32_t kSpanBytes = T * 8 * TILES * 4;
    constexpr int kLog2 = kSpanBytes == 4096 ? 5 : (kSpanBytes == 8192 ? 4 : 3);
    static_assert((kSpanBytes << kLog2) == kXcdRunBytes, "span size");
    uint32_t span = blockIdx.x;
    if (RUN)
        span = xcd_run_order<kLog2>(span, g.spans, run_phase<kLog2>(g.a, kSpanBytes));
    ProbeLane l;
    const int64_t first = (int64_t)span * (T * 8 * TILES) + (int64_t)part * (T * 8);
    const uint32_t row = threadIdx.x >> 4, lane16 = threadIdx.x & 15;
    l.elt = first + row * kGroup + lane16 * 4;
    l.code = (first >> 1) + row * (kGroup / 2) + lane16 * 2;
    l.grp = first / kGroup + row;
    l.first = lane16 == 0;
    return l;
}

template <int T, int TILES, bool RUN>
__global__ __launch_bounds__(T) void probe_read_kernel(ProbeArgs g)
{
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        const float4 x = load4(g.a + l.elt), y = load4(g.a + l.elt + 64);
        // never true for finite data; keeps the loads alive
        if (x.x + x.y + x.z + x.w + y.x + y.y + y.z + y.w == 0x1.234568p+100f)
            g.a[l.elt] = 0.0f;
    }
}

template <int T, int TILES, bool RUN>
__global__ __launch_bounds__(T) void probe_write_kernel(ProbeArgs g)
{
    const float4 v = make_float4(1.0f, 1.0f, 1.0f, 1.0f);
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        store4(g.a + l.elt, v);
        store4(g.a + l.elt + 64, v);
    }
}

template <int T, int TILES, bool RUN>
__global__ __launch_bounds__(T) void probe_copy_kernel(ProbeArgs g)
{
    float4 x[TILES], y[TILES];
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        x[part] = load4(g.b + l.elt);
        y[part] = load4(g.b + l.elt + 64);
    }
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        store4(g.a + l.elt, x[part]);
        store4(g.a + l.elt + 64, y[part]);
    }
}

template <int T, int TILES, bool RUN>
__global__ __launch_bounds__(T) void probe_update_kernel(ProbeArgs g)
{
    float4 x[TILES], y[TILES];
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        x[part] = load4(g.a + l.elt);
        y[part] = load4(g.a + l.elt + 64);
        const float4 u = load4(g.b + l.elt), w = load4(g.b + l.elt + 64);
        x[part].x += u.x; x[part].y += u.y; x[part].z += u.z; x[part].w += u.w;
        y[part].x += w.x; y[part].y += w.y; y[part].z += w.z; y[part].w += w.w;
    }
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        store4(g.a + l.elt, x[part]);
        store4(g.a + l.elt + 64, y[part]);
    }
}

// DWORD: one 4-byte code access per lane and state instead of two 2-byte ones (what a kernel that
// trades the halves between neighbouring lanes would issue): 18 instead of 22 vector-memory
// instructions per wave and tile.
template <int T, int TILES, bool RUN, bool DWORD>
__global__ __launch_bounds__(T) void probe_fused_mix_kernel(ProbeArgs g)
{
    float4 x[TILES], y[TILES];
    uint32_t m0[TILES], m1[TILES], v0[TILES], v1[TILES];
    float sm[TILES], sv[TILES];
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        x[part] = load4(g.a + l.elt);
        y[part] = load4(g.a + l.elt + 64);
        const float4 u = load4(g.b + l.elt), w = load4(g.b + l.elt + 64);
        if (DWORD) {
            const int64_t word = l.code + (threadIdx.x & 15) * 2;  // the lane's dword in its group's 64 code bytes
            m0[part] = load_u32(reinterpret_cast<const uint32_t *>(g.c0 + word));
            v0[part] = load_u32(reinterpret_cast<const uint32_t *>(g.c1 + word));
            m1[part] = v1[part] = 0;
        } else {
            const uint16_t *m = reinterpret_cast<const uint16_t *>(g.c0 + l.code);
            const uint16_t *v = reinterpret_cast<const uint16_t *>(g.c1 + l.code);
            m0[part] = load_u16(m); m1[part] = load_u16(m + 16);
            v0[part] = load_u16(v); v1[part] = load_u16(v + 16);
        }
        sm[part] = g.s0[l.grp];
        sv[part] = g.s1[l.grp];
        x[part].x = x[part].x * sm[part] + u.x; x[part].y = x[part].y * sm[part] + u.y;
        x[part].z = x[part].z * sm[part] + u.z; x[part].w = x[part].w * sm[part] + u.w;
        y[part].x = y[part].x * sv[part] + w.x; y[part].y = y[part].y * sv[part] + w.y;
        y[part].z = y[part].z * sv[part] + w.z; y[part].w = y[part].w * sv[part] + w.w;
    }
#pragma unroll
    for (int part = 0; part < TILES; ++part) {
        const ProbeLane l = probe_lane<T, TILES, RUN>(g, part);
        store4(g.a + l.elt, x[part]);
        store4(g.a + l.elt + 64, y[part]);
        if (DWORD) {
            const int64_t word = l.code + (threadIdx.x & 15) * 2;
            store_u32(reinterpret_cast<uint32_t *>(g.c0 + word), m0[part] ^ v0[part]);
            store_u32(reinterpret_cast<uint32_t *>(g.c1 + word), v0[part] + m0[part]);
        } else {
            uint16_t *m = reinterpret_cast<uint16_t *>(g.c0 + l.code), *v = reinterpret_cast<uint16_t *>(g.c1 + l.code);
            store_u16(m, m0[part] ^ v1[part]);
            store_u16(m + 16, m1[part] ^ v0[part]);
            store_u16(v, v0[part] + m0[part]);
            store_u16(v + 16, v1[part] + m1[part]);
        }
        if (l.first) {
            g.s0[l.grp] = sv[part];
            g.s1[l.grp] = sm[part];
        }
    }
}

template <int T, int TILES, bool RUN>
static int probe_launch(int pattern, const ProbeArgs &g, size_t lds, hipStream_t s)
{
    const void *fn = nullptr;
    switch (pattern) {
    case LPMM_PROBE_READ: fn = (const void *)probe_read_kernel<T, TILES, RUN>; break;
    case LPMM_PROBE_WRITE: fn = (const void *)probe_write_kernel<T, TILES, RUN>; break;
    case LPMM_PROBE_COPY: fn = (const void *)probe_copy_kernel<T, TILES, RUN>; break;
    case LPMM_PROBE_UPDATE: fn = (const void *)probe_update_kernel<T, TILES, RUN>; break;
    case LPMM_PROBE_FUSED_MIX: fn = (const void *)probe_fused_mix_kernel<T, TILES, RUN, false>; break;
    case LPMM_PROBE_FUSED_MIX_DWORD: fn = (const void *)probe_fused_mix_kernel<T, TILES, RUN, true>; break;
    default: return LPMM_ERR_ARG;
    }
    if (lds > 64 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return LPMM_ERR_LAUNCH;
    }
    const dim3 grid(g.spans), block(T);
    switch (pattern) {
    case LPMM_PROBE_READ: hipLaunchKernelGGL((probe_read_kernel<T, TILES, RUN>), grid, block, lds, s, g); break;
    case LPMM_PROBE_WRITE: hipLaunchKernelGGL((probe_write_kernel<T, TILES, RUN>), grid, block, lds, s, g); break;
    case LPMM_PROBE_COPY: hipLaunchKernelGGL((probe_copy_kernel<T, TILES, RUN>), grid, block, lds, s, g); break;
    case LPMM_PROBE_UPDATE: hipLaunchKernelGGL((probe_update_kernel<T, TILES, RUN>), grid, block, lds, s, g); break;
    case LPMM_PROBE_FUSED_MIX:
        hipLaunchKernelGGL((probe_fused_mix_kernel<T, TILES, RUN, false>), grid, block, lds, s, g);
        break;
    default: hipLaunchKernelGGL((probe_fused_mix_kernel<T, TILES, RUN, true>), grid, block, lds, s, g); break;
    }
    return launch_status();
}

template <int T, int TILES>
static int probe_shape(int pattern, bool run, ProbeArgs &g, int64_t n, size_t lds, hipStream_t s)
{
    g.spans = (uint32_t)(n / (T * 8 * TILES));
    return run ? probe_launch<T, TILES, true>(pattern, g, lds, s) : probe_launch<T, TILES, false>(pattern, g, lds, s);
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_stream_probe(int kind, float *a, const float *b, uint8_t *codes0, uint8_t *codes1, float *scale0,
                                 float *scale1, int64_t n, int64_t lds_bytes, void *stream)
{
    const int pattern = kind & 0xff, shape = kind & LPMM_PROBE_SHAPE_MASK;
    const bool run = (kind & LPMM_PROBE_RUN_ORDER) != 0;
    if ((kind & ~(0xff | LPMM_PROBE_SHAPE_MASK | LPMM_PROBE_RUN_ORDER)) != 0 || pattern > LPMM_PROBE_FUSED_MIX_DWORD)
        return LPMM_ERR_ARG;
    // 4096 elements: the largest span of the shapes
    if (n <= 0 || n % 4096 != 0 || n / 1024 > 0x7fffffffLL || lds_bytes < 0 || lds_bytes > 160 * 1024)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(a);
    LPMM_REQUIRE_ALIGN(a, 16);
    const bool mix = pattern == LPMM_PROBE_FUSED_MIX || pattern == LPMM_PROBE_FUSED_MIX_DWORD;
    if (pattern == LPMM_PROBE_COPY || pattern == LPMM_PROBE_UPDATE || mix) {
        LPMM_REQUIRE_PTR(b);
        LPMM_REQUIRE_ALIGN(b, 16);
    }
    if (mix) {
        LPMM_REQUIRE_PTR(codes0);
        LPMM_REQUIRE_PTR(codes1);
        LPMM_REQUIRE_PTR(scale0);
        LPMM_REQUIRE_PTR(scale1);
        LPMM_REQUIRE_ALIGN(codes0, 4);
        LPMM_REQUIRE_ALIGN(codes1, 4);
        LPMM_REQUIRE_ALIGN(scale0, 4);
        LPMM_REQUIRE_ALIGN(scale1, 4);
    }
    ProbeArgs g = {a, b, codes0, codes1, scale0, scale1, 0};
    const size_t lds = (size_t)lds_bytes;
    hipStream_t s = (hipStream_t)stream;
    switch (shape) {
    case LPMM_PROBE_SHAPE_256: return probe_shape<256, 1>(pattern, run, g, n, lds, s);
    case LPMM_PROBE_SHAPE_512: return probe_shape<512, 1>(pattern, run, g, n, lds, s);
    case LPMM_PROBE_SHAPE_128: return probe_shape<128, 1>(pattern, run, g, n, lds, s);
    case LPMM_PROBE_SHAPE_256X2: return probe_shape<256, 2>(pattern, run, g, n, lds, s);
    default: return LPMM_ERR_ARG;
    }
}
