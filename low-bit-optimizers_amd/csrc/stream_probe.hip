// Streaming-rate calibration kernels for gfx950.  Diagnostic only: no counterpart in the
// reference.  They move bytes the way the fused 4-bit AdamW step moves them (256-thread
// workgroups, one tile of 2048 elements per workgroup, a lane owns the 16-byte pieces [4l, 4l+4)
// and [64+4l, 64+4l+4) of its 128-element group, nontemporal accesses, one-shot grid) and do no
// arithmetic worth the name, so that their rate is what the memory system gives to that access
// pattern: read only, write only, copy, the in-place update p += g (two reads per write), and
// the seven streams of the fused step (p and g read, p written, two code arrays and two scale
// arrays read and written: 9.0625 bytes read and 5.0625 written per element).  A dynamic LDS
// allocation the kernels never touch caps the number of workgroups resident on a CU.
#include "lpmm_codec.hpp"

namespace lpmm {

constexpr int kProbeThreads = 256;
constexpr int kProbeTile = 2048;

extern __shared__ uint32_t probe_unused_lds[];

struct ProbeLane {
    int64_t elt;   // first element of the lane's first piece
    int64_t code;  // byte offset of its first code half-word
    int64_t grp;   // its group
    bool first;    // lane 0 of its group's 16 lanes
};

__device__ __forceinline__ ProbeLane probe_lane()
{
    ProbeLane l;
    const int64_t tile = (int64_t)blockIdx.x * kProbeTile;
    const uint32_t row = threadIdx.x >> 4, lane16 = threadIdx.x & 15;
    l.elt = tile + row * kGroup + lane16 * 4;
    l.code = (tile >> 1) + row * (kGroup / 2) + lane16 * 2;
    l.grp = tile / kGroup + row;
    l.first = lane16 == 0;
    return l;
}

__global__ __launch_bounds__(kProbeThreads) void probe_read_kernel(float *a)
{
    const ProbeLane l = probe_lane();
    const float4 x = load4(a + l.elt), y = load4(a + l.elt + 64);
    // never true for finite data; keeps the loads alive
    if (x.x + x.y + x.z + x.w + y.x + y.y + y.z + y.w == 0x1.234568p+100f)
        a[l.elt] = 0.0f;
}

__global__ __launch_bounds__(kProbeThreads) void probe_write_kernel(float *a, float value)
{
    const ProbeLane l = probe_lane();
    const float4 v = make_float4(value, value, value, value);
    store4(a + l.elt, v);
    store4(a + l.elt + 64, v);
}

__global__ __launch_bounds__(kProbeThreads) void probe_copy_kernel(float *a, const float *b)
{
    const ProbeLane l = probe_lane();
    const float4 x = load4(b + l.elt), y = load4(b + l.elt + 64);
    store4(a + l.elt, x);
    store4(a + l.elt + 64, y);
}

__global__ __launch_bounds__(kProbeThreads) void probe_update_kernel(float *a, const float *b)
{
    const ProbeLane l = probe_lane();
    float4 x = load4(a + l.elt), y = load4(a + l.elt + 64);
    const float4 u = load4(b + l.elt), w = load4(b + l.elt + 64);
    x.x += u.x; x.y += u.y; x.z += u.z; x.w += u.w;
    y.x += w.x; y.y += w.y; y.z += w.z; y.w += w.w;
    store4(a + l.elt, x);
    store4(a + l.elt + 64, y);
}

__global__ __launch_bounds__(kProbeThreads) void probe_fused_mix_kernel(float *a, const float *b, uint8_t *c0, uint8_t *c1,
                                                                        float *s0, float *s1)
{
    const ProbeLane l = probe_lane();
    float4 x = load4(a + l.elt), y = load4(a + l.elt + 64);
    const float4 u = load4(b + l.elt), w = load4(b + l.elt + 64);
    uint16_t *m = reinterpret_cast<uint16_t *>(c0 + l.code), *v = reinterpret_cast<uint16_t *>(c1 + l.code);
    const uint32_t m0 = load_u16(m), m1 = load_u16(m + 16), v0 = load_u16(v), v1 = load_u16(v + 16);
    const float sm = s0[l.grp], sv = s1[l.grp];
    x.x = x.x * sm + u.x; x.y = x.y * sm + u.y; x.z = x.z * sm + u.z; x.w = x.w * sm + u.w;
    y.x = y.x * sv + w.x; y.y = y.y * sv + w.y; y.z = y.z * sv + w.z; y.w = y.w * sv + w.w;
    store4(a + l.elt, x);
    store4(a + l.elt + 64, y);
    store_u16(m, m0 ^ v1);
    store_u16(m + 16, m1 ^ v0);
    store_u16(v, v0 + m0);
    store_u16(v + 16, v1 + m1);
    if (l.first) {
        s0[l.grp] = sv;
        s1[l.grp] = sm;
    }
}

// The same seven streams with one 4-byte code access per lane and state instead of two 2-byte
// ones (what a kernel that trades the halves between neighbouring lanes would issue): 18 instead
// of 22 vector-memory instructions per wave.
__global__ __launch_bounds__(kProbeThreads) void probe_fused_mix_dword_kernel(float *a, const float *b, uint8_t *c0,
                                                                              uint8_t *c1, float *s0, float *s1)
{
    const ProbeLane l = probe_lane();
    float4 x = load4(a + l.elt), y = load4(a + l.elt + 64);
    const float4 u = load4(b + l.elt), w = load4(b + l.elt + 64);
    const int64_t word = l.code + (threadIdx.x & 15) * 2;  // byte offset of the lane's dword in its group's 64 code bytes
    uint32_t *m = reinterpret_cast<uint32_t *>(c0 + word), *v = reinterpret_cast<uint32_t *>(c1 + word);
    const uint32_t m0 = __builtin_nontemporal_load(m), v0 = __builtin_nontemporal_load(v);
    const float sm = s0[l.grp], sv = s1[l.grp];
    x.x = x.x * sm + u.x; x.y = x.y * sm + u.y; x.z = x.z * sm + u.z; x.w = x.w * sm + u.w;
    y.x = y.x * sv + w.x; y.y = y.y * sv + w.y; y.z = y.z * sv + w.z; y.w = y.w * sv + w.w;
    store4(a + l.elt, x);
    store4(a + l.elt + 64, y);
    __builtin_nontemporal_store(m0 ^ v0, m);
    __builtin_nontemporal_store(v0 + m0, v);
    if (l.first) {
        s0[l.grp] = sv;
        s1[l.grp] = sm;
    }
}

}  // namespace lpmm

using namespace lpmm;

extern "C" int lpmm_stream_probe(int kind, float *a, const float *b, uint8_t *codes0, uint8_t *codes1, float *scale0,
                                 float *scale1, int64_t n, int64_t lds_bytes, void *stream)
{
    if (n <= 0 || n % kProbeTile != 0 || n / kProbeTile > 0x7fffffffLL || lds_bytes < 0 || lds_bytes > 160 * 1024)
        return LPMM_ERR_SIZE;
    LPMM_REQUIRE_PTR(a);
    LPMM_REQUIRE_ALIGN(a, 16);
    const bool mix = kind == LPMM_PROBE_FUSED_MIX || kind == LPMM_PROBE_FUSED_MIX_DWORD;
    if (kind == LPMM_PROBE_COPY || kind == LPMM_PROBE_UPDATE || mix) {
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
    const dim3 grid((uint32_t)(n / kProbeTile)), block(kProbeThreads);
    const size_t lds = (size_t)lds_bytes;
    hipStream_t s = (hipStream_t)stream;
    const void *fn = nullptr;
    switch (kind) {
    case LPMM_PROBE_READ: fn = (const void *)probe_read_kernel; break;
    case LPMM_PROBE_WRITE: fn = (const void *)probe_write_kernel; break;
    case LPMM_PROBE_COPY: fn = (const void *)probe_copy_kernel; break;
    case LPMM_PROBE_UPDATE: fn = (const void *)probe_update_kernel; break;
    case LPMM_PROBE_FUSED_MIX: fn = (const void *)probe_fused_mix_kernel; break;
    case LPMM_PROBE_FUSED_MIX_DWORD: fn = (const void *)probe_fused_mix_dword_kernel; break;
    default: return LPMM_ERR_ARG;
    }
    if (lds > 64 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return LPMM_ERR_LAUNCH;
    }
    switch (kind) {
    case LPMM_PROBE_READ: hipLaunchKernelGGL(probe_read_kernel, grid, block, lds, s, a); break;
    case LPMM_PROBE_WRITE: hipLaunchKernelGGL(probe_write_kernel, grid, block, lds, s, a, 1.0f); break;
    case LPMM_PROBE_COPY: hipLaunchKernelGGL(probe_copy_kernel, grid, block, lds, s, a, b); break;
    case LPMM_PROBE_UPDATE: hipLaunchKernelGGL(probe_update_kernel, grid, block, lds, s, a, b); break;
    case LPMM_PROBE_FUSED_MIX:
        hipLaunchKernelGGL(probe_fused_mix_kernel, grid, block, lds, s, a, b, codes0, codes1, scale0, scale1);
        break;
    default:
        hipLaunchKernelGGL(probe_fused_mix_dword_kernel, grid, block, lds, s, a, b, codes0, codes1, scale0, scale1);
        break;
    }
    return launch_status();
}
