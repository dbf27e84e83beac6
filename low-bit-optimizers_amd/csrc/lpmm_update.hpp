// Elementwise AdamW arithmetic of the two host paths of the reference, shared by the kernels.
#pragma once

#include "lpmm_codec.hpp"

#include <math.h>

namespace lpmm {

// ---------------------------------------------------------------------------------------
// Fused path (lpmm/cpp_extension/fused_adamw_kernel.cu:119-128): float scalars, bias
// corrections c1 = 1 - beta1^step, c2s = sqrt(1 - beta2^step).
// ---------------------------------------------------------------------------------------
struct Hyper {
    float beta1, beta2, omb1, omb2, lr, wd, eps, c1, c2s, rc2s;  // omb = 1 - beta; rc2s = 1 / c2s (host division)
};

#ifndef LPMM_P_MODE
#define LPMM_P_MODE 1  // 0: IEEE sqrt/div, 1: approximation + residual correction, 2: approximation only
#endif

// The two moments of one element, operation by operation as the reference writes them.
__device__ __forceinline__ void adamw_moments(float g, float &m, float &v, const Hyper &h)
{
    m = h.beta1 * m + h.omb1 * g;
    v = h.beta2 * v + h.omb2 * g * g;
}

// The parameter of one element from the updated moments, in the reference's operation order.
__device__ __forceinline__ float adamw_param(float p, float m, float v, const Hyper &h)
{
#if LPMM_P_MODE == 0
    const float denom = (sqrtf(v) / h.c2s + h.eps) * h.c1;
    const float update = (m / denom) + (h.wd * p);
#elif LPMM_P_MODE == 1
    const float denom = (div_by_rc(sqrt_fast(v), h.c2s, h.rc2s) + h.eps) * h.c1;
    const float update = div_fast(m, denom) + (h.wd * p);
#else
    const float denom = (__builtin_amdgcn_sqrtf(v) * h.rc2s + h.eps) * h.c1;
    const float update = m * __builtin_amdgcn_rcpf(denom) + (h.wd * p);
#endif
    return p - (h.lr * update);
}

// AdamW on one element; returns the new parameter, updates m and v in place.
__device__ __forceinline__ float adamw_elt(float p, float g, float &m, float &v, const Hyper &h)
{
    adamw_moments(g, m, v, h);
    return adamw_param(p, m, v, h);
}

// The same parameter update with the per-tensor constants folded on the host,
//     denom = sqrt(v) * (c1 / c2s) + eps * c1,   p - lr * (m / denom + wd * p)  as two fmas,
// and the hardware's square root and reciprocal (1 ulp each) without correction steps: 6 instructions
// instead of 19.  The result differs from adamw_param's by the rounding of at most four operations of
// the update term: |difference| <= 4e-7 * lr * |m / denom| + 1 ulp of p, far inside the 1e-6 relative
// bound on updated parameters.  The moments, and with them every code and scale, do not depend on it.
__device__ __forceinline__ float adamw_param_folded(float p, float m, float v, float lr, float wd, float fa, float fb)
{
    const float denom = __builtin_fmaf(__builtin_amdgcn_sqrtf(v), fa, fb);
    const float update = __builtin_fmaf(wd, p, m * __builtin_amdgcn_rcpf(denom));
    return __builtin_fmaf(-lr, update, p);
}

// bias corrections exactly as the reference computes them per thread
// (fused_adamw_kernel.cu:103-104), done once on the host
inline void bias_corrections(float beta1, float beta2, float step, float *c1, float *c2s)
{
    *c1 = 1.0f - powf(beta1, step);
    *c2s = sqrtf(1.0f - powf(beta2, step));
}

// ---------------------------------------------------------------------------------------
// Non-fused path (lpmm/optim/adamw.py:367-369, :412-422), with the roundings of the PyTorch
// CPU kernels its op sequence runs: multiply by the float-cast Python scalar, lerp as
// fma(w, g - m, m) for w < 0.5, addcmul as v + (value*g)*g, true division by the float-cast
// sqrt(bias_correction2), addcdiv as p + (value*m)/denom; bias corrections in double.
// ---------------------------------------------------------------------------------------
struct NfHyper {
    float decay, w1, b2, w2, neg_step_size, bc2_sqrt, rbc2_sqrt, eps;  // rbc2_sqrt = 1 / bc2_sqrt, correctly rounded
};

inline NfHyper make_nf_hyper(double beta1, double beta2, double lr, double wd, double eps, double step)
{
    NfHyper h;
    h.decay = (float)(1.0 - lr * wd);
    h.w1 = (float)(1.0 - beta1);
    h.b2 = (float)beta2;
    h.w2 = (float)(1.0 - beta2);
    const double bc1 = 1.0 - pow(beta1, step);
    const double bc2 = 1.0 - pow(beta2, step);
    h.neg_step_size = (float)(-(lr / bc1));
    h.bc2_sqrt = (float)sqrt(bc2);
    h.rbc2_sqrt = 1.0f / h.bc2_sqrt;
    h.eps = (float)eps;
    return h;
}

__device__ __forceinline__ float lerp_w(float a, float b, float w)
{
    return (fabsf(w) < 0.5f) ? __builtin_fmaf(w, b - a, a) : __builtin_fmaf(w - 1.0f, b - a, b);
}

// v.mul_(beta2).addcmul_(g, g, value=1 - beta2)
__device__ __forceinline__ void nonfused_second_moment(float &v, float g, const NfHyper &h)
{
    const float vi = v * h.b2;
    v = vi + (h.w2 * g) * g;
}

// One element of the non-fused update; p, m and v are updated in place.
__device__ __forceinline__ void nonfused_elt(float &p, float g, float &m, float &v, const NfHyper &h)
{
    const float pi = p * h.decay;
    m = lerp_w(m, g, h.w1);
    nonfused_second_moment(v, g, h);
    const float denom = div_by_rc(sqrt_fast(v), h.bc2_sqrt, h.rbc2_sqrt) + h.eps;
    p = pi + div_fast(h.neg_step_size * m, denom);
}

}  // namespace lpmm
