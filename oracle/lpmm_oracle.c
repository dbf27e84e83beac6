/*
 * CPU oracle for the 4-bit optimizer-state hot path of lpmm (thu-ml/low-bit-optimizers).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a scalar C restatement of the reference's
 * arithmetic, used only as the checker by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py.  Nothing in the shipped package may import, link or call
 * it; the product path is the HIP library and fails loudly when that is missing.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see oracle/Makefile).  Contraction is off
 * so that every float operation below rounds exactly once, as written; the only fused
 * operations are the explicit fmaf() calls, placed where the reference's PyTorch CPU path
 * uses a fused multiply-add (Tensor.lerp_).
 *
 * Each function names the reference lines it follows (paths relative to the reference
 * repository root).
 *
 * Parity status (what pins each function, apart from the HIP kernels being compared to it):
 *   qmapping            brute force against the closed form "number of fp32 midpoints < x",
 *                       every map point, every midpoint and its two neighbours, NaN, +-0.
 *   pack/unpack         exhaustive 256-byte round trip, length formulas, pad codes; the
 *                       any-width versions additionally against the 4-bit ones at width 4
 *                       and against a bit-by-bit Python restatement for widths 1..8.
 *   adamw_fp32_step     torch.optim.AdamW (library routine) over 100 steps.
 *   adamw4bit_step      closed form of the first step from zero state; equals
 *                       adamw_fp32_step when the state is representable; one-cell bound.
 *   quant/dequant group numpy abs/reshape/max restatement; max element decodes to scale.
 *   rank1               numpy row/col max + minimum.outer; 1-D reduces to group-128.
 *   nonfused_step       PyTorch CPU op sequence (library ops) of the reference's
 *                       _single_tensor_adamw4bit, to 1e-6 relative.
 *   factored_step       closed form v = row*col/mean(row) (Adafactor); rank-one g^2 case.
 *   nonfused_update_f16 PyTorch CPU op sequence on float16 tensors, bit for bit; the two
 *                       conversions against numpy.float16 on all 65536 halfs and on floats
 *                       around every rounding boundary.
 *   adamw4bit_step_f16  equals adamw4bit_step with the map rounded to half on inputs whose
 *                       later roundings vanish (states and gradients on a coarse binary grid,
 *                       betas 0.5 and 0.75); a numpy.float16 restatement operation by operation.
 *                       Against a real CUDA build of the half instantiation: parity unpinned.
 *   sgd_update          PyTorch CPU op sequence (library ops) of the reference's
 *                       _single_tensor_sgd4bit, bit for bit.
 *   philox / SR pack    Random123's known-answer vectors for philox4x32-10; torch.randint on
 *                       the GPU for cuRAND's state conventions; noise = 0.5 reduces the
 *                       stochastic search to round-to-nearest on the linear scale; the
 *                       empirical mean of the decoded codes equals x.  Against a real CUDA
 *                       build: parity unpinned (no CUDA here).
 * The reference ships no tests, golden vectors or fixtures for any of these.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LPMM_GROUP 128
#define LPMM_PACK_GROUP 2048

/* ------------------------------------------------------------------------------------ */
/* Code assignment.                                                                     */
/* lpmm/cpp_extension/fused_adamw_kernel.cu:27-49 (q_mapping) and                       */
/* lpmm/cpp_extension/quantization_kernel.cu:397-427 (quantize_bsearch<false>).         */
/* Returns the reference's int result: -1 for NaN input (the reference reads qmap[-1]   */
/* there and returns lo-1 = -1 whatever that read yields, because NaN compares false).  */
/* ------------------------------------------------------------------------------------ */
int lpmm_oracle_qmapping(const float *qmap, int bits, float x)
{
    int lo = 0;
    int hi = 1 << bits;

    if (x <= qmap[lo])
        return lo;
    if (qmap[hi - 1] <= x)
        return hi - 1;

    while (lo < hi) {
        int mi = (lo + hi) >> 1;
        if (qmap[mi] <= x)
            lo = mi + 1;
        else
            hi = mi;
    }
    if (lo == 0)
        return -1; /* only reachable for NaN */
    float mid_val = (qmap[lo - 1] + qmap[lo]) * 0.5f;
    return (mid_val < x) ? lo : lo - 1;
}

/* 4-bit code as stored: the reference masks the int with 0xF
 * (fused_adamw_kernel.cu:157-163, quantization_kernel.cu:452-453), so NaN -> 15. */
static inline uint8_t code4(const float *qmap, float x)
{
    return (uint8_t)(lpmm_oracle_qmapping(qmap, 4, x) & 0xF);
}

void lpmm_oracle_qmapping_many(const float *qmap, const float *x, int64_t n, uint8_t *codes)
{
    for (int64_t i = 0; i < n; ++i)
        codes[i] = code4(qmap, x[i]);
}

/* ------------------------------------------------------------------------------------ */
/* pack_nonlinear / unpack_nonlinear, 4-bit, non-stochastic.                            */
/* lpmm/cpp_extension/quantization_kernel.cu:430-459 (kernel), :461-477 (sizes),        */
/* :604-628 (unpack kernel).  x holds n_padded already-normalised values; out holds     */
/* n_padded/2 + 1 bytes; byte i = code(x[2i]) | code(x[2i+1]) << 4.  The reference      */
/* leaves the last byte uninitialised; it is written as 0 here.                         */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_pack_nonlinear_4bit(const float *x, const float *qmap, int64_t n_padded,
                                     uint8_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n_padded / 2; ++i)
        out[i] = (uint8_t)(code4(qmap, x[2 * i]) | (code4(qmap, x[2 * i + 1]) << 4));
    out[n_padded / 2] = 0;
}

void lpmm_oracle_unpack_nonlinear_4bit(const uint8_t *codes, const float *qmap, int64_t n,
                                       float *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        out[i] = qmap[(codes[i >> 1] >> ((i & 1) * 4)) & 0xF];
}

/* ------------------------------------------------------------------------------------ */
/* pack_nonlinear / unpack_nonlinear for any width 1..8, non-stochastic.                 */
/* lpmm/cpp_extension/quantization_kernel.cu:592-601, :695-705 (dispatch on the width):  */
/* widths that divide 8 and are below 8 go to the packing kernels (:430-459, :604-628:   */
/* 8/bits codes per byte, code j masked and shifted by j*bits), every other width to the */
/* one-code-per-byte kernels (:516-533: the int result cast to uint8_t, so -1 for NaN    */
/* becomes 255; :656-669: qmap[byte]).  out holds n_padded*storage_bits/8 + 1 bytes, the */
/* last one (uninitialised in the reference) written as 0.                               */
/* The reference's unpack reads qmap[255] for a NaN code of a width below 8, past the    */
/* end of the map; that read is undefined there and restated here as the map's last      */
/* entry (index masked to the width).                                                    */
/* ------------------------------------------------------------------------------------ */
static inline int width_is_packed(int bits)
{
    return 8 % bits == 0 && bits < 8;
}

void lpmm_oracle_pack_nonlinear(const float *x, const float *qmap, int bits, int64_t n_padded,
                                uint8_t *out)
{
    if (width_is_packed(bits)) {
        const int per = 8 / bits;
        const int mask = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
        for (int64_t b = 0; b < n_padded / per; ++b) {
            uint8_t byte = 0;
            for (int j = 0; j < per; ++j)
                byte |= (uint8_t)((lpmm_oracle_qmapping(qmap, bits, x[b * per + j]) & mask) << (j * bits));
            out[b] = byte;
        }
        out[n_padded / per] = 0;
    } else {
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n_padded; ++i)
            out[i] = (uint8_t)lpmm_oracle_qmapping(qmap, bits, x[i]);
        out[n_padded] = 0;
    }
}

void lpmm_oracle_unpack_nonlinear(const uint8_t *codes, const float *qmap, int bits, int64_t n,
                                  float *out)
{
    const int mask = (1 << bits) - 1;
    if (width_is_packed(bits)) {
        const int per = 8 / bits;
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; ++i)
            out[i] = qmap[(codes[i / per] >> ((i % per) * bits)) & mask];
    } else {
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; ++i)
            out[i] = qmap[codes[i] & mask];
    }
}

/* ------------------------------------------------------------------------------------ */
/* Stochastic rounding (quantize_bsearch<true>, quantization_kernel.cu:418-421) with the   */
/* random stream the reference draws it from: curandStatePhilox4_32_10_t initialised per   */
/* thread with curand_init(seed, thread id, offset) and read with curand_uniform           */
/* (quantization_kernel.cu:443-451, :526-531).  cuRAND itself is not part of the reference */
/* tree; its generator is the published Philox4x32-10 of Salmon et al. (SC'11, Random123), */
/* restated here, with cuRAND's documented conventions: key = the two halves of the seed,  */
/* counter words {x, y} = block index within the subsequence (offset / 4), {z, w} = the    */
/* subsequence, the four outputs of a block consumed in the order x, y, z, w starting at   */
/* offset % 4, and uniform = u * 2^-32 + 2^-33 in float, i.e. (0, 1].                      */
/* Pinned by: the three known-answer vectors of Random123 for philox4x32-10; PyTorch's     */
/* device generator on the GPU (torch.randint, which draws the raw outputs from the same    */
/* state layout) for the counter/subsequence/ordering conventions.  The uniform conversion  */
/* is cuRAND's documented one; the device library under PyTorch-ROCm differs from it in the */
/* last place, so it is compared to within that.                                            */
/* ------------------------------------------------------------------------------------ */
static inline void philox_round(uint32_t c[4], const uint32_t k[2])
{
    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k[0];
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k[1];
    const uint32_t n3 = (uint32_t)p0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
}

void lpmm_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]};
    uint32_t k[2] = {key[0], key[1]};
    for (int r = 0; r < 10; ++r) {
        if (r > 0) {
            k[0] += 0x9E3779B9u;
            k[1] += 0xBB67AE85u;
        }
        philox_round(c, k);
    }
    out[0] = c[0]; out[1] = c[1]; out[2] = c[2]; out[3] = c[3];
}

/* draw number j (0-based) of the state curand_init(seed, subsequence, offset) gives */
uint32_t lpmm_oracle_philox_draw(uint64_t seed, uint64_t subsequence, uint64_t offset, uint64_t j)
{
    const uint64_t pos = offset + j;  /* position in the subsequence, in 32-bit outputs */
    const uint64_t block = pos >> 2;
    const uint32_t ctr[4] = {(uint32_t)block, (uint32_t)(block >> 32), (uint32_t)subsequence,
                             (uint32_t)(subsequence >> 32)};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t out[4];
    lpmm_oracle_philox4x32_10(ctr, key, out);
    return out[pos & 3];
}

float lpmm_oracle_philox_uniform(uint64_t seed, uint64_t subsequence, uint64_t offset, uint64_t j)
{
    const float u = (float)lpmm_oracle_philox_draw(seed, subsequence, offset, j);
    return u * 0x1p-32f + 0x1p-33f;
}

/* quantize_bsearch<true> (quantization_kernel.cu:397-421).  NaN gives -1 as in the
 * non-stochastic search (the reference reads qmap[-1] there; __float2int_rn(NaN) is 0, so it
 * returns lo - 1 = -1 whatever that read yields). */
int lpmm_oracle_qmapping_sr(const float *qmap, int bits, float x, float noise)
{
    int lo = 0;
    int hi = 1 << bits;

    if (x <= qmap[lo])
        return lo;
    if (qmap[hi - 1] <= x)
        return hi - 1;
    while (lo < hi) {
        int mi = (lo + hi) >> 1;
        if (qmap[mi] <= x)
            lo = mi + 1;
        else
            hi = mi;
    }
    if (lo == 0)
        return -1;
    const float proba = (x - qmap[lo - 1]) / (qmap[lo] - qmap[lo - 1]);
    const float t = (proba + noise) - 0.5f;
    const int flag = (int)rintf(t); /* __float2int_rn: to nearest, ties to even */
    return flag ? lo : lo - 1;
}

/* pack_nonlinear(..., stochastic=True) for any width: thread t of the reference's launch
 * handles work_per_thread consecutive values (4 * 8/bits for the packing widths 1, 2, 4,
 * quantization_kernel.cu:437-441; 4 for the one-code-per-byte widths, :525) and draws one
 * uniform per value, in order, from subsequence t (:443-451, :526-531). */
void lpmm_oracle_pack_nonlinear_sr(const float *x, const float *qmap, int bits, int64_t n_padded,
                                   uint64_t seed, uint64_t offset, uint8_t *out)
{
    const int packed = width_is_packed(bits);
    const int per = packed ? 8 / bits : 1;
    const int wpt = 4 * per;
    const int mask = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n_padded / per; ++b) {
        uint8_t byte = 0;
        for (int j = 0; j < per; ++j) {
            const int64_t i = b * per + j;
            const float noise = lpmm_oracle_philox_uniform(seed, (uint64_t)(i / wpt), offset, (uint64_t)(i % wpt));
            const int q = lpmm_oracle_qmapping_sr(qmap, bits, x[i], noise);
            byte |= packed ? (uint8_t)((q & mask) << (j * bits)) : (uint8_t)q;
        }
        out[b] = byte;
    }
    out[n_padded / per] = 0;
}

/* ------------------------------------------------------------------------------------ */
/* Fused fp32-state AdamW step.  lpmm/cpp_extension/fused_adamw_kernel.cu:52-78.        */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_adamw_fp32_step(float *p, const float *g, float *m, float *v, int64_t n,
                                 float beta1, float beta2, float lr, float weight_decay,
                                 float eps, float step)
{
    const float correction1 = 1.0f - powf(beta1, step);
    const float correction2_sqrt = sqrtf(1.0f - powf(beta2, step));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        m[i] = beta1 * m[i] + (1 - beta1) * g[i];
        v[i] = beta2 * v[i] + (1 - beta2) * g[i] * g[i];
        float denom = (sqrtf(v[i]) / correction2_sqrt + eps) * correction1;
        float update = (m[i] / denom) + (weight_decay * p[i]);
        p[i] = p[i] - (lr * update);
    }
}

/* ------------------------------------------------------------------------------------ */
/* Fused 4-bit AdamW step.  lpmm/cpp_extension/fused_adamw_kernel.cu:81-174; state      */
/* sizes from lpmm/optim/adamw.py:508-523 ((n+1)/2 bytes, ceil(n/128) scales).          */
/* One 128-element block = one scale; low nibble of a byte = even element.  Elements    */
/* past n do not exist: they add 0 to the block maxima and leave their nibble 0.        */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_adamw4bit_step(float *p, const float *g, uint8_t *m_codes, uint8_t *v_codes,
                                float *m_scale, float *v_scale, const float *qmap_m,
                                const float *qmap_v, int64_t n, float beta1, float beta2,
                                float lr, float weight_decay, float eps, float step)
{
    const float correction1 = 1.0f - powf(beta1, step);
    const float correction2_sqrt = sqrtf(1.0f - powf(beta2, step));
    const int64_t blocks = (n + LPMM_GROUP - 1) / LPMM_GROUP;

#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < blocks; ++b) {
        const int64_t base = b * LPMM_GROUP;
        const int cnt = (int)((n - base) < LPMM_GROUP ? (n - base) : LPMM_GROUP);
        float mm[LPMM_GROUP], vv[LPMM_GROUP];
        float absmax_m = 0.0f, absmax_v = 0.0f;
        const float sm = m_scale[b], sv = v_scale[b];

        for (int k = 0; k < cnt; ++k) {
            const int64_t i = base + k;
            const uint8_t byte_m = m_codes[i >> 1], byte_v = v_codes[i >> 1];
            const int sh = (int)(i & 1) * 4;
            float ea = qmap_m[(byte_m >> sh) & 0xF] * sm;
            ea = beta1 * ea + (1 - beta1) * g[i];
            float es = qmap_v[(byte_v >> sh) & 0xF] * sv;
            es = beta2 * es + (1 - beta2) * g[i] * g[i];

            float denom = (sqrtf(es) / correction2_sqrt + eps) * correction1;
            float update = (ea / denom) + (weight_decay * p[i]);
            p[i] = p[i] - (lr * update);

            mm[k] = ea;
            vv[k] = es;
            absmax_m = fmaxf(absmax_m, fabsf(ea));
            absmax_v = fmaxf(absmax_v, es);
        }
        for (int k = 0; k < cnt; k += 2) {
            const int64_t i = base + k;
            uint8_t bm = code4(qmap_m, mm[k] / absmax_m);
            uint8_t bv = code4(qmap_v, vv[k] / absmax_v);
            if (k + 1 < cnt) {
                bm |= (uint8_t)(code4(qmap_m, mm[k + 1] / absmax_m) << 4);
                bv |= (uint8_t)(code4(qmap_v, vv[k + 1] / absmax_v) << 4);
            }
            m_codes[i >> 1] = bm;
            v_codes[i >> 1] = bv;
        }
        m_scale[b] = absmax_m;
        v_scale[b] = absmax_v;
    }
}

/* ------------------------------------------------------------------------------------ */
/* Group-wise ("group") quantisation into the non-fused packed layout.                  */
/* lpmm/functional.py:184-189 (scale: zero-pad to a multiple of gp_sz, per-group        */
/* max|x| of shape (G,1), true division), :404-422 (group_tensor), :359-369             */
/* (re-group to 2048 with zero padding, pack).  codes holds NG*1024+1 bytes with        */
/* NG = ceil(G*gp_sz/2048); max1 holds G floats.                                        */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_quant_group(const float *x, int64_t n, int64_t gp_sz, const float *qmap,
                             uint8_t *codes, float *max1)
{
    const int64_t G = (n + gp_sz - 1) / gp_sz;
    const int64_t scaled = G * gp_sz;
    const int64_t NG = (scaled + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP;
    const int64_t n_padded = NG * LPMM_PACK_GROUP;

#pragma omp parallel for schedule(static)
    for (int64_t gidx = 0; gidx < G; ++gidx) {
        float mx = 0.0f; /* padding contributes |0| */
        const int64_t lo = gidx * gp_sz;
        const int64_t hi = (lo + gp_sz < n) ? lo + gp_sz : n;
        for (int64_t i = lo; i < hi; ++i)
            mx = fmaxf(mx, fabsf(x[i]));
        max1[gidx] = mx;
    }
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n_padded / 2; ++b) {
        uint8_t byte = 0;
        for (int h = 0; h < 2; ++h) {
            const int64_t i = 2 * b + h;
            float val;
            if (i < n)
                val = x[i] / max1[i / gp_sz];
            else if (i < scaled)
                val = 0.0f / max1[i / gp_sz]; /* pad of the last group, divided too */
            else
                val = 0.0f; /* pad added by the re-grouping to 2048 */
            byte |= (uint8_t)(code4(qmap, val) << (4 * h));
        }
        codes[b] = byte;
    }
    codes[n_padded / 2] = 0;
}

/* lpmm/functional.py:393-400 (unpack, slice to scaled_shape), :115-118 (x.mul(max1),
 * slice to the parameter's numel). */
void lpmm_oracle_dequant_group(const uint8_t *codes, const float *max1, const float *qmap,
                               int64_t n, int64_t gp_sz, float *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        out[i] = qmap[(codes[i >> 1] >> ((i & 1) * 4)) & 0xF] * max1[i / gp_sz];
}

/* ------------------------------------------------------------------------------------ */
/* Rank-1 ("rank1") scaling of a 2-D tensor R x C.                                      */
/* lpmm/functional.py:190-203 (dim>=2 branch), :512-531 (per-dimension max|x|),         */
/* :503-509 (scale tensor = elementwise min of the broadcast maxima).                   */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_rank1_stats(const float *x, int64_t R, int64_t C, float *rowmax, float *colmax)
{
    for (int64_t c = 0; c < C; ++c)
        colmax[c] = 0.0f;
    for (int64_t r = 0; r < R; ++r) {
        float mx = 0.0f;
        for (int64_t c = 0; c < C; ++c) {
            float a = fabsf(x[r * C + c]);
            mx = fmaxf(mx, a);
            colmax[c] = fmaxf(colmax[c], a);
        }
        rowmax[r] = mx;
    }
}

void lpmm_oracle_quant_rank1(const float *x, int64_t R, int64_t C, const float *rowmax,
                             const float *colmax, const float *qmap, uint8_t *codes)
{
    const int64_t n = R * C;
    const int64_t NG = (n + LPMM_PACK_GROUP - 1) / LPMM_PACK_GROUP;
    const int64_t n_padded = NG * LPMM_PACK_GROUP;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < n_padded / 2; ++b) {
        uint8_t byte = 0;
        for (int h = 0; h < 2; ++h) {
            const int64_t i = 2 * b + h;
            float val = 0.0f;
            if (i < n) {
                const float rm = rowmax[i / C], cm = colmax[i % C];
                const float st = (cm < rm) ? cm : rm; /* torch.min(row, col) */
                val = x[i] / st;
            }
            byte |= (uint8_t)(code4(qmap, val) << (4 * h));
        }
        codes[b] = byte;
    }
    codes[n_padded / 2] = 0;
}

/* lpmm/functional.py:97-106 (x.mul(st)). */
void lpmm_oracle_dequant_rank1(const uint8_t *codes, const float *rowmax, const float *colmax,
                               const float *qmap, int64_t R, int64_t C, float *out)
{
    const int64_t n = R * C;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const float rm = rowmax[i / C], cm = colmax[i % C];
        const float st = (cm < rm) ? cm : rm;
        out[i] = qmap[(codes[i >> 1] >> ((i & 1) * 4)) & 0xF] * st;
    }
}

/* ------------------------------------------------------------------------------------ */
/* Elementwise part of the non-fused step.  lpmm/optim/adamw.py:367-369, :412-422.      */
/* The reference runs these as PyTorch ops; the roundings below are those of the        */
/* PyTorch CPU kernels: Tensor.mul_(python float) multiplies by the float-cast scalar;  */
/* lerp_ with weight < 0.5 is fma(w, g-m, m); addcmul_ is v + (value*g)*g; the division */
/* by sqrt(bias_correction2) is a true division by the float-cast scalar; addcdiv_ is   */
/* p + (value*m)/denom.  Bias corrections are Python doubles (adamw.py:415-419).        */
/* m and v are full fp32 tensors here (already dequantised / to be quantised).          */
/* ------------------------------------------------------------------------------------ */
static inline float lerp_small_w(float a, float b, float w)
{
    return (fabsf(w) < 0.5f) ? fmaf(w, b - a, a) : fmaf(w - 1.0f, b - a, b);
}

void lpmm_oracle_nonfused_update(float *p, const float *g, float *m, float *v, int64_t n,
                                 double beta1, double beta2, double lr, double weight_decay,
                                 double eps, double step)
{
    const float decay = (float)(1.0 - lr * weight_decay);
    const float w1 = (float)(1.0 - beta1);
    const float b2 = (float)beta2;
    const float w2 = (float)(1.0 - beta2);
    const double bc1 = 1.0 - pow(beta1, step);
    const double bc2 = 1.0 - pow(beta2, step);
    const float neg_step_size = (float)(-(lr / bc1));
    const float bc2_sqrt = (float)sqrt(bc2);
    const float epsf = (float)eps;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        float pi = p[i] * decay;
        float mi = lerp_small_w(m[i], g[i], w1);
        float vi = v[i] * b2;
        vi = vi + (w2 * g[i]) * g[i];
        float denom = sqrtf(vi) / bc2_sqrt + epsf;
        pi = pi + (neg_step_size * mi) / denom;
        p[i] = pi;
        m[i] = mi;
        v[i] = vi;
    }
}

/* ------------------------------------------------------------------------------------ */
/* The same elementwise part on float16 tensors (float16 parameters with fused=False:   */
/* the reference's op sequence then runs PyTorch's half kernels, lpmm/optim/adamw.py     */
/* :367-369, :412-422).  Every op of PyTorch on half tensors converts its operands to    */
/* float, computes as the float kernel does and rounds the result to half once, so the   */
/* chain below is the float chain above with a rounding to half after each op; Python    */
/* scalars enter as floats, never as halfs.  Conversions: IEEE binary16, round to        */
/* nearest even, subnormals kept (c10::Half, numpy.float16).                             */
/* ------------------------------------------------------------------------------------ */
static inline float h2f(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0x1Fu) {
        bits = sign | 0x7F800000u | (man << 13);
    } else if (exp != 0) {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    } else {
        /* zero or subnormal: man * 2^-24, exact in float */
        float f = (float)man * 0x1p-24f;
        memcpy(&bits, &f, 4);
        bits |= sign;
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

static inline uint16_t f2h(float f)
{
    uint32_t bits;
    memcpy(&bits, &f, 4);
    const uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    const uint32_t a = bits & 0x7FFFFFFFu;
    if (a > 0x7F800000u)
        return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu)); /* NaN stays NaN (quiet) */
    if (a >= 0x47800000u)                                          /* |f| >= 65536: infinity (65520 rounds there below) */
        return (uint16_t)(sign | 0x7C00u);
    if (a < 0x38800000u) {
        /* below the smallest normal half (2^-14): the result is round(|f| * 2^24) units of 2^-24; */
        /* adding 0.5f places those units at the last place of the float sum, which rounds to nearest even */
        float af;
        memcpy(&af, &a, 4);
        const float t = af + 0.5f;
        uint32_t tb;
        memcpy(&tb, &t, 4);
        return (uint16_t)(sign | (tb - 0x3F000000u));
    }
    /* normal: drop 13 mantissa bits with round to nearest even; a carry runs into the exponent */
    const uint32_t r = a + 0xFFFu + ((a >> 13) & 1u);
    return (uint16_t)(sign | ((r - 0x38000000u) >> 13));
}

void lpmm_oracle_f16_to_f32(const uint16_t *h, float *f, int64_t n)
{
    for (int64_t i = 0; i < n; ++i)
        f[i] = h2f(h[i]);
}

void lpmm_oracle_f32_to_f16(const float *f, uint16_t *h, int64_t n)
{
    for (int64_t i = 0; i < n; ++i)
        h[i] = f2h(f[i]);
}

static inline float rh(float x) { return h2f(f2h(x)); }

void lpmm_oracle_nonfused_update_f16(uint16_t *p, const uint16_t *g, uint16_t *m, uint16_t *v, int64_t n,
                                     double beta1, double beta2, double lr, double weight_decay,
                                     double eps, double step)
{
    const float decay = (float)(1.0 - lr * weight_decay);
    const float w1 = (float)(1.0 - beta1);
    const float b2 = (float)beta2;
    const float w2 = (float)(1.0 - beta2);
    const double bc1 = 1.0 - pow(beta1, step);
    const double bc2 = 1.0 - pow(beta2, step);
    const float neg_step_size = (float)(-(lr / bc1));
    const float bc2_sqrt = (float)sqrt(bc2);
    const float epsf = (float)eps;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const float gi = h2f(g[i]);
        const float pi = rh(h2f(p[i]) * decay);            /* param.mul_(1 - lr * weight_decay) */
        const float mi = rh(lerp_small_w(h2f(m[i]), gi, w1)); /* exp_avg.lerp_(grad, 1 - beta1) */
        float vi = rh(h2f(v[i]) * b2);                      /* exp_avg_sq.mul_(beta2) */
        vi = rh(vi + (w2 * gi) * gi);                       /* .addcmul_(grad, grad, value=1 - beta2) */
        float denom = rh(sqrtf(vi));                        /* exp_avg_sq.sqrt() */
        denom = rh(denom / bc2_sqrt);                       /* / bias_correction2_sqrt */
        denom = rh(denom + epsf);                           /* .add_(eps) */
        p[i] = f2h(pi + (neg_step_size * mi) / denom);      /* param.addcdiv_(exp_avg, denom, value=-step_size) */
        m[i] = f2h(mi);
        v[i] = f2h(vi);
    }
}

/* ------------------------------------------------------------------------------------ */
/* The fused 4-bit step instantiated on at::Half                                         */
/* (lpmm/cpp_extension/fused_adamw_kernel.cu:80-174 with T = at::Half, dispatch :222).   */
/* c10::Half arithmetic converts to float and back: Half * Half is the float product     */
/* rounded to half, float * Half and Half / float are float; an assignment to T rounds.  */
/*   T m = (T)qmap[idx] * scale[b];            map entry to half, product to half  (:119) */
/*   m = beta1 * m + (1 - beta1) * g[i];       float, rounded on assignment        (:120) */
/*   T v = (T)qmap[idx] * scale[b]; v = beta2 * v + (1 - beta2) * g[i] * g[i];   (:121-123) */
/*   denom, update in float; p[i] = p[i] - lr * update rounded on the store      (:125-127) */
/*   maxima and the normalised values (float)m / absmax in float                 (:148-157) */
/*   scale[b] = (T)absmax: exact, a maximum of halfs                             (:169-170) */
/* Layout as lpmm_oracle_adamw4bit_step; p, g and the scales are binary16 bit patterns.  */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_adamw4bit_step_f16(uint16_t *p, const uint16_t *g, uint8_t *m_codes, uint8_t *v_codes,
                                    uint16_t *m_scale, uint16_t *v_scale, const float *qmap_m,
                                    const float *qmap_v, int64_t n, float beta1, float beta2,
                                    float lr, float weight_decay, float eps, float step)
{
    const float correction1 = 1.0f - powf(beta1, step);
    const float correction2_sqrt = sqrtf(1.0f - powf(beta2, step));
    const int64_t blocks = (n + LPMM_GROUP - 1) / LPMM_GROUP;

#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < blocks; ++b) {
        const int64_t base = b * LPMM_GROUP;
        const int cnt = (int)((n - base) < LPMM_GROUP ? (n - base) : LPMM_GROUP);
        float mm[LPMM_GROUP], vv[LPMM_GROUP];
        float absmax_m = 0.0f, absmax_v = 0.0f;
        const float sm = h2f(m_scale[b]), sv = h2f(v_scale[b]);

        for (int k = 0; k < cnt; ++k) {
            const int64_t i = base + k;
            const uint8_t byte_m = m_codes[i >> 1], byte_v = v_codes[i >> 1];
            const int sh = (int)(i & 1) * 4;
            const float gi = h2f(g[i]), pi = h2f(p[i]);
            float ea = rh(rh(qmap_m[(byte_m >> sh) & 0xF]) * sm);
            ea = rh(beta1 * ea + (1 - beta1) * gi);
            float es = rh(rh(qmap_v[(byte_v >> sh) & 0xF]) * sv);
            es = rh(beta2 * es + (1 - beta2) * gi * gi);

            float denom = (sqrtf(es) / correction2_sqrt + eps) * correction1;
            float update = (ea / denom) + (weight_decay * pi);
            p[i] = f2h(pi - (lr * update));

            mm[k] = ea;
            vv[k] = es;
            absmax_m = fmaxf(absmax_m, fabsf(ea));
            absmax_v = fmaxf(absmax_v, es);
        }
        for (int k = 0; k < cnt; k += 2) {
            const int64_t i = base + k;
            uint8_t bm = code4(qmap_m, mm[k] / absmax_m);
            uint8_t bv = code4(qmap_v, vv[k] / absmax_v);
            if (k + 1 < cnt) {
                bm |= (uint8_t)(code4(qmap_m, mm[k + 1] / absmax_m) << 4);
                bv |= (uint8_t)(code4(qmap_v, vv[k + 1] / absmax_v) << 4);
            }
            m_codes[i >> 1] = bm;
            v_codes[i >> 1] = bv;
        }
        m_scale[b] = f2h(absmax_m);
        v_scale[b] = f2h(absmax_v);
    }
}

/* ------------------------------------------------------------------------------------ */
/* 4-bit SGD with momentum: the elementwise part of lpmm/optim/sgd.py:133-187            */
/* (_single_tensor_sgd4bit) on fp32 buffers, with the roundings of the PyTorch kernels   */
/* its op sequence runs: Tensor.add(other, alpha=s) is fma(s, other, self) with s cast   */
/* to float (alpha = 1 gives the same value as a plain add), mul_ is one multiply.       */
/*   d = -g if maximize else g;  d = d.add(p, alpha=wd) if wd != 0          (:152-155)   */
/*   first step: buf = d                                                    (:161-163)   */
/*   else:       buf.mul_(momentum).add_(d, alpha=1-dampening)              (:173)       */
/*   d = d.add(buf, alpha=momentum) if nesterov else buf                    (:176-179)   */
/*   p.add_(d, alpha=-lr)                                                   (:181)       */
/* buf is a full fp32 tensor here (already dequantised / to be quantised).               */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_sgd_update(float *p, const float *g, float *buf, int64_t n, double momentum,
                            double dampening, double lr, double weight_decay, int nesterov,
                            int maximize, int first_step)
{
    const float mom = (float)momentum;
    const float w = (float)(1.0 - dampening);
    const float wd = (float)weight_decay;
    const float neg_lr = (float)(-lr);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        float d = maximize ? -g[i] : g[i];
        if (weight_decay != 0.0)
            d = fmaf(wd, p[i], d);
        float b;
        if (first_step) {
            b = d;
        } else {
            b = buf[i] * mom;
            b = fmaf(w, d, b);
        }
        const float u = nesterov ? fmaf(mom, b, d) : b;
        p[i] = fmaf(neg_lr, u, p[i]);
        buf[i] = b;
    }
}

/* ------------------------------------------------------------------------------------ */
/* Factored second moment, 2-D R x C.  lpmm/optim/adamw.py:579-627, :571-576, :367-369. */
/* Row/col means of g^2 are accumulated in double and rounded once to float (PyTorch's  */
/* own float summation order is not restated; the difference is below the 1e-6          */
/* tolerance that applies to the parameters).  m is a full fp32 tensor here.            */
/* ------------------------------------------------------------------------------------ */
void lpmm_oracle_factored_stats(const float *g, int64_t R, int64_t C, float *row_mean,
                                float *col_mean)
{
    double *col = (double *)calloc((size_t)C, sizeof(double));
    for (int64_t r = 0; r < R; ++r) {
        double s = 0.0;
        for (int64_t c = 0; c < C; ++c) {
            float u = g[r * C + c] * g[r * C + c];
            s += (double)u;
            col[c] += (double)u;
        }
        row_mean[r] = (float)(s / (double)C);
    }
    for (int64_t c = 0; c < C; ++c)
        col_mean[c] = (float)(col[c] / (double)R);
    free(col);
}

/* exp_avg_sq_row/col EMA (adamw.py:609-610): row.mul_(beta2).add_(mean, alpha=1-beta2),
 * the add with alpha being fma(mean, alpha, row*beta2) in PyTorch's CPU kernel.
 * Returns mean(row) after the update, in float, accumulated in double. */
float lpmm_oracle_factored_ema(float *row, float *col, const float *row_mean,
                               const float *col_mean, int64_t R, int64_t C, double beta2)
{
    const float b2 = (float)beta2, w2 = (float)(1.0 - beta2);
    double s = 0.0;
    for (int64_t r = 0; r < R; ++r) {
        row[r] = fmaf(row_mean[r], w2, row[r] * b2);
        s += (double)row[r];
    }
    for (int64_t c = 0; c < C; ++c)
        col[c] = fmaf(col_mean[c], w2, col[c] * b2);
    return (float)(s / (double)R);
}

/* Parameter/first-moment update with v = (row/mean(row)) * col (adamw.py:571-576,
 * :607, :612-619), after the decoupled decay p *= 1 - lr*wd (adamw.py:369 / :478). */
void lpmm_oracle_factored_update(float *p, const float *g, float *m, const float *row,
                                 const float *col, float row_mean_all, int64_t R, int64_t C,
                                 double beta1, double beta2, double lr, double weight_decay,
                                 double eps, double step)
{
    const float decay = (float)(1.0 - lr * weight_decay);
    const float w1 = (float)(1.0 - beta1);
    const double bc1 = 1.0 - pow(beta1, step);
    const double bc2 = 1.0 - pow(beta2, step);
    const float neg_step_size = (float)(-(lr / bc1));
    const float bc2_sqrt = (float)sqrt(bc2);
    const float epsf = (float)eps;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        const float rf = row[r] / row_mean_all;
        for (int64_t c = 0; c < C; ++c) {
            const int64_t i = r * C + c;
            float pi = p[i] * decay;
            float mi = lerp_small_w(m[i], g[i], w1);
            float vi = rf * col[c];
            float denom = sqrtf(vi) / bc2_sqrt + epsf;
            p[i] = pi + (neg_step_size * mi) / denom;
            m[i] = mi;
        }
    }
}

int lpmm_oracle_max_threads(void)
{
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void lpmm_oracle_set_threads(int n)
{
#ifdef _OPENMP
    extern void omp_set_num_threads(int);
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}
