/*
 * lpmm_hip.h -- C ABI of the MI355X (gfx950) kernels for lpmm's 4-bit optimizer-state
 * hot path.  Plain pointers and sizes only: no torch types, no exceptions, no global
 * state; every call is asynchronous on the given HIP stream and re-entrant.
 *
 * All pointers are DEVICE pointers unless a parameter is documented as host memory.
 * `stream` is a hipStream_t passed as void* (NULL = the HIP null stream).
 * Every function returns an lpmm_status; 0 means the work was enqueued.
 * Argument validation happens before any HIP call, so bad arguments are reported
 * without touching a GPU.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * thu-ml/low-bit-optimizers repository root).
 */
#ifndef LPMM_HIP_H
#define LPMM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LPMM_HIP_ABI_VERSION 2

/* One quantisation group of the fused path = 128 elements = one scale
 * (lpmm/cpp_extension/fused_adamw_kernel.cu:216-219). */
#define LPMM_GROUP 128
/* Padding unit of the non-fused packed layout (lpmm/functional.py:362). */
#define LPMM_PACK_GROUP 2048
/* Most tensors one multi-tensor launch record can hold. */
#define LPMM_MULTI_MAX 48

typedef enum lpmm_status {
    LPMM_OK = 0,
    LPMM_ERR_NULL = 1,      /* a required pointer is NULL */
    LPMM_ERR_ALIGN = 2,     /* a pointer does not meet its stated alignment */
    LPMM_ERR_SIZE = 3,      /* a size/count is negative, zero where it may not be, or too big */
    LPMM_ERR_LAUNCH = 4,    /* the HIP runtime reported an error at launch */
    LPMM_ERR_ARG = 5        /* an enum/flag argument has an unknown value */
} lpmm_status;

const char *lpmm_status_string(int status);
int lpmm_abi_version(void);

/* ---------------------------------------------------------------------------------------
 * (a) Fused 4-bit AdamW step on one tensor, in place.
 * Replaces fused_adamw.adamw4bit_single_tensor
 *   (lpmm/cpp_extension/fused_adamw.cc:44-78, kernel fused_adamw_kernel.cu:81-174).
 *   p, g            fp32[n]                       (p updated in place; g read only)
 *   m_codes,v_codes uint8[(n+1)/2]                two 4-bit codes per byte, low nibble = even index
 *   m_scale,v_scale fp32[ceil(n/128)]             one scale per 128 elements
 *   qmap_m, qmap_v  fp32[16]                      ascending quantisation maps
 *   step            the reference's float step count (>= 1)
 * p and g need 4-byte alignment; 16-byte alignment of p and g and 4-byte alignment of the
 * code arrays selects the vectorised path (any torch allocation has it).
 * ------------------------------------------------------------------------------------- */
int lpmm_adamw4bit_step(float *p, const float *g, uint8_t *m_codes, uint8_t *v_codes,
                        float *m_scale, float *v_scale, const float *qmap_m,
                        const float *qmap_v, int64_t n, float beta1, float beta2, float lr,
                        float weight_decay, float eps, float step, void *stream);

/* The same operator on float16 tensors: the reference dispatches its 4-bit kernel on at::Half as
 * well (fused_adamw_kernel.cu:222-230), with p, g and both scale arrays of that type and the
 * maps float32 (fused_adamw.cc:60-65).  The instantiation rounds a map entry to half before it
 * meets the scale ((T)qmap[idx] * scale, a product of halfs), rounds the moments and the
 * parameter to half where they are assigned to T and computes everything else in float, the
 * normalised values included (fused_adamw_kernel.cu:119-128, :148-167).
 *   p, g            float16[n]
 *   m_scale,v_scale float16[ceil(n/128)]
 * Codes, maps and step as above.  p and g need 2-byte alignment, the code arrays too. */
int lpmm_adamw4bit_f16_step(void *p, const void *g, uint8_t *m_codes, uint8_t *v_codes,
                            void *m_scale, void *v_scale, const float *qmap_m,
                            const float *qmap_v, int64_t n, float beta1, float beta2, float lr,
                            float weight_decay, float eps, float step, void *stream);

/* One record of a multi-tensor launch; the array of records is HOST memory. */
typedef struct lpmm_adamw4bit_tensor {
    float *p;
    const float *g;
    uint8_t *m_codes;
    uint8_t *v_codes;
    float *m_scale;
    float *v_scale;
    int64_t n;
    float step;
    float reserved;
} lpmm_adamw4bit_tensor;

/* The same step over `count` tensors (host array `tensors`) in as few launches as
 * possible.  Replaces the per-tensor Python loop of _fused_adamw4bit
 * (lpmm/optim/adamw.py:463-542), one reference launch per tensor.  Each tensor carries
 * its own step (adamw.py:498); hyper-parameters are per parameter group, as in the
 * reference. */
int lpmm_adamw4bit_step_multi(const lpmm_adamw4bit_tensor *tensors, int64_t count,
                              const float *qmap_m, const float *qmap_v, float beta1,
                              float beta2, float lr, float weight_decay, float eps,
                              void *stream);

/* Fused fp32-state AdamW step (tensors at or under the quantisation threshold).
 * Replaces fused_adamw.adamw_single_tensor
 *   (lpmm/cpp_extension/fused_adamw.cc:15-41, kernel fused_adamw_kernel.cu:52-78). */
int lpmm_adamw_fp32_step(float *p, const float *g, float *m, float *v, int64_t n, float beta1,
                         float beta2, float lr, float weight_decay, float eps, float step,
                         void *stream);

typedef struct lpmm_adamw_fp32_tensor {
    float *p;
    const float *g;
    float *m;
    float *v;
    int64_t n;
    float step;
    float reserved;
} lpmm_adamw_fp32_tensor;

/* Multi-tensor form of the fp32-state step (the `else` branch of _fused_adamw4bit,
 * lpmm/optim/adamw.py:543-561). */
int lpmm_adamw_fp32_step_multi(const lpmm_adamw_fp32_tensor *tensors, int64_t count,
                               float beta1, float beta2, float lr, float weight_decay,
                               float eps, void *stream);

/* The same step for IEEE half-precision tensors: the p, g, m and v of every record point to
 * fp16[n] (2-byte aligned); all arithmetic is float.  Replaces fused_adamw.adamw_single_tensor
 * for at::Half tensors (the kernel template instantiated by AT_DISPATCH_FLOATING_TYPES_AND_HALF,
 * lpmm/cpp_extension/fused_adamw_kernel.cu:52-78, :188): every element read converts to float,
 * every write rounds to half, and the parameter update reads the moments back after their
 * rounding.  (The 4-bit operator cannot run half tensors in the reference either: its float32
 * scales are read through the parameters' type, :229-230.) */
int lpmm_adamw_fp16_step_multi(const lpmm_adamw_fp32_tensor *tensors, int64_t count, float beta1,
                               float beta2, float lr, float weight_decay, float eps, void *stream);

/* ---------------------------------------------------------------------------------------
 * (b) Stand-alone quantise / dequantise in the non-fused packed layout
 *     (NG*1024 + 1 bytes, NG = ceil(numel_scaled/2048); lpmm/functional.py:359-369,
 *     quantization_kernel.cu:475-477).  The trailing byte is written as 0.
 * ------------------------------------------------------------------------------------- */

/* Replaces ext_quantization.pack_nonlinear for bits = 4, stochastic = false
 *   (lpmm/cpp_extension/quantization.cc:54-63, quantization_kernel.cu:430-513).
 * x: fp32[n_padded] already normalised, n_padded a multiple of 8; out: n_padded/2 + 1 bytes. */
int lpmm_pack_nonlinear_4bit(const float *x, const float *qmap, int64_t n_padded, uint8_t *out,
                             void *stream);

/* Replaces ext_quantization.unpack_nonlinear for bits = 4
 *   (lpmm/cpp_extension/quantization.cc:65-76, quantization_kernel.cu:604-653).
 * out[i] = qmap[code_i] for i < n (n = num_groups * group_size in the reference call). */
int lpmm_unpack_nonlinear_4bit(const uint8_t *codes, const float *qmap, int64_t n, float *out,
                               void *stream);

/* vectorwise_quant with scale_type 'group' in one pass: per-group max|x| -> max1, x/max1,
 * code search, pack.  Replaces lpmm/functional.py:184-189 + :359-369 (abs, max, div, cat,
 * pack_nonlinear as separate passes).  gp_sz = 128 * 2^k, at most 4096; codes: ceil(G*gp_sz/2048)*1024 + 1 bytes; max1: fp32[G],
 * G = ceil(n/gp_sz). */
int lpmm_quant_group(const float *x, int64_t n, int64_t gp_sz, const float *qmap, uint8_t *codes,
                     float *max1, void *stream);

/* vectorwise_dequant with scale_type 'group': out[i] = qmap[code_i] * max1[i / gp_sz].
 * Replaces lpmm/functional.py:393-400 + :115-118. */
int lpmm_dequant_group(const uint8_t *codes, const float *max1, const float *qmap, int64_t n,
                       int64_t gp_sz, float *out, void *stream);

/* Rank-1 statistics of a row-major R x C tensor: rowmax[r] = max_c |x|, colmax[c] = max_r |x|.
 * Replaces get_sm3_statistics / _max_reduce_except_dim (lpmm/functional.py:512-531).
 * colmax is accumulated with atomics on the bit patterns of non-negative floats and is
 * cleared by the call itself. */
int lpmm_rank1_stats(const float *x, int64_t rows, int64_t cols, float *rowmax, float *colmax,
                     void *stream);

/* Rank-1 normalise + search + pack: code(x[r,c] / min(rowmax[r], colmax[c])).
 * Replaces lpmm/functional.py:199-203 + :503-509 + :359-369.  codes: ceil(R*C/2048)*1024+1. */
int lpmm_quant_rank1(const float *x, int64_t rows, int64_t cols, const float *rowmax,
                     const float *colmax, const float *qmap, uint8_t *codes, void *stream);

/* out[r,c] = qmap[code] * min(rowmax[r], colmax[c]).  Replaces lpmm/functional.py:97-106. */
int lpmm_dequant_rank1(const uint8_t *codes, const float *rowmax, const float *colmax,
                       const float *qmap, int64_t rows, int64_t cols, float *out, void *stream);

/* Rank-1 statistics of a contiguous tensor of 1..LPMM_RANK1_ND_MAX dimensions:
 * stats[i][j] = max |x| over the elements whose i-th index is j (stats[i] holds shape[i] floats).
 * Replaces get_sm3_statistics (lpmm/functional.py:512-531) for tensors the 2-D entry point
 * above does not cover; the statistics are cleared by the call itself.  `shape` and `stats` are
 * host arrays of ndim entries.  `work` is NULL or device memory for numel / shape[ndim-1] floats:
 * with it, a last dimension of 32 or more goes through the 2-D kernel (x is still read once). */
#define LPMM_RANK1_ND_MAX 8
int lpmm_rank1_stats_nd(const float *x, int ndim, const int64_t *shape, float *const *stats, float *work,
                        void *stream);

/* row_scale[r] = min over the leading dimensions i < ndim-1 of stats[i][index_i(r)], r running
 * over the rows of the (numel / shape[ndim-1]) x shape[ndim-1] view; NaN if any of them is
 * (torch.min).  With row_scale as `rowmax` and stats[ndim-1] as `colmax`, lpmm_quant_rank1 /
 * lpmm_dequant_rank1 (and their _bits forms) on that 2-D view apply the reference's scale
 * min_i stats[i] (lpmm/functional.py:503-509) to the N-D tensor.  stats[ndim-1] is not read. */
int lpmm_rank1_row_scale_nd(const float *const *stats, int ndim, const int64_t *shape, float *row_scale,
                            void *stream);

/* Statistics and scale of short vectors, many per call (no counterpart in the reference).  For
 * each record: stats[i][j] = max |x| over the elements of the vector x (row-major, shape[0..ndim))
 * whose i-th index is j, written in full, and scale[e] = the minimum of element e's statistics (NaN
 * if any of them is).  That is lpmm_rank1_stats_nd followed by lpmm_rank1_row_scale_nd over all of the
 * vector's dimensions, in one launch for up to 32 vectors -- what lies between the two passes of
 * lpmm_nonfused_adamw4bit_rank1_pass_multi for tensors of more than two dimensions, whose trailing
 * dimensions are the vector's.  ndim 1..7, at most 8192 statistics entries per vector (the sum of
 * its dimensions), fewer than 2^31 elements; one workgroup works through a vector, so the call
 * is for vectors of thousands of values (a long one is better served by the two calls it stands
 * for); records live in host memory and are consumed during the call. */
typedef struct lpmm_rank1_small_vector {
    const float *x;
    float *scale;
    float *stats[LPMM_RANK1_ND_MAX - 1];
    int64_t shape[LPMM_RANK1_ND_MAX - 1];
    int32_t ndim;
    int32_t reserved;
} lpmm_rank1_small_vector;
int lpmm_rank1_small_fold_scale_multi(const lpmm_rank1_small_vector *vectors, int64_t count, void *stream);

/* ---------------------------------------------------------------------------------------
 * The same six operations for any code width 1..8(lpmm/configs/default_{5,6,7,8}b.yml use
 * 5..8).  Storage follows lpmm/cpp_extension/quantization_kernel.cu:592-601, :695-705:
 * widths 1, 2, 4 pack 8/bits codes per byte (code j of a byte at bit j*bits), every other
 * width stores one code per byte; arrays hold n_padded*storage_bits/8 + 1 bytes and must be
 * 8-byte aligned.  qmap: 2^bits ascending floats.  Codes come from the reference's search
 * (:397-427); for NaN it stores the all-ones code (packed) or 255 (one code per byte), which
 * decodes here as map entry 2^bits - 1 (the reference would read past a shorter map).
 * ------------------------------------------------------------------------------------- */
int lpmm_pack_nonlinear(const float *x, const float *qmap, int bits, int64_t n_padded, uint8_t *out,
                        void *stream);
/* pack_nonlinear(..., stochastic=True): lpmm/cpp_extension/quantization.cc:54-63 with
 * quantize_bsearch<true> (quantization_kernel.cu:418-421): between map entries q[lo-1] <= x <
 * q[lo] the code is lo with probability (x - q[lo-1]) / (q[lo] - q[lo-1]).  The random numbers
 * are the ones the reference draws (:443-451, :526-531): Philox4x32-10 keyed by `seed`, one
 * subsequence per reference thread (4 * codes-per-byte consecutive values), starting `offset`
 * outputs into each subsequence -- the (seed, offset) pair the reference takes from torch's
 * default device generator (:480-487).  n_padded: a multiple of 32. */
int lpmm_pack_nonlinear_sr(const float *x, const float *qmap, int bits, int64_t n_padded, uint64_t seed,
                           uint64_t offset, uint8_t *out, void *stream);
int lpmm_unpack_nonlinear(const uint8_t *codes, const float *qmap, int bits, int64_t n, float *out,
                          void *stream);
int lpmm_quant_group_bits(const float *x, int64_t n, int64_t gp_sz, const float *qmap, int bits,
                          uint8_t *codes, float *max1, void *stream);
int lpmm_dequant_group_bits(const uint8_t *codes, const float *max1, const float *qmap, int bits,
                            int64_t n, int64_t gp_sz, float *out, void *stream);
int lpmm_quant_rank1_bits(const float *x, int64_t rows, int64_t cols, const float *rowmax,
                          const float *colmax, const float *qmap, int bits, uint8_t *codes, void *stream);

/* Code tables (no counterpart in the reference, whose kernels search the map for every value).
 * For a map that qualifies -- strictly increasing, as create_dynamic_map gives
 * (lpmm/functional.py:272-300) -- the code of the search of quantization_kernel.cu:397-427 is the
 * number of midpoints below x, and one read of a table over the sign, the exponent and the
 * leading bits - 2 mantissa bits of x finds it.  The table belongs to the map: build it once
 * (one small launch) and pass it with the map to the _table entry points below, which otherwise
 * equal the entry points without the suffix and give the same bytes; NULL, a table built for
 * another width or one of a map that does not qualify means the search.  table:
 * LPMM_CODE_TABLE_BYTES device bytes, 16-byte aligned, written in full; its last word says what
 * the builder found (search / the evenly spaced map's closed form / table).  A table that was
 * built from a different map of the same width gives wrong codes without an error. */
#define LPMM_CODE_TABLE_BYTES 12288
int lpmm_code_table_build(const float *qmap, int bits, void *table, void *stream);
int lpmm_quant_group_bits_table(const float *x, int64_t n, int64_t gp_sz, const float *qmap, int bits,
                                const void *table, uint8_t *codes, float *max1, void *stream);
int lpmm_quant_rank1_bits_table(const float *x, int64_t rows, int64_t cols, const float *rowmax,
                                const float *colmax, const float *qmap, int bits, const void *table,
                                uint8_t *codes, void *stream);
int lpmm_dequant_rank1_bits(const uint8_t *codes, const float *rowmax, const float *colmax,
                            const float *qmap, int bits, int64_t rows, int64_t cols, float *out,
                            void *stream);

/* ---------------------------------------------------------------------------------------
 * Non-fused step, elementwise part on fp32 m and v (already dequantised):
 * decoupled decay, lerp, EMA of g*g, bias-corrected update.
 * Replaces the PyTorch op sequence of _single_tensor_adamw4bit
 *   (lpmm/optim/adamw.py:367-369, :412-422).  Scalars are doubles, as in Python.
 * ------------------------------------------------------------------------------------- */
int lpmm_nonfused_update(float *p, const float *g, float *m, float *v, int64_t n, double beta1,
                         double beta2, double lr, double weight_decay, double eps, double step,
                         void *stream);

/* The same update for a list of tensors in one launch per 64 tensors (the many small
 * tensors that keep fp32 states); records as for lpmm_adamw_fp32_step_multi. */
int lpmm_nonfused_update_multi(const lpmm_adamw_fp32_tensor *tensors, int64_t count, double beta1,
                               double beta2, double lr, double weight_decay, double eps, void *stream);

/* The whole non-fused step on 4-bit states in one pass, for the configuration the reference
 * uses by default when fused=False is combined with block-wise second-moment scaling (both
 * moments 4-bit, 'group' scaling, gp_sz 128, real-nearest): dequantise m and v, the update
 * above, re-quantise, for a list of tensors in one launch per LPMM_MULTI_MAX tensors.
 * Replaces the body of _single_tensor_adamw4bit for such tensors
 *   (lpmm/optim/adamw.py:394-436: vectorwise_dequant x2, the op sequence, vectorwise_quant x2).
 * Records are lpmm_adamw4bit_tensor with the non-fused state layout:
 *   m_codes, v_codes: ceil(n/2048)*1024 + 1 bytes each (lpmm/functional.py:503-509), written
 *                     in full by every call, padding included;
 *   m_scale, v_scale: the (ceil(n/128), 1) "max1" tensors.
 * Before the first step the scales must be zero and the codes those of 0.0 (0x77 bytes for
 * the standard first-moment map, 0x00 for the second): that state decodes to the all-zero
 * moments the reference starts from. */
int lpmm_nonfused_adamw4bit_step_multi(const lpmm_adamw4bit_tensor *tensors, int64_t count,
                                       const float *qmap_m, const float *qmap_v, double beta1,
                                       double beta2, double lr, double weight_decay, double eps,
                                       void *stream);

/* The whole non-fused step with the reference's default scalings (lpmm/configs/default.yml:
 * first moment 4-bit 'group' gp_sz 128, second moment 4-bit 'rank1') on row-major R x C
 * tensors whose column count is a multiple of 128, in two passes over HBM: update + first
 * moment + statistics of the new second moment, then re-quantisation of the second moment.
 * Replaces, for such tensors, the body of _single_tensor_adamw4bit
 *   (lpmm/optim/adamw.py:394-436) including get_sm3_statistics (lpmm/functional.py:503-509
 *   for the packed layout, :190-203 for the rank-1 scale).
 * v_rowmax (R floats) / v_colmax (C floats) are the statistics the v codes are currently
 * scaled by (max_dims of the reference's metadata); the call leaves the statistics of the
 * new second moment in v_rowmax_next / v_colmax_next (cleared by the call, must not alias
 * the current ones) and the v codes scaled by them: the caller swaps the two pairs.
 * Code arrays: ceil(R*C/2048)*1024 + 1 bytes, 4-byte aligned, written in full.  Before the
 * first step all scales and statistics must be zero and the codes those of 0.0. */
typedef struct lpmm_nonfused_rank1_tensor {
    float *p;
    const float *g;
    uint8_t *m_codes;
    float *m_max1;
    uint8_t *v_codes;
    const float *v_rowmax;
    const float *v_colmax;
    float *v_rowmax_next;
    float *v_colmax_next;
    int64_t rows;
    int64_t cols;
    float step;
    float reserved;
} lpmm_nonfused_rank1_tensor;

int lpmm_nonfused_adamw4bit_rank1_step_multi(const lpmm_nonfused_rank1_tensor *tensors, int64_t count,
                                             const float *qmap_m, const float *qmap_v, double beta1,
                                             double beta2, double lr, double weight_decay, double eps,
                                             void *stream);

/* One pass of lpmm_nonfused_adamw4bit_rank1_step_multi at a time (no counterpart in the
 * reference, which has no passes): pass 1 clears the next statistics, updates p, re-quantises m and
 * leaves the row and column maxima of the new second moment in v_rowmax_next / v_colmax_next;
 * pass 2 recomputes the new second moment from g and the old codes and statistics and quantises
 * it with whatever v_rowmax_next / v_colmax_next hold then.  Between the two a caller may replace
 * the maxima by scales derived from them: a tensor of more than two dimensions, viewed as
 * shape[0] x (numel / shape[0]), has the reference's scale min over all dimensions
 * (lpmm/functional.py:503-531) when its column scale is the minimum over the trailing dimensions'
 * statistics -- lpmm_rank1_row_scale_nd on shape[1:] gives it before pass 1 (as v_colmax) and,
 * from the statistics that lpmm_rank1_stats_nd folds out of pass 1's column maxima, before
 * pass 2 (as v_colmax_next; see lpmm/optim/adamw.py::_rank1_nd_steps).  Both calls take the same
 * records, apart from the pointers the caller redirects. */
int lpmm_nonfused_adamw4bit_rank1_pass_multi(const lpmm_nonfused_rank1_tensor *tensors, int64_t count,
                                             const float *qmap_m, const float *qmap_v, double beta1,
                                             double beta2, double lr, double weight_decay, double eps,
                                             int pass, void *stream);

/* The non-fused step on float16 parameters (4-bit states, first moment 'group' gp_sz 128).  With
 * fused=False the reference's op sequence runs PyTorch's half kernels: every op computes in float
 * and rounds its result to half once, Python scalars enter as floats
 *   (lpmm/optim/adamw.py:367-369, :394-434);
 * states, scales and statistics are half tensors, the normalised values are rounded to half by the
 * division and widened to float for the search
 *   (lpmm/functional.py:184-203, lpmm/cpp_extension/quantization_kernel.cu:450),
 * and a dequantised value is the float product of the map entry and the half scale, rounded to
 * half (lpmm/functional.py:97-118, :150).  These two entry points are that chain in one and in two
 * passes over HBM; p, g, the scales and the statistics are IEEE binary16 arrays, the code arrays
 * have the layout of the float entry points above, the first-step convention is theirs too.
 *
 * lpmm_nonfused_adamw4bit_f16_step_multi: second moment 'group' gp_sz 128 (also a vector under
 * 'rank1'); one pass; any n; up to 48 tensors per launch.
 * lpmm_nonfused_adamw4bit_rank1_f16_step_multi: second moment 'rank1' on row-major R x C tensors
 * whose column count is a multiple of 128; two passes.  v_rowmax / v_colmax (R / C halfs) are the
 * statistics the v codes are scaled by, v_rowmax_next / v_colmax_next receive those of the new
 * second moment (must not alias the current ones: the caller swaps the pairs); `work` is scratch
 * of ((R + 3) / 4 * 4 + C) floats, 16-byte aligned, whose contents do not matter before and
 * after the call.  p, g and v_colmax 16-byte aligned, the code arrays, m_max1 and v_rowmax 4-byte,
 * the next statistics 2-byte. */
typedef struct lpmm_adamw4bit_f16_tensor {
    void *p;
    const void *g;
    uint8_t *m_codes;
    uint8_t *v_codes;
    void *m_max1;
    void *v_max1;
    int64_t n;
    float step;
    float reserved;
} lpmm_adamw4bit_f16_tensor;

int lpmm_nonfused_adamw4bit_f16_step_multi(const lpmm_adamw4bit_f16_tensor *tensors, int64_t count,
                                           const float *qmap_m, const float *qmap_v, double beta1,
                                           double beta2, double lr, double weight_decay, double eps,
                                           void *stream);

typedef struct lpmm_nonfused_rank1_f16_tensor {
    void *p;
    const void *g;
    uint8_t *m_codes;
    void *m_max1;
    uint8_t *v_codes;
    const void *v_rowmax;
    const void *v_colmax;
    void *v_rowmax_next;
    void *v_colmax_next;
    float *work;
    int64_t rows;
    int64_t cols;
    float step;
    float reserved;
} lpmm_nonfused_rank1_f16_tensor;

int lpmm_nonfused_adamw4bit_rank1_f16_step_multi(const lpmm_nonfused_rank1_f16_tensor *tensors,
                                                 int64_t count, const float *qmap_m,
                                                 const float *qmap_v, double beta1, double beta2,
                                                 double lr, double weight_decay, double eps,
                                                 void *stream);

/* The non-fused step with an fp32 first moment and a 4-bit second moment: the configurations
 * that quantise the second moment only (QUANT.M.ENABLE False: lpmm/configs/
 * 2nd_moment_only_group_128.yml and 2nd_moment_only_default.yml).  In _single_tensor_adamw4bit
 * exp_avg then is the state tensor itself, updated in place by lerp_ (lpmm/optim/adamw.py:397-399,
 * :412), and only exp_avg_sq is dequantised and quantised again (:402-409, :430-434).  Same
 * arithmetic, state layouts and first-step convention as the two entry points above, with
 * m: float[n] in place of the first moment's codes and scales.
 *
 * lpmm_nonfused_adamw_v4bit_step_multi: second moment with 'group' scaling, gp_sz 128; one
 * pass; any n; up to 48 tensors per launch.
 * lpmm_nonfused_adamw_v4bit_rank1_step_multi: second moment with 'rank1' scaling on row-major
 * R x C tensors whose column count is a multiple of 128; two passes; the statistics trade
 * places as in lpmm_nonfused_adamw4bit_rank1_step_multi; p, g and m 16-byte aligned. */
typedef struct lpmm_adamw_v4bit_tensor {
    float *p;
    const float *g;
    float *m;
    uint8_t *v_codes;
    float *v_max1;
    int64_t n;
    float step;
    float reserved;
} lpmm_adamw_v4bit_tensor;

int lpmm_nonfused_adamw_v4bit_step_multi(const lpmm_adamw_v4bit_tensor *tensors, int64_t count,
                                         const float *qmap_v, double beta1, double beta2, double lr,
                                         double weight_decay, double eps, void *stream);

typedef struct lpmm_rank1_v4bit_tensor {
    float *p;
    const float *g;
    float *m;
    uint8_t *v_codes;
    const float *v_rowmax;
    const float *v_colmax;
    float *v_rowmax_next;
    float *v_colmax_next;
    int64_t rows;
    int64_t cols;
    float step;
    float reserved;
} lpmm_rank1_v4bit_tensor;

int lpmm_nonfused_adamw_v4bit_rank1_step_multi(const lpmm_rank1_v4bit_tensor *tensors, int64_t count,
                                               const float *qmap_v, double beta1, double beta2,
                                               double lr, double weight_decay, double eps,
                                               void *stream);

/* The two-pass step above with a first moment whose 'group' scaling spans m_group_size =
 * 256, 512, 1024, 2048 or 4096 values of the flattened tensor (lpmm/configs/
 * 1st_moment_group_{256,512,1024,2048,4096}.yml; group_tensor, lpmm/functional.py:404-422).
 * A group then spans several 128-column pieces and, where the column count is not a multiple
 * of the group size, tensor rows: the update pass merges the groups' maxima of the new first
 * moment into m_max1_next (cleared by the call, must not alias m_max1), and the second pass
 * recomputes the first moment from g and the old codes and scales, bit-identically, and
 * overwrites its codes scaled by m_max1_next -- the caller swaps m_max1 / m_max1_next like the
 * statistics of the second moment.  m_codes: ceil(ceil(R*C / m_group_size) * m_group_size / 2048)
 * * 1024 + 1 bytes, 4-byte aligned, written in full; m_max1, m_max1_next: float[ceil(R*C /
 * m_group_size)].  Everything else as in lpmm_nonfused_adamw4bit_rank1_step_multi.
 *
 * This entry point also takes column counts that are no multiple of 128 (any multiple of 8, e.g.
 * 1600 or 1000), with m_group_size 128 as well: the 128-value groups of the flattened tensor then
 * straddle tensor rows, which is the same global dependency.  A call with such a tensor runs
 * more general (somewhat slower) kernels on all its tensors. */
typedef struct lpmm_rank1_mgroup_tensor {
    float *p;
    const float *g;
    uint8_t *m_codes;
    const float *m_max1;
    float *m_max1_next;
    uint8_t *v_codes;
    const float *v_rowmax;
    const float *v_colmax;
    float *v_rowmax_next;
    float *v_colmax_next;
    int64_t rows;
    int64_t cols;
    float step;
    float reserved;
} lpmm_rank1_mgroup_tensor;

int lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi(const lpmm_rank1_mgroup_tensor *tensors,
                                                    int64_t count, const float *qmap_m,
                                                    const float *qmap_v, int64_t m_group_size,
                                                    double beta1, double beta2, double lr,
                                                    double weight_decay, double eps, void *stream);

/* lpmm_nonfused_adamw4bit_rank1_step_multi for code widths of 5 to 8 bits (lpmm/configs/
 * default_{5,6,7,8}b.yml): qmap_m / qmap_v hold 2^bits_m / 2^bits_v entries; the code arrays hold
 * one code per byte (lpmm/cpp_extension/quantization_kernel.cu:516-533, :656-669):
 * ceil(R*C/2048)*2048 + 1 bytes each, 4-byte aligned, written in full.  Codes are found by the
 * reference's search (:397-427), so maps with repeated entries behave as there.  Everything
 * else (records, statistics, first-step convention) as in the 4-bit entry point. */
int lpmm_nonfused_adamw_bits_rank1_step_multi(const lpmm_nonfused_rank1_tensor *tensors,
                                              int64_t count, const float *qmap_m, int bits_m,
                                              const float *qmap_v, int bits_v, double beta1,
                                              double beta2, double lr, double weight_decay,
                                              double eps, void *stream);
/* The same with the code tables of the two maps (lpmm_code_table_build; either may be NULL). */
int lpmm_nonfused_adamw_bits_rank1_step_multi_table(const lpmm_nonfused_rank1_tensor *tensors,
                                                    int64_t count, const float *qmap_m, int bits_m,
                                                    const void *table_m, const float *qmap_v,
                                                    int bits_v, const void *table_v, double beta1,
                                                    double beta2, double lr, double weight_decay,
                                                    double eps, void *stream);

/* ---------------------------------------------------------------------------------------
 * (c) Factored second moment on a row-major R x C tensor.
 * Replaces _single_quantized_factored_update (lpmm/optim/adamw.py:579-627) and
 * _approx_sq_grad (:571-576).
 * ------------------------------------------------------------------------------------- */

/* Pass 1: row/col means of g*g folded into the EMAs
 *   row = beta2*row + (1-beta2)*mean_c(g^2), col likewise (adamw.py:608-610),
 * and *row_mean_all = mean(row) after the update (adamw.py:574).
 * workspace: device scratch of lpmm_factored_workspace_bytes(rows, cols) bytes. */
int64_t lpmm_factored_workspace_bytes(int64_t rows, int64_t cols);
int lpmm_factored_stats(const float *g, int64_t rows, int64_t cols, float *row, float *col,
                        float *row_mean_all, double beta2, void *workspace, void *stream);

/* lpmm_factored_stats without the workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  The partial sums go to an array of
 * LPMM_FACTORED_STATIC_BYTES that the library's code object holds on every GPU it runs on until
 * the process ends; the call allocates and frees nothing.  Shapes whose
 * lpmm_factored_workspace_bytes(rows, cols) exceeds that size return LPMM_ERR_SIZE.  All calls
 * on one GPU share the array: calls that overlap on one GPU (different streams) race.  Same
 * results as lpmm_factored_stats.
 * The first call on each GPU looks the array's address up (hipGetSymbolAddress, which may load the
 * code object): make that call outside any stream capture, as a warm-up on a small input.  Every
 * later call on that GPU only enqueues three kernels on `stream` and may be recorded into a HIP
 * graph; replays use the same array. */
#define LPMM_FACTORED_STATIC_BYTES (32u << 20)
int lpmm_factored_stats_static(const float *g, int64_t rows, int64_t cols, float *row, float *col,
                               float *row_mean_all, double beta2, void *stream);

/* Pass 2: p *= 1-lr*wd; m = dequant(m_codes); m.lerp_(g, 1-beta1);
 * v = row/row_mean_all * col; p += -lr/bc1 * m / (sqrt(v)/sqrt(bc2) + eps); m re-quantised
 * with 'group' scaling, gp_sz 128, into the non-fused packed layout (adamw.py:596-625).
 * first_step != 0 means m starts at zero and m_codes/m_max1 are only written. */
int lpmm_factored_update(float *p, const float *g, uint8_t *m_codes, float *m_max1,
                         const float *qmap_m, const float *row, const float *col,
                         const float *row_mean_all, int64_t rows, int64_t cols, double beta1,
                         double beta2, double lr, double weight_decay, double eps, double step,
                         int first_step, void *stream);

/* Both passes for a list of row-major R x C tensors whose column count is a multiple of 128
 * and whose first moment is quantised (4-bit, 'group', gp_sz 128): statistics and update of
 * all tensors in four launches per group of up to 24 tensors
 * instead of four per tensor.  Same results as
 * lpmm_factored_stats followed by lpmm_factored_update.  workspace: device scratch of
 * lpmm_factored_workspace_bytes(rows, cols) bytes per tensor, 8-byte aligned, not shared
 * between the tensors of one call; p, g and col 16-byte aligned. */
typedef struct lpmm_factored_tensor {
    float *p;
    const float *g;
    uint8_t *m_codes;
    float *m_max1;
    float *row;
    float *col;
    void *workspace;
    int64_t rows;
    int64_t cols;
    float step;
    int32_t first_step;
} lpmm_factored_tensor;

int lpmm_factored_step_multi(const lpmm_factored_tensor *tensors, int64_t count, const float *qmap_m,
                             double beta1, double beta2, double lr, double weight_decay, double eps,
                             void *stream);

/* The same pass with an fp32 first moment (m read and written as floats): tensors at or
 * under the quantisation threshold, or first-moment quantisation disabled
 * (the `else: exp_avg = q_exp_avg` branch, lpmm/optim/adamw.py:603-604). */
int lpmm_factored_update_fp32m(float *p, const float *g, float *m, const float *row,
                               const float *col, const float *row_mean_all, int64_t rows,
                               int64_t cols, double beta1, double beta2, double lr,
                               double weight_decay, double eps, double step, void *stream);

/* ---------------------------------------------------------------------------------------
 * (d) SGD with a 4-bit momentum buffer, one pass, for a list of tensors.
 * Replaces the per-tensor op chain of _single_tensor_sgd4bit (lpmm/optim/sgd.py:133-187) for
 * tensors whose buffer is quantised with 4 bits, 'group' scaling, gp_sz 128, round to nearest:
 *   d = -g if maximize else g;  d += weight_decay * p (if weight_decay != 0)     (:152-155)
 *   buf = d on the first step, else buf = dequant(codes) * momentum + (1 - dampening) * d  (:161-173)
 *   d = d + momentum * buf if nesterov else buf;  p += -lr * d                   (:176-181)
 *   codes, max1 = quantise(buf)                                                  (:184-187)
 * Every multiply-add of the chain is one fused operation with the float-cast scalar, as in
 * PyTorch's kernels.  m_codes: int8[ceil(n / 2048) * 1024 + 1] (the packed layout of
 * vectorwise_quant), m_max1: float[ceil(n / 128)]; first_step != 0 means the buffer does not
 * exist yet and both are only written.  momentum must not be 0 (the reference keeps no buffer
 * then).  Up to 64 tensors per launch. */
typedef struct lpmm_sgd4bit_tensor {
    float *p;
    const float *g;
    uint8_t *m_codes;
    float *m_max1;
    int64_t n;
    int32_t first_step;
    int32_t reserved;
} lpmm_sgd4bit_tensor;

int lpmm_sgd4bit_step_multi(const lpmm_sgd4bit_tensor *tensors, int64_t count, const float *qmap,
                            double momentum, double dampening, double lr, double weight_decay,
                            int nesterov, int maximize, void *stream);

/* ---------------------------------------------------------------------------------------
 * Diagnostic (no counterpart in the reference): compares the library's near-exact sqrt and
 * division sequences (hardware approximation + one fma correction of the residual) with the
 * correctly rounded operations on the device.  counts: 11 zero-initialised device uint64:
 *   [0] sqrt inputs tried (every sqrt_stride-th positive normal float), [1] results that
 *   differ from sqrtf, [2] of those, by more than 1 ulp, [3] of those, with an input of at
 *   least 2^-100 (below that the residual underflows; such a second moment is far below any
 *   eps); [4] division pairs tried, [5] results that differ from x/d, [6] of those, by more
 *   than 1 ulp; [7] pairs tried for the reciprocal-based group division, [8] results that
 *   differ from x/y (must stay 0); [9] floats tried for the Newton-corrected reciprocal of the
 *   group maximum (every float in [2^-60, 2^60]), [10] results that differ from 1/y (must
 *   stay 0).
 * ------------------------------------------------------------------------------------- */
int lpmm_selftest_arithmetic(unsigned long long *counts, uint32_t sqrt_stride, uint64_t pairs,
                             uint32_t seed, void *stream);

/* Diagnostic (no counterpart in the reference): runs the code assignment exactly as the kernels
 * run it (LDS tables, saturating byte conversion, byte permute, median-of-three clamp) against
 * the plain count of midpoints below x -- the reference search of
 * lpmm/cpp_extension/fused_adamw_kernel.cu:27-49 -- on the device.  counts: 10 zero-initialised
 * device uint64:
 *   [0] values tried with the standard first-moment map: all 2^32 bit patterns, NaNs included
 *   (they must give code 15), [1] wrong codes; [2], [3] the same with the standard
 *   second-moment map; [4] values <= 1 tried with the bare closed form of the second-moment
 *   code, [5] wrong codes; [6] values tried through the division by the group maximum with the
 *   first-moment map (256 maxima: both ends of the range that divides by the corrected
 *   reciprocal with their neighbours, zero, subnormal, huge, infinite, random; numerators
 *   within 128 floats of every midpoint * maximum and random), [7] wrong codes; [8], [9] the
 *   same with the second-moment map.  Every odd entry must stay 0. */
int lpmm_selftest_encoders(unsigned long long *counts, void *stream);

/* Diagnostic (no counterpart in the reference): builds the code table of a map as
 * lpmm_code_table_build does and runs the one-read code assignment against the search of
 * lpmm/cpp_extension/quantization_kernel.cu:397-427 as the library restates it, on the device, for
 * all 2^32 bit patterns of x (NaNs included).  qmap: 2^bits floats, 3 <= bits <= 8.  counts: 3
 * zero-initialised device uint64: [0] patterns tried, [1] codes that differ (must stay 0),
 * [2] 1 if the map qualifies for a table; for a map that does not, nothing is tried. */
int lpmm_selftest_bucket_encoder(const float *qmap, int bits, unsigned long long *counts, void *stream);

/* Diagnostic (no counterpart in the reference): streaming-rate calibration.  Kernels that move
 * bytes the way the fused 4-bit step moves them (256-thread workgroups, 2048-element tiles, the
 * same lane-to-address layout, nontemporal accesses, one-shot grid) with no arithmetic to speak
 * of, so that their rate is what the memory system gives to the access pattern itself:
 *   LPMM_PROBE_READ       a read                                   4 B/element
 *   LPMM_PROBE_WRITE      a written                                4 B/element
 *   LPMM_PROBE_COPY       a = b                                    8 B/element
 *   LPMM_PROBE_UPDATE     a += b in place (2 reads : 1 write)     12 B/element
 *   LPMM_PROBE_FUSED_MIX  the seven streams of lpmm_adamw4bit_step: a, b read, a written,
 *                         codes0/1 (n/2 bytes each) and scale0/1 (n/128 floats each) read and
 *                         written                                 14.125 B/element
 *   LPMM_PROBE_FUSED_MIX_DWORD  the same with one 4-byte code access per lane and state
 *                         instead of two 2-byte ones              14.125 B/element
 * kind = pattern | workgroup shape | tile order:
 *   LPMM_PROBE_SHAPE_256    256 threads on one 2048-element tile (the fused step's own shape; the default)
 *   LPMM_PROBE_SHAPE_512    512 threads on two adjacent tiles
 *   LPMM_PROBE_SHAPE_128    128 threads on half a tile
 *   LPMM_PROBE_SHAPE_256X2  256 threads that load two adjacent tiles before they store either
 *   LPMM_PROBE_RUN_ORDER    the workgroups take their spans so that every XCD streams 128 KB runs of a (the
 *                           fused step's tile order); without it workgroup i takes span i
 * n: a multiple of 4096; a, b: fp32[n], 16-byte aligned; code arrays 4-byte aligned.  lds_bytes (0..163840) of dynamic LDS
 * that the kernels never touch cap the workgroups resident per CU at floor(160 KB / lds_bytes)
 * (0: the hardware's own limit).  Buffers a pattern does not use may be NULL. */
enum {
    LPMM_PROBE_READ = 0, LPMM_PROBE_WRITE = 1, LPMM_PROBE_COPY = 2, LPMM_PROBE_UPDATE = 3, LPMM_PROBE_FUSED_MIX = 4,
    LPMM_PROBE_FUSED_MIX_DWORD = 5,
    LPMM_PROBE_SHAPE_256 = 0x000, LPMM_PROBE_SHAPE_512 = 0x100, LPMM_PROBE_SHAPE_128 = 0x200,
    LPMM_PROBE_SHAPE_256X2 = 0x300, LPMM_PROBE_SHAPE_MASK = 0x300,
    LPMM_PROBE_RUN_ORDER = 0x1000
};
int lpmm_stream_probe(int kind, float *a, const float *b, uint8_t *codes0, uint8_t *codes1, float *scale0,
                      float *scale1, int64_t n, int64_t lds_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LPMM_HIP_H */
