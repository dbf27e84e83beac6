// Shared by the two-pass rank-1 step kernels (nonfused_rank1.hip: 4-bit states, the tuned passes;
// nonfused_rank1_bits.hip: 5-8-bit states; nonfused_rank1_ragged.hip: column counts that are no
// multiple of 128): the tensor records of a launch, the tile geometry and small helpers.
#pragma once
#include "lpmm_update.hpp"

namespace lpmm {

constexpr int kThreads = 256;
constexpr int kEltsPerLane = 8;
constexpr int kDppRows = kThreads / 16;  // 128-column groups a workgroup handles per pass
constexpr int kR1Max = 32;               // tensors per launch
// Tile policy: widest tile (lg of 128-column groups), tensor rows per workgroup (more where one pass
// of a narrow tile covers more), workgroups taken to be resident together.
#ifndef LPMM_R1_LG
#define LPMM_R1_LG 1
#endif
#ifndef LPMM_R1_ROWS
#define LPMM_R1_ROWS 64
#endif
#ifndef LPMM_R1_RESIDENT
#define LPMM_R1_RESIDENT 256
#endif
constexpr int kPolicyLgWide = LPMM_R1_LG;
constexpr uint32_t kPolicyRows = LPMM_R1_ROWS, kPolicyResident = LPMM_R1_RESIDENT;
constexpr uint32_t kPolicyRowsM32 = LPMM_R1_ROWS / 2;  // fp32 first moment
static_assert(LPMM_R1_LG >= 1 && LPMM_R1_LG <= 3, "a tile is 256 to 1024 columns wide at most");
constexpr int kMaxLgWide = kPolicyLgWide;   // the LDS column arrays hold 128 << kMaxLgWide columns
constexpr int kMaxWide = 1 << kMaxLgWide;
// Per-column data of a tile lives in LDS, not in registers (occupancy): the current column
// statistics in the unused bytes between the maps and the encode table, further arrays after
// the table.
constexpr uint32_t kColBytes = kMaxWide * kGroup * 4;
constexpr uint32_t kColOld = kLdsQ1 + 64;
static_assert(kColOld + kColBytes <= kEncLdsBegin, "column statistics overlap the encode table");
constexpr uint32_t kColExtra = (kLdsBytes + 15) / 16 * 16;  // first byte after the table
// Column maxima of the tile, one slot of 8 x 16 words (+16 words of skew, so that the DPP rows
// of a wave hit different banks) per column group: word k * 16 + lane16 of a slot is element k
// of lane lane16.
constexpr uint32_t kRedSlotWords = kGroup + 16;

// A workgroup covers tile_rows rows x (128 << lg_wide) columns: per pass, (16 >> lg_wide) rows of
// (1 << lg_wide) adjacent groups each.
struct TileShape {
    uint32_t lg_wide : 8;
    uint32_t tile_rows : 24;  // max(the policy's rows, rows of one pass)
    uint32_t comb;            // row blocks whose passes interleave
};

struct TensorR1 {
    float *p;
    const float *g;
    uint8_t *mc;  // fp32 first moment: the moment itself (float[rows * cols]), ms unused
    float *ms;
    float *ms_new;  // first-moment groups wider than 128 values: the scales of the new first moment
    uint8_t *vc;
    const float *row_old;
    const float *col_old;
    float *row_new;
    float *col_new;
    int64_t rows;
    uint32_t col_blocks;  // columns / 128
    float neg_step_size, bc2_sqrt, rbc2_sqrt;
    uint32_t m_lg;  // the first moment's group holds 128 << m_lg values
    uint32_t col_tail;  // columns in the last 128-column block (128 unless the column count is ragged)
    TileShape tile;
};

// How the first moment is kept: 4-bit codes in groups of 128 values (re-quantised where it is
// updated), fp32 (read and written as floats), or 4-bit codes in wider groups (256 .. 4096
// values of the flattened tensor: a group spans several DPP rows, tiles and, where the column
// count is not a multiple of the group size, tensor rows.  The update pass only merges the
// groups' maxima into the next scales, the second pass recomputes the moment from g and the old
// codes, bit-identically, and writes its codes -- what both passes do for the second moment).
enum MomentMode { kMCodes128 = 0, kMFloat = 1, kMCodesWide = 2 };

struct MultiR1 {
    TensorR1 t[kR1Max];
    uint32_t tile_start[kR1Max + 1];  // prefix sum of tiles per tensor; unused slots hold the total
    int count;
    float decay, w1, b2, w2, eps;
};

static_assert(sizeof(MultiR1) + 3 * sizeof(void *) + 2 * sizeof(int) <= 4096, "kernel arguments exceed 4 KB");
static_assert(kR1Max <= kWave, "one tile_start entry per lane");

// tensor of this workgroup (uniform): the number of later tensors whose first tile is not
// after this one
__device__ __forceinline__ int find_tensor(const MultiR1 &args)
{
    const int lane = threadIdx.x & (kWave - 1);
    const bool started = lane + 1 < kR1Max && args.tile_start[lane + 1] <= blockIdx.x;
    return __popcll(__ballot(started));
}

__device__ __forceinline__ void unpack8(const float4 &a, const float4 &b, float (&o)[kEltsPerLane])
{
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}

// Where a DPP row of this workgroup works: column group `cg` (fixed), rows row0, row0 + step, ...
struct Geometry {
    int64_t row0;
    uint32_t cg, col_tile;
    int step, passes, wide;
};

__device__ __forceinline__ Geometry geometry(const TileShape &ts, uint32_t col_blocks, uint32_t tile, int drow)
{
    Geometry q;
    q.wide = 1 << ts.lg_wide;
    const uint32_t col_tiles = (col_blocks + q.wide - 1) >> ts.lg_wide;
    const uint32_t rb = tile / col_tiles;
    q.col_tile = tile - rb * col_tiles;
    q.cg = q.col_tile * q.wide + (drow & (q.wide - 1));
    const int pass_rows = kDppRows >> ts.lg_wide;
    q.passes = (int)ts.tile_rows / pass_rows;
    // block k of group grp: pass i covers the rows from (grp * passes * comb + i * comb + k) * pass_rows on
    const uint32_t grp = rb / ts.comb, k = rb - grp * ts.comb;
    q.row0 = (int64_t)grp * ts.tile_rows * ts.comb + (int64_t)k * pass_rows + (drow >> ts.lg_wide);
    q.step = pass_rows * (int)ts.comb;
    return q;
}

__device__ __forceinline__ Geometry geometry(const TensorR1 &t, uint32_t tile, int drow)
{
    return geometry(t.tile, t.col_blocks, tile, drow);
}

// Folded rows.  A tensor of R x C values with C = 64 modulo 128 and R even is the same memory as
// the row-major matrix of R / 2 double rows of 2 C values, and 2 C is a multiple of 128: the
// 128-value groups of the first moment, cut from the flattened tensor (lpmm/functional.py:404-422),
// never straddle a double row, so the kernels for whole column blocks apply to that matrix (GPT-2-XL's
// d = 1600 and 3 d = 4800).  What changes is where a value's statistics sit: a DPP row's 128 values
// are two halves of 64 (a lane's first and second run of four), half h of column block cg of double
// row r lies in tensor row 2 r + (128 cg + 64 h >= C) at column (128 cg + 64 h) mod C.  The record
// keeps the tensor's own shape (col_blocks = ceil(C / 128), col_tail = 64); kernels instantiated
// with FOLD read it this way, tensors with whole column blocks in the same launch as before.
struct Fold {
    bool on;
    uint32_t real_cols, col_blocks;  // columns of the tensor; column blocks of the matrix the kernel works on
    int64_t rows;                    // rows of that matrix
};

template <bool FOLD>
__device__ __forceinline__ Fold fold_of(const TensorR1 &t)
{
    Fold f;
    f.on = FOLD && t.col_tail != (uint32_t)kGroup;
    f.real_cols = (t.col_blocks - 1) * kGroup + t.col_tail;
    f.col_blocks = f.on ? 2 * t.col_blocks - 1 : t.col_blocks;
    f.rows = f.on ? t.rows >> 1 : t.rows;
    return f;
}

// column of the tensor for column c of the matrix (c < 2 C)
__device__ __forceinline__ uint32_t fold_col(const Fold &f, uint32_t c) { return c >= f.real_cols ? c - f.real_cols : c; }

// tensor rows of the two halves of column block cg in row r of the matrix
__device__ __forceinline__ void fold_rows(const Fold &f, int64_t r, uint32_t cg, int64_t &r0, int64_t &r1)
{
    if (f.on) {
        r0 = 2 * r + (cg * kGroup >= f.real_cols ? 1 : 0);
        r1 = 2 * r + (cg * kGroup + 64 >= f.real_cols ? 1 : 0);
    } else {
        r0 = r1 = r;
    }
}

// Row maxima of a tile.  An atomic maximum on global memory goes out to the fabric (the L2s of
// the XCDs are not coherent with each other), and the passes of a tile produce one per tensor row,
// column group and pass: 0.008 per element, a tenth of the first pass's DRAM transactions together
// with its partial writes.  So the maxima of a tile's rows meet in LDS first -- slot 2 * (row of
// the tile) + (tensor row of a double row: folded rows only) -- and one global atomic per row and
// tile follows the passes, issued by neighbouring threads for neighbouring rows (LLaMA-7B-shaped
// set 21.23 -> 20.85 ms per step, GPT-2-XL-shaped set 6.30 -> 5.71 ms).
constexpr int kRowSlots = 2 * (int)kPolicyRows;
static_assert(kRowSlots <= kThreads, "one thread per row slot");
static_assert(kPolicyRows >= (uint32_t)kDppRows, "a tile holds the policy's rows: one slot pair per row");

__device__ __forceinline__ int row_slot(const TileShape &ts, int pass, int drow)
{
    return 2 * (pass * (kDppRows >> ts.lg_wide) + (drow >> ts.lg_wide));
}

// after the passes and a barrier: rows = rows of the matrix the tile works on; fold: its rows are double rows
__device__ __forceinline__ void flush_row_maxima(const uint32_t *rowred, const TileShape &ts, const Geometry &q, int drow,
                                                 int64_t rows, bool fold, float *__restrict__ row_new)
{
    if (threadIdx.x >= (uint32_t)kRowSlots)
        return;
    const int pr = kDppRows >> ts.lg_wide;
    const int local = threadIdx.x >> 1, half = threadIdx.x & 1;
    const int pass = local / pr, in_pass = local - pass * pr;
    // the first row of the tile's first pass: row0 of this thread's DPP row less its place in the pass
    const int64_t r = (q.row0 - (drow >> ts.lg_wide)) + (int64_t)pass * q.step + in_pass;
    if (pass < q.passes && r < rows && (half == 0 || fold))
        atomic_max_nonneg(row_new + (fold ? 2 * r + half : r), __uint_as_float(rowred[threadIdx.x]));
}

// Codes of a plain 0.0 into the padding [n, n_padded) of a packed array and 0 into the extra
// last byte; one workgroup.  n and n_padded are multiples of 8, the array is 4-byte aligned.
__device__ __forceinline__ void write_padding(uint8_t *codes, int64_t n, int64_t n_padded, uint32_t zero_word)
{
    for (int64_t i = n + (int64_t)threadIdx.x * kEltsPerLane; i < n_padded; i += kThreads * kEltsPerLane)
        *reinterpret_cast<uint32_t *>(codes + (i >> 1)) = zero_word;
    if (threadIdx.x == 0)
        codes[n_padded / 2] = 0;
}

// The launches of the other kernel families (defined next to their kernels); tiles = workgroups.
void launch_rank1_bits(const MultiR1 &args, uint32_t tiles, const float *qmap_m, const float *qmap_v, int bits_m,
                       int bits_v, const uint32_t *table_m, const uint32_t *table_v, hipStream_t stream);
void launch_rank1_ragged(const MultiR1 &args, uint32_t tiles, const float *qmap_m, const float *qmap_v,
                         hipStream_t stream);
// float16 parameters (nonfused_half.hip): p, g, the first moment's scales and the current statistics
// of the records point at halfs, the next statistics at float work arrays
void launch_rank1_half(const MultiR1 &args, uint32_t tiles, const float *qmap_m, const float *qmap_v, hipStream_t stream);
int rank1_step_multi_half(const lpmm_nonfused_rank1_tensor *tensors, int64_t count, const float *qmap_m,
                          const float *qmap_v, double beta1, double beta2, double lr, double weight_decay, double eps,
                          void *stream);

}  // namespace lpmm
