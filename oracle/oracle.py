"""ctypes/numpy front end of the CPU oracle (oracle/lpmm_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker.  The shipped package never imports it.

All arrays are C-contiguous numpy arrays; "in place" functions mutate their arguments
exactly like the reference's kernels mutate the tensors they are given.

Functions restated here in numpy rather than in C, and what pins them (tests/test_oracle_*.py):
  adamw_fp16_step     the float step of the C oracle on inputs exactly representable in half, and a
                      float16 round trip of it operation by operation (moments re-read after rounding).
  rank1_*_nd          on a 2-D tensor the 2-D C functions bit for bit; on 3-D/4-D tensors the
                      reference's op sequence run by PyTorch's CPU kernels and a loop over all indices.
  *_f16               float16 scaling around the C search: each op in float with one rounding to half
                      (numpy.float16 arithmetic), against the same ops of PyTorch's CPU half kernels
                      bit for bit (codes, scales, statistics and three whole steps).
  map construction    the bit patterns the reference's recipe gives when PyTorch's ops run it
                      (tests/golden/qmaps.json).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblpmm_oracle.so")

GROUP = 128
PACK_GROUP = 2048


def build(force=False):
    """Compile oracle/lpmm_oracle.c with the committed Makefile."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "liblpmm_oracle.so"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    return lib


_lib = _load()

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")
_i64 = ctypes.c_int64
_f = ctypes.c_float
_d = ctypes.c_double


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_qmapping = _sig("lpmm_oracle_qmapping", ctypes.c_int, _f32p, ctypes.c_int, _f)
_qmapping_many = _sig("lpmm_oracle_qmapping_many", None, _f32p, _f32p, _i64, _u8p)
_pack = _sig("lpmm_oracle_pack_nonlinear_4bit", None, _f32p, _f32p, _i64, _u8p)
_unpack = _sig("lpmm_oracle_unpack_nonlinear_4bit", None, _u8p, _f32p, _i64, _f32p)
_pack_bits = _sig("lpmm_oracle_pack_nonlinear", None, _f32p, _f32p, ctypes.c_int, _i64, _u8p)
_unpack_bits = _sig("lpmm_oracle_unpack_nonlinear", None, _u8p, _f32p, ctypes.c_int, _i64, _f32p)
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")
_u64 = ctypes.c_uint64
_philox = _sig("lpmm_oracle_philox4x32_10", None, _u32p, _u32p, _u32p)
_philox_draw = _sig("lpmm_oracle_philox_draw", ctypes.c_uint32, _u64, _u64, _u64, _u64)
_philox_uniform = _sig("lpmm_oracle_philox_uniform", _f, _u64, _u64, _u64, _u64)
_qmapping_sr = _sig("lpmm_oracle_qmapping_sr", ctypes.c_int, _f32p, ctypes.c_int, _f, _f)
_pack_sr = _sig("lpmm_oracle_pack_nonlinear_sr", None, _f32p, _f32p, ctypes.c_int, _i64, _u64, _u64, _u8p)
_adamw_fp32 = _sig("lpmm_oracle_adamw_fp32_step", None, _f32p, _f32p, _f32p, _f32p, _i64,
                   _f, _f, _f, _f, _f, _f)
_adamw4bit = _sig("lpmm_oracle_adamw4bit_step", None, _f32p, _f32p, _u8p, _u8p, _f32p, _f32p,
                  _f32p, _f32p, _i64, _f, _f, _f, _f, _f, _f)
_quant_group = _sig("lpmm_oracle_quant_group", None, _f32p, _i64, _i64, _f32p, _u8p, _f32p)
_dequant_group = _sig("lpmm_oracle_dequant_group", None, _u8p, _f32p, _f32p, _i64, _i64, _f32p)
_rank1_stats = _sig("lpmm_oracle_rank1_stats", None, _f32p, _i64, _i64, _f32p, _f32p)
_quant_rank1 = _sig("lpmm_oracle_quant_rank1", None, _f32p, _i64, _i64, _f32p, _f32p, _f32p, _u8p)
_dequant_rank1 = _sig("lpmm_oracle_dequant_rank1", None, _u8p, _f32p, _f32p, _f32p, _i64, _i64,
                      _f32p)
_nonfused_update = _sig("lpmm_oracle_nonfused_update", None, _f32p, _f32p, _f32p, _f32p, _i64,
                        _d, _d, _d, _d, _d, _d)
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_nonfused_update_f16 = _sig("lpmm_oracle_nonfused_update_f16", None, _u16p, _u16p, _u16p, _u16p, _i64,
                            _d, _d, _d, _d, _d, _d)
_adamw4bit_f16 = _sig("lpmm_oracle_adamw4bit_step_f16", None, _u16p, _u16p, _u8p, _u8p, _u16p, _u16p,
                      _f32p, _f32p, _i64, _f, _f, _f, _f, _f, _f)
_f16_to_f32 = _sig("lpmm_oracle_f16_to_f32", None, _u16p, _f32p, _i64)
_f32_to_f16 = _sig("lpmm_oracle_f32_to_f16", None, _f32p, _u16p, _i64)
_sgd_update = _sig("lpmm_oracle_sgd_update", None, _f32p, _f32p, _f32p, _i64, _d, _d, _d, _d, ctypes.c_int,
                   ctypes.c_int, ctypes.c_int)
_factored_stats = _sig("lpmm_oracle_factored_stats", None, _f32p, _i64, _i64, _f32p, _f32p)
_factored_ema = _sig("lpmm_oracle_factored_ema", _f, _f32p, _f32p, _f32p, _f32p, _i64, _i64, _d)
_factored_update = _sig("lpmm_oracle_factored_update", None, _f32p, _f32p, _f32p, _f32p, _f32p,
                        _f, _i64, _i64, _d, _d, _d, _d, _d, _d)
_max_threads = _sig("lpmm_oracle_max_threads", ctypes.c_int)
_set_threads = _sig("lpmm_oracle_set_threads", None, ctypes.c_int)


def max_threads():
    return int(_max_threads())


def set_threads(n):
    _set_threads(int(n))


# --------------------------------------------------------------------------------------
# Quantisation maps.  lpmm/functional.py:244-268 (create_general_qmap), :272-315
# (create_dynamic_map), :644-656 (create_pow_map).
# --------------------------------------------------------------------------------------
def _linspace_f32(start, end, steps):
    """torch.linspace for float32 on CPU, scalar formula: step = (end-start)/(steps-1) in
    float32; the first half counts up from start, the second half counts down from end.
    PyTorch's vectorised path (grids of 8 or more points) rounds differently; the 4-bit maps
    only use grids of 2, 3 and 5 points, and the 17-point grid of the v map is exact."""
    f = np.float32
    start, end = f(start), f(end)
    if steps == 1:
        return np.array([start], dtype=f)
    step = f((end - start) / f(steps - 1))
    out = np.empty(steps, dtype=f)
    half = steps // 2
    for i in range(steps):
        if i < half:
            out[i] = f(start + f(step * f(i)))
        else:
            out[i] = f(end - f(step * f(steps - i - 1)))
    return out


def create_dynamic_map(signed=True, max_exponent_bits=3, total_bits=4):
    """lpmm/functional.py:272-315.  The float32 means are scaled by the float32-cast power
    of ten (tensor * python scalar), widened to double by .tolist(), sorted, and narrowed
    back to float32 by torch.Tensor(data)."""
    f = np.float32
    data = []
    non_sign_bits = total_bits - (1 if signed else 0)
    additional_items = 2 ** (non_sign_bits - max_exponent_bits) - 1
    if not signed:
        additional_items = 2 * additional_items
    for i in range(max_exponent_bits):
        if signed:
            fraction_items = int(2 ** (i + non_sign_bits - max_exponent_bits) + 1)
        else:
            fraction_items = int(2 ** (i + non_sign_bits - max_exponent_bits + 1) + 1)
        scale = f(10 ** (-(max_exponent_bits - 1) + i))
        b = _linspace_f32(0.1, 1, fraction_items)
        means = ((b[:-1] + b[1:]) / f(2.0)).astype(f)
        data += [float(v) for v in (scale * means).astype(f)]
        if signed:
            data += [float(v) for v in (f(-scale) * means).astype(f)]
        if additional_items > 0:
            b = _linspace_f32(0.1, 1, additional_items + 1)
            means = ((b[:-1] + b[1:]) / f(2.0)).astype(f)
            data += [float(v) for v in (scale * means).astype(f)]
            if signed:
                data += [float(v) for v in (f(-scale) * means).astype(f)]
    data.append(0.0)
    data.append(1.0)
    data.sort()
    return np.array(data, dtype=np.float32)


def create_pow_map(b=4, signed=False, p=1):
    """lpmm/functional.py:644-656 (the 'no zero' versions)."""
    f = np.float32
    if signed:
        q = _linspace_f32(-1, 1, 2 ** b)
        if p != 1:
            q = (np.sign(q) * np.abs(q) ** f(p)).astype(f)
    else:
        q = _linspace_f32(0, 1, 2 ** b + 1)[1:]
        if p != 1:
            q = (q ** f(p)).astype(f)
    return np.ascontiguousarray(q, dtype=f)


def qmap_m():
    """First-moment map: create_general_qmap('nonlinear', 4, True) (functional.py:250-251)."""
    return create_dynamic_map(True, 3, 4)


def qmap_v():
    """Second-moment map: create_general_qmap('power-1', 4, False) (functional.py:257-258)."""
    return create_pow_map(4, False, 1)


def midpoints(qmap):
    q = np.asarray(qmap, dtype=np.float32)
    return ((q[:-1] + q[1:]) * np.float32(0.5)).astype(np.float32)


# --------------------------------------------------------------------------------------
# thin wrappers
# --------------------------------------------------------------------------------------
def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def qmapping_scalar(qmap, x, bits=4):
    """The reference's int return value (-1 for NaN)."""
    return int(_qmapping(_c(qmap, np.float32), bits, float(np.float32(x))))


def qmapping(qmap, x):
    x = _c(x, np.float32).reshape(-1)
    out = np.empty(x.size, dtype=np.uint8)
    _qmapping_many(_c(qmap, np.float32), x, x.size, out)
    return out


def pack_nonlinear_4bit(x, qmap):
    x = _c(x, np.float32).reshape(-1)
    assert x.size % 8 == 0
    out = np.empty(x.size // 2 + 1, dtype=np.uint8)
    _pack(x, _c(qmap, np.float32), x.size, out)
    return out


def unpack_nonlinear_4bit(codes, qmap, n):
    out = np.empty(n, dtype=np.float32)
    _unpack(_c(codes, np.uint8), _c(qmap, np.float32), n, out)
    return out


def storage_bits(bits):
    """quantization_kernel.cu:592-601: widths 1, 2, 4 are packed, the others take a byte."""
    return bits if bits in (1, 2, 4) else 8


def pack_nonlinear(x, qmap, bits):
    """Codes of already-normalised values, any width; x.size a multiple of 8."""
    x = _c(x, np.float32).reshape(-1)
    assert x.size % 8 == 0 and len(qmap) == 2 ** bits
    out = np.empty(x.size * storage_bits(bits) // 8 + 1, dtype=np.uint8)
    _pack_bits(x, _c(qmap, np.float32), bits, x.size, out)
    return out


def philox4x32_10(ctr, key):
    """One Philox4x32-10 block: ctr 4 words, key 2 words -> 4 words."""
    out = np.empty(4, np.uint32)
    _philox(_c(ctr, np.uint32), _c(key, np.uint32), out)
    return out


def philox_draw(seed, subsequence, offset, j):
    """32-bit output number j of the state curand_init(seed, subsequence, offset) gives."""
    return int(_philox_draw(seed, subsequence, offset, j))


def philox_uniform(seed, subsequence, offset, j):
    """curand_uniform of that output: u * 2^-32 + 2^-33 in float, (0, 1]."""
    return float(_philox_uniform(seed, subsequence, offset, j))


def qmapping_sr(qmap, x, noise, bits=4):
    """quantize_bsearch<true>: the int the reference returns (-1 for NaN)."""
    return int(_qmapping_sr(_c(qmap, np.float32), bits, x, noise))


def pack_nonlinear_sr(x, qmap, bits, seed, offset):
    """pack_nonlinear(..., stochastic=True) with the Philox stream (seed, offset)."""
    x = _c(x, np.float32).reshape(-1)
    assert x.size % 32 == 0 and len(qmap) == 2 ** bits
    out = np.empty(x.size * storage_bits(bits) // 8 + 1, dtype=np.uint8)
    _pack_sr(x, _c(qmap, np.float32), bits, x.size, seed, offset, out)
    return out


def unpack_nonlinear(codes, qmap, bits, n):
    out = np.empty(n, dtype=np.float32)
    _unpack_bits(_c(codes, np.uint8), _c(qmap, np.float32), bits, n, out)
    return out


def _pad_to(x, multiple):
    rem = (-x.size) % multiple
    return np.concatenate([x, np.zeros(rem, x.dtype)]) if rem else x


def quant_group_bits(x, qmap, bits, gp_sz=GROUP):
    """vectorwise_quant with 'group' scaling for any width, composed as the reference composes
    it (lpmm/functional.py:184-189, :404-422, :359-369): zero-pad to whole groups, max|x| per
    group, true division (0/0 -> NaN), zero-pad to whole 2048-value pack groups, pack."""
    x = _c(x, np.float32).reshape(-1)
    grouped = _pad_to(x, gp_sz).reshape(-1, gp_sz)
    max1 = np.abs(grouped).max(axis=1).astype(np.float32)
    with np.errstate(invalid="ignore", divide="ignore"):
        normed = (grouped / max1[:, None]).astype(np.float32).reshape(-1)
    return pack_nonlinear(_pad_to(normed, PACK_GROUP), qmap, bits), max1


def dequant_group_bits(codes, max1, qmap, bits, n, gp_sz=GROUP):
    """lpmm/functional.py:393-400, :115-118."""
    g = max1.size
    vals = unpack_nonlinear(codes, qmap, bits, g * gp_sz).reshape(g, gp_sz)
    return (vals * _c(max1, np.float32).reshape(-1, 1)).astype(np.float32).reshape(-1)[:n]


def quant_rank1_bits(x, rowmax, colmax, qmap, bits):
    """lpmm/functional.py:190-203, :503-509 for any width."""
    x = _c(x, np.float32)
    st = np.where(colmax[None, :] < rowmax[:, None], colmax[None, :], rowmax[:, None]).astype(np.float32)
    with np.errstate(invalid="ignore", divide="ignore"):
        normed = (x / st).astype(np.float32).reshape(-1)
    return pack_nonlinear(_pad_to(normed, PACK_GROUP), qmap, bits)


def dequant_rank1_bits(codes, rowmax, colmax, qmap, bits, r, c):
    st = np.where(colmax[None, :] < rowmax[:, None], colmax[None, :], rowmax[:, None]).astype(np.float32)
    return (unpack_nonlinear(codes, qmap, bits, r * c).reshape(r, c) * st).astype(np.float32)


def rank1_stats_nd(x):
    """get_sm3_statistics (lpmm/functional.py:512-531) for any number of dimensions: for each
    dimension the maximum of |x| over all the others, as 1-D arrays."""
    a = np.abs(_c(x, np.float32))
    return [a.max(axis=tuple(j for j in range(a.ndim) if j != i)).astype(np.float32) for i in range(a.ndim)]


def rank1_scale_nd(stats, shape):
    """_compute_sm3_scale_tensor (lpmm/functional.py:503-509): the statistics broadcast to the
    tensor's shape and folded with an elementwise minimum, dimension 0 first; torch.min returns NaN
    where either operand is NaN, as numpy.minimum does."""
    scale = None
    for i, st in enumerate(stats):
        keep = [1] * len(shape)
        keep[i] = shape[i]
        other = np.broadcast_to(_c(st, np.float32).reshape(keep), shape)
        scale = other if scale is None else np.minimum(scale, other)
    return np.ascontiguousarray(scale, dtype=np.float32)


def quant_rank1_nd_bits(x, stats, qmap, bits):
    """lpmm/functional.py:190-203 + :359-369 for a tensor of any number of dimensions."""
    x = _c(x, np.float32)
    with np.errstate(invalid="ignore", divide="ignore"):
        normed = (x / rank1_scale_nd(stats, x.shape)).astype(np.float32).reshape(-1)
    return pack_nonlinear(_pad_to(normed, PACK_GROUP), qmap, bits)


def dequant_rank1_nd_bits(codes, stats, qmap, bits, shape):
    """lpmm/functional.py:97-106 for a tensor of any number of dimensions."""
    n = int(np.prod(shape))
    return (unpack_nonlinear(codes, qmap, bits, n).reshape(shape) * rank1_scale_nd(stats, shape)).astype(np.float32)


def adamw_fp32_step(p, g, m, v, beta1, beta2, lr, wd, eps, step):
    _adamw_fp32(p, g, m, v, p.size, beta1, beta2, lr, wd, eps, step)


_libm = ctypes.CDLL("libm.so.6")
_libm.powf.restype = ctypes.c_float
_libm.powf.argtypes = [ctypes.c_float, ctypes.c_float]


def _powf(a, b):
    return np.float32(_libm.powf(float(a), float(b)))


def adamw_fp16_step(p, g, m, v, beta1, beta2, lr, wd, eps, step):
    """adamw_cuda_kernel<at::Half> (lpmm/cpp_extension/fused_adamw_kernel.cu:52-78, instantiated by
    the dispatch at :188) on float16 arrays, in place.  c10::Half converts to float for every
    arithmetic operator and rounds to nearest even on assignment, so: the moments are formed in
    float and stored as half (:66-67); the update reads them back *after* that rounding (:72-73),
    runs in float with the float scalars of the fp32 step, and the parameter is rounded to half on
    its store (:74).  numpy float32 arithmetic rounds every operation once, like the kernel built
    without contraction."""
    f = np.float32
    assert p.dtype == g.dtype == m.dtype == v.dtype == np.float16
    b1, b2, lr_, wd_, eps_, st = f(beta1), f(beta2), f(lr), f(wd), f(eps), f(step)
    omb1, omb2 = f(1) - b1, f(1) - b2
    gf, pf = g.astype(f), p.astype(f)
    m[...] = (b1 * m.astype(f) + omb1 * gf).astype(np.float16)
    v[...] = (b2 * v.astype(f) + (omb2 * gf) * gf).astype(np.float16)
    c1 = f(1) - _powf(b1, st)  # the C library's powf, as in the C restatement of the fp32 step
    c2s = np.sqrt(f(1) - _powf(b2, st), dtype=f)
    denom = (np.sqrt(v.astype(f), dtype=f) / c2s + eps_) * c1
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        update = m.astype(f) / denom + wd_ * pf
        p[...] = (pf - lr_ * update).astype(np.float16)


def adamw4bit_step(p, g, m_codes, v_codes, m_scale, v_scale, qm, qv, beta1, beta2, lr, wd, eps,
                   step):
    n = p.size
    assert g.size == n and m_codes.size == (n + 1) // 2 and v_codes.size == (n + 1) // 2
    assert m_scale.size == (n + GROUP - 1) // GROUP and v_scale.size == m_scale.size
    _adamw4bit(p, g, m_codes, v_codes, m_scale, v_scale, _c(qm, np.float32), _c(qv, np.float32), n,
               beta1, beta2, lr, wd, eps, step)


def packed_nbytes_nonfused(n, gp_sz=GROUP):
    g = (n + gp_sz - 1) // gp_sz
    ng = (g * gp_sz + PACK_GROUP - 1) // PACK_GROUP
    return ng * (PACK_GROUP // 2) + 1


def quant_group(x, qmap, gp_sz=GROUP):
    x = _c(x, np.float32).reshape(-1)
    n = x.size
    g = (n + gp_sz - 1) // gp_sz
    codes = np.empty(packed_nbytes_nonfused(n, gp_sz), dtype=np.uint8)
    max1 = np.empty(g, dtype=np.float32)
    _quant_group(x, n, gp_sz, _c(qmap, np.float32), codes, max1)
    return codes, max1


def dequant_group(codes, max1, qmap, n, gp_sz=GROUP):
    out = np.empty(n, dtype=np.float32)
    _dequant_group(_c(codes, np.uint8), _c(max1, np.float32).reshape(-1), _c(qmap, np.float32), n,
                   gp_sz, out)
    return out


def rank1_stats(x):
    x = _c(x, np.float32)
    r, c = x.shape
    rowmax = np.empty(r, dtype=np.float32)
    colmax = np.empty(c, dtype=np.float32)
    _rank1_stats(x, r, c, rowmax, colmax)
    return rowmax, colmax


def quant_rank1(x, rowmax, colmax, qmap):
    x = _c(x, np.float32)
    r, c = x.shape
    codes = np.empty(packed_nbytes_nonfused(r * c, 1), dtype=np.uint8)
    _quant_rank1(x, r, c, rowmax, colmax, _c(qmap, np.float32), codes)
    return codes


def dequant_rank1(codes, rowmax, colmax, qmap, r, c):
    out = np.empty((r, c), dtype=np.float32)
    _dequant_rank1(_c(codes, np.uint8), rowmax, colmax, _c(qmap, np.float32), r, c, out)
    return out


def nonfused_update(p, g, m, v, beta1, beta2, lr, wd, eps, step):
    _nonfused_update(p, g, m, v, p.size, beta1, beta2, lr, wd, eps, step)


def sgd_update(p, g, buf, momentum, dampening, lr, wd, nesterov, maximize, first_step):
    """Elementwise part of _single_tensor_sgd4bit (lpmm/optim/sgd.py:133-187) on fp32 buffers, in place."""
    _sgd_update(p, g, buf, p.size, momentum, dampening, lr, wd, int(bool(nesterov)), int(bool(maximize)),
                int(bool(first_step)))


def factored_stats(g):
    r, c = g.shape
    row_mean = np.empty(r, dtype=np.float32)
    col_mean = np.empty(c, dtype=np.float32)
    _factored_stats(g, r, c, row_mean, col_mean)
    return row_mean, col_mean


def factored_ema(row, col, row_mean, col_mean, beta2):
    return float(_factored_ema(row, col, row_mean, col_mean, row.size, col.size, beta2))


def factored_update(p, g, m, row, col, row_mean_all, beta1, beta2, lr, wd, eps, step):
    r, c = p.shape
    _factored_update(p, g, m, row, col, row_mean_all, r, c, beta1, beta2, lr, wd, eps, step)


# --------------------------------------------------------------------------------------
# Whole non-fused steps on one tensor, composed from the pieces above the way
# lpmm/optim/adamw.py:332-436 and :579-627 compose them.
# --------------------------------------------------------------------------------------
class NonFusedState:
    """Optimizer state of one tensor in the non-fused layout (adamw.py:119-129,
    functional.py:32-34, :240): packed codes of NG*1024+1 bytes plus max1 (G,) for 'group'
    scaling, (rowmax, colmax) for 'rank1' on a 2-D tensor, (codes, [stat_0, ...]) for 'rank1' on
    a tensor of more dimensions."""

    def __init__(self, shape, v_scale_type="group", factored=False, bits=4):
        self.bits = bits  # code width of both moments (lpmm/configs/default_{5,6,7,8}b.yml)
        self.shape = tuple(shape)
        self.n = int(np.prod(self.shape))
        self.step = 0
        self.v_scale_type = v_scale_type
        self.factored = factored and len(self.shape) >= 2
        self.m = None  # (codes, max1)
        self.v = None  # (codes, max1) or (codes, rowmax, colmax)
        if self.factored:
            self.row = np.zeros(self.shape[0], dtype=np.float32)
            self.col = np.zeros(self.shape[1], dtype=np.float32)


def _v_is_rank1(state):
    return state.v_scale_type == "rank1" and len(state.shape) >= 2


def nonfused_step(p, g, state, qm, qv, lr, beta1, beta2, eps, wd):
    """One step of _single_tensor_adamw4bit on one quantised tensor.  p is updated in place."""
    state.step += 1
    n = state.n
    pf, gf = p.reshape(-1), np.ascontiguousarray(g, dtype=np.float32).reshape(-1)
    if state.factored:
        return _factored_step(p, g, state, qm, lr, beta1, beta2, eps, wd)
    b = state.bits
    if b == 4:
        deq_g = lambda s, q: dequant_group(s[0], s[1], q, n)
        deq_r = lambda s, q, r, c: dequant_rank1(s[0], s[1], s[2], q, r, c)
        q_g = quant_group
        q_r = quant_rank1
    else:
        deq_g = lambda s, q: dequant_group_bits(s[0], s[1], q, b, n)
        deq_r = lambda s, q, r, c: dequant_rank1_bits(s[0], s[1], s[2], q, b, r, c)
        q_g = lambda x, q: quant_group_bits(x, q, b)
        q_r = lambda x, rm, cm, q: quant_rank1_bits(x, rm, cm, q, b)
    m = np.zeros(n, np.float32) if state.m is None else deq_g(state.m, qm)
    if state.v is None:
        v = np.zeros(n, np.float32)
    elif _v_is_rank1(state) and len(state.shape) > 2:
        v = dequant_rank1_nd_bits(state.v[0], state.v[1], qv, b, state.shape).reshape(-1)
    elif _v_is_rank1(state):
        r, c = state.shape
        v = np.ascontiguousarray(deq_r(state.v, qv, r, c)).reshape(-1)
    else:
        v = deq_g(state.v, qv)
    nonfused_update(pf, gf, m, v, beta1, beta2, lr, wd, eps, float(state.step))
    state.m = q_g(m, qm)
    if _v_is_rank1(state) and len(state.shape) > 2:
        vn = v.reshape(state.shape)
        stats = rank1_stats_nd(vn)
        state.v = (quant_rank1_nd_bits(vn, stats, qv, b), stats)
    elif _v_is_rank1(state):
        r, c = state.shape
        v2 = v.reshape(r, c)
        rowmax, colmax = rank1_stats(v2)
        state.v = (q_r(v2, rowmax, colmax, qv), rowmax, colmax)
    else:
        state.v = q_g(v, qv)
    return m, v


def _factored_step(p, g, state, qm, lr, beta1, beta2, eps, wd):
    n = state.n
    r, c = state.shape
    g2 = np.ascontiguousarray(g, dtype=np.float32).reshape(r, c)
    m = np.zeros(n, np.float32) if state.m is None else dequant_group(state.m[0], state.m[1], qm, n)
    row_mean, col_mean = factored_stats(g2)
    mean_all = factored_ema(state.row, state.col, row_mean, col_mean, beta2)
    factored_update(p.reshape(r, c), g2, m, state.row, state.col, mean_all, beta1, beta2, lr, wd,
                    eps, float(state.step))
    state.m = quant_group(m, qm)
    return m, None


# --------------------------------------------------------------------------------------
# float16 parameters on the non-fused path: the reference's chain runs PyTorch's half kernels
# (lpmm/optim/adamw.py:394-434, lpmm/functional.py:184-203, :97-118).  Every op converts to float,
# computes and rounds to half once; states, scales and statistics are float16; the pack kernel
# widens each normalised (half) value to float before the search
# (lpmm/cpp_extension/quantization_kernel.cu:450); the unpacked map values are float32, their
# product with the float16 scale is float32 (type promotion) and takes the state's type last
# (lpmm/functional.py:150).
# --------------------------------------------------------------------------------------
f16 = np.float16


def f16_to_f32(h):
    h = _c(h, np.float16).reshape(-1)
    out = np.empty(h.size, np.float32)
    _f16_to_f32(h.view(np.uint16), out, h.size)
    return out


def f32_to_f16(x):
    x = _c(x, np.float32).reshape(-1)
    out = np.empty(x.size, np.uint16)
    _f32_to_f16(x, out, x.size)
    return out.view(np.float16)


def nonfused_update_f16(p, g, m, v, beta1, beta2, lr, wd, eps, step):
    """Elementwise part of the step on float16 arrays, in place."""
    for a in (p, g, m, v):
        assert a.dtype == np.float16 and a.flags.c_contiguous
    _nonfused_update_f16(p.reshape(-1).view(np.uint16), g.reshape(-1).view(np.uint16), m.reshape(-1).view(np.uint16),
                         v.reshape(-1).view(np.uint16), p.size, beta1, beta2, lr, wd, eps, step)


def _pack_padded(normed16, qmap):
    """functional.py:361-363 on half values: widen, zero-pad to whole pack groups, search, pack."""
    return pack_nonlinear_4bit(_pad_to(normed16.astype(np.float32).reshape(-1), PACK_GROUP), qmap)


def quant_group_f16(x, qmap, gp_sz=GROUP):
    """functional.py:184-189 then :359-369 on a float16 tensor: (codes, float16 max1 of G values)."""
    grouped = _pad_to(_c(x, np.float16).reshape(-1), gp_sz).reshape(-1, gp_sz)
    max1 = np.abs(grouped).max(axis=1)
    with np.errstate(invalid="ignore", divide="ignore"):
        normed = (grouped.astype(np.float32) / max1.astype(np.float32)[:, None]).astype(np.float16)
    return _pack_padded(normed, qmap), max1


def dequant_group_f16(codes, max1, qmap, n, gp_sz=GROUP):
    """functional.py:393-400, :115-118, :150: float32 map value times float16 scale, in float, then to half."""
    g = max1.size
    vals = unpack_nonlinear_4bit(codes, qmap, g * gp_sz).reshape(g, gp_sz)
    return (vals * _c(max1, np.float16).reshape(-1, 1).astype(np.float32)).astype(np.float16).reshape(-1)[:n]


def rank1_stats_f16(x):
    a = np.abs(_c(x, np.float16))
    return a.max(axis=1), a.max(axis=0)


def _rank1_scale_f16(rowmax, colmax):
    r, c = rowmax.astype(np.float32), colmax.astype(np.float32)
    return np.where(c[None, :] < r[:, None], c[None, :], r[:, None])


def quant_rank1_f16(x, rowmax, colmax, qmap):
    """functional.py:190-203 on a float16 matrix."""
    x = _c(x, np.float16)
    with np.errstate(invalid="ignore", divide="ignore"):
        normed = (x.astype(np.float32) / _rank1_scale_f16(rowmax, colmax)).astype(np.float16)
    return _pack_padded(normed, qmap)


def dequant_rank1_f16(codes, rowmax, colmax, qmap, r, c):
    vals = unpack_nonlinear_4bit(codes, qmap, (r * c + 7) // 8 * 8)[: r * c].reshape(r, c)
    return (vals * _rank1_scale_f16(rowmax, colmax)).astype(np.float16)


def nonfused_step_f16(p, g, state, qm, qv, lr, beta1, beta2, eps, wd):
    """One step of _single_tensor_adamw4bit on one quantised float16 tensor (4-bit states, first
    moment 'group' 128, second 'group' 128 or 'rank1' on a matrix).  p (float16) is updated in place;
    state is a NonFusedState whose scales and statistics are float16 arrays."""
    assert p.dtype == np.float16 and g.dtype == np.float16 and state.bits == 4 and not state.factored
    state.step += 1
    n = state.n
    rank1 = _v_is_rank1(state)
    assert not rank1 or len(state.shape) == 2
    m = np.zeros(n, np.float16) if state.m is None else dequant_group_f16(state.m[0], state.m[1], qm, n)
    if state.v is None:
        v = np.zeros(n, np.float16)
    elif rank1:
        r, c = state.shape
        v = np.ascontiguousarray(dequant_rank1_f16(state.v[0], state.v[1], state.v[2], qv, r, c)).reshape(-1)
    else:
        v = dequant_group_f16(state.v[0], state.v[1], qv, n)
    m, v = np.ascontiguousarray(m), np.ascontiguousarray(v)
    nonfused_update_f16(p.reshape(-1), np.ascontiguousarray(g).reshape(-1), m, v, beta1, beta2, lr, wd, eps,
                        float(state.step))
    state.m = quant_group_f16(m, qm)
    if rank1:
        v2 = v.reshape(state.shape)
        rowmax, colmax = rank1_stats_f16(v2)
        state.v = (quant_rank1_f16(v2, rowmax, colmax, qv), rowmax, colmax)
    else:
        state.v = quant_group_f16(v, qv)
    return m, v


def adamw4bit_step_f16(p, g, m_codes, v_codes, m_scale, v_scale, qm, qv, beta1, beta2, lr, wd, eps, step):
    """The fused 4-bit operator instantiated on half (lpmm/cpp_extension/fused_adamw_kernel.cu:80-174,
    T = at::Half): p, g and the scales are float16 arrays, updated in place like the codes."""
    for a in (p, g, m_scale, v_scale):
        assert a.dtype == np.float16 and a.flags.c_contiguous
    _adamw4bit_f16(p.reshape(-1).view(np.uint16), g.reshape(-1).view(np.uint16), m_codes, v_codes,
                   m_scale.reshape(-1).view(np.uint16), v_scale.reshape(-1).view(np.uint16), _c(qm, np.float32),
                   _c(qv, np.float32), p.size, beta1, beta2, lr, wd, eps, step)
