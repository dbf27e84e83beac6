"""Quantise / dequantise entry points of the 4-bit optimizer-state path.

Same functions and keyword protocol as the slice of lpmm/functional.py the optimizer uses:
`vectorwise_quant(x, **kw) -> (packed int8, metadata)` (lpmm/functional.py:26-59),
`vectorwise_dequant(qx, **kw) -> x` (:62-151) and `create_general_qmap` (:244-268), for
1..8-bit codes (4-bit is the optimizers' default and the fast path), 'real-nearest' rounding
and the scale types 'group' and 'rank1'.  The packed layout and the metadata dict are the
reference's: for 4 bits int8[NG*1024 + 1] with two codes per byte (low nibble = even index),
for widths that do not divide 8 one code per byte; `max1` of shape (G, 1) for 'group',
`max_dims` for 'rank1', `scaled_shape`, `dtype`, `stride`.

Where the reference chains abs / max / div / cat / pack (and unpack / mul) as separate
passes, each call here is one HIP kernel (two for rank-1 quantisation: statistics, then
normalise + search + pack; tensors of 3..8 dimensions add a kernel that folds the leading
dimensions' statistics into one scale per row of the (numel / last, last) view).
"""
import ctypes
import math

import torch

from . import _native
from .cpp_extension import quantization as ext_quantization

PACK_GROUP = 2048
RANK1_ND_MAX = 8  # dimensions the rank-1 kernels take (LPMM_RANK1_ND_MAX)

_NONLINEAR_TYPES = ("nonlinear", "power-1", "power-2", "power-3", "float-point", "nonlinear-nozero")


# --------------------------------------------------------------------------------------
# quantisation maps
# --------------------------------------------------------------------------------------
def create_dynamic_map(signed=True, max_exponent_bits=7, total_bits=8):
    """Dynamic-exponent map (lpmm/functional.py:272-315): per decade 10^-(E-1)..10^0 the means
    of a float32 linspace(0.1, 1) grid whose resolution doubles with the decade, mirrored
    when signed, plus 0 and 1.  The float32 -> double -> float32 round trip of the
    reference (tensor * scalar, .tolist(), torch.Tensor) is kept, since it fixes the bits."""
    non_sign_bits = total_bits - (1 if signed else 0)
    extra = 2 ** (non_sign_bits - max_exponent_bits) - 1
    if not signed:
        extra *= 2
    values = [0.0, 1.0]

    def add_means(count, decade):
        edges = torch.linspace(0.1, 1, count)
        means = decade * ((edges[:-1] + edges[1:]) / 2.0)
        values.extend(means.tolist())
        if signed:
            values.extend((-means).tolist())

    for i in range(max_exponent_bits):
        decade = 10 ** (i - (max_exponent_bits - 1))
        shift = i + non_sign_bits - max_exponent_bits
        add_means(int(2 ** shift + 1) if signed else int(2 ** (shift + 1) + 1), decade)
        if extra > 0:
            add_means(extra + 1, decade)
    return torch.Tensor(sorted(values))


def create_pow_map(b, signed, p):
    """Power map without zero (lpmm/functional.py:644-656): unsigned -> linspace(0,1,2^b+1)[1:]^p."""
    if signed:
        qmap = torch.linspace(-1, 1, 2 ** b)
        if p != 1:
            qmap = qmap.sign() * (qmap.abs() ** p)
    else:
        qmap = torch.linspace(0, 1, 2 ** b + 1)[1:]
        if p != 1:
            qmap = qmap ** p
    return qmap


def create_general_qmap(quant_type, bit, signed):
    """lpmm/functional.py:244-268 for the map families this build quantises with."""
    if bit == 1:
        return torch.Tensor([-1.0, 1.0]) if signed else torch.Tensor([0.0, 1.0])
    if quant_type == "linear":
        return None
    if quant_type == "nonlinear":
        return create_dynamic_map(signed, bit - 1, bit if signed else bit - 1)
    if quant_type == "nonlinear-nozero":
        mapping = create_dynamic_map(signed, bit - 1, bit if signed else bit - 1)
        if not signed:
            mapping[0] = mapping[1]
        return mapping
    if quant_type in ("power-1", "power-2", "power-3"):
        return create_pow_map(bit, signed, int(quant_type[-1]))
    raise ValueError(f"Not support {quant_type} quant type.")


# --------------------------------------------------------------------------------------
# grouping helpers (lpmm/functional.py:404-431)
# --------------------------------------------------------------------------------------
def group_tensor(input, gp_sz):
    """Flatten, zero-pad to a multiple of gp_sz, view as (num_groups, gp_sz)."""
    if not gp_sz > 0:
        raise ValueError("group size need to be a positive integer, but found {}".format(gp_sz))
    flat = input.flatten()
    rem = flat.shape[0] % gp_sz
    if rem != 0:
        flat = torch.cat([flat, torch.zeros([gp_sz - rem], dtype=input.dtype, device=input.device)], dim=0)
    return flat.view(-1, gp_sz)


def recon_grouped_tensor(grouped_tensor, shape):
    """First shape.numel() values of the flattened groups, viewed as shape."""
    return grouped_tensor.flatten()[: shape.numel()].view(shape)


# --------------------------------------------------------------------------------------
# rank-1 statistics (lpmm/functional.py:503-531)
# --------------------------------------------------------------------------------------
def _max_reduce_except_dim(tensor, dim):
    result = tensor
    rank = tensor.dim()
    if rank > 0:
        assert dim < rank
        for d in range(rank):
            if d != dim:
                result = result.max(dim=d, keepdim=True).values
    return result


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _shape_array(shape):
    return (ctypes.c_int64 * len(shape))(*shape)


def get_sm3_statistics(x, **kwargs):
    """max|x| over all dimensions but one, for each dimension (keepdim shapes).  float32 CUDA
    tensors of 2..8 dimensions take HIP kernels that read x once."""
    on_hip = x.is_cuda and x.dtype == torch.float32 and x.numel() > 0
    if x.dim() == 2 and on_hip:
        xc = x.contiguous()
        rows, cols = xc.shape
        rowmax = torch.empty((rows, 1), dtype=torch.float32, device=x.device)
        colmax = torch.empty((1, cols), dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            st = _native.lib().lpmm_rank1_stats(xc.data_ptr(), rows, cols, rowmax.data_ptr(), colmax.data_ptr(),
                                                _native.current_stream(x.device))
        _native.check(st, "rank1_stats")
        return [rowmax, colmax]
    if 2 < x.dim() <= RANK1_ND_MAX and on_hip:
        xc = x.contiguous()
        shape = tuple(xc.shape)
        stats = []
        for i, d in enumerate(shape):
            keep = [1] * len(shape)
            keep[i] = d
            stats.append(torch.empty(keep, dtype=torch.float32, device=x.device))
        work = None
        if shape[-1] >= 32:  # long last dimension: the 2-D kernel plus a fold of its row maxima
            work = torch.empty((xc.numel() // shape[-1],), dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            st = _native.lib().lpmm_rank1_stats_nd(xc.data_ptr(), len(shape), _shape_array(shape), _ptr_array(stats),
                                                   work.data_ptr() if work is not None else None,
                                                   _native.current_stream(x.device))
        _native.check(st, "rank1_stats_nd")
        return stats
    qx = x.abs()
    return [_max_reduce_except_dim(qx, i) for i in range(x.dim())]


def _row_scale_nd(max_dims, shape):
    """For a tensor of more than two dimensions: per row of its (numel / shape[-1], shape[-1])
    view the smallest statistic of the leading dimensions.  With the last dimension's
    statistics as column maxima the 2-D kernels then scale by min over all dimensions, which
    is _compute_sm3_scale_tensor (lpmm/functional.py:503-509)."""
    if len(shape) > RANK1_ND_MAX:
        raise NotImplementedError(f"rank-1 scaling of a {len(shape)}-D tensor: the kernels take up to "
                                  f"{RANK1_ND_MAX} dimensions")
    dev = max_dims[0].device
    stats = [m.to(torch.float32).contiguous() for m in max_dims]
    for m, d in zip(stats, shape):
        if m.numel() != d:
            raise ValueError(f"max_dims do not belong to a tensor of shape {tuple(shape)}")
    rows = math.prod(shape[:-1])
    row_scale = torch.empty((rows,), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        st = _native.lib().lpmm_rank1_row_scale_nd(_ptr_array(stats), len(shape), _shape_array(tuple(shape)),
                                                   row_scale.data_ptr(), _native.current_stream(dev))
    _native.check(st, "rank1_row_scale_nd")
    return row_scale, stats[-1]


def _compute_sm3_scale_tensor(max_dims):
    scale = max_dims[0].clone()
    for other in max_dims[1:]:
        scale = torch.min(scale, other)
    return scale


# --------------------------------------------------------------------------------------
# code search + packing on already-normalised values (lpmm/functional.py:359-400)
# --------------------------------------------------------------------------------------
_ROUND_TYPES = ("real-nearest", "real-sr")  # the two that go through the packing operator


def nonlinear_quant(qx, qmap, b, round_type="sr"):
    if round_type not in _ROUND_TYPES:
        raise NotImplementedError(f"round_type {round_type!r}: this build implements {_ROUND_TYPES} only")
    return ext_quantization.pack_nonlinear(group_tensor(qx, PACK_GROUP), qmap, b, round_type == "real-sr")


def nonlinear_dequant(qx, qmap, b, shape, round_type="sr"):
    if not round_type.startswith("real"):
        raise NotImplementedError(f"round_type {round_type!r}: this build implements {_ROUND_TYPES} only")
    num_groups = (shape.numel() + PACK_GROUP - 1) // PACK_GROUP
    return recon_grouped_tensor(ext_quantization.unpack_nonlinear(qx, qmap, b, num_groups, PACK_GROUP), shape)


# --------------------------------------------------------------------------------------
# vectorwise_quant / vectorwise_dequant
# --------------------------------------------------------------------------------------
def _select_qmap(kwargs):
    qmap = kwargs["qmap"]
    if not isinstance(qmap, torch.Tensor):
        qmap = qmap[(kwargs["b"], kwargs["signed"])][kwargs["quant_type"]]
    return qmap


def _require_supported(kwargs, x):
    if kwargs["quant_type"] not in _NONLINEAR_TYPES:
        raise ValueError(f"Not support {kwargs['quant_type']} quant type.")
    if not 1 <= kwargs["b"] <= 8:
        raise ValueError(f"code width must be 1..8 bits, got {kwargs['b']}")
    if kwargs["round_type"] not in _ROUND_TYPES:
        raise NotImplementedError(
            f"round_type {kwargs['round_type']!r}: this build implements {_ROUND_TYPES} only")
    if not x.is_cuda:
        raise RuntimeError("x must be a CUDA tensor! (the quantised optimizer path has no CPU implementation)")


def storage_bits(b):
    """Bits a code occupies in the packed tensor: widths that divide 8 (1, 2, 4) are packed,
    every other width takes a whole byte (lpmm/cpp_extension/quantization_kernel.cu:592-601)."""
    return b if b in (1, 2, 4) else 8


def packed_nbytes(numel_scaled, b=4):
    """Bytes of the packed tensor for numel_scaled normalised values of b-bit codes."""
    return (numel_scaled + PACK_GROUP - 1) // PACK_GROUP * (PACK_GROUP * storage_bits(b) // 8) + 1


_CODE_TABLES = {}
_CODE_TABLES_MAX = 64


def code_table(qmap, b):
    """The code table of a device map for the quantisers and step kernels of widths other than 4
    (lpmm_code_table_build): built by one small launch the first time a map tensor is seen and kept
    with that tensor, so that the kernels find a code with one table read instead of the
    reference's search (lpmm/cpp_extension/quantization_kernel.cu:397-427; same codes).  The entry
    holds the map tensor itself: its memory cannot be handed to another map while the table lives,
    and a map that was modified in place (tensor version) gets a new table."""
    key = (qmap.data_ptr(), qmap._version, int(b))
    hit = _CODE_TABLES.get(key)
    if hit is not None:
        return hit[1]
    if qmap.dtype != torch.float32 or not qmap.is_cuda or not qmap.is_contiguous() or qmap.numel() != 2 ** b:
        raise ValueError("lpmm: code_table needs a contiguous float32 CUDA map of 2^b entries")
    table = torch.empty(_native.CODE_TABLE_BYTES // 4, dtype=torch.int32, device=qmap.device)
    with torch.cuda.device(qmap.device):
        st = _native.lib().lpmm_code_table_build(qmap.data_ptr(), int(b), table.data_ptr(),
                                                 _native.current_stream(qmap.device))
    _native.check(st, "code_table_build")
    if len(_CODE_TABLES) >= _CODE_TABLES_MAX:
        _CODE_TABLES.pop(next(iter(_CODE_TABLES)))
    _CODE_TABLES[key] = (qmap, table)
    return table


def _group_gp_sz_ok(gp_sz):
    return gp_sz in (128, 256, 512, 1024, 2048, 4096)


def quant_group_(x, qmap, gp_sz, codes=None, max1=None, b=4):
    """'group' scaling in one kernel.  x: contiguous float32 CUDA tensor.  Optionally writes
    into caller-owned `codes` / `max1` buffers of the right size."""
    n = x.numel()
    groups = (n + gp_sz - 1) // gp_sz
    if codes is None:
        codes = torch.empty((packed_nbytes(groups * gp_sz, b),), dtype=torch.int8, device=x.device)
    if max1 is None:
        max1 = torch.empty((groups, 1), dtype=torch.float32, device=x.device)
    lib = _native.lib()
    with torch.cuda.device(x.device):
        stream = _native.current_stream(x.device)
        if b == 4:
            st = lib.lpmm_quant_group(x.data_ptr(), n, gp_sz, qmap.data_ptr(), codes.data_ptr(), max1.data_ptr(),
                                      stream)
        else:
            st = lib.lpmm_quant_group_bits_table(x.data_ptr(), n, gp_sz, qmap.data_ptr(), b,
                                                 code_table(qmap, b).data_ptr(), codes.data_ptr(), max1.data_ptr(),
                                                 stream)
    _native.check(st, "quant_group")
    return codes, max1


def quant_rank1_(x, qmap, codes=None, b=4):
    """'rank1' scaling of a contiguous float32 CUDA tensor of two or more dimensions:
    statistics kernel(s), then normalise + search + pack kernel (more than two dimensions: on
    the (numel / shape[-1], shape[-1]) view with the leading dimensions' minima as row scale)."""
    max_dims = get_sm3_statistics(x)
    if x.dim() == 2:
        rows, cols = x.shape
        rowmax, colmax = max_dims
    else:
        rows, cols = x.numel() // x.shape[-1], x.shape[-1]
        rowmax, colmax = _row_scale_nd(max_dims, x.shape)
    if codes is None:
        codes = torch.empty((packed_nbytes(rows * cols, b),), dtype=torch.int8, device=x.device)
    lib = _native.lib()
    with torch.cuda.device(x.device):
        stream = _native.current_stream(x.device)
        if b == 4:
            st = lib.lpmm_quant_rank1(x.data_ptr(), rows, cols, rowmax.data_ptr(), colmax.data_ptr(),
                                      qmap.data_ptr(), codes.data_ptr(), stream)
        else:
            st = lib.lpmm_quant_rank1_bits_table(x.data_ptr(), rows, cols, rowmax.data_ptr(), colmax.data_ptr(),
                                                 qmap.data_ptr(), b, code_table(qmap, b).data_ptr(),
                                                 codes.data_ptr(), stream)
    _native.check(st, "quant_rank1")
    return codes, max_dims


def vectorwise_quant(x, **kwargs):
    """Quantise x; returns (packed codes, generated metadata).  lpmm/functional.py:26-59 with
    quant_scaling's 'group' (:184-189) and 'rank1' (:190-203) branches."""
    _require_supported(kwargs, x)
    qmap = _select_qmap(kwargs)
    md = {"dtype": x.dtype, "stride": x.stride()}
    src = x.detach()
    if src.dtype not in (torch.float32, torch.float16, torch.float64):
        raise NotImplementedError(f"{src.dtype} states: the quantisers take float32, float16 and float64")
    # float16 and float64 states (half or double parameters on the non-fused path): the scaling runs as PyTorch device ops
    # of that type, one rounding per op, exactly the reference's chain (lpmm/functional.py:184-203);
    # the search and the packing widen each value to float, as the reference's half kernel does
    fp32 = src.dtype is torch.float32
    src = src.contiguous()
    scale_type = kwargs["scale_type"]
    b = kwargs["b"]
    as_group = scale_type == "group" or (scale_type == "rank1" and src.dim() == 1)
    if scale_type == "rank1":
        md["dim"] = src.dim()
    # stochastic rounding: scaling by PyTorch device ops as in the reference
    # (lpmm/functional.py:184-203), the search and packing by the HIP operator
    nearest = kwargs["round_type"] == "real-nearest" and fp32
    if as_group:
        gp_sz = kwargs["gp_sz"] if scale_type == "group" else 128
        if nearest and _group_gp_sz_ok(gp_sz):
            codes, max1 = quant_group_(src, qmap, gp_sz, b=b)
        else:  # any other group size: PyTorch reductions, HIP search + pack
            grouped = group_tensor(src, gp_sz)
            max1 = _max_reduce_except_dim(grouped.abs(), 0)
            codes = nonlinear_quant(grouped.div(max1), qmap, b, round_type=kwargs["round_type"])
        md["max1"] = max1
        md["scaled_shape"] = torch.Size((max1.shape[0], gp_sz))
    elif scale_type == "rank1":
        if nearest and 2 <= src.dim() <= RANK1_ND_MAX and src.numel() > 0:
            codes, max_dims = quant_rank1_(src, qmap, b=b)
        else:
            max_dims = get_sm3_statistics(src)
            codes = nonlinear_quant(src.div(_compute_sm3_scale_tensor(max_dims)), qmap, b,
                                    round_type=kwargs["round_type"])
        md["max_dims"] = max_dims
        md["max1"] = None
        md["scaled_shape"] = src.shape
    else:
        raise NotImplementedError(f"scale_type {scale_type!r}: this build implements 'group' and 'rank1'")
    return codes, md


def vectorwise_dequant(qx, denormalized=True, **kwargs):
    """Dequantise packed codes to a tensor of kwargs['shape'] (the parameter's shape) with the
    strides kwargs['stride'] records (None: contiguous).  lpmm/functional.py:62-151."""
    _require_supported(kwargs, qx)
    qmap = _select_qmap(kwargs)
    dtype, stride = kwargs["dtype"], kwargs["stride"]
    scaled_shape = kwargs["scaled_shape"]
    scale_type = kwargs["scale_type"]
    codes = qx.detach()
    dev = codes.device
    b = kwargs["b"]
    lib = _native.lib()
    as_group = scale_type == "group" or (scale_type == "rank1" and kwargs["dim"] == 1)
    if not denormalized:
        return nonlinear_dequant(codes, qmap, b, shape=scaled_shape, round_type=kwargs["round_type"])
    if as_group:
        shape = kwargs["shape"]
        gp_sz = scaled_shape[1]
        n = shape.numel()
        if gp_sz % 128 == 0 and kwargs["max1"].dtype is torch.float32:
            x = torch.empty(shape, dtype=torch.float32, device=dev)
            with torch.cuda.device(dev):
                stream = _native.current_stream(dev)
                if b == 4:
                    st = lib.lpmm_dequant_group(codes.data_ptr(), kwargs["max1"].data_ptr(), qmap.data_ptr(), n,
                                                gp_sz, x.data_ptr(), stream)
                else:
                    st = lib.lpmm_dequant_group_bits(codes.data_ptr(), kwargs["max1"].data_ptr(), qmap.data_ptr(),
                                                     b, n, gp_sz, x.data_ptr(), stream)
            _native.check(st, "dequant_group")
        else:
            x = nonlinear_dequant(codes, qmap, b, shape=scaled_shape, round_type=kwargs["round_type"])
            x = recon_grouped_tensor(x.mul(kwargs["max1"]), shape)
    elif scale_type == "rank1":
        max_dims = kwargs["max_dims"]
        if (2 <= len(scaled_shape) <= RANK1_ND_MAX and numel(scaled_shape) > 0
                and all(m.dtype is torch.float32 for m in max_dims)):
            if len(scaled_shape) == 2:
                rows, cols = scaled_shape
                rowmax, colmax = max_dims
            else:
                rows, cols = numel(scaled_shape[:-1]), scaled_shape[-1]
                rowmax, colmax = _row_scale_nd(max_dims, scaled_shape)
            x = torch.empty(scaled_shape, dtype=torch.float32, device=dev)
            with torch.cuda.device(dev):
                stream = _native.current_stream(dev)
                if b == 4:
                    st = lib.lpmm_dequant_rank1(codes.data_ptr(), rowmax.data_ptr(), colmax.data_ptr(),
                                                qmap.data_ptr(), rows, cols, x.data_ptr(), stream)
                else:
                    st = lib.lpmm_dequant_rank1_bits(codes.data_ptr(), rowmax.data_ptr(), colmax.data_ptr(),
                                                     qmap.data_ptr(), b, rows, cols, x.data_ptr(), stream)
            _native.check(st, "dequant_rank1")
        else:
            x = nonlinear_dequant(codes, qmap, b, shape=scaled_shape, round_type=kwargs["round_type"])
            x = x.mul(_compute_sm3_scale_tensor(max_dims))
    else:
        raise NotImplementedError(f"scale_type {scale_type!r}: this build implements 'group' and 'rank1'")

    if stride is not None and x.stride() != stride:
        recon = torch.empty_strided(x.shape, stride, dtype=dtype, layout=torch.strided, device=dev)
        recon.copy_(x)
        return recon
    return x.to(dtype=dtype)


def numel(shape):
    return math.prod(shape)
