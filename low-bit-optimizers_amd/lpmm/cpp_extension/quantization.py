"""lpmm.cpp_extension.quantization: pack_nonlinear / unpack_nonlinear of the reference's
pybind module (lpmm/cpp_extension/quantization.cc:54-83) for 4-bit, round-to-nearest codes.
Both allocate and return a new tensor on the input's device and leave the inputs untouched."""
import torch

from .. import _native
from ._checks import check_cuda_tensor_dim_float, check_cuda_tensor_dim_type, same_device

__all__ = ["pack_nonlinear", "unpack_nonlinear"]


def _require_4bit(bits):
    if bits > 8:
        raise RuntimeError("Expected bits <= 8 to be true, but got false.")
    if bits != 4:
        raise NotImplementedError(f"this build packs 4-bit codes only, got bits={bits}")


def pack_nonlinear(data, qmap, bits, stochastic):
    """data: float32 (num_groups, group_size), already normalised.  Returns int8 of
    bits*numel/8 + 1 bytes (lpmm/cpp_extension/quantization_kernel.cu:475-477); the final byte,
    left uninitialised by the reference, is 0.  Unlike the reference this does not touch
    torch's default random generator."""
    _require_4bit(bits)
    check_cuda_tensor_dim_float(data, "data", 2)
    check_cuda_tensor_dim_float(qmap, "qmap", 1)
    if stochastic:
        raise NotImplementedError("stochastic rounding is not part of this build")
    if data.size(1) % 8 != 0:
        raise RuntimeError("Expected group_size % work_per_thread == 0 to be true, but got false.")
    if qmap.numel() != 16:
        raise RuntimeError("4-bit quantisation maps must have 16 entries")
    dev = same_device(data, qmap)
    n = data.numel()
    out = torch.empty((n // 2 + 1,), dtype=torch.int8, device=dev)
    with torch.cuda.device(dev):
        st = _native.lib().lpmm_pack_nonlinear_4bit(data.data_ptr(), qmap.data_ptr(), n, out.data_ptr(),
                                                    _native.current_stream(dev))
    _native.check(st, "pack_nonlinear")
    return out


def unpack_nonlinear(data, qmap, bits, num_groups, group_size):
    """data: int8 1-D packed codes.  Returns float32 (num_groups, group_size) of qmap[code]
    (lpmm/cpp_extension/quantization_kernel.cu:604-653)."""
    _require_4bit(bits)
    check_cuda_tensor_dim_type(data, "data", 1, torch.int8)
    check_cuda_tensor_dim_float(qmap, "qmap", 1)
    n = int(num_groups) * int(group_size)
    if data.numel() * 2 < n:
        raise RuntimeError(f"packed data holds {data.numel() * 2} codes, fewer than the {n} requested")
    if qmap.numel() != 16:
        raise RuntimeError("4-bit quantisation maps must have 16 entries")
    dev = same_device(data, qmap)
    out = torch.empty((int(num_groups), int(group_size)), dtype=qmap.dtype, device=dev)
    with torch.cuda.device(dev):
        st = _native.lib().lpmm_unpack_nonlinear_4bit(data.data_ptr(), qmap.data_ptr(), n, out.data_ptr(),
                                                      _native.current_stream(dev))
    _native.check(st, "unpack_nonlinear")
    return out
