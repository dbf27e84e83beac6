"""lpmm.cpp_extension.quantization: pack_nonlinear / unpack_nonlinear of the reference's
pybind module (lpmm/cpp_extension/quantization.cc:54-83) for codes of 1..8 bits, rounded to
nearest or stochastically.  Both allocate and return a new tensor on the input's device and
leave the inputs untouched."""
import torch

from .. import _native
from ._checks import check_cuda_tensor_dim_float, check_cuda_tensor_dim_type, same_device

__all__ = ["pack_nonlinear", "unpack_nonlinear"]


def _check_bits(bits, qmap):
    if bits > 8:
        raise RuntimeError("Expected bits <= 8 to be true, but got false.")
    if bits < 1:
        raise RuntimeError(f"bits must be at least 1, got {bits}")
    if qmap.numel() < 2 ** bits:
        raise RuntimeError(f"{bits}-bit quantisation maps must have {2 ** bits} entries, got {qmap.numel()}")


def _storage_bits(bits):
    # widths that divide 8 are packed, the others take a byte per code
    # (lpmm/cpp_extension/quantization_kernel.cu:592-601)
    return bits if bits in (1, 2, 4) else 8


def pack_nonlinear(data, qmap, bits, stochastic):
    """data: float32, float16 or float64 (num_groups, group_size), already normalised.  Returns int8 of
    storage_bits*numel/8 + 1 bytes (lpmm/cpp_extension/quantization_kernel.cu:475-477, :549-550; storage_bits
    is `bits` for 1, 2 and 4 and 8 otherwise); the final byte,
    left uninitialised by the reference, is 0.

    stochastic=True draws its random numbers as the reference does
    (lpmm/cpp_extension/quantization_kernel.cu:480-487): a (seed, offset) pair from torch's default
    generator of the device, whose offset advances by group_size * work_per_thread rounded up
    to a multiple of 4.  With stochastic=False the generator is left alone (the reference
    advances it there too, although its kernel ignores the numbers).

    Half data: the reference's kernel is instantiated for at::Half as well and widens every value to
    float before the search (lpmm/cpp_extension/quantization_kernel.cu:489-507, :450); the widening is
    exact, so the codes are those of data.float(), which is what runs here.  The map must be float32
    there too (qmap.data_ptr<float>())."""
    check_cuda_tensor_dim_float(data, "data", 2, fp32_only=False)
    check_cuda_tensor_dim_float(qmap, "qmap", 1)
    if data.dtype is not torch.float32:
        # half: exact widening; double: rounded to float, which is the kernel's `const float x = data[i]`
        # (lpmm/cpp_extension/quantization_kernel.cu:450, dispatched for double as well, :492)
        data = data.float()
    _check_bits(bits, qmap)
    if data.size(1) % (4 * (8 // _storage_bits(bits))) != 0 or data.numel() % 8 != 0:
        raise RuntimeError("Expected group_size % work_per_thread == 0 to be true, but got false.")
    dev = same_device(data, qmap)
    n = data.numel()
    out = torch.empty((n * _storage_bits(bits) // 8 + 1,), dtype=torch.int8, device=dev)
    with torch.cuda.device(dev):
        if stochastic:
            if n % 32 != 0:
                raise RuntimeError("stochastic rounding needs a multiple of 32 values")
            work_per_thread = 4 * (8 // _storage_bits(bits))
            gen = torch.cuda.default_generators[dev.index if dev.index is not None else torch.cuda.current_device()]
            seed, offset = gen.initial_seed(), gen.get_offset()
            gen.set_offset(offset + (data.size(1) * work_per_thread + 3) // 4 * 4)
            st = _native.lib().lpmm_pack_nonlinear_sr(data.data_ptr(), qmap.data_ptr(), bits, n, seed, offset,
                                                      out.data_ptr(), _native.current_stream(dev))
        elif bits == 4:
            st = _native.lib().lpmm_pack_nonlinear_4bit(data.data_ptr(), qmap.data_ptr(), n, out.data_ptr(),
                                                        _native.current_stream(dev))
        else:
            st = _native.lib().lpmm_pack_nonlinear(data.data_ptr(), qmap.data_ptr(), bits, n, out.data_ptr(),
                                                   _native.current_stream(dev))
    _native.check(st, "pack_nonlinear")
    return out


def unpack_nonlinear(data, qmap, bits, num_groups, group_size):
    """data: int8 1-D packed codes.  Returns float32 (num_groups, group_size) of qmap[code]
    (lpmm/cpp_extension/quantization_kernel.cu:604-653)."""
    check_cuda_tensor_dim_type(data, "data", 1, torch.int8)
    check_cuda_tensor_dim_float(qmap, "qmap", 1)
    _check_bits(bits, qmap)
    n = int(num_groups) * int(group_size)
    held = data.numel() * 8 // _storage_bits(bits)
    if held < n:
        raise RuntimeError(f"packed data holds {held} codes, fewer than the {n} requested")
    if n % 8 != 0:
        raise RuntimeError("Expected group_size % work_per_thread == 0 to be true, but got false.")
    dev = same_device(data, qmap)
    out = torch.empty((int(num_groups), int(group_size)), dtype=qmap.dtype, device=dev)
    with torch.cuda.device(dev):
        if bits == 4:
            st = _native.lib().lpmm_unpack_nonlinear_4bit(data.data_ptr(), qmap.data_ptr(), n, out.data_ptr(),
                                                          _native.current_stream(dev))
        else:
            st = _native.lib().lpmm_unpack_nonlinear(data.data_ptr(), qmap.data_ptr(), bits, n, out.data_ptr(),
                                                     _native.current_stream(dev))
    _native.check(st, "unpack_nonlinear")
    return out
