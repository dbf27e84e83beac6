"""lpmm.cpp_extension.fused_adamw: the two fused-step operators of the reference's pybind
module (lpmm/cpp_extension/fused_adamw.cc:82-83), same positional signatures, in-place on the
caller's tensors, returning None.  Work is enqueued on torch's current stream of the
tensors' device."""
import numpy as np
import torch

from .. import _native
from ._checks import check_cuda_tensor_float, same_device

__all__ = ["adamw_single_tensor", "adamw4bit_single_tensor"]


def adamw_single_tensor(p, g, exp_avg, exp_avg_sq, beta1, beta2, lr, weight_decay, eps, step):
    """Fused AdamW step on states of the parameters' type (lpmm/cpp_extension/fused_adamw.cc:15-41):
    float32, or float16 as the reference's dispatch also instantiates
    (lpmm/cpp_extension/fused_adamw_kernel.cu:188); all four tensors must have the same type."""
    for t, name in ((p, "p"), (exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq"), (g, "g")):
        check_cuda_tensor_float(t, name, fp32_only=False)
        if t.dtype != p.dtype:
            raise RuntimeError(f"expected scalar type {p.dtype} but found {t.dtype} for {name}")
    n = p.numel()
    if exp_avg.numel() != n:
        raise RuntimeError("number of elements in exp_avg and p tensors should be equal")
    if exp_avg_sq.numel() != n:
        raise RuntimeError("number of elements in exp_avg_sq and p tensors should be equal")
    if g.numel() != n:
        raise RuntimeError("number of elements in g and p tensors should be equal")
    dev = same_device(p, g, exp_avg, exp_avg_sq)
    with torch.cuda.device(dev):
        if p.dtype is torch.float16:
            table = np.array([(p.data_ptr(), g.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), n, step, 0.0)],
                             dtype=_native.ADAMW_FP32_TENSOR)
            st = _native.lib().lpmm_adamw_fp16_step_multi(table.ctypes.data, 1, beta1, beta2, lr, weight_decay, eps,
                                                          _native.current_stream(dev))
        else:
            st = _native.lib().lpmm_adamw_fp32_step(
                p.data_ptr(), g.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), n,
                beta1, beta2, lr, weight_decay, eps, step, _native.current_stream(dev))
    _native.check(st, "adamw_single_tensor")


def adamw4bit_single_tensor(p, g, exp_avg, exp_avg_sq, exp_avg_scale, exp_avg_sq_scale,
                            exp_avg_qmap, exp_avg_sq_qmap, beta1, beta2, lr, weight_decay, eps, step):
    """Fused 4-bit AdamW step (lpmm/cpp_extension/fused_adamw.cc:44-78).

    exp_avg / exp_avg_sq hold two 4-bit codes per byte and must have numel == p.numel() // 2,
    the reference's own check (fused_adamw.cc:68-71; a tensor with an odd number of elements
    therefore fails here exactly as it does there).  The scales must have one entry per 128
    elements (lpmm/cpp_extension/fused_adamw_kernel.cu:218-219)."""
    # float32, or float16 as the reference's dispatch also instantiates (fused_adamw_kernel.cu:222): p, g and
    # the scales then share that type (data_ptr<scalar_t>(), :224-230), the maps stay float32 (:231-232)
    half = p.dtype is torch.float16
    check_cuda_tensor_float(p, "p", fp32_only=not half)
    for t, name in ((g, "g"), (exp_avg_scale, "exp_avg_scale"), (exp_avg_sq_scale, "exp_avg_sq_scale")):
        check_cuda_tensor_float(t, name, fp32_only=not half)
        if t.dtype != p.dtype:
            raise RuntimeError(f"expected scalar type {p.dtype} but found {t.dtype} for {name}")
    check_cuda_tensor_float(exp_avg_qmap, "exp_avg_qmap")
    check_cuda_tensor_float(exp_avg_sq_qmap, "exp_avg_sq_qmap")
    n = p.numel()
    if exp_avg.numel() != n // 2:
        raise RuntimeError("number of elements in exp_avg and p tensors should be equal")
    if exp_avg_sq.numel() != n // 2:
        raise RuntimeError("number of elements in exp_avg_sq and p tensors should be equal")
    if g.numel() != n:
        raise RuntimeError("number of elements in g and p tensors should be equal")
    if n >= 2 ** 31:
        raise RuntimeError("parameter tensor is too large to be indexed with int32")
    blocks = (n + 127) // 128
    if exp_avg_scale.numel() != blocks or exp_avg_sq_scale.numel() != blocks:
        raise RuntimeError("Expected grid_dim == exp_avg_scale.numel() to be true, but got false.")
    for t, name in ((exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq")):
        if t.element_size() != 1 or not t.is_cuda or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous CUDA tensor of 1-byte elements")
    if exp_avg_qmap.numel() != 16 or exp_avg_sq_qmap.numel() != 16:
        raise RuntimeError("4-bit quantisation maps must have 16 entries")
    dev = same_device(p, g, exp_avg, exp_avg_sq, exp_avg_scale, exp_avg_sq_scale, exp_avg_qmap,
                      exp_avg_sq_qmap)
    with torch.cuda.device(dev):
        step_fn = _native.lib().lpmm_adamw4bit_f16_step if half else _native.lib().lpmm_adamw4bit_step
        st = step_fn(
            p.data_ptr(), g.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(),
            exp_avg_scale.data_ptr(), exp_avg_sq_scale.data_ptr(), exp_avg_qmap.data_ptr(),
            exp_avg_sq_qmap.data_ptr(), n, beta1, beta2, lr, weight_decay, eps, step,
            _native.current_stream(dev))
    _native.check(st, "adamw4bit_single_tensor")
