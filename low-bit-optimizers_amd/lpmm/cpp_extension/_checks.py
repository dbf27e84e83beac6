"""Tensor checks of the operator boundary, same conditions and messages as the reference's
CHECK_CUDA_TENSOR_* macros (lpmm/cpp_extension/common.h:2-27); failures raise RuntimeError
like TORCH_CHECK does."""
import torch


def check_cuda_tensor_float(t, name, *, fp32_only=True):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor!")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous!")
    if t.dtype not in (torch.float32, torch.float16, torch.float64):
        raise RuntimeError(f"The type of {name} is not kFloat32, kFloat16 or kFloat64!")
    if fp32_only and t.dtype != torch.float32:
        kind = "kFloat16" if t.dtype is torch.float16 else "kFloat64"
        raise RuntimeError(f"The type of {name} is {kind}: float32 is required here (half tensors are accepted "
                           "where the reference can run them: adamw_single_tensor and the data of pack_nonlinear; "
                           "double tensors as the data of pack_nonlinear)")


def check_cuda_tensor_dim_float(t, name, n_dim, *, fp32_only=True):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor!")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous!")
    if t.dim() != n_dim:
        raise RuntimeError(f"The dimension of {name} is not correct!")
    check_cuda_tensor_float(t, name, fp32_only=fp32_only)


def check_cuda_tensor_dim_type(t, name, n_dim, dtype):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor!")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous!")
    if t.dim() != n_dim:
        raise RuntimeError(f"The dimension of {name} is not correct!")
    if t.dtype != dtype:
        raise RuntimeError(f"The type of {name} is not correct!")


def same_device(*tensors):
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on the same device, got {dev} and {t.device}")
    return dev
