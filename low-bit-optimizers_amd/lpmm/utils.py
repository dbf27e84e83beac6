"""Small helpers with the names and meanings of the reference's lpmm/utils.py: device-memory
bookkeeping (lpmm/utils.py:12-45), rank helpers (:48-58) and quantisation-error metrics
(:78-116)."""
import torch
import torch.nn.functional as F

_ITEM_BYTES = {torch.float32: 4, torch.int32: 4, torch.bfloat16: 2, torch.float16: 2, torch.int16: 2, torch.int8: 1}


def empty_cache(ratio):
    """Release torch's cached device memory when less than `ratio` of it is in use."""
    if ratio is None:
        return
    reserved = torch.cuda.memory_reserved(0)
    if reserved > 0 and torch.cuda.memory_allocated(0) / reserved < ratio:
        torch.cuda.empty_cache()


def get_memory_usage(print_info=False):
    """Bytes currently allocated by torch on device 0."""
    allocated = torch.cuda.memory_allocated(0)
    if print_info:
        print("allocated: %.2f MB" % (allocated / 2 ** 20), flush=True)
        print("reserved:  %.2f MB" % (torch.cuda.memory_reserved(0) / 2 ** 20), flush=True)
    return allocated


def compute_tensor_bytes(tensors):
    """Bytes held by a tensor or a list of tensors; as in the reference only the 4-, 2- and
    1-byte types it lists are counted (float32/int32, bf16/fp16/int16, int8), others as 0."""
    if not isinstance(tensors, (list, tuple)):
        tensors = [tensors]
    return sum(x.numel() * _ITEM_BYTES.get(x.dtype, 0) for x in tensors)


def get_rank():
    return torch.distributed.get_rank() if torch.distributed.is_initialized() else 0


def get_world_size():
    return torch.distributed.get_world_size() if torch.distributed.is_initialized() else 1


def print0(*args, **kwargs):
    if get_rank() == 0:
        print(*args, **kwargs)


def min_fn(a, b):
    return a < b


def max_fn(a, b):
    return a > b


def get_metric_fn(metric_op):
    if metric_op == "min":
        return min_fn
    if metric_op == "max":
        return max_fn
    raise NotImplementedError


def sqnr(x, qx):
    """Signal-to-quantisation-noise ratio in dB."""
    return 20 * torch.log10(torch.norm(x) / torch.norm(x - qx))


def relerr(x, qx):
    return torch.abs(x - qx).norm() / torch.abs(x).norm()


def jsd(x, qx):
    x, qx = x.flatten(), qx.flatten()
    m = 0.5 * (x + qx)
    return 0.5 * (F.kl_div(x, m) + F.kl_div(qx, m))


def abserr(x, qx):
    return torch.abs(x - qx).mean()


def get_metric_from_q_and_dq(x, op, average, **kwargs):
    """Mean relative error of op(x) against op(dequantise(quantise(x))) over `average`
    round trips (lpmm/utils.py:102-116 always measures 'relerr')."""
    from .functional import vectorwise_dequant, vectorwise_quant

    total = 0.0
    for _ in range(average):
        qx, md = vectorwise_quant(x, **kwargs)
        total += relerr(op(x), op(vectorwise_dequant(qx, **md)))
    return total / average
