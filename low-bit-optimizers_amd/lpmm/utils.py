"""Helpers that users of lpmm import next to the optimizers: device-memory bookkeeping, rank
queries and quantisation-error metrics.  Names, arguments and results follow the reference's
lpmm/utils.py (memory: lines 12-45, ranks: 48-58, metrics: 61-116)."""
import operator

import torch

# element sizes the reference's byte counter knows (lpmm/utils.py:38-43); any other dtype counts as 0
_COUNTED_ITEMSIZE = {
    torch.float32: 4, torch.int32: 4,
    torch.bfloat16: 2, torch.float16: 2, torch.int16: 2,
    torch.int8: 1,
}
_MIB = float(1 << 20)


def _device0_memory():
    return torch.cuda.memory_allocated(0), torch.cuda.memory_reserved(0)


def empty_cache(ratio):
    """Hand torch's cached blocks of device 0 back to the driver when less than `ratio` of the
    reserved memory is in use; `None` switches the check off."""
    if ratio is not None:
        in_use, reserved = _device0_memory()
        if reserved > 0 and in_use < ratio * reserved:
            torch.cuda.empty_cache()


def get_memory_usage(print_info=False):
    """Bytes torch has allocated on device 0 right now."""
    in_use, reserved = _device0_memory()
    if print_info:
        print(f"allocated: {in_use / _MIB:.2f} MB", flush=True)
        print(f"reserved:  {reserved / _MIB:.2f} MB", flush=True)
    return in_use


def compute_tensor_bytes(tensors):
    """Bytes held by one tensor or by a list/tuple of tensors."""
    seq = tensors if isinstance(tensors, (list, tuple)) else (tensors,)
    return sum(t.numel() * _COUNTED_ITEMSIZE.get(t.dtype, 0) for t in seq)


def _dist_query(name, single_process_value):
    dist = torch.distributed
    return getattr(dist, name)() if dist.is_available() and dist.is_initialized() else single_process_value


def get_rank():
    return _dist_query("get_rank", 0)


def get_world_size():
    return _dist_query("get_world_size", 1)


def print0(*args, **kwargs):
    """print on rank 0 only."""
    if get_rank() == 0:
        print(*args, **kwargs)


min_fn = operator.lt  # "a is better than b" when smaller is better
max_fn = operator.gt  # ... when larger is better


def get_metric_fn(metric_op):
    try:
        return {"min": min_fn, "max": max_fn}[metric_op]
    except KeyError:
        raise NotImplementedError(metric_op) from None


def _err(x, qx):
    return x - qx


def sqnr(x, qx):
    """Signal-to-quantisation-noise ratio in dB: 20 log10(|x| / |x - qx|)."""
    return 20 * torch.log10(torch.linalg.vector_norm(x) / torch.linalg.vector_norm(_err(x, qx)))


def relerr(x, qx):
    """|x - qx| / |x| in the Euclidean norm."""
    return torch.linalg.vector_norm(_err(x, qx)) / torch.linalg.vector_norm(x)


def abserr(x, qx):
    """Mean absolute error."""
    return _err(x, qx).abs().mean()


def jsd(x, qx):
    """Jensen-Shannon style divergence of two flattened tensors, built from torch's kl_div with
    its default arguments as in the reference (lpmm/utils.py:90-95)."""
    a, b = x.reshape(-1), qx.reshape(-1)
    mid = (a + b) / 2
    kl = torch.nn.functional.kl_div
    return (kl(a, mid) + kl(b, mid)) / 2


def get_metric_from_q_and_dq(x, op, average, **kwargs):
    """Relative error of op(x) against op(dequantise(quantise(x))), averaged over `average`
    round trips (the reference measures 'relerr' whatever else it lists, lpmm/utils.py:103-116)."""
    from .functional import vectorwise_dequant, vectorwise_quant

    target = op(x)
    runs = []
    for _ in range(average):
        codes, meta = vectorwise_quant(x, **kwargs)
        runs.append(relerr(target, op(vectorwise_dequant(codes, **meta))))
    return sum(runs) / average
