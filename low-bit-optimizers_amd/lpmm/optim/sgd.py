"""SGD with a 4-bit momentum buffer.

Drop-in for lpmm.optim.SGD (lpmm/optim/sgd.py:11-187): same constructor and state keys
(`momentum_buffer`, `momentum_buffer_qstate`), non-fused only (fused=True raises, as there).
The momentum buffer uses the first-moment quantisation config (QUANT.M).  Contiguous float32
tensors whose buffer is quantised with 4 bits, 'group' scaling over 128 values and round to
nearest (the default configuration) take one HIP kernel per 64 tensors that reads p, g and the
packed buffer once and writes p and the buffer back (lpmm_sgd4bit_step_multi: 13 bytes per
parameter).  Every other case runs the reference's own chain of PyTorch ops on the device
(lpmm/optim/sgd.py:152-187) around the HIP dequantise / quantise kernels of lpmm.functional.
Both produce the same state layout.
"""
from typing import Optional

import numpy as np
import torch

from .. import _native
from ..functional import packed_nbytes, vectorwise_dequant, vectorwise_quant
from .optimizer import LowBitOptimizer

__all__ = ["SGD"]


class SGD(LowBitOptimizer):
    def __init__(
        self,
        params,
        lr,
        momentum=0,
        dampening=0,
        weight_decay=0,
        nesterov=False,
        qconfig=None,
        *,
        maximize: bool = False,
        fused: Optional[bool] = False,
    ):
        if lr < 0.0:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        if weight_decay < 0.0:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        if fused is True:
            raise ValueError("Not support fused SGD currently.")
        defaults = dict(lr=lr, momentum=momentum, weight_decay=weight_decay, dampening=dampening,
                        nesterov=nesterov, maximize=maximize)
        super().__init__(params, defaults, qconfig)

    def get_subqconfig(self, optimizer_state_name):
        if optimizer_state_name == "momentum_buffer":
            return self.qconfig.QUANT.M
        raise ValueError(f"unknown optimizer state {optimizer_state_name!r}")

    @torch.no_grad()
    def step(self, closure=None):
        """Performs a single optimization step."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        md = self.get_qmetadata_by_state_name("momentum_buffer")
        one_pass_config = (md["b"] == 4 and md["scale_type"] == "group" and md["gp_sz"] == 128
                           and md["round_type"] == "real-nearest")
        for group in self.param_groups:
            momentum, dampening = group["momentum"], group["dampening"]
            batched = {}  # (device, map address) -> records of the one-pass kernel
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("SGD does not support sparse gradients")
                state = self.state[p]
                if len(state) == 0:
                    state["momentum_buffer"] = torch.zeros((), dtype=torch.float, device=p.device)
                    self.init_qstate(p, "momentum_buffer")
                qstate = state["momentum_buffer_qstate"]
                enabled = self.override_q_enable.get(id(p), qstate["enable"])

                if (one_pass_config and enabled and momentum != 0 and p.is_cuda and p.dtype is torch.float32
                        and p.grad.dtype is torch.float32 and p.is_contiguous() and p.grad.is_contiguous()):
                    first = state["momentum_buffer"].numel() <= 1
                    if first:
                        groups = (p.numel() + 127) // 128
                        state["momentum_buffer"] = torch.empty((packed_nbytes(groups * 128),), dtype=torch.int8,
                                                               device=p.device)
                        qstate["overhead"].clear()
                        qstate["overhead"].update({"dtype": p.dtype, "stride": p.stride(),
                                                   "max1": torch.empty((groups, 1), dtype=torch.float32, device=p.device),
                                                   "scaled_shape": torch.Size((groups, 128))})
                    batched.setdefault((p.device, qstate["qmap"].data_ptr()), []).append(
                        (p.data_ptr(), p.grad.data_ptr(), state["momentum_buffer"].data_ptr(),
                         qstate["overhead"]["max1"].data_ptr(), p.numel(), 1 if first else 0, 0))
                    continue

                d_p = p.grad if not group["maximize"] else -p.grad
                if group["weight_decay"] != 0:
                    d_p = d_p.add(p, alpha=group["weight_decay"])
                if momentum != 0:
                    q_buf = state["momentum_buffer"]
                    if q_buf.numel() <= 1:
                        # the first step stores the (decayed) gradient itself (sgd.py:161-163)
                        buf = torch.clone(d_p).detach()
                    else:
                        if enabled:
                            kw = dict(qstate["overhead"])
                            kw.update(md)
                            buf = vectorwise_dequant(q_buf, qmap=qstate["qmap"], shape=p.shape, **kw)
                        else:
                            buf = q_buf
                        buf.mul_(momentum).add_(d_p, alpha=1 - dampening)
                    d_p = d_p.add(buf, alpha=momentum) if group["nesterov"] else buf
                    if enabled:
                        qx, gen = vectorwise_quant(buf, qmap=qstate["qmap"], shape=p.shape, **md)
                        state["momentum_buffer"] = qx
                        qstate["overhead"].clear()
                        qstate["overhead"].update(gen)
                    else:
                        state["momentum_buffer"] = buf
                p.add_(d_p, alpha=-group["lr"])

            for (dev, qmap_ptr), records in batched.items():
                table = np.array(records, dtype=_native.SGD4BIT_TENSOR)
                with torch.cuda.device(dev):
                    st = _native.lib().lpmm_sgd4bit_step_multi(
                        table.ctypes.data, len(records), qmap_ptr, momentum, dampening, group["lr"],
                        group["weight_decay"], int(bool(group["nesterov"])), int(bool(group["maximize"])),
                        _native.current_stream(dev))
                _native.check(st, "SGD step")
        return loss
