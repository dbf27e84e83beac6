"""The reference's non-fused PyTorch path, re-typed as plain PyTorch CPU ops.

TEST INFRASTRUCTURE ONLY (checker and CPU baseline); the shipped package never imports it.

The reference's `_single_tensor_adamw4bit` (lpmm/optim/adamw.py:332-436) is a sequence of
PyTorch library ops plus two calls into its CUDA-only pack/unpack extension
(lpmm/functional.py:363, :396), which rejects CPU tensors
(lpmm/cpp_extension/common.h:22-27).  Here the same op sequence runs on CPU tensors and the
pack/unpack step is done by the C oracle, which produces the same packed layout.  The
PyTorch ops themselves are library code, not reference code; their roundings are what pins
`lpmm_oracle_nonfused_update` in oracle/lpmm_oracle.c.
"""
import math

import numpy as np
import torch

from . import oracle as O


def _group(x, gp_sz):
    """functional.py:404-422: flatten, zero-pad to a multiple of gp_sz, view (G, gp_sz)."""
    flat = x.flatten()
    rem = flat.numel() % gp_sz
    if rem:
        flat = torch.cat([flat, torch.zeros(gp_sz - rem, dtype=x.dtype)])
    return flat.view(-1, gp_sz)


def _pack(normed, qmap):
    """functional.py:361-363: re-group to 2048 and pack two 4-bit codes per byte."""
    grouped = _group(normed, O.PACK_GROUP)
    # half data is widened to float by the reference's kernel (quantization_kernel.cu:450)
    return torch.from_numpy(O.pack_nonlinear_4bit(grouped.float().numpy(), qmap))


def _unpack(codes, qmap, numel):
    """functional.py:393-397 + :425-431: unpack NG*2048 values, keep the first numel."""
    ng = (numel + O.PACK_GROUP - 1) // O.PACK_GROUP
    return torch.from_numpy(O.unpack_nonlinear_4bit(codes.numpy(), qmap, ng * O.PACK_GROUP))[:numel]


def quant_group(x, qmap, gp_sz=128):
    """functional.py:184-189 then :359-369."""
    gx = _group(x, gp_sz)
    max1 = gx.abs().max(dim=1, keepdim=True).values
    return _pack(gx.div(max1), qmap), max1


def dequant_group(codes, max1, qmap, shape, gp_sz=128):
    """functional.py:393-400, :115-118."""
    g = max1.shape[0]
    # the unpacked values are float32; times half statistics they stay float32 (type promotion), and
    # the result takes the state's type at the end (functional.py:150)
    x = _unpack(codes, qmap, g * gp_sz).view(g, gp_sz).mul(max1)
    return x.flatten()[: math.prod(shape)].view(shape).to(max1.dtype)


def quant_rank1(x, qmap):
    """functional.py:190-203 (dim >= 2), :503-531."""
    ax = x.abs()
    max_dims = []
    for i in range(x.dim()):
        r = ax
        for d in range(x.dim()):
            if d != i:
                r = r.max(dim=d, keepdim=True).values
        max_dims.append(r)
    st = max_dims[0].clone()
    for md in max_dims[1:]:
        st = torch.min(st, md)
    return _pack(x.div(st), qmap), max_dims


def dequant_rank1(codes, max_dims, qmap, shape):
    """functional.py:97-106."""
    st = max_dims[0].clone()
    for md in max_dims[1:]:
        st = torch.min(st, md)
    return _unpack(codes, qmap, math.prod(shape)).view(shape).mul(st).to(st.dtype)


class TorchNonFusedAdamW:
    """One-tensor-at-a-time driver of the op sequence, for quantised tensors only
    (numel > 4096).  v_scale_type 'group' is the built-in default (lpmm/config.py:58),
    'rank1' is lpmm/configs/default.yml:11-18."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2,
                 v_scale_type="group", factor_second_moment=False):
        self.params = list(params)
        self.lr, self.betas, self.eps, self.wd = lr, betas, eps, weight_decay
        self.v_scale_type = v_scale_type
        self.factor = factor_second_moment
        self.qm, self.qv = O.qmap_m(), O.qmap_v()
        self.state = [dict(step=0) for _ in self.params]

    @torch.no_grad()
    def step(self, grads):
        beta1, beta2 = self.betas
        lr, eps, wd = self.lr, self.eps, self.wd
        for p, g, st in zip(self.params, grads, self.state):
            st["step"] += 1
            step = st["step"]
            p.mul_(1 - lr * wd)  # adamw.py:369
            factored = self.factor and p.dim() >= 2
            if "m" in st:
                m = dequant_group(st["m"][0], st["m"][1], self.qm, p.shape).clone()
            else:
                m = torch.zeros_like(p)
            bc1 = 1 - beta1 ** step
            bc2 = 1 - beta2 ** step
            step_size = lr / bc1
            bc2_sqrt = math.sqrt(bc2)
            if factored:  # adamw.py:579-627
                if "row" not in st:
                    st["row"] = torch.zeros(p.shape[:-1])
                    st["col"] = torch.zeros(p.shape[:-2] + p.shape[-1:])
                m.lerp_(g, 1 - beta1)
                update = g ** 2
                st["row"].mul_(beta2).add_(update.mean(dim=-1), alpha=1 - beta2)
                st["col"].mul_(beta2).add_(update.mean(dim=-2), alpha=1 - beta2)
                r_factor = (st["row"] / st["row"].mean(dim=-1, keepdim=True)).unsqueeze(-1)
                v = torch.mul(r_factor, st["col"].unsqueeze(-2))
            else:  # adamw.py:402-413
                if "v" not in st:
                    v = torch.zeros_like(p)
                elif self.v_scale_type == "rank1" and p.dim() >= 2:
                    v = dequant_rank1(st["v"][0], st["v"][1], self.qv, p.shape)
                else:
                    v = dequant_group(st["v"][0], st["v"][1], self.qv, p.shape).clone()
                m.lerp_(g, 1 - beta1)
                v.mul_(beta2).addcmul_(g, g, value=1 - beta2)
            denom = (v.sqrt() / bc2_sqrt).add_(eps)
            p.addcdiv_(m, denom, value=-step_size)
            st["m"] = quant_group(m, self.qm)
            if not factored:
                if self.v_scale_type == "rank1" and p.dim() >= 2:
                    st["v"] = quant_rank1(v, self.qv)
                else:
                    st["v"] = quant_group(v, self.qv)
            st["m_fp32"], st["v_fp32"] = m, v


def as_numpy(t):
    return np.ascontiguousarray(t.detach().cpu().numpy())
