"""AdamW with 4-bit optimizer states on MI355X.

Drop-in for lpmm.optim.AdamW (lpmm/optim/adamw.py:14-230): same constructor, same
per-parameter state keys (`step`, `exp_avg`, `exp_avg_sq`, `exp_avg_qstate`,
`exp_avg_sq_qstate`, `exp_avg_sq_row`, `exp_avg_sq_col`), same packed layouts:

* fused=True   -> `exp_avg`/`exp_avg_sq` int8[(numel+1)//2], scales float32[ceil(numel/128)]
                  in `*_qstate["overhead"]["max1"]` (lpmm/optim/adamw.py:508-523); tensors with
                  numel <= threshold keep fp32 states (:543-561).
* fused=False  -> `vectorwise_quant` layout and metadata (lpmm/optim/adamw.py:425-434).
* factor_second_moment=True on >= 2-D tensors -> fp32 row/col statistics (:124-126, :579-627).

What differs is the execution: all fused tensors of a parameter group go to the GPU in a
handful of multi-tensor launches instead of one launch per tensor, and each quantise /
dequantise / update of the non-fused path is one HIP kernel instead of a chain of
PyTorch passes.
"""
import math
import weakref
from typing import Optional

import numpy as np
import torch

from .. import _native
from ..functional import RANK1_ND_MAX, _ptr_array, _shape_array, code_table, packed_nbytes, vectorwise_dequant, vectorwise_quant
from .optimizer import LowBitOptimizer

__all__ = ["AdamW"]


def _two_pass_columns(rows, cols):
    """Column counts the two-pass kernels take on a rows x cols matrix: whole 128-column blocks, or
    half a block left over with an even row count (taken as double rows)."""
    return cols % 128 == 0 or (cols % 128 == 64 and rows % 2 == 0)


def _two_pass_nd(shape):
    """Tensors of more than two dimensions that take the two passes on their shape[0] x rest view.  The
    kernels' tiles are 64 rows tall: a large tensor with a handful of rows (a stack of a few matrices)
    fills an eighth of every tile and pays one column atomic per few elements -- measured 1.20 against
    0.47 ms for 3 x 4096 x 4096 and 0.66 against 0.58 ms for 8 x 2048 x 4096, level at 16 rows -- so it
    stays with the staged path; small tensors gain from the batched launches whatever their shape."""
    rows, numel = shape[0], 1
    for d in shape:
        numel *= d
    if rows == 0 or not _two_pass_columns(rows, numel // rows):
        return False
    return rows >= 16 or numel <= (1 << 20)


def _is_placeholder(t):
    # a state that has not been materialised yet is a 0-dim tensor (adamw.py:121, :128);
    # the reference tests numel() <= 1 (adamw.py:394, :402, :509, :544)
    return t.numel() <= 1


_ZERO_BYTE = {}


def _zero_byte(qmap):
    """int8 value of a packed byte whose two codes both select the map entry nearest 0.0
    (what quantising a zero tensor stores); looked up once per map tensor.  The cache entry
    remembers which tensor object it was made for: an address the allocator hands to another
    map later does not hit it."""
    key = (qmap.device, qmap.data_ptr(), qmap._version)
    hit = _ZERO_BYTE.get(key)
    if hit is None or hit[0]() is not qmap:
        code = int(torch.argmin(qmap.abs()).item())
        byte = code | (code << 4)
        hit = _ZERO_BYTE[key] = (weakref.ref(qmap), byte - 256 if byte > 127 else byte)
    return hit[1]


class _Batch(list):
    """Records of one pending launch, plus what becomes true once that launch has been enqueued: states
    whose statistics trade places with a second buffer point to the new buffer only after the kernels
    that fill it are on the stream.  A check that raises before the launch, or a launch that returns an
    error, leaves those states as they were (old codes with the statistics they are scaled by)."""

    def __init__(self):
        super().__init__()
        self.commits = []

    def launched(self):
        for commit in self.commits:
            commit()
        self.commits.clear()


class AdamW(LowBitOptimizer):
    def __init__(
        self,
        params,
        lr=1e-3,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=1e-2,
        use_first_moment=True,
        factor_second_moment=False,
        qconfig=None,
        *,
        fused: Optional[bool] = False,
    ):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        if not 0.0 <= weight_decay:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, fused=fused,
                        use_first_moment=use_first_moment, factor_second_moment=factor_second_moment)
        super().__init__(params, defaults, qconfig)

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault("fused", None)
        for s in self.state.values():
            if "step" in s and not torch.is_tensor(s["step"]):
                s["step"] = torch.tensor(float(s["step"]))

    def get_subqconfig(self, optimizer_state_name):
        if optimizer_state_name == "exp_avg":
            return self.qconfig.QUANT.M
        if optimizer_state_name == "exp_avg_sq":
            return self.qconfig.QUANT.SQM
        raise ValueError(f"unknown optimizer state {optimizer_state_name!r}")

    @staticmethod
    def _get_options(param_group, param_shape):
        factored = len(param_shape) >= 2 and param_group["factor_second_moment"]
        return factored, param_group["use_first_moment"]

    # ---- state ---------------------------------------------------------------------------
    def _state_of(self, group, p):
        """The parameter's state, created on first use (lpmm/optim/adamw.py:114-129), and whether its
        second moment is factored (decided once, when the state is created: the keys tell)."""
        state = self.state[p]
        if len(state) != 0:
            return state, "exp_avg_sq_row" in state
        factored, _ = self._get_options(group, p.shape)
        state["step"] = torch.tensor(0.0)  # on the host: reading it never syncs the GPU
        state["exp_avg"] = torch.zeros((), dtype=torch.float, device=p.device)
        self.init_qstate(p, "exp_avg")
        if factored:
            state["exp_avg_sq_row"] = torch.zeros(p.shape[:-1], device=p.device)
            state["exp_avg_sq_col"] = torch.zeros(p.shape[:-2] + p.shape[-1:], device=p.device)
        else:
            state["exp_avg_sq"] = torch.zeros((), dtype=torch.float, device=p.device)
        self.init_qstate(p, "exp_avg_sq")
        return state, factored

    def _next_step(self, state):
        """state["step"] += 1 and its value as a Python float.  The count is a 0-dim float32 tensor
        on the host, as in the reference (lpmm/optim/adamw.py:119); it is advanced through a numpy
        view of the same memory, which costs a fraction of a tensor operation, and the view is
        rebuilt whenever the tensor has been replaced (load_state_dict)."""
        t = state["step"]
        views = self.__dict__.setdefault("_step_views", {})
        hit = views.get(id(state))
        if hit is None or hit[0] is not t:
            if t.device.type != "cpu" or t.dtype != torch.float32 or t.dim() != 0:
                t += 1
                return t.item()
            hit = views[id(state)] = (t, t.numpy())
        view = hit[1]
        view += 1.0
        return float(view)

    def _enabled(self, p, state, name):
        if id(p) in self.override_q_enable:
            return self.override_q_enable[id(p)]
        return state[f"{name}_qstate"]["enable"]

    # ---- step ----------------------------------------------------------------------------
    @torch.no_grad()
    def step(self, closure=None):
        """Performs a single optimization step."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        for group in self.param_groups:
            work = []
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("AdamW does not support sparse gradients")
                state, factored = self._state_of(group, p)
                work.append((p, p.grad, state, factored))
            if not work:
                continue
            if group["fused"]:
                self._step_fused(group, work)
            else:
                self._step_single(group, work)
        return loss

    # ---- fused path (lpmm/optim/adamw.py:439-561) ---------------------------------------
    def _step_fused(self, group, work):
        beta1, beta2 = group["betas"]
        lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
        md_m = self.get_qmetadata_by_state_name("exp_avg")
        md_v = self.get_qmetadata_by_state_name("exp_avg_sq")
        quant, plain, plain16 = {}, {}, {}  # device -> list of records
        factored_work = []
        lib = _native.lib()

        def launch_quant(key, records):
            dev, qm_ptr, qv_ptr = key
            table = np.array(records, dtype=_native.ADAMW4BIT_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_adamw4bit_step_multi(table.ctypes.data, len(records), qm_ptr, qv_ptr, beta1, beta2,
                                                   lr, wd, eps, _native.current_stream(dev))
            _native.check(st, "fused 4-bit AdamW step")

        for p, grad, state, factored in work:
            step = self._next_step(state)
            if factored:
                # the fused kernel does not cover the factored case (adamw.py:472-495)
                factored_work.append((p, grad, state, step))
                continue
            en_m, en_v = self._enabled(p, state, "exp_avg"), self._enabled(p, state, "exp_avg_sq")
            if en_m != en_v:
                raise ValueError("For same tensor, exp_avg and exp_avg_sq should be both quantized or "
                                 f"unquantized simultaneously, but get ({en_m} {en_v})")
            if en_m:
                self._check_fp32_cuda(p, grad, "the 4-bit fused operator reads its float32 scales through the "
                                      "parameters' type, in the reference as well "
                                      "(lpmm/cpp_extension/fused_adamw_kernel.cu:229-230)")
                if md_m["b"] != 4 or md_v["b"] != 4:
                    # the reference's fused kernel reads and writes 4-bit codes whatever the
                    # configuration says (fused_adamw_kernel.cu:113, :157); refuse instead
                    raise ValueError("fused=True supports 4-bit states only; use fused=False for "
                                     f"{md_m['b']}-bit exp_avg / {md_v['b']}-bit exp_avg_sq")
                if md_m["scale_type"] != "group":
                    print("Warning: fused_adamw4bit only support block-wise scaling, but get exp_avg "
                          f"scale_type {md_m['scale_type']}.")
                if md_v["scale_type"] != "group":
                    print("Warning: fused_adamw4bit only support block-wise scaling, but get exp_avg_sq "
                          f"scale_type {md_v['scale_type']}.")
                n = p.numel()
                if n % 2 != 0:
                    # the reference's operator demands numel(exp_avg) == numel(p) // 2
                    # (lpmm/cpp_extension/fused_adamw.cc:68-71) while (numel+1)//2 bytes are allocated
                    raise RuntimeError("number of elements in exp_avg and p tensors should be equal")
                nbytes, blocks = (n + 1) // 2, (n + 127) // 128
                if _is_placeholder(state["exp_avg"]):
                    state["exp_avg"] = torch.zeros((nbytes,), dtype=torch.int8, device=p.device)
                if _is_placeholder(state["exp_avg_sq"]):
                    state["exp_avg_sq"] = torch.zeros((nbytes,), dtype=torch.int8, device=p.device)
                oh_m, oh_v = state["exp_avg_qstate"]["overhead"], state["exp_avg_sq_qstate"]["overhead"]
                if "max1" not in oh_m:
                    oh_m["max1"] = torch.zeros((blocks,), dtype=torch.float32, device=p.device)
                if "max1" not in oh_v:
                    oh_v["max1"] = torch.zeros((blocks,), dtype=torch.float32, device=p.device)
                key = (p.device, state["exp_avg_qstate"]["qmap"].data_ptr(),
                       state["exp_avg_sq_qstate"]["qmap"].data_ptr())
                pending = quant.setdefault(key, [])
                pending.append(
                    (p.data_ptr(), grad.data_ptr(), state["exp_avg"].data_ptr(), state["exp_avg_sq"].data_ptr(),
                     oh_m["max1"].data_ptr(), oh_v["max1"].data_ptr(), n, step, 0.0))
                if len(pending) == _native.MULTI_MAX:
                    # one launch's worth: enqueue it now, so that the GPU works while the host
                    # walks the remaining tensors
                    launch_quant(key, pending)
                    pending.clear()
            else:
                # fp32 states in the parameters' type: float32, or float16 as the reference's operator
                # also accepts (lpmm/cpp_extension/fused_adamw_kernel.cu:188, common.h:15-27)
                half = p.dtype is torch.float16
                if not half:
                    self._check_fp32_cuda(p, grad)
                elif not (grad.dtype is torch.float16 and p.is_cuda and grad.is_cuda and p.is_contiguous()
                          and grad.is_contiguous()):
                    raise RuntimeError("p and g must be contiguous CUDA tensors of the same type (float16)")
                if _is_placeholder(state["exp_avg"]):
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                if _is_placeholder(state["exp_avg_sq"]):
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                if state["exp_avg"].dtype is not p.dtype or state["exp_avg_sq"].dtype is not p.dtype:
                    raise RuntimeError("exp_avg and exp_avg_sq must have the parameter's type")
                (plain16 if half else plain).setdefault(p.device, []).append(
                    (p.data_ptr(), grad.data_ptr(), state["exp_avg"].data_ptr(), state["exp_avg_sq"].data_ptr(),
                     p.numel(), step, 0.0))

        self._factored_steps(group, factored_work)
        for key, records in quant.items():
            if records:
                launch_quant(key, records)
        for dev, records in plain.items():
            table = np.array(records, dtype=_native.ADAMW_FP32_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_adamw_fp32_step_multi(table.ctypes.data, len(records), beta1, beta2, lr, wd, eps,
                                                    _native.current_stream(dev))
            _native.check(st, "fused fp32 AdamW step")
        for dev, records in plain16.items():
            table = np.array(records, dtype=_native.ADAMW_FP32_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_adamw_fp16_step_multi(table.ctypes.data, len(records), beta1, beta2, lr, wd, eps,
                                                    _native.current_stream(dev))
            _native.check(st, "fused fp16 AdamW step")

    @staticmethod
    def _check_fp32_cuda(p, grad, why="the HIP kernels of this path compute in float32 (float16 and float64 parameters "
                         "take the reference's own chain of PyTorch ops on the non-fused path, float16 also the "
                         "fp32-state operator under fused=True; the factored second moment and bfloat16 are "
                         "float32 only)",
                         strided_ok=False):
        if (p.dtype is torch.float32 and grad.dtype is torch.float32 and p.is_cuda and grad.is_cuda
                and (strided_ok or (p.is_contiguous() and grad.is_contiguous()))):
            return
        for t, name in ((p, "p"), (grad, "g")):
            if not t.is_cuda:
                raise RuntimeError(f"{name} must be a CUDA tensor!")
            if not strided_ok and not t.is_contiguous():
                raise RuntimeError(f"{name} must be contiguous!")
            if t.dtype != torch.float32:
                raise RuntimeError(f"The type of {name} is {t.dtype}, float32 is required here: {why}")

    @classmethod
    def _dense_operands(cls, p, grad, held):
        """The parameter and its gradient as the non-fused kernels take them: contiguous float32.
        The reference's non-fused step is a chain of PyTorch ops and accepts any strides
        (lpmm/optim/adamw.py:394-422; its quantiser flattens in index order, functional.py:404-422).
        A strided operand is copied to a contiguous tensor in index order, which leaves every
        value and every quantisation group as they are there.  `held` keeps the copies alive until
        the step's kernels are enqueued (launches are deferred and take raw pointers); the updated
        copy of a strided parameter is written back then (_write_back)."""
        cls._check_fp32_cuda(p, grad, strided_ok=True)
        if p.is_contiguous() and grad.is_contiguous():
            return p, grad
        dense = p if p.is_contiguous() else p.detach().contiguous()
        grad = grad.contiguous()
        held.append((p if dense is not p else None, dense, grad))
        return dense, grad

    @staticmethod
    def _write_back(held):
        for p, dense, _ in held:
            if p is not None:
                p.copy_(dense)
        held.clear()

    @staticmethod
    def _state_stride(p):
        """Strides the reference records for a state of p: those of
        zeros_like(p, memory_format=preserve_format) (lpmm/optim/adamw.py:395, functional.py:32)."""
        if p.is_contiguous():
            return p.stride()
        return torch.empty_like(p, device="meta", memory_format=torch.preserve_format).stride()

    # ---- non-fused path (lpmm/optim/adamw.py:332-436) -----------------------------------
    def _step_single(self, group, work):
        beta1, beta2 = group["betas"]
        lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
        md_m = self.get_qmetadata_by_state_name("exp_avg")
        md_v = self.get_qmetadata_by_state_name("exp_avg_sq")
        lib = _native.lib()
        # both moments 4-bit, first moment block-wise over 128 values, second moment either the
        # same or rank-1 on a 2-D tensor with a multiple of 128 columns: dequantise, update and
        # re-quantise in one kernel (two for rank-1), all such tensors of the group per launch
        def fits(md):
            return md["b"] == 4 and md["round_type"] == "real-nearest"

        m_group128 = fits(md_m) and md_m["scale_type"] == "group" and md_m["gp_sz"] == 128
        v_group128 = fits(md_v) and md_v["scale_type"] == "group" and md_v["gp_sz"] == 128
        v_rank1 = fits(md_v) and md_v["scale_type"] == "rank1"
        # first-moment groups of 256 .. 4096 values (configs/1st_moment_group_*.yml)
        m_group_wide = fits(md_m) and md_m["scale_type"] == "group" and md_m["gp_sz"] in (256, 512, 1024, 2048, 4096)
        batched, batched_rank1, plain = {}, {}, {}
        batched_m32, batched_rank1_m32 = {}, {}  # fp32 first moment, quantised second moment
        batched_rank1_mgroup = {}
        # 5 to 8 bits (configs/default_{5,6,7,8}b.yml): one code per byte, the same two passes
        def wide_codes(md):
            return md["b"] in (5, 6, 7, 8) and md["round_type"] == "real-nearest"

        bits_rank1 = (wide_codes(md_m) and md_m["scale_type"] == "group" and md_m["gp_sz"] == 128
                      and wide_codes(md_v) and md_v["scale_type"] == "rank1")
        batched_rank1_bits = {}
        factored_work = []
        nd_work = {}  # tensors of more than two dimensions that take the two passes (per device and maps)
        held = []  # contiguous copies of strided operands

        def launch_group(key, records):
            dev, qm_ptr, qv_ptr = key
            table = np.array(records, dtype=_native.ADAMW4BIT_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw4bit_step_multi(table.ctypes.data, len(records), qm_ptr, qv_ptr, beta1,
                                                            beta2, lr, wd, eps, _native.current_stream(dev))
            _native.check(st, "non-fused 4-bit AdamW step")

        def launch_rank1(key, records):
            dev, qm_ptr, qv_ptr = key
            table = np.array(records, dtype=_native.NONFUSED_RANK1_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw4bit_rank1_step_multi(table.ctypes.data, len(records), qm_ptr, qv_ptr,
                                                                  beta1, beta2, lr, wd, eps,
                                                                  _native.current_stream(dev))
            _native.check(st, "non-fused 4-bit AdamW step (rank-1 second moment)")
            records.launched()

        half_flat, half_rank1 = {}, {}  # float16 parameters

        def launch_half_flat(key, records):
            dev, qm_ptr, qv_ptr = key
            table = np.array(records, dtype=_native.ADAMW4BIT_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw4bit_f16_step_multi(table.ctypes.data, len(records), qm_ptr, qv_ptr, beta1,
                                                                beta2, lr, wd, eps, _native.current_stream(dev))
            _native.check(st, "non-fused 4-bit AdamW step on float16 parameters")

        def launch_half_rank1(key, records):
            dev, qm_ptr, qv_ptr = key
            table = np.array(records, dtype=_native.NONFUSED_RANK1_F16_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw4bit_rank1_f16_step_multi(table.ctypes.data, len(records), qm_ptr, qv_ptr,
                                                                      beta1, beta2, lr, wd, eps,
                                                                      _native.current_stream(dev))
            _native.check(st, "non-fused 4-bit AdamW step on float16 parameters (rank-1 second moment)")
            records.launched()

        def launch_group_m32(key, records):
            dev, qv_ptr = key
            table = np.array(records, dtype=_native.ADAMW_V4BIT_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw_v4bit_step_multi(table.ctypes.data, len(records), qv_ptr, beta1, beta2,
                                                              lr, wd, eps, _native.current_stream(dev))
            _native.check(st, "non-fused AdamW step (fp32 first moment, 4-bit second moment)")

        def launch_rank1_m32(key, records):
            dev, qv_ptr = key
            table = np.array(records, dtype=_native.RANK1_V4BIT_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw_v4bit_rank1_step_multi(table.ctypes.data, len(records), qv_ptr, beta1,
                                                                    beta2, lr, wd, eps, _native.current_stream(dev))
            _native.check(st, "non-fused AdamW step (fp32 first moment, rank-1 4-bit second moment)")
            records.launched()

        def launch_rank1_mgroup(key, records):
            dev, qm_ptr, qv_ptr = key[:3]
            table = np.array(records, dtype=_native.RANK1_MGROUP_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi(
                    table.ctypes.data, len(records), qm_ptr, qv_ptr, md_m["gp_sz"], beta1, beta2, lr, wd, eps,
                    _native.current_stream(dev))
            _native.check(st, "non-fused 4-bit AdamW step (wide first-moment groups, rank-1 second moment)")
            records.launched()

        def launch_rank1_bits(key, records):
            dev, qm_ptr, qv_ptr, tm_ptr, tv_ptr = key
            table = np.array(records, dtype=_native.NONFUSED_RANK1_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_adamw_bits_rank1_step_multi_table(
                    table.ctypes.data, len(records), qm_ptr, md_m["b"], tm_ptr, qv_ptr, md_v["b"], tv_ptr, beta1, beta2,
                    lr, wd, eps, _native.current_stream(dev))
            _native.check(st, "non-fused AdamW step (5-8-bit states, rank-1 second moment)")
            records.launched()

        for p, grad, state, factored in work:
            step = self._next_step(state)
            if factored:
                factored_work.append((p, grad, state, step))
                continue
            if p.dtype in (torch.float16, torch.float64):
                # float16 with the default kinds of states: the chain of half ops as one or two HIP passes
                kind = self._half_kernel_kind(p, grad, state, m_group128, v_group128, v_rank1)
                if kind is None:
                    self._half_step(group, p, grad, state, step, md_m, md_v)
                    continue
                key = (p.device, state["exp_avg_qstate"]["qmap"].data_ptr(),
                       state["exp_avg_sq_qstate"]["qmap"].data_ptr())
                if kind == "flat":
                    pending = half_flat.setdefault(key, [])
                    pending.append(self._nonfused_record(p, p, grad, state, step, v_rank1))
                    if len(pending) == _native.MULTI_MAX:
                        launch_half_flat(key, pending)
                        pending.clear()
                else:
                    pending = half_rank1.setdefault(key, _Batch())
                    mc, ms = self._group_state(p, state, "exp_avg")
                    pending.append((p.data_ptr(), grad.data_ptr(), mc, ms) + self._rank1_state_f16(p, state, pending)
                                   + (p.shape[0], p.shape[1], step, 0.0))
                    if len(pending) == _native.RANK1_MULTI_MAX:
                        launch_half_rank1(key, pending)
                        pending.clear()
                continue
            dense, grad = self._dense_operands(p, grad, held)
            en_m, en_v = self._enabled(p, state, "exp_avg"), self._enabled(p, state, "exp_avg_sq")
            if m_group128 and en_m and en_v:
                key = (p.device, state["exp_avg_qstate"]["qmap"].data_ptr(),
                       state["exp_avg_sq_qstate"]["qmap"].data_ptr())
                # a vector under 'rank1' is scaled block-wise over 128 values (lpmm/functional.py:192-197)
                if v_group128 or (v_rank1 and p.dim() == 1):
                    pending = batched.setdefault(key, [])
                    pending.append(self._nonfused_record(p, dense, grad, state, step, v_rank1))
                    if len(pending) == _native.MULTI_MAX:  # one launch's worth: enqueue it now
                        launch_group(key, pending)
                        pending.clear()
                    continue
                if v_rank1 and 2 < p.dim() <= RANK1_ND_MAX and _two_pass_nd(p.shape):
                    # a convolution weight and its like, viewed as shape[0] x the rest
                    nd_work.setdefault(key, []).append((p, dense, grad, state, step))
                    continue
                # whole 128-column blocks, or half a block left over with an even row count (taken
                # as double rows: GPT-2-XL's 1600 and 4800 columns)
                if v_rank1 and p.dim() == 2 and (p.shape[1] % 128 == 0
                                                 or (p.shape[1] % 128 == 64 and p.shape[0] % 2 == 0)):
                    pending = batched_rank1.setdefault(key, _Batch())
                    pending.append(self._nonfused_rank1_record(p, dense, grad, state, step, pending))
                    if len(pending) == _native.RANK1_MULTI_MAX:
                        launch_rank1(key, pending)
                        pending.clear()
                    continue
            if bits_rank1 and en_m and en_v and p.dim() == 2 and p.shape[1] % 128 == 0:
                qm, qv = state["exp_avg_qstate"]["qmap"], state["exp_avg_sq_qstate"]["qmap"]
                key = (p.device, qm.data_ptr(), qv.data_ptr(), code_table(qm, md_m["b"]).data_ptr(),
                       code_table(qv, md_v["b"]).data_ptr())
                pending = batched_rank1_bits.setdefault(key, _Batch())
                mc, ms = self._group_state(p, state, "exp_avg", b=md_m["b"])
                pending.append((dense.data_ptr(), grad.data_ptr(), mc, ms) + self._rank1_state(p, state, pending, b=md_v["b"])
                               + (p.shape[0], p.shape[1], step, 0.0))
                if len(pending) == _native.RANK1_MULTI_MAX:
                    launch_rank1_bits(key, pending)
                    pending.clear()
                continue
            # wide first-moment groups, or rows that are no whole number of 128-value groups (a multiple
            # of 8 columns; the two kinds go to different launches: the second takes more general kernels)
            ragged = p.dim() == 2 and p.shape[1] % 128 != 0 and p.shape[1] % 8 == 0
            if (en_m and en_v and v_rank1 and p.dim() == 2
                    and ((m_group_wide and p.shape[1] % 128 == 0) or ((m_group_wide or m_group128) and ragged))):
                key = (p.device, state["exp_avg_qstate"]["qmap"].data_ptr(),
                       state["exp_avg_sq_qstate"]["qmap"].data_ptr(), ragged)
                pending = batched_rank1_mgroup.setdefault(key, _Batch())
                mc, _ = self._group_state(p, state, "exp_avg", md_m["gp_sz"])
                # the scales trade places with a second buffer, like the second moment's statistics
                oh = state["exp_avg_qstate"]["overhead"]
                cur = oh["max1"]
                nxt = self._spare_scales.get(p)
                if nxt is None or nxt.device != cur.device or nxt.shape != cur.shape:
                    nxt = torch.empty_like(cur)

                def commit(p=p, oh=oh, cur=cur, nxt=nxt):
                    self._spare_scales[p] = cur
                    oh["max1"] = nxt

                pending.commits.append(commit)
                pending.append((dense.data_ptr(), grad.data_ptr(), mc, cur.data_ptr(), nxt.data_ptr())
                               + self._rank1_state(p, state, pending) + (p.shape[0], p.shape[1], step, 0.0))
                if len(pending) == _native.RANK1_MULTI_MAX:
                    launch_rank1_mgroup(key, pending)
                    pending.clear()
                continue
            m = self._materialise(p, state, "exp_avg", en_m, md_m)
            if not en_m and en_v:
                # only the second moment is quantised: the first is read and written as floats
                key = (p.device, state["exp_avg_sq_qstate"]["qmap"].data_ptr())
                if v_group128 or (v_rank1 and p.dim() == 1):
                    pending = batched_m32.setdefault(key, [])
                    pending.append((dense.data_ptr(), grad.data_ptr(), m.data_ptr())
                                   + self._group_state(p, state, "exp_avg_sq", rank1_vector=v_rank1)
                                   + (p.numel(), step, 0.0))
                    if len(pending) == _native.V4BIT_MULTI_MAX:
                        launch_group_m32(key, pending)
                        pending.clear()
                    continue
                if v_rank1 and p.dim() == 2 and p.shape[1] % 128 == 0 and m.data_ptr() % 16 == 0:
                    pending = batched_rank1_m32.setdefault(key, _Batch())
                    pending.append((dense.data_ptr(), grad.data_ptr(), m.data_ptr()) + self._rank1_state(p, state, pending)
                                   + (p.shape[0], p.shape[1], step, 0.0))
                    if len(pending) == _native.RANK1_MULTI_MAX:
                        launch_rank1_m32(key, pending)
                        pending.clear()
                    continue
            v = self._materialise(p, state, "exp_avg_sq", en_v, md_v)
            if not en_m and not en_v and m.is_contiguous() and v.is_contiguous():
                # fp32 states (small tensors): all of them in one launch
                plain.setdefault(p.device, []).append(
                    (dense.data_ptr(), grad.data_ptr(), m.data_ptr(), v.data_ptr(), p.numel(), step, 0.0))
                continue
            with torch.cuda.device(p.device):
                st = lib.lpmm_nonfused_update(dense.data_ptr(), grad.data_ptr(), m.data_ptr(), v.data_ptr(), p.numel(),
                                              beta1, beta2, lr, wd, eps, step, _native.current_stream(p.device))
            _native.check(st, "non-fused AdamW update")
            if en_m:
                self._requantise(p, state, "exp_avg", m, md_m)
            if en_v:
                self._requantise(p, state, "exp_avg_sq", v, md_v)
        self._factored_steps(group, factored_work)
        for key, items in nd_work.items():
            self._rank1_nd_steps(group, key, items)
        for dev, records in plain.items():
            table = np.array(records, dtype=_native.ADAMW_FP32_TENSOR)
            with torch.cuda.device(dev):
                st = lib.lpmm_nonfused_update_multi(table.ctypes.data, len(records), beta1, beta2, lr, wd, eps,
                                                    _native.current_stream(dev))
            _native.check(st, "non-fused AdamW update")
        for key, records in batched.items():
            if records:
                launch_group(key, records)
        for key, records in batched_rank1.items():
            if records:
                launch_rank1(key, records)
        for key, records in half_flat.items():
            if records:
                launch_half_flat(key, records)
        for key, records in half_rank1.items():
            if records:
                launch_half_rank1(key, records)
        for key, records in batched_rank1_mgroup.items():
            if records:
                launch_rank1_mgroup(key, records)
        for key, records in batched_rank1_bits.items():
            if records:
                launch_rank1_bits(key, records)
        for key, records in batched_m32.items():
            if records:
                launch_group_m32(key, records)
        for key, records in batched_rank1_m32.items():
            if records:
                launch_rank1_m32(key, records)
        self._write_back(held)

    def _half_kernel_kind(self, p, grad, state, m_group128, v_group128, v_rank1):
        """Which HIP step takes a float16 parameter on the non-fused path: "flat" (one pass: both moments
        block-wise over 128 values, a vector under 'rank1' included), "rank1" (two passes: a matrix with
        a multiple of 128 columns), or None for the chain of PyTorch ops (float64, strided operands,
        unquantised or differently scaled states, states whose scales are not halfs)."""
        if p.dtype is not torch.float16 or grad.dtype is not torch.float16 or not (p.is_cuda and grad.is_cuda):
            return None
        if not (p.is_contiguous() and grad.is_contiguous() and m_group128):
            return None
        if not (self._enabled(p, state, "exp_avg") and self._enabled(p, state, "exp_avg_sq")):
            return None
        for name in ("exp_avg", "exp_avg_sq"):
            if state[f"{name}_qstate"]["qmap"].dtype is not torch.float32:
                return None
            if not _is_placeholder(state[name]):
                oh = state[f"{name}_qstate"]["overhead"]
                scales = [oh["max1"]] if oh.get("max1") is not None else list(oh.get("max_dims", ()))
                if oh.get("dtype") is not torch.float16 or any(t.dtype is not torch.float16 for t in scales):
                    return None
        if v_group128 or (v_rank1 and p.dim() == 1):
            return "flat"
        if (v_rank1 and p.dim() == 2 and p.shape[1] % 128 == 0 and p.shape[0] > 0
                and p.data_ptr() % 16 == 0 and grad.data_ptr() % 16 == 0):
            return "rank1"
        return None

    def _rank1_state_f16(self, p, state, batch):
        """_rank1_state for float16 parameters: half statistics, and a float work array in which the
        kernels take the maxima of the new second moment (kept until the launch is enqueued)."""
        rows, cols = p.shape
        dev = p.device
        qs_v = state["exp_avg_sq_qstate"]
        if _is_placeholder(state["exp_avg_sq"]):
            state["exp_avg_sq"] = torch.full((packed_nbytes(p.numel(), 4),), _zero_byte(qs_v["qmap"]),
                                             dtype=torch.int8, device=dev)
            qs_v["overhead"].clear()
            qs_v["overhead"].update({"dtype": p.dtype, "stride": self._state_stride(p), "dim": 2, "max1": None,
                                     "max_dims": [torch.zeros((rows, 1), dtype=torch.float16, device=dev),
                                                  torch.zeros((1, cols), dtype=torch.float16, device=dev)],
                                     "scaled_shape": p.shape})
        oh = qs_v["overhead"]
        cur = oh["max_dims"]
        nxt = self._spare_stats.get(p)
        if nxt is None or nxt[0].device != dev or nxt[0].dtype is not torch.float16:
            nxt = [torch.empty_like(cur[0]), torch.empty_like(cur[1])]
        work = torch.empty(((rows + 3) // 4 * 4 + cols,), dtype=torch.float32, device=dev)

        def commit(work=work):  # holds the work array until the kernels are on the stream
            self._spare_stats[p] = cur
            oh["max_dims"] = nxt

        batch.commits.append(commit)
        return (state["exp_avg_sq"].data_ptr(), cur[0].data_ptr(), cur[1].data_ptr(), nxt[0].data_ptr(),
                nxt[1].data_ptr(), work.data_ptr())

    def _half_step(self, group, p, grad, state, step, md_m, md_v):
        """float16 (and float64) parameters on the non-fused path.  The reference runs them through
        PyTorch's kernels of that type, every op rounding to it once (lpmm/optim/adamw.py:367-369,
        :394-434), with states, statistics and the scaling in that type (lpmm/functional.py:184-203,
        :97-118); its pack kernel converts every normalised value to float before the search
        (lpmm/cpp_extension/quantization_kernel.cu:450).  The same chain of PyTorch device ops runs
        here, so every rounding falls where it falls there; the code search, packing and unpacking
        are the HIP operators."""
        if not (p.is_cuda and grad.is_cuda):
            raise RuntimeError("p and g must be CUDA tensors!")
        if grad.dtype is not p.dtype:
            raise RuntimeError(f"The type of g is {grad.dtype}: {p.dtype} parameters need gradients of their type "
                               "(the reference's lerp_ raises for mixed types as well)")
        beta1, beta2 = group["betas"]
        lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
        p.mul_(1 - lr * wd)
        moments = []
        for name, md in (("exp_avg", md_m), ("exp_avg_sq", md_v)):
            t = state[name]
            if _is_placeholder(t):
                t = torch.zeros_like(p, memory_format=torch.preserve_format)
            elif self._enabled(p, state, name):
                qstate = state[f"{name}_qstate"]
                kw = dict(qstate["overhead"])
                kw.update(md)
                t = vectorwise_dequant(t, qmap=qstate["qmap"], shape=p.shape, **kw)
            moments.append(t)
        m, v = moments
        m.lerp_(grad, 1 - beta1)
        v.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
        bias_correction1 = 1 - beta1 ** step
        bias_correction2 = 1 - beta2 ** step
        denom = (v.sqrt() / math.sqrt(bias_correction2)).add_(eps)
        p.addcdiv_(m, denom, value=-(lr / bias_correction1))
        for name, t, md in (("exp_avg", m, md_m), ("exp_avg_sq", v, md_v)):
            if self._enabled(p, state, name):
                qstate = state[f"{name}_qstate"]
                qx, gen = vectorwise_quant(t, qmap=qstate["qmap"], shape=p.shape, **md)
                state[name] = qx
                qstate["overhead"].clear()
                qstate["overhead"].update(gen)
            else:
                state[name] = t

    def _group_state(self, p, state, name, gp_sz=128, b=4, rank1_vector=False):
        """Pointers to the codes and scales of a state with block-wise scaling over gp_sz values;
        creates the state on first use: an all-zero moment in the layout and with the metadata
        vectorwise_quant gives it (lpmm/optim/adamw.py:425-434).  With zero scales every code decodes
        to zero, and the first step overwrites the codes in full: for widths other than 4 bits the
        array starts as zero bytes."""
        groups = (p.numel() + gp_sz - 1) // gp_sz
        qstate = state[f"{name}_qstate"]
        if _is_placeholder(state[name]):
            state[name] = torch.full((packed_nbytes(groups * gp_sz, b),), _zero_byte(qstate["qmap"]) if b == 4 else 0,
                                     dtype=torch.int8, device=p.device)
            oh = qstate["overhead"]
            oh.clear()
            oh.update({"dtype": p.dtype, "stride": self._state_stride(p),
                       # scales take the state's type (lpmm/functional.py:187: a maximum of the tensor's values)
                       "max1": torch.zeros((groups, 1), device=p.device,
                                           dtype=torch.float16 if p.dtype is torch.float16 else torch.float32),
                       "scaled_shape": torch.Size((groups, gp_sz))})
            if rank1_vector:  # the 'rank1' branch records the dimension count (lpmm/functional.py:191)
                oh["dim"] = 1
        return state[name].data_ptr(), qstate["overhead"]["max1"].data_ptr()

    def _rank1_state(self, p, state, batch, b=4):
        """Pointers to the codes of a rank-1 scaled second moment, the statistics they are scaled
        by and the pair of buffers that receives the next statistics; creates the state on first
        use.  The kernels leave the statistics of the new second moment in the second pair; the
        pairs trade places once the launch is enqueued (`batch.launched()`), so that the state's
        `max_dims` always are the statistics its codes are scaled by, also after a step that raised."""
        rows, cols = p.shape
        dev = p.device
        qs_v = state["exp_avg_sq_qstate"]
        if _is_placeholder(state["exp_avg_sq"]):
            state["exp_avg_sq"] = torch.full((packed_nbytes(p.numel(), b),), _zero_byte(qs_v["qmap"]) if b == 4 else 0,
                                             dtype=torch.int8, device=dev)
            qs_v["overhead"].clear()
            qs_v["overhead"].update({"dtype": p.dtype, "stride": self._state_stride(p), "dim": 2, "max1": None,
                                     "max_dims": [torch.zeros((rows, 1), dtype=torch.float32, device=dev),
                                                  torch.zeros((1, cols), dtype=torch.float32, device=dev)],
                                     "scaled_shape": p.shape})
        oh = qs_v["overhead"]
        cur = oh["max_dims"]
        nxt = self._spare_stats.get(p)
        if nxt is None or nxt[0].device != dev:
            nxt = [torch.empty_like(cur[0]), torch.empty_like(cur[1])]

        def commit():
            self._spare_stats[p] = cur
            oh["max_dims"] = nxt

        batch.commits.append(commit)
        return (state["exp_avg_sq"].data_ptr(), cur[0].data_ptr(), cur[1].data_ptr(), nxt[0].data_ptr(),
                nxt[1].data_ptr())

    def _nonfused_record(self, p, dense, grad, state, step, rank1_vector=False):
        """The tensor's record for the one-pass non-fused step."""
        mc, ms = self._group_state(p, state, "exp_avg")
        vc, vs = self._group_state(p, state, "exp_avg_sq", rank1_vector=rank1_vector)
        return (dense.data_ptr(), grad.data_ptr(), mc, vc, ms, vs, p.numel(), step, 0.0)

    def _nonfused_rank1_record(self, p, dense, grad, state, step, batch):
        """The tensor's record for the two-pass step with a rank-1 second moment."""
        mc, ms = self._group_state(p, state, "exp_avg")
        return (dense.data_ptr(), grad.data_ptr(), mc, ms) + self._rank1_state(p, state, batch) + (
            p.shape[0], p.shape[1], step, 0.0)

    def _rank1_nd_steps(self, group, key, items):
        """The two-pass step on tensors of 3 to 8 dimensions (default configuration: first moment in
        groups of 128 values, rank-1 second moment).  The reference's scale of such a tensor is the
        minimum over all its dimensions' statistics (lpmm/functional.py:503-531).  Viewed as
        shape[0] x (numel / shape[0]) that is min(statistic of row, column scale) with the column
        scale the minimum over the trailing dimensions' statistics, so the kernels for matrices apply,
        one pass at a time: the column scale of the current statistics goes in as the column
        statistics of pass 1; what pass 1 leaves as column maxima of the new second moment is folded
        into the next statistics of the trailing dimensions (lpmm_rank1_stats_nd on a vector of
        shape[1:]), and their column scale is what pass 2 divides by.  The statistics of dimension 0
        are the row statistics of the passes as they are."""
        dev, qm_ptr, qv_ptr = key
        lib = _native.lib()
        beta1, beta2 = group["betas"]
        lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
        batch = _Batch()
        first, second, between = [], [], []
        with torch.cuda.device(dev):
            stream = _native.current_stream(dev)
            for p, dense, grad, state, step in items:
                rows, cols = p.shape[0], p.numel() // p.shape[0]
                trailing = tuple(p.shape[1:]) + (1,)  # lpmm_rank1_row_scale_nd leaves the last dimension out
                mc, ms = self._group_state(p, state, "exp_avg")
                vc, cur, nxt = self._rank1_nd_state(p, state, batch)
                scratch = self._nd_scratch.get(p)
                if scratch is None or scratch["work"].device != p.device:
                    scratch = self._nd_scratch[p] = {
                        "work": torch.empty((3, cols), dtype=torch.float32, device=p.device), "scale_of": None, "row": 0}
                work = scratch["work"]
                # rows of `work`: the column scale of the current statistics, the column maxima of the new
                # second moment, the column scale of the next statistics.  The last step's third row is this
                # step's first as long as the state still holds the statistics that step left
                if scratch["scale_of"] is cur:
                    old_row = scratch["row"]
                else:
                    old_row = 0
                    st = lib.lpmm_rank1_row_scale_nd(_ptr_array(cur[1:] + [cur[0]]), len(trailing),
                                                     _shape_array(trailing), work[0].data_ptr(), stream)
                    _native.check(st, "rank1_row_scale_nd")
                raw_row, new_row = [r for r in range(3) if r != old_row]
                head = (dense.data_ptr(), grad.data_ptr(), mc, ms, vc, cur[0].data_ptr(), work[old_row].data_ptr(),
                        nxt[0].data_ptr())
                tail = (rows, cols, step, 0.0)
                first.append(head + (work[raw_row].data_ptr(),) + tail)
                second.append(head + (work[new_row].data_ptr(),) + tail)
                between.append((p, nxt, work[raw_row], work[new_row], trailing))

                def remember(scratch=scratch, nxt=nxt, new_row=new_row):
                    scratch["scale_of"], scratch["row"] = nxt, new_row

                batch.commits.append(remember)
            for pass_no, records in ((1, first), (2, second)):
                for i in range(0, len(records), _native.RANK1_MULTI_MAX):
                    chunk = np.array(records[i:i + _native.RANK1_MULTI_MAX], dtype=_native.NONFUSED_RANK1_TENSOR)
                    st = lib.lpmm_nonfused_adamw4bit_rank1_pass_multi(chunk.ctypes.data, len(chunk), qm_ptr, qv_ptr, beta1,
                                                                      beta2, lr, wd, eps, pass_no, stream)
                    _native.check(st, f"non-fused 4-bit AdamW step on tensors of more than two dimensions, pass {pass_no}")
                if pass_no == 1:
                    # the column maxima of the new second moment -> next statistics of the trailing dimensions
                    # -> their column scale: one launch for all tensors whose statistics fit a workgroup's LDS
                    # (every convolution weight), two calls per tensor otherwise
                    small = []
                    for p, nxt, raw, scale, trailing in between:
                        dims = tuple(p.shape[1:])
                        # one workgroup per vector: for the few thousand values of a convolution weight's
                        # trailing dimensions, not for the millions of a stack of matrices
                        if sum(dims) <= _native.RANK1_SMALL_SLOTS and raw.numel() <= _native.RANK1_SMALL_VALUES:
                            pad = 7 - len(dims)
                            small.append((raw.data_ptr(), scale.data_ptr(), tuple(t.data_ptr() for t in nxt[1:]) + (0,) * pad,
                                          dims + (1,) * pad, len(dims), 0))
                            continue
                        st = lib.lpmm_rank1_stats_nd(raw.data_ptr(), p.dim() - 1, _shape_array(dims),
                                                     _ptr_array(nxt[1:]), None, stream)
                        _native.check(st, "rank1_stats_nd")
                        st = lib.lpmm_rank1_row_scale_nd(_ptr_array(nxt[1:] + [nxt[0]]), len(trailing),
                                                         _shape_array(trailing), scale.data_ptr(), stream)
                        _native.check(st, "rank1_row_scale_nd")
                    if small:
                        vectors = np.array(small, dtype=_native.RANK1_SMALL_VECTOR)
                        st = lib.lpmm_rank1_small_fold_scale_multi(vectors.ctypes.data, len(small), stream)
                        _native.check(st, "rank1_small_fold_scale_multi")
        batch.launched()

    def _rank1_nd_state(self, p, state, batch):
        """_rank1_state for a tensor of more than two dimensions: one statistic per dimension, in the
        shapes get_sm3_statistics gives them (lpmm/functional.py:512-531)."""
        dev = p.device
        qs_v = state["exp_avg_sq_qstate"]
        if _is_placeholder(state["exp_avg_sq"]):
            state["exp_avg_sq"] = torch.full((packed_nbytes(p.numel(), 4),), _zero_byte(qs_v["qmap"]), dtype=torch.int8,
                                             device=dev)
            stats = []
            for i, n in enumerate(p.shape):
                keep = [1] * p.dim()
                keep[i] = n
                stats.append(torch.zeros(keep, dtype=torch.float32, device=dev))
            qs_v["overhead"].clear()
            qs_v["overhead"].update({"dtype": p.dtype, "stride": self._state_stride(p), "dim": p.dim(), "max1": None,
                                     "max_dims": stats, "scaled_shape": p.shape})
        oh = qs_v["overhead"]
        cur = oh["max_dims"]
        nxt = self._spare_stats.get(p)
        if nxt is None or len(nxt) != len(cur) or nxt[0].device != dev:
            nxt = [torch.empty_like(t) for t in cur]

        def commit():
            self._spare_stats[p] = cur
            oh["max_dims"] = nxt

        batch.commits.append(commit)
        return state["exp_avg_sq"].data_ptr(), cur, nxt

    @property
    def _nd_scratch(self):
        # three vectors of numel / shape[0] floats per tensor of more than two dimensions (the column
        # scale of the current statistics, the column maxima of the new second moment, the column
        # scale of the next statistics) and which statistics the kept scale belongs to; not part of
        # the optimizer state
        d = self.__dict__.get("_nd_scratch_by_param")
        if d is None:
            d = self.__dict__["_nd_scratch_by_param"] = {}
        return d

    @property
    def _spare_stats(self):
        # second pair of row/column statistics per parameter; not part of the optimizer state
        # (its contents are only meaningful during a step)
        d = self.__dict__.get("_spare_stats_by_param")
        if d is None:
            d = self.__dict__["_spare_stats_by_param"] = {}
        return d

    @property
    def _spare_scales(self):
        # second buffer of first-moment scales per parameter (wide groups); not part of the state
        d = self.__dict__.get("_spare_scales_by_param")
        if d is None:
            d = self.__dict__["_spare_scales_by_param"] = {}
        return d

    def _materialise(self, p, state, name, enabled, md):
        """Contiguous fp32 tensor of a state for the update, in the parameter's index order:
        zeros at the first step, the dequantised tensor when quantised, the state itself
        otherwise (adamw.py:394-409).  The reference gives the tensor the strides its metadata
        records; the kernels here work on the contiguous form of the same values."""
        t = state[name]
        if _is_placeholder(t):
            state[name] = t = torch.zeros_like(p, memory_format=torch.contiguous_format)
            return t
        if enabled:
            qstate = state[f"{name}_qstate"]
            kw = dict(qstate["overhead"])
            kw.update(md)
            kw["stride"] = None  # no re-striding of the temporary
            return vectorwise_dequant(t, qmap=qstate["qmap"], shape=p.shape, **kw)
        if not t.is_contiguous():  # e.g. loaded from a checkpoint of a strided parameter
            state[name] = t = t.contiguous()
        return t

    def _requantise(self, p, state, name, x, md):
        qstate = state[f"{name}_qstate"]
        qx, gen = vectorwise_quant(x, qmap=qstate["qmap"], shape=p.shape, **md)
        gen["stride"] = self._state_stride(p)
        state[name] = qx
        qstate["overhead"].clear()
        qstate["overhead"].update(gen)

    # ---- factored second moment (lpmm/optim/adamw.py:579-627) ---------------------------
    def _factored_steps(self, group, items):
        """Factored tensors of a parameter group: 2-D tensors with a multiple of 128 columns and a
        4-bit block-wise first moment go to the multi-tensor kernels together, the others one
        by one."""
        if not items:
            return
        beta1, beta2 = group["betas"]
        lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
        md_m = self.get_qmetadata_by_state_name("exp_avg")
        m_fits = (md_m["scale_type"] == "group" and md_m["gp_sz"] == 128 and md_m["b"] == 4
                  and md_m["round_type"] == "real-nearest")
        lib = _native.lib()
        batched = {}
        held = []  # contiguous copies of strided operands
        for p, grad, state, step in items:
            dense, grad = self._dense_operands(p, grad, held)
            if not (m_fits and p.dim() == 2 and p.shape[1] % 128 == 0 and self._enabled(p, state, "exp_avg")):
                self._factored_step(group, p, dense, grad, state, step)
                continue
            rows, cols = p.shape
            qstate = state["exp_avg_qstate"]
            first = _is_placeholder(state["exp_avg"])
            if first:
                groups = p.numel() // 128
                state["exp_avg"] = torch.empty((packed_nbytes(p.numel()),), dtype=torch.int8, device=p.device)
                qstate["overhead"].clear()
                qstate["overhead"].update({"dtype": p.dtype, "stride": self._state_stride(p),
                                           "max1": torch.empty((groups, 1), dtype=torch.float32, device=p.device),
                                           "scaled_shape": torch.Size((groups, 128))})
            key = (p.device, qstate["qmap"].data_ptr())
            ws = (lib.lpmm_factored_workspace_bytes(rows, cols) + 255) // 256 * 256
            batched.setdefault(key, []).append(
                [dense.data_ptr(), grad.data_ptr(), state["exp_avg"].data_ptr(), qstate["overhead"]["max1"].data_ptr(),
                 state["exp_avg_sq_row"].data_ptr(), state["exp_avg_sq_col"].data_ptr(), ws, rows, cols, step,
                 1 if first else 0])
        for (dev, qm_ptr), records in batched.items():
            with torch.cuda.device(dev):
                work = torch.empty((sum(r[6] for r in records),), dtype=torch.uint8, device=dev)
                offset = work.data_ptr()
                for r in records:
                    r[6], offset = offset, offset + r[6]
                table = np.array([tuple(r) for r in records], dtype=_native.FACTORED_TENSOR)
                st = lib.lpmm_factored_step_multi(table.ctypes.data, len(records), qm_ptr, beta1, beta2, lr, wd, eps,
                                                  _native.current_stream(dev))
            _native.check(st, "factored step")
        self._write_back(held)

    def _factored_step(self, group, p, dense, grad, state, step):
        """One factored tensor outside the multi-tensor launch; `dense` is p or its contiguous copy."""
        beta1, beta2 = group["betas"]
        lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
        lib = _native.lib()
        dev = p.device
        rows, cols = p.shape[-2], p.shape[-1]
        batch = p.numel() // (rows * cols)  # leading dimensions: independent R x C matrices
        row, col = state["exp_avg_sq_row"], state["exp_avg_sq_col"]
        en_m = self._enabled(p, state, "exp_avg")
        md_m = self.get_qmetadata_by_state_name("exp_avg")
        qstate = state["exp_avg_qstate"]
        one_pass = (batch == 1 and en_m and md_m["scale_type"] == "group" and md_m["gp_sz"] == 128
                    and md_m["b"] == 4 and md_m["round_type"] == "real-nearest")
        with torch.cuda.device(dev):
            stream = _native.current_stream(dev)
            work = torch.empty((lib.lpmm_factored_workspace_bytes(rows, cols),), dtype=torch.uint8, device=dev)
            mean_all = torch.empty((batch,), dtype=torch.float32, device=dev)
            for b in range(batch):
                st = lib.lpmm_factored_stats(grad.data_ptr() + 4 * b * rows * cols, rows, cols,
                                             row.data_ptr() + 4 * b * rows, col.data_ptr() + 4 * b * cols,
                                             mean_all.data_ptr() + 4 * b, beta2, work.data_ptr(), stream)
                _native.check(st, "factored statistics")
            if one_pass:
                first = _is_placeholder(state["exp_avg"])
                groups = (p.numel() + 127) // 128
                if first:
                    state["exp_avg"] = torch.empty((packed_nbytes(groups * 128),), dtype=torch.int8, device=dev)
                    max1 = torch.empty((groups, 1), dtype=torch.float32, device=dev)
                else:
                    max1 = qstate["overhead"]["max1"]
                st = lib.lpmm_factored_update(dense.data_ptr(), grad.data_ptr(), state["exp_avg"].data_ptr(),
                                              max1.data_ptr(), qstate["qmap"].data_ptr(), row.data_ptr(),
                                              col.data_ptr(), mean_all.data_ptr(), rows, cols, beta1, beta2, lr, wd,
                                              eps, step, 1 if first else 0, stream)
                _native.check(st, "factored update")
                qstate["overhead"].clear()
                qstate["overhead"].update({"dtype": p.dtype, "stride": self._state_stride(p), "max1": max1,
                                           "scaled_shape": torch.Size((groups, 128))})
                return
            m = self._materialise(p, state, "exp_avg", en_m, md_m)
            for b in range(batch):
                off = 4 * b * rows * cols
                st = lib.lpmm_factored_update_fp32m(dense.data_ptr() + off, grad.data_ptr() + off, m.data_ptr() + off,
                                                    row.data_ptr() + 4 * b * rows, col.data_ptr() + 4 * b * cols,
                                                    mean_all.data_ptr() + 4 * b, rows, cols, beta1, beta2, lr, wd,
                                                    eps, step, stream)
                _native.check(st, "factored update")
            if en_m:
                self._requantise(p, state, "exp_avg", m, md_m)
