"""Base class of the low-bit optimizers: quantisation config, per-state quantisation
records and checkpointing.  Same public surface as lpmm/optim/optimizer.py:14-163."""
from collections import defaultdict
from collections.abc import Iterable
from copy import deepcopy
from itertools import chain

import torch

from ..config import config_from_mapping, get_config, to_plain
from ..functional import create_general_qmap

__all__ = ["LowBitOptimizer"]


def _quantize_enabled(p, prior_enable, threshold):
    """A state is quantised iff its config enables it and the tensor has more than
    `threshold` elements (lpmm/optim/optimizer.py:156-163)."""
    if not prior_enable:
        return False
    if threshold is not None and p.numel() <= threshold:
        return False
    return True


class LowBitOptimizer(torch.optim.Optimizer):
    def __init__(self, params, defaults, config):
        super().__init__(params, defaults)
        self.qconfig = get_config(config)
        self.override_q_enable = {}
        self.qmaps = {}

    # ---- per-state quantisation records ------------------------------------------------
    def override_quantize_enable(self, module, param_name, enable):
        """Force quantisation on/off for one parameter before its state exists
        (lpmm/optim/optimizer.py:28-34)."""
        p = getattr(module, param_name)
        assert p is not None
        assert isinstance(p, torch.Tensor)
        if len(self.state[p]) != 0:
            raise ValueError("overriding enabling of quantized parameters is prohibited after state initialization.")
        self.override_q_enable[id(p)] = enable

    def get_qmetadata_by_state_name(self, optimizer_state_name):
        """The six fields the quantise/dequantise entry points take
        (lpmm/optim/optimizer.py:56-66)."""
        sub = self.get_subqconfig(optimizer_state_name)
        return dict(
            b=sub.BITS,
            scale_type=sub.SCALE_TYPE.DEFAULT,
            quant_type=sub.QUANT_TYPE.DEFAULT,
            round_type=sub.ROUND_TYPE,
            gp_sz=sub.GROUP_SIZE,
            signed=sub.SIGNED,
        )

    def init_qstate(self, p, state_name):
        """Create state[f"{state_name}_qstate"] = {enable, overhead, qmap}; maps are cached per
        (quant_type, bits, signed) and moved to the parameter's device
        (lpmm/optim/optimizer.py:36-54)."""
        sub = self.get_subqconfig(state_name)
        md = self.get_qmetadata_by_state_name(state_name)
        key = (md["quant_type"], md["b"], md["signed"])
        if key not in self.qmaps:
            self.qmaps[key] = create_general_qmap(*key)
        self.qmaps[key] = self.qmaps[key].to(p.device)
        self.state[p][f"{state_name}_qstate"] = {
            "enable": _quantize_enabled(p, sub.ENABLE, sub.THRESHOLD),
            "overhead": dict(),
            "qmap": self.qmaps[key],
        }

    # ---- checkpointing -----------------------------------------------------------------
    def state_dict(self):
        """torch's state dict plus 'qconfig' (lpmm/optim/optimizer.py:68-71).  The config is
        stored as a plain nested dict with the reference's keys, so that the checkpoint holds
        builtin types and tensors only and loads with `torch.load(..., weights_only=True)`;
        the reference stores its yacs CfgNode object, which needs yacs to unpickle."""
        out = super().state_dict()
        out["qconfig"] = to_plain(self.qconfig)
        return out

    def load_state_dict(self, state_dict):
        """Restore a state_dict().  Tensors move to their parameter's device; floating-point
        state follows the parameter's dtype, except `step`, the packed int8 code tensors and the
        quantisation maps, which are kept as they are (lpmm/optim/optimizer.py:73-136)."""
        # any mapping with the reference's keys: the plain dict written by state_dict() above, a
        # config node of this package, or a yacs CfgNode (a dict subclass) from a reference checkpoint
        self.qconfig = config_from_mapping(state_dict["qconfig"])
        state_dict = deepcopy(state_dict)
        groups, saved_groups = self.param_groups, state_dict["param_groups"]
        if len(groups) != len(saved_groups):
            raise ValueError("loaded state dict has a different number of parameter groups")
        if any(len(g["params"]) != len(s["params"]) for g, s in zip(groups, saved_groups)):
            raise ValueError("loaded state dict contains a parameter group "
                             "that doesn't match the size of optimizer's group")
        id_map = dict(zip(chain.from_iterable(g["params"] for g in saved_groups),
                          chain.from_iterable(g["params"] for g in groups)))

        def place(param, value, key=None):
            if isinstance(value, torch.Tensor):
                if key == "step":
                    return value
                if key == "qmap":
                    # the maps stay float32 whatever the parameter's type: the kernels (here and in the
                    # reference, lpmm/cpp_extension/quantization_kernel.cu:496, :648: data_ptr<float>()) read them as floats,
                    # and a map rounded to half would decode the saved codes to other values.  The reference
                    # casts them with the rest (:107-108) and cannot step float16 parameters after a load.
                    return value.to(param.device)
                if param.is_floating_point() and value.dtype != torch.int8:
                    value = value.to(param.dtype)
                return value.to(param.device)
            if isinstance(value, dict):
                return {k: place(param, v, key=k) for k, v in value.items()}
            if isinstance(value, Iterable) and not isinstance(value, (str, bytes)):
                return type(value)(place(param, v) for v in value)
            return value

        state = defaultdict(dict)
        for k, v in state_dict["state"].items():
            if k in id_map:
                state[id_map[k]] = place(id_map[k], v)
            else:
                state[k] = v
        new_groups = []
        for g, s in zip(groups, saved_groups):
            s["params"] = g["params"]
            new_groups.append(s)
        self.__setstate__({"state": state, "param_groups": new_groups})
        self._intern_qmaps()

    def _intern_qmaps(self):
        """After a load every state holds its own copy of its quantisation map.  States whose
        map has the same contents share one tensor again (the optimizer's cached map where it
        is the same), as they do after init_qstate: the multi-tensor launches group tensors by
        their maps, and hundreds of 64-byte device tensors would be wasted otherwise."""
        pool = {}
        for key, qmap in self.qmaps.items():
            if isinstance(qmap, torch.Tensor):
                pool[(qmap.device, qmap.dtype, tuple(qmap.tolist()))] = qmap
        for state in self.state.values():
            if not isinstance(state, dict):
                continue
            for name, qstate in state.items():
                if not (isinstance(name, str) and name.endswith("_qstate") and isinstance(qstate, dict)):
                    continue
                qmap = qstate.get("qmap")
                if not isinstance(qmap, torch.Tensor):
                    continue
                key = (qmap.device, qmap.dtype, tuple(qmap.tolist()))
                qstate["qmap"] = shared = pool.setdefault(key, qmap)
                # states created after the load (init_qstate) should pick up the same tensor
                try:
                    md = self.get_qmetadata_by_state_name(name[: -len("_qstate")])
                except (ValueError, NotImplementedError):
                    continue
                ckey = (md["quant_type"], md["b"], md["signed"])
                if ckey not in self.qmaps:
                    self.qmaps[ckey] = create_general_qmap(*ckey)
                cached = self.qmaps[ckey]
                if cached is not shared and tuple(cached.tolist()) == key[2] and cached.dtype == shared.dtype:
                    self.qmaps[ckey] = shared

    # ---- to be provided by subclasses --------------------------------------------------
    @torch.no_grad()
    def step(self, closure=None):
        raise NotImplementedError("The step method needs overriding")

    def get_subqconfig(self, optimizer_state_name):
        raise NotImplementedError("The get_subconfig method needs overriding")
