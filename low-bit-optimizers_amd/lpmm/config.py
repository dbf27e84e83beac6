"""Quantisation config of the 4-bit optimizer-state path, without yacs.

Mirrors the part of lpmm/config.py that the optimizer reads: the per-state nodes QUANT.M
(first moment) and QUANT.SQM (second moment) with the keys ENABLE, THRESHOLD, BITS,
SCALE_TYPE.DEFAULT, QUANT_TYPE.DEFAULT, ROUND_TYPE, GROUP_SIZE, SIGNED
(lpmm/config.py:35-65), built-in defaults equal to the reference's `_C`, and YAML files
merged over them with `BASE` inheritance (lpmm/config.py:82-94).  `get_config(None)`
returns the defaults, `get_config("file.yml")` the merged config (lpmm/config.py:181-189).
Unlike the reference, building a config prints nothing and writes no file.
"""
import copy
import os

import yaml

__all__ = ["Node", "get_config", "config_from_mapping", "to_plain", "CONFIG_DIR"]

CONFIG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "configs")


class Node(dict):
    """Nested dict with attribute access (the subset of yacs' CfgNode the optimizer uses)."""

    def __getattr__(self, name):
        try:
            return self[name]
        except KeyError:
            raise AttributeError(name) from None

    def __setattr__(self, name, value):
        self[name] = value

    def clone(self):
        return copy.deepcopy(self)

    def merge(self, other):
        for key, value in other.items():
            if isinstance(value, dict) and isinstance(self.get(key), dict):
                self[key].merge(value)
            else:
                self[key] = _to_node(value)
        return self

    def __str__(self):
        return yaml.safe_dump(_to_plain(self), default_flow_style=False, sort_keys=True)


def _to_node(value):
    if isinstance(value, dict):
        return Node({k: _to_node(v) for k, v in value.items()})
    return value


def _to_plain(value):
    if isinstance(value, dict):
        return {k: _to_plain(v) for k, v in value.items()}
    return value


def to_plain(config):
    """The config as nested builtin dicts (what a checkpoint stores)."""
    return _to_plain(config)


def config_from_mapping(mapping):
    """A config node from any nested mapping that carries the optimizer's keys (a plain dict
    from a checkpoint, a Node, a yacs CfgNode).  Raises if QUANT.M / QUANT.SQM are missing."""
    if not isinstance(mapping, dict):
        raise TypeError(f"qconfig of a checkpoint must be a mapping, not {type(mapping).__name__}")
    node = _to_node(_to_plain(mapping))
    for state in ("M", "SQM"):
        sub = node.get("QUANT", {}).get(state)
        missing = [k for k in ("ENABLE", "THRESHOLD", "BITS", "SCALE_TYPE", "QUANT_TYPE", "ROUND_TYPE", "GROUP_SIZE",
                               "SIGNED") if sub is None or k not in sub]
        if missing:
            raise ValueError(f"qconfig of the checkpoint lacks QUANT.{state} keys {missing}")
    return node


def _state_node(bits, scale_type, quant_type, round_type, group_size, signed, enable=True):
    return dict(
        ENABLE=enable,
        THRESHOLD=4096,
        EXCLUDE_SUFFIX=[""],
        EXCLUDE_REGEX=[""],
        BITS=bits,
        SCALE_TYPE=dict(DEFAULT=scale_type, DEFAULT_ONLY=True),
        QUANT_TYPE=dict(DEFAULT=quant_type, DEFAULT_ONLY=True),
        ROUND_TYPE=round_type,
        GROUP_SIZE=group_size,
        SIGNED=signed,
    )


# Built-in defaults: the values of lpmm/config.py:7-79.  Note SQM.SCALE_TYPE.DEFAULT is
# 'group' here; 'rank1' comes only from configs/default.yml.
_DEFAULTS = _to_node(dict(
    BASE=[""],
    QUANT=dict(
        INIT_STATES=["param"],
        P=_state_node(8, "group", "linear", "sr", 64, True, enable=False),
        G=dict(ENABLE=False, THRESHOLD=4096),
        M=_state_node(4, "group", "nonlinear", "real-nearest", 128, True),
        SQM=_state_node(4, "group", "power-1", "real-nearest", 128, False),
        DEBUG=dict(TRUNCATED_RATE_STAT_ITER=False, ROW_ABSMAX_STAT_ITER=False,
                   ROW_ABSMAX_STAT_EPOCH=False),
    ),
    TRAIN=dict(),
    OUTPUT=".",
    TAG="",
    LOCAL_RANK=0,
))


def _merge_file(config, path):
    with open(path, "r") as f:
        loaded = yaml.safe_load(f) or {}
    for base in loaded.get("BASE", [""]):
        if base:
            _merge_file(config, os.path.join(os.path.dirname(path), base))
    config.merge(loaded)


def get_config(args=None):
    """None -> built-in defaults; str -> defaults merged with that YAML file."""
    config = _DEFAULTS.clone()
    if isinstance(args, str):
        _merge_file(config, args)
    elif isinstance(args, dict):
        config.merge(args)
    elif args is not None:
        raise TypeError("qconfig must be None, a path to a YAML file or a Node/dict, "
                        f"not {type(args).__name__}")
    return config
