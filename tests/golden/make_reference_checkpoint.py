#!/usr/bin/env python3
"""Writes tests/golden/reference_shaped_checkpoints.pt: two optimizer state dicts laid out by
hand the way the reference's lpmm.optim.AdamW.state_dict() lays them out, as builtin
containers and tensors only (readable with torch.load(..., weights_only=True)).

Nothing here imports or runs the reference; the layout is typed from its sources:

* top level {'state', 'param_groups', 'qconfig'}: torch's Optimizer.state_dict() plus the
  'qconfig' entry (lpmm/optim/optimizer.py:68-71).  The reference stores its yacs CfgNode there,
  a dict subclass; the fixture holds the same keys and values (lpmm/config.py:7-79, with
  lpmm/configs/default.yml:11-18 merged for the second dict) as a plain nested dict.
* param_groups: the constructor's defaults plus 'params' as indices (lpmm/optim/adamw.py:38-46).
* per-parameter state, in creation order (lpmm/optim/adamw.py:114-129, lpmm/optim/optimizer.py:36-54):
  'step' (0-dim float32 on the host), 'exp_avg', 'exp_avg_qstate' = {'enable', 'overhead', 'qmap'},
  'exp_avg_sq', 'exp_avg_sq_qstate'.
* "fused": quantised tensors hold int8[(numel+1)//2] codes and float32[ceil(numel/128)] scales in
  overhead['max1'] (lpmm/optim/adamw.py:508-523); tensors at or under the threshold hold float32
  moments (:543-547) and an empty overhead.
* "nonfused_default": what vectorwise_quant leaves after a step with lpmm/configs/default.yml
  (lpmm/optim/adamw.py:425-434, lpmm/functional.py:32-34, :184-203, :240, :359-369): int8 codes of
  ceil(numel_scaled/2048)*1024 + 1 bytes (the last byte is uninitialised there; 0x5A here),
  overhead {'dtype', 'stride', 'max1' (G,1), 'scaled_shape' (G,128)} for the first moment and
  {'dtype', 'stride', 'dim', 'max_dims' [(R,1), (1,C)], 'max1' None, 'scaled_shape'} for the
  rank-1 second moment.

The moments behind the codes are seeded random tensors quantised by this repository's CPU oracle,
so every state is self-consistent (each group's largest element carries code 15 or 0).
Run from the repository root:  python tests/golden/make_reference_checkpoint.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import oracle as O  # noqa: E402

SHAPES = [(40, 256), (1600,)]
STEP = 5.0


def state_node(bits, scale_type, quant_type, round_type, group_size, signed, enable):
    return {"ENABLE": enable, "THRESHOLD": 4096, "EXCLUDE_SUFFIX": [""], "EXCLUDE_REGEX": [""], "BITS": bits,
            "SCALE_TYPE": {"DEFAULT": scale_type, "DEFAULT_ONLY": True},
            "QUANT_TYPE": {"DEFAULT": quant_type, "DEFAULT_ONLY": True},
            "ROUND_TYPE": round_type, "GROUP_SIZE": group_size, "SIGNED": signed}


def qconfig(v_scale_type):
    return {
        "BASE": [""],
        "QUANT": {
            "INIT_STATES": ["param"],
            "P": state_node(8, "group", "linear", "sr", 64, True, False),
            "G": {"ENABLE": False, "THRESHOLD": 4096},
            "M": state_node(4, "group", "nonlinear", "real-nearest", 128, True, True),
            "SQM": state_node(4, v_scale_type, "power-1", "real-nearest", 128, False, True),
            "DEBUG": {"TRUNCATED_RATE_STAT_ITER": False, "ROW_ABSMAX_STAT_ITER": False,
                      "ROW_ABSMAX_STAT_EPOCH": False},
        },
        "TRAIN": {},
        "OUTPUT": ".",
        "TAG": "",
        "LOCAL_RANK": 0,
    }


def group(fused):
    return {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 1e-2, "fused": fused,
            "use_first_moment": True, "factor_second_moment": False, "params": [0, 1]}


def int8(codes):
    return torch.from_numpy(np.ascontiguousarray(codes).view(np.int8).copy())


def main():
    rng = np.random.default_rng(20240531)
    qm, qv = O.qmap_m(), O.qmap_v()
    tqm, tqv = torch.from_numpy(qm.copy()), torch.from_numpy(qv.copy())
    r, c = SHAPES[0]
    n = r * c
    m = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    v = ((rng.standard_normal(n) * 1e-3) ** 2).astype(np.float32)
    m_small = (rng.standard_normal(SHAPES[1][0]) * 1e-3).astype(np.float32)
    v_small = ((rng.standard_normal(SHAPES[1][0]) * 1e-3) ** 2).astype(np.float32)

    def small_state():
        return {"step": torch.tensor(STEP), "exp_avg": torch.from_numpy(m_small.copy()),
                "exp_avg_qstate": {"enable": False, "overhead": {}, "qmap": tqm.clone()},
                "exp_avg_sq": torch.from_numpy(v_small.copy()),
                "exp_avg_sq_qstate": {"enable": False, "overhead": {}, "qmap": tqv.clone()}}

    # fused layout: the padded non-fused codes without their padding and trailing byte
    mc, m_max1 = O.quant_group(m, qm)
    vc, v_max1 = O.quant_group(v, qv)
    fused = {
        "state": {
            0: {"step": torch.tensor(STEP), "exp_avg": int8(mc[: n // 2]),
                "exp_avg_qstate": {"enable": True, "overhead": {"max1": torch.from_numpy(m_max1.copy())},
                                   "qmap": tqm.clone()},
                "exp_avg_sq": int8(vc[: n // 2]),
                "exp_avg_sq_qstate": {"enable": True, "overhead": {"max1": torch.from_numpy(v_max1.copy())},
                                      "qmap": tqv.clone()}},
            1: small_state(),
        },
        "param_groups": [group(True)],
        "qconfig": qconfig("group"),
    }

    rowmax, colmax = O.rank1_stats(v.reshape(r, c))
    vc1 = O.quant_rank1(v.reshape(r, c), rowmax, colmax, qv).copy()
    mc_nf = mc.copy()
    mc_nf[-1] = 0x5A  # the byte past the codes is never initialised by the reference's packing operator
    vc1[-1] = 0x5A
    groups = (n + 127) // 128
    nonfused = {
        "state": {
            0: {"step": torch.tensor(STEP), "exp_avg": int8(mc_nf),
                "exp_avg_qstate": {"enable": True,
                                   "overhead": {"dtype": torch.float32, "stride": (c, 1),
                                                "max1": torch.from_numpy(m_max1.copy()).reshape(groups, 1),
                                                "scaled_shape": torch.Size((groups, 128))},
                                   "qmap": tqm.clone()},
                "exp_avg_sq": int8(vc1),
                "exp_avg_sq_qstate": {"enable": True,
                                      "overhead": {"dtype": torch.float32, "stride": (c, 1), "dim": 2,
                                                   "max_dims": [torch.from_numpy(rowmax.copy()).reshape(r, 1),
                                                                torch.from_numpy(colmax.copy()).reshape(1, c)],
                                                   "max1": None, "scaled_shape": torch.Size((r, c))},
                                      "qmap": tqv.clone()}},
            1: small_state(),
        },
        "param_groups": [group(False)],
        "qconfig": qconfig("rank1"),
    }
    out = os.path.join(HERE, "reference_shaped_checkpoints.pt")
    torch.save({"fused": fused, "nonfused_default": nonfused}, out)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
