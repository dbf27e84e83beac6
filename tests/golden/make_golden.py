#!/usr/bin/env python3
"""Writes the fixtures in this directory.

qmaps.json         bit patterns of the two standard 4-bit maps and their fp32 midpoints.  Source:
                   the construction recipe of the reference (lpmm/functional.py:272-315, :644-656)
                   executed op for op with PyTorch CPU ops in this script (torch.linspace in
                   float32, tensor * python scalar, .tolist(), torch.Tensor(sorted list)); nothing
                   is imported from the reference.
fused_step_small.npz  a seeded 3-step run of the fused 4-bit AdamW step on 1000 elements, produced
                   by the CPU oracle after it passed tests/test_oracle_*.py; lets the GPU tests
                   check the kernels without the oracle's shared library.
nonfused_steps_small.npz  seeded 3-step runs of the non-fused step on a 17 x 256 tensor, by the same
                   oracle: second moment block-wise ("group"), rank-1 ("rank1", the reference's
                   default configuration) and factored ("factored"); packed codes and scales /
                   statistics after every step, parameters after the last.
"""
import json
import os
import struct
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))


def hexes(values):
    return ["%08x" % struct.unpack("<I", struct.pack("<f", float(v)))[0] for v in values]


def dynamic_map_signed_4bit():
    data = []
    for i in range(3):  # max_exponent_bits = 3, non_sign_bits = 3, no additional items
        boundaries = torch.linspace(0.1, 1, 2 ** i + 1)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        data += ((10 ** (-2 + i)) * means).tolist()
        data += (-(10 ** (-2 + i)) * means).tolist()
    data.append(0)
    data.append(1.0)
    data.sort()
    return torch.Tensor(data)


def main():
    qm = dynamic_map_signed_4bit()
    qv = torch.linspace(0, 1, 17)[1:]
    mid = lambda q: (q[:-1] + q[1:]) * 0.5
    json.dump({"qmap_m_hex": hexes(qm.tolist()), "mid_m_hex": hexes(mid(qm).tolist()),
               "qmap_v_hex": hexes(qv.tolist()), "mid_v_hex": hexes(mid(qv).tolist())},
              open(os.path.join(HERE, "qmaps.json"), "w"), indent=1)

    from oracle import oracle as O

    rng = np.random.default_rng(2024)
    n = 1000
    p = (rng.standard_normal(n) * 0.02).astype(np.float32)
    grads = (rng.standard_normal((3, n)) * 1e-3).astype(np.float32)
    grads[1, 128:256] = 0.0
    mc, vc = np.zeros(n // 2, np.uint8), np.zeros(n // 2, np.uint8)
    ms, vs = np.zeros(8, np.float32), np.zeros(8, np.float32)
    out = {"p0": p.copy(), "grads": grads}
    for s in range(3):
        O.adamw4bit_step(p, grads[s], mc, vc, ms, vs, O.qmap_m(), O.qmap_v(), 0.9, 0.999, 1e-3, 0.01, 1e-8,
                         float(s + 1))
        out[f"p{s + 1}"], out[f"mc{s + 1}"], out[f"vc{s + 1}"] = p.copy(), mc.copy(), vc.copy()
        out[f"ms{s + 1}"], out[f"vs{s + 1}"] = ms.copy(), vs.copy()
    np.savez_compressed(os.path.join(HERE, "fused_step_small.npz"), **out)

    rng = np.random.default_rng(4242)
    shape = (17, 256)  # 4352 elements: just above the quantisation threshold of 4096
    p0 = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    grads = (rng.standard_normal((3,) + shape) * 1e-3).astype(np.float32)
    grads *= np.exp(rng.standard_normal((3, shape[0], 1)) * 0.7).astype(np.float32)  # rows of different size
    grads[2, 5] = 0.0
    out = {"p0": p0, "grads": grads}
    for kind in ("group", "rank1", "factored"):
        p = p0.copy()
        st = O.NonFusedState(shape, v_scale_type="rank1" if kind == "rank1" else "group", factored=kind == "factored")
        for s in range(3):
            O.nonfused_step(p, grads[s], st, O.qmap_m(), O.qmap_v(), 1e-3, 0.9, 0.999, 1e-8, 0.01)
            k = f"{kind}{s + 1}"
            out[f"mc_{k}"], out[f"ms_{k}"] = st.m[0].copy(), st.m[1].copy()
            if kind == "factored":
                out[f"row_{k}"], out[f"col_{k}"] = st.row.copy(), st.col.copy()
            else:
                out[f"vc_{k}"] = st.v[0].copy()
                for j, a in enumerate(st.v[1:]):
                    out[f"vs{j}_{k}"] = a.copy()
        out[f"p_{kind}3"] = p.copy()
    np.savez_compressed(os.path.join(HERE, "nonfused_steps_small.npz"), **out)


if __name__ == "__main__":
    main()
