"""Checkpoint round trips on the GPU (lpmm/optim/optimizer.py:68-136 of the reference):

* state_dict -> torch.save -> torch.load(weights_only=True) -> load_state_dict -> continue must
  leave the same bytes as an uninterrupted run, for every way the optimizer keeps its states:
  fused, non-fused with the default configuration (rank-1 second moment: `max_dims` plus the
  second pair of statistics buffers the two-pass kernels swap in), non-fused with block-wise
  second moment, factored second moment; also when the file is loaded onto the host first.
* a state dict laid out by hand the way the reference lays it out (tests/golden/
  make_reference_checkpoint.py) loads and continues exactly as the CPU oracle continues it.
"""
import os

import numpy as np
import pytest
import torch

from util import assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

H = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_shaped_checkpoints.pt")


def _config(name):
    import lpmm

    return os.path.join(os.path.dirname(lpmm.config.__file__), "configs", name)


MODES = {
    "fused": dict(fused=True),
    "nonfused_rank1": dict(fused=False, qconfig="default.yml"),
    "nonfused_group": dict(fused=False, qconfig="2nd_moment_group_128.yml"),
    "nonfused_rank1_fp32_m": dict(fused=False, qconfig="2nd_moment_only_default.yml"),
    "nonfused_group_fp32_m": dict(fused=False, qconfig="2nd_moment_only_group_128.yml"),
    "nonfused_rank1_m_group_512": dict(fused=False, qconfig="1st_moment_group_512.yml"),
    "nonfused_rank1_6bit": dict(fused=False, qconfig="default_6b.yml"),
    # float16 parameters: the half step kernels (and, for the ragged and 3-D tensors, the chain of PyTorch ops)
    "nonfused_rank1_half": dict(fused=False, qconfig="default.yml", half=True),
    "nonfused_group_half": dict(fused=False, qconfig="2nd_moment_group_128.yml", half=True),
    "factored": dict(fused=False, factor_second_moment=True),
    "factored_fused": dict(fused=True, factor_second_moment=True),
}
# 2-D with a multiple of 128 columns (multi-tensor kernels), 2-D with ragged columns and a 3-D
# tensor (staged paths), a quantised vector, an fp32-state vector
SHAPES = [(96, 256), (70, 130), (3, 40, 64), (8192,), (1600,)]


def _make(mode, params):
    import lpmm

    kw = dict(MODES[mode])
    if "qconfig" in kw:
        kw["qconfig"] = _config(kw["qconfig"])
    hyper = dict(H)
    if kw.pop("half", False):
        hyper["eps"] = 1e-3  # float16 rounds 1e-8 to zero
    return lpmm.optim.AdamW(params, **hyper, **kw)


def _flat_state(opt, params):
    """Every tensor of the optimizer state, by a stable name."""
    out = {}

    def walk(prefix, value):
        if isinstance(value, torch.Tensor):
            out[prefix] = value
        elif isinstance(value, dict):
            for k, v in value.items():
                walk(f"{prefix}.{k}", v)
        elif isinstance(value, (list, tuple)):
            for i, v in enumerate(value):
                walk(f"{prefix}[{i}]", v)

    for i, p in enumerate(params):
        walk(f"p{i}", opt.state[p])
    return out


@pytest.mark.parametrize("map_location", [None, "cpu"])
@pytest.mark.parametrize("mode", sorted(MODES))
def test_resume_through_a_file_equals_uninterrupted_run(mode, map_location, tmp_path):
    if mode == "fused":
        shapes = [s for s in SHAPES if int(np.prod(s)) % 2 == 0]
    else:
        shapes = SHAPES
    rng = np.random.default_rng(12)
    dtype = np.float16 if MODES[mode].get("half") else np.float32
    start = [(rng.standard_normal(s) * 0.02).astype(dtype) for s in shapes]
    grads = [[(rng.standard_normal(s) * (3e-2 if dtype is np.float16 else 1e-3)).astype(dtype) for s in shapes]
             for _ in range(6)]

    def run(opt, params, steps):
        for k in steps:
            for p, g in zip(params, grads[k]):
                p.grad = to_dev(g)
            opt.step()

    params_a = [torch.nn.Parameter(to_dev(x)) for x in start]
    opt_a = _make(mode, params_a)
    run(opt_a, params_a, range(6))

    params_b = [torch.nn.Parameter(to_dev(x)) for x in start]
    opt_b = _make(mode, params_b)
    run(opt_b, params_b, range(3))
    path = str(tmp_path / "opt.pt")
    torch.save({"opt": opt_b.state_dict(), "params": [p.detach() for p in params_b]}, path)
    del opt_b

    # a file of tensors and builtin containers only: the weights-only loader reads it
    ckpt = torch.load(path, weights_only=True, map_location=map_location)
    assert type(ckpt["opt"]["qconfig"]) is dict
    params_c = [torch.nn.Parameter(p.to("cuda").clone()) for p in ckpt["params"]]
    opt_c = _make(mode, params_c)
    opt_c.load_state_dict(ckpt["opt"])
    # after the load, states with the same map share one tensor again (one launch group per map pair)
    maps = {opt_c.state[p][f"{name}_qstate"]["qmap"].data_ptr() for p in params_c for name in ("exp_avg", "exp_avg_sq")}
    assert len(maps) == 2
    assert all(opt_c.state[p][f"{name}_qstate"]["qmap"].is_cuda for p in params_c for name in ("exp_avg", "exp_avg_sq"))
    run(opt_c, params_c, range(3, 6))
    torch.cuda.synchronize()

    for i, (pa, pc) in enumerate(zip(params_a, params_c)):
        assert torch.equal(pa, pc), f"parameter {i} {tuple(pa.shape)} differs after the resumed run"
    sa, sc = _flat_state(opt_a, params_a), _flat_state(opt_c, params_c)
    assert sa.keys() == sc.keys()
    for name in sa:
        assert sa[name].dtype == sc[name].dtype and sa[name].shape == sc[name].shape, name
        if name.endswith(".step"):
            assert float(sa[name]) == float(sc[name]) == 6.0 and sc[name].device.type == "cpu"
        else:
            assert torch.equal(sa[name], sc[name].to(sa[name].device)), f"state {name} differs after the resumed run"


@pytest.mark.parametrize("map_location", [None, "cpu"])
def test_sgd_resume_through_a_file_equals_uninterrupted_run(map_location, tmp_path):
    """lpmm.optim.SGD with a 4-bit momentum buffer: tensors on the one-pass kernel (contiguous, quantised),
    a strided one on the chain of PyTorch ops, and one with an fp32 buffer."""
    import lpmm

    shapes = [(96, 256), (8192,), (70, 130), (1600,)]
    rng = np.random.default_rng(13)
    start = [(rng.standard_normal(s) * 0.02).astype(np.float32) for s in shapes]
    grads = [[(rng.standard_normal(s) * 1e-2).astype(np.float32) for s in shapes] for _ in range(6)]

    def make(params):
        return lpmm.optim.SGD(params, lr=0.05, momentum=0.9, dampening=0.1, weight_decay=1e-4, nesterov=True)

    def fresh(values):
        params = [torch.nn.Parameter(to_dev(x)) for x in values]
        # the third tensor lives transposed in its storage: not contiguous
        params[2] = torch.nn.Parameter(to_dev(np.ascontiguousarray(values[2].T)).t())
        assert not params[2].is_contiguous()
        return params

    def run(opt, params, steps):
        for k in steps:
            for i, (p, g) in enumerate(zip(params, grads[k])):
                p.grad = to_dev(np.ascontiguousarray(g.T)).t() if i == 2 else to_dev(g)
            opt.step()

    params_a = fresh(start)
    opt_a = make(params_a)
    run(opt_a, params_a, range(6))

    params_b = fresh(start)
    opt_b = make(params_b)
    run(opt_b, params_b, range(3))
    path = str(tmp_path / "sgd.pt")
    torch.save({"opt": opt_b.state_dict(), "params": [p.detach().contiguous() for p in params_b]}, path)
    del opt_b

    ckpt = torch.load(path, weights_only=True, map_location=map_location)
    params_c = fresh([to_np(p) for p in ckpt["params"]])
    opt_c = make(params_c)
    opt_c.load_state_dict(ckpt["opt"])
    run(opt_c, params_c, range(3, 6))
    torch.cuda.synchronize()

    for i, (pa, pc) in enumerate(zip(params_a, params_c)):
        assert torch.equal(pa, pc), f"parameter {i} {tuple(pa.shape)} differs after the resumed run"
    sa, sc = _flat_state(opt_a, params_a), _flat_state(opt_c, params_c)
    assert sa.keys() == sc.keys()
    for name in sa:
        assert sa[name].dtype == sc[name].dtype and sa[name].shape == sc[name].shape, name
        assert torch.equal(sa[name], sc[name].to(sa[name].device)), f"state {name} differs after the resumed run"
    assert opt_c.state[params_c[0]]["momentum_buffer"].dtype == torch.int8
    assert opt_c.state[params_c[3]]["momentum_buffer"].dtype == torch.float32


def test_reference_shaped_fused_checkpoint_continues_like_the_oracle(oracle, qmaps):
    import lpmm

    qm, qv = qmaps
    ckpt = torch.load(GOLDEN, weights_only=True)["fused"]
    rng = np.random.default_rng(3)
    shapes = [(40, 256), (1600,)]
    host_p = [(rng.standard_normal(s) * 0.02).astype(np.float32) for s in shapes]
    params = [torch.nn.Parameter(to_dev(x)) for x in host_p]
    opt = lpmm.optim.AdamW(params, fused=True)  # hyper-parameters come from the checkpoint's group
    opt.load_state_dict(ckpt)
    assert opt.qconfig.QUANT.SQM.SCALE_TYPE.DEFAULT == "group" and opt.param_groups[0]["fused"] is True
    s0 = ckpt["state"][0]
    mc, vc = s0["exp_avg"].numpy().view(np.uint8).copy(), s0["exp_avg_sq"].numpy().view(np.uint8).copy()
    ms = s0["exp_avg_qstate"]["overhead"]["max1"].numpy().copy()
    vs = s0["exp_avg_sq_qstate"]["overhead"]["max1"].numpy().copy()
    m1, v1 = ckpt["state"][1]["exp_avg"].numpy().copy(), ckpt["state"][1]["exp_avg_sq"].numpy().copy()
    ho = (0.9, 0.999, 1e-3, 1e-2, 1e-8)
    for step in (6.0, 7.0):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        before = [x.copy() for x in host_p]
        oracle.adamw4bit_step(host_p[0].reshape(-1), grads[0].reshape(-1), mc, vc, ms, vs, qm, qv, *ho, step)
        oracle.adamw_fp32_step(host_p[1], grads[1], m1, v1, *ho, step)
        torch.cuda.synchronize()
        st = opt.state[params[0]]
        assert float(st["step"]) == step
        np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), mc)
        np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), vc)
        np.testing.assert_array_equal(to_np(st["exp_avg_qstate"]["overhead"]["max1"]), ms)
        np.testing.assert_array_equal(to_np(st["exp_avg_sq_qstate"]["overhead"]["max1"]), vs)
        np.testing.assert_array_equal(to_np(opt.state[params[1]]["exp_avg"]), m1)
        np.testing.assert_array_equal(to_np(opt.state[params[1]]["exp_avg_sq"]), v1)
        for p, want, b in zip(params, host_p, before):
            assert_rel(to_np(p.detach()), want, "p", scale=b)


def test_reference_shaped_nonfused_checkpoint_continues_like_the_oracle(oracle, qmaps):
    import lpmm

    qm, qv = qmaps
    ckpt = torch.load(GOLDEN, weights_only=True)["nonfused_default"]
    rng = np.random.default_rng(4)
    shapes = [(40, 256), (1600,)]
    host_p = [(rng.standard_normal(s) * 0.02).astype(np.float32) for s in shapes]
    params = [torch.nn.Parameter(to_dev(x)) for x in host_p]
    opt = lpmm.optim.AdamW(params, fused=False)  # built-in defaults; the checkpoint brings the rank-1 setting
    opt.load_state_dict(ckpt)
    assert opt.qconfig.QUANT.SQM.SCALE_TYPE.DEFAULT == "rank1" and opt.param_groups[0]["fused"] is False
    s0 = ckpt["state"][0]
    ref = oracle.NonFusedState(shapes[0], v_scale_type="rank1")
    ref.step = 5
    oh_m, oh_v = s0["exp_avg_qstate"]["overhead"], s0["exp_avg_sq_qstate"]["overhead"]
    ref.m = (s0["exp_avg"].numpy().view(np.uint8).copy(), oh_m["max1"].numpy().reshape(-1).copy())
    ref.v = (s0["exp_avg_sq"].numpy().view(np.uint8).copy(), oh_v["max_dims"][0].numpy().reshape(-1).copy(),
             oh_v["max_dims"][1].numpy().reshape(-1).copy())
    m1, v1 = ckpt["state"][1]["exp_avg"].numpy().copy(), ckpt["state"][1]["exp_avg_sq"].numpy().copy()
    n = int(np.prod(shapes[0]))
    for step in (6.0, 7.0):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        before = [x.copy() for x in host_p]
        oracle.nonfused_step(host_p[0], grads[0], ref, qm, qv, 1e-3, 0.9, 0.999, 1e-8, 1e-2)
        oracle.nonfused_update(host_p[1], grads[1], m1, v1, 0.9, 0.999, 1e-3, 1e-2, 1e-8, step)
        torch.cuda.synchronize()
        st = opt.state[params[0]]
        assert float(st["step"]) == step
        oh = st["exp_avg_sq_qstate"]["overhead"]
        # all codes up to the byte past them, which the reference leaves uninitialised
        np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8)[: n // 2], ref.m[0][: n // 2])
        np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8)[: n // 2], ref.v[0][: n // 2])
        np.testing.assert_array_equal(to_np(st["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), ref.m[1])
        np.testing.assert_array_equal(to_np(oh["max_dims"][0]).reshape(-1), ref.v[1])
        np.testing.assert_array_equal(to_np(oh["max_dims"][1]).reshape(-1), ref.v[2])
        np.testing.assert_array_equal(to_np(opt.state[params[1]]["exp_avg"]), m1)
        np.testing.assert_array_equal(to_np(opt.state[params[1]]["exp_avg_sq"]), v1)
        for p, want, b in zip(params, host_p, before):
            assert_rel(to_np(p.detach()), want, "p", scale=b)
