"""End-to-end GPU tests of lpmm.optim.AdamW against the CPU oracle: fused, non-fused
(group and rank-1 second moment) and factored paths, state layout, checkpointing,
the 100-step trajectory criterion and the golden fixture."""
import os

import numpy as np
import pytest
import torch

from util import assert_codes, assert_params, assert_rel, nibbles, to_dev, to_np

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
H = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
HO = (0.9, 0.999, 1e-3, 0.01, 1e-8)  # oracle order: beta1, beta2, lr, wd, eps


def _params(shapes, rng):
    host = [(rng.standard_normal(s) * 0.02).astype(np.float32) for s in shapes]
    return host, [torch.nn.Parameter(to_dev(h)) for h in host]


def test_fused_optimizer_matches_oracle_and_layout(oracle, qmaps):
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(0)
    shapes = [(64, 130), (1600,), (6400,), (40, 40), (130, 128)]  # 8320 q, 1600 fp32, 6400 q (50 groups), 1600 fp32, 16640 q
    host, params = _params(shapes, rng)
    opt = lpmm.optim.AdamW(params, fused=True, **H)
    ref = []
    for h in host:
        n = h.size
        if n > 4096:
            ref.append(dict(mc=np.zeros(n // 2, np.uint8), vc=np.zeros(n // 2, np.uint8),
                            ms=np.zeros((n + 127) // 128, np.float32), vs=np.zeros((n + 127) // 128, np.float32)))
        else:
            ref.append(dict(m=np.zeros(n, np.float32), v=np.zeros(n, np.float32)))
    for step in range(1, 6):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        for p, h, g, r in zip(params, host, grads, ref):
            before = h.copy()
            if "mc" in r:
                oracle.adamw4bit_step(h.reshape(-1), g.reshape(-1), r["mc"], r["vc"], r["ms"], r["vs"], qm, qv, *HO, float(step))
            else:
                oracle.adamw_fp32_step(h.reshape(-1), g.reshape(-1), r["m"], r["v"], *HO, float(step))
            # one step from identical inputs; the next one starts from the oracle's parameters
            assert_params(to_np(p), h, before, f"p step {step}")
            p.data.copy_(to_dev(h))
    torch.cuda.synchronize()
    for p, h, r in zip(params, host, ref):
        st = opt.state[p]
        assert float(st["step"]) == 5.0 and st["step"].device.type == "cpu"
        if "mc" in r:
            n = h.size
            assert st["exp_avg"].dtype == torch.int8 and st["exp_avg"].shape == ((n + 1) // 2,)
            assert st["exp_avg_qstate"]["overhead"]["max1"].shape == ((n + 127) // 128,)
            assert_codes(to_np(st["exp_avg"]), r["mc"], n, "m codes")
            assert_codes(to_np(st["exp_avg_sq"]), r["vc"], n, "v codes")
            assert_rel(to_np(st["exp_avg_qstate"]["overhead"]["max1"]), r["ms"], "m scales")
            assert_rel(to_np(st["exp_avg_sq_qstate"]["overhead"]["max1"]), r["vs"], "v scales")
        else:
            assert st["exp_avg"].dtype == torch.float32 and st["exp_avg"].shape == p.shape
            np.testing.assert_array_equal(to_np(st["exp_avg"]).reshape(-1), r["m"])
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).reshape(-1), r["v"])
        assert_rel(to_np(p), h, "p", scale=h)


def test_fused_optimizer_error_behaviour(oracle):
    import lpmm

    # odd numel > 4096: the reference allocates (n+1)//2 bytes and then fails its own size check
    p = torch.nn.Parameter(torch.zeros(4099, device="cuda"))
    p.grad = torch.zeros_like(p)
    with pytest.raises(RuntimeError, match="number of elements in exp_avg and p"):
        lpmm.optim.AdamW([p], fused=True).step()
    # m and v must be quantised together on the fused path
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "2nd_moment_only_group_128.yml")
    q = torch.nn.Parameter(torch.zeros(128, 64, device="cuda"))
    q.grad = torch.zeros_like(q)
    with pytest.raises(ValueError, match="both quantized or unquantized"):
        lpmm.optim.AdamW([q], fused=True, qconfig=cfg).step()
    # non-contiguous gradient
    r = torch.nn.Parameter(torch.zeros(128, 64, device="cuda"))
    r.grad = torch.zeros(64, 128, device="cuda").t()
    with pytest.raises(RuntimeError, match="contiguous"):
        lpmm.optim.AdamW([r], fused=True).step()


@pytest.mark.parametrize("v_scale", ["rank1", "group"])
def test_nonfused_optimizer_matches_oracle(oracle, qmaps, v_scale):
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(1)
    shapes = [(96, 160), (11008,), (2000,)]
    host, params = _params(shapes, rng)
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs",
                       "default.yml" if v_scale == "rank1" else "2nd_moment_group_128.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **H)
    states = [oracle.NonFusedState(s, v_scale_type=v_scale) for s in shapes[:2]]
    m_small, v_small = np.zeros(2000, np.float32), np.zeros(2000, np.float32)
    for step in range(1, 5):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        for h, g, st in zip(host[:2], grads[:2], states):
            oracle.nonfused_step(h, g, st, qm, qv, H["lr"], 0.9, 0.999, H["eps"], H["weight_decay"])
        oracle.nonfused_update(host[2], grads[2], m_small, v_small, 0.9, 0.999, H["lr"], H["weight_decay"], H["eps"], float(step))
    torch.cuda.synchronize()
    # 2-D tensor
    s0 = opt.state[params[0]]
    n0 = host[0].size
    assert s0["exp_avg"].dtype == torch.int8 and s0["exp_avg"].numel() == (n0 + 2047) // 2048 * 1024 + 1
    np.testing.assert_array_equal(to_np(s0["exp_avg"]).view(np.uint8), states[0].m[0])
    np.testing.assert_array_equal(to_np(s0["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), states[0].m[1])
    oh = s0["exp_avg_sq_qstate"]["overhead"]
    np.testing.assert_array_equal(to_np(s0["exp_avg_sq"]).view(np.uint8), states[0].v[0])
    if v_scale == "rank1":
        assert oh["dim"] == 2 and oh["max1"] is None and oh["scaled_shape"] == torch.Size(shapes[0])
        np.testing.assert_array_equal(to_np(oh["max_dims"][0]).reshape(-1), states[0].v[1])
        np.testing.assert_array_equal(to_np(oh["max_dims"][1]).reshape(-1), states[0].v[2])
    else:
        assert oh["max1"].shape == ((n0 + 127) // 128, 1) and oh["scaled_shape"] == torch.Size(((n0 + 127) // 128, 128))
        np.testing.assert_array_equal(to_np(oh["max1"]).reshape(-1), states[0].v[1])
    assert_rel(to_np(params[0]), host[0], 'p 2-D', scale=host[0])
    # 1-D tensor: rank1 falls back to group-128
    s1 = opt.state[params[1]]
    if v_scale == "rank1":
        assert s1["exp_avg_sq_qstate"]["overhead"]["dim"] == 1  # as the reference's 'rank1' branch records it
    np.testing.assert_array_equal(to_np(s1["exp_avg_sq"]).view(np.uint8), states[1].v[0])
    np.testing.assert_array_equal(to_np(s1["exp_avg_sq_qstate"]["overhead"]["max1"]).reshape(-1), states[1].v[1])
    assert_rel(to_np(params[1]), host[1], 'p 1-D', scale=host[1])
    # small tensor keeps fp32 states
    s2 = opt.state[params[2]]
    assert s2["exp_avg"].dtype == torch.float32
    np.testing.assert_array_equal(to_np(s2["exp_avg"]), m_small)
    np.testing.assert_array_equal(to_np(s2["exp_avg_sq"]), v_small)
    assert_rel(to_np(params[2]), host[2], 'p small', scale=host[2])


def test_nonfused_optimizer_routes_every_column_count(oracle, qmaps):
    """fused=False under the default configuration with the column counts that take different kernels:
    whole 128-column blocks, 64 modulo 128 with an even row count (taken as double rows), the same
    with an odd row count and 32 modulo 128 (ragged rows) -- all in one optimizer, against the oracle."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(11)
    shapes = [(48, 256), (64, 192), (40, 320), (33, 192), (96, 160), (130, 1600)]
    host, params = _params(shapes, rng)
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "default.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **H)
    states = [oracle.NonFusedState(s, v_scale_type="rank1") for s in shapes]
    for step in range(1, 5):
        grads = [(rng.standard_normal(s) * 1e-3 * np.exp(rng.standard_normal((s[0], 1)))).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        for h, g, st in zip(host, grads, states):
            oracle.nonfused_step(h, g, st, qm, qv, H["lr"], 0.9, 0.999, H["eps"], H["weight_decay"])
    torch.cuda.synchronize()
    for i, shape in enumerate(shapes):
        s = opt.state[params[i]]
        np.testing.assert_array_equal(to_np(s["exp_avg"]).view(np.uint8), states[i].m[0], err_msg=str(shape))
        np.testing.assert_array_equal(to_np(s["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), states[i].m[1])
        oh = s["exp_avg_sq_qstate"]["overhead"]
        np.testing.assert_array_equal(to_np(s["exp_avg_sq"]).view(np.uint8), states[i].v[0], err_msg=str(shape))
        np.testing.assert_array_equal(to_np(oh["max_dims"][0]).reshape(-1), states[i].v[1], err_msg=str(shape))
        np.testing.assert_array_equal(to_np(oh["max_dims"][1]).reshape(-1), states[i].v[2], err_msg=str(shape))
        assert_rel(to_np(params[i]), host[i], f"p {shape}", scale=host[i])


def test_nonfused_rank1_on_tensors_of_more_than_two_dimensions(oracle, qmaps):
    """Default configuration (rank-1 second moment) on 3-D and 4-D parameters: statistics,
    quantiser and dequantiser run in HIP (N-D statistics kernels plus the 2-D kernels on the
    flattened view) and leave the oracle's codes and statistics."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(21)
    # the first five take the two passes on their shape[0] x rest view (rest a multiple of 128, or 64 modulo
    # 128 with an even shape[0]: double rows), the last two the staged path
    shapes = [(6, 40, 64), (64, 64, 3, 3), (16, 4, 8, 32), (12, 3, 128), (6, 2, 4, 4, 32), (32, 16, 3, 3), (4, 24, 130)]
    shapes += [(48, 16, 3, 3), (16, 8, 8, 8)] * 15  # 35 tensors on the two passes: more than one launch holds
    shapes += [(4, 300, 256)]  # trailing dimensions of 76800 values: folded by the general statistics kernels
    host, params = _params(shapes, rng)
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "default.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **H)
    states = [oracle.NonFusedState(s, v_scale_type="rank1") for s in shapes]
    for step in range(1, 4):
        # structure along every dimension, so that each statistic decides the scale somewhere
        grads = []
        for s in shapes:
            g = rng.standard_normal(s) * 1e-3
            for d_ in range(len(s)):
                keep = [1] * len(s)
                keep[d_] = s[d_]
                g = g * np.exp(0.7 * rng.standard_normal(keep))
            grads.append(g.astype(np.float32))
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        before = [h.copy() for h in host]
        for h, g, st in zip(host, grads, states):
            oracle.nonfused_step(h, g, st, qm, qv, H["lr"], 0.9, 0.999, H["eps"], H["weight_decay"])
        torch.cuda.synchronize()
        for i, (p, h, st, b) in enumerate(zip(params, host, states, before)):
            what = f"tensor {i} {shapes[i]} step {step}"
            s = opt.state[p]
            n = h.size
            oh = s["exp_avg_sq_qstate"]["overhead"]
            assert oh["dim"] == len(shapes[i]) and oh["scaled_shape"] == torch.Size(shapes[i]) and oh["max1"] is None
            for d, (got, want) in enumerate(zip(oh["max_dims"], st.v[1])):
                keep = [1] * len(shapes[i])
                keep[d] = shapes[i][d]
                assert tuple(got.shape) == tuple(keep)
                np.testing.assert_array_equal(to_np(got).reshape(-1), want, err_msg=f"statistics {d} of {what}")
            np.testing.assert_array_equal(to_np(s["exp_avg"]).view(np.uint8)[: (n + 1) // 2], st.m[0][: (n + 1) // 2])
            np.testing.assert_array_equal(to_np(s["exp_avg_sq"]).view(np.uint8)[: (n + 1) // 2], st.v[0][: (n + 1) // 2])
            assert_rel(to_np(p.detach()), h, "p of " + what, scale=b)


STRIDED_MODES = {
    "rank1": dict(fused=False, qconfig="default.yml"),
    "group": dict(fused=False, qconfig="2nd_moment_group_128.yml"),
    "rank1_fp32_m": dict(fused=False, qconfig="2nd_moment_only_default.yml"),
    "group_fp32_m": dict(fused=False, qconfig="2nd_moment_only_group_128.yml"),
    "rank1_m_group_512": dict(fused=False, qconfig="1st_moment_group_512.yml"),
    "rank1_6bit": dict(fused=False, qconfig="default_6b.yml"),
    "factored": dict(fused=False, factor_second_moment=True),
    "factored_on_fused": dict(fused=True, factor_second_moment=True),
}


@pytest.mark.parametrize("mode", sorted(STRIDED_MODES))
def test_strided_parameters_equal_their_contiguous_twins(mode):
    """Non-contiguous parameters and gradients on the non-fused paths (the reference's PyTorch
    ops take any strides, lpmm/optim/adamw.py:394-422, and its quantiser flattens in index
    order): the same values in a contiguous tensor must give the same bytes, the strided
    parameter is updated in its own storage, and the states record the strides the reference
    records (those of zeros_like(p, preserve_format))."""
    import lpmm

    kw = dict(STRIDED_MODES[mode])
    if "qconfig" in kw:
        kw["qconfig"] = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", kw["qconfig"])
    rng = np.random.default_rng(8)
    dev = "cuda"
    # a transposed matrix (dense, permuted strides), every other column of a wider matrix (gaps),
    # a permuted 3-D tensor, a strided small vector with fp32 states, a transposed ragged matrix, a
    # transposed matrix whose rows are a multiple of 8 but not of 128 values long
    bases = [to_dev((rng.standard_normal((256, 96)) * 0.02).astype(np.float32)),
             to_dev((rng.standard_normal((64, 512)) * 0.02).astype(np.float32)),
             to_dev((rng.standard_normal((40, 6, 64)) * 0.02).astype(np.float32)),
             to_dev((rng.standard_normal((4000,)) * 0.02).astype(np.float32)),
             to_dev((rng.standard_normal((130, 70)) * 0.02).astype(np.float32)),
             to_dev((rng.standard_normal((136, 64)) * 0.02).astype(np.float32))]
    views = [lambda t: t.t(), lambda t: t[:, ::2], lambda t: t.permute(1, 0, 2), lambda t: t[::2], lambda t: t.t(),
             lambda t: t.t()]
    if mode == "factored":
        bases, views = bases[:2] + bases[3:], views[:2] + views[3:]
    elif mode == "factored_on_fused":
        # tensors that are not factored go to the fused operator there, which demands contiguous
        # operands in the reference as well (lpmm/cpp_extension/common.h:4)
        bases, views = bases[:2] + bases[4:], views[:2] + views[4:]
    strided = [torch.nn.Parameter(v(b)) for v, b in zip(views, bases)]
    assert not any(p.is_contiguous() for p in strided)
    twins = [torch.nn.Parameter(p.detach().contiguous().clone()) for p in strided]
    opt_s = lpmm.optim.AdamW(strided, **H, **kw)
    opt_t = lpmm.optim.AdamW(twins, **H, **kw)
    for step in range(3):
        for i, (p, t) in enumerate(zip(strided, twins)):
            g = to_dev((rng.standard_normal(tuple(p.shape)) * 1e-3).astype(np.float32))
            t.grad = g
            if i % 2 == 0:  # a gradient with the parameter's strides, else a contiguous one
                gs = torch.empty_strided(p.shape, p.stride(), device=dev)
                gs.copy_(g)
                p.grad = gs
            else:
                p.grad = g.clone()
        opt_s.step()
        opt_t.step()
    torch.cuda.synchronize()
    for i, (p, t, v, b) in enumerate(zip(strided, twins, views, bases)):
        assert not p.is_contiguous() and p.data_ptr() == b.data_ptr()
        assert torch.equal(p.detach(), t.detach()), f"parameter {i} differs from its contiguous twin"
        assert torch.equal(v(b), t.detach()), f"parameter {i}: the strided storage was not updated"
        ss, st = opt_s.state[p], opt_t.state[t]
        assert ss.keys() == st.keys()
        for name in ("exp_avg", "exp_avg_sq", "exp_avg_sq_row", "exp_avg_sq_col"):
            if name in ss:
                assert ss[name].shape == st[name].shape
                n = ss[name].numel() - (1 if ss[name].dtype == torch.int8 else 0)  # the byte past the codes
                assert torch.equal(ss[name].reshape(-1)[:n], st[name].reshape(-1)[:n]), f"{name} of parameter {i}"
        for name in ("exp_avg", "exp_avg_sq"):
            oh_s, oh_t = ss[f"{name}_qstate"]["overhead"], st.get(f"{name}_qstate", {}).get("overhead", {})
            for key in ("max1", "max_dims"):
                if oh_s.get(key) is not None:
                    a = oh_s[key] if isinstance(oh_s[key], list) else [oh_s[key]]
                    c = oh_t[key] if isinstance(oh_t[key], list) else [oh_t[key]]
                    assert all(torch.equal(x, y) for x, y in zip(a, c)), f"{key} of {name} of parameter {i}"
            if "stride" in oh_s:
                want = torch.empty_like(p, device="meta", memory_format=torch.preserve_format).stride()
                assert tuple(oh_s["stride"]) == tuple(want)
    # dequantising through the public function restores the recorded strides
    import lpmm.functional as F

    s0 = opt_s.state[strided[0]]
    name = "exp_avg" if s0["exp_avg"].dtype == torch.int8 else "exp_avg_sq"  # a quantised state of this mode
    if s0[name].dtype == torch.int8:
        md = opt_s.get_qmetadata_by_state_name(name)
        m = F.vectorwise_dequant(s0[name], qmap=s0[f"{name}_qstate"]["qmap"], shape=strided[0].shape,
                                 **{**s0[f"{name}_qstate"]["overhead"], **md})
        assert m.stride() == strided[0].stride() and m.shape == strided[0].shape


@pytest.mark.parametrize("fused", [False, True])
def test_factored_optimizer_matches_oracle(oracle, qmaps, fused):
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(2)
    shapes = [(128, 344), (344, 128), (50, 60), (11008,)]  # quantised m x2, fp32 m (3000 <= 4096), 1-D: 4-bit m and v
    host, params = _params(shapes, rng)
    opt = lpmm.optim.AdamW(params, fused=fused, factor_second_moment=True, **H)
    states = [oracle.NonFusedState(s, factored=True) for s in shapes[:2]]
    row2, col2, m2 = np.zeros(50, np.float32), np.zeros(60, np.float32), np.zeros(3000, np.float32)
    st1d = oracle.NonFusedState(shapes[3], v_scale_type="group")
    fz = dict(mc=np.zeros(5504, np.uint8), vc=np.zeros(5504, np.uint8), ms=np.zeros(86, np.float32), vs=np.zeros(86, np.float32))
    for step in range(1, 4):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        for h, g, st in zip(host[:2], grads[:2], states):
            oracle.nonfused_step(h, g, st, qm, qv, H["lr"], 0.9, 0.999, H["eps"], H["weight_decay"])
        rm, cm = oracle.factored_stats(grads[2])
        mean_all = oracle.factored_ema(row2, col2, rm, cm, 0.999)
        oracle.factored_update(host[2], grads[2], m2, row2, col2, mean_all, 0.9, 0.999, H["lr"], H["weight_decay"], H["eps"], float(step))
        if fused:
            before = host[3].copy()
            oracle.adamw4bit_step(host[3], grads[3], fz["mc"], fz["vc"], fz["ms"], fz["vs"], qm, qv, *HO, float(step))
            assert_params(to_np(params[3]), host[3], before, f"p 1-D step {step}")
            params[3].data.copy_(to_dev(host[3]))
        else:
            oracle.nonfused_step(host[3], grads[3], st1d, qm, qv, H["lr"], 0.9, 0.999, H["eps"], H["weight_decay"])
    torch.cuda.synchronize()
    for p, h, st in zip(params[:2], host[:2], states):
        s = opt.state[p]
        assert "exp_avg_sq" not in s and s["exp_avg_sq_row"].shape == (h.shape[0],) and s["exp_avg_sq_col"].shape == (h.shape[1],)
        assert_rel(to_np(s["exp_avg_sq_row"]), st.row, "row", tol=1e-6)
        assert_rel(to_np(s["exp_avg_sq_col"]), st.col, "col", tol=1e-6)
        np.testing.assert_array_equal(to_np(s["exp_avg"]).view(np.uint8), st.m[0])  # m does not depend on v
        np.testing.assert_array_equal(to_np(s["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), st.m[1])
        assert_rel(to_np(p), h, "p", scale=h)
    s = opt.state[params[2]]
    assert s["exp_avg"].dtype == torch.float32
    np.testing.assert_array_equal(to_np(s["exp_avg"]).reshape(-1), m2)
    assert_rel(to_np(params[2]), host[2], "p small", scale=host[2])
    s = opt.state[params[3]]
    if fused:
        np.testing.assert_array_equal(to_np(s["exp_avg_sq"]).view(np.uint8), fz["vc"])
    else:
        np.testing.assert_array_equal(to_np(s["exp_avg_sq"]).view(np.uint8), st1d.v[0])
    assert_rel(to_np(params[3]), host[3], "p 1-D", scale=host[3])


def test_trajectory_100_steps(oracle, qmaps):
    """Dequantised m and v over 100 steps stay within 1e-4 relative of the oracle's (measured
    against the scale of each 128-group, since m has entries near zero)."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(3)
    shape = (256, 512)
    n = shape[0] * shape[1]
    host, params = _params([shape], rng)
    h = host[0].reshape(-1)
    opt = lpmm.optim.AdamW(params, fused=True, **H)
    mc, vc = np.zeros(n // 2, np.uint8), np.zeros(n // 2, np.uint8)
    ms, vs = np.zeros(n // 128, np.float32), np.zeros(n // 128, np.float32)
    total_flips = 0
    for step in range(1, 101):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        params[0].grad = to_dev(g.reshape(shape))
        opt.step()
        oracle.adamw4bit_step(h, g, mc, vc, ms, vs, qm, qv, *HO, float(step))
        if step % 20 == 0:
            st = opt.state[params[0]]
            gm = oracle.dequant_group(to_np(st["exp_avg"]).view(np.uint8), to_np(st["exp_avg_qstate"]["overhead"]["max1"]), qm, n)
            gv = oracle.dequant_group(to_np(st["exp_avg_sq"]).view(np.uint8), to_np(st["exp_avg_sq_qstate"]["overhead"]["max1"]), qv, n)
            assert_rel(gm, oracle.dequant_group(mc, ms, qm, n), f"m trajectory step {step}", tol=1e-4, scale=ms.repeat(128))
            assert_rel(gv, oracle.dequant_group(vc, vs, qv, n), f"v trajectory step {step}", tol=1e-4, scale=vs.repeat(128))
            assert_rel(to_np(params[0]).reshape(-1), h, f"p trajectory step {step}", tol=1e-6, scale=np.full(n, 0.02))
            total_flips += int(np.sum(nibbles(to_np(st["exp_avg"]), n) != nibbles(mc, n)))
    print("code differences after 100 unsynchronised steps:", total_flips)


def test_golden_fixture_on_gpu(qmaps):
    """The committed fixture (tests/golden/fused_step_small.npz), through the reference-named
    operator lpmm.cpp_extension.fused_adamw.adamw4bit_single_tensor."""
    from lpmm.cpp_extension import fused_adamw

    gold = np.load(os.path.join(HERE, "golden", "fused_step_small.npz"))
    n = gold["p0"].size
    p = to_dev(gold["p0"])
    mc = torch.zeros(n // 2, dtype=torch.int8, device="cuda")
    vc = torch.zeros_like(mc)
    ms, vs = torch.zeros(8, device="cuda"), torch.zeros(8, device="cuda")
    qm, qv = to_dev(qmaps[0]), to_dev(qmaps[1])
    for s in range(3):
        g = to_dev(gold["grads"][s])
        fused_adamw.adamw4bit_single_tensor(p, g, mc, vc, ms, vs, qm, qv, 0.9, 0.999, 1e-3, 0.01, 1e-8, float(s + 1))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(mc).view(np.uint8), gold[f"mc{s + 1}"])
        np.testing.assert_array_equal(to_np(vc).view(np.uint8), gold[f"vc{s + 1}"])
        np.testing.assert_array_equal(to_np(ms), gold[f"ms{s + 1}"])
        np.testing.assert_array_equal(to_np(vs), gold[f"vs{s + 1}"])
        assert_rel(to_np(p), gold[f"p{s + 1}"], "p", scale=gold["p0"])
    with pytest.raises(RuntimeError):  # wrong scale length (lpmm/cpp_extension/fused_adamw_kernel.cu:218-219)
        fused_adamw.adamw4bit_single_tensor(p, g, mc, vc, ms[:7], vs, qm, qv, 0.9, 0.999, 1e-3, 0.01, 1e-8, 4.0)
    with pytest.raises(RuntimeError):  # numel mismatch
        fused_adamw.adamw4bit_single_tensor(p, g[:-2], mc, vc, ms, vs, qm, qv, 0.9, 0.999, 1e-3, 0.01, 1e-8, 4.0)


@pytest.mark.parametrize("kind", ["group", "rank1", "factored"])
def test_golden_nonfused_fixture_on_gpu(kind):
    """The committed non-fused fixture (tests/golden/nonfused_steps_small.npz) through
    lpmm.optim.AdamW(fused=False): block-wise second moment (one-pass kernel), rank-1 second
    moment (two-pass kernels, the default configuration) and factored second moment."""
    import lpmm

    gold = np.load(os.path.join(HERE, "golden", "nonfused_steps_small.npz"))
    cfg_dir = os.path.join(os.path.dirname(lpmm.config.__file__), "configs")
    p = torch.nn.Parameter(to_dev(gold["p0"]))
    if kind == "factored":
        opt = lpmm.optim.AdamW([p], fused=False, factor_second_moment=True, **H)
    else:
        cfg = os.path.join(cfg_dir, "default.yml" if kind == "rank1" else "2nd_moment_group_128.yml")
        opt = lpmm.optim.AdamW([p], fused=False, qconfig=cfg, **H)
    for s in range(3):
        p.grad = to_dev(gold["grads"][s])
        opt.step()
        torch.cuda.synchronize()
        st = opt.state[p]
        k = f"{kind}{s + 1}"
        np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), gold[f"mc_{k}"], err_msg=f"m codes {k}")
        np.testing.assert_array_equal(to_np(st["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), gold[f"ms_{k}"])
        if kind == "factored":
            # sums of squares in double, folded in another order than the oracle's loop
            assert_rel(to_np(st["exp_avg_sq_row"]), gold[f"row_{k}"], f"row {k}", tol=2e-7)
            assert_rel(to_np(st["exp_avg_sq_col"]), gold[f"col_{k}"], f"col {k}", tol=2e-7)
            continue
        np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), gold[f"vc_{k}"], err_msg=f"v codes {k}")
        oh = st["exp_avg_sq_qstate"]["overhead"]
        if kind == "rank1":
            np.testing.assert_array_equal(to_np(oh["max_dims"][0]).reshape(-1), gold[f"vs0_{k}"])
            np.testing.assert_array_equal(to_np(oh["max_dims"][1]).reshape(-1), gold[f"vs1_{k}"])
        else:
            np.testing.assert_array_equal(to_np(oh["max1"]).reshape(-1), gold[f"vs0_{k}"])
    assert_rel(to_np(p.detach()), gold[f"p_{kind}3"], f"p {kind}", scale=gold["p0"])


def test_checkpoint_resume_on_gpu(oracle):
    """state_dict -> load_state_dict -> continue gives the same bytes as an uninterrupted run."""
    import lpmm

    rng = np.random.default_rng(4)
    shapes = [(64, 130), (1600,)]
    host, params_a = _params(shapes, rng)
    params_b = [torch.nn.Parameter(p.detach().clone()) for p in params_a]
    opt_a = lpmm.optim.AdamW(params_a, fused=True, **H)
    opt_b = lpmm.optim.AdamW(params_b, fused=True, **H)
    grads = [[(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes] for _ in range(4)]

    def run(opt, params, steps):
        for k in steps:
            for p, g in zip(params, grads[k]):
                p.grad = to_dev(g)
            opt.step()

    run(opt_a, params_a, range(4))
    run(opt_b, params_b, range(2))
    sd = opt_b.state_dict()
    params_c = [torch.nn.Parameter(p.detach().clone()) for p in params_b]
    opt_c = lpmm.optim.AdamW(params_c, fused=True, **H)
    opt_c.load_state_dict(sd)
    run(opt_c, params_c, range(2, 4))
    torch.cuda.synchronize()
    for pa, pc in zip(params_a, params_c):
        assert torch.equal(pa, pc)
        sa, sc = opt_a.state[pa], opt_c.state[pc]
        assert torch.equal(sa["exp_avg"], sc["exp_avg"]) and torch.equal(sa["exp_avg_sq"], sc["exp_avg_sq"])
        assert sc["exp_avg"].dtype == sa["exp_avg"].dtype and float(sc["step"]) == 4.0


@pytest.mark.parametrize("nesterov", [False, True])
def test_sgd_4bit_momentum(oracle, qmaps, nesterov):
    """lpmm.optim.SGD: momentum buffer quantised with the first-moment config; the update is a
    chain of PyTorch device ops as in the reference, restated here in numpy float32."""
    import lpmm

    qm = qmaps[0]
    rng = np.random.default_rng(8)
    shapes = [(96, 160), (1000,)]
    host, params = _params(shapes, rng)
    lr, mom, wd, damp = 0.05, 0.9, 1e-4, 0.1
    opt = lpmm.optim.SGD(params, lr=lr, momentum=mom, dampening=damp, weight_decay=wd, nesterov=nesterov)
    bufs = [None, None]
    f = np.float32
    for step in range(4):
        grads = [(rng.standard_normal(s) * 1e-2).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for i, (h, g) in enumerate(zip(host, grads)):
            d_p = g + f(wd) * h
            if bufs[i] is None:
                buf = d_p.copy()
            else:
                prev = oracle.dequant_group(bufs[i][0], bufs[i][1], qm, h.size).reshape(h.shape) if i == 0 else bufs[i]
                buf = (prev * f(mom) + f(1 - damp) * d_p).astype(np.float32)
            upd = (d_p + f(mom) * buf).astype(np.float32) if nesterov else buf
            yard = np.maximum(np.abs(h), f(lr) * np.abs(upd))  # operands of the subtraction below
            h -= f(lr) * upd
            st = opt.state[params[i]]
            if i == 0:
                bufs[i] = oracle.quant_group(buf.reshape(-1), qm)
                got_buf = oracle.dequant_group(to_np(st["momentum_buffer"]).view(np.uint8),
                                               to_np(st["momentum_buffer_qstate"]["overhead"]["max1"]).reshape(-1), qm, h.size)
                want_buf = oracle.dequant_group(bufs[i][0], bufs[i][1], qm, h.size)
                # PyTorch's device kernels may fuse multiply-adds: compare the dequantised buffers on the
                # scale of their groups, then continue from the optimizer's own state
                assert_rel(got_buf, want_buf, "momentum buffer", tol=1e-5, scale=bufs[i][1].repeat(128)[: h.size])
                assert np.mean(nibbles(to_np(st["momentum_buffer"]), h.size) != nibbles(bufs[i][0], h.size)) < 1e-3
                assert st["momentum_buffer"].dtype == torch.int8
                bufs[i] = (to_np(st["momentum_buffer"]).view(np.uint8).copy(),
                           to_np(st["momentum_buffer_qstate"]["overhead"]["max1"]).reshape(-1).copy())
            else:
                assert st["momentum_buffer"].dtype == torch.float32
                assert_rel(to_np(st["momentum_buffer"]), buf, "fp32 momentum buffer", tol=1e-6, scale=np.abs(buf).mean() + 0 * buf)
                bufs[i] = to_np(st["momentum_buffer"]).copy()
            assert_rel(to_np(params[i]), h, "p", tol=1e-6, scale=yard)
            h[...] = to_np(params[i])
    with pytest.raises(ValueError):
        lpmm.optim.SGD(params, lr=0.1, fused=True)


@pytest.mark.parametrize("mode", ["fused", "nonfused_group", "nonfused_rank1", "factored"])
def test_steps_are_reproducible_bit_for_bit(mode):
    """Two optimizers fed the same parameters and gradients end in identical parameters and
    states: the row/column maxima of the rank-1 path are merged with an order-free integer
    atomic max and the factored sums are folded in a fixed order, so nothing depends on the
    order in which workgroups happen to run."""
    import lpmm

    cfg_dir = os.path.join(os.path.dirname(lpmm.config.__file__), "configs")
    kw = dict(H)
    if mode == "fused":
        kw.update(fused=True)
    elif mode == "nonfused_group":
        kw.update(fused=False, qconfig=os.path.join(cfg_dir, "2nd_moment_group_128.yml"))
    elif mode == "nonfused_rank1":
        kw.update(fused=False, qconfig=os.path.join(cfg_dir, "default.yml"))
    else:
        kw.update(fused=True, factor_second_moment=True)
    shapes = [(1024, 2048), (300, 4224), (2048, 1152), (6400,), (1600,)]
    gen = torch.Generator(device="cuda").manual_seed(5)
    init = [torch.randn(s, device="cuda", generator=gen) * 0.02 for s in shapes]
    grads = [[torch.randn(s, device="cuda", generator=gen) * 1e-3 * (1 + 10 * (i == 1)) for s in shapes]
             for i in range(3)]

    def run():
        params = [torch.nn.Parameter(t.clone()) for t in init]
        opt = lpmm.optim.AdamW(params, **kw)
        for gs in grads:
            for p, g in zip(params, gs):
                p.grad = g.clone()
            opt.step()
        torch.cuda.synchronize()
        out = []
        for p in params:
            st = opt.state[p]
            out.append(p.detach().clone())
            for name in sorted(st):
                if name == "step":
                    continue
                v = st[name]
                found = [v] if torch.is_tensor(v) else []
                if isinstance(v, dict):  # a qstate: the scales live in its overhead
                    for o in v.get("overhead", {}).values():
                        found += [o] if torch.is_tensor(o) else [x for x in o if torch.is_tensor(x)] if isinstance(o, (list, tuple)) else []
                out.extend(x.clone() for x in found)
        return out

    a, b = run(), run()
    assert len(a) == len(b) and len(a) > len(shapes)
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and x.shape == y.shape
        assert torch.equal(x.view(torch.uint8) if x.dtype == torch.int8 else x, y.view(torch.uint8) if y.dtype == torch.int8 else y)


@pytest.mark.parametrize("fused", [True, False])
def test_param_groups_missing_grads_and_closure(oracle, qmaps, fused):
    """Two parameter groups with their own hyper-parameters, a parameter that gets its first
    gradient two steps late (its own step count, lpmm/optim/adamw.py:119, :498) and a closure:
    every tensor must follow the oracle run with its group's hyper-parameters and its own
    step number."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(21)
    shapes = [(96, 128), (70, 256), (5000,)]  # all quantised (numel > 4096)
    host, params = _params(shapes, rng)
    groups = [dict(params=[params[0], params[2]], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01),
              dict(params=[params[1]], lr=3e-4, betas=(0.8, 0.99), eps=1e-6, weight_decay=0.0)]
    hyper = [(0.9, 0.999, 1e-3, 0.01, 1e-8), (0.8, 0.99, 3e-4, 0.0, 1e-6), (0.9, 0.999, 1e-3, 0.01, 1e-8)]
    kw = dict(fused=True) if fused else dict(
        fused=False, qconfig=os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "2nd_moment_group_128.yml"))
    opt = lpmm.optim.AdamW(groups, **kw)
    steps_done = [0, 0, 0]
    if fused:
        ref = [dict(mc=np.zeros((h.size + 1) // 2, np.uint8), vc=np.zeros((h.size + 1) // 2, np.uint8),
                    ms=np.zeros((h.size + 127) // 128, np.float32), vs=np.zeros((h.size + 127) // 128, np.float32))
               for h in host]
    else:
        ref = [dict(m=None, v=None) for _ in host]
    calls = []
    for it in range(4):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for i, (p, g) in enumerate(zip(params, grads)):
            p.grad = None if (i == 2 and it < 2) else to_dev(g)

        def closure():
            calls.append(it)
            return torch.tensor(float(it))

        loss = opt.step(closure)
        assert float(loss) == float(it)
        for i, (h, g, r) in enumerate(zip(host, grads, ref)):
            if i == 2 and it < 2:
                continue
            steps_done[i] += 1
            b1, b2, lr, wd, eps = hyper[i]
            if fused:
                before = h.copy()
                oracle.adamw4bit_step(h.reshape(-1), g.reshape(-1), r["mc"], r["vc"], r["ms"], r["vs"], qm, qv,
                                      b1, b2, lr, wd, eps, float(steps_done[i]))
                assert_params(to_np(params[i]), h, before, f"p of tensor {i}, call {it}")
                params[i].data.copy_(to_dev(h))
            else:
                n = h.size
                m = np.zeros(n, np.float32) if r["m"] is None else oracle.dequant_group(r["m"][0], r["m"][1], qm, n)
                v = np.zeros(n, np.float32) if r["v"] is None else oracle.dequant_group(r["v"][0], r["v"][1], qv, n)
                oracle.nonfused_update(h.reshape(-1), g.reshape(-1), m, v, b1, b2, lr, wd, eps, float(steps_done[i]))
                r["m"], r["v"] = oracle.quant_group(m, qm), oracle.quant_group(v, qv)
    torch.cuda.synchronize()
    assert calls == [0, 1, 2, 3]
    for i, (p, h, r) in enumerate(zip(params, host, ref)):
        st = opt.state[p]
        assert float(st["step"]) == float(steps_done[i]) == (2.0 if i == 2 else 4.0)
        assert_rel(to_np(p), h, f"p of tensor {i}", scale=h)
        if fused:
            assert_codes(to_np(st["exp_avg"]), r["mc"], h.size, "m codes")
            assert_codes(to_np(st["exp_avg_sq"]), r["vc"], h.size, "v codes")
        else:
            np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), r["m"][0])
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), r["v"][0])


def test_half_parameters_on_the_fused_path(oracle):
    """float16 parameters: tensors at or under the threshold keep half states and go through the
    half instantiation of the fp32-state operator, as in the reference
    (lpmm/optim/adamw.py:543-561, lpmm/cpp_extension/fused_adamw_kernel.cu:188); a tensor whose
    states would be quantised is refused, as the reference's 4-bit operator fails on it
    (float32 scales read through the parameters' type, :229-230); the non-fused path is float32
    only here."""
    import lpmm
    from lpmm.cpp_extension import fused_adamw

    rng = np.random.default_rng(17)
    shapes = [(1600,), (64, 64), (3, 5, 7)]
    host = [(rng.standard_normal(s) * 0.02).astype(np.float16) for s in shapes]
    params = [torch.nn.Parameter(to_dev(h)) for h in host]
    opt = lpmm.optim.AdamW(params, fused=True, **H)
    ms = [np.zeros(h.size, np.float16) for h in host]
    vs = [np.zeros(h.size, np.float16) for h in host]
    for step in range(1, 5):
        grads = [(rng.standard_normal(s) * 1e-2).astype(np.float16) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for p, h, g, m, v in zip(params, host, grads, ms, vs):
            oracle.adamw_fp16_step(h.reshape(-1), g.reshape(-1), m, v, H["betas"][0], H["betas"][1], H["lr"],
                                   H["weight_decay"], H["eps"], float(step))
            st = opt.state[p]
            assert st["exp_avg"].dtype == torch.float16 and st["exp_avg"].shape == p.shape
            np.testing.assert_array_equal(to_np(st["exp_avg"]).reshape(-1), m)
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).reshape(-1), v)
            np.testing.assert_array_equal(to_np(p.detach()), h)
    # the reference-named operator accepts half as well
    p = to_dev(host[0].copy()); g = to_dev((rng.standard_normal(shapes[0]) * 1e-2).astype(np.float16))
    m = torch.zeros_like(p); v = torch.zeros_like(p)
    want_p, want_m, want_v = host[0].copy(), np.zeros(1600, np.float16), np.zeros(1600, np.float16)
    fused_adamw.adamw_single_tensor(p, g, m, v, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0)
    oracle.adamw_fp16_step(want_p, to_np(g), want_m, want_v, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(p), want_p)
    with pytest.raises(RuntimeError, match="expected scalar type"):
        fused_adamw.adamw_single_tensor(p, g.float(), m, v, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0)
    # quantised states with half parameters: refused, with the reason
    big = torch.nn.Parameter(torch.zeros(128, 64, dtype=torch.float16, device="cuda"))
    big.grad = torch.zeros_like(big)
    with pytest.raises(RuntimeError, match="float32 is required"):
        lpmm.optim.AdamW([big], fused=True).step()
    # ... and so is the factored second moment with half parameters
    with pytest.raises(RuntimeError, match="float32 is required"):
        lpmm.optim.AdamW([big], fused=False, factor_second_moment=True).step()
    bf = torch.nn.Parameter(torch.zeros(128, 64, dtype=torch.bfloat16, device="cuda"))
    bf.grad = torch.zeros_like(bf)
    with pytest.raises(RuntimeError, match="float32 is required"):
        lpmm.optim.AdamW([bf], fused=False).step()


@pytest.mark.parametrize("v_scale", ["rank1", "group"])
def test_half_parameters_on_the_nonfused_path(v_scale):
    """float16 parameters with fused=False: the reference's own chain of float16 PyTorch ops
    (lpmm/optim/adamw.py:394-434, lpmm/functional.py:184-203, :97-118), here on the device with the HIP
    pack / unpack operators, against the same chain run by PyTorch's CPU kernels with the C oracle's
    pack / unpack.  Both round to half after every op; a float-level last-bit difference between the two
    libraries' kernels can cross a half rounding boundary now and then, so values are compared to a few
    half ulps of the operands (measured: at most 2.5), codes to a small budget (measured: under 1e-4), and every step starts from the device's own state."""
    import lpmm
    from oracle.nonfused_torch import TorchNonFusedAdamW

    torch.manual_seed(5)
    shapes = [(96, 160), (11008,), (2000,)]  # quantised 2-D, quantised 1-D, fp16 states
    hyper = dict(lr=1e-2, betas=(0.9, 0.999), eps=1e-3, weight_decay=0.01)
    host = [(torch.randn(s) * 0.5).half() for s in shapes]
    params = [torch.nn.Parameter(h.cuda()) for h in host]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs",
                       "default.yml" if v_scale == "rank1" else "2nd_moment_group_128.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **hyper)
    ref = TorchNonFusedAdamW([h.clone() for h in host[:2]], v_scale_type=v_scale, **hyper)
    ulp = 2.0 ** -10
    for step in range(1, 4):
        grads = [(torch.randn(s) * 0.3).half() for s in shapes]
        for p, g in zip(params, grads):
            p.grad = g.cuda()
        before = [q.float().abs() for q in ref.params]
        opt.step()
        ref.step(grads[:2])
        torch.cuda.synchronize()
        for i in range(2):
            st, rs = opt.state[params[i]], ref.state[i]
            n = host[i].numel()
            assert params[i].dtype == torch.float16 and st["exp_avg"].dtype == torch.int8
            got_p, want_p = params[i].detach().cpu().float(), ref.params[i].float()
            # one half ulp of the larger operand: a step that cancels most of a parameter leaves a small result
            yard = torch.maximum(want_p.abs(), before[i]).clamp_min(2.0 ** -14)
            assert torch.all((got_p - want_p).abs() <= 4 * ulp * yard), f"p {i} step {step}"
            oh_m, oh_v = st["exp_avg_qstate"]["overhead"], st["exp_avg_sq_qstate"]["overhead"]
            assert oh_m["max1"].dtype == torch.float16 and oh_m["dtype"] == torch.float16
            gm1, wm1 = oh_m["max1"].cpu().float().reshape(-1), rs["m"][1].float().reshape(-1)
            assert torch.all((gm1 - wm1).abs() <= 2 * ulp * wm1.abs()), f"m scales {i} step {step}"
            dm = np.mean(nibbles(to_np(st["exp_avg"]), n) != nibbles(rs["m"][0].numpy(), n))
            dv = np.mean(nibbles(to_np(st["exp_avg_sq"]), n) != nibbles(rs["v"][0].numpy(), n))
            assert dm < 2e-3 and dv < 2e-3, (i, step, dm, dv)
            if v_scale == "rank1" and i == 0:
                assert oh_v["dim"] == 2 and oh_v["max_dims"][0].dtype == torch.float16
            # continue from the device's state
            ref.params[i].copy_(params[i].detach().cpu())
            rs["m"] = (st["exp_avg"].cpu().clone(), oh_m["max1"].cpu().clone())
            if v_scale == "rank1" and i == 0:
                rs["v"] = (st["exp_avg_sq"].cpu().clone(), [m.cpu().clone() for m in oh_v["max_dims"]])
            else:
                rs["v"] = (st["exp_avg_sq"].cpu().clone(), oh_v["max1"].cpu().clone())
        small = opt.state[params[2]]
        assert small["exp_avg"].dtype == torch.float16 and small["exp_avg_sq"].dtype == torch.float16
    assert all(torch.isfinite(p).all() for p in params)


@pytest.mark.parametrize("v_scale", ["rank1", "group"])
def test_half_parameters_take_the_hip_step_kernels(oracle, qmaps, v_scale):
    """float16 parameters with fused=False whose states have the default kinds (first moment block-wise
    over 128 values, second moment block-wise or rank-1 on a matrix with a multiple of 128 columns) go
    through the one- and two-pass HIP kernels: parameters, codes, half scales and half statistics bit
    for bit against the oracle's float16 restatement of the reference's chain
    (lpmm/optim/adamw.py:394-434), four steps, one optimizer holding matrices, a vector, a matrix that
    stays with the chain of PyTorch ops (160 columns under 'rank1') and a tensor with half states."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(31)
    shapes = [(96, 256), (40, 1024), (11008,), (64, 160), (2000,)]
    hyper = dict(lr=1e-2, betas=(0.9, 0.999), eps=1e-3, weight_decay=0.01)
    host = [(rng.standard_normal(s) * 0.5).astype(np.float16) for s in shapes]
    params = [torch.nn.Parameter(to_dev(h.copy())) for h in host]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs",
                       "default.yml" if v_scale == "rank1" else "2nd_moment_group_128.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **hyper)
    states = [oracle.NonFusedState(s, v_scale) for s in shapes[:4]]
    exact = [0, 1, 2] if v_scale == "rank1" else [0, 1, 2, 3]  # tensors on the kernels

    def same(got, want, what):
        got, want = np.ascontiguousarray(got).reshape(-1), np.ascontiguousarray(want).reshape(-1)
        assert got.dtype == want.dtype == np.float16, what
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), what

    for step in range(1, 5):
        grads = [(rng.standard_normal(s) * 0.3 * 10.0 ** (1 - step)).astype(np.float16) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for i in exact:
            oracle.nonfused_step_f16(host[i], grads[i], states[i], qm, qv, hyper["lr"], 0.9, 0.999, hyper["eps"], 0.01)
            st = opt.state[params[i]]
            what = f"step {step} tensor {i}"
            same(to_np(params[i].detach()), host[i], what + ": p")
            oh_m, oh_v = st["exp_avg_qstate"]["overhead"], st["exp_avg_sq_qstate"]["overhead"]
            assert oh_m["dtype"] is torch.float16 and oh_v["dtype"] is torch.float16
            same(to_np(oh_m["max1"]), states[i].m[1], what + ": m max1")
            np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), states[i].m[0], err_msg=what + ": m codes")
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), states[i].v[0], err_msg=what + ": v codes")
            if v_scale == "rank1" and len(shapes[i]) == 2:
                assert oh_v["max1"] is None and oh_v["dim"] == 2
                assert oh_v["max_dims"][0].shape == (shapes[i][0], 1) and oh_v["max_dims"][1].shape == (1, shapes[i][1])
                same(to_np(oh_v["max_dims"][0]), states[i].v[1], what + ": row statistics")
                same(to_np(oh_v["max_dims"][1]), states[i].v[2], what + ": column statistics")
            else:
                same(to_np(oh_v["max1"]), states[i].v[1], what + ": v max1")
    assert all(torch.isfinite(p).all() for p in params)
    # the states read back as the reference's metadata describes them: half tensors of the parameter's shape
    from lpmm.functional import vectorwise_dequant

    st = opt.state[params[0]]
    kw = dict(st["exp_avg_qstate"]["overhead"])
    kw.update(opt.get_qmetadata_by_state_name("exp_avg"))
    m = vectorwise_dequant(st["exp_avg"], qmap=st["exp_avg_qstate"]["qmap"], shape=params[0].shape, **kw)
    assert m.dtype is torch.float16 and m.shape == params[0].shape
    same(to_np(m), oracle.dequant_group_f16(states[0].m[0], states[0].m[1], qm, host[0].size), "dequantised m")


def test_half_and_float_parameters_in_one_group(oracle, qmaps):
    """A parameter group that holds float16 and float32 tensors (fused=False, default configuration): each
    goes to the kernels of its type, and both match their oracles bit for bit over three steps."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(33)
    shape = (64, 256)
    hyper = dict(lr=1e-2, betas=(0.9, 0.999), eps=1e-3, weight_decay=0.01)
    host_h = (rng.standard_normal(shape) * 0.5).astype(np.float16)
    host_f = (rng.standard_normal(shape) * 0.5).astype(np.float32)
    ph, pf = torch.nn.Parameter(to_dev(host_h.copy())), torch.nn.Parameter(to_dev(host_f.copy()))
    opt = lpmm.optim.AdamW([pf, ph], fused=False, **hyper,
                           qconfig=os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "default.yml"))
    st_h, st_f = oracle.NonFusedState(shape, "rank1"), oracle.NonFusedState(shape, "rank1")
    for step in range(1, 4):
        gh = (rng.standard_normal(shape) * 0.1).astype(np.float16)
        gf = (rng.standard_normal(shape) * 0.1).astype(np.float32)
        ph.grad, pf.grad = to_dev(gh), to_dev(gf)
        opt.step()
        torch.cuda.synchronize()
        oracle.nonfused_step_f16(host_h, gh, st_h, qm, qv, hyper["lr"], 0.9, 0.999, hyper["eps"], 0.01)
        oracle.nonfused_step(host_f, gf, st_f, qm, qv, hyper["lr"], 0.9, 0.999, hyper["eps"], 0.01)
        assert np.array_equal(to_np(ph.detach()).view(np.uint16), host_h.view(np.uint16)), step
        assert_params(to_np(pf.detach()), host_f, host_f, f"float parameter, step {step}")
        for p, st in ((ph, st_h), (pf, st_f)):
            s = opt.state[p]
            np.testing.assert_array_equal(to_np(s["exp_avg"]).view(np.uint8), st.m[0])
            np.testing.assert_array_equal(to_np(s["exp_avg_sq"]).view(np.uint8), st.v[0])
            dims = s["exp_avg_sq_qstate"]["overhead"]["max_dims"]
            assert dims[0].dtype is p.dtype and s["exp_avg_qstate"]["overhead"]["max1"].dtype is p.dtype
            np.testing.assert_array_equal(to_np(dims[0]).reshape(-1), st.v[1])
            np.testing.assert_array_equal(to_np(dims[1]).reshape(-1), st.v[2])
        pf.data.copy_(torch.from_numpy(host_f))  # the float update is near-exact: continue from the oracle's values


@pytest.mark.parametrize("v_scale", ["rank1", "group"])
def test_double_parameters_on_the_nonfused_path(v_scale):
    """float64 parameters with fused=False: the reference's chain of PyTorch ops in double
    (lpmm/optim/adamw.py:394-434; its pack kernel rounds every normalised value to float before the
    search, lpmm/cpp_extension/quantization_kernel.cu:450), here on the device with the HIP pack /
    unpack operators, against the same chain run by PyTorch's CPU kernels with the C oracle's pack /
    unpack.  Double arithmetic is correctly rounded on both sides; what can differ is an op that
    one library fuses and the other does not, so values are compared to 1e-13 relative and codes
    to a small budget, and every step starts from the device's own state."""
    import lpmm
    from oracle.nonfused_torch import TorchNonFusedAdamW

    torch.manual_seed(6)
    shapes = [(96, 160), (11008,), (2000,)]  # quantised 2-D, quantised 1-D, double states
    hyper = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    host = [(torch.randn(s) * 0.02).double() for s in shapes]
    params = [torch.nn.Parameter(h.cuda()) for h in host]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs",
                       "default.yml" if v_scale == "rank1" else "2nd_moment_group_128.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **hyper)
    ref = TorchNonFusedAdamW([h.clone() for h in host[:2]], v_scale_type=v_scale, **hyper)
    for step in range(1, 4):
        grads = [(torch.randn(s) * 1e-3).double() for s in shapes]
        for p, g in zip(params, grads):
            p.grad = g.cuda()
        opt.step()
        ref.step(grads[:2])
        torch.cuda.synchronize()
        for i in range(2):
            st, rs = opt.state[params[i]], ref.state[i]
            n = host[i].numel()
            assert params[i].dtype == torch.float64 and st["exp_avg"].dtype == torch.int8
            got_p, want_p = params[i].detach().cpu(), ref.params[i]
            assert torch.all((got_p - want_p).abs() <= 1e-13 * want_p.abs().clamp_min(1e-6)), f"p {i} step {step}"
            oh_m, oh_v = st["exp_avg_qstate"]["overhead"], st["exp_avg_sq_qstate"]["overhead"]
            assert oh_m["max1"].dtype == torch.float64 and oh_m["dtype"] == torch.float64
            gm1, wm1 = oh_m["max1"].cpu().reshape(-1), rs["m"][1].reshape(-1)
            assert torch.all((gm1 - wm1).abs() <= 1e-14 * wm1.abs()), f"m scales {i} step {step}"
            dm = np.mean(nibbles(to_np(st["exp_avg"]), n) != nibbles(rs["m"][0].numpy(), n))
            dv = np.mean(nibbles(to_np(st["exp_avg_sq"]), n) != nibbles(rs["v"][0].numpy(), n))
            assert dm < 1e-4 and dv < 1e-4, (i, step, dm, dv)
            if v_scale == "rank1" and i == 0:
                assert oh_v["dim"] == 2 and oh_v["max_dims"][0].dtype == torch.float64
            # continue from the device's state
            ref.params[i].copy_(params[i].detach().cpu())
            rs["m"] = (st["exp_avg"].cpu().clone(), oh_m["max1"].cpu().clone())
            if v_scale == "rank1" and i == 0:
                rs["v"] = (st["exp_avg_sq"].cpu().clone(), [m.cpu().clone() for m in oh_v["max_dims"]])
            else:
                rs["v"] = (st["exp_avg_sq"].cpu().clone(), oh_v["max1"].cpu().clone())
        small = opt.state[params[2]]
        assert small["exp_avg"].dtype == torch.float64 and small["exp_avg_sq"].dtype == torch.float64
    assert all(torch.isfinite(p).all() for p in params)
    with pytest.raises(RuntimeError, match="float32 is required"):
        bad = lpmm.optim.AdamW([torch.nn.Parameter(host[1].cuda())], fused=True, **hyper)
        bad.param_groups[0]["params"][0].grad = host[1].cuda()
        bad.step()


@pytest.mark.parametrize("config", ["default.yml", "1st_moment_group_1024.yml"])
def test_failed_launch_leaves_the_statistics_with_their_codes(config):
    """The two-pass kernels write the next row/column statistics (and, with wide first-moment groups, the
    next scales) into a second buffer that trades places with the state's.  A launch that returns an error
    must leave the state pointing at the statistics its codes are scaled by: the step after the failure
    continues exactly like a run that never failed."""
    import lpmm
    from lpmm import _native

    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", config)
    entry = ("lpmm_nonfused_adamw4bit_rank1_step_multi" if config == "default.yml"
             else "lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi")
    rng = np.random.default_rng(31)
    shapes = [(64, 256), (96, 128)]
    host, params = _params(shapes, rng)
    _, twins = _params(shapes, np.random.default_rng(31))
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **H)
    ref = lpmm.optim.AdamW(twins, fused=False, qconfig=cfg, **H)
    lib = _native.lib()

    def step_both(which):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for o, ps in which:
            for p, g in zip(ps, grads):
                p.grad = to_dev(g)
            o.step()
        return grads

    step_both([(opt, params), (ref, twins)])
    before = [(opt.state[p]["exp_avg_sq_qstate"]["overhead"]["max_dims"][0].data_ptr(),
               opt.state[p]["exp_avg_qstate"]["overhead"]["max1"].data_ptr(),
               to_np(opt.state[p]["exp_avg_sq_qstate"]["overhead"]["max_dims"][0]).copy()) for p in params]
    real = getattr(lib, entry)
    setattr(lib, entry, lambda *a: 5)  # any status but LPMM_OK
    try:
        for p in params:
            p.grad = torch.zeros_like(p)
        with pytest.raises(RuntimeError):
            opt.step()
    finally:
        setattr(lib, entry, real)
    torch.cuda.synchronize()
    for p, (rows_ptr, max1_ptr, rows) in zip(params, before):
        oh_v, oh_m = opt.state[p]["exp_avg_sq_qstate"]["overhead"], opt.state[p]["exp_avg_qstate"]["overhead"]
        assert oh_v["max_dims"][0].data_ptr() == rows_ptr and oh_m["max1"].data_ptr() == max1_ptr
        np.testing.assert_array_equal(to_np(oh_v["max_dims"][0]), rows)
    # the failed call counted a step for every tensor; give the twin the same count, then both continue alike
    for p, t in zip(params, twins):
        ref.state[t]["step"] += 1
        assert float(opt.state[p]["step"]) == float(ref.state[t]["step"])
    step_both([(opt, params), (ref, twins)])
    torch.cuda.synchronize()
    for p, t in zip(params, twins):
        assert torch.equal(p.detach(), t.detach())
        assert torch.equal(opt.state[p]["exp_avg_sq"], ref.state[t]["exp_avg_sq"])
        assert torch.equal(opt.state[p]["exp_avg"], ref.state[t]["exp_avg"])
        for a, b in zip(opt.state[p]["exp_avg_sq_qstate"]["overhead"]["max_dims"],
                        ref.state[t]["exp_avg_sq_qstate"]["overhead"]["max_dims"]):
            assert torch.equal(a, b)
