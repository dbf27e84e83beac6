"""The two fused benchmark configurations as whole parameter sets.

* GPT-2-XL-shaped set (48 layers, d = 1600, 50257 x 1600 embedding; 580 tensors, 290 of them
  1600-long vectors with fp32 states): every distinct shape through
  lpmm.optim.AdamW(fused=True) against the CPU oracle, and the full set for 20 steps against
  single-tensor C-ABI calls on copies.
* LLaMA-7B-shaped set (291 tensors, 6.7e9 parameters): the full set through the optimizer's
  multi-tensor launches against single-tensor C-ABI calls on copies, bit for bit.

The path under test is _fused_adamw4bit of the reference (lpmm/optim/adamw.py:439-561): one
launch per tensor there, launches of up to 48 (4-bit states) / 64 (fp32 states) tensors here.
"""
import numpy as np
import pytest
import torch

from util import assert_codes, assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

HO = (0.9, 0.999, 1e-3, 0.01, 1e-8)  # beta1, beta2, lr, weight decay, eps


def gpt2xl_shapes():
    d = 1600
    shapes = [(50257, d), (1024, d)]
    for _ in range(48):
        shapes += [(d,), (d,), (d, 3 * d), (3 * d,), (d, d), (d,), (d,), (d,), (d, 4 * d), (4 * d,), (4 * d, d), (d,)]
    shapes += [(d,), (d,)]
    return shapes


def llama7b_shapes():
    shapes = [(32000, 4096)]
    for _ in range(32):
        shapes += [(4096, 4096)] * 4 + [(11008, 4096)] * 2 + [(4096, 11008)] + [(4096,)] * 2
    shapes += [(4096,), (32000, 4096)]
    return shapes


def test_shape_lists_are_the_configurations():
    g, l = gpt2xl_shapes(), llama7b_shapes()
    assert len(g) == 580 and sum(int(np.prod(s)) for s in g) == 1_557_611_200
    assert sum(1 for s in g if np.prod(s) <= 4096) == 290
    assert len(l) == 291 and sum(int(np.prod(s)) for s in l) == 6_738_415_616
    assert sum(1 for s in l if np.prod(s) > 4096) == 226


def _make_optimizer(params):
    import lpmm

    return lpmm.optim.AdamW(params, lr=HO[2], betas=(HO[0], HO[1]), eps=HO[4], weight_decay=HO[3], fused=True)


def test_gpt2xl_distinct_shapes_match_oracle(oracle, qmaps):
    """All nine distinct GPT-2-XL shapes in one optimizer (one ragged multi-tensor launch: the
    embedding and the 4800-long bias end in a 64-element group; plus one fp32-state launch),
    three steps, against the oracle tensor by tensor.  Seeds follow the configuration:
    parameter i from seed 10000+i, its gradient at step s from seed 20000+1000*s+i."""
    qm, qv = qmaps
    d = 1600
    shapes = [(50257, d), (1024, d), (d, 3 * d), (3 * d,), (d, d), (d, 4 * d), (4 * d,), (4 * d, d), (d,)]
    refs, params = [], []
    for i, shape in enumerate(shapes):
        n = int(np.prod(shape))
        p0 = (np.random.default_rng(10000 + i).standard_normal(n, dtype=np.float32) * 0.02).astype(np.float32)
        params.append(torch.nn.Parameter(to_dev(p0).view(shape)))
        if n > 4096:
            refs.append(dict(n=n, p=p0, mc=np.zeros(n // 2, np.uint8), vc=np.zeros(n // 2, np.uint8),
                             ms=np.zeros((n + 127) // 128, np.float32), vs=np.zeros((n + 127) // 128, np.float32)))
        else:
            refs.append(dict(n=n, p=p0, m=np.zeros(n, np.float32), v=np.zeros(n, np.float32)))
    opt = _make_optimizer(params)
    for step in (1, 2, 3):
        grads = []
        for i, (p, r) in enumerate(zip(params, refs)):
            g = (np.random.default_rng(20000 + 1000 * step + i).standard_normal(r["n"], dtype=np.float32)
                 * 1e-3).astype(np.float32)
            grads.append(g)
            p.grad = to_dev(g).view(p.shape)
        opt.step()
        torch.cuda.synchronize()
        for i, (p, r, g) in enumerate(zip(params, refs, grads)):
            what = f"tensor {i} {tuple(p.shape)} step {step}"
            before = r["p"].copy()
            st = opt.state[p]
            if "mc" in r:
                oracle.adamw4bit_step(r["p"], g, r["mc"], r["vc"], r["ms"], r["vs"], qm, qv, *HO, float(step))
                assert st["exp_avg"].dtype == torch.int8 and st["exp_avg"].numel() == r["n"] // 2
                flips = assert_codes(to_np(st["exp_avg"]), r["mc"], r["n"], "m codes of " + what)
                flips += assert_codes(to_np(st["exp_avg_sq"]), r["vc"], r["n"], "v codes of " + what)
                assert_rel(to_np(st["exp_avg_qstate"]["overhead"]["max1"]), r["ms"], "m scales of " + what)
                assert_rel(to_np(st["exp_avg_sq_qstate"]["overhead"]["max1"]), r["vs"], "v scales of " + what)
                assert flips == 0, f"{flips} codes of {what} differ from the oracle"
            else:
                oracle.adamw_fp32_step(r["p"], g, r["m"], r["v"], *HO, float(step))
                np.testing.assert_array_equal(to_np(st["exp_avg"]), r["m"], err_msg=what)
                np.testing.assert_array_equal(to_np(st["exp_avg_sq"]), r["v"], err_msg=what)
            assert_rel(to_np(p.detach()).reshape(-1), r["p"], "p of " + what, scale=before)
            # the next step starts from the oracle's parameters on both sides
            p.data.copy_(to_dev(r["p"]).view(p.shape))


def _single_tensor_copies(params):
    """Per tensor: copies of the parameter and fresh states for single-tensor C-ABI calls."""
    out = []
    for p in params:
        n = p.numel()
        if n > 4096:
            out.append(dict(n=n, p=p.detach().clone(), mc=torch.zeros(n // 2, dtype=torch.int8, device=p.device),
                            vc=torch.zeros(n // 2, dtype=torch.int8, device=p.device),
                            ms=torch.zeros((n + 127) // 128, device=p.device),
                            vs=torch.zeros((n + 127) // 128, device=p.device)))
        else:
            out.append(dict(n=n, p=p.detach().clone(), m=torch.zeros(n, device=p.device),
                            v=torch.zeros(n, device=p.device)))
    return out


def _single_tensor_step(lib, copies, params, dqm, dqv, step):
    stream = torch.cuda.current_stream().cuda_stream
    for c, p in zip(copies, params):
        g = p.grad
        if "mc" in c:
            st = lib.lpmm_adamw4bit_step(c["p"].data_ptr(), g.data_ptr(), c["mc"].data_ptr(), c["vc"].data_ptr(),
                                         c["ms"].data_ptr(), c["vs"].data_ptr(), dqm.data_ptr(), dqv.data_ptr(),
                                         c["n"], *HO, float(step), stream)
        else:
            st = lib.lpmm_adamw_fp32_step(c["p"].data_ptr(), g.data_ptr(), c["m"].data_ptr(), c["v"].data_ptr(),
                                          c["n"], *HO, float(step), stream)
        assert st == 0


def _assert_set_equal(opt, params, copies, step):
    for i, (p, c) in enumerate(zip(params, copies)):
        st = opt.state[p]
        what = f"tensor {i} {tuple(p.shape)} step {step}"
        assert torch.equal(p.detach().view(-1), c["p"].view(-1)), "p of " + what
        if "mc" in c:
            assert torch.equal(st["exp_avg"], c["mc"]), "m codes of " + what
            assert torch.equal(st["exp_avg_sq"], c["vc"]), "v codes of " + what
            assert torch.equal(st["exp_avg_qstate"]["overhead"]["max1"], c["ms"]), "m scales of " + what
            assert torch.equal(st["exp_avg_sq_qstate"]["overhead"]["max1"], c["vs"]), "v scales of " + what
        else:
            assert torch.equal(st["exp_avg"].view(-1), c["m"]), "m of " + what
            assert torch.equal(st["exp_avg_sq"].view(-1), c["v"]), "v of " + what


def test_gpt2xl_whole_set_equals_single_tensor_calls(qmaps):
    """The configuration as written: 580 tensors, parameters N(0, 0.02), gradients N(0, 1e-3)
    reseeded every step, 20 steps.  The optimizer (7 launches of up to 48 quantised tensors, one
    of them ragged, and 5 of up to 64 fp32-state vectors per step) must leave exactly the bytes
    that 580 single-tensor calls per step leave on copies."""
    from lpmm import _native

    lib = _native.lib()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    params = []
    for i, shape in enumerate(gpt2xl_shapes()):
        gen.manual_seed(10000 + i)
        params.append(torch.nn.Parameter(torch.randn(shape, device=dev, generator=gen) * 0.02))
    copies = _single_tensor_copies(params)
    opt = _make_optimizer(params)
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    for step in range(1, 21):
        for i, p in enumerate(params):
            gen.manual_seed(20000 + 1000 * step + i)
            p.grad = torch.randn(p.shape, device=dev, generator=gen) * 1e-3
        opt.step()
        _single_tensor_step(lib, copies, params, dqm, dqv, step)
        if step in (1, 2, 20):
            torch.cuda.synchronize()
            _assert_set_equal(opt, params, copies, step)
    # the moments have really moved: no quantised state is still all zero
    assert all(int(opt.state[p]["exp_avg_sq"].ne(0).sum()) > 0 for p in params if p.numel() > 4096)


def test_llama7b_whole_set_equals_single_tensor_calls(qmaps):
    """All 291 LLaMA-7B-shaped tensors (6.7e9 parameters, launches of 48 tensors with up to 7e5
    tiles) with heavy-tailed gradients (Student-t, 3 degrees of freedom, x 1e-3), three steps."""
    from lpmm import _native

    lib = _native.lib()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    params = []
    for i, shape in enumerate(llama7b_shapes()):
        gen.manual_seed(10000 + i)
        params.append(torch.nn.Parameter(torch.randn(shape, device=dev, generator=gen) * 0.02))
    copies = _single_tensor_copies(params)
    opt = _make_optimizer(params)
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    for p in params:
        p.grad = torch.empty_like(p)
    for step in (1, 2, 3):
        for i, p in enumerate(params):
            gen.manual_seed(20000 + 1000 * step + i)
            z = torch.randn(p.shape, device=dev, generator=gen)
            s = torch.zeros(p.shape, device=dev)
            for _ in range(3):
                a = torch.randn(p.shape, device=dev, generator=gen)
                s.addcmul_(a, a)
            p.grad.copy_(z.div_(s.div_(3.0).sqrt_()).mul_(1e-3))
            del z, s, a
        opt.step()
        _single_tensor_step(lib, copies, params, dqm, dqv, step)
        torch.cuda.synchronize()
        _assert_set_equal(opt, params, copies, step)


# ---------------------------------------------------------------------------------------
# The factored configuration as a whole set (lpmm/optim/adamw.py:579-627 for the matrices,
# :332-436 / :439-561 for the vectors, which keep a 4-bit or fp32 second moment).
# ---------------------------------------------------------------------------------------
def factored_shapes():
    shapes = []
    for _ in range(32):
        shapes += [(4096, 11008), (11008, 4096), (4096, 4096), (11008,), (4096,)]
    return shapes


def _factored_copies(params, fused, qm):
    """Per tensor: a copy of the parameter and fresh states in the layouts the single-tensor entry points take."""
    from lpmm import _native
    from lpmm.functional import packed_nbytes
    from lpmm.optim.adamw import _zero_byte

    lib = _native.lib()
    out = []
    for p in params:
        n, dev = p.numel(), p.device
        c = dict(n=n, p=p.detach().clone())
        if p.dim() == 2:
            rows, cols = p.shape
            c.update(kind="factored", mc=torch.empty(packed_nbytes(n), dtype=torch.int8, device=dev),
                     ms=torch.empty(n // 128, device=dev), row=torch.zeros(rows, device=dev),
                     col=torch.zeros(cols, device=dev), mean=torch.zeros(1, device=dev),
                     work=torch.empty(lib.lpmm_factored_workspace_bytes(rows, cols), dtype=torch.uint8, device=dev))
        elif n > 4096 and fused:
            c.update(kind="fused4", mc=torch.zeros(n // 2, dtype=torch.int8, device=dev),
                     vc=torch.zeros(n // 2, dtype=torch.int8, device=dev), ms=torch.zeros(n // 128, device=dev),
                     vs=torch.zeros(n // 128, device=dev))
        elif n > 4096:
            zero = _zero_byte(qm)
            c.update(kind="nonfused4", mc=torch.full((packed_nbytes(n),), zero, dtype=torch.int8, device=dev),
                     vc=torch.full((packed_nbytes(n),), 0, dtype=torch.int8, device=dev),
                     ms=torch.zeros(n // 128, device=dev), vs=torch.zeros(n // 128, device=dev))
        else:
            c.update(kind="fp32", m=torch.zeros(n, device=dev), v=torch.zeros(n, device=dev))
        out.append(c)
    return out


def _factored_single_step(lib, nat, copies, params, dqm, dqv, step, fused):
    stream = torch.cuda.current_stream().cuda_stream
    b1, b2, lr, wd, eps = HO
    for c, p in zip(copies, params):
        g = p.grad
        if c["kind"] == "factored":
            rows, cols = p.shape
            st = lib.lpmm_factored_stats(g.data_ptr(), rows, cols, c["row"].data_ptr(), c["col"].data_ptr(),
                                         c["mean"].data_ptr(), b2, c["work"].data_ptr(), stream)
            assert st == 0
            st = lib.lpmm_factored_update(c["p"].data_ptr(), g.data_ptr(), c["mc"].data_ptr(), c["ms"].data_ptr(),
                                          dqm.data_ptr(), c["row"].data_ptr(), c["col"].data_ptr(),
                                          c["mean"].data_ptr(), rows, cols, b1, b2, lr, wd, eps, float(step),
                                          1 if step == 1 else 0, stream)
        elif c["kind"] == "fused4":
            st = lib.lpmm_adamw4bit_step(c["p"].data_ptr(), g.data_ptr(), c["mc"].data_ptr(), c["vc"].data_ptr(),
                                         c["ms"].data_ptr(), c["vs"].data_ptr(), dqm.data_ptr(), dqv.data_ptr(),
                                         c["n"], *HO, float(step), stream)
        elif c["kind"] == "nonfused4":
            rec = np.array([(c["p"].data_ptr(), g.data_ptr(), c["mc"].data_ptr(), c["vc"].data_ptr(),
                             c["ms"].data_ptr(), c["vs"].data_ptr(), c["n"], float(step), 0.0)],
                           dtype=nat.ADAMW4BIT_TENSOR)
            st = lib.lpmm_nonfused_adamw4bit_step_multi(rec.ctypes.data, 1, dqm.data_ptr(), dqv.data_ptr(), b1, b2,
                                                        lr, wd, eps, stream)
        elif fused:
            st = lib.lpmm_adamw_fp32_step(c["p"].data_ptr(), g.data_ptr(), c["m"].data_ptr(), c["v"].data_ptr(),
                                          c["n"], *HO, float(step), stream)
        else:
            st = lib.lpmm_nonfused_update(c["p"].data_ptr(), g.data_ptr(), c["m"].data_ptr(), c["v"].data_ptr(),
                                          c["n"], b1, b2, lr, wd, eps, float(step), stream)
        assert st == 0


def _assert_factored_set_equal(opt, params, copies, step):
    for i, (p, c) in enumerate(zip(params, copies)):
        st = opt.state[p]
        what = f"tensor {i} {tuple(p.shape)} step {step}"
        assert float(st["step"]) == float(step)
        assert torch.equal(p.detach().view(-1), c["p"].view(-1)), "p of " + what
        if c["kind"] == "factored":
            assert "exp_avg_sq" not in st
            assert torch.equal(st["exp_avg_sq_row"].view(-1), c["row"]), "row statistics of " + what
            assert torch.equal(st["exp_avg_sq_col"].view(-1), c["col"]), "column statistics of " + what
            assert torch.equal(st["exp_avg"], c["mc"]), "m codes of " + what
            assert torch.equal(st["exp_avg_qstate"]["overhead"]["max1"].view(-1), c["ms"]), "m scales of " + what
        elif c["kind"] in ("fused4", "nonfused4"):
            assert torch.equal(st["exp_avg"], c["mc"]), "m codes of " + what
            assert torch.equal(st["exp_avg_sq"], c["vc"]), "v codes of " + what
            assert torch.equal(st["exp_avg_qstate"]["overhead"]["max1"].view(-1), c["ms"]), "m scales of " + what
            assert torch.equal(st["exp_avg_sq_qstate"]["overhead"]["max1"].view(-1), c["vs"]), "v scales of " + what
        else:
            assert torch.equal(st["exp_avg"].view(-1), c["m"]), "m of " + what
            assert torch.equal(st["exp_avg_sq"].view(-1), c["v"]), "v of " + what


@pytest.mark.parametrize("fused", [True, False])
def test_factored_whole_set_equals_single_tensor_calls(qmaps, fused):
    """The factored configuration as written: 32 x {4096 x 11008, 11008 x 4096, 4096 x 4096} with a factored
    second moment, 32 vectors of 11008 values that keep 4-bit moments and 32 of 4096 values with fp32 moments
    (3.4e9 parameters), gradients N(0, 1e-3) reseeded every step, 20 steps through
    lpmm.optim.AdamW(factor_second_moment=True).  The optimizer's launches (96 matrices in groups of 24 with
    four launches each and a workspace carved per tensor, the vectors in multi-tensor launches of their own)
    must leave exactly the bytes that single-tensor calls leave on copies: lpmm_factored_stats +
    lpmm_factored_update per matrix, the 4-bit and fp32 step entry points per vector."""
    import lpmm
    from lpmm import _native

    lib = _native.lib()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    params = []
    for i, shape in enumerate(factored_shapes()):
        gen.manual_seed(10000 + i)
        params.append(torch.nn.Parameter(torch.randn(shape, device=dev, generator=gen) * 0.02))
    assert sum(p.numel() for p in params) == 32 * (2 * 4096 * 11008 + 4096 * 4096 + 11008 + 4096)
    opt = lpmm.optim.AdamW(params, lr=HO[2], betas=(HO[0], HO[1]), eps=HO[4], weight_decay=HO[3], fused=fused,
                           factor_second_moment=True)
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    copies = _factored_copies(params, fused, dqm)
    for p in params:
        p.grad = torch.empty_like(p)
    for step in range(1, 21):
        for i, p in enumerate(params):
            gen.manual_seed(20000 + 1000 * step + i)
            p.grad.normal_(0.0, 1e-3, generator=gen)
        opt.step()
        _factored_single_step(lib, _native, copies, params, dqm, dqv, step, fused)
        if step in (1, 2, 20):
            torch.cuda.synchronize()
            _assert_factored_set_equal(opt, params, copies, step)
    # the states really are the factored ones and have moved
    st = opt.state[params[0]]
    assert st["exp_avg_sq_row"].shape[0] == 4096 and st["exp_avg_sq_col"].shape[0] == 11008
    assert float(st["exp_avg_sq_row"].min()) > 0.0 and int(st["exp_avg"].ne(0).sum()) > 0
