"""Parity at the benchmark configurations' real tensor sizes: every distinct LLaMA-7B shape
through the fused step, 2^26 values through the stand-alone quantisers, a 4096 x 11008
tensor through the factored step -- each compared with the CPU oracle on seeded inputs, plus
size-independent properties (quantise -> dequantise -> quantise is idempotent; the largest
element of every group decodes to its scale)."""
import numpy as np
import pytest
import torch

from util import assert_codes, assert_params, assert_rel, nibbles, to_dev, to_np

pytestmark = pytest.mark.gpu

HO = (0.9, 0.999, 1e-3, 0.01, 1e-8)


def _student_t(rng, n):
    z = rng.standard_normal((4, n), dtype=np.float32)
    return (z[0] / np.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3.0) * 1e-3).astype(np.float32)


@pytest.mark.parametrize("shape", [(32000, 4096), (4096, 4096), (11008, 4096), (4096, 11008)])
def test_fused_step_llama_shapes(oracle, qmaps, shape):
    from lpmm import _native

    lib = _native.lib()
    qm, qv = qmaps
    n = shape[0] * shape[1]
    rng = np.random.default_rng(shape[0] + 3 * shape[1])
    p_ref = (rng.standard_normal(n, dtype=np.float32) * 0.02).astype(np.float32)
    mc_ref, vc_ref = np.zeros(n // 2, np.uint8), np.zeros(n // 2, np.uint8)
    ms_ref, vs_ref = np.zeros(n // 128, np.float32), np.zeros(n // 128, np.float32)
    p, mc, vc, ms, vs = (to_dev(a) for a in (p_ref, mc_ref, vc_ref, ms_ref, vs_ref))
    dqm, dqv = to_dev(qm), to_dev(qv)
    for step in (1, 2, 3):
        g_np = _student_t(rng, n)
        g = to_dev(g_np)
        st = lib.lpmm_adamw4bit_step(p.data_ptr(), g.data_ptr(), mc.data_ptr(), vc.data_ptr(), ms.data_ptr(),
                                     vs.data_ptr(), dqm.data_ptr(), dqv.data_ptr(), n, *HO, float(step),
                                     torch.cuda.current_stream().cuda_stream)
        assert st == 0
        p_before = p_ref.copy()
        oracle.adamw4bit_step(p_ref, g_np, mc_ref, vc_ref, ms_ref, vs_ref, qm, qv, *HO, float(step))
        torch.cuda.synchronize()
        flips = assert_codes(to_np(mc), mc_ref, n, f"m codes step {step}")
        flips += assert_codes(to_np(vc), vc_ref, n, f"v codes step {step}")
        assert_rel(to_np(ms), ms_ref, "m scales")
        assert_rel(to_np(vs), vs_ref, "v scales")
        assert_params(to_np(p), p_ref, p_before, f"p step {step}")
        p.copy_(torch.from_numpy(p_ref))
        if flips:
            for d, h in ((mc, mc_ref), (vc, vc_ref), (ms, ms_ref), (vs, vs_ref)):
                d.copy_(torch.from_numpy(h))
    # property: the group maximum decodes to the scale (code 15 on the v map)
    cv = nibbles(to_np(vc), n).reshape(-1, 128)
    assert np.all(cv.max(axis=1) == 15)


def test_nonfused_default_config_4096x4096(oracle, qmaps):
    """The first benchmark configuration as it is written: non-fused lpmm.optim.AdamW with the
    default configuration file (m block-wise 128 with the signed map, v rank-1 with the linear
    map), one 4096 x 4096 fp32 parameter ~ N(0, 0.02), gradients ~ N(0, 1e-3) reseeded each
    step, lr 1e-3, betas (0.9, 0.999), wd 0.01, 10 steps -- against the oracle's staged
    sequence on the same inputs."""
    import os

    import lpmm

    qm, qv = qmaps
    shape = (4096, 4096)
    p_ref = (torch.randn(shape, generator=torch.Generator().manual_seed(0)) * 0.02).numpy()
    p = torch.nn.Parameter(to_dev(p_ref))
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "default.yml")
    opt = lpmm.optim.AdamW([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, fused=False, qconfig=cfg)
    state = oracle.NonFusedState(shape, v_scale_type="rank1")
    n = p_ref.size
    for step in range(1, 11):
        g_np = (torch.randn(shape, generator=torch.Generator().manual_seed(1000 + step)) * 1e-3).numpy()
        p.grad = to_dev(g_np)
        opt.step()
        p_before = p_ref.copy()
        oracle.nonfused_step(p_ref, g_np, state, qm, qv, 1e-3, 0.9, 0.999, 1e-8, 0.01)
        torch.cuda.synchronize()
        st = opt.state[p]
        oh = st["exp_avg_sq_qstate"]["overhead"]
        np.testing.assert_array_equal(to_np(oh["max_dims"][0]).reshape(-1), state.v[1], err_msg=f"row maxima step {step}")
        np.testing.assert_array_equal(to_np(oh["max_dims"][1]).reshape(-1), state.v[2], err_msg=f"col maxima step {step}")
        np.testing.assert_array_equal(to_np(st["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), state.m[1])
        assert_codes(to_np(st["exp_avg"]), state.m[0], n, f"m codes step {step}")
        assert_codes(to_np(st["exp_avg_sq"]), state.v[0], n, f"v codes step {step}")
        assert_rel(to_np(p.detach()), p_ref, f"p step {step}", scale=p_before)


def test_quant_roundtrip_64m(oracle, qmaps):
    import lpmm.functional as F

    n = 1 << 26
    rng = np.random.default_rng(1)
    signed = rng.standard_normal(n, dtype=np.float32)
    signed[rng.permutation(n)[: n // 1000]] *= 50.0
    unsigned = (rng.standard_normal(n, dtype=np.float32) ** 2).astype(np.float32)
    qm, qv = to_dev(qmaps[0]), to_dev(qmaps[1])
    md_m = dict(b=4, scale_type="group", quant_type="nonlinear", round_type="real-nearest", gp_sz=128, signed=True)
    md_vg = dict(b=4, scale_type="group", quant_type="power-1", round_type="real-nearest", gp_sz=128, signed=False)
    md_vr = dict(md_vg, scale_type="rank1")
    for name, x, dq, hq, md in (("signed", signed, qm, qmaps[0], md_m), ("unsigned", unsigned, qv, qmaps[1], md_vg)):
        dx = to_dev(x)
        qx, gen = F.vectorwise_quant(dx, qmap=dq, shape=dx.shape, **md)
        want_codes, want_max1 = oracle.quant_group(x, hq, 128)
        np.testing.assert_array_equal(to_np(gen["max1"]).reshape(-1), want_max1)
        np.testing.assert_array_equal(to_np(qx).view(np.uint8), want_codes)
        back = F.vectorwise_dequant(qx, qmap=dq, shape=dx.shape, **{**gen, **md})
        want_back = oracle.dequant_group(want_codes, want_max1, hq, n)
        np.testing.assert_array_equal(to_np(back), want_back)
        # round-trip error equals the oracle's (lpmm/utils.py:84-87 formula)
        rel = np.linalg.norm(x.astype(np.float64) - want_back) / np.linalg.norm(x.astype(np.float64))
        got = float((dx.double() - back.double()).norm() / dx.double().norm())
        assert abs(got - rel) <= 1e-9 * rel
        if name == "unsigned":
            # idempotence on the unsigned map (its largest element decodes to exactly the scale;
            # on the signed map a negative maximum decodes to -0.8875 * scale, so the scale shrinks)
            qx2, gen2 = F.vectorwise_quant(back, qmap=dq, shape=dx.shape, **md)
            assert torch.equal(gen2["max1"], gen["max1"]) and torch.equal(qx2, qx)
    # rank-1 on the unsigned data viewed 8192 x 8192
    x2 = unsigned.reshape(8192, 8192)
    dx = to_dev(x2)
    qx, gen = F.vectorwise_quant(dx, qmap=qv, shape=dx.shape, **md_vr)
    row, col = oracle.rank1_stats(x2)
    np.testing.assert_array_equal(to_np(gen["max_dims"][0]).reshape(-1), row)
    np.testing.assert_array_equal(to_np(gen["max_dims"][1]).reshape(-1), col)
    want_codes = oracle.quant_rank1(x2, row, col, qmaps[1])
    np.testing.assert_array_equal(to_np(qx).view(np.uint8), want_codes)
    back = F.vectorwise_dequant(qx, qmap=qv, shape=dx.shape, **{**gen, **md_vr})
    np.testing.assert_array_equal(to_np(back), oracle.dequant_rank1(want_codes, row, col, qmaps[1], 8192, 8192))


@pytest.mark.parametrize("shape", [(4096, 11008), (11008, 4096), (4096, 4096)])
def test_factored_step_llama_shapes(oracle, qmaps, shape):
    """The three matrix shapes of the factored configuration at full size, three steps each, against
    the oracle (the tall 11008 x 4096 has the most row tiles, the wide 4096 x 11008 the most column tiles)."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(9 + shape[0])
    host = (rng.standard_normal(shape, dtype=np.float32) * 0.02).astype(np.float32)
    param = torch.nn.Parameter(to_dev(host))
    opt = lpmm.optim.AdamW([param], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01,
                           factor_second_moment=True, fused=True)
    state = oracle.NonFusedState(shape, factored=True)
    for step in range(1, 4):
        g = (rng.standard_normal(shape, dtype=np.float32) * 1e-3).astype(np.float32)
        param.grad = to_dev(g)
        before = host.copy()
        opt.step()
        oracle.nonfused_step(host, g, state, qm, qv, 1e-3, 0.9, 0.999, 1e-8, 0.01)
        torch.cuda.synchronize()
        s = opt.state[param]
        assert_rel(to_np(s["exp_avg_sq_row"]), state.row, "row", tol=1e-6)
        assert_rel(to_np(s["exp_avg_sq_col"]), state.col, "col", tol=1e-6)
        np.testing.assert_array_equal(to_np(s["exp_avg"]).view(np.uint8), state.m[0])
        np.testing.assert_array_equal(to_np(s["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), state.m[1])
        assert_rel(to_np(param), host, "p", scale=before)


def test_indexing_beyond_two_to_the_31_elements(qmaps):
    """One tensor of 2^31 + 4160 elements (its byte offsets pass 2^33, its last group holds 64
    values) must come out exactly as the same buffers processed as two tensors split at a
    group boundary: groups are independent, and the two halves are indexed with small numbers,
    the regime the oracle comparisons cover.  Fused step (two steps, the second from non-zero
    states), then the block-wise quantiser and dequantiser on the same number of values."""
    from lpmm import _native

    lib = _native.lib()
    stream = torch.cuda.current_stream().cuda_stream
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    n = (1 << 31) + 4160
    cut = (1 << 30) + 128 * 5  # a group boundary that is not a tile boundary
    gen = torch.Generator(device="cuda").manual_seed(31)
    g = torch.empty(n, device="cuda")
    p0 = torch.empty(n, device="cuda")
    chunk = 1 << 28
    for lo in range(0, n, chunk):  # filled in pieces: bounded temporaries
        hi = min(n, lo + chunk)
        p0[lo:hi] = torch.randn(hi - lo, device="cuda", generator=gen) * 0.02
        g[lo:hi] = torch.randn(hi - lo, device="cuda", generator=gen) * 1e-3
    groups = (n + 127) // 128

    def fresh():
        return dict(p=p0.clone(), mc=torch.zeros(n // 2, dtype=torch.uint8, device="cuda"),
                    vc=torch.zeros(n // 2, dtype=torch.uint8, device="cuda"),
                    ms=torch.zeros(groups, device="cuda"), vs=torch.zeros(groups, device="cuda"))

    a, b = fresh(), fresh()
    for step in (1.0, 2.0):
        st = lib.lpmm_adamw4bit_step(a["p"].data_ptr(), g.data_ptr(), a["mc"].data_ptr(), a["vc"].data_ptr(),
                                     a["ms"].data_ptr(), a["vs"].data_ptr(), dqm.data_ptr(), dqv.data_ptr(), n, *HO,
                                     step, stream)
        assert st == 0, lib.lpmm_status_string(st)
        recs = []
        for lo, hi in ((0, cut), (cut, n)):
            recs.append((b["p"].data_ptr() + 4 * lo, g.data_ptr() + 4 * lo, b["mc"].data_ptr() + lo // 2,
                         b["vc"].data_ptr() + lo // 2, b["ms"].data_ptr() + 4 * (lo // 128),
                         b["vs"].data_ptr() + 4 * (lo // 128), hi - lo, step, 0.0))
        table = np.array(recs, dtype=_native.ADAMW4BIT_TENSOR)
        st = lib.lpmm_adamw4bit_step_multi(table.ctypes.data, 2, dqm.data_ptr(), dqv.data_ptr(), *HO, stream)
        assert st == 0, lib.lpmm_status_string(st)
        torch.cuda.synchronize()
        for k in ("p", "mc", "vc", "ms", "vs"):
            assert torch.equal(a[k], b[k]), f"{k} differs after step {step}"
    # the states are non-trivial: the last (64-value) group has a scale and the codes of its missing half stay 0
    assert float(a["vs"][-1]) > 0 and int(a["mc"][-1]) != 0
    del a, b, p0
    torch.cuda.empty_cache()

    # block-wise quantiser / dequantiser in the non-fused layout, split at a 2048-value pack boundary
    cutq = (1 << 30) + 2048 * 3
    nbytes = (n + 2047) // 2048 * 1024 + 1
    codes_a = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    codes_b = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    max_a, max_b = torch.zeros(groups, device="cuda"), torch.zeros(groups, device="cuda")
    assert lib.lpmm_quant_group(g.data_ptr(), n, 128, dqm.data_ptr(), codes_a.data_ptr(), max_a.data_ptr(), stream) == 0
    assert lib.lpmm_quant_group(g.data_ptr() + 4 * cutq, n - cutq, 128, dqm.data_ptr(), codes_b.data_ptr() + cutq // 2,
                                max_b.data_ptr() + 4 * (cutq // 128), stream) == 0
    # the first part second: its trailing byte (always written as 0) lands on the first code byte of the second part
    tail = codes_b[cutq // 2].clone()
    assert lib.lpmm_quant_group(g.data_ptr(), cutq, 128, dqm.data_ptr(), codes_b.data_ptr(), max_b.data_ptr(), stream) == 0
    codes_b[cutq // 2] = tail
    torch.cuda.synchronize()
    assert torch.equal(codes_a, codes_b) and torch.equal(max_a, max_b)
    out_a = torch.empty(n, device="cuda")
    assert lib.lpmm_dequant_group(codes_a.data_ptr(), max_a.data_ptr(), dqm.data_ptr(), n, 128, out_a.data_ptr(), stream) == 0
    out_b = torch.empty(n, device="cuda")
    assert lib.lpmm_dequant_group(codes_a.data_ptr(), max_a.data_ptr(), dqm.data_ptr(), cutq, 128, out_b.data_ptr(), stream) == 0
    assert lib.lpmm_dequant_group(codes_a.data_ptr() + cutq // 2, max_a.data_ptr() + 4 * (cutq // 128), dqm.data_ptr(),
                                  n - cutq, 128, out_b.data_ptr() + 4 * cutq, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b)
    # and the round trip is what quantisation promises: every value within its group's scale
    err = (out_a[: 1 << 20] - g[: 1 << 20]).abs().max()
    assert float(err) <= float(max_a[: 1 << 13].max())


@pytest.mark.parametrize("shape", [(64, 1024, 1024), (512, 512, 3, 3), (16, 8, 128, 4096)])
def test_rank1_nd_statistics_at_size(oracle, qmaps, shape):
    """Rank-1 statistics, quantise and dequantise of 3-D and 4-D tensors of 2.4e6 .. 6.7e7 values through
    lpmm.functional against the N-D oracle (the stacked-matrix shapes take the 2-D kernel plus the fold of its row
    maxima, the convolution-shaped one the one-pass kernel on the tensor itself)."""
    import lpmm.functional as F

    rng = np.random.default_rng(len(shape) * 100 + shape[0])
    x = (rng.standard_normal(shape, dtype=np.float32) ** 2).astype(np.float32)
    x *= np.exp(rng.standard_normal((shape[0],) + (1,) * (len(shape) - 1))).astype(np.float32)
    dx = to_dev(x)
    md = dict(b=4, scale_type="rank1", quant_type="power-1", round_type="real-nearest", gp_sz=128, signed=False)
    dq = to_dev(qmaps[1])
    codes, gen = F.vectorwise_quant(dx, qmap=dq, shape=dx.shape, **md)
    want_stats = oracle.rank1_stats_nd(x)
    for i, (got, want) in enumerate(zip(gen["max_dims"], want_stats)):
        np.testing.assert_array_equal(to_np(got).reshape(-1), want, err_msg=f"statistics of dimension {i}")
    want_codes = oracle.quant_rank1_nd_bits(x, want_stats, qmaps[1], 4)
    np.testing.assert_array_equal(to_np(codes).view(np.uint8), want_codes)
    back = F.vectorwise_dequant(codes, qmap=dq, shape=dx.shape, **{**gen, **md})
    np.testing.assert_array_equal(to_np(back), oracle.dequant_rank1_nd_bits(want_codes, want_stats, qmaps[1], 4, shape))


@pytest.mark.parametrize("v_scale", ["rank1", "group"])
def test_half_step_kernels_at_4096x11008(oracle, qmaps, v_scale):
    """float16 parameters with fused=False at a LLaMA-7B MLP shape through the optimizer (the two-pass half
    kernels under the default configuration, the one-pass kernel with a block-wise second moment) against
    the oracle's float16 restatement of the reference's chain, two steps, bit for bit."""
    import os

    import lpmm

    qm, qv = qmaps
    shape = (4096, 11008)
    rng = np.random.default_rng(77)
    host = (rng.standard_normal(shape, dtype=np.float32) * 0.02).astype(np.float16)
    p = torch.nn.Parameter(to_dev(host.copy()))
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs",
                       "default.yml" if v_scale == "rank1" else "2nd_moment_group_128.yml")
    hyper = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-3, weight_decay=0.01)
    opt = lpmm.optim.AdamW([p], fused=False, qconfig=cfg, **hyper)
    state = oracle.NonFusedState(shape, v_scale)

    def same(got, want, what):
        got, want = np.ascontiguousarray(got).reshape(-1), np.ascontiguousarray(want).reshape(-1)
        assert got.dtype == want.dtype == np.float16, what
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), what

    for step in (1, 2):
        g = (rng.standard_normal(shape, dtype=np.float32) * 0.05).astype(np.float16)
        p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        oracle.nonfused_step_f16(host, g, state, qm, qv, hyper["lr"], 0.9, 0.999, hyper["eps"], 0.01)
        st = opt.state[p]
        same(to_np(p.detach()), host, f"step {step}: p")
        same(to_np(st["exp_avg_qstate"]["overhead"]["max1"]), state.m[1], f"step {step}: m max1")
        np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), state.m[0])
        np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), state.v[0])
        oh_v = st["exp_avg_sq_qstate"]["overhead"]
        if v_scale == "rank1":
            same(to_np(oh_v["max_dims"][0]), state.v[1], f"step {step}: row statistics")
            same(to_np(oh_v["max_dims"][1]), state.v[2], f"step {step}: column statistics")
        else:
            same(to_np(oh_v["max1"]), state.v[1], f"step {step}: v max1")
