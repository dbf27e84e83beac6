"""Pins of the oracle's step, quantise and statistics functions (no GPU): closed forms,
library routines (torch.optim.AdamW, PyTorch CPU ops, numpy), invariants, special cases."""
import os

import numpy as np
import pytest
import torch

from util import assert_codes, assert_rel, nibbles

HERE = os.path.dirname(os.path.abspath(__file__))
H = dict(beta1=0.9, beta2=0.999, lr=1e-3, wd=0.01, eps=1e-8)
f32 = np.float32


def test_pack_layout_exhaustive(oracle, qmaps):
    """All 256 byte values survive unpack -> pack; low nibble = even element; sizes."""
    for q in qmaps:
        allbytes = np.arange(256, dtype=np.uint8)
        vals = oracle.unpack_nonlinear_4bit(allbytes, q, 512)
        assert np.array_equal(vals[0::2], q[allbytes & 0xF]) and np.array_equal(vals[1::2], q[allbytes >> 4])
        packed = oracle.pack_nonlinear_4bit(vals, q)
        assert packed.size == 512 // 2 + 1 and packed[-1] == 0
        assert np.array_equal(packed[:-1], allbytes)
    assert oracle.packed_nbytes_nonfused(4096 * 4096) == 8388609  # NG*1024 + 1
    assert oracle.packed_nbytes_nonfused(2 ** 26) == 33554433
    assert oracle.packed_nbytes_nonfused(4097) == 3 * 1024 + 1


def test_fp32_step_equals_torch_adamw(oracle):
    """lpmm_oracle_adamw_fp32_step against the library routine torch.optim.AdamW, and against
    the recurrences evaluated in double.

    The reference kernel takes its scalars as C floats and forms 1-beta in float
    (lpmm/cpp_extension/fused_adamw_kernel.cu:68-69): with beta2 = 0.999 that is
    1 - fl32(0.999) = 0.00099998712, 1.29e-5 below the 0.001 PyTorch uses, so v (and only v)
    differs from torch.optim.AdamW by that relative amount; everything else agrees to
    rounding.  The double recurrence below uses the float-rounded constants and pins v."""
    torch.manual_seed(0)
    n = 5000
    p0 = torch.randn(n) * 0.02
    pt = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([pt], lr=H["lr"], betas=(H["beta1"], H["beta2"]), eps=H["eps"], weight_decay=H["wd"])
    p, m, v = p0.numpy().copy(), np.zeros(n, f32), np.zeros(n, f32)
    b1, b2 = float(f32(H["beta1"])), float(f32(H["beta2"]))
    omb1, omb2 = float(f32(1) - f32(H["beta1"])), float(f32(1) - f32(H["beta2"]))
    md, vd = np.zeros(n), np.zeros(n)
    for s in range(1, 101):
        g = torch.randn(n) * 1e-3
        pt.grad = g.clone()
        opt.step()
        gn = g.numpy().copy()
        oracle.adamw_fp32_step(p, gn, m, v, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], float(s))
        md = b1 * md + omb1 * gn.astype(np.float64)
        vd = b2 * vd + omb2 * gn.astype(np.float64) ** 2
        if s == 1:
            assert_rel(p, pt.detach().numpy(), "p after one step", tol=1e-6, scale=p0.numpy())
    # m is a signed sum: entries near zero are compared on the scale of a typical entry
    typical = np.full(n, np.abs(md).mean())
    assert_rel(m, md, "m vs double recurrence", tol=2e-6, scale=typical)
    assert_rel(v, vd, "v vs double recurrence", tol=2e-6)
    st = opt.state[pt]
    assert_rel(m, st["exp_avg"].numpy(), "m vs torch", tol=1e-5, scale=typical)
    assert_rel(v, st["exp_avg_sq"].numpy(), "v vs torch", tol=1.29e-5 + 2e-6)
    # rounding differences of the two algebraically equal update forms accumulate like a random walk
    assert np.max(np.abs(p - pt.detach().numpy())) <= 1e-5 * np.max(np.abs(p))


def test_fused_first_step_closed_form(oracle, qmaps):
    """From zero state: m1 = (1-b1) g, v1 = (1-b2) g^2,
    p1 = p0 - lr (m1 / ((sqrt(v1)/sqrt(1-b2) + eps)(1-b1)) + wd p0), evaluated in double."""
    qm, qv = qmaps
    rng = np.random.default_rng(1)
    n = 128 * 9 + 50
    p0 = (rng.standard_normal(n) * 0.02).astype(f32)
    g = (rng.standard_normal(n) * 1e-3).astype(f32)
    p = p0.copy()
    nb, ng = (n + 1) // 2, (n + 127) // 128
    mc, vc, ms, vs = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8), np.zeros(ng, f32), np.zeros(ng, f32)
    oracle.adamw4bit_step(p, g, mc, vc, ms, vs, qm, qv, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], 1.0)
    gd, pd = g.astype(np.float64), p0.astype(np.float64)
    b1, b2 = float(f32(H["beta1"])), float(f32(H["beta2"]))
    m1, v1 = (1 - b1) * gd, (1 - b2) * gd * gd
    want = pd - H["lr"] * (m1 / ((np.sqrt(v1) / np.sqrt(1 - b2) + H["eps"]) * (1 - b1)) + H["wd"] * pd)
    assert_rel(p, want, "p1 closed form", tol=1e-6, scale=p0)
    # scales are the group maxima of m1 / v1, and the maximal element decodes to the scale
    pad = np.zeros(ng * 128)
    pad[:n] = np.abs(m1)
    assert_rel(ms, pad.reshape(ng, 128).max(1), "m scale", tol=1e-6)
    pad[:n] = v1
    assert_rel(vs, pad.reshape(ng, 128).max(1), "v scale", tol=1e-6)
    cm, cv = nibbles(mc, n), nibbles(vc, n)
    for grp in range(ng):
        sl = slice(grp * 128, min(n, (grp + 1) * 128))
        k = np.argmax(np.abs(m1[sl]))
        assert cm[sl][k] == (15 if m1[sl][k] > 0 else 0)  # +1.0*scale or -0.8875*scale
        assert cv[sl][np.argmax(v1[sl])] == 15
    assert np.all(cv[v1 * 16 < vs.repeat(128)[:n] * 0.5] == 0)  # zero is excluded: small values take code 0


def test_fused_step_is_dequant_fp32step_quant(oracle, qmaps):
    """The fused step equals: dequantise (group-128) -> fp32 AdamW step -> group absmax quantise,
    each of which is pinned separately."""
    qm, qv = qmaps
    rng = np.random.default_rng(2)
    n = 128 * 40
    p = (rng.standard_normal(n) * 0.02).astype(f32)
    nb, ng = n // 2, n // 128
    mc, vc = rng.integers(0, 256, nb, dtype=np.uint8), rng.integers(0, 256, nb, dtype=np.uint8)
    ms = np.abs(rng.standard_normal(ng) * 1e-3).astype(f32)
    vs = np.abs(rng.standard_normal(ng) * 1e-6).astype(f32)
    g = (rng.standard_normal(n) * 1e-3).astype(f32)
    m = oracle.dequant_group(mc, ms, qm, n)
    v = oracle.dequant_group(vc, vs, qv, n)
    p2 = p.copy()
    oracle.adamw_fp32_step(p2, g, m, v, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], 3.0)
    want_mc, want_ms = oracle.quant_group(m, qm)
    want_vc, want_vs = oracle.quant_group(v, qv)
    oracle.adamw4bit_step(p, g, mc, vc, ms, vs, qm, qv, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], 3.0)
    assert np.array_equal(p, p2)
    assert np.array_equal(ms, want_ms) and np.array_equal(vs, want_vs)
    assert np.array_equal(mc, want_mc[:nb]) and np.array_equal(vc, want_vc[:nb])


def test_fused_state_stays_within_one_cell_of_fp32_adamw(oracle, qmaps):
    qm, qv = qmaps
    rng = np.random.default_rng(3)
    n = 128 * 16
    p = (rng.standard_normal(n) * 0.02).astype(f32)
    pf, mf, vf = p.copy(), np.zeros(n, f32), np.zeros(n, f32)
    mc, vc, ms, vs = np.zeros(n // 2, np.uint8), np.zeros(n // 2, np.uint8), np.zeros(16, f32), np.zeros(16, f32)
    for s in range(1, 4):
        g = (rng.standard_normal(n) * 1e-3).astype(f32)
        m_prev = oracle.dequant_group(mc, ms, qm, n)
        v_prev = oracle.dequant_group(vc, vs, qv, n)
        oracle.adamw4bit_step(p, g, mc, vc, ms, vs, qm, qv, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], float(s))
        m_new = f32(H["beta1"]) * m_prev + (1 - f32(H["beta1"])) * g
        v_new = f32(H["beta2"]) * v_prev + (1 - f32(H["beta2"])) * g * g
        # dequantised new state is within one cell (largest gap of the map x scale) of the exact EMA
        assert np.all(np.abs(oracle.dequant_group(mc, ms, qm, n) - m_new) <= 0.225 / 2 * ms.repeat(128) * 1.0001 + 1e-30)
        assert np.all(np.abs(oracle.dequant_group(vc, vs, qv, n) - v_new) <= 0.0625 * vs.repeat(128) * 1.0001 + 1e-30)


def test_golden_fused_fixture(oracle, qmaps):
    gold = np.load(os.path.join(HERE, "golden", "fused_step_small.npz"))
    qm, qv = qmaps
    n = gold["p0"].size
    p = gold["p0"].copy()
    mc, vc, ms, vs = np.zeros(n // 2, np.uint8), np.zeros(n // 2, np.uint8), np.zeros(8, f32), np.zeros(8, f32)
    for s in range(3):
        oracle.adamw4bit_step(p, gold["grads"][s].copy(), mc, vc, ms, vs, qm, qv, 0.9, 0.999, 1e-3, 0.01, 1e-8, float(s + 1))
        for name, arr in (("p", p), ("mc", mc), ("vc", vc), ("ms", ms), ("vs", vs)):
            assert np.array_equal(arr, gold[f"{name}{s + 1}"]), f"{name} step {s + 1}"
    # the zeroed gradient group of step 2 keeps a decayed, still representable state
    assert gold["ms2"][1] > 0


def test_quant_group_equals_numpy(oracle, qmaps):
    rng = np.random.default_rng(4)
    for q, x in ((qmaps[0], rng.standard_normal(5000).astype(f32)), (qmaps[1], (rng.standard_normal(5000) ** 2).astype(f32))):
        for gp in (128, 256, 2048):
            codes, max1 = oracle.quant_group(x, q, gp)
            g = (x.size + gp - 1) // gp
            pad = np.zeros(g * gp, f32)
            pad[: x.size] = x
            want_max = np.abs(pad).reshape(g, gp).max(1)
            assert np.array_equal(max1, want_max)
            ng = (g * gp + 2047) // 2048
            normed = np.zeros(ng * 2048, f32)
            normed[: g * gp] = (pad.reshape(g, gp) / want_max[:, None]).reshape(-1)
            assert np.array_equal(nibbles(codes, ng * 2048), oracle.qmapping(q, normed))
            assert codes.size == ng * 1024 + 1
            back = oracle.dequant_group(codes, max1, q, x.size, gp)
            assert np.array_equal(back, (q[nibbles(codes, x.size)] * want_max.repeat(gp)[: x.size]).astype(f32))
    # an all-zero group: 0/0 -> NaN -> code 15, scale 0, decodes to 0
    z = np.zeros(256, f32)
    z[128:] = 1.0
    codes, max1 = oracle.quant_group(z, qmaps[0])
    assert max1[0] == 0 and np.all(nibbles(codes, 128) == 15)
    assert np.all(oracle.dequant_group(codes, max1, qmaps[0], 256)[:128] == 0)


def test_rank1_equals_numpy_and_special_cases(oracle, qmaps):
    qv = qmaps[1]
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((37, 53)) ** 2).astype(f32)
    row, col = oracle.rank1_stats(x)
    assert np.array_equal(row, x.max(1)) and np.array_equal(col, x.max(0))
    st = np.minimum.outer(row, col)
    codes = oracle.quant_rank1(x, row, col, qv)
    ng = (x.size + 2047) // 2048
    normed = np.zeros(ng * 2048, f32)
    normed[: x.size] = (x / st).reshape(-1)
    assert np.array_equal(nibbles(codes, ng * 2048), oracle.qmapping(qv, normed))
    assert np.array_equal(oracle.dequant_rank1(codes, row, col, qv, 37, 53), (qv[nibbles(codes, x.size)].reshape(37, 53) * st).astype(f32))
    # a rank-one tensor |x| = r c^T with max(r) = max(c) = 1 has st = min(r_i, c_j) >= x_ij, and
    # x / st <= 1 with the row and column maxima hitting exactly 1
    r, c = rng.random(20).astype(f32), rng.random(30).astype(f32)
    r[3], c[7] = 1.0, 1.0
    y = np.outer(r, c).astype(f32)
    row, col = oracle.rank1_stats(y)
    assert np.array_equal(row, r) and np.array_equal(col, c)
    n = y / np.minimum.outer(row, col)
    assert n.max() == 1.0 and np.all(n <= 1.0) and np.all(n[3, :] <= 1) and n[3, 7] == 1.0
    assert nibbles(oracle.quant_rank1(y, row, col, qv), y.size).reshape(20, 30)[3, 7] == 15


def test_rank1_nd_reduces_to_2d_and_to_library_ops(oracle, qmaps):
    """The N-D restatement of rank-1 scaling: on a 2-D tensor it is the (pinned) 2-D C
    functions bit for bit; on 3-D and 4-D tensors its statistics and scale are what the
    reference's op sequence gives when PyTorch's CPU kernels run it (max over every other
    dimension with keepdim, then a chain of torch.min: lpmm/functional.py:503-531), and what a
    loop over all indices gives; a separable tensor a_i b_j c_k has the factors as statistics."""
    qv = qmaps[1]
    rng = np.random.default_rng(11)
    x2 = (rng.standard_normal((37, 53)) ** 2).astype(f32)
    x2[4, :] = 0.0
    stats = oracle.rank1_stats_nd(x2)
    row, col = oracle.rank1_stats(x2)
    assert np.array_equal(stats[0], row) and np.array_equal(stats[1], col)
    codes = oracle.quant_rank1_nd_bits(x2, stats, qv, 4)
    assert np.array_equal(codes, oracle.quant_rank1(x2, row, col, qv))
    assert np.array_equal(oracle.dequant_rank1_nd_bits(codes, stats, qv, 4, x2.shape),
                          oracle.dequant_rank1(codes, row, col, qv, 37, 53))
    for shape in [(3, 5, 7), (2, 3, 4, 5), (6, 1, 9)]:
        x = (rng.standard_normal(shape) ** 2).astype(f32)
        x[(0,) * len(shape)] = 0.0
        stats = oracle.rank1_stats_nd(x)
        scale = oracle.rank1_scale_nd(stats, shape)
        # the reference's op sequence on PyTorch CPU kernels
        t = torch.from_numpy(x).abs()
        max_dims = []
        for i in range(t.dim()):
            red = t
            for d in range(t.dim()):
                if d != i:
                    red = red.max(dim=d, keepdim=True).values
            max_dims.append(red)
        ts = max_dims[0].clone()
        for other in max_dims[1:]:
            ts = torch.min(ts, other)
        for st, md in zip(stats, max_dims):
            assert np.array_equal(st, md.numpy().reshape(-1))
        assert np.array_equal(scale, ts.numpy())
        # a loop over all indices
        want = [np.zeros(d, f32) for d in shape]
        for idx in np.ndindex(*shape):
            for i, j in enumerate(idx):
                want[i][j] = max(want[i][j], abs(x[idx]))
        for st, w in zip(stats, want):
            assert np.array_equal(st, w)
        for idx in np.ndindex(*shape):
            assert scale[idx] == min(want[i][j] for i, j in enumerate(idx))
        # codes: the map search on x / scale, zero padding to the pack group
        codes = oracle.quant_rank1_nd_bits(x, stats, qv, 4)
        normed = np.zeros(2048, f32)
        with np.errstate(invalid="ignore"):
            normed[: x.size] = (x / scale).reshape(-1)
        assert np.array_equal(nibbles(codes, 2048), oracle.qmapping(qv, normed))
        back = oracle.dequant_rank1_nd_bits(codes, stats, qv, 4, shape)
        assert np.array_equal(back, (qv[nibbles(codes, x.size)].reshape(shape) * scale).astype(f32))
    a, b, c = rng.random(6).astype(f32), rng.random(5).astype(f32), rng.random(4).astype(f32)
    a[2] = b[0] = c[3] = 1.0
    # powers of two keep the products exact
    a, b, c = (np.exp2(np.floor(np.log2(v))).astype(f32) for v in (a, b, c))
    y = (a[:, None, None] * b[None, :, None] * c[None, None, :]).astype(f32)
    stats = oracle.rank1_stats_nd(y)
    assert np.array_equal(stats[0], a) and np.array_equal(stats[1], b) and np.array_equal(stats[2], c)
    assert nibbles(oracle.quant_rank1_nd_bits(y, stats, qv, 4), y.size).reshape(y.shape)[2, 0, 3] == 15
    # a NaN: max and min of PyTorch's CPU kernels both hand it on, so every slice through it gets a NaN scale
    z = (rng.standard_normal((4, 3, 5)) ** 2).astype(f32)
    z[1, 2, 3] = np.nan
    stats = oracle.rank1_stats_nd(z)
    t = torch.from_numpy(z).abs()
    ts = None
    for i in range(3):
        red = t
        for d in range(3):
            if d != i:
                red = red.max(dim=d, keepdim=True).values
        assert np.array_equal(stats[i], red.numpy().reshape(-1), equal_nan=True)
        ts = red.clone() if ts is None else torch.min(ts, red)
    scale = oracle.rank1_scale_nd(stats, z.shape)
    assert np.array_equal(scale, ts.numpy(), equal_nan=True)
    assert np.isnan(scale).sum() == 4 * 3 * 5 - 3 * 2 * 4


def test_nonfused_c_update_follows_torch_cpu_ops(oracle, qmaps):
    """The C restatement of the non-fused step against the same op sequence run by PyTorch's
    CPU kernels (library ops), on a 2-D tensor, group-128 m and rank-1 v, 4 steps."""
    from oracle.nonfused_torch import TorchNonFusedAdamW

    qm, qv = qmaps
    torch.manual_seed(0)
    shape = (96, 160)
    p_t = torch.randn(shape) * 0.02
    p_c = p_t.numpy().copy()
    topt = TorchNonFusedAdamW([p_t], lr=H["lr"], betas=(H["beta1"], H["beta2"]), eps=H["eps"], weight_decay=H["wd"],
                              v_scale_type="rank1")
    state = oracle.NonFusedState(shape, v_scale_type="rank1")
    flips = 0
    for s in range(4):
        g = torch.randn(shape) * 1e-3
        p_before = p_c.copy()
        topt.step([g])
        m_c, v_c = oracle.nonfused_step(p_c, g.numpy(), state, qm, qv, H["lr"], H["beta1"], H["beta2"], H["eps"], H["wd"])
        ts = topt.state[0]
        assert_rel(p_c, p_t.numpy(), f"p step {s}", tol=1e-6, scale=p_before)
        assert_rel(m_c, ts["m_fp32"].numpy(), f"m step {s}", tol=1e-6)
        assert_rel(v_c, ts["v_fp32"].numpy(), f"v step {s}", tol=1e-6)
        # a last-bit difference of a PyTorch kernel may flip a code that sits on a rounding
        # boundary; with 15360 elements the tie budget rounds to zero, so count instead
        flips += int(np.sum(nibbles(state.m[0], p_c.size) != nibbles(ts["m"][0].numpy(), p_c.size)))
        flips += int(np.sum(nibbles(state.v[0], p_c.size) != nibbles(ts["v"][0].numpy(), p_c.size)))
        # resynchronise so that each step is compared on identical inputs
        state.m = (ts["m"][0].numpy().view(np.uint8).copy(), ts["m"][1].numpy().reshape(-1).copy())
        state.v = (ts["v"][0].numpy().view(np.uint8).copy(), ts["v"][1][0].numpy().reshape(-1).copy(),
                   ts["v"][1][1].numpy().reshape(-1).copy())
        p_c[...] = p_t.numpy()
    assert flips <= 2, flips


@pytest.mark.parametrize("nesterov", [False, True])
@pytest.mark.parametrize("maximize", [False, True])
@pytest.mark.parametrize("dampening, wd", [(0.0, 0.0), (0.1, 1e-4), (0.0, 0.05)])
def test_sgd_c_update_follows_torch_cpu_ops(oracle, nesterov, maximize, dampening, wd):
    """The elementwise part of the 4-bit SGD step against the reference's own op sequence
    (lpmm/optim/sgd.py:152-181) run by PyTorch's CPU kernels, bit for bit, over three steps
    (the first stores the decayed gradient itself): Tensor.add(alpha=) is one fused
    multiply-add with the float-cast scalar, mul_ one multiply.  Sizes cover the vectorised
    body of the library kernels and their scalar tails."""
    rng = np.random.default_rng(31)
    lr, mom = 0.05, 0.9
    for n in (1, 7, 64, 1000, 4099):
        p = rng.standard_normal(n).astype(f32)
        tp, tbuf, buf = torch.from_numpy(p.copy()), None, np.zeros(n, f32)
        for step in range(3):
            g = (rng.standard_normal(n) * 1e-2).astype(f32)
            tg = torch.from_numpy(g)
            d_p = tg if not maximize else -tg
            if wd != 0:
                d_p = d_p.add(tp, alpha=wd)
            if tbuf is None:
                tbuf = torch.clone(d_p).detach()
            else:
                tbuf.mul_(mom).add_(d_p, alpha=1 - dampening)
            d_p = d_p.add(tbuf, alpha=mom) if nesterov else tbuf
            tp.add_(d_p, alpha=-lr)
            oracle.sgd_update(p, g, buf, mom, dampening, lr, wd, nesterov, maximize, step == 0)
            assert np.array_equal(buf, tbuf.numpy()), (n, step)
            assert np.array_equal(p, tp.numpy()), (n, step)


def test_factored_closed_forms(oracle):
    rng = np.random.default_rng(7)
    r, c = 24, 40
    # for g^2 = a b^T (rank one) the factored estimate reproduces the EMA of g^2 exactly
    a, b = rng.random(r) + 0.5, rng.random(c) + 0.5
    g = np.sqrt(np.outer(a, b)).astype(f32)
    row, col = np.zeros(r, f32), np.zeros(c, f32)
    row_mean, col_mean = oracle.factored_stats(g)
    g2 = (g.astype(np.float64)) ** 2
    assert_rel(row_mean, g2.mean(1), "row mean", tol=2e-7)
    assert_rel(col_mean, g2.mean(0), "col mean", tol=2e-7)
    mean_all = oracle.factored_ema(row, col, row_mean, col_mean, H["beta2"])
    assert_rel(row, (1 - H["beta2"]) * g2.mean(1), "row EMA", tol=1e-6)
    assert_rel([mean_all], [row.astype(np.float64).mean()], "mean(row)", tol=2e-7)
    vhat = np.outer(row.astype(np.float64) / mean_all, col.astype(np.float64))
    assert_rel(vhat, (1 - H["beta2"]) * g2, "rank-one reconstruction", tol=5e-6)
    # one update step against the closed form in double
    p0 = (rng.standard_normal((r, c)) * 0.02).astype(f32)
    p, m = p0.copy(), np.zeros(r * c, f32)
    oracle.factored_update(p, g, m, row, col, mean_all, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], 1.0)
    m1 = (1 - H["beta1"]) * g.astype(np.float64)
    denom = np.sqrt(vhat) / np.sqrt(1 - H["beta2"]) + H["eps"]
    want = p0 * (1 - H["lr"] * H["wd"]) - H["lr"] / (1 - H["beta1"]) * m1 / denom
    assert_rel(p, want, "p", tol=1e-6, scale=p0)
    assert_rel(m, m1.reshape(-1), "m", tol=1e-6)


def test_factored_c_follows_torch_cpu_ops(oracle, qmaps):
    from oracle.nonfused_torch import TorchNonFusedAdamW

    torch.manual_seed(1)
    shape = (64, 96)
    p_t = torch.randn(shape) * 0.02
    p_c = p_t.numpy().copy()
    topt = TorchNonFusedAdamW([p_t], lr=H["lr"], betas=(H["beta1"], H["beta2"]), eps=H["eps"], weight_decay=H["wd"],
                              factor_second_moment=True)
    state = oracle.NonFusedState(shape, factored=True)
    for s in range(3):
        g = torch.randn(shape) * 1e-3
        p_before = p_c.copy()
        topt.step([g])
        oracle.nonfused_step(p_c, g.numpy(), state, qmaps[0], qmaps[1], H["lr"], H["beta1"], H["beta2"], H["eps"], H["wd"])
        ts = topt.state[0]
        assert_rel(state.row, ts["row"].numpy(), "row", tol=1e-6)
        assert_rel(state.col, ts["col"].numpy(), "col", tol=1e-6)
        assert_rel(p_c, p_t.numpy(), "p", tol=1e-6, scale=p_before)
        assert_codes(state.m[0], ts["m"][0].numpy(), p_c.size, "m codes") if p_c.size >= 10 ** 5 else None
        state.m = (ts["m"][0].numpy().view(np.uint8).copy(), ts["m"][1].numpy().reshape(-1).copy())
        state.row[...] = ts["row"].numpy()
        state.col[...] = ts["col"].numpy()
        p_c[...] = p_t.numpy()


@pytest.mark.parametrize("kind", ["group", "rank1", "factored"])
def test_golden_nonfused_fixture(oracle, qmaps, kind):
    """The committed non-fused fixture (tests/golden/nonfused_steps_small.npz) is what the oracle
    produces today: guards the oracle and the fixture against drifting apart."""
    gold = np.load(os.path.join(HERE, "golden", "nonfused_steps_small.npz"))
    p = gold["p0"].copy()
    st = oracle.NonFusedState(p.shape, v_scale_type="rank1" if kind == "rank1" else "group", factored=kind == "factored")
    for s in range(3):
        oracle.nonfused_step(p, gold["grads"][s], st, qmaps[0], qmaps[1], 1e-3, 0.9, 0.999, 1e-8, 0.01)
        k = f"{kind}{s + 1}"
        np.testing.assert_array_equal(st.m[0], gold[f"mc_{k}"])
        np.testing.assert_array_equal(st.m[1], gold[f"ms_{k}"])
        if kind == "factored":
            np.testing.assert_array_equal(st.row, gold[f"row_{k}"])
            np.testing.assert_array_equal(st.col, gold[f"col_{k}"])
        else:
            np.testing.assert_array_equal(st.v[0], gold[f"vc_{k}"])
            for j, a in enumerate(st.v[1:]):
                np.testing.assert_array_equal(a, gold[f"vs{j}_{k}"])
    np.testing.assert_array_equal(p, gold[f"p_{kind}3"])


def test_fp16_step_pinned_by_the_fp32_step(oracle):
    """The float16 restatement of adamw_cuda_kernel<at::Half> against the C restatement of the
    float kernel, where the two must agree: with beta1 = beta2 = 0.5 and dyadic moments and
    gradients the new moments are exactly representable in half, so rounding them changes
    nothing and the half step's parameter is the float step's parameter rounded to half once.
    A wrong rounding point, operand order or bias correction in the half restatement fails it."""
    rng = np.random.default_rng(0)
    n = 8192
    m = (rng.integers(-64, 64, n) / 64).astype(np.float16)
    g = (rng.integers(-32, 32, n) / 32).astype(np.float16)
    v = (rng.integers(1, 64, n) / 64).astype(np.float16)
    p = rng.standard_normal(n).astype(np.float16)
    for step in (1.0, 3.0, 40.0):
        p32, g32, m32, v32 = (a.astype(np.float32) for a in (p, g, m, v))
        oracle.adamw_fp32_step(p32, g32, m32, v32, 0.5, 0.5, 1e-2, 0.01, 1e-8, step)
        ph, mh, vh = p.copy(), m.copy(), v.copy()
        oracle.adamw_fp16_step(ph, g, mh, vh, 0.5, 0.5, 1e-2, 0.01, 1e-8, step)
        np.testing.assert_array_equal(mh.astype(np.float32), m32)
        np.testing.assert_array_equal(vh.astype(np.float32), v32)
        np.testing.assert_array_equal(ph, p32.astype(np.float16))
        assert np.any(ph != p)


def test_fp16_step_reads_the_rounded_moments(oracle):
    """With ordinary hyper-parameters the new moments are not representable in half.  They must
    equal the float step's moments rounded to half once, and the parameter must come from those
    rounded moments (lpmm/cpp_extension/fused_adamw_kernel.cu:66-73 reads exp_avg and exp_avg_sq
    back from memory): an update formed from the unrounded moments differs somewhere."""
    rng = np.random.default_rng(1)
    n = 4096
    p = (rng.standard_normal(n) * 0.02).astype(np.float16)
    g = (rng.standard_normal(n) * 1e-2).astype(np.float16)
    m = (rng.standard_normal(n) * 1e-2).astype(np.float16)
    v = (rng.standard_normal(n) ** 2 * 1e-4).astype(np.float16)
    ph, mh, vh = p.copy(), m.copy(), v.copy()
    oracle.adamw_fp16_step(ph, g, mh, vh, 0.9, 0.999, 1e-3, 0.01, 1e-8, 5.0)
    p32, g32, m32, v32 = (a.astype(np.float32) for a in (p, g, m, v))
    oracle.adamw_fp32_step(p32, g32, m32, v32, 0.9, 0.999, 1e-3, 0.01, 1e-8, 5.0)
    np.testing.assert_array_equal(mh, m32.astype(np.float16))
    np.testing.assert_array_equal(vh, v32.astype(np.float16))
    f = np.float32
    c1 = f(1) - f(0.9) ** f(5)
    c2s = np.sqrt(f(1) - f(0.999) ** f(5))

    def update(mm, vv):
        pf = p.astype(f)
        return (pf - f(1e-3) * (mm / ((np.sqrt(vv) / c2s + f(1e-8)) * c1) + f(0.01) * pf)).astype(np.float16)

    from_rounded = update(mh.astype(f), vh.astype(f))
    assert np.mean(from_rounded == ph) > 0.999  # the C library's powf and ** may differ in the last place
    assert np.any(update(m32, v32) != from_rounded)


def test_half_conversions_are_numpy_float16(oracle):
    """The oracle's binary16 <-> binary32 conversions against numpy.float16: every half, and floats at and next to
    every half, every midpoint between neighbouring halfs, the overflow threshold and random values."""
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    f = oracle.f16_to_f32(h)
    assert np.array_equal(f.view(np.uint32), h.astype(f32).view(np.uint32))
    rng = np.random.default_rng(0)
    fs = np.sort(f[np.isfinite(f)])
    mid = ((fs[:-1].astype(np.float64) + fs[1:].astype(np.float64)) / 2).astype(f32)
    up, down = f32(np.inf), f32(-np.inf)
    with np.errstate(invalid="ignore"):
        x = np.concatenate([
            rng.standard_normal(1 << 18).astype(f32) * np.exp(rng.standard_normal(1 << 18) * 6).astype(f32),
            f, np.nextafter(f, up), np.nextafter(f, down), mid, np.nextafter(mid, up), np.nextafter(mid, down),
            np.array([65519.99, 65520, 65520.01, 1e9, -1e9, np.inf, -np.inf, 0.0, -0.0, 2.0 ** -25, 2.0 ** -24], f32)])
    with np.errstate(over="ignore"):
        got, want = oracle.f32_to_f16(x), x.astype(np.float16)
    assert np.all((got.view(np.uint16) == want.view(np.uint16)) | (np.isnan(got) & np.isnan(want)))


@pytest.mark.parametrize("v_scale", ["rank1", "group"])
@pytest.mark.parametrize("eps", [1e-3, 1e-8])
def test_nonfused_half_step_is_the_torch_cpu_half_chain(oracle, qmaps, v_scale, eps):
    """nonfused_step_f16 (C update with a rounding to half after every op, numpy float16 scaling, the C search)
    against the reference's op sequence run by PyTorch's CPU half kernels: parameters, both moments, codes,
    scales and statistics bit for bit over four steps with shrinking gradients.  With eps = 1e-8 (the default,
    which float16 rounds to zero) elements whose second moment is zero divide by zero; both sides agree on the
    infinities and NaNs as well."""
    from oracle.nonfused_torch import TorchNonFusedAdamW

    qm, qv = qmaps
    torch.manual_seed(5)
    shapes = [(96, 160), (11008,), (33, 256), (5000,), (45, 100)]  # the last two end in a partial group
    hyper = dict(lr=1e-2, betas=(0.9, 0.999), eps=eps, weight_decay=0.01)
    host = [(torch.randn(s) * 0.5).half() for s in shapes]
    ref = TorchNonFusedAdamW([h.clone() for h in host], v_scale_type=v_scale, **hyper)
    ps = [h.numpy().copy() for h in host]
    states = [oracle.NonFusedState(s, v_scale) for s in shapes]

    def same(a, b):
        a, b = np.ascontiguousarray(a).reshape(-1), np.ascontiguousarray(b).reshape(-1)
        assert a.dtype == b.dtype == np.float16
        return np.all((a.view(np.uint16) == b.view(np.uint16)) | (np.isnan(a) & np.isnan(b)))

    for step in range(1, 5):
        grads = [(torch.randn(s) * 0.3 * 10.0 ** -step).half() for s in shapes]
        ref.step(grads)
        for i, s in enumerate(shapes):
            m, v = oracle.nonfused_step_f16(ps[i], grads[i].numpy(), states[i], qm, qv, hyper["lr"], 0.9, 0.999, eps, 0.01)
            rs = ref.state[i]
            assert same(ps[i], ref.params[i].numpy()), (step, s)
            assert same(m, rs["m_fp32"].numpy()) and same(v, rs["v_fp32"].numpy()), (step, s)
            assert np.array_equal(states[i].m[0], rs["m"][0].numpy()) and same(states[i].m[1], rs["m"][1].numpy())
            assert np.array_equal(states[i].v[0], rs["v"][0].numpy()), (step, s)
            if v_scale == "rank1" and len(s) == 2:
                assert same(states[i].v[1], rs["v"][1][0].numpy()) and same(states[i].v[2], rs["v"][1][1].numpy())
            else:
                assert same(states[i].v[1], rs["v"][1].numpy())
        if eps == 1e-3:
            assert all(np.isfinite(p).all() for p in ps)


def test_fused_half_step_reduces_to_the_float_step(oracle):
    """adamw4bit_step_f16 (the operator's at::Half instantiation) against the pinned float step.  With
    maps, scales, states and gradients on a coarse binary grid and betas of 0.5 and 0.75 every moment
    is exactly representable in half, so the roundings at the assignments change nothing: codes and
    scales equal the float step's, and the parameter is the float step's rounded to half once.  A wrong
    operand, bias correction, nibble or rounding point in the half restatement fails it."""
    rng = np.random.default_rng(41)
    qm = (np.arange(16) / 8 - 1).astype(f32)  # -1 ... 0.875, three fractional bits
    qv = ((np.arange(16) + 1) / 16).astype(f32)
    for n in (128 * 6, 128 * 3 + 70, 50):
        nb, ng = (n + 1) // 2, (n + 127) // 128
        mc = rng.integers(0, 256, nb, dtype=np.uint8)
        vc = rng.integers(0, 256, nb, dtype=np.uint8)
        ms, vs = np.full(ng, 0.25, f32), np.full(ng, 0.25, f32)
        p = (rng.integers(-512, 512, n) / 1024).astype(f32)
        g = (rng.integers(-16, 16, n) / 16).astype(f32)
        ph, gh = p.astype(np.float16), g.astype(np.float16)
        mch, vch, msh, vsh = mc.copy(), vc.copy(), ms.astype(np.float16), vs.astype(np.float16)
        hyper = (0.5, 0.75, 1e-2, 0.0625, 1e-3, 3.0)
        oracle.adamw4bit_step(p, g, mc, vc, ms, vs, qm, qv, *hyper)
        oracle.adamw4bit_step_f16(ph, gh, mch, vch, msh, vsh, qm, qv, *hyper)
        assert np.array_equal(mch, mc) and np.array_equal(vch, vc), n
        assert np.array_equal(msh.astype(f32), ms) and np.array_equal(vsh.astype(f32), vs), n
        assert np.array_equal(ph.view(np.uint16), p.astype(np.float16).view(np.uint16)), n


def test_fused_half_step_against_numpy_half_arithmetic(oracle, qmaps):
    """The same function on random states and gradients against numpy.float16 arithmetic, operation by
    operation as c10::Half defines it (Half * Half: float product rounded to half; float * Half, Half /
    float: float; assignment to T: one rounding): the map entries are rounded to half before the
    product, the normalised values are not rounded, elements past the end leave their nibble 0."""
    qm, qv = qmaps
    rng = np.random.default_rng(42)
    h16 = np.float16
    b1, b2, lr, wd, eps, step = f32(0.9), f32(0.999), f32(1e-3), f32(0.01), f32(1e-8), f32(2.0)
    for n in (128 * 5, 128 * 2 + 38):
        nb, ng = (n + 1) // 2, (n + 127) // 128
        mc, vc = rng.integers(0, 256, nb, dtype=np.uint8), rng.integers(0, 256, nb, dtype=np.uint8)
        ms = np.abs(rng.standard_normal(ng) * 1e-2).astype(h16)
        vs = np.abs(rng.standard_normal(ng) * 1e-3).astype(h16)
        p = (rng.standard_normal(n) * 0.1).astype(h16)
        g = (rng.standard_normal(n) * 0.05).astype(h16)
        # numpy restatement
        cm, cv = nibbles(mc, n), nibbles(vc, n)
        grp = np.arange(n) // 128
        m0 = (qm[cm].astype(h16) * ms[grp])  # half * half -> half
        v0 = (qv[cv].astype(h16) * vs[grp])
        gf = g.astype(f32)
        m = (b1 * m0.astype(f32) + (f32(1) - b1) * gf).astype(h16)
        v = (b2 * v0.astype(f32) + (f32(1) - b2) * gf * gf).astype(h16)
        c1 = f32(1) - f32(np.float32(b1) ** step)
        c2s = np.sqrt(f32(1) - f32(np.float32(b2) ** step), dtype=f32)
        denom = (np.sqrt(v.astype(f32)) / c2s + eps) * c1
        update = m.astype(f32) / denom + wd * p.astype(f32)
        want_p = (p.astype(f32) - lr * update).astype(h16)
        pad = np.zeros(ng * 128, f32)
        pad[:n] = np.abs(m.astype(f32))
        want_ms = pad.reshape(ng, 128).max(1)
        pad[:n] = v.astype(f32)
        want_vs = pad.reshape(ng, 128).max(1)
        with np.errstate(invalid="ignore", divide="ignore"):
            want_cm = oracle.qmapping(qm, m.astype(f32) / want_ms[grp])
            want_cv = oracle.qmapping(qv, v.astype(f32) / want_vs[grp])
        oracle.adamw4bit_step_f16(p, g, mc, vc, ms, vs, qm, qv, float(b1), float(b2), float(lr), float(wd), float(eps), float(step))
        assert np.array_equal(p.view(np.uint16), want_p.view(np.uint16)), n
        assert np.array_equal(ms.astype(f32), want_ms) and np.array_equal(vs.astype(f32), want_vs), n
        assert np.array_equal(nibbles(mc, n), want_cm) and np.array_equal(nibbles(vc, n), want_cv), n
        if n % 2:
            assert mc[-1] >> 4 == 0 and vc[-1] >> 4 == 0
