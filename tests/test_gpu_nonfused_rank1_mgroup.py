"""GPU parity of the two-pass non-fused 4-bit AdamW step with first-moment groups of 256 .. 4096
values and a rank-1 second moment (lpmm/configs/1st_moment_group_*.yml) against the CPU oracle's
separate stages (dequantise, update, statistics, quantise), called through the C ABI on torch
device memory.  Codes (in full, padding included), scales and statistics bit for bit."""
import os

import numpy as np
import pytest
import torch

from util import assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

H = dict(beta1=0.9, beta2=0.999, lr=1e-3, wd=0.01, eps=1e-8)
GROUP_SIZES = [256, 512, 1024, 2048, 4096]


def _native():
    from lpmm import _native

    return _native


def _nbytes(n, gp):
    padded = (n + gp - 1) // gp * gp
    return (padded + 2047) // 2048 * 1024 + 1


class _Tensor:
    def __init__(self, rows, cols, gp, rng):
        self.rows, self.cols, self.n, self.gp = rows, cols, rows * cols, gp
        self.host_p = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
        self.ref_m = None  # (codes, max1)
        self.ref_v = None  # (codes, rowmax, colmax)
        self.p = to_dev(self.host_p)
        groups = (self.n + gp - 1) // gp
        # before the first step: zero scales and statistics, codes of 0.0; padding and the spare
        # buffers hold a pattern the kernels have to overwrite
        mc = np.full(_nbytes(self.n, gp), 0xA5, np.uint8)
        vc = np.full(_nbytes(self.n, 128), 0xA5, np.uint8)
        mc[: self.n // 2] = 0x77
        vc[: self.n // 2] = 0x00
        self.mc, self.vc = to_dev(mc), to_dev(vc)
        self.scales = to_dev(np.zeros(groups, np.float32))
        self.spare_scales = to_dev(np.full(groups, 7.0, np.float32))
        self.stats = [to_dev(np.zeros(rows, np.float32)), to_dev(np.zeros(cols, np.float32))]
        self.spare = [to_dev(np.full(rows, 7.0, np.float32)), to_dev(np.full(cols, 7.0, np.float32))]
        self.g = None

    def record(self, g, step):
        self.g = to_dev(g)
        cur, nxt = self.stats, self.spare
        self.stats, self.spare = nxt, cur
        ms, ms_next = self.scales, self.spare_scales
        self.scales, self.spare_scales = ms_next, ms
        return (self.p.data_ptr(), self.g.data_ptr(), self.mc.data_ptr(), ms.data_ptr(), ms_next.data_ptr(),
                self.vc.data_ptr(), cur[0].data_ptr(), cur[1].data_ptr(), nxt[0].data_ptr(), nxt[1].data_ptr(),
                self.rows, self.cols, float(step), 0.0)

    def oracle_step(self, oracle, g, qm, qv, step):
        n, r, c = self.n, self.rows, self.cols
        m = np.zeros(n, np.float32) if self.ref_m is None else oracle.dequant_group(*self.ref_m, qm, n, self.gp)
        v = np.zeros(n, np.float32) if self.ref_v is None else oracle.dequant_rank1(*self.ref_v, qv, r, c).reshape(-1)
        oracle.nonfused_update(self.host_p.reshape(-1), g.reshape(-1), m, v, H["beta1"], H["beta2"], H["lr"],
                               H["wd"], H["eps"], float(step))
        self.ref_m = oracle.quant_group(m, qm, self.gp)
        v2 = v.reshape(r, c)
        rowmax, colmax = oracle.rank1_stats(v2)
        self.ref_v = (oracle.quant_rank1(v2, rowmax, colmax, qv), rowmax, colmax)

    def check(self, what):
        np.testing.assert_array_equal(to_np(self.stats[0]), self.ref_v[1], err_msg=f"{what}: v row statistics")
        np.testing.assert_array_equal(to_np(self.stats[1]), self.ref_v[2], err_msg=f"{what}: v column statistics")
        np.testing.assert_array_equal(to_np(self.scales), self.ref_m[1], err_msg=f"{what}: m max1")
        got = to_np(self.mc)
        assert got.size == self.ref_m[0].size, what
        np.testing.assert_array_equal(got, self.ref_m[0], err_msg=f"{what}: m codes")
        np.testing.assert_array_equal(to_np(self.vc), self.ref_v[0], err_msg=f"{what}: v codes")
        got = to_np(self.p)
        assert_rel(got, self.host_p, f"{what}: p", scale=self.host_p)
        bad = int(np.sum(got != self.host_p))
        assert bad <= max(1, self.n // 100000), (what, bad)
        self.p.copy_(torch.from_numpy(self.host_p))


def _step_all(oracle, tensors, grads, gp, qm, qv, dqm, dqv, step):
    nat = _native()
    lib = nat.lib()
    table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.RANK1_MGROUP_TENSOR)
    st = lib.lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi(table.ctypes.data, len(tensors), dqm.data_ptr(),
                                                             dqv.data_ptr(), gp, H["beta1"], H["beta2"], H["lr"],
                                                             H["wd"], H["eps"], torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.lpmm_status_string(st)
    for t, g in zip(tensors, grads):
        t.oracle_step(oracle, g, qm, qv, step)
    torch.cuda.synchronize()


def _grad(rng, t, zero_rows=0):
    # row and column structure, so that both statistics matter for the scale
    g = rng.standard_normal((t.rows, t.cols)) * 1e-3
    g *= np.exp(rng.standard_normal((t.rows, 1))) * np.exp(rng.standard_normal((1, t.cols)))
    g = g.astype(np.float32)
    if zero_rows:
        g[-zero_rows:] = 0.0
    return g


@pytest.mark.parametrize("gp", GROUP_SIZES)
def test_mgroup_two_pass_matches_staged_oracle(oracle, qmaps, gp):
    """Tensors smaller than one group, with a cut last group (its padding takes the group's
    scale), with columns that are no multiple of the group size (groups span rows), with more
    row blocks than interleave, and with more than one pass per tile."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(61)
    shapes = [(1, 128), (3, 128), (16, 256), (65, 384), (100, 1280), (513, 1024), (67, 4224), (2500, 640),
              (33, 8192)]
    tensors = [_Tensor(r, c, gp, rng) for r, c in shapes]
    for step in range(1, 4):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, gp, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"group {gp}, {t.rows}x{t.cols} step {step}")


@pytest.mark.parametrize("gp", [256, 4096])
def test_mgroup_all_zero_groups(oracle, qmaps, gp):
    """Rows whose gradient stays zero: their first-moment groups have scale 0 and 0/0 gives
    code 15, in the cut last group for its padding as well."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(62)
    tensors = [_Tensor(r, c, gp, rng) for r, c in [(40, 384), (70, 128), (9, 4224)]]
    zero_rows = [34, 66, 3]
    for step in (1, 2):
        grads = [_grad(rng, t, z) for t, z in zip(tensors, zero_rows)]
        _step_all(oracle, tensors, grads, gp, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"group {gp}, {t.rows}x{t.cols} step {step}")


@pytest.mark.parametrize("gp", [128, 512, 4096])
def test_ragged_columns_match_staged_oracle(oracle, qmaps, gp):
    """Column counts that are no multiple of 128 (multiples of 8): the first moment's groups
    straddle rows, the last 128-column block of a row is cut, and the end of the tensor cuts a
    group (its padding takes the group's scale).  With whole tiles, ragged row counts, fewer
    columns than one block, and a tensor that is a multiple of 128 columns in the same call."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(66)
    shapes = [(5, 136), (7, 72), (1, 8), (40, 1600), (130, 200), (300, 1000), (64, 4800), (2500, 328), (33, 256),
              (513, 1096)]
    tensors = [_Tensor(r, c, gp, rng) for r, c in shapes]
    for step in range(1, 4):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, gp, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"group {gp}, {t.rows}x{t.cols} step {step}")


def test_ragged_columns_all_zero_groups(oracle, qmaps):
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(67)
    tensors = [_Tensor(r, c, 128, rng) for r, c in [(40, 200), (70, 72), (9, 1608)]]
    zero_rows = [34, 66, 3]
    for step in (1, 2):
        grads = [_grad(rng, t, z) for t, z in zip(tensors, zero_rows)]
        _step_all(oracle, tensors, grads, 128, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_ragged_columns_optimizer_with_the_default_configuration(oracle, qmaps):
    """lpmm.optim.AdamW(fused=False, qconfig=default.yml) on GPT-2-XL-like shapes (d = 1600): the
    two-pass kernels for ragged rows; states in the reference's layout, equal to the oracle."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(68)
    shapes = [(48, 1600), (1600, 200), (10, 4800)]
    holders = [_Tensor(r, c, 128, rng) for r, c in shapes]
    params = [torch.nn.Parameter(to_dev(h.host_p)) for h in holders]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "default.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, lr=H["lr"], betas=(H["beta1"], H["beta2"]),
                           eps=H["eps"], weight_decay=H["wd"])
    for step in range(1, 4):
        grads = [_grad(rng, h) for h in holders]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for i, (h, p, g) in enumerate(zip(holders, params, grads)):
            h.oracle_step(oracle, g, qm, qv, step)
            st = opt.state[p]
            what = f"tensor {i} step {step}"
            oh = st["exp_avg_qstate"]["overhead"]
            assert tuple(oh["max1"].shape) == ((h.n + 127) // 128, 1), what
            np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), h.ref_m[0], err_msg=f"{what}: m codes")
            np.testing.assert_array_equal(to_np(oh["max1"]).reshape(-1), h.ref_m[1], err_msg=f"{what}: m max1")
            ov = st["exp_avg_sq_qstate"]["overhead"]
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), h.ref_v[0], err_msg=f"{what}: v codes")
            np.testing.assert_array_equal(to_np(ov["max_dims"][0]).reshape(-1), h.ref_v[1], err_msg=what)
            np.testing.assert_array_equal(to_np(ov["max_dims"][1]).reshape(-1), h.ref_v[2], err_msg=what)
            assert_rel(to_np(p), h.host_p, f"{what}: p", scale=h.host_p)
            with torch.no_grad():
                p.copy_(torch.from_numpy(h.host_p))


def test_mgroup_more_tensors_than_one_launch(oracle, qmaps):
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(63)
    tensors = [_Tensor(int(r), 128 * int(cb), 512, rng)
               for r, cb in zip(rng.integers(1, 200, 40), rng.integers(1, 6, 40))]
    for step in (1, 2):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, 512, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_mgroup_full_size(oracle, qmaps):
    """4096 x 11008 (11008 is no multiple of 512: every other group spans two rows)."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(64)
    t = _Tensor(4096, 11008, 512, rng)
    for step in (1, 2):
        g = (rng.standard_normal((t.rows, t.cols)) * 1e-3).astype(np.float32)
        _step_all(oracle, [t], [g], 512, qm, qv, dqm, dqv, step)
        t.check(f"step {step}")


def test_mgroup_optimizer(oracle, qmaps):
    """lpmm.optim.AdamW(fused=False, qconfig=1st_moment_group_512.yml): 2-D tensors take the
    kernels above, a ragged one stays on the staged path; both equal the oracle and their
    states have the reference's layout and metadata."""
    import lpmm

    qm, qv = qmaps
    rng = np.random.default_rng(65)
    shapes = [(96, 256), (130, 70), (33, 1152)]
    holders = [_Tensor(r, c, 512, rng) for r, c in shapes]
    params = [torch.nn.Parameter(to_dev(h.host_p)) for h in holders]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", "1st_moment_group_512.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, lr=H["lr"], betas=(H["beta1"], H["beta2"]),
                           eps=H["eps"], weight_decay=H["wd"])
    for step in range(1, 4):
        grads = [_grad(rng, h) for h in holders]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for i, (h, p, g) in enumerate(zip(holders, params, grads)):
            h.oracle_step(oracle, g, qm, qv, step)
            st = opt.state[p]
            what = f"tensor {i} step {step}"
            groups = (h.n + 511) // 512
            oh = st["exp_avg_qstate"]["overhead"]
            assert st["exp_avg"].dtype == torch.int8 and tuple(oh["max1"].shape) == (groups, 1), what
            assert tuple(oh["scaled_shape"]) == (groups, 512), what
            np.testing.assert_array_equal(to_np(st["exp_avg"]).view(np.uint8), h.ref_m[0], err_msg=f"{what}: m codes")
            np.testing.assert_array_equal(to_np(oh["max1"]).reshape(-1), h.ref_m[1], err_msg=f"{what}: m max1")
            ov = st["exp_avg_sq_qstate"]["overhead"]
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), h.ref_v[0], err_msg=f"{what}: v codes")
            np.testing.assert_array_equal(to_np(ov["max_dims"][0]).reshape(-1), h.ref_v[1], err_msg=what)
            np.testing.assert_array_equal(to_np(ov["max_dims"][1]).reshape(-1), h.ref_v[2], err_msg=what)
            assert_rel(to_np(p), h.host_p, f"{what}: p", scale=h.host_p)
            with torch.no_grad():
                p.copy_(torch.from_numpy(h.host_p))


def test_mgroup_argument_checks(qmaps):
    nat = _native()
    lib = nat.lib()
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    stream = torch.cuda.current_stream().cuda_stream
    f5 = (H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"])
    p = torch.zeros(256, device="cuda")
    mc = torch.zeros(_nbytes(256, 256), dtype=torch.uint8, device="cuda")
    vc = torch.zeros(_nbytes(256, 128), dtype=torch.uint8, device="cuda")
    ms = [torch.zeros(1, device="cuda") for _ in range(2)]
    row = [torch.zeros(2, device="cuda") for _ in range(2)]
    col = [torch.zeros(128, device="cuda") for _ in range(2)]
    ok = (p.data_ptr(), p.data_ptr(), mc.data_ptr(), ms[0].data_ptr(), ms[1].data_ptr(), vc.data_ptr(),
          row[0].data_ptr(), col[0].data_ptr(), row[1].data_ptr(), col[1].data_ptr(), 2, 128, 1.0, 0.0)

    def call(records, gp=256):
        table = np.array(records, dtype=nat.RANK1_MGROUP_TENSOR)
        return lib.lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi(table.ctypes.data, len(records), dqm.data_ptr(),
                                                                   dqv.data_ptr(), gp, *f5, stream)

    for gp in (0, 64, 300, 384, 8192):
        assert call([ok], gp) != 0, gp  # 128 .. 4096 in powers of two only
    assert call([ok[:4] + (0,) + ok[5:]]) != 0  # no buffer for the next scales
    assert call([ok[:4] + (ms[0].data_ptr(),) + ok[5:]]) != 0  # the scales alias
    assert call([ok[:11] + (100, 1.0, 0.0)]) != 0  # columns not a multiple of 8
    assert call([ok[:10] + (0, 128, 1.0, 0.0)]) == 0  # an empty tensor is skipped
    torch.cuda.synchronize()
