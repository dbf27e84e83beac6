"""GPU parity of the non-fused AdamW step with an fp32 first moment and a 4-bit second moment
(the configurations that quantise the second moment only) against the CPU oracle's separate
stages -- dequantise v, the update on fp32 arrays, (statistics,) quantise v -- called through
the C ABI on torch device memory.  First moment, scales, statistics and the packed buffers are
compared bit for bit, the buffers in full (padding codes and the extra last byte included)."""
import numpy as np
import pytest
import torch

from util import assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

H = dict(beta1=0.9, beta2=0.999, lr=1e-3, wd=0.01, eps=1e-8)


def _native():
    from lpmm import _native

    return _native


def _nbytes(n):
    return (n + 2047) // 2048 * 1024 + 1


def _check_p(t, what):
    got = to_np(t.p).reshape(-1)
    want = t.host_p.reshape(-1)
    assert_rel(got, want, f"{what}: p", scale=want)
    # sqrt and the divisions of the update are near-exact: a stray last-bit difference at most
    bad = int(np.sum(got != want))
    assert bad <= max(1, t.n // 100000), (what, bad)
    t.p.copy_(torch.from_numpy(t.host_p))


class _Flat:
    """A tensor of n elements with a block-wise scaled second moment."""

    def __init__(self, n, rng, offset=0):
        self.n, self.offset = n, offset
        self.host_p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        self.host_m = np.zeros(n, np.float32)
        self.ref_v = None  # (codes, max1)
        self.p = self._dev(self.host_p)
        self.m = self._dev(self.host_m)
        vc = np.full(_nbytes(n), 0xA5, np.uint8)  # a pattern the kernel has to overwrite
        vc[: (n + 1) // 2] = 0
        self.vc = to_dev(vc)
        self.vs = to_dev(np.zeros((n + 127) // 128, np.float32))
        self.g = None

    def _dev(self, a):
        buf = torch.empty(a.size + self.offset, dtype=torch.float32, device="cuda")
        view = buf[self.offset:]
        view.copy_(torch.from_numpy(a))
        return view

    def record(self, g, step):
        self.g = self._dev(g)
        return (self.p.data_ptr(), self.g.data_ptr(), self.m.data_ptr(), self.vc.data_ptr(), self.vs.data_ptr(),
                self.n, float(step), 0.0)

    def oracle_step(self, oracle, g, qv, step):
        n = self.n
        v = np.zeros(n, np.float32) if self.ref_v is None else oracle.dequant_group(*self.ref_v, qv, n)
        oracle.nonfused_update(self.host_p, g, self.host_m, v, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"],
                               float(step))
        self.ref_v = oracle.quant_group(v, qv)

    def check(self, what):
        np.testing.assert_array_equal(to_np(self.m), self.host_m, err_msg=f"{what}: m")
        np.testing.assert_array_equal(to_np(self.vs), self.ref_v[1], err_msg=f"{what}: v max1")
        np.testing.assert_array_equal(to_np(self.vc), self.ref_v[0], err_msg=f"{what}: v codes")
        _check_p(self, what)


def _step_flat(oracle, tensors, grads, qv, dqv, step):
    nat = _native()
    lib = nat.lib()
    table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.ADAMW_V4BIT_TENSOR)
    st = lib.lpmm_nonfused_adamw_v4bit_step_multi(table.ctypes.data, len(tensors), dqv.data_ptr(), H["beta1"],
                                                  H["beta2"], H["lr"], H["wd"], H["eps"],
                                                  torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.lpmm_status_string(st)
    for t, g in zip(tensors, grads):
        t.oracle_step(oracle, g, qv, step)
    torch.cuda.synchronize()


def _flat_grad(rng, n):
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    if n > 300:
        g[rng.integers(0, n, 3)] *= 50.0
        g[128:256] = 0.0  # a group whose second moment stays zero: scale 0, 0/0 -> code 15
    return g


@pytest.mark.parametrize("offset", [0, 1])
def test_group_step_matches_staged_oracle(oracle, qmaps, offset):
    qv = qmaps[1]
    dqv = to_dev(qv)
    rng = np.random.default_rng(51 + offset)
    # below one group, odd, one over a group / a tile, whole tiles, large
    sizes = [1, 2, 127, 129, 2047, 2048, 2049, 4097, 128 * 37, 2048 * 5, 100003, 4096 * 300 + 64]
    tensors = [_Flat(n, rng, offset=offset) for n in sizes]
    for step in range(1, 5):
        grads = [_flat_grad(rng, t.n) for t in tensors]
        _step_flat(oracle, tensors, grads, qv, dqv, step)
        for t in tensors:
            t.check(f"n={t.n} offset={offset} step {step}")


def test_group_step_more_tensors_than_one_launch_with_their_own_step_counts(oracle, qmaps):
    qv = qmaps[1]
    dqv = to_dev(qv)
    rng = np.random.default_rng(52)
    tensors = [_Flat(int(n), rng) for n in rng.integers(1, 9000, size=110)]
    nat = _native()
    for rnd in range(3):
        steps = [rnd + 1 + (i % 4) * 10 for i in range(len(tensors))]
        grads = [_flat_grad(rng, t.n) for t in tensors]
        table = np.array([t.record(g, s) for t, g, s in zip(tensors, grads, steps)], dtype=nat.ADAMW_V4BIT_TENSOR)
        st = nat.lib().lpmm_nonfused_adamw_v4bit_step_multi(table.ctypes.data, len(tensors), dqv.data_ptr(),
                                                            H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"],
                                                            torch.cuda.current_stream().cuda_stream)
        nat.check(st, "lpmm_nonfused_adamw_v4bit_step_multi")
        torch.cuda.synchronize()
        for i, (t, g, s) in enumerate(zip(tensors, grads, steps)):
            t.oracle_step(oracle, g, qv, s)
            t.check(f"tensor {i} n={t.n} round {rnd}")


def test_group_step_full_size(oracle, qmaps):
    """4096 x 11008 (the largest LLaMA-7B MLP shape) for two steps."""
    qv = qmaps[1]
    dqv = to_dev(qv)
    rng = np.random.default_rng(53)
    t = _Flat(4096 * 11008, rng)
    for step in (1, 2):
        g = _flat_grad(rng, t.n)
        _step_flat(oracle, [t], [g], qv, dqv, step)
        t.check(f"step {step}")


class _Matrix:
    """A rows x cols tensor with a rank-1 scaled second moment."""

    def __init__(self, rows, cols, rng):
        self.rows, self.cols, self.n = rows, cols, rows * cols
        self.host_p = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
        self.host_m = np.zeros(self.n, np.float32)
        self.ref_v = None  # (codes, rowmax, colmax)
        self.p = to_dev(self.host_p)
        self.m = to_dev(self.host_m)
        vc = np.full(_nbytes(self.n), 0xA5, np.uint8)
        vc[: self.n // 2] = 0
        self.vc = to_dev(vc)
        self.stats = [to_dev(np.zeros(rows, np.float32)), to_dev(np.zeros(cols, np.float32))]
        self.spare = [to_dev(np.full(rows, 7.0, np.float32)), to_dev(np.full(cols, 7.0, np.float32))]
        self.g = None

    def record(self, g, step):
        self.g = to_dev(g)
        cur, nxt = self.stats, self.spare
        self.stats, self.spare = nxt, cur
        return (self.p.data_ptr(), self.g.data_ptr(), self.m.data_ptr(), self.vc.data_ptr(), cur[0].data_ptr(),
                cur[1].data_ptr(), nxt[0].data_ptr(), nxt[1].data_ptr(), self.rows, self.cols, float(step), 0.0)

    def oracle_step(self, oracle, g, qv, step):
        n, r, c = self.n, self.rows, self.cols
        v = np.zeros(n, np.float32) if self.ref_v is None else oracle.dequant_rank1(*self.ref_v, qv, r, c).reshape(-1)
        oracle.nonfused_update(self.host_p.reshape(-1), g.reshape(-1), self.host_m, v, H["beta1"], H["beta2"],
                               H["lr"], H["wd"], H["eps"], float(step))
        v2 = v.reshape(r, c)
        rowmax, colmax = oracle.rank1_stats(v2)
        self.ref_v = (oracle.quant_rank1(v2, rowmax, colmax, qv), rowmax, colmax)

    def check(self, what):
        np.testing.assert_array_equal(to_np(self.stats[0]), self.ref_v[1], err_msg=f"{what}: v row statistics")
        np.testing.assert_array_equal(to_np(self.stats[1]), self.ref_v[2], err_msg=f"{what}: v column statistics")
        np.testing.assert_array_equal(to_np(self.m), self.host_m, err_msg=f"{what}: m")
        np.testing.assert_array_equal(to_np(self.vc), self.ref_v[0], err_msg=f"{what}: v codes")
        _check_p(self, what)


def _step_matrices(oracle, tensors, grads, qv, dqv, step):
    nat = _native()
    lib = nat.lib()
    table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.RANK1_V4BIT_TENSOR)
    st = lib.lpmm_nonfused_adamw_v4bit_rank1_step_multi(table.ctypes.data, len(tensors), dqv.data_ptr(), H["beta1"],
                                                        H["beta2"], H["lr"], H["wd"], H["eps"],
                                                        torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.lpmm_status_string(st)
    for t, g in zip(tensors, grads):
        t.oracle_step(oracle, g, qv, step)
    torch.cuda.synchronize()


def _matrix_grad(rng, t):
    # row and column structure, so that both statistics matter for the scale
    g = rng.standard_normal((t.rows, t.cols)) * 1e-3
    g *= np.exp(rng.standard_normal((t.rows, 1))) * np.exp(rng.standard_normal((1, t.cols)))
    return g.astype(np.float32)


def test_rank1_step_matches_staged_oracle(oracle, qmaps):
    qv = qmaps[1]
    dqv = to_dev(qv)
    rng = np.random.default_rng(54)
    # fewer rows than one pass / one tile, ragged row counts, several column blocks, whole tiles,
    # more row blocks than interleave in one group
    shapes = [(1, 128), (3, 128), (16, 256), (65, 384), (100, 1280), (513, 1024), (2048, 640), (67, 4224),
              (2500, 4096)]
    tensors = [_Matrix(r, c, rng) for r, c in shapes]
    for step in range(1, 4):
        grads = [_matrix_grad(rng, t) for t in tensors]
        _step_matrices(oracle, tensors, grads, qv, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_rank1_step_more_tensors_than_one_launch(oracle, qmaps):
    qv = qmaps[1]
    dqv = to_dev(qv)
    rng = np.random.default_rng(55)
    tensors = [_Matrix(int(r), 128 * int(cb), rng) for r, cb in zip(rng.integers(1, 200, 40), rng.integers(1, 5, 40))]
    for step in (1, 2):
        grads = [_matrix_grad(rng, t) for t in tensors]
        _step_matrices(oracle, tensors, grads, qv, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_argument_checks(qmaps):
    nat = _native()
    lib = nat.lib()
    dqv = to_dev(qmaps[1])
    stream = torch.cuda.current_stream().cuda_stream
    f5 = (H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"])
    p = torch.zeros(256, device="cuda")
    vc = torch.zeros(_nbytes(256), dtype=torch.uint8, device="cuda")
    vs = torch.zeros(2, device="cuda")
    ok = (p.data_ptr(), p.data_ptr(), p.data_ptr(), vc.data_ptr(), vs.data_ptr(), 256, 1.0, 0.0)

    def flat(records, count=None, qmap=dqv.data_ptr()):
        table = np.array(records, dtype=nat.ADAMW_V4BIT_TENSOR)
        return lib.lpmm_nonfused_adamw_v4bit_step_multi(table.ctypes.data, len(records) if count is None else count,
                                                        qmap, *f5, stream)

    assert flat([ok], count=0) == 0
    assert flat([ok], count=-1) != 0
    assert flat([ok], qmap=0) != 0
    assert flat([ok[:2] + (0,) + ok[3:]]) != 0  # no first moment
    assert flat([ok[:3] + (vc.data_ptr() + 1,) + ok[4:]]) != 0  # codes not 2-byte aligned
    assert flat([ok[:5] + (-5, 1.0, 0.0)]) != 0
    assert flat([ok[:5] + (0, 1.0, 0.0)]) == 0  # an empty tensor is skipped

    row = [torch.zeros(2, device="cuda") for _ in range(2)]
    col = [torch.zeros(128, device="cuda") for _ in range(2)]
    okm = (p.data_ptr(), p.data_ptr(), p.data_ptr(), vc.data_ptr(), row[0].data_ptr(), col[0].data_ptr(),
           row[1].data_ptr(), col[1].data_ptr(), 2, 128, 1.0, 0.0)

    def matrix(records):
        table = np.array(records, dtype=nat.RANK1_V4BIT_TENSOR)
        return lib.lpmm_nonfused_adamw_v4bit_rank1_step_multi(table.ctypes.data, len(records), dqv.data_ptr(), *f5,
                                                              stream)

    assert matrix([okm[:2] + (0,) + okm[3:]]) != 0  # no first moment
    assert matrix([okm[:2] + (p.data_ptr() + 4,) + okm[3:]]) != 0  # first moment not 16-byte aligned
    assert matrix([okm[:9] + (100, 1.0, 0.0)]) != 0  # columns not a multiple of 128
    assert matrix([okm[:6] + (row[0].data_ptr(),) + okm[7:]]) != 0  # the statistics alias
    assert matrix([okm[:8] + (0, 128, 1.0, 0.0)]) == 0  # an empty tensor is skipped
    torch.cuda.synchronize()


@pytest.mark.parametrize("config", ["2nd_moment_only_group_128.yml", "2nd_moment_only_default.yml"])
def test_optimizer_with_second_moment_only_configurations(oracle, qmaps, config):
    """lpmm.optim.AdamW(fused=False) under the shipped configurations that quantise the second
    moment only: tensors the kernels above take, tensors that stay on the staged path (a ragged
    2-D tensor and a 1-D tensor under rank-1 scaling) and a small tensor with fp32 states all
    equal the oracle; the first moment is an fp32 state tensor throughout."""
    import os

    import lpmm

    qv = qmaps[1]
    rng = np.random.default_rng(56)
    rank1 = config == "2nd_moment_only_default.yml"
    shapes = [(96, 256), (130, 70), (5000,), (2000,)]
    holders = []
    for s in shapes:
        as_matrix = rank1 and len(s) == 2
        holders.append(_Matrix(s[0], s[1], rng) if as_matrix else _Flat(int(np.prod(s)), rng))
    params = [torch.nn.Parameter(to_dev(h.host_p.reshape(s))) for h, s in zip(holders, shapes)]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", config)
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, lr=H["lr"], betas=(H["beta1"], H["beta2"]),
                           eps=H["eps"], weight_decay=H["wd"])
    v_small = np.zeros(2000, np.float32)
    for step in range(1, 4):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for h, g in zip(holders[:3], grads[:3]):
            h.oracle_step(oracle, g if isinstance(h, _Matrix) else g.reshape(-1), qv, step)
        small = holders[3]
        oracle.nonfused_update(small.host_p, grads[3], small.host_m, v_small, H["beta1"], H["beta2"], H["lr"],
                               H["wd"], H["eps"], float(step))
        for i, (h, p) in enumerate(zip(holders, params)):
            st = opt.state[p]
            what = f"{config} tensor {i} step {step}"
            assert st["exp_avg"].dtype == torch.float32 and st["exp_avg"].shape == p.shape, what
            np.testing.assert_array_equal(to_np(st["exp_avg"]).reshape(-1), h.host_m, err_msg=f"{what}: m")
            assert_rel(to_np(p).reshape(-1), h.host_p.reshape(-1), f"{what}: p", scale=h.host_p.reshape(-1))
            if i == 3:
                np.testing.assert_array_equal(to_np(st["exp_avg_sq"]), v_small, err_msg=f"{what}: v")
                continue
            assert st["exp_avg_sq"].dtype == torch.int8
            np.testing.assert_array_equal(to_np(st["exp_avg_sq"]).view(np.uint8), h.ref_v[0], err_msg=f"{what}: v codes")
            oh = st["exp_avg_sq_qstate"]["overhead"]
            if isinstance(h, _Matrix):
                np.testing.assert_array_equal(to_np(oh["max_dims"][0]).reshape(-1), h.ref_v[1], err_msg=what)
                np.testing.assert_array_equal(to_np(oh["max_dims"][1]).reshape(-1), h.ref_v[2], err_msg=what)
            else:
                np.testing.assert_array_equal(to_np(oh["max1"]).reshape(-1), h.ref_v[1], err_msg=what)
            # the device parameter goes on from the oracle's value: a stray last-bit difference
            # of the update must not grow into a different code later
            with torch.no_grad():
                p.copy_(torch.from_numpy(h.host_p.reshape(p.shape)))
