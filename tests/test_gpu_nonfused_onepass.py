"""GPU parity of the one-pass non-fused 4-bit AdamW step (dequantise -> update -> re-quantise
of both moments, block-wise scaling over 128 values) against the CPU oracle's three separate
stages, called through the C ABI on torch device memory.  The packed buffers are compared
in full: padding codes and the extra last byte included."""
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


def _oracle_step(oracle, p, g, st, qm, qv, step):
    """st = [m_codes, m_max1, v_codes, v_max1] (None before the first step); p updated in place."""
    n = p.size
    m = np.zeros(n, np.float32) if st[0] is None else oracle.dequant_group(st[0], st[1], qm, n)
    v = np.zeros(n, np.float32) if st[2] is None else oracle.dequant_group(st[2], st[3], qv, n)
    oracle.nonfused_update(p, g, m, v, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], float(step))
    st[0], st[1] = oracle.quant_group(m, qm)
    st[2], st[3] = oracle.quant_group(v, qv)


class _Tensor:
    def __init__(self, n, rng, zero_byte_m=0x77, offset=0):
        self.n = n
        self.host_p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        self.ref = [None, None, None, None]
        self.offset = offset
        self.p = self._dev(self.host_p)
        ng = (n + 127) // 128
        # the state before the first step: zero scales, codes of 0.0; the rest of the buffer
        # is filled with a pattern the kernel has to overwrite
        self.mc = self._dev(np.full(_nbytes(n), 0xA5, np.uint8))
        self.vc = self._dev(np.full(_nbytes(n), 0xA5, np.uint8))
        self.mc[: (n + 1) // 2] = zero_byte_m
        self.vc[: (n + 1) // 2] = 0
        self.ms = self._dev(np.zeros(ng, np.float32))
        self.vs = self._dev(np.zeros(ng, np.float32))
        self.g = None

    def _dev(self, a):
        buf = torch.empty(a.size + self.offset, dtype=torch.from_numpy(a).dtype, device="cuda")
        view = buf[self.offset:]
        view.copy_(torch.from_numpy(a))
        return view

    def record(self, g, step):
        self.g = self._dev(g)
        return (self.p.data_ptr(), self.g.data_ptr(), self.mc.data_ptr(), self.vc.data_ptr(), self.ms.data_ptr(),
                self.vs.data_ptr(), self.n, float(step), 0.0)

    def check(self, what):
        np.testing.assert_array_equal(to_np(self.mc), self.ref[0], err_msg=f"{what}: m codes")
        np.testing.assert_array_equal(to_np(self.vc), self.ref[2], err_msg=f"{what}: v codes")
        np.testing.assert_array_equal(to_np(self.ms), self.ref[1], err_msg=f"{what}: m max1")
        np.testing.assert_array_equal(to_np(self.vs), self.ref[3], err_msg=f"{what}: v max1")
        got = to_np(self.p)
        assert_rel(got, self.host_p, f"{what}: p", scale=self.host_p)
        # sqrt and the divisions of the update are near-exact: a stray last-bit difference at most
        bad = int(np.sum(got != self.host_p))
        assert bad <= max(1, self.n // 100000), (what, bad)
        self.p.copy_(torch.from_numpy(self.host_p))


def _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step):
    nat = _native()
    lib = nat.lib()
    table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.ADAMW4BIT_TENSOR)
    st = lib.lpmm_nonfused_adamw4bit_step_multi(table.ctypes.data, len(tensors), dqm.data_ptr(), dqv.data_ptr(),
                                                H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"],
                                                torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.lpmm_status_string(st)
    for t, g in zip(tensors, grads):
        _oracle_step(oracle, t.host_p, g, t.ref, qm, qv, step)
    torch.cuda.synchronize()


@pytest.mark.parametrize("offset", [0, 1])
def test_onepass_matches_three_stage_oracle(oracle, qmaps, offset):
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(11 + offset)
    # ragged sizes: below one group, odd, one over a group / a tile, whole tiles, large
    sizes = [1, 2, 127, 129, 2047, 2048, 2049, 4097, 128 * 37, 2048 * 5, 100003, 4096 * 300 + 64]
    tensors = [_Tensor(n, rng, offset=offset) for n in sizes]
    for step in range(1, 5):
        grads = [(rng.standard_normal(t.n) * 1e-3).astype(np.float32) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"n={t.n} step {step}")


def test_onepass_more_tensors_than_one_launch(oracle, qmaps):
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(12)
    tensors = [_Tensor(int(n), rng) for n in rng.integers(1, 9000, size=60)]
    for step in (1, 2):
        grads = [(rng.standard_normal(t.n) * 1e-3).astype(np.float32) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"n={t.n} step {step}")


def test_onepass_zero_groups_and_outliers(oracle, qmaps):
    """All-zero groups quantise to code 15 with scale 0 (0/0 in the reference's division),
    also inside a partial last group; single large entries stretch a group's scale."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(13)
    n = 128 * 21 + 37
    t = _Tensor(n, rng)
    for step in range(1, 4):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        g[128 * 3:128 * 5] = 0.0
        g[128 * 21:] = 0.0  # the partial last group
        g[128 * 7 + 5] = 30.0
        g[128 * 9 + 100] = -1e-12
        _step_all(oracle, [t], [g], qm, qv, dqm, dqv, step)
        t.check(f"step {step}")
    assert np.all(t.ref[1][3:5] == 0.0) and t.ref[0][128 * 3 // 2] == 0xFF


@pytest.mark.parametrize("which", ["linear", "shifted"])
def test_onepass_other_maps(oracle, which):
    """Maps other than the two standard ones take the search fallback; the padding holds the
    code of 0.0 under the map in use."""
    if which == "linear":
        qm = oracle.create_pow_map(4, True, 1)  # a signed linear map
    else:
        qm = np.linspace(-0.2, 1.0, 16).astype(np.float32)  # the code of 0.0 is not 7
    qv = (oracle.qmap_v() ** 2).astype(np.float32)
    assert qm.size == 16 and qv.size == 16
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(14)
    zero_code = int(np.sum((qm[:-1] + qm[1:]) * np.float32(0.5) < 0))
    tensors = [_Tensor(n, rng, zero_byte_m=zero_code | (zero_code << 4)) for n in (300, 5000, 2048 * 3)]
    for step in range(1, 4):
        grads = [(rng.standard_normal(t.n) * 1e-3).astype(np.float32) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"n={t.n} step {step}")


def test_onepass_argument_checks(qmaps):
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.lpmm_nonfused_adamw4bit_step_multi(None, 0, dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999, 1e-3, 0.0,
                                                  1e-8, s) == 0
    assert lib.lpmm_nonfused_adamw4bit_step_multi(None, 1, dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999, 1e-3, 0.0,
                                                  1e-8, s) != 0
    assert lib.lpmm_nonfused_adamw4bit_step_multi(None, -1, dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999, 1e-3, 0.0,
                                                  1e-8, s) != 0
    rec = np.array([(0, 0, 0, 0, 0, 0, 100, 1.0, 0.0)], dtype=nat.ADAMW4BIT_TENSOR)
    assert lib.lpmm_nonfused_adamw4bit_step_multi(rec.ctypes.data, 1, dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999,
                                                  1e-3, 0.0, 1e-8, s) != 0
