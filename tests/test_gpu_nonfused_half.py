"""GPU parity of the non-fused AdamW step on float16 parameters (4-bit states; second moment block-wise
in one pass, rank-1 in two) against the CPU oracle's float16 restatement of the reference's op chain
(oracle.nonfused_step_f16: every op in float with one rounding to half, half scales and statistics),
called through the C ABI on torch device memory.  Parameters, scales, statistics and the packed
buffers are compared bit for bit, the buffers in full (padding codes and the extra last byte
included); a NaN equals a NaN.  Last, the fused 4-bit operator's instantiation on half tensors against
the oracle's restatement of it."""
import numpy as np
import pytest
import torch

from util import to_dev, to_np

pytestmark = pytest.mark.gpu

f16 = np.float16


def _native():
    from lpmm import _native

    return _native


def _nbytes(n):
    return (n + 2047) // 2048 * 1024 + 1


def _same_halfs(got, want, what):
    got, want = np.ascontiguousarray(got).reshape(-1), np.ascontiguousarray(want).reshape(-1)
    assert got.dtype == want.dtype == f16, what
    ok = (got.view(np.uint16) == want.view(np.uint16)) | (np.isnan(got) & np.isnan(want))
    assert ok.all(), (what, int((~ok).sum()), got[~ok][:5], want[~ok][:5])


def _dev_halfs(a, offset=0):
    buf = torch.empty(a.size + offset, dtype=torch.float16, device="cuda")
    view = buf[offset:]
    view.copy_(torch.from_numpy(np.ascontiguousarray(a).reshape(-1)))
    return view


def _codes(n, zero_byte):
    c = np.full(_nbytes(n), 0xA5, np.uint8)  # a pattern the kernels have to overwrite
    c[: (n + 1) // 2] = zero_byte
    return to_dev(c)


class _Flat:
    """A tensor of n halfs, both moments block-wise over 128 values."""

    def __init__(self, oracle, n, rng, offset=0):
        self.n, self.offset = n, offset
        self.host_p = (rng.standard_normal(n) * 0.5).astype(f16)
        self.state = oracle.NonFusedState((n,), "group")
        self.p = _dev_halfs(self.host_p, offset)
        self.mc, self.vc = _codes(n, 0x77), _codes(n, 0x00)
        groups = (n + 127) // 128
        self.ms = torch.zeros(groups, dtype=torch.float16, device="cuda")
        self.vs = torch.zeros(groups, dtype=torch.float16, device="cuda")
        self.g = None

    def record(self, g, step):
        self.g = _dev_halfs(g, self.offset)
        return (self.p.data_ptr(), self.g.data_ptr(), self.mc.data_ptr(), self.vc.data_ptr(), self.ms.data_ptr(),
                self.vs.data_ptr(), self.n, float(step), 0.0)

    def check(self, what):
        st = self.state
        _same_halfs(to_np(self.ms), st.m[1], f"{what}: m max1")
        _same_halfs(to_np(self.vs), st.v[1], f"{what}: v max1")
        np.testing.assert_array_equal(to_np(self.mc), st.m[0], err_msg=f"{what}: m codes")
        np.testing.assert_array_equal(to_np(self.vc), st.v[0], err_msg=f"{what}: v codes")
        _same_halfs(to_np(self.p), self.host_p, f"{what}: p")


@pytest.mark.parametrize("eps", [1e-3, 1e-8])
def test_one_pass_half_step(oracle, qmaps, eps):
    """Whole tiles, a ragged end, fewer values than a group, pointers that allow no 8-byte accesses;
    four steps with shrinking gradients, so that second moments underflow to zero in half.  With the
    default eps (zero as a half) such elements divide by zero: the infinities and NaNs are compared too."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(21)
    hyper = dict(lr=1e-2, beta1=0.9, beta2=0.999, wd=0.01)
    tensors = [_Flat(oracle, 2048 * 3, rng), _Flat(oracle, 5000, rng), _Flat(oracle, 100, rng),
               _Flat(oracle, 11008, rng, offset=1), _Flat(oracle, 2048 * 2 + 128, rng, offset=3)]
    for step in range(1, 5):
        grads = [(rng.standard_normal(t.n) * 0.3 * 10.0 ** -step).astype(f16) for t in tensors]
        grads[0][128:384] = 0  # two groups that never see a gradient: scale 0, 0 / 0 -> the NaN code throughout
        grads[1][4992:] = 0    # ... and the partial last group of a ragged tensor
        records = [t.record(g, step) for t, g in zip(tensors, grads)]
        table = np.array(records, dtype=nat.ADAMW4BIT_TENSOR)
        st = lib.lpmm_nonfused_adamw4bit_f16_step_multi(table.ctypes.data, len(records), dqm.data_ptr(), dqv.data_ptr(),
                                                        hyper["beta1"], hyper["beta2"], hyper["lr"], hyper["wd"], eps,
                                                        nat.current_stream(torch.device("cuda:0")))
        assert st == 0
        torch.cuda.synchronize()
        for i, (t, g) in enumerate(zip(tensors, grads)):
            oracle.nonfused_step_f16(t.host_p, g, t.state, qm, qv, hyper["lr"], hyper["beta1"], hyper["beta2"], eps,
                                     hyper["wd"])
            t.check(f"step {step} tensor {i} (n = {t.n})")
    if eps == 1e-3:
        assert all(np.isfinite(t.host_p).all() for t in tensors)
    else:
        assert any(not np.isfinite(t.host_p).all() for t in tensors)
    st = tensors[0].state
    assert st.m[1][1] == 0 and st.v[1][2] == 0 and np.all(st.m[0][64:192] == 0xFF) and np.all(st.v[0][64:192] == 0xFF)


class _Matrix:
    """A matrix of halfs: first moment block-wise, second moment rank-1."""

    def __init__(self, oracle, rows, cols, rng):
        self.rows, self.cols, self.n = rows, cols, rows * cols
        self.host_p = (rng.standard_normal((rows, cols)) * 0.5).astype(f16)
        self.state = oracle.NonFusedState((rows, cols), "rank1")
        self.p = _dev_halfs(self.host_p)
        self.mc, self.vc = _codes(self.n, 0x77), _codes(self.n, 0x00)
        self.ms = torch.zeros(self.n // 128, dtype=torch.float16, device="cuda")
        self.stats = [torch.zeros(rows, dtype=torch.float16, device="cuda"),
                      torch.zeros(cols, dtype=torch.float16, device="cuda")]
        self.next = [torch.full((rows,), 7.0, dtype=torch.float16, device="cuda"),
                     torch.full((cols,), 7.0, dtype=torch.float16, device="cuda")]
        self.work = torch.full(((rows + 3) // 4 * 4 + cols,), 3.0, dtype=torch.float32, device="cuda")
        self.g = None

    def record(self, g, step):
        self.g = _dev_halfs(g)
        return (self.p.data_ptr(), self.g.data_ptr(), self.mc.data_ptr(), self.ms.data_ptr(), self.vc.data_ptr(),
                self.stats[0].data_ptr(), self.stats[1].data_ptr(), self.next[0].data_ptr(), self.next[1].data_ptr(),
                self.work.data_ptr(), self.rows, self.cols, float(step), 0.0)

    def launched(self):
        self.stats, self.next = self.next, self.stats

    def check(self, what):
        st = self.state
        _same_halfs(to_np(self.ms), st.m[1], f"{what}: m max1")
        np.testing.assert_array_equal(to_np(self.mc), st.m[0], err_msg=f"{what}: m codes")
        _same_halfs(to_np(self.stats[0]), st.v[1], f"{what}: row statistics")
        _same_halfs(to_np(self.stats[1]), st.v[2], f"{what}: column statistics")
        np.testing.assert_array_equal(to_np(self.vc), st.v[0], err_msg=f"{what}: v codes")
        _same_halfs(to_np(self.p), self.host_p, f"{what}: p")


@pytest.mark.parametrize("eps", [1e-3, 1e-8])
def test_two_pass_half_step(oracle, qmaps, eps):
    """Matrices with one column block, with more blocks than a tile is wide, with fewer rows than a
    tile, with a row count that is no multiple of the rows of a pass; 34 tensors (two launch groups),
    four steps with shrinking gradients, a row and a column of zero gradients."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(22)
    hyper = dict(lr=1e-2, beta1=0.9, beta2=0.999, wd=0.01)
    shapes = [(96, 256), (33, 128), (200, 384), (64, 1024), (7, 640), (130, 128)] + [(20, 128)] * 28
    tensors = [_Matrix(oracle, r, c, rng) for r, c in shapes]
    for step in range(1, 5):
        grads = [(rng.standard_normal((t.rows, t.cols)) * 0.3 * 10.0 ** -step).astype(f16) for t in tensors]
        grads[0][5, :] = 0
        grads[0][:, 9] = 0
        records = [t.record(g, step) for t, g in zip(tensors, grads)]
        table = np.array(records, dtype=nat.NONFUSED_RANK1_F16_TENSOR)
        st = lib.lpmm_nonfused_adamw4bit_rank1_f16_step_multi(
            table.ctypes.data, len(records), dqm.data_ptr(), dqv.data_ptr(), hyper["beta1"], hyper["beta2"],
            hyper["lr"], hyper["wd"], eps, nat.current_stream(torch.device("cuda:0")))
        assert st == 0
        torch.cuda.synchronize()
        for i, (t, g) in enumerate(zip(tensors, grads)):
            t.launched()
            oracle.nonfused_step_f16(t.host_p, g, t.state, qm, qv, hyper["lr"], hyper["beta1"], hyper["beta2"], eps,
                                     hyper["wd"])
            if i < 8 or step == 4:
                t.check(f"step {step} tensor {i} {t.rows} x {t.cols}")


def test_half_steps_reject_bad_arguments(qmaps):
    nat = _native()
    lib = nat.lib()
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    s = nat.current_stream(torch.device("cuda:0"))
    h = (0.9, 0.999, 1e-3, 0.01, 1e-8)
    p = torch.zeros(256, dtype=torch.float16, device="cuda")
    codes = torch.zeros(1025, dtype=torch.uint8, device="cuda")
    sc = torch.zeros(2, dtype=torch.float16, device="cuda")
    ok = (p.data_ptr(), p.data_ptr(), codes.data_ptr(), codes.data_ptr(), sc.data_ptr(), sc.data_ptr(), 256, 1.0, 0.0)

    def flat(rec, count=1, qm=dqm.data_ptr()):
        table = np.array([rec], dtype=nat.ADAMW4BIT_TENSOR)
        return lib.lpmm_nonfused_adamw4bit_f16_step_multi(table.ctypes.data, count, qm, dqv.data_ptr(), *h, s)

    assert flat(ok, count=0) == 0
    assert flat(ok, count=-1) == 3
    assert flat(ok, qm=None) == 1
    assert flat((0,) + ok[1:]) == 1
    assert flat(ok[:6] + (-1,) + ok[7:]) == 3
    assert flat((p.data_ptr() + 1,) + ok[1:]) == 2
    assert flat(ok[:6] + (0,) + ok[7:]) == 0  # an empty tensor is skipped

    stats = [torch.zeros(2, dtype=torch.float16, device="cuda") for _ in range(2)]
    cs = [torch.zeros(128, dtype=torch.float16, device="cuda") for _ in range(2)]
    work = torch.zeros(4 + 128, dtype=torch.float32, device="cuda")
    okr = (p.data_ptr(), p.data_ptr(), codes.data_ptr(), sc.data_ptr(), codes.data_ptr(), stats[0].data_ptr(),
           cs[0].data_ptr(), stats[1].data_ptr(), cs[1].data_ptr(), work.data_ptr(), 2, 128, 1.0, 0.0)

    def matrix(rec, count=1):
        table = np.array([rec], dtype=nat.NONFUSED_RANK1_F16_TENSOR)
        return lib.lpmm_nonfused_adamw4bit_rank1_f16_step_multi(table.ctypes.data, count, dqm.data_ptr(), dqv.data_ptr(),
                                                                *h, s)

    assert matrix(okr, count=0) == 0
    assert matrix(okr[:11] + (64,) + okr[12:]) == 3  # the column count must be a multiple of 128
    assert matrix(okr[:9] + (0,) + okr[10:]) == 1  # no work array
    assert matrix(okr[:9] + (work.data_ptr() + 4,) + okr[10:]) == 2
    assert matrix(okr[:7] + (stats[0].data_ptr(),) + okr[8:]) == 5  # the next statistics alias the current ones
    assert matrix((0,) + okr[1:]) == 1
    torch.cuda.synchronize()


@pytest.mark.parametrize("n", [2048 * 3, 128 * 21 + 38, 100, 2])
def test_fused_operator_on_half_tensors(oracle, qmaps, n):
    """The reference-named operator on float16 p, g and scales (the at::Half instantiation of the fused
    4-bit kernel, lpmm/cpp_extension/fused_adamw_kernel.cu:80-174, :222-230) against the oracle's
    restatement of that instantiation: codes, half scales and parameters bit for bit over three steps;
    whole tiles, a group that the end of the tensor cuts, fewer values than a group, one byte."""
    from lpmm.cpp_extension import fused_adamw

    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(51 + n)
    nb, ng = n // 2, (n + 127) // 128
    hp = (rng.standard_normal(n) * 0.1).astype(f16)
    hmc, hvc = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8)
    hms, hvs = np.zeros(ng, f16), np.zeros(ng, f16)
    p = to_dev(hp.copy())
    mc, vc = to_dev(hmc.copy()), to_dev(hvc.copy())
    ms, vs = to_dev(hms.copy()), to_dev(hvs.copy())
    guard = to_dev(np.full(64, 0x5A, np.uint8))  # a small allocation made right after the codes: must stay as it is
    hyper = (0.9, 0.999, 1e-3, 0.01, 1e-8)
    for step in range(1, 4):
        hg = (rng.standard_normal(n) * 0.05).astype(f16)
        g = to_dev(hg)
        fused_adamw.adamw4bit_single_tensor(p, g, mc, vc, ms, vs, dqm, dqv, *hyper, float(step))
        torch.cuda.synchronize()
        oracle.adamw4bit_step_f16(hp, hg, hmc, hvc, hms, hvs, qm, qv, *hyper, float(step))
        what = f"n = {n}, step {step}"
        np.testing.assert_array_equal(to_np(mc), hmc, err_msg=what + ": m codes")
        np.testing.assert_array_equal(to_np(vc), hvc, err_msg=what + ": v codes")
        _same_halfs(to_np(ms), hms, what + ": m scales")
        _same_halfs(to_np(vs), hvs, what + ": v scales")
        _same_halfs(to_np(p), hp, what + ": p")
    assert np.all(to_np(guard) == 0x5A)
    # types: the gradient and the scales share the parameter's type, the maps stay float32
    with pytest.raises(RuntimeError, match="expected scalar type"):
        fused_adamw.adamw4bit_single_tensor(p, g.float(), mc, vc, ms, vs, dqm, dqv, *hyper, 4.0)
    with pytest.raises(RuntimeError, match="expected scalar type"):
        fused_adamw.adamw4bit_single_tensor(p, g, mc, vc, ms.float(), vs, dqm, dqv, *hyper, 4.0)
    with pytest.raises(RuntimeError, match="float32 is required"):
        fused_adamw.adamw4bit_single_tensor(p, g, mc, vc, ms, vs, dqm.half(), dqv, *hyper, 4.0)


@pytest.mark.parametrize("eps", [1e-3, 1e-8])
def test_one_pass_half_step_on_every_gradient_value(oracle, qmaps, eps):
    """Every float16 gradient of magnitude up to 256 (subnormals and both zeros included; beyond that the
    second moment overflows in half), in shuffled order, on states that three ordinary steps have filled:
    parameters, codes and scales bit for bit.  The sweep takes the square root, the two divisions and the
    encoders of the kernel through 46 octaves of second moments, down to the ones that underflow to zero."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(61)
    mags = np.arange(0, 0x5C01, dtype=np.uint16)  # 0 ... 256.0
    sweep = np.concatenate([mags, mags | 0x8000]).view(f16)
    reps = 3
    t = _Flat(oracle, sweep.size * reps, rng)
    hyper = dict(lr=1e-2, beta1=0.9, beta2=0.999, wd=0.01)
    for step in range(1, 6):
        if step <= 3:
            g = (rng.standard_normal(t.n) * 0.3).astype(f16)
        else:
            g = np.concatenate([rng.permutation(sweep) for _ in range(reps)])
        table = np.array([t.record(g, step)], dtype=nat.ADAMW4BIT_TENSOR)
        st = lib.lpmm_nonfused_adamw4bit_f16_step_multi(table.ctypes.data, 1, dqm.data_ptr(), dqv.data_ptr(),
                                                        hyper["beta1"], hyper["beta2"], hyper["lr"], hyper["wd"], eps,
                                                        nat.current_stream(torch.device("cuda:0")))
        assert st == 0
        torch.cuda.synchronize()
        oracle.nonfused_step_f16(t.host_p, g, t.state, qm, qv, hyper["lr"], hyper["beta1"], hyper["beta2"], eps,
                                 hyper["wd"])
        t.check(f"step {step}")
    assert np.isfinite(t.state.v[1].astype(np.float32)).all() and float(t.state.v[1].max()) > 50.0


def test_fused_operator_on_every_half_gradient_value(oracle, qmaps):
    """The same sweep through the fused operator's half instantiation (float eps: no division by zero)."""
    from lpmm.cpp_extension import fused_adamw

    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(62)
    mags = np.arange(0, 0x5C01, dtype=np.uint16)
    sweep = np.concatenate([mags, mags | 0x8000]).view(f16)
    n = sweep.size * 2
    nb, ng = n // 2, (n + 127) // 128
    hp = (rng.standard_normal(n) * 0.1).astype(f16)
    hmc, hvc, hms, hvs = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8), np.zeros(ng, f16), np.zeros(ng, f16)
    p, mc, vc, ms, vs = (to_dev(a.copy()) for a in (hp, hmc, hvc, hms, hvs))
    hyper = (0.9, 0.999, 1e-3, 0.01, 1e-8)
    for step in range(1, 5):
        hg = (rng.standard_normal(n) * 0.05).astype(f16) if step <= 2 else np.concatenate([rng.permutation(sweep) for _ in range(2)])
        fused_adamw.adamw4bit_single_tensor(p, to_dev(hg), mc, vc, ms, vs, dqm, dqv, *hyper, float(step))
        torch.cuda.synchronize()
        oracle.adamw4bit_step_f16(hp, hg, hmc, hvc, hms, hvs, qm, qv, *hyper, float(step))
        np.testing.assert_array_equal(to_np(mc), hmc, err_msg=f"step {step}: m codes")
        np.testing.assert_array_equal(to_np(vc), hvc, err_msg=f"step {step}: v codes")
        _same_halfs(to_np(ms), hms, f"step {step}: m scales")
        _same_halfs(to_np(vs), hvs, f"step {step}: v scales")
        _same_halfs(to_np(p), hp, f"step {step}: p")
