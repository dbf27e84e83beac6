"""GPU parity of the two-pass non-fused AdamW step with 5- to 8-bit states (one code per byte;
first moment block-wise over 128 values, second moment rank-1: lpmm/configs/default_{5,6,7,8}b.yml)
against the CPU oracle's separate stages (dequantise, update, statistics, quantise), called
through the C ABI on torch device memory.  Codes (in full, padding included), scales and
statistics bit for bit."""
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
    return (n + 2047) // 2048 * 2048 + 1


def _maps(oracle, bits):
    """The maps the optimizer builds for these widths (lpmm/optim/optimizer.py:156-163)."""
    return oracle.create_dynamic_map(True, bits - 1, bits), oracle.create_pow_map(bits, False, 1)


class _Tensor:
    def __init__(self, rows, cols, bits, rng):
        self.rows, self.cols, self.n, self.bits = rows, cols, rows * cols, bits
        self.host_p = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
        self.ref_m = None  # (codes, max1)
        self.ref_v = None  # (codes, rowmax, colmax)
        self.p = to_dev(self.host_p)
        # before the first step: zero scales and statistics, under which any code decodes to
        # zero; the buffers hold a pattern the kernels have to overwrite
        self.mc = to_dev(np.full(_nbytes(self.n), 0xA5, np.uint8))
        self.vc = to_dev(np.full(_nbytes(self.n), 0xA5, np.uint8))
        self.ms = to_dev(np.zeros(self.n // 128, np.float32))
        self.stats = [to_dev(np.zeros(rows, np.float32)), to_dev(np.zeros(cols, np.float32))]
        self.spare = [to_dev(np.full(rows, 7.0, np.float32)), to_dev(np.full(cols, 7.0, np.float32))]
        self.g = None

    def record(self, g, step):
        self.g = to_dev(g)
        cur, nxt = self.stats, self.spare
        self.stats, self.spare = nxt, cur
        return (self.p.data_ptr(), self.g.data_ptr(), self.mc.data_ptr(), self.ms.data_ptr(), self.vc.data_ptr(),
                cur[0].data_ptr(), cur[1].data_ptr(), nxt[0].data_ptr(), nxt[1].data_ptr(), self.rows, self.cols,
                float(step), 0.0)

    def oracle_step(self, oracle, g, qm, qv, step):
        n, r, c, b = self.n, self.rows, self.cols, self.bits
        m = np.zeros(n, np.float32) if self.ref_m is None else oracle.dequant_group_bits(*self.ref_m, qm, b, n)
        v = (np.zeros(n, np.float32) if self.ref_v is None
             else np.ascontiguousarray(oracle.dequant_rank1_bits(*self.ref_v, qv, b, r, c)).reshape(-1))
        oracle.nonfused_update(self.host_p.reshape(-1), g.reshape(-1), m, v, H["beta1"], H["beta2"], H["lr"],
                               H["wd"], H["eps"], float(step))
        self.ref_m = oracle.quant_group_bits(m, qm, b)
        v2 = v.reshape(r, c)
        rowmax, colmax = oracle.rank1_stats(v2)
        self.ref_v = (oracle.quant_rank1_bits(v2, rowmax, colmax, qv, b), rowmax, colmax)

    def check(self, what):
        np.testing.assert_array_equal(to_np(self.stats[0]), self.ref_v[1], err_msg=f"{what}: v row statistics")
        np.testing.assert_array_equal(to_np(self.stats[1]), self.ref_v[2], err_msg=f"{what}: v column statistics")
        np.testing.assert_array_equal(to_np(self.ms), self.ref_m[1], err_msg=f"{what}: m max1")
        got = to_np(self.mc)
        assert got.size == self.ref_m[0].size, what
        np.testing.assert_array_equal(got, self.ref_m[0], err_msg=f"{what}: m codes")
        np.testing.assert_array_equal(to_np(self.vc), self.ref_v[0], err_msg=f"{what}: v codes")
        got = to_np(self.p)
        assert_rel(got, self.host_p, f"{what}: p", scale=self.host_p)
        bad = int(np.sum(got != self.host_p))
        assert bad <= max(1, self.n // 100000), (what, bad)
        self.p.copy_(torch.from_numpy(self.host_p))


def _code_table(dq, bits):
    nat = _native()
    table = torch.empty(nat.CODE_TABLE_BYTES // 4, dtype=torch.int32, device="cuda")
    assert nat.lib().lpmm_code_table_build(dq.data_ptr(), bits, table.data_ptr(),
                                           torch.cuda.current_stream().cuda_stream) == 0
    return table


def _step_all(oracle, tensors, grads, bits, qm, qv, dqm, dqv, step, with_tables=False):
    """with_tables: the code tables of the two maps (one table read per value instead of the search;
    the dynamic-exponent map of the first moment qualifies, the second moment's evenly spaced map
    takes its closed form either way)."""
    nat = _native()
    lib = nat.lib()
    table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.NONFUSED_RANK1_TENSOR)
    stream = torch.cuda.current_stream().cuda_stream
    if with_tables:
        tm, tv = _code_table(dqm, bits), _code_table(dqv, bits)
        assert int(tm[-1]) == (bits << 8 | 2) and int(tv[-1]) == (bits << 8 | 1)
        st = lib.lpmm_nonfused_adamw_bits_rank1_step_multi_table(
            table.ctypes.data, len(tensors), dqm.data_ptr(), bits, tm.data_ptr(), dqv.data_ptr(), bits, tv.data_ptr(),
            H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], stream)
    else:
        st = lib.lpmm_nonfused_adamw_bits_rank1_step_multi(table.ctypes.data, len(tensors), dqm.data_ptr(), bits,
                                                           dqv.data_ptr(), bits, H["beta1"], H["beta2"], H["lr"],
                                                           H["wd"], H["eps"], stream)
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


@pytest.mark.parametrize("with_tables", [False, True])
@pytest.mark.parametrize("bits", [5, 6, 7, 8])
def test_bits_two_pass_matches_staged_oracle(oracle, bits, with_tables):
    qm, qv = _maps(oracle, bits)
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(70 + bits)
    # fewer rows than one pass / one tile, ragged row counts, several column blocks, whole tiles,
    # more row blocks than interleave in one group
    shapes = [(1, 128), (3, 128), (16, 256), (65, 384), (100, 1280), (513, 1024), (67, 4224), (2500, 640)]
    tensors = [_Tensor(r, c, bits, rng) for r, c in shapes]
    for step in range(1, 4):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, bits, qm, qv, dqm, dqv, step, with_tables)
        for t in tensors:
            t.check(f"{bits} bits, {t.rows}x{t.cols} step {step}")


@pytest.mark.parametrize("with_tables", [False, True])
@pytest.mark.parametrize("bits", [5, 8])
def test_bits_all_zero_rows(oracle, bits, with_tables):
    """Rows whose gradient stays zero: scale 0, 0/0 -> NaN -> the byte 255."""
    qm, qv = _maps(oracle, bits)
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(80 + bits)
    tensors = [_Tensor(r, c, bits, rng) for r, c in [(40, 384), (70, 128)]]
    for step in (1, 2):
        grads = [_grad(rng, t, z) for t, z in zip(tensors, (34, 3))]
        _step_all(oracle, tensors, grads, bits, qm, qv, dqm, dqv, step, with_tables)
        for t in tensors:
            t.check(f"{bits} bits, {t.rows}x{t.cols} step {step}")


def test_bits_more_tensors_than_one_launch_and_full_size(oracle):
    bits = 6
    qm, qv = _maps(oracle, bits)
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(90)
    tensors = [_Tensor(int(r), 128 * int(cb), bits, rng)
               for r, cb in zip(rng.integers(1, 200, 40), rng.integers(1, 5, 40))]
    tensors.append(_Tensor(4096, 4096, bits, rng))
    for step in (1, 2):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, bits, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_bits_argument_checks(oracle):
    nat = _native()
    lib = nat.lib()
    qm, qv = _maps(oracle, 8)
    dqm, dqv = to_dev(qm), to_dev(qv)
    stream = torch.cuda.current_stream().cuda_stream
    f5 = (H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"])
    p = torch.zeros(256, device="cuda")
    mc = torch.zeros(_nbytes(256), dtype=torch.uint8, device="cuda")
    vc = torch.zeros(_nbytes(256), dtype=torch.uint8, device="cuda")
    ms = torch.zeros(2, device="cuda")
    row = [torch.zeros(2, device="cuda") for _ in range(2)]
    col = [torch.zeros(128, device="cuda") for _ in range(2)]
    ok = (p.data_ptr(), p.data_ptr(), mc.data_ptr(), ms.data_ptr(), vc.data_ptr(), row[0].data_ptr(),
          col[0].data_ptr(), row[1].data_ptr(), col[1].data_ptr(), 2, 128, 1.0, 0.0)

    def call(records, bm=8, bv=8):
        table = np.array(records, dtype=nat.NONFUSED_RANK1_TENSOR)
        return lib.lpmm_nonfused_adamw_bits_rank1_step_multi(table.ctypes.data, len(records), dqm.data_ptr(), bm,
                                                             dqv.data_ptr(), bv, *f5, stream)

    for bm, bv in [(4, 8), (8, 4), (9, 8), (0, 0), (3, 3)]:
        assert call([ok], bm, bv) != 0, (bm, bv)
    assert call([ok[:2] + (0,) + ok[3:]]) != 0
    assert call([ok[:10] + (100, 1.0, 0.0)]) != 0  # columns not a multiple of 128
    assert call([ok[:9] + (0, 128, 1.0, 0.0)]) == 0  # an empty tensor is skipped
    torch.cuda.synchronize()
