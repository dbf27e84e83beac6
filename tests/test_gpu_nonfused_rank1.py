"""GPU parity of the two-pass non-fused 4-bit AdamW step with a rank-1 second moment against
the CPU oracle's separate stages (dequantise, update, statistics, quantise), called through
the C ABI on torch device memory.  Packed buffers are compared in full, padding included."""
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


class _Tensor:
    def __init__(self, rows, cols, rng, zero_byte_m=0x77, zero_byte_v=0x00):
        self.rows, self.cols, self.n = rows, cols, rows * cols
        self.host_p = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
        self.ref_m = None  # (codes, max1)
        self.ref_v = None  # (codes, rowmax, colmax)
        self.p = to_dev(self.host_p)
        # before the first step: zero scales and statistics, codes of 0.0; padding and the
        # spare statistics hold a pattern the kernels have to overwrite
        mc = np.full(_nbytes(self.n), 0xA5, np.uint8)
        vc = np.full(_nbytes(self.n), 0xA5, np.uint8)
        mc[: self.n // 2] = zero_byte_m
        vc[: self.n // 2] = zero_byte_v
        self.mc, self.vc = to_dev(mc), to_dev(vc)
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
        n, r, c = self.n, self.rows, self.cols
        m = np.zeros(n, np.float32) if self.ref_m is None else oracle.dequant_group(*self.ref_m, qm, n)
        v = np.zeros(n, np.float32) if self.ref_v is None else oracle.dequant_rank1(*self.ref_v, qv, r, c).reshape(-1)
        oracle.nonfused_update(self.host_p.reshape(-1), g.reshape(-1), m, v, H["beta1"], H["beta2"], H["lr"],
                               H["wd"], H["eps"], float(step))
        self.ref_m = oracle.quant_group(m, qm)
        v2 = v.reshape(r, c)
        rowmax, colmax = oracle.rank1_stats(v2)
        self.ref_v = (oracle.quant_rank1(v2, rowmax, colmax, qv), rowmax, colmax)

    def check(self, what):
        np.testing.assert_array_equal(to_np(self.stats[0]), self.ref_v[1], err_msg=f"{what}: v row statistics")
        np.testing.assert_array_equal(to_np(self.stats[1]), self.ref_v[2], err_msg=f"{what}: v column statistics")
        np.testing.assert_array_equal(to_np(self.ms), self.ref_m[1], err_msg=f"{what}: m max1")
        np.testing.assert_array_equal(to_np(self.mc), self.ref_m[0], err_msg=f"{what}: m codes")
        np.testing.assert_array_equal(to_np(self.vc), self.ref_v[0], err_msg=f"{what}: v codes")
        got = to_np(self.p)
        assert_rel(got, self.host_p, f"{what}: p", scale=self.host_p)
        bad = int(np.sum(got != self.host_p))
        assert bad <= max(1, self.n // 100000), (what, bad)
        self.p.copy_(torch.from_numpy(self.host_p))


def _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step):
    nat = _native()
    lib = nat.lib()
    table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.NONFUSED_RANK1_TENSOR)
    st = lib.lpmm_nonfused_adamw4bit_rank1_step_multi(table.ctypes.data, len(tensors), dqm.data_ptr(),
                                                      dqv.data_ptr(), H["beta1"], H["beta2"], H["lr"], H["wd"],
                                                      H["eps"], torch.cuda.current_stream().cuda_stream)
    assert st == 0, lib.lpmm_status_string(st)
    for t, g in zip(tensors, grads):
        t.oracle_step(oracle, g, qm, qv, step)
    torch.cuda.synchronize()


def _grad(rng, t):
    # row and column structure, so that both statistics matter for the scale
    g = rng.standard_normal((t.rows, t.cols)) * 1e-3
    g *= np.exp(rng.standard_normal((t.rows, 1))) * np.exp(rng.standard_normal((1, t.cols)))
    return g.astype(np.float32)


def test_rank1_two_pass_matches_staged_oracle(oracle, qmaps):
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(21)
    # fewer rows than one pass / one tile, ragged row counts, several column blocks, whole tiles
    shapes = [(1, 128), (3, 128), (16, 256), (64, 128), (65, 384), (100, 1280), (130, 128), (513, 1024), (2048, 640),
              (70, 2048), (67, 4224)]
    tensors = [_Tensor(r, c, rng) for r, c in shapes]
    for step in range(1, 5):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_rank1_folded_rows(oracle, qmaps):
    """Column counts of 64 modulo 128 with an even row count (GPT-2-XL's 1600 and 4800): the kernels take
    two tensor rows as one row of whole column blocks; the statistics of a value sit at its own row and
    column.  Fewer double rows than one pass, more than one tile, one and several column tiles, tensors
    with whole column blocks in the same launch."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(29)
    shapes = [(2, 64), (2, 192), (6, 1600), (65, 384), (64, 192), (130, 320), (66, 4800), (258, 1600), (16, 256),
              (1024, 1600), (200, 6464)]
    tensors = [_Tensor(r, c, rng) for r, c in shapes]
    for step in range(1, 4):
        grads = [_grad(rng, t) for t in tensors]
        if step == 2:
            grads[5][7, :] = 0.0  # a row and a column of zeros, one of each half of a double row
            grads[5][:, 300] = 0.0
            grads[7][100:102, :] = 0.0
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_rank1_one_pass_at_a_time(oracle, qmaps):
    """lpmm_nonfused_adamw4bit_rank1_pass_multi: pass 1 and pass 2 as separate calls give what the
    two-pass call gives (here with nothing done in between)."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(31)
    tensors = [_Tensor(r, c, rng) for r, c in [(65, 384), (64, 192), (130, 128)]]
    s = torch.cuda.current_stream().cuda_stream
    for step in (1, 2, 3):
        grads = [_grad(rng, t) for t in tensors]
        table = np.array([t.record(g, step) for t, g in zip(tensors, grads)], dtype=nat.NONFUSED_RANK1_TENSOR)
        for pass_no in (1, 2):
            st = lib.lpmm_nonfused_adamw4bit_rank1_pass_multi(table.ctypes.data, len(tensors), dqm.data_ptr(), dqv.data_ptr(),
                                                              H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], pass_no, s)
            assert st == 0, lib.lpmm_status_string(st)
        for t, g in zip(tensors, grads):
            t.oracle_step(oracle, g, qm, qv, step)
        torch.cuda.synchronize()
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")
    assert lib.lpmm_nonfused_adamw4bit_rank1_pass_multi(table.ctypes.data, len(tensors), dqm.data_ptr(), dqv.data_ptr(),
                                                        H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], 3, s) == 5


def test_rank1_interleaved_row_blocks_with_ragged_last_group(oracle, qmaps):
    """Tensors with more row blocks than interleave in one group: several groups, the last one
    short of blocks and ending in a ragged block (2500 = 39 * 64 + 4 rows over 16 column tiles,
    1100 = 17 * 64 + 12 rows over 32 column tiles, 64 * 11 + 1 rows over 43 column tiles of which
    the last is half empty)."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(23)
    tensors = [_Tensor(r, c, rng) for r, c in [(2500, 4096), (1100, 8192), (705, 11008)]]
    for step in (1, 2):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_rank1_more_tensors_than_one_launch(oracle, qmaps):
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(22)
    tensors = [_Tensor(int(r), 128 * int(cb), rng) for r, cb in zip(rng.integers(1, 200, 40), rng.integers(1, 5, 40))]
    for step in (1, 2, 3):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")


def test_rank1_zero_rows_columns_and_outliers(oracle, qmaps):
    """A row or column whose second moment is all zero has scale 0: 0/0 -> code 15, as in the
    reference; single large gradients dominate a row's and a column's statistic."""
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(23)
    t = _Tensor(70, 256, rng)
    for step in range(1, 4):
        g = _grad(rng, t)
        g[5, :] = 0.0
        g[:, 130] = 0.0
        g[20:40, 0:128] = 0.0  # whole 128-groups of m stay zero
        g[7, 9] = 50.0
        g[60, 200] = 1e-15
        _step_all(oracle, [t], [g], qm, qv, dqm, dqv, step)
        t.check(f"step {step}")
    assert t.ref_v[1][5] == 0.0 and t.ref_v[2][130] == 0.0


def test_rank1_other_maps(oracle):
    qm = np.linspace(-0.2, 1.0, 16).astype(np.float32)  # the code of 0.0 is not 7
    qv = (oracle.qmap_v() ** 2).astype(np.float32)
    zm = int(np.sum((qm[:-1] + qm[1:]) * np.float32(0.5) < 0))
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(24)
    tensors = [_Tensor(r, c, rng, zero_byte_m=zm | (zm << 4)) for r, c in ((5, 128), (77, 256))]
    for step in range(1, 4):
        grads = [_grad(rng, t) for t in tensors]
        _step_all(oracle, tensors, grads, qm, qv, dqm, dqv, step)
        for t in tensors:
            t.check(f"{t.rows}x{t.cols} step {step}")
    # one standard map, one not
    qm_std, qv_std = oracle.qmap_m(), oracle.qmap_v()
    for maps in ((qm_std, qv), (qm, qv_std)):
        t = _Tensor(33, 384, rng, zero_byte_m=0x77 if maps[0] is qm_std else zm | (zm << 4))
        dm, dv = to_dev(maps[0]), to_dev(maps[1])
        for step in (1, 2):
            g = _grad(rng, t)
            _step_all(oracle, [t], [g], maps[0], maps[1], dm, dv, step)
            t.check(f"mixed maps step {step}")


def test_rank1_argument_checks(qmaps):
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    s = torch.cuda.current_stream().cuda_stream
    call = lib.lpmm_nonfused_adamw4bit_rank1_step_multi
    tail = (dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999, 1e-3, 0.0, 1e-8, s)
    assert call(None, 0, *tail) == 0
    assert call(None, 1, *tail) != 0
    buf = torch.zeros(4096, dtype=torch.float32, device="cuda")
    ptr = buf.data_ptr()
    ok = (ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr + 2048, ptr + 4096, 4, 128, 1.0, 0.0)
    bad_cols = ok[:10] + (100,) + ok[11:]
    odd_rows_of_half_blocks = ok[:9] + (3, 192) + ok[11:]  # 64 modulo 128 columns need an even row count
    aliased = ok[:7] + (ptr, ptr) + ok[9:]
    for rec in (bad_cols, odd_rows_of_half_blocks, aliased):
        table = np.array([rec], dtype=nat.NONFUSED_RANK1_TENSOR)
        assert call(table.ctypes.data, 1, *tail) != 0
