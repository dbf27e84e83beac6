"""GPU parity of the non-fused elementwise update and of the factored second-moment step
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from util import assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

H = dict(beta1=0.9, beta2=0.999, lr=1e-3, wd=0.01, eps=1e-8)


def _lib():
    from lpmm import _native

    return _native.lib()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def test_nonfused_update_matches_oracle(oracle):
    lib = _lib()
    rng = np.random.default_rng(5)
    for n in (1, 1000, 4096 * 33 + 5):
        p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        m = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        v = (rng.standard_normal(n) ** 2 * 1e-6).astype(np.float32)
        dp, dm, dv = to_dev(p), to_dev(m), to_dev(v)
        mismatches = 0
        for step in (1.0, 2.0, 77.0):
            g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
            dg = to_dev(g)
            st = lib.lpmm_nonfused_update(dp.data_ptr(), dg.data_ptr(), dm.data_ptr(), dv.data_ptr(), n, H["beta1"],
                                          H["beta2"], H["lr"], H["wd"], H["eps"], step, _stream())
            assert st == 0
            oracle.nonfused_update(p, g, m, v, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], step)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(to_np(dm), m)
            np.testing.assert_array_equal(to_np(dv), v)
            got_p = to_np(dp)
            assert_rel(got_p, p, "p", scale=p)
            mismatches += int(np.sum(got_p != p))
            dp.copy_(torch.from_numpy(p))
        # the update's sqrt and divisions are near-exact: at most a stray last-bit difference
        assert mismatches <= max(1, n // 100000), mismatches


def test_nonfused_update_multi_matches_oracle(oracle):
    """Many small fp32-state tensors in one call (more than one launch holds), each with its
    own step count."""
    from lpmm import _native

    lib = _lib()
    rng = np.random.default_rng(6)
    sizes = [int(n) for n in rng.integers(1, 5000, size=70)] + [4096 * 3 + 1]
    host, dev = [], []
    for n in sizes:
        arrs = [(rng.standard_normal(n) * 0.02).astype(np.float32), (rng.standard_normal(n) * 1e-3).astype(np.float32),
                (rng.standard_normal(n) * 1e-3).astype(np.float32), (rng.standard_normal(n) ** 2 * 1e-6).astype(np.float32)]
        host.append(arrs)
        dev.append([to_dev(a) for a in arrs])
    steps = [float(1 + i % 9) for i in range(len(sizes))]
    table = np.array([(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), n, st, 0.0)
                      for d, n, st in zip(dev, sizes, steps)], dtype=_native.ADAMW_FP32_TENSOR)
    st = lib.lpmm_nonfused_update_multi(table.ctypes.data, len(sizes), H["beta1"], H["beta2"], H["lr"], H["wd"],
                                        H["eps"], _stream())
    assert st == 0
    torch.cuda.synchronize()
    for (p, g, m, v), d, step in zip(host, dev, steps):
        oracle.nonfused_update(p, g, m, v, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], step)
        np.testing.assert_array_equal(to_np(d[2]), m)
        np.testing.assert_array_equal(to_np(d[3]), v)
        assert_rel(to_np(d[0]), p, "p", scale=p)


@pytest.mark.parametrize("shape", [(64, 128), (100, 70), (513, 1025), (1024, 2752), (2752, 1024)])
def test_factored_step_matches_oracle(oracle, qmaps, shape):
    lib = _lib()
    qm = qmaps[0]
    dqm = to_dev(qm)
    r, c = shape
    n = r * c
    rng = np.random.default_rng(r + c)
    p = (rng.standard_normal((r, c)) * 0.02).astype(np.float32)
    row, col = np.zeros(r, np.float32), np.zeros(c, np.float32)
    dp, drow, dcol = to_dev(p), to_dev(row), to_dev(col)
    groups = (n + 127) // 128
    nbytes = (groups * 128 + 2047) // 2048 * 1024 + 1
    codes = torch.full((nbytes,), 0x55, dtype=torch.uint8, device="cuda")
    max1 = torch.zeros(groups, dtype=torch.float32, device="cuda")
    mean_all = torch.zeros(1, dtype=torch.float32, device="cuda")
    work = torch.empty(lib.lpmm_factored_workspace_bytes(r, c), dtype=torch.uint8, device="cuda")
    m_state = None
    for step in range(1, 5):
        g = (rng.standard_normal((r, c)) * 1e-3 * (1 + rng.random((r, 1)) * 3)).astype(np.float32)
        dg = to_dev(g)
        assert lib.lpmm_factored_stats(dg.data_ptr(), r, c, drow.data_ptr(), dcol.data_ptr(), mean_all.data_ptr(),
                                       H["beta2"], work.data_ptr(), _stream()) == 0
        assert lib.lpmm_factored_update(dp.data_ptr(), dg.data_ptr(), codes.data_ptr(), max1.data_ptr(),
                                        dqm.data_ptr(), drow.data_ptr(), dcol.data_ptr(), mean_all.data_ptr(), r, c,
                                        H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"], float(step),
                                        1 if step == 1 else 0, _stream()) == 0
        # oracle
        row_mean, col_mean = oracle.factored_stats(g)
        mean_ref = oracle.factored_ema(row, col, row_mean, col_mean, H["beta2"])
        m = np.zeros(n, np.float32) if m_state is None else oracle.dequant_group(m_state[0], m_state[1], qm, n)
        oracle.factored_update(p, g, m, row, col, mean_ref, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"],
                               float(step))
        m_state = oracle.quant_group(m, qm)
        torch.cuda.synchronize()
        # row/col sums are accumulated in double in a different (fixed) order than the oracle's
        # sequential loop: equal after rounding to float except for rare last-bit differences
        assert_rel(to_np(drow), row, f"row step {step}", tol=2e-7)
        assert_rel(to_np(dcol), col, f"col step {step}", tol=2e-7)
        assert_rel(to_np(mean_all), [mean_ref], f"mean step {step}", tol=2e-7)
        assert_rel(to_np(dp), p, f"p step {step}")
        # the first moment does not depend on the second: bit-exact
        np.testing.assert_array_equal(to_np(max1), m_state[1])
        np.testing.assert_array_equal(to_np(codes), m_state[0])
        # continue from the oracle's statistics so that the comparison stays one step deep
        drow.copy_(torch.from_numpy(row)); dcol.copy_(torch.from_numpy(col)); dp.copy_(torch.from_numpy(p))


def test_factored_step_multi_matches_oracle(oracle, qmaps):
    """Statistics + update of many tensors per call (more than one launch group holds), each
    with its own step count, against the oracle."""
    from lpmm import _native

    lib = _lib()
    qm = qmaps[0]
    dqm = to_dev(qm)
    rng = np.random.default_rng(9)
    shapes = [(64, 128), (1, 128), (33, 256), (513, 1024), (100, 2176), (300, 4224)]
    shapes += [(int(r), 128 * int(cb)) for r, cb in zip(rng.integers(1, 120, 24), rng.integers(1, 4, 24))]
    tensors = []
    for r, c in shapes:
        n = r * c
        t = dict(r=r, c=c, n=n, p=(rng.standard_normal((r, c)) * 0.02).astype(np.float32),
                 row=np.zeros(r, np.float32), col=np.zeros(c, np.float32), m_state=None,
                 step0=int(rng.integers(0, 5)))
        t["dp"], t["drow"], t["dcol"] = to_dev(t["p"]), to_dev(t["row"]), to_dev(t["col"])
        t["codes"] = torch.full(((n + 2047) // 2048 * 1024 + 1,), 0x55, dtype=torch.uint8, device="cuda")
        t["max1"] = torch.zeros(n // 128, dtype=torch.float32, device="cuda")
        t["work"] = torch.empty(lib.lpmm_factored_workspace_bytes(r, c), dtype=torch.uint8, device="cuda")
        tensors.append(t)
    for it in range(1, 4):
        grads, recs = [], []
        for t in tensors:
            g = (rng.standard_normal((t["r"], t["c"])) * 1e-3 * (1 + rng.random((t["r"], 1)) * 3)).astype(np.float32)
            t["g"], t["dg"] = g, to_dev(g)
            recs.append((t["dp"].data_ptr(), t["dg"].data_ptr(), t["codes"].data_ptr(), t["max1"].data_ptr(),
                         t["drow"].data_ptr(), t["dcol"].data_ptr(), t["work"].data_ptr(), t["r"], t["c"],
                         float(t["step0"] + it), 1 if it == 1 else 0))
        table = np.array(recs, dtype=_native.FACTORED_TENSOR)
        st = lib.lpmm_factored_step_multi(table.ctypes.data, len(recs), dqm.data_ptr(), H["beta1"], H["beta2"],
                                          H["lr"], H["wd"], H["eps"], _stream())
        assert st == 0, lib.lpmm_status_string(st)
        torch.cuda.synchronize()
        for t in tensors:
            what = f'{t["r"]}x{t["c"]} iteration {it}'
            row_mean, col_mean = oracle.factored_stats(t["g"])
            mean_ref = oracle.factored_ema(t["row"], t["col"], row_mean, col_mean, H["beta2"])
            m = (np.zeros(t["n"], np.float32) if t["m_state"] is None
                 else oracle.dequant_group(t["m_state"][0], t["m_state"][1], qm, t["n"]))
            oracle.factored_update(t["p"], t["g"], m, t["row"], t["col"], mean_ref, H["beta1"], H["beta2"], H["lr"],
                                   H["wd"], H["eps"], float(t["step0"] + it))
            t["m_state"] = oracle.quant_group(m, qm)
            assert_rel(to_np(t["drow"]), t["row"], f"row {what}", tol=2e-7)
            assert_rel(to_np(t["dcol"]), t["col"], f"col {what}", tol=2e-7)
            assert_rel(to_np(t["dp"]), t["p"], f"p {what}")
            np.testing.assert_array_equal(to_np(t["max1"]), t["m_state"][1], err_msg=what)
            np.testing.assert_array_equal(to_np(t["codes"]), t["m_state"][0], err_msg=what)
            t["drow"].copy_(torch.from_numpy(t["row"])); t["dcol"].copy_(torch.from_numpy(t["col"]))
            t["dp"].copy_(torch.from_numpy(t["p"]))


def test_factored_fp32m_matches_oracle(oracle):
    lib = _lib()
    r, c = 48, 64
    rng = np.random.default_rng(9)
    p = (rng.standard_normal((r, c)) * 0.02).astype(np.float32)
    m = np.zeros(r * c, np.float32)
    row, col = np.zeros(r, np.float32), np.zeros(c, np.float32)
    dp, dm, drow, dcol = to_dev(p), to_dev(m), to_dev(row), to_dev(col)
    mean_all = torch.zeros(1, dtype=torch.float32, device="cuda")
    work = torch.empty(lib.lpmm_factored_workspace_bytes(r, c), dtype=torch.uint8, device="cuda")
    for step in range(1, 4):
        g = (rng.standard_normal((r, c)) * 1e-3).astype(np.float32)
        dg = to_dev(g)
        assert lib.lpmm_factored_stats(dg.data_ptr(), r, c, drow.data_ptr(), dcol.data_ptr(), mean_all.data_ptr(),
                                       H["beta2"], work.data_ptr(), _stream()) == 0
        assert lib.lpmm_factored_update_fp32m(dp.data_ptr(), dg.data_ptr(), dm.data_ptr(), drow.data_ptr(),
                                              dcol.data_ptr(), mean_all.data_ptr(), r, c, H["beta1"], H["beta2"],
                                              H["lr"], H["wd"], H["eps"], float(step), _stream()) == 0
        row_mean, col_mean = oracle.factored_stats(g)
        mean_ref = oracle.factored_ema(row, col, row_mean, col_mean, H["beta2"])
        oracle.factored_update(p, g, m, row, col, mean_ref, H["beta1"], H["beta2"], H["lr"], H["wd"], H["eps"],
                               float(step))
        torch.cuda.synchronize()
        assert_rel(to_np(drow), row, "row", tol=2e-7)
        assert_rel(to_np(dp), p, "p")
        np.testing.assert_array_equal(to_np(dm), m)
        drow.copy_(torch.from_numpy(row)); dcol.copy_(torch.from_numpy(col)); dp.copy_(torch.from_numpy(p))


def test_factored_step_multi_large_batches_equal_single_tensor_calls(qmaps):
    """Tensors whose gradients exceed the byte budget of one launch batch: the multi-tensor
    call (several batches, update pass walking back to front) must leave exactly what
    lpmm_factored_stats + lpmm_factored_update leave tensor by tensor."""
    from lpmm import _native

    lib = _lib()
    dqm = to_dev(qmaps[0])
    gen = torch.Generator(device="cuda").manual_seed(77)
    shapes = [(4096, 8192), (2048, 11008), (4096, 8192), (8192, 4096), (4096, 8192), (1000, 1152), (4096, 8192)]
    assert sum(r * c * 4 for r, c in shapes) > (384 << 20) * 3 // 2  # at least two batches

    def fresh(r, c):
        n = r * c
        t = dict(r=r, c=c, p=torch.randn(r, c, device="cuda", generator=gen) * 0.02,
                 row=torch.rand(r, device="cuda", generator=gen) * 1e-6,
                 col=torch.rand(c, device="cuda", generator=gen) * 1e-6,
                 codes=torch.randint(0, 256, (n // 2048 * 1024 + (1024 if n % 2048 else 0) + 1,), dtype=torch.uint8,
                                     device="cuda", generator=gen),
                 max1=torch.rand(n // 128, device="cuda", generator=gen) * 1e-3,
                 g=torch.randn(r, c, device="cuda", generator=gen) * 1e-3,
                 work=torch.empty(lib.lpmm_factored_workspace_bytes(r, c), dtype=torch.uint8, device="cuda"))
        return t

    a = [fresh(r, c) for r, c in shapes]
    b = [{k: (v.clone() if torch.is_tensor(v) else v) for k, v in t.items()} for t in a]
    recs = [(t["p"].data_ptr(), t["g"].data_ptr(), t["codes"].data_ptr(), t["max1"].data_ptr(), t["row"].data_ptr(),
             t["col"].data_ptr(), t["work"].data_ptr(), t["r"], t["c"], 7.0, 0) for t in a]
    table = np.array(recs, dtype=_native.FACTORED_TENSOR)
    st = lib.lpmm_factored_step_multi(table.ctypes.data, len(recs), dqm.data_ptr(), H["beta1"], H["beta2"], H["lr"],
                                      H["wd"], H["eps"], _stream())
    assert st == 0, lib.lpmm_status_string(st)
    mean_all = torch.zeros(1, dtype=torch.float32, device="cuda")
    for t in b:
        assert lib.lpmm_factored_stats(t["g"].data_ptr(), t["r"], t["c"], t["row"].data_ptr(), t["col"].data_ptr(),
                                       mean_all.data_ptr(), H["beta2"], t["work"].data_ptr(), _stream()) == 0
        assert lib.lpmm_factored_update(t["p"].data_ptr(), t["g"].data_ptr(), t["codes"].data_ptr(),
                                        t["max1"].data_ptr(), dqm.data_ptr(), t["row"].data_ptr(), t["col"].data_ptr(),
                                        mean_all.data_ptr(), t["r"], t["c"], H["beta1"], H["beta2"], H["lr"], H["wd"],
                                        H["eps"], 7.0, 0, _stream()) == 0
    torch.cuda.synchronize()
    for x, y in zip(a, b):
        for k in ("p", "row", "col", "codes", "max1"):
            assert torch.equal(x[k], y[k]), f'{k} of {x["r"]}x{x["c"]}'
