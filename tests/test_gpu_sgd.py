"""GPU parity of the one-pass SGD step with a 4-bit momentum buffer (lpmm_sgd4bit_step_multi)
against the CPU oracle's three stages (dequantise -> the reference's op chain on fp32 buffers
-> quantise), called through the C ABI on torch device memory, bit for bit: parameters,
scales and the packed buffer in full, padding codes and the extra last byte included.  The
oracle's op chain is itself pinned against PyTorch's CPU kernels
(tests/test_oracle_steps.py::test_sgd_c_update_follows_torch_cpu_ops)."""
import numpy as np
import pytest
import torch

from util import to_dev, to_np

pytestmark = pytest.mark.gpu


def _native():
    from lpmm import _native

    return _native


def _nbytes(n):
    return (n + 2047) // 2048 * 1024 + 1


class _Tensor:
    def __init__(self, n, rng, offset=0):
        self.n = n
        self.host_p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        self.ref = None  # (codes, max1) of the oracle's buffer
        self.offset = offset  # in floats: 1 makes p and g unaligned for 16-byte accesses
        self.p_store = to_dev(np.concatenate([np.zeros(offset, np.float32), self.host_p]))
        self.p = self.p_store[offset:]
        # a pattern the kernel has to overwrite everywhere
        self.mc = to_dev(np.full(_nbytes(n), 0xA5, np.uint8))
        self.ms = to_dev(np.full((n + 127) // 128, np.nan, np.float32))
        self.g_store = None

    def grad(self, rng):
        g = (rng.standard_normal(self.n) * 1e-2).astype(np.float32)
        if self.n > 300:
            g[rng.integers(0, self.n, 3)] *= 50.0
            g[128:256] = 0.0  # a group of zeros: code 15 throughout, scale 0, once the buffer decays to zero
        self.g_store = to_dev(np.concatenate([np.zeros(self.offset, np.float32), g]))
        return g

    def record(self, first):
        return (self.p.data_ptr(), self.g_store[self.offset:].data_ptr(), self.mc.data_ptr(), self.ms.data_ptr(),
                self.n, 1 if first else 0, 0)

    def oracle_step(self, oracle, g, qm, hyper, first):
        buf = np.zeros(self.n, np.float32) if first else oracle.dequant_group(self.ref[0], self.ref[1], qm, self.n)
        oracle.sgd_update(self.host_p, g, buf, hyper["momentum"], hyper["dampening"], hyper["lr"], hyper["wd"],
                          hyper["nesterov"], hyper["maximize"], first)
        self.ref = oracle.quant_group(buf, qm)

    def check(self, what):
        assert np.array_equal(to_np(self.p), self.host_p), f"{what}: parameters"
        assert np.array_equal(to_np(self.ms), self.ref[1]), f"{what}: scales"
        got = to_np(self.mc)
        assert got.size == self.ref[0].size
        assert np.array_equal(got, self.ref[0]), f"{what}: packed buffer ({np.flatnonzero(got != self.ref[0])[:5]})"
        if self.offset:
            assert not to_np(self.p_store[: self.offset]).any(), f"{what}: wrote in front of the parameter"


def _launch(tensors, first, dqm, hyper):
    nat = _native()
    table = np.array([t.record(first) for t in tensors], dtype=nat.SGD4BIT_TENSOR)
    st = nat.lib().lpmm_sgd4bit_step_multi(table.ctypes.data, len(tensors), dqm.data_ptr(), hyper["momentum"],
                                           hyper["dampening"], hyper["lr"], hyper["wd"], int(hyper["nesterov"]),
                                           int(hyper["maximize"]), torch.cuda.current_stream().cuda_stream)
    nat.check(st, "lpmm_sgd4bit_step_multi")
    torch.cuda.synchronize()


HYPERS = [
    dict(momentum=0.9, dampening=0.0, lr=0.05, wd=0.0, nesterov=False, maximize=False),
    dict(momentum=0.9, dampening=0.1, lr=0.05, wd=1e-4, nesterov=True, maximize=False),
    dict(momentum=0.8, dampening=0.0, lr=0.01, wd=0.05, nesterov=False, maximize=True),
]


@pytest.mark.parametrize("hyper", HYPERS)
def test_sgd_step_matches_oracle(oracle, qmaps, hyper):
    """Sizes around every boundary of the layout (one element, a cut group, a cut pack group,
    whole tiles), aligned and unaligned pointers, four steps (the first creates the buffer)."""
    qm = qmaps[0]
    dqm = to_dev(qm)
    rng = np.random.default_rng(41)
    sizes = [1, 2, 7, 127, 128, 129, 1000, 2047, 2048, 2049, 4096 * 3 + 1, 70000, 2048 * 40]
    tensors = [_Tensor(n, rng) for n in sizes] + [_Tensor(n, rng, offset=1) for n in (5, 300, 2048 * 3, 9999)]
    for step in range(4):
        grads = [t.grad(rng) for t in tensors]
        _launch(tensors, step == 0, dqm, hyper)
        for t, g in zip(tensors, grads):
            t.oracle_step(oracle, g, qm, hyper, step == 0)
            t.check(f"n={t.n} offset={t.offset} step {step}")


def test_sgd_more_tensors_than_one_launch_and_mixed_first_steps(oracle, qmaps):
    """150 tensors (three launches of at most 64), some of which see their first gradient later
    than the others: per-tensor first_step flags."""
    qm = qmaps[0]
    dqm = to_dev(qm)
    hyper = HYPERS[1]
    rng = np.random.default_rng(42)
    tensors = [_Tensor(int(n), rng) for n in rng.integers(1, 6000, 150)]
    started = [False] * len(tensors)
    for step in range(3):
        active = [i for i in range(len(tensors)) if step > 0 or i % 3 != 0]
        grads = {i: tensors[i].grad(rng) for i in active}
        nat = _native()
        table = np.array([tensors[i].record(not started[i]) for i in active], dtype=nat.SGD4BIT_TENSOR)
        st = nat.lib().lpmm_sgd4bit_step_multi(table.ctypes.data, len(active), dqm.data_ptr(), hyper["momentum"],
                                               hyper["dampening"], hyper["lr"], hyper["wd"], 1, 0,
                                               torch.cuda.current_stream().cuda_stream)
        nat.check(st, "lpmm_sgd4bit_step_multi")
        torch.cuda.synchronize()
        for i in active:
            tensors[i].oracle_step(oracle, grads[i], qm, hyper, not started[i])
            started[i] = True
            tensors[i].check(f"tensor {i} n={tensors[i].n} step {step}")


def test_sgd_full_size_matches_oracle(oracle, qmaps):
    """4096 x 11008 (the largest LLaMA-7B MLP shape) for two steps."""
    qm = qmaps[0]
    dqm = to_dev(qm)
    rng = np.random.default_rng(43)
    t = _Tensor(4096 * 11008, rng)
    for step in range(2):
        g = t.grad(rng)
        _launch([t], step == 0, dqm, HYPERS[1])
        t.oracle_step(oracle, g, qm, HYPERS[1], step == 0)
        t.check(f"step {step}")


def test_sgd_optimizer_takes_the_one_pass_kernel_and_interchanges_with_the_op_chain(oracle, qmaps):
    """lpmm.optim.SGD on eligible tensors (2-D, 1-D and 3-D) equals the oracle bit for bit, and
    the state the one-pass kernel writes is the one the staged path reads: the library's own
    vectorwise_dequant decodes it with the recorded metadata."""
    import lpmm

    qm = qmaps[0]
    rng = np.random.default_rng(44)
    hyper = dict(momentum=0.9, dampening=0.1, lr=0.05, wd=1e-4, nesterov=True, maximize=False)
    shapes = [(96, 160), (5000,), (33, 7, 31)]
    host = [(rng.standard_normal(s) * 0.02).astype(np.float32) for s in shapes]
    params = [torch.nn.Parameter(to_dev(h)) for h in host]
    opt = lpmm.optim.SGD(params, lr=hyper["lr"], momentum=hyper["momentum"], dampening=hyper["dampening"],
                         weight_decay=hyper["wd"], nesterov=True)
    refs = [None] * len(shapes)
    for step in range(3):
        grads = [(rng.standard_normal(s) * 1e-2).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        torch.cuda.synchronize()
        for i, (h, g) in enumerate(zip(host, grads)):
            n = h.size
            buf = np.zeros(n, np.float32) if refs[i] is None else oracle.dequant_group(refs[i][0], refs[i][1], qm, n)
            flat = h.reshape(-1)
            oracle.sgd_update(flat, g.reshape(-1), buf, hyper["momentum"], hyper["dampening"], hyper["lr"], hyper["wd"],
                              True, False, refs[i] is None)
            refs[i] = oracle.quant_group(buf, qm)
            st = opt.state[params[i]]
            assert st["momentum_buffer"].dtype == torch.int8
            assert np.array_equal(to_np(st["momentum_buffer"]).view(np.uint8), refs[i][0]), (i, step)
            oh = st["momentum_buffer_qstate"]["overhead"]
            assert tuple(oh["max1"].shape) == ((n + 127) // 128, 1) and tuple(oh["scaled_shape"]) == ((n + 127) // 128, 128)
            assert np.array_equal(to_np(oh["max1"]).reshape(-1), refs[i][1]), (i, step)
            assert np.array_equal(to_np(params[i]), h), (i, step)
    # the same state under the op chain: dequantise with the library's own operator
    from lpmm.functional import vectorwise_dequant

    md = opt.get_qmetadata_by_state_name("momentum_buffer")
    for i, p in enumerate(params):
        st = opt.state[p]
        kw = dict(st["momentum_buffer_qstate"]["overhead"])
        kw.update(md)
        buf = vectorwise_dequant(st["momentum_buffer"], qmap=st["momentum_buffer_qstate"]["qmap"], shape=p.shape, **kw)
        want = oracle.dequant_group(refs[i][0], refs[i][1], qm, host[i].size).reshape(host[i].shape)
        assert np.array_equal(to_np(buf), want)


def test_sgd_argument_checks(qmaps):
    nat = _native()
    lib = nat.lib()
    dqm = to_dev(qmaps[0])
    stream = torch.cuda.current_stream().cuda_stream
    p = torch.zeros(256, device="cuda")
    mc = torch.zeros(_nbytes(256), dtype=torch.uint8, device="cuda")
    ms = torch.zeros(2, device="cuda")
    ok = (p.data_ptr(), p.data_ptr(), mc.data_ptr(), ms.data_ptr(), 256, 1, 0)

    def call(records, count=None, qmap=dqm.data_ptr()):
        table = np.array(records, dtype=nat.SGD4BIT_TENSOR)
        return lib.lpmm_sgd4bit_step_multi(table.ctypes.data, len(records) if count is None else count, qmap, 0.9, 0.0,
                                           0.1, 0.0, 0, 0, stream)

    assert call([ok], count=0) == 0
    assert call([ok], count=-1) != 0
    assert call([ok], qmap=0) != 0
    assert call([(0,) + ok[1:]]) != 0
    assert call([ok[:2] + (0,) + ok[3:]]) != 0
    assert call([ok[:2] + (mc.data_ptr() + 1,) + ok[3:]]) != 0  # codes not 2-byte aligned
    assert call([ok[:4] + (-5, 1, 0)]) != 0
    assert call([ok[:4] + (0, 1, 0)]) == 0  # an empty tensor is skipped
    torch.cuda.synchronize()
