"""GPU parity of stochastic rounding (pack_nonlinear(..., stochastic=True)): the HIP kernel
against the CPU oracle bit for bit, the oracle's Philox conventions against PyTorch's device
generator, and the path through lpmm.functional and the optimizer."""
import numpy as np
import pytest
import torch

from util import to_dev, to_np

pytestmark = pytest.mark.gpu


def _lib():
    from lpmm import _native

    return _native.lib()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _nbytes(n_padded, bits):
    return n_padded * (bits if bits in (1, 2, 4) else 8) // 8 + 1


def test_philox_conventions_match_the_device_generator(oracle):
    """torch.randint on the device draws curand4 from a Philox state initialised with
    (seed, thread index, offset) and hands component c of thread i to element i + c * T, T the
    number of threads of its launch (256 per block, as many blocks as there are elements / 256,
    capped at what the device holds at once).  So a tensor of 4 T elements shows all four
    components of the first block of every subsequence, and a second call the next block.
    With a range of 2^27 (small enough for torch to use one 32-bit output per element) the element
    is the raw output modulo 2^27.  (The block function
    itself, all 32 bits, is pinned by the known-answer vectors of the CPU tests.)"""
    dev = torch.device("cuda:0")
    prop = torch.cuda.get_device_properties(dev)
    T = prop.multi_processor_count * (prop.max_threads_per_multi_processor // 256) * 256
    seed = 123456789
    torch.manual_seed(seed)
    first = to_np(torch.randint(0, 2 ** 27, (4 * T,), device=dev))
    second = to_np(torch.randint(0, 2 ** 27, (4 * T,), device=dev))  # the generator's offset advanced by 4
    torch.manual_seed(seed)
    uni = to_np(torch.rand(4 * T, device=dev))
    rng = np.random.default_rng(0)
    for i in [0, 1, 2, 255, 256, T - 1] + [int(v) for v in rng.integers(0, T, 60)]:
        for c in range(4):
            for got, off in ((first, 0), (second, 4)):
                assert int(got[i + c * T]) == oracle.philox_draw(seed, i, off, c) & 0x7FFFFFF, (i, c, off)
            # the uniform conversion: the reference's generator library computes u * 2^-32 + 2^-33
            # (restated in the oracle and the kernel); the device library here may differ from that
            # in the last place, which is as close as this comparison can be
            want = oracle.philox_uniform(seed, i, 0, c)
            assert abs(float(uni[i + c * T]) - want) <= 2.0 ** -24 * max(want, 2.0 ** -8), (i, c)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("seed,offset", [(0, 0), (0x9E3779B97F4A7C15, 16384), (42, 3), (7, (1 << 34) + 6)])
def test_pack_sr_matches_oracle(oracle, bits, seed, offset):
    lib = _lib()
    qmap = np.asarray(oracle.create_pow_map(bits, True, 1), np.float32)
    rng = np.random.default_rng(bits * 131 + offset % 97)
    for n in (32, 2048, 2048 * 3 + 64):
        x = rng.uniform(-1.05, 1.05, n).astype(np.float32)
        x[::97] = qmap[rng.integers(0, qmap.size, x[::97].size)]  # exact map points
        x[5] = np.nan
        want = oracle.pack_nonlinear_sr(x, qmap, bits, seed, offset)
        dx, dq = to_dev(x), to_dev(qmap)
        out = torch.full((_nbytes(n, bits) + 7,), 0x55, dtype=torch.uint8, device="cuda")
        st = lib.lpmm_pack_nonlinear_sr(dx.data_ptr(), dq.data_ptr(), bits, n, seed, offset, out.data_ptr(), _stream())
        assert st == 0, lib.lpmm_status_string(st)
        got = to_np(out)
        np.testing.assert_array_equal(got[:_nbytes(n, bits)], want, err_msg=f"bits {bits} n {n}")
        assert np.all(got[_nbytes(n, bits):] == 0x55), "wrote past the end"


def test_pack_sr_argument_errors():
    lib = _lib()
    x = torch.zeros(64, device="cuda")
    q = torch.linspace(-1, 1, 16, device="cuda")
    out = torch.zeros(64, dtype=torch.uint8, device="cuda")
    assert lib.lpmm_pack_nonlinear_sr(x.data_ptr(), q.data_ptr(), 4, 48, 0, 0, out.data_ptr(), _stream()) == 3
    assert lib.lpmm_pack_nonlinear_sr(x.data_ptr(), q.data_ptr(), 9, 64, 0, 0, out.data_ptr(), _stream()) == 3
    assert lib.lpmm_pack_nonlinear_sr(None, q.data_ptr(), 4, 64, 0, 0, out.data_ptr(), _stream()) == 1


def test_operator_draws_from_the_default_generator(oracle, qmaps):
    """The operator shim takes (seed, offset) from torch's default generator of the device and
    advances the offset by group_size * work_per_thread, as the reference's launcher does
    (quantization_kernel.cu:480-487)."""
    from lpmm.cpp_extension import quantization as ext

    qm = np.asarray(qmaps[0], np.float32)
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (3, 2048)).astype(np.float32)
    torch.manual_seed(2024)
    gen = torch.cuda.default_generators[0]
    off0 = gen.get_offset()
    a = ext.pack_nonlinear(to_dev(x), to_dev(qm), 4, True)
    assert gen.get_offset() == off0 + 2048 * 8
    b = ext.pack_nonlinear(to_dev(x), to_dev(qm), 4, True)
    assert gen.get_offset() == off0 + 2 * 2048 * 8
    np.testing.assert_array_equal(to_np(a).view(np.uint8), oracle.pack_nonlinear_sr(x, qm, 4, 2024, off0))
    np.testing.assert_array_equal(to_np(b).view(np.uint8), oracle.pack_nonlinear_sr(x, qm, 4, 2024, off0 + 2048 * 8))
    assert not np.array_equal(to_np(a), to_np(b))
    # the nearest path leaves the generator alone
    ext.pack_nonlinear(to_dev(x), to_dev(qm), 4, False)
    assert gen.get_offset() == off0 + 2 * 2048 * 8


@pytest.mark.parametrize("scale_type,shape", [("group", (300, 70)), ("rank1", (96, 200)), ("rank1", (5000,))])
def test_vectorwise_quant_real_sr(oracle, qmaps, scale_type, shape):
    """round_type 'real-sr' through lpmm.functional: the scaling is the same as for
    'real-nearest' (same scales), every decoded value is one of the two map entries around the
    normalised value, and the mean over repeated quantisations approaches x."""
    import lpmm.functional as F

    signed = scale_type == "group"
    qmap = to_dev(np.asarray(qmaps[0] if signed else qmaps[1], np.float32))
    rng = np.random.default_rng(11)
    x = rng.standard_normal(shape).astype(np.float32)
    if not signed:
        # inside the range of the zero-excluded map after scaling (values below its first entry,
        # 1/16 of the scale, go to code 0 whatever the rounding)
        x = rng.uniform(0.2, 1.0, shape).astype(np.float32)
    dx = to_dev(x)
    kw = dict(qmap=qmap, shape=dx.shape, b=4, signed=signed, quant_type="nonlinear" if signed else "power-1",
              scale_type=scale_type, gp_sz=128, enable=True)
    torch.manual_seed(1)
    qn, mdn = F.vectorwise_quant(dx, round_type="real-nearest", **kw)
    acc = np.zeros(x.shape, np.float64)
    reps = 24
    for _ in range(reps):
        qs, mds = F.vectorwise_quant(dx, round_type="real-sr", **kw)
        assert qs.shape == qn.shape and qs.dtype == qn.dtype
        for k in ("max1", "max_dims"):
            if mdn.get(k) is not None:
                a, b = mdn[k], mds[k]
                if isinstance(a, (list, tuple)):
                    for u, v in zip(a, b):
                        assert torch.equal(u, v)
                else:
                    assert torch.equal(a, b)
        full = dict(kw)
        full.update(mds)
        dec = to_np(F.vectorwise_dequant(qs, round_type="real-sr", **full))
        assert dec.shape == x.shape
        acc += dec
    full = dict(kw)
    full.update(mdn)
    near = to_np(F.vectorwise_dequant(qn, round_type="real-nearest", **full))
    # unbiased: the averaged reconstruction is much closer to x than one nearest rounding
    err_sr = np.abs(acc / reps - x).mean()
    err_near = np.abs(near - x).mean()
    assert err_sr < 0.5 * err_near, (err_sr, err_near)


def test_optimizer_with_real_sr_config(tmp_path, qmaps):
    """A configuration with ROUND_TYPE real-sr runs the staged non-fused step (dequantise,
    update, re-quantise stochastically); the states stay within one quantisation cell of the
    round-to-nearest run."""
    import lpmm

    cfg = tmp_path / "sr.yml"
    cfg.write_text("QUANT:\n  M:\n    ROUND_TYPE: real-sr\n  SQM:\n    ROUND_TYPE: real-sr\n")
    torch.manual_seed(0)
    p0 = torch.randn(64, 256, device="cuda") * 0.02
    outs = []
    for qc in (str(cfg), None):
        p = torch.nn.Parameter(p0.clone())
        opt = lpmm.optim.AdamW([p], lr=1e-3, betas=(0.9, 0.999), weight_decay=0.01, fused=False, qconfig=qc)
        g = torch.Generator(device="cuda").manual_seed(5)
        for _ in range(3):
            p.grad = torch.randn(p.shape, device="cuda", generator=g) * 1e-3
            opt.step()
        st = opt.state[p]
        assert st["exp_avg"].dtype == torch.int8 and st["exp_avg"].numel() > 1
        outs.append(to_np(p.detach()))
        assert np.isfinite(outs[-1]).all()
    assert not np.array_equal(outs[0], outs[1])
    np.testing.assert_allclose(outs[0], outs[1], rtol=0, atol=3 * 3e-3)  # three steps of at most ~lr each
