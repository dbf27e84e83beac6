"""GPU parity of the stand-alone quantise / dequantise kernels (non-fused packed layout)
against the CPU oracle, through the C ABI and through lpmm.functional."""
import numpy as np
import pytest
import torch

from util import assert_codes, assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu


def _lib():
    from lpmm import _native

    return _native.lib()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _signed(rng, n):
    x = rng.standard_normal(n).astype(np.float32)
    idx = rng.permutation(n)[: max(1, n // 1000)]
    x[idx] *= 50.0  # 0.1 % outliers x50
    return x


def _unsigned(rng, n):
    return (rng.standard_normal(n) ** 2).astype(np.float32)


@pytest.mark.parametrize("n", [8, 2048, 2048 * 5, 2048 * 3 + 8 * 11])
def test_pack_unpack_match_oracle(oracle, qmaps, n):
    lib = _lib()
    rng = np.random.default_rng(n)
    for qmap, x in ((qmaps[0], np.clip(rng.standard_normal(n) * 0.4, -1, 1).astype(np.float32)),
                    (qmaps[1], rng.random(n).astype(np.float32))):
        if n > 64:
            x[:16] = qmap  # exact map points
            x[16:31] = oracle.midpoints(qmap)  # exact ties -> lower code
            x[40] = np.nan  # NaN -> code 15
            x[41], x[42] = 2.0, -2.0
        want = oracle.pack_nonlinear_4bit(x, qmap)
        dx, dq = to_dev(x), to_dev(qmap)
        out = torch.full((n // 2 + 1,), 0x55, dtype=torch.uint8, device="cuda")
        assert lib.lpmm_pack_nonlinear_4bit(dx.data_ptr(), dq.data_ptr(), n, out.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(out), want)
        back = torch.empty(n, dtype=torch.float32, device="cuda")
        assert lib.lpmm_unpack_nonlinear_4bit(out.data_ptr(), dq.data_ptr(), n, back.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(back), oracle.unpack_nonlinear_4bit(want, qmap, n))


@pytest.mark.parametrize("n,gp_sz", [(4097, 128), (128 * 33, 128), (2048 * 7 + 100, 128), (4096 * 4096 // 16, 128),
                                     (10000, 256), (2048 * 5 + 3, 512), (70000, 1024), (50000, 2048), (50000, 4096),
                                     (4096 * 3, 4096), (100, 4096)])
def test_quant_dequant_group(oracle, qmaps, n, gp_sz):
    lib = _lib()
    rng = np.random.default_rng(n + gp_sz)
    for qmap, x in ((qmaps[0], _signed(rng, n)), (qmaps[1], _unsigned(rng, n))):
        if n > 2 * gp_sz:
            x[gp_sz: 2 * gp_sz] = 0.0  # an all-zero group: 0/0 -> code 15, max1 = 0
        want_codes, want_max1 = oracle.quant_group(x, qmap, gp_sz)
        dx, dq = to_dev(x), to_dev(qmap)
        codes = torch.full((want_codes.size,), 0x55, dtype=torch.uint8, device="cuda")
        max1 = torch.empty(want_max1.size, dtype=torch.float32, device="cuda")
        st = lib.lpmm_quant_group(dx.data_ptr(), n, gp_sz, dq.data_ptr(), codes.data_ptr(), max1.data_ptr(), _stream())
        assert st == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(max1), want_max1)
        np.testing.assert_array_equal(to_np(codes), want_codes)  # includes pad codes and the trailing byte
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        st = lib.lpmm_dequant_group(codes.data_ptr(), max1.data_ptr(), dq.data_ptr(), n, gp_sz, out.data_ptr(), _stream())
        assert st == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(out), oracle.dequant_group(want_codes, want_max1, qmap, n, gp_sz))


@pytest.mark.parametrize("shape", [(64, 80), (33, 1000), (1000, 33), (257, 1029), (2048, 2048), (4096, 1600)])
def test_rank1(oracle, qmaps, shape):
    lib = _lib()
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    r, c = shape
    for qmap, x in ((qmaps[1], _unsigned(rng, r * c).reshape(r, c)), (qmaps[0], _signed(rng, r * c).reshape(r, c))):
        x[3, :] = 0.0  # an all-zero row: scale 0 there
        if c > 5:
            x[:, 5] = 0.0
        want_row, want_col = oracle.rank1_stats(x)
        dx, dq = to_dev(x), to_dev(qmap)
        rowmax = torch.full((r,), -1.0, dtype=torch.float32, device="cuda")
        colmax = torch.full((c,), -1.0, dtype=torch.float32, device="cuda")
        assert lib.lpmm_rank1_stats(dx.data_ptr(), r, c, rowmax.data_ptr(), colmax.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(rowmax), want_row)
        np.testing.assert_array_equal(to_np(colmax), want_col)
        want_codes = oracle.quant_rank1(x, want_row, want_col, qmap)
        codes = torch.full((want_codes.size,), 0x55, dtype=torch.uint8, device="cuda")
        assert lib.lpmm_quant_rank1(dx.data_ptr(), r, c, rowmax.data_ptr(), colmax.data_ptr(), dq.data_ptr(),
                                    codes.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(codes), want_codes)
        out = torch.empty((r, c), dtype=torch.float32, device="cuda")
        assert lib.lpmm_dequant_rank1(codes.data_ptr(), rowmax.data_ptr(), colmax.data_ptr(), dq.data_ptr(), r, c,
                                      out.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(out), oracle.dequant_rank1(want_codes, want_row, want_col, qmap, r, c))


ND_SHAPES = [(6, 50, 40), (64, 64, 3, 3), (5, 7, 2049), (3, 4, 5, 6, 7), (2, 1, 3000, 2), (2, 2, 2, 2, 2, 2, 2, 33),
             (3, 1, 1, 5000), (4, 512, 1024), (7, 4100)]


@pytest.mark.parametrize("with_work", [False, True])
@pytest.mark.parametrize("shape", ND_SHAPES)
def test_rank1_nd(oracle, qmaps, shape, with_work):
    """Rank-1 statistics of tensors of up to 8 dimensions (one-pass kernel, and the 2-D kernel
    plus a fold of its row maxima when a workspace is passed), the row scale derived from them
    and the 2-D quantise / dequantise kernels on the flattened view, against the N-D oracle."""
    import ctypes

    lib = _lib()
    rng = np.random.default_rng(sum(shape) + len(shape))
    n = int(np.prod(shape))
    nd = len(shape)
    shape_arr = (ctypes.c_int64 * nd)(*shape)
    for qmap, bits, x in ((qmaps[1], 4, _unsigned(rng, n).reshape(shape)), (qmaps[0], 4, _signed(rng, n).reshape(shape)),
                          (oracle.create_pow_map(5, False, 1), 5, _unsigned(rng, n).reshape(shape))):
        x[(0,) * nd] = 0.0
        x[(slice(None),) * (nd - 1) + (shape[-1] - 1,)] = 0.0  # an all-zero slice of the last dimension: scale 0
        want_stats = oracle.rank1_stats_nd(x)
        dx, dq = to_dev(x), to_dev(qmap)
        stats = [torch.full((d,), -1.0, dtype=torch.float32, device="cuda") for d in shape]
        ptrs = (ctypes.c_void_p * nd)(*[t.data_ptr() for t in stats])
        work = torch.full((n // shape[-1],), -1.0, dtype=torch.float32, device="cuda") if with_work else None
        st = lib.lpmm_rank1_stats_nd(dx.data_ptr(), nd, shape_arr, ptrs, work.data_ptr() if with_work else None,
                                     _stream())
        assert st == 0
        torch.cuda.synchronize()
        for i, (got, want) in enumerate(zip(stats, want_stats)):
            np.testing.assert_array_equal(to_np(got), want, err_msg=f"statistics of dimension {i}")
        rows, cols = n // shape[-1], shape[-1]
        row_scale = torch.full((rows,), -1.0, dtype=torch.float32, device="cuda")
        assert lib.lpmm_rank1_row_scale_nd(ptrs, nd, shape_arr, row_scale.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        lead = oracle.rank1_scale_nd(want_stats[:-1], shape[:-1]) if nd > 1 else None
        np.testing.assert_array_equal(to_np(row_scale), lead.reshape(-1))
        want_codes = oracle.quant_rank1_nd_bits(x, want_stats, qmap, bits)
        codes = torch.full((want_codes.size,), 0x55, dtype=torch.uint8, device="cuda")
        out = torch.empty(shape, dtype=torch.float32, device="cuda")
        if bits == 4:
            assert lib.lpmm_quant_rank1(dx.data_ptr(), rows, cols, row_scale.data_ptr(), stats[-1].data_ptr(),
                                        dq.data_ptr(), codes.data_ptr(), _stream()) == 0
            assert lib.lpmm_dequant_rank1(codes.data_ptr(), row_scale.data_ptr(), stats[-1].data_ptr(), dq.data_ptr(),
                                          rows, cols, out.data_ptr(), _stream()) == 0
        else:
            assert lib.lpmm_quant_rank1_bits(dx.data_ptr(), rows, cols, row_scale.data_ptr(), stats[-1].data_ptr(),
                                             dq.data_ptr(), bits, codes.data_ptr(), _stream()) == 0
            assert lib.lpmm_dequant_rank1_bits(codes.data_ptr(), row_scale.data_ptr(), stats[-1].data_ptr(),
                                               dq.data_ptr(), bits, rows, cols, out.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(codes), want_codes)
        np.testing.assert_array_equal(to_np(out), oracle.dequant_rank1_nd_bits(want_codes, want_stats, qmap, bits, shape))


def test_rank1_small_fold_scale_multi(oracle):
    """Statistics of every dimension and the scale (their minimum per element) of short vectors, more
    vectors than one launch holds, against the N-D oracle; signed values and NaN included (|x|, and a
    NaN statistic makes the scale NaN as torch.min does)."""
    from lpmm import _native

    lib = _lib()
    rng = np.random.default_rng(77)
    shapes = [(64, 3, 3), (16, 1, 1), (7,), (5, 4, 3, 2, 2), (4096, 3, 3), (2, 2, 2, 2, 2, 2, 2), (640,)] * 6
    shapes = shapes[:40]
    xs, outs, records = [], [], []
    for i, shape in enumerate(shapes):
        x = (rng.standard_normal(shape) * np.exp(rng.standard_normal(shape))).astype(np.float32)
        x[(0,) * len(shape)] = 0.0
        if i == 3:
            x[(1,) * len(shape)] = np.nan
        dx = to_dev(x)
        stats = [torch.full((d,), -1.0, dtype=torch.float32, device="cuda") for d in shape]
        scale = torch.full((x.size,), -1.0, dtype=torch.float32, device="cuda")
        pad = 7 - len(shape)
        records.append((dx.data_ptr(), scale.data_ptr(), tuple(t.data_ptr() for t in stats) + (0,) * pad,
                        tuple(shape) + (1,) * pad, len(shape), 0))
        xs.append((x, dx))
        outs.append((stats, scale))
    table = np.array(records, dtype=_native.RANK1_SMALL_VECTOR)
    assert lib.lpmm_rank1_small_fold_scale_multi(table.ctypes.data, len(records), _stream()) == 0
    torch.cuda.synchronize()
    for (x, _), (stats, scale), shape in zip(xs, outs, shapes):
        want = oracle.rank1_stats_nd(x)
        for i, (got, w) in enumerate(zip(stats, want)):
            np.testing.assert_array_equal(to_np(got), w, err_msg=f"{shape}: statistics of dimension {i}")
        np.testing.assert_array_equal(to_np(scale), oracle.rank1_scale_nd(want, shape).reshape(-1), err_msg=str(shape))
    # arguments: no dimensions, more statistics than a workgroup keeps, a missing pointer
    ok = records[0]
    for bad, status in ((ok[:4] + (0, 0), 5), (ok[:3] + ((8190, 2, 1, 1, 1, 1, 1),) + ok[4:], 3), ((0,) + ok[1:], 1)):
        table = np.array([bad], dtype=_native.RANK1_SMALL_VECTOR)
        assert lib.lpmm_rank1_small_fold_scale_multi(table.ctypes.data, 1, _stream()) == status
    assert lib.lpmm_rank1_small_fold_scale_multi(None, 0, _stream()) == 0


def test_rank1_nd_rejects_bad_arguments():
    import ctypes

    lib = _lib()
    x = torch.zeros(64, device="cuda")
    stats = [torch.zeros(4, device="cuda") for _ in range(3)]
    ptrs = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in stats])
    shape = (ctypes.c_int64 * 3)(4, 4, 4)
    assert lib.lpmm_rank1_stats_nd(x.data_ptr(), 0, shape, ptrs, None, _stream()) == 5
    assert lib.lpmm_rank1_stats_nd(x.data_ptr(), 9, shape, ptrs, None, _stream()) == 5
    assert lib.lpmm_rank1_stats_nd(None, 3, shape, ptrs, None, _stream()) == 1
    assert lib.lpmm_rank1_stats_nd(x.data_ptr(), 3, (ctypes.c_int64 * 3)(4, 0, 4), ptrs, None, _stream()) == 3
    assert lib.lpmm_rank1_stats_nd(x.data_ptr(), 3, (ctypes.c_int64 * 3)(2 ** 31, 2 ** 31, 4), ptrs, None, _stream()) == 3
    assert lib.lpmm_rank1_stats_nd(x.data_ptr(), 3, shape, (ctypes.c_void_p * 3)(stats[0].data_ptr(), None, None), None,
                                   _stream()) == 1
    assert lib.lpmm_rank1_row_scale_nd(ptrs, 1, shape, x.data_ptr(), _stream()) == 5
    assert lib.lpmm_rank1_row_scale_nd(ptrs, 3, shape, None, _stream()) == 1
    torch.cuda.synchronize()


def test_functional_round_trip_metadata(oracle, qmaps):
    """vectorwise_quant / vectorwise_dequant: layout, metadata and values as the reference
    defines them (lpmm/functional.py:26-151)."""
    import lpmm.functional as F

    rng = np.random.default_rng(0)
    qm, qv = to_dev(qmaps[0]), to_dev(qmaps[1])
    md_m = dict(b=4, scale_type="group", quant_type="nonlinear", round_type="real-nearest", gp_sz=128, signed=True)
    md_v = dict(b=4, scale_type="rank1", quant_type="power-1", round_type="real-nearest", gp_sz=128, signed=False)

    x = _signed(rng, 300 * 70).reshape(300, 70)
    dx = to_dev(x)
    qx, gen = F.vectorwise_quant(dx, qmap=qm, shape=dx.shape, **md_m)
    g = (x.size + 127) // 128
    assert qx.dtype == torch.int8 and qx.numel() == (x.size + 2047) // 2048 * 1024 + 1
    assert gen["max1"].shape == (g, 1) and gen["scaled_shape"] == torch.Size((g, 128))
    assert gen["dtype"] == torch.float32 and gen["stride"] == dx.stride()
    want_codes, want_max1 = oracle.quant_group(x, qmaps[0], 128)
    np.testing.assert_array_equal(to_np(qx).view(np.uint8), want_codes)
    back = F.vectorwise_dequant(qx, qmap=qm, shape=dx.shape, **{**gen, **md_m})
    assert back.shape == dx.shape
    np.testing.assert_array_equal(to_np(back).reshape(-1), oracle.dequant_group(want_codes, want_max1, qmaps[0], x.size))

    v = _unsigned(rng, 300 * 70).reshape(300, 70)
    dv = to_dev(v)
    qv_codes, gen = F.vectorwise_quant(dv, qmap=qv, shape=dv.shape, **md_v)
    assert gen["dim"] == 2 and gen["max1"] is None and gen["scaled_shape"] == dv.shape
    assert gen["max_dims"][0].shape == (300, 1) and gen["max_dims"][1].shape == (1, 70)
    row, col = oracle.rank1_stats(v)
    np.testing.assert_array_equal(to_np(qv_codes).view(np.uint8), oracle.quant_rank1(v, row, col, qmaps[1]))
    back = F.vectorwise_dequant(qv_codes, qmap=qv, shape=dv.shape, **{**gen, **md_v})
    np.testing.assert_array_equal(to_np(back), oracle.dequant_rank1(to_np(qv_codes).view(np.uint8), row, col, qmaps[1], 300, 70))

    # rank1 on a 1-D tensor falls back to group-128 (lpmm/functional.py:192-197)
    b = _unsigned(rng, 11008)
    db = to_dev(b)
    qb, gen = F.vectorwise_quant(db, qmap=qv, shape=db.shape, **md_v)
    assert gen["dim"] == 1 and gen["max1"].shape == (86, 1)
    np.testing.assert_array_equal(to_np(qb).view(np.uint8), oracle.quant_group(b, qmaps[1], 128)[0])
    back = F.vectorwise_dequant(qb, qmap=qv, shape=db.shape, **{**gen, **md_v})
    np.testing.assert_array_equal(to_np(back), oracle.dequant_group(to_np(qb).view(np.uint8), to_np(gen["max1"]), qmaps[1], b.size))

    # 3-D rank1: N-D statistics kernels, then the 2-D kernels on the (6*50, 40) view
    w = _unsigned(rng, 6 * 50 * 40).reshape(6, 50, 40)
    dw = to_dev(w)
    qw, gen = F.vectorwise_quant(dw, qmap=qv, shape=dw.shape, **md_v)
    st = np.minimum(np.minimum(w.max(axis=(1, 2), keepdims=True), w.max(axis=(0, 2), keepdims=True)),
                    w.max(axis=(0, 1), keepdims=True))
    ng = (w.size + 2047) // 2048
    padded = np.zeros(ng * 2048, np.float32)
    padded[: w.size] = (w / st).reshape(-1)
    np.testing.assert_array_equal(to_np(qw).view(np.uint8), oracle.pack_nonlinear_4bit(padded, qmaps[1]))
    back = F.vectorwise_dequant(qw, qmap=qv, shape=dw.shape, **{**gen, **md_v})
    want = oracle.unpack_nonlinear_4bit(to_np(qw).view(np.uint8), qmaps[1], w.size).reshape(w.shape) * st
    np.testing.assert_array_equal(to_np(back), want.astype(np.float32))
    assert gen["dim"] == 3 and [tuple(m.shape) for m in gen["max_dims"]] == [(6, 1, 1), (1, 50, 1), (1, 1, 40)]
    for m, want_st in zip(gen["max_dims"], oracle.rank1_stats_nd(w)):
        np.testing.assert_array_equal(to_np(m).reshape(-1), want_st)


def test_shim_pack_unpack_signatures(oracle, qmaps):
    """lpmm.cpp_extension.quantization keeps the reference's positional signatures
    (lpmm/cpp_extension/quantization.cc:54-83) and its size conventions."""
    from lpmm.cpp_extension import quantization as ext

    rng = np.random.default_rng(1)
    x = rng.random((3, 2048)).astype(np.float32)
    dq = to_dev(qmaps[1])
    packed = ext.pack_nonlinear(to_dev(x), dq, 4, False)
    assert packed.dtype == torch.int8 and packed.shape == (3 * 1024 + 1,)
    np.testing.assert_array_equal(to_np(packed).view(np.uint8), oracle.pack_nonlinear_4bit(x, qmaps[1]))
    un = ext.unpack_nonlinear(packed, dq, 4, 3, 2048)
    assert un.shape == (3, 2048) and un.dtype == torch.float32
    # half data is widened to float before the search, as in the reference's at::Half instantiation
    xh = to_dev(x).half()
    for bits, qmap in ((4, qmaps[1]), (5, oracle.create_pow_map(5, False, 1))):
        got = ext.pack_nonlinear(xh, to_dev(qmap), bits, False)
        want = oracle.pack_nonlinear(to_np(xh).astype(np.float32).reshape(-1), qmap, bits)
        np.testing.assert_array_equal(to_np(got).view(np.uint8), want)
    with pytest.raises(RuntimeError, match="kFloat16"):
        ext.pack_nonlinear(to_dev(x), dq.half(), 4, False)  # the map must be float32 there as well
    # double data is rounded to float before the search (the reference's kernel: `const float x = data[i]`)
    xd = to_dev(x).double() * (1.0 + 2.0 ** -30)
    got = ext.pack_nonlinear(xd, dq, 4, False)
    want = oracle.pack_nonlinear_4bit(xd.float().cpu().numpy().reshape(-1), qmaps[1])
    np.testing.assert_array_equal(to_np(got).view(np.uint8), want)
    with pytest.raises(RuntimeError, match="kFloat64"):
        ext.pack_nonlinear(to_dev(x), dq.double(), 4, False)
    with pytest.raises(RuntimeError):
        ext.pack_nonlinear(torch.from_numpy(x), dq, 4, False)  # CPU tensor
    with pytest.raises(RuntimeError):
        ext.pack_nonlinear(to_dev(x).reshape(-1), dq, 4, False)  # wrong dimension
    with pytest.raises(RuntimeError):
        ext.unpack_nonlinear(packed.to(torch.uint8), dq, 4, 3, 2048)  # not int8


def test_quant_group_other_map(oracle):
    """A non-standard map goes through the generic search of the same kernels."""
    lib = _lib()
    rng = np.random.default_rng(12)
    qmap = oracle.create_pow_map(4, True, 1)
    n = 2048 * 3 + 700
    x = _signed(rng, n)
    want_codes, want_max1 = oracle.quant_group(x, qmap, 128)
    dx, dq = to_dev(x), to_dev(qmap)
    codes = torch.empty(want_codes.size, dtype=torch.uint8, device="cuda")
    max1 = torch.empty(want_max1.size, dtype=torch.float32, device="cuda")
    assert lib.lpmm_quant_group(dx.data_ptr(), n, 128, dq.data_ptr(), codes.data_ptr(), max1.data_ptr(), _stream()) == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(codes), want_codes)
    np.testing.assert_array_equal(to_np(max1), want_max1)
    normed = np.clip(rng.standard_normal(2048) * 0.5, -1.5, 1.5).astype(np.float32)
    out = torch.empty(1025, dtype=torch.uint8, device="cuda")
    assert lib.lpmm_pack_nonlinear_4bit(to_dev(normed).data_ptr(), dq.data_ptr(), 2048, out.data_ptr(), _stream()) == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(out), oracle.pack_nonlinear_4bit(normed, qmap))


def test_quant_group_extreme_scales(oracle, qmaps):
    lib = _lib()
    rng = np.random.default_rng(13)
    for scale in (1e-30, 1e-20, 1e20, 1e30):
        for qmap, x in ((qmaps[0], (rng.standard_normal(4096) * scale).astype(np.float32)),
                        (qmaps[1], (rng.random(4096) * scale).astype(np.float32))):
            want_codes, want_max1 = oracle.quant_group(x, qmap, 128)
            dx, dq = to_dev(x), to_dev(qmap)
            codes = torch.empty(want_codes.size, dtype=torch.uint8, device="cuda")
            max1 = torch.empty(want_max1.size, dtype=torch.float32, device="cuda")
            assert lib.lpmm_quant_group(dx.data_ptr(), 4096, 128, dq.data_ptr(), codes.data_ptr(), max1.data_ptr(), _stream()) == 0
            torch.cuda.synchronize()
            np.testing.assert_array_equal(to_np(codes), want_codes)
            np.testing.assert_array_equal(to_np(max1), want_max1)
