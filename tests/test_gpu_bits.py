"""GPU parity of the any-width (1..8 bit) quantise / dequantise kernels against the CPU oracle,
through the C ABI, the operator shim and the optimizer (lpmm/configs/default_{5,8}b.yml)."""
import os

import numpy as np
import pytest
import torch

from util import assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

BITS = [1, 2, 3, 4, 5, 6, 7, 8]


def _lib():
    from lpmm import _native

    return _native.lib()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _nbytes(n_padded, bits):
    return n_padded * (bits if bits in (1, 2, 4) else 8) // 8 + 1


@pytest.mark.parametrize("bits", BITS)
def test_pack_unpack_bits(oracle, bits):
    lib = _lib()
    rng = np.random.default_rng(bits)
    for signed in (True, False):
        qmap = oracle.create_pow_map(bits, signed, 1)
        mids = oracle.midpoints(qmap)
        n = 2048 * 3 + 8 * 5
        x = rng.uniform(-1.2, 1.2, n).astype(np.float32)
        special = np.concatenate([qmap, mids, np.nextafter(mids, np.float32(2)), [np.nan, np.inf, -np.inf, 0.0, -0.0]])
        x[:special.size] = special[:n]
        want = oracle.pack_nonlinear(x, qmap, bits)
        dq = to_dev(qmap)
        out = torch.full((want.size,), 0x5A, dtype=torch.uint8, device="cuda")
        assert lib.lpmm_pack_nonlinear(to_dev(x).data_ptr(), dq.data_ptr(), bits, n, out.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(out), want)
        back = torch.empty(n, dtype=torch.float32, device="cuda")
        assert lib.lpmm_unpack_nonlinear(out.data_ptr(), dq.data_ptr(), bits, n, back.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(back), oracle.unpack_nonlinear(want, qmap, bits, n))


@pytest.mark.parametrize("kind", ["even", "dynamic", "pow2_signed", "pow3_unsigned"])
@pytest.mark.parametrize("bits", [1, 2, 3, 5, 6, 7, 8])
def test_code_assignment_on_a_dense_sample(oracle, bits, kind):
    """The evenly spaced map without zero takes a closed form instead of the search, other maps
    the descent through the map's entries: every 251st float bit pattern (negative values,
    infinities and NaNs included) and the 17 floats around every midpoint and every entry of the
    map, against the oracle's search."""
    lib = _lib()
    if kind == "even":
        qmap = oracle.create_pow_map(bits, False, 1)
        assert np.array_equal(qmap, (np.arange(1, 2 ** bits + 1) / 2 ** bits).astype(np.float32))
    elif kind == "dynamic":
        if bits < 2:
            pytest.skip("the dynamic-exponent map needs a sign bit and an exponent bit")
        qmap = oracle.create_dynamic_map(True, bits - 1, bits)
    elif kind == "pow2_signed":
        qmap = oracle.create_pow_map(bits, True, 2)
    else:
        qmap = oracle.create_pow_map(bits, False, 3)
    assert qmap.size == 2 ** bits
    mids = oracle.midpoints(qmap)
    sample = np.arange(0, 2 ** 32, 251, dtype=np.uint64).astype(np.uint32)
    near = (np.concatenate([mids, qmap]).view(np.uint32)[:, None].astype(np.int64) + np.arange(-8, 9)[None, :]).reshape(-1)
    bitsx = np.concatenate([sample, near.astype(np.uint32)])
    bitsx = np.concatenate([bitsx, np.zeros((-bitsx.size) % 2048, np.uint32)])
    x = bitsx.view(np.float32)
    want = oracle.pack_nonlinear(x, qmap, bits)
    out = torch.full((want.size,), 0x5A, dtype=torch.uint8, device="cuda")
    assert lib.lpmm_pack_nonlinear(to_dev(x).data_ptr(), to_dev(qmap).data_ptr(), bits, x.size, out.data_ptr(),
                                   _stream()) == 0
    torch.cuda.synchronize()
    got = to_np(out)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, (bits, bad[:5], got[bad[:5]], want[bad[:5]])


@pytest.mark.parametrize("bits", BITS)
@pytest.mark.parametrize("n,gp_sz", [(4097, 128), (2048 * 5 + 3, 512), (50000, 2048), (4096 * 3 + 17, 4096), (100, 128),
                                     (2048 * 4, 128), (2048 * 3 + 128 * 5, 256), (2048 * 7 + 130, 1024)])
def test_quant_dequant_group_bits(oracle, bits, n, gp_sz):
    lib = _lib()
    rng = np.random.default_rng(n + bits)
    for signed in (True, False):
        qmap = oracle.create_pow_map(bits, signed, 2 if bits > 2 else 1)
        x = (rng.standard_normal(n) * 0.1).astype(np.float32)
        x = x if signed else x * x
        if n > 2 * gp_sz:
            x[gp_sz:2 * gp_sz] = 0.0  # an all-zero group: 0/0 -> NaN code, max1 = 0
        want_codes, want_max1 = oracle.quant_group_bits(x, qmap, bits, gp_sz)
        dx, dq = to_dev(x), to_dev(qmap)
        codes = torch.full((want_codes.size,), 0x5A, dtype=torch.uint8, device="cuda")
        max1 = torch.empty(want_max1.size, dtype=torch.float32, device="cuda")
        st = lib.lpmm_quant_group_bits(dx.data_ptr(), n, gp_sz, dq.data_ptr(), bits, codes.data_ptr(), max1.data_ptr(),
                                       _stream())
        assert st == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(max1), want_max1)
        np.testing.assert_array_equal(to_np(codes), want_codes)  # padding and the last byte included
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        st = lib.lpmm_dequant_group_bits(codes.data_ptr(), max1.data_ptr(), dq.data_ptr(), bits, n, gp_sz,
                                         out.data_ptr(), _stream())
        assert st == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(out), oracle.dequant_group_bits(want_codes, want_max1, qmap, bits, n, gp_sz))


@pytest.mark.parametrize("bits", [3, 5, 6, 7, 8])
def test_bucket_table_equals_the_search_on_all_floats(oracle, bits):
    """Maps that qualify are encoded with one table read (sign, exponent and leading mantissa bits
    pick a bucket that holds at most one midpoint) instead of the search: both on the device over
    all 2^32 bit patterns.  The reference's signed dynamic-exponent maps must qualify; a map with a
    repeated entry must not (the search's answer for it depends on more than the midpoints)."""
    lib = _lib()
    dynamic = oracle.create_dynamic_map(True, bits - 1, bits)
    repeated = dynamic.copy()
    repeated[3] = repeated[2]
    cases = [(dynamic, True), (oracle.create_pow_map(bits, True, 2), None), (oracle.create_pow_map(bits, False, 3), None),
             (oracle.create_pow_map(bits, False, 1), None), (repeated, False)]
    for qmap, qualifies in cases:
        assert qmap.size == 2 ** bits
        counts = torch.zeros(3, dtype=torch.int64, device="cuda")
        assert lib.lpmm_selftest_bucket_encoder(to_dev(qmap).data_ptr(), bits, counts.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        tried, wrong, ok = counts.tolist()
        if qualifies is not None:
            assert bool(ok) == qualifies
        assert (tried, wrong) == ((2 ** 32, 0) if ok else (0, 0))


def _code_table(dq, bits):
    from lpmm import _native

    table = torch.full((_native.CODE_TABLE_BYTES // 4,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    assert _lib().lpmm_code_table_build(dq.data_ptr(), bits, table.data_ptr(), _stream()) == 0
    return table


@pytest.mark.parametrize("bits", BITS)
def test_code_table_says_what_the_map_allows(oracle, bits):
    """Last word of a table: bits << 8 | 0 (search), 1 (the evenly spaced map's closed form), 2 (table)."""
    even = oracle.create_pow_map(bits, False, 1)
    cases = [(even, 1)]
    if bits >= 2:
        dynamic = oracle.create_dynamic_map(True, bits - 1, bits)
        repeated = dynamic.copy()
        repeated[1] = repeated[0]
        cases += [(dynamic, 2 if bits >= 3 else 0), (repeated, 0)]
    for qmap, mode in cases:
        table = _code_table(to_dev(qmap), bits)
        torch.cuda.synchronize()
        assert int(table[-1]) == (bits << 8 | mode), (bits, mode, hex(int(table[-1])))
    lib = _lib()
    assert lib.lpmm_code_table_build(to_dev(even).data_ptr(), 9, table.data_ptr(), _stream()) != 0
    assert lib.lpmm_code_table_build(to_dev(even).data_ptr(), bits, table.data_ptr() + 4, _stream()) != 0


@pytest.mark.parametrize("with_table", [False, True])
@pytest.mark.parametrize("bits", [5, 6, 7, 8])
@pytest.mark.parametrize("gp_sz", [128, 512])
def test_quant_group_bits_with_the_dynamic_map(oracle, bits, gp_sz, with_table):
    """Whole tiles through the row-layout kernel with the map of configs/default_{5,6,7,8}b.yml:
    groups whose maximum is 1 hold every entry of the map, every midpoint and the floats next to
    them, so that their quotients are those values exactly; random groups follow."""
    lib = _lib()
    rng = np.random.default_rng(bits * 7 + gp_sz)
    qmap = oracle.create_dynamic_map(True, bits - 1, bits)
    mids = oracle.midpoints(qmap)
    two = np.float32(2)
    special = np.concatenate([qmap, mids, np.nextafter(mids, two), np.nextafter(mids, -two), np.nextafter(qmap, two),
                              np.nextafter(qmap, -two), [0.0, -0.0, 1e-30, -1e-30, 2.0 ** -24, -2.0 ** -24]]).astype(np.float32)
    special = special[np.abs(special) <= 1.0]
    per = gp_sz - 1
    groups = -(-special.size // per)
    head = np.zeros((groups, gp_sz), np.float32)
    head[:, 0] = 1.0
    head[:, 1:].reshape(-1)[:special.size] = special
    n = 2048 * 24 + 136
    x = (rng.standard_t(3, n) * 1e-3).astype(np.float32)
    x[:head.size] = head.reshape(-1)
    assert head.size < n - 4096
    want_codes, want_max1 = oracle.quant_group_bits(x, qmap, bits, gp_sz)
    codes = torch.full((want_codes.size,), 0x5A, dtype=torch.uint8, device="cuda")
    max1 = torch.empty(want_max1.size, dtype=torch.float32, device="cuda")
    dq = to_dev(qmap)
    if with_table:
        table = _code_table(dq, bits)
        assert int(table[-1]) == (bits << 8 | 2)
        st = lib.lpmm_quant_group_bits_table(to_dev(x).data_ptr(), n, gp_sz, dq.data_ptr(), bits, table.data_ptr(),
                                             codes.data_ptr(), max1.data_ptr(), _stream())
    else:
        st = lib.lpmm_quant_group_bits(to_dev(x).data_ptr(), n, gp_sz, dq.data_ptr(), bits, codes.data_ptr(),
                                       max1.data_ptr(), _stream())
    assert st == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(max1), want_max1)
    np.testing.assert_array_equal(to_np(codes), want_codes)


def test_a_table_of_another_width_or_of_a_map_that_does_not_qualify_means_the_search(oracle):
    lib = _lib()
    rng = np.random.default_rng(5)
    n = 2048 * 6
    x = (rng.standard_t(3, n) * 1e-3).astype(np.float32)
    dx = to_dev(x)
    dynamic8 = oracle.create_dynamic_map(True, 7, 8)
    repeated = oracle.create_dynamic_map(True, 5, 6)
    repeated[5] = repeated[4]
    for qmap, bits, table_map, table_bits in [(oracle.create_dynamic_map(True, 5, 6), 6, dynamic8, 8), (repeated, 6, repeated, 6)]:
        want_codes, want_max1 = oracle.quant_group_bits(x, qmap, bits, 128)
        table = _code_table(to_dev(table_map), table_bits)
        codes = torch.full((want_codes.size,), 0x5A, dtype=torch.uint8, device="cuda")
        max1 = torch.empty(want_max1.size, dtype=torch.float32, device="cuda")
        assert lib.lpmm_quant_group_bits_table(dx.data_ptr(), n, 128, to_dev(qmap).data_ptr(), bits, table.data_ptr(),
                                               codes.data_ptr(), max1.data_ptr(), _stream()) == 0
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(codes), want_codes)


def test_width_4_generic_kernels_equal_the_fast_path(oracle, qmaps):
    """The any-width kernels at width 4 and the 4-bit kernels give the same bytes."""
    lib = _lib()
    rng = np.random.default_rng(44)
    n = 2048 * 9 + 77
    for qmap, x in ((qmaps[0], (rng.standard_normal(n) * 0.1).astype(np.float32)),
                    (qmaps[1], (rng.standard_normal(n) ** 2).astype(np.float32))):
        dx, dq = to_dev(x), to_dev(qmap)
        nb = (n + 2047) // 2048 * 1024 + 1
        a = torch.zeros(nb, dtype=torch.uint8, device="cuda")
        b = torch.zeros(nb, dtype=torch.uint8, device="cuda")
        ma = torch.empty((n + 127) // 128, dtype=torch.float32, device="cuda")
        mb = torch.empty_like(ma)
        assert lib.lpmm_quant_group(dx.data_ptr(), n, 128, dq.data_ptr(), a.data_ptr(), ma.data_ptr(), _stream()) == 0
        assert lib.lpmm_quant_group_bits(dx.data_ptr(), n, 128, dq.data_ptr(), 4, b.data_ptr(), mb.data_ptr(),
                                         _stream()) == 0
        torch.cuda.synchronize()
        assert torch.equal(a, b) and torch.equal(ma, mb)


@pytest.mark.parametrize("bits", [2, 3, 5, 8])
@pytest.mark.parametrize("shape", [(64, 80), (33, 1000), (257, 1029), (70, 256), (5, 2176), (130, 128)])
def test_rank1_bits(oracle, bits, shape):
    _rank1_bits_case(oracle, bits, shape, oracle.create_pow_map(bits, False, 1), False)


@pytest.mark.parametrize("with_table", [False, True])
@pytest.mark.parametrize("bits", [5, 8])
@pytest.mark.parametrize("shape", [(70, 256), (5, 2176), (130, 128), (33, 1000)])
def test_rank1_bits_with_the_dynamic_map(oracle, bits, shape, with_table):
    """A signed map under the rank-1 scaling (values of both signs), with and without its code table."""
    _rank1_bits_case(oracle, bits, shape, oracle.create_dynamic_map(True, bits - 1, bits), with_table, signed=True)


def _rank1_bits_case(oracle, bits, shape, qmap, with_table, signed=False):
    lib = _lib()
    r, c = shape
    rng = np.random.default_rng(r + bits)
    x = ((rng.standard_normal(shape) * np.exp(rng.standard_normal((r, 1))) * np.exp(rng.standard_normal((1, c)))) ** 2
         ).astype(np.float32)
    if signed:
        x *= rng.choice([-1.0, 1.0], shape).astype(np.float32)
    x[3, :] = 0.0
    x[:, 7] = 0.0
    x[4, :] *= 1e-25  # a row whose scales lie below the range of the reciprocal-based division
    rowmax, colmax = oracle.rank1_stats(x)
    want = oracle.quant_rank1_bits(x, rowmax, colmax, qmap, bits)
    dx, dq, dr, dc = to_dev(x), to_dev(qmap), to_dev(rowmax), to_dev(colmax)
    codes = torch.full((want.size,), 0x5A, dtype=torch.uint8, device="cuda")
    if with_table:
        table = _code_table(dq, bits)
        st = lib.lpmm_quant_rank1_bits_table(dx.data_ptr(), r, c, dr.data_ptr(), dc.data_ptr(), dq.data_ptr(), bits,
                                             table.data_ptr(), codes.data_ptr(), _stream())
    else:
        st = lib.lpmm_quant_rank1_bits(dx.data_ptr(), r, c, dr.data_ptr(), dc.data_ptr(), dq.data_ptr(), bits,
                                       codes.data_ptr(), _stream())
    assert st == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(codes), want)
    out = torch.empty(shape, dtype=torch.float32, device="cuda")
    st = lib.lpmm_dequant_rank1_bits(codes.data_ptr(), dr.data_ptr(), dc.data_ptr(), dq.data_ptr(), bits, r, c,
                                     out.data_ptr(), _stream())
    assert st == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(to_np(out), oracle.dequant_rank1_bits(want, rowmax, colmax, qmap, bits, r, c))


def test_operator_shim_other_widths(oracle):
    from lpmm.cpp_extension import quantization as ext

    rng = np.random.default_rng(3)
    for bits in (2, 6, 8):
        qmap = oracle.create_pow_map(bits, True, 1)
        x = rng.uniform(-1, 1, (3, 2048)).astype(np.float32)
        packed = ext.pack_nonlinear(to_dev(x), to_dev(qmap), bits, False)
        assert packed.dtype == torch.int8 and packed.numel() == _nbytes(3 * 2048, bits)
        np.testing.assert_array_equal(to_np(packed).view(np.uint8), oracle.pack_nonlinear(x, qmap, bits))
        un = ext.unpack_nonlinear(packed, to_dev(qmap), bits, 3, 2048)
        np.testing.assert_array_equal(to_np(un).reshape(-1), oracle.unpack_nonlinear(to_np(packed).view(np.uint8), qmap, bits, 3 * 2048))
    with pytest.raises(RuntimeError):
        ext.pack_nonlinear(to_dev(x), to_dev(oracle.create_pow_map(4, True, 1)), 9, False)
    with pytest.raises(RuntimeError):
        ext.pack_nonlinear(to_dev(x), to_dev(oracle.create_pow_map(4, True, 1)), 5, False)  # map too short


@pytest.mark.parametrize("bits", [5, 8])
def test_nonfused_optimizer_other_widths(oracle, bits):
    """lpmm.optim.AdamW(fused=False) with the 5- and 8-bit configurations against the oracle's
    staged step; the maps are the ones the optimizer built."""
    import lpmm

    H = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    rng = np.random.default_rng(bits)
    # a ragged matrix and a vector (staged path), a matrix the two-pass kernels take
    shapes = [(96, 160), (11008,), (64, 256)]
    host = [(rng.standard_normal(s) * 0.02).astype(np.float32) for s in shapes]
    params = [torch.nn.Parameter(to_dev(h)) for h in host]
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", f"default_{bits}b.yml")
    opt = lpmm.optim.AdamW(params, fused=False, qconfig=cfg, **H)
    states = [oracle.NonFusedState(s, v_scale_type="rank1", bits=bits) for s in shapes]
    qm = qv = None
    for step in range(1, 4):
        grads = [(rng.standard_normal(s) * 1e-3).astype(np.float32) for s in shapes]
        for p, g in zip(params, grads):
            p.grad = to_dev(g)
        opt.step()
        if qm is None:
            s0 = opt.state[params[0]]
            qm, qv = to_np(s0["exp_avg_qstate"]["qmap"]), to_np(s0["exp_avg_sq_qstate"]["qmap"])
            assert qm.size == 2 ** bits and qv.size == 2 ** bits
        for h, g, st in zip(host, grads, states):
            oracle.nonfused_step(h, g, st, qm, qv, H["lr"], 0.9, 0.999, H["eps"], H["weight_decay"])
    torch.cuda.synchronize()
    for p, h, st, shape in zip(params, host, states, shapes):
        s = opt.state[p]
        n = h.size
        assert s["exp_avg"].dtype == torch.int8 and s["exp_avg"].numel() == (n + 2047) // 2048 * 2048 + 1
        np.testing.assert_array_equal(to_np(s["exp_avg"]).view(np.uint8), st.m[0])
        np.testing.assert_array_equal(to_np(s["exp_avg_qstate"]["overhead"]["max1"]).reshape(-1), st.m[1])
        np.testing.assert_array_equal(to_np(s["exp_avg_sq"]).view(np.uint8), st.v[0])
        assert_rel(to_np(p), h, "p", scale=h)
    with pytest.raises(ValueError, match="4-bit states only"):
        bad = lpmm.optim.AdamW([torch.nn.Parameter(to_dev(host[1]))], fused=True, qconfig=cfg, **H)
        bad.param_groups[0]["params"][0].grad = to_dev(host[1])
        bad.step()
