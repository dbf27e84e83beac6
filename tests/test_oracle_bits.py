"""Pins the any-width (1..8 bit) pack / unpack / quantise functions of the CPU oracle:
against a bit-by-bit Python restatement of the reference's storage rule, against the 4-bit
functions at width 4, and through round trips and closed forms."""
import numpy as np
import pytest


def _maps(oracle, bits):
    """A signed and an unsigned ascending map of 2^bits entries."""
    return oracle.create_pow_map(bits, True, 1), oracle.create_pow_map(bits, False, 1)


def _py_search(qmap, bits, x):
    """quantization_kernel.cu:397-427 line by line in Python floats-as-float32."""
    f = np.float32
    lo, hi = 0, 1 << bits
    if x <= qmap[lo]:
        return lo
    if qmap[hi - 1] <= x:
        return hi - 1
    while lo < hi:
        mi = (lo + hi) >> 1
        if qmap[mi] <= x:
            lo = mi + 1
        else:
            hi = mi
    if lo == 0:
        return -1
    mid = f(f(qmap[lo - 1] + qmap[lo]) * f(0.5))
    return lo if mid < x else lo - 1


def _py_pack(x, qmap, bits):
    codes = [_py_search(qmap, bits, v) for v in x]
    if bits in (1, 2, 4):
        per, mask = 8 // bits, (1 << bits) - 1
        out = [sum(((codes[b * per + j] & mask) << (j * bits)) for j in range(per)) for b in range(len(x) // per)]
    else:
        out = [c & 0xFF for c in codes]
    return np.array(out + [0], dtype=np.uint8)


@pytest.mark.parametrize("bits", range(1, 9))
def test_pack_matches_bitwise_restatement(oracle, bits):
    rng = np.random.default_rng(bits)
    for qmap in _maps(oracle, bits):
        x = np.concatenate([rng.uniform(-1.3, 1.3, 200), qmap, oracle.midpoints(qmap),
                            np.nextafter(oracle.midpoints(qmap), np.float32(2)), [0.0, -0.0, np.nan, np.inf, -np.inf]])
        x = np.resize(x.astype(np.float32), (x.size + 7) // 8 * 8)
        got = oracle.pack_nonlinear(x, qmap, bits)
        np.testing.assert_array_equal(got, _py_pack(x, qmap, bits))
        assert got.size == x.size * (bits if bits in (1, 2, 4) else 8) // 8 + 1


@pytest.mark.parametrize("bits", range(1, 9))
def test_search_equals_midpoint_count_on_ascending_maps(oracle, bits):
    rng = np.random.default_rng(100 + bits)
    for qmap in _maps(oracle, bits):
        mids = oracle.midpoints(qmap)
        x = np.concatenate([rng.uniform(-1.2, 1.2, 500).astype(np.float32), qmap, mids,
                            np.nextafter(mids, np.float32(-2)), np.nextafter(mids, np.float32(2))])
        want = (mids[None, :] < x[:, None]).sum(axis=1)
        got = np.array([oracle.qmapping_scalar(qmap, v, bits) for v in x])
        np.testing.assert_array_equal(got, want)
        assert oracle.qmapping_scalar(qmap, np.nan, bits) == -1


def test_search_with_repeated_entries(oracle):
    """The 'nonlinear-nozero' unsigned maps repeat their first entry (functional.py:254-256):
    the upper-bound search still returns the reference's answer, which the midpoint count
    would not (x equal to the repeated value)."""
    qmap = oracle.create_pow_map(3, False, 1).copy()
    qmap[0] = qmap[1]
    for x in (qmap[0], np.nextafter(qmap[0], np.float32(2)), np.float32(0.0), np.float32(0.3)):
        assert oracle.qmapping_scalar(qmap, x, 3) == _py_search(qmap, 3, x)
    assert oracle.qmapping_scalar(qmap, qmap[0], 3) == 0  # x <= qmap[0] returns first


@pytest.mark.parametrize("bits", range(1, 9))
def test_round_trip_and_nan_codes(oracle, bits):
    for qmap in _maps(oracle, bits):
        reps = np.resize(qmap, (qmap.size + 7) // 8 * 8)
        codes = oracle.pack_nonlinear(reps, qmap, bits)
        np.testing.assert_array_equal(oracle.unpack_nonlinear(codes, qmap, bits, reps.size), reps)
        nan = oracle.pack_nonlinear(np.full(8, np.nan, np.float32), qmap, bits)
        assert np.all(nan[:-1] == 0xFF) and nan[-1] == 0  # all-ones code / (uint8_t)-1
        np.testing.assert_array_equal(oracle.unpack_nonlinear(nan, qmap, bits, 8), np.full(8, qmap[-1]))


def test_width_4_equals_the_4bit_functions(oracle, qmaps):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(128 * 37 + 5) * 0.1).astype(np.float32)
    x[256:384] = 0.0
    for qmap, data in ((qmaps[0], x), (qmaps[1], x * x)):
        c4, m4 = oracle.quant_group(data, qmap)
        cb, mb = oracle.quant_group_bits(data, qmap, 4)
        np.testing.assert_array_equal(c4, cb)
        np.testing.assert_array_equal(m4, mb)
        np.testing.assert_array_equal(oracle.dequant_group(c4, m4, qmap, data.size),
                                      oracle.dequant_group_bits(cb, mb, qmap, 4, data.size))
    v = (x[:128 * 36] ** 2).reshape(36, 128)
    v[5, :] = 0.0
    rm, cm = oracle.rank1_stats(v)
    c4 = oracle.quant_rank1(v, rm, cm, qmaps[1])
    np.testing.assert_array_equal(c4, oracle.quant_rank1_bits(v, rm, cm, qmaps[1], 4))
    np.testing.assert_array_equal(oracle.dequant_rank1(c4, rm, cm, qmaps[1], 36, 128),
                                  oracle.dequant_rank1_bits(c4, rm, cm, qmaps[1], 4, 36, 128))


@pytest.mark.parametrize("bits", [3, 5, 8])
def test_group_quantisation_properties(oracle, bits):
    """Closed forms that hold for any width: the element of largest magnitude of a group gets
    the last (or first) code and decodes to +-scale * |q|; the error of every element is at
    most half the widest cell times the scale; an all-zero group stores NaN codes, scale 0."""
    rng = np.random.default_rng(bits)
    qmap = oracle.create_pow_map(bits, True, 1)
    x = (rng.standard_normal(128 * 9) * 0.3).astype(np.float32)
    x[128:256] = 0.0
    codes, max1 = oracle.quant_group_bits(x, qmap, bits)
    assert codes.size == 2048 + 1 and max1[1] == 0.0 and np.all(codes[128:256] == 0xFF)
    back = oracle.dequant_group_bits(codes, max1, qmap, bits, x.size)
    cell = np.max(np.diff(qmap))
    scale = np.repeat(max1, 128)
    assert np.all(np.abs(back - x) <= 0.5 * cell * scale * (1 + 1e-6) + 1e-12)
    for g in (0, 2, 5):
        i = g * 128 + int(np.argmax(np.abs(x[g * 128:(g + 1) * 128])))
        assert codes[i] == (2 ** bits - 1 if x[i] > 0 else 0)
    assert np.all(codes[128 * 9:2048] == oracle.qmapping_scalar(qmap, 0.0, bits))  # padding: code of a plain 0.0
