"""Pins the stochastic-rounding part of the CPU oracle: the Philox4x32-10 generator against the
known-answer vectors Random123 publishes, cuRAND's state conventions through their invariants,
and quantize_bsearch<true> through the closed form of its acceptance probability.  (The
conventions themselves -- which counter words hold the subsequence, the order the four outputs
of a block are used in, the uniform conversion -- are pinned against PyTorch's device generator
in the GPU tests.)"""
import numpy as np
import pytest

# Random123 kat_vectors, philox4x32 with 10 rounds: (counter, key, expected)
PHILOX_KAT = [
    ([0x00000000] * 4, [0x00000000] * 2, [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(oracle, ctr, key, want):
    assert [int(v) for v in oracle.philox4x32_10(ctr, key)] == want


def test_draws_follow_the_counter_layout(oracle):
    """Output j of (seed, subsequence, offset) is word (offset + j) % 4 of the block with counter
    {(offset + j) / 4 as 64 bits, subsequence as 64 bits} and key {seed lo, seed hi}."""
    seed, sub = 0x0123456789ABCDEF, 0x00000002_00000005
    for offset, j in [(0, 0), (0, 3), (0, 4), (3, 0), (3, 2), (16384, 7), ((1 << 34) + 1, 9)]:
        pos = offset + j
        blk = oracle.philox4x32_10([(pos >> 2) & 0xFFFFFFFF, pos >> 34, sub & 0xFFFFFFFF, sub >> 32],
                                   [seed & 0xFFFFFFFF, seed >> 32])
        assert oracle.philox_draw(seed, sub, offset, j) == int(blk[pos & 3])
        assert oracle.philox_draw(seed, sub, offset, j) == oracle.philox_draw(seed, sub, 0, pos)


def test_uniform_is_in_half_open_unit_interval(oracle):
    u = np.array([oracle.philox_uniform(7, s, 0, j) for s in range(64) for j in range(8)], np.float32)
    assert u.min() > 0.0 and u.max() <= 1.0
    assert abs(u.mean() - 0.5) < 0.05
    # the conversion itself: u32 -> float (to nearest), times 2^-32, plus 2^-33
    d = oracle.philox_draw(7, 3, 0, 5)
    assert oracle.philox_uniform(7, 3, 0, 5) == float(np.float32(np.float32(d) * np.float32(2.0 ** -32))
                                                      + np.float32(2.0 ** -33))


def test_sr_search_acceptance_rule(oracle, qmaps):
    """Between q[lo-1] <= x < q[lo] the code is lo iff proba + noise - 0.5 rounds (to nearest
    even) to a nonzero integer, i.e. iff noise > 1 - proba: probability proba under a uniform
    (0, 1] noise.  Map points and values outside the map are not random at all."""
    for qmap in qmaps:
        q = np.asarray(qmap, np.float32)
        for k in range(16):
            for noise in (2.0 ** -33, 0.25, 0.5, 1.0):
                assert oracle.qmapping_sr(q, float(q[k]), noise) == k
        assert oracle.qmapping_sr(q, float(q[0]) - 1.0, 0.7) == 0
        assert oracle.qmapping_sr(q, float(q[15]) + 1.0, 0.7) == 15
        assert oracle.qmapping_sr(q, float("nan"), 0.7) == -1
        rng = np.random.default_rng(5)
        for _ in range(300):
            lo = int(rng.integers(1, 16))
            a, b = float(q[lo - 1]), float(q[lo])
            x = np.float32(a + (b - a) * rng.uniform(0.02, 0.98))
            proba = float((np.float32(x) - np.float32(a)) / (np.float32(b) - np.float32(a)))
            noise = float(np.float32(rng.uniform(0.001, 1.0)))
            if abs(noise - (1.0 - proba)) < 1e-5:
                continue  # within rounding of the boundary
            assert oracle.qmapping_sr(q, float(x), noise) == (lo if noise > 1.0 - proba else lo - 1)
        # noise = 1/2 makes it round-to-nearest on the linear scale between the two entries
        x = np.float32(q[8] + np.float32(0.75) * (q[9] - q[8]))
        assert oracle.qmapping_sr(q, float(x), 0.5) == 9
        x = np.float32(q[8] + np.float32(0.25) * (q[9] - q[8]))
        assert oracle.qmapping_sr(q, float(x), 0.5) == 8


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 8])
def test_sr_pack_uses_one_subsequence_per_reference_thread(oracle, bits):
    """Value i draws output i % wpt of subsequence i / wpt, wpt = 4 * codes per byte
    (quantization_kernel.cu:437-451, :525-531); the bytes are laid out as by the nearest packer."""
    qmap = np.asarray(oracle.create_pow_map(bits, True, 1), np.float32)
    rng = np.random.default_rng(bits)
    n = 256
    x = rng.uniform(-1.1, 1.1, n).astype(np.float32)
    seed, offset = 0xDEADBEEF12345, 20
    got = oracle.pack_nonlinear_sr(x, qmap, bits, seed, offset)
    per = 8 // bits if bits in (1, 2, 4) else 1
    wpt = 4 * per
    codes = [oracle.qmapping_sr(qmap, float(x[i]), oracle.philox_uniform(seed, i // wpt, offset, i % wpt), bits)
             for i in range(n)]
    mask = (1 << bits) - 1
    if per > 1:
        want = [sum(((codes[b * per + j] & mask) << (j * bits)) for j in range(per)) for b in range(n // per)]
    else:
        want = [c & 0xFF for c in codes]
    assert np.array_equal(got, np.array(want + [0], np.uint8))
    # map points are not random: same bytes as the nearest packer
    pts = np.resize(qmap, n).astype(np.float32)
    assert np.array_equal(oracle.pack_nonlinear_sr(pts, qmap, bits, seed, offset), oracle.pack_nonlinear(pts, qmap, bits))


def test_sr_is_unbiased(oracle, qmaps):
    """E[decode(code)] = x for x inside the map's range: the mean over 4096 independent streams
    is within 4 standard errors of x."""
    q = np.asarray(qmaps[1], np.float32)  # (k+1)/16
    x = np.float32(0.4)  # between 6/16 and 7/16: proba 0.4
    n = 4096
    codes = oracle.pack_nonlinear_sr(np.full(n, x, np.float32), q, 4, 99, 0)
    dec = oracle.unpack_nonlinear(codes, q, 4, n)
    assert set(np.unique(dec)) == {np.float32(0.375), np.float32(0.4375)}
    se = 0.0625 * np.sqrt(0.4 * 0.6 / n)
    assert abs(dec.astype(np.float64).mean() - 0.4) < 4 * se
