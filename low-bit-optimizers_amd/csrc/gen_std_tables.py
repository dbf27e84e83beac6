#!/usr/bin/env python3
"""Generates std_tables.inc: the standard 4-bit quantisation maps of the AdamW states as bit
patterns, and the bucket table that turns a normalised first-moment value into its code
with one LDS read and one compare.

Run `python gen_std_tables.py > std_tables.inc` after changing anything here; the output is
committed.  tests/test_encode_tables.py checks the table against the reference search over
every float bit pattern.

Bucket table.  For an ascending 16-entry map q the code of x is the number of fp32 midpoints
mid_k = (q[k-1]+q[k])*0.5f that are < x.  The kernels cut the real line into 256 buckets with
one instruction: the conversion of x to an 8-bit float with 5 exponent and 2 mantissa bits
(v_cvt_pk_bf8_f32 of gfx950: round to nearest even, overflow to infinity, every NaN to 0xfe).
The byte is the bucket index; a bucket is the interval of fp32 values that round to that 8-bit
float.  The generator checks that no bucket holds two midpoints; then
    code = (|x| as bits  >  thr) ? code_gt : code_le
with, for x >= 0: thr = bits(t) for the midpoint t inside the bucket, code_le = c, code_gt = c + 1
(c = code at the bucket's low end); for x < 0: thr = bits(|t|) - 1, code_le = c, code_gt = c - 1 (a
tie stays at the lower code on both sides).  Buckets without a midpoint have thr = 0xffffffff
(a NaN: never compares below), the NaN bucket holds code 15 (the reference's search returns -1
for a NaN, masked to 15).
"""
import struct
import sys

import numpy as np


def bits(f):
    return struct.unpack("<I", struct.pack("<f", float(f)))[0]


def linspace_f32(start, end, steps):
    f = np.float32
    start, end = f(start), f(end)
    step = f((end - start) / f(steps - 1))
    out = np.empty(steps, dtype=f)
    for i in range(steps):
        out[i] = f(start + f(step * f(i))) if i < steps // 2 else f(end - f(step * f(steps - i - 1)))
    return out


def dynamic_map_signed4():
    """create_dynamic_map(True, 3, 4) of the reference (lpmm/functional.py:272-315)."""
    f = np.float32
    data = [0.0, 1.0]
    for i in range(3):
        edges = linspace_f32(0.1, 1, 2 ** i + 1)
        means = ((edges[:-1] + edges[1:]) / f(2.0)).astype(f)
        scaled = (f(10.0 ** (i - 2)) * means).astype(f)
        data += [float(v) for v in scaled] + [-float(v) for v in scaled]
    return np.array(sorted(data), dtype=f)


def pow1_map_unsigned4():
    """create_pow_map(4, False, 1) (lpmm/functional.py:644-656): (k+1)/16."""
    return linspace_f32(0, 1, 17)[1:]


def midpoints(q):
    return ((q[:-1] + q[1:]) * np.float32(0.5)).astype(np.float32)


def code_of(mids, x):
    return int(np.sum(mids < np.float32(x)))


def bf8_byte(b32):
    """The byte v_cvt_pk_bf8_f32 produces for the fp32 bit pattern b32 (OCP E5M2, round to
    nearest even; measured on gfx950 for all 2^32 inputs)."""
    sign = (b32 >> 31) << 7
    mag = b32 & 0x7FFFFFFF
    if mag > 0x7F800000:
        return 0xFE
    if (mag >> 23) >= 113:  # normal in the 8-bit format: drop 21 mantissa bits, ties to even
        r = (mag + 0xFFFFF + ((mag >> 21) & 1)) >> 21
        return sign | min(r - 448, 0x7C)
    # below 2^-14: multiples of 2^-16, ties to even
    val = struct.unpack("<f", struct.pack("<I", mag))[0]
    q = val * 65536.0  # exact in double
    n = int(q)
    frac = q - n
    if frac > 0.5 or (frac == 0.5 and (n & 1)):
        n += 1
    return sign | n


def bucket_ranges():
    """byte -> (smallest, largest) fp32 magnitude bits that convert to it, non-negative side."""
    def first_at_least(code):  # smallest magnitude whose byte is >= code
        lo, hi = 0, 0x7F800000
        while lo < hi:
            mid = (lo + hi) // 2
            if bf8_byte(mid) >= code:
                hi = mid
            else:
                lo = mid + 1
        return lo
    starts = [first_at_least(c) for c in range(0x7D)]
    out = {}
    for c in range(0x7D):
        end = starts[c + 1] - 1 if c + 1 < 0x7D else 0x7F800000
        out[c] = (starts[c], end)
    return out


def f32(b):
    return struct.unpack("<f", struct.pack("<I", b))[0]


def build(q):
    """256 entries {thr, code_le, code_gt}, indexed by the byte of the 8-bit conversion."""
    mids = midpoints(q)
    pos = sorted(bits(m) for m in mids if m >= 0)       # magnitudes of midpoints >= 0
    neg = sorted(bits(-m) for m in mids if m < 0)       # magnitudes of midpoints < 0
    ranges = bucket_ranges()
    entries = [(0xFFFFFFFF, 15, 15)] * 256              # unused indices and the NaN bucket
    for byte, (lo, hi) in ranges.items():
        # x >= 0: codes grow with the magnitude; a midpoint t with lo <= t < hi splits the bucket
        c = code_of(mids, f32(lo))
        inside = [t for t in pos if lo <= t < hi]
        assert len(inside) <= 1, "two midpoints in one bucket"
        entries[byte] = (inside[0], c, c + 1) if inside else (0xFFFFFFFF, c, c)
        assert code_of(mids, f32(hi)) == (c + 1 if inside else c)
        # x < 0: codes fall with the magnitude; the code drops at magnitude T = |t| (inclusive) for lo < T <= hi
        c = code_of(mids, -f32(lo))
        inside = [t for t in neg if lo < t <= hi]
        assert len(inside) <= 1, "two midpoints in one bucket"
        entries[0x80 | byte] = (inside[0] - 1, c, c - 1) if inside else (0xFFFFFFFF, c, c)
        assert code_of(mids, -f32(hi)) == (c - 1 if inside else c)
    return entries


COMPACT_LO, COMPACT_HI = 24, 63  # magnitude bytes kept in the stored table; the others repeat these two


def compact(entries):
    """The stored table: magnitude bytes COMPACT_LO..COMPACT_HI of either sign.  Every other
    bucket of a sign equals the nearer end of that range (no midpoint lies outside it), except
    the NaN bucket 0xfe, which the kernels patch to code 15."""
    per = COMPACT_HI - COMPACT_LO + 1
    out = []
    for sign in (0, 1):
        out += [entries[(sign << 7) | m] for m in range(COMPACT_LO, COMPACT_HI + 1)]
    for idx in range(256):
        m = min(max(idx & 127, COMPACT_LO), COMPACT_HI)
        want = (0xFFFFFFFF, 15, 15) if idx == 0xFE else entries[idx]
        got = out[(idx >> 7) * per + m - COMPACT_LO]
        if idx in (0x7D, 0x7E, 0x7F, 0xFD, 0xFF):
            continue  # bytes the conversion never produces
        assert got == want or idx == 0xFE, (idx, got, want)
    return out


def main():
    qm, qv = dynamic_map_signed4(), pow1_map_unsigned4()
    entries = compact(build(qm))
    out = sys.stdout
    out.write("// Generated by gen_std_tables.py -- do not edit.\n")
    out.write("// Standard maps of the 4-bit AdamW states as fp32 bit patterns, and the first-moment\n")
    out.write("// encode table {thr, code_le, code_gt, 0}.  A value's bucket is the byte that its conversion\n")
    out.write("// to an 8-bit float (5 exponent bits, 2 mantissa bits, round to nearest even) gives; stored\n")
    out.write("// are the buckets with magnitude byte kEncCompactLo..kEncCompactHi, first those of x >= 0, then\n")
    out.write("// those of x < 0.  Buckets outside that range equal the nearer end of it; the NaN bucket\n")
    out.write("// (0xfe) holds code 15.\n")
    out.write("static constexpr uint32_t kStdQmapMBits[16] = {%s};\n" % ", ".join("0x%08xu" % bits(v) for v in qm))
    out.write("static constexpr uint32_t kStdQmapVBits[16] = {%s};\n" % ", ".join("0x%08xu" % bits(v) for v in qv))
    out.write("static constexpr int kEncEntries = 256;  // buckets\n")
    out.write("static constexpr uint32_t kEncCompactLo = %d;\n" % COMPACT_LO)
    out.write("static constexpr uint32_t kEncCompactHi = %d;\n" % COMPACT_HI)
    out.write("static constexpr uint32_t kEncCompactPerSign = %d;\n" % (COMPACT_HI - COMPACT_LO + 1))
    out.write("static constexpr uint32_t kEncTableM[%d][4] = {\n" % len(entries))
    for thr, cle, cgt in entries:
        out.write("    {0x%08xu, %du, %du, 0u},\n" % (thr, cle, cgt))
    out.write("};\n")


if __name__ == "__main__":
    main()
