"""Independent restatements used ONLY to pin the C oracle (they share no code with it).

* lane_numpy: the 64 lanes advance together as numpy float32 vectors; every multiply and every add is one
  correctly rounded IEEE binary32 operation (numpy never fuses them).
* lane_python_double: each binary32 operation is done in Python doubles and rounded through struct — for + and x,
  rounding the double result to binary32 equals the correctly rounded binary32 result (53 >= 2*24+2).
* exact_dot_fraction: exact rational arithmetic.
"""
import struct
from fractions import Fraction

import numpy as np


def half_bits_to_float(h):
    return float(np.array([h], dtype=np.uint16).view(np.float16)[0])


def _f32(v):
    return struct.unpack("<f", struct.pack("<f", v))[0]


def nibble(qrow, i):
    return (int(qrow[i >> 3]) >> (4 * (i & 7))) & 0xF


def lane_numpy(qrow, zrow, srow_f32, x_bits, group):
    k = len(x_bits)
    idx = np.arange(k)
    nib = (np.asarray(qrow, dtype=np.uint32)[idx >> 3] >> ((idx & 7) * 4).astype(np.uint32)) & np.uint32(0xF)
    z = np.asarray(zrow, dtype=np.int64)[idx // group]
    sc = np.asarray(srow_f32, dtype=np.float32)[idx // group]
    w = (nib.astype(np.int64) - z).astype(np.float32) * sc
    xf = np.asarray(x_bits, dtype=np.uint16).view(np.float16).astype(np.float32)
    acc = np.zeros(64, np.float32)
    for j in range(k // 64):
        p = w[j * 64:(j + 1) * 64] * xf[j * 64:(j + 1) * 64]
        acc = acc + p
    return acc.astype(np.float64)


def tree_pairwise_halving(v):
    a = [float(t) for t in v]
    width = 32
    while width >= 1:
        a = [a[i] + a[i + width] for i in range(width)]
        width //= 2
    return a[0]


def lane_python_double(qrow, zrow, srow_f32, x_bits, group):
    k = len(x_bits)
    lanes = []
    for l in range(64):
        acc = 0.0
        for i in range(l, k, 64):
            g = i // group
            w = _f32(float(nibble(qrow, i) - int(zrow[g])) * float(srow_f32[g]))
            p = _f32(w * half_bits_to_float(int(x_bits[i])))
            acc = _f32(acc + p)
        lanes.append(acc)
    return lanes


def exact_dot_fraction(qrow, zrow, srow_f32, x_bits, group):
    k = len(x_bits)
    tot = Fraction(0)
    for i in range(k):
        g = i // group
        tot += (nibble(qrow, i) - int(zrow[g])) * Fraction(float(srow_f32[g])) * Fraction(
            half_bits_to_float(int(x_bits[i])))
    return tot


def xorshift64(seed):
    """Generator written out in the reference's lane tests (crates/core/src/quant/lane.rs:101-107, 150-156)."""
    s = seed & 0xFFFFFFFFFFFFFFFF
    while True:
        s ^= (s << 13) & 0xFFFFFFFFFFFFFFFF
        s ^= s >> 7
        s ^= (s << 17) & 0xFFFFFFFFFFFFFFFF
        yield s


def test_to_f16(v):
    """The truncating-exponent half conversion the lane tests use for their inputs (lane.rs:76-96): round half up on
    the mantissa, flush below the normal range to signed zero, saturate to infinity."""
    b = struct.unpack("<I", struct.pack("<f", v))[0]
    sign = (b >> 16) & 0x8000
    exp = ((b >> 23) & 0xFF) - 127 + 15
    man = b & 0x7FFFFF
    if exp <= 0:
        return sign
    if exp >= 31:
        return sign | 0x7C00
    m = (man >> 13) + ((man >> 12) & 1)
    if m & 0x400:
        m &= 0x3FF
        exp += 1
    return sign | (exp << 10) | m


test_to_f16.__test__ = False
