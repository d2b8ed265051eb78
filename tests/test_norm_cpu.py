"""Pins the oracle's norm_resid (assets/norm.cu:4-48, 97-148) independently of its own text."""
import numpy as np
import pytest

from llm170_amd import gen


def fma_f32(a, b, c):
    """round_f32(a*b + c) for float32 arrays without libm: the product of two f32 is exact in f64; the f64 sum is
    made round-to-odd with the error term of a two-sum, after which the rounding to f32 is the correct single one."""
    a, b, c = (np.asarray(v, np.float32).astype(np.float64) for v in (a, b, c))
    p = a * b
    s = p + c
    bb = s - p
    err = (p - (s - bb)) + (c - bb)  # two-sum: p + c == s + err exactly
    bits = s.view(np.uint64) if s.ndim else np.array(s).view(np.uint64)
    bits = bits.copy()
    inexact = err != 0
    # round to odd: an inexact sum whose last bit is even moves one step towards the true value
    even = (bits & np.uint64(1)) == 0
    towards_larger_magnitude = (err > 0) == (s > 0)
    step = np.where(towards_larger_magnitude, np.uint64(1), np.uint64(0xFFFFFFFFFFFFFFFF))  # +1 / -1 on the bit pattern
    fix = inexact & even
    bits = np.where(fix, bits + step, bits)
    return bits.view(np.float64).astype(np.float32)


def test_fma_helper_against_exact_rationals():
    from fractions import Fraction
    r = np.random.default_rng(5)
    a = r.standard_normal(400).astype(np.float32) * np.float32(3e3)
    b = r.standard_normal(400).astype(np.float32)
    c = (-(a.astype(np.float64) * b.astype(np.float64))).astype(np.float32) * np.float32(1 + 2.0 ** -20)  # cancellation
    got = fma_f32(a, b, c)
    for i in range(400):
        exact = Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(c[i]))
        # correctly rounded f32 of an exact rational: compare against both neighbours
        g = Fraction(float(got[i]))
        lo, hi = np.nextafter(got[i], np.float32(-np.inf)), np.nextafter(got[i], np.float32(np.inf))
        assert abs(exact - g) <= abs(exact - Fraction(float(lo))) and abs(exact - g) <= abs(exact - Fraction(float(hi)))


def norm_resid_numpy(x, nw, ab, w_off, fused=True, tree=True):
    x, ab = np.asarray(x, np.float32), np.asarray(ab, np.float32)
    t, hidden = x.shape
    v = x + ab
    xn = np.empty_like(v)
    for r in range(t):
        part = np.zeros(1024, np.float32)
        for j in range((hidden + 1023) // 1024):
            seg = v[r, j * 1024:(j + 1) * 1024]
            if fused:
                part[:seg.size] = fma_f32(seg, seg, part[:seg.size])
            else:
                part[:seg.size] = part[:seg.size] + seg * seg
        if tree:
            st = 512
            while st > 0:
                part[:st] = part[:st] + part[st:2 * st]
                st >>= 1
            total = part[0]
        else:
            total = np.float32(0)
            for p_ in part:
                total = np.float32(total + p_)
        inv = np.float32(1.0) / np.sqrt(np.float32(total / np.float32(hidden)) + np.float32(1e-6), dtype=np.float32)
        xn[r] = (v[r] * inv) * nw[w_off:w_off + hidden]
    return v, xn


def _inputs(t, hidden, seed):
    x = gen.normal_f32(seed, (t, hidden)) * np.float32(3.0)
    ab = gen.normal_f32(seed + 1, (t, hidden))
    nw = (np.float32(1.0) + gen.normal_f32(seed + 2, (2 * hidden,)) * np.float32(0.1)).astype(np.float32)
    return x, ab, nw


@pytest.mark.parametrize("t,hidden,w_off", [(3, 5120, 0), (2, 2048, 2048), (2, 1000, 7), (1, 8192, 0), (4, 64, 0)])
def test_norm_resid_against_numpy_restatement(orc, t, hidden, w_off):
    x, ab, nw = _inputs(t, hidden, 40 + hidden)
    x_new, xn, xn32, xn16 = orc.norm_resid(x, nw, ab, w_off)
    v, want = norm_resid_numpy(x, nw, ab, w_off)
    assert np.array_equal(x_new.view(np.uint32), v.view(np.uint32))
    assert np.array_equal(xn.view(np.uint32), want.view(np.uint32))
    h = want.astype(np.float16)
    assert np.array_equal(xn16, h.view(np.uint16))
    assert np.array_equal(xn32.view(np.uint32), h.astype(np.float32).view(np.uint32))
    # the formula itself, in float64
    v64 = v.astype(np.float64)
    ref = v64 / np.sqrt((v64 * v64).mean(axis=1, keepdims=True) + 1e-6) * nw[w_off:w_off + hidden].astype(np.float64)
    assert np.all(np.abs(xn - ref) <= 4 * np.spacing(np.abs(ref).astype(np.float32)) + 1e-30)


def test_norm_resid_order_matters(orc):
    """What the restatement fixes is observable: without the fused multiply-add, or with a sequential instead of a
    tree sum, some row's scale changes in the last bits."""
    x, ab, nw = _inputs(64, 5120, 900)
    _, xn, _, _ = orc.norm_resid(x, nw, ab, 0)
    _, unfused = norm_resid_numpy(x, nw, ab, 0, fused=False)
    _, seq = norm_resid_numpy(x, nw, ab, 0, tree=False)
    assert not np.array_equal(xn, unfused)
    assert not np.array_equal(xn, seq)


def test_norm_resid_closed_forms(orc):
    hidden = 2048
    ones = np.ones((2, hidden), np.float32)
    z = np.zeros_like(ones)
    nw = np.full(hidden, 2.0, np.float32)
    x_new, xn, xn32, xn16 = orc.norm_resid(ones, nw, z, 0)
    inv = np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(1e-6), dtype=np.float32)
    assert np.array_equal(x_new, ones) and np.all(xn == np.float32(inv * np.float32(2.0)))
    # a zero row: inv = 1/sqrt(1e-6), output exactly zero; residual: x + ab with ab = -x is exactly zero
    x_new, xn, _, xn16 = orc.norm_resid(ones, nw, -ones, 0)
    assert np.all(x_new == 0) and np.all(xn == 0) and np.all(xn16 == 0)
