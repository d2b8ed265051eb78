"""Pins the CPU oracle (oracle/lane_oracle.c) against the reference's known answers and against independent
restatements.  CPU only."""
import json
import os
import struct
from fractions import Fraction

import numpy as np
import pytest

from llm170_amd import gen
from tests import independent as ind

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "lane_vectors.json")))


def bits(v):
    return struct.unpack("<I", struct.pack("<f", float(v)))[0]


def from_bits(b):
    return struct.unpack("<f", struct.pack("<I", b))[0]


# ---------------------------------------------------------------- casts
def test_half_to_f32_kats(orc):
    for h, want in GOLD["half_to_f32"]:
        assert bits(orc.half_to_f32(h)) == want


def test_half_to_f32_all_patterns_match_ieee(orc):
    got = orc.half_to_f32_bits_all()
    want = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16).astype(np.float32).view(np.uint32)
    nan = (np.arange(65536) & 0x7C00 == 0x7C00) & (np.arange(65536) & 0x3FF != 0)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN: payload shifted into the f32 mantissa (deq.rs:23); numpy additionally quiets it
    h = np.arange(65536)[nan]
    assert np.array_equal(got[nan], ((h >> 15) << 31 | 0xFF << 23 | (h & 0x3FF) << 13).astype(np.uint32))


def test_f32_to_f16_edges(orc):
    for fb, want in GOLD["f32_to_f16_edges"]:
        assert orc.f32_to_f16(from_bits(fb)) == want, hex(fb)
    for a, b in GOLD["f32_to_f16_equal_pairs"]:
        assert orc.f32_to_f16(from_bits(a)) == orc.f32_to_f16(from_bits(b))


def test_f32_to_f16_roundtrips_all_non_nan(orc):
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    keep = ~((h & 0x7C00 == 0x7C00) & (h & 0x3FF != 0))
    v = h.view(np.float16).astype(np.float32)
    back = orc.f32_to_f16_array(v[keep])
    assert np.array_equal(back, h[keep])


def test_f32_to_f16_is_rne_on_random_floats(orc):
    r = gen.stream(7, 200000)
    f = (r & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    # keep exponents inside and just around the half range so ties/subnormals/overflow are all hit
    e = (f >> 23) & 0xFF
    f = (f & ~np.uint32(0xFF << 23)) | (((e % 48) + 127 - 28).astype(np.uint32) << 23)
    v = f.view(np.float32)
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f32_to_f16_array(v), want)
    # exact ties: halfway between adjacent halves must go to the even one
    for hb in (0x3C00, 0x3C01, 0x0001, 0x0002, 0x03FF, 0x7BFE):
        lo = float(np.array([hb], np.uint16).view(np.float16)[0])
        hi = float(np.array([hb + 1], np.uint16).view(np.float16)[0])
        mid = np.float32((lo + hi) / 2)
        assert float(mid) == (lo + hi) / 2
        assert orc.f32_to_f16(mid) == (hb if hb % 2 == 0 else hb + 1)


def test_bf16_to_f32(orc):
    assert orc.bf16_to_f32(0x3F80) == 1.0
    assert bits(orc.bf16_to_f32(0xC049)) == 0xC0490000


# ---------------------------------------------------------------- dequant
def test_dequant_rows_known_answers(orc):
    for row in GOLD["dequant_rows"]:
        q = np.array(row["q"], np.uint32).view(np.uint8)
        s = np.array(row["s"], np.uint16).view(np.uint8)
        out = orc.dequant_row_split(q, s, 0, row["k"], row["group"], row["scale_bf16"])
        assert np.array_equal(out, np.array(row["expect"], np.float32))


def test_dequant_matches_numpy_unpack_times_scale(orc):
    for (n, k, g) in [(8, 512, 128), (8, 256, 32)]:
        q, s, _ = gen.make_linear(n, k, g, 1)
        want = gen.unpack_nibbles(q, k).astype(np.float32) * np.repeat(gen.f16_bits_to_f32(s), g, axis=1)
        got = orc.dequant_matrix(q, s, n, k, g)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        assert np.array_equal(gen.pack_nibbles(gen.unpack_nibbles(q, k)), q)


def test_pack_order_matches_fixture_packer():
    # scripts/gen_tiny_w4a16.py:44-48: element i of a row -> bits 4*(i&7) of word i>>3, stored value+8
    vals = (np.arange(16).reshape(1, 16) % 16) - 8
    q = gen.pack_nibbles(vals)
    assert q[0, 0] == 0x76543210 and q[0, 1] == 0xFEDCBA98


# ---------------------------------------------------------------- lane order
def test_center_is_zero(orc):
    c = GOLD["center"]
    assert bits(orc.dot_row_lane(c["q"], c["z"], c["s"], c["x"])) == c["expect_bits"]


def test_reference_lane_tests(orc):
    t1 = GOLD["lane_test_g128_f16"]
    got = orc.dot_row_lane(t1["q"], t1["z"], t1["s_f16"], t1["x"])
    assert bits(got) == t1["expect_bits"]
    rel = abs(float(got) - t1["scalar_f64_sum"]) / max(abs(t1["scalar_f64_sum"]), 1e-9)
    assert rel < 1e-6  # assertion of lane.rs:133-137
    sf = [orc.half_to_f32(h) for h in t1["s_f16"]]
    parts = orc.lane_parts(t1["q"], t1["z"], sf, t1["x"], 128)
    assert [bits(p) for p in parts] == t1["lane_bits"]

    t2 = GOLD["lane_test_g32_bf16"]
    sf = [orc.bf16_to_f32(h) for h in t2["s_bf16"]]
    got = orc.dot_row_lane_group(t2["q"], t2["z"], sf, t2["x"], 32)
    assert bits(got) == t2["expect_bits"]
    assert [bits(p) for p in orc.lane_parts(t2["q"], t2["z"], sf, t2["x"], 32)] == t2["lane_bits"]


def test_seeded_rows_match_golden(orc):
    cache = {}
    for r in GOLD["seeded_rows"]["rows"]:
        key = (r["n"], r["k"], r["group"])
        if key not in cache:
            cache[key] = gen.make_linear(r["n"], r["k"], r["group"], 2)
        q, s, x = cache[key]
        sf = gen.f16_bits_to_f32(s[r["row"]])
        got = orc.dot_row_lane_group(q[r["row"]], [8] * (r["k"] // r["group"]), sf, x[r["tok"]], r["group"])
        assert bits(got) == r["expect_bits"]


def test_lane_matches_independent_emulations(orc):
    for seed, (k, g) in enumerate([(128, 128), (256, 32), (1024, 128), (768, 32), (640, 64)]):
        q, s, x = gen.make_linear(1, k, g, 1, seed=seed + 11)
        z = (gen.stream(seed, k // g) % np.uint64(16)).astype(np.uint32)
        sf = gen.f16_bits_to_f32(s[0])
        c = orc.lane_parts(q[0], z, sf, x[0], g)
        assert np.array_equal(c, ind.lane_numpy(q[0], z, sf, x[0], g))
        assert np.array_equal(c, np.array(ind.lane_python_double(q[0], z, sf, x[0], g)))


def test_lane_is_not_fused_and_not_sequential(orc):
    """A fused multiply-add, or summing in index order, gives different bits on ordinary inputs — so agreement with
    the emulations above is not vacuous."""
    k, g = 2048, 128
    differs_fma = differs_seq = 0
    for seed in range(20):
        q, s, x = gen.make_linear(1, k, g, 1, seed=1000 + seed)
        sf = gen.f16_bits_to_f32(s[0])
        z8 = [8] * (k // g)
        got = orc.dot_row_lane_group(q[0], z8, sf, x[0], g)
        w = gen.unpack_nibbles(q, k)[0].astype(np.float32) * np.repeat(sf, g)
        xf = gen.f16_bits_to_f32(x[0])
        lanes = []
        for l in range(64):
            acc = 0.0
            for i in range(l, k, 64):
                acc = ind._f32(acc + float(w[i]) * float(xf[i]))  # single rounding = fused
            lanes.append(acc)
        fused = np.float32(ind.tree_pairwise_halving(lanes))
        seq = np.float32(0)
        for i in range(k):
            seq = seq + w[i] * xf[i]
        differs_fma += bits(fused) != bits(got)
        differs_seq += bits(seq) != bits(got)
    assert differs_fma > 0 and differs_seq > 0


def test_dot_against_exact_rational(orc):
    for seed, (k, g) in enumerate([(256, 128), (256, 32), (512, 64)]):
        q, s, x = gen.make_linear(1, k, g, 1, seed=seed + 99)
        sf = gen.f16_bits_to_f32(s[0])
        z8 = [8] * (k // g)
        exact = ind.exact_dot_fraction(q[0], z8, sf, x[0], g)
        got = orc.dot_row_lane_group(q[0], z8, sf, x[0], g)
        scale = sum(abs(Fraction(float(a))) for a in (gen.unpack_nibbles(q, k)[0].astype(np.float32) * np.repeat(sf, g) *
                                                       gen.f16_bits_to_f32(x[0])))
        assert abs(Fraction(float(got)) - exact) <= scale * Fraction(1, 2 ** 20)
        # Neumaier f64 dot (exact.rs:27-53) is within a few f64 ulps of the rational value
        e = orc.exact_dot(q[0].view(np.uint8), s[0].view(np.uint8), gen.f16_bits_to_f32(x[0]), k, g, False)
        assert abs(Fraction(e) - exact) <= abs(exact) * Fraction(1, 2 ** 48) + Fraction(1, 2 ** 60)


def test_closed_form_integer_sum(orc):
    """Scales 1.0 and x 1.0 => exactly sum(nibble - 8) (closed form of probe.rs:1293-1308)."""
    k = 4096
    q = gen.weights_q(5, 3, k)
    for o in range(3):
        got = orc.dot_row_lane(q[o], [8] * (k // 128), [0x3C00] * (k // 128), [0x3C00] * k)
        assert float(got) == float(gen.unpack_nibbles(q, k)[o].astype(np.int64).sum())


def test_power_of_two_scales_are_exact(orc):
    """Power-of-two scales and activations: every product and partial sum is exact, so the result equals the f64
    sum (closed form used by the reference's self-check, gpu/bench.rs:81-114)."""
    k, g = 1024, 32
    q = gen.weights_q(6, 2, k)
    e = (gen.stream(8, k // g) % np.uint64(5)).astype(np.int64)
    s = gen.f32_to_f16_bits(np.ldexp(1.0, -e).astype(np.float32))
    xe = (gen.stream(9, k) % np.uint64(4)).astype(np.int64)
    xs = np.where(gen.stream(10, k) & np.uint64(1), 1.0, -1.0)
    x = gen.f32_to_f16_bits((xs * np.ldexp(1.0, -xe)).astype(np.float32))
    for o in range(2):
        want = float((gen.unpack_nibbles(q, k)[o].astype(np.float64) * np.repeat(np.ldexp(1.0, -e), g) *
                      gen.f16_bits_to_f32(x).astype(np.float64)).sum())
        got = orc.dot_row_lane_group(q[o], [8] * (k // g), gen.f16_bits_to_f32(s), x, g)
        assert float(got) == want


# ---------------------------------------------------------------- tree64
def test_tree64_exact_when_exactly_summable(orc):
    import math
    v = (gen.stream(3, 64) >> np.uint64(40)).astype(np.float64) - 2.0 ** 23
    assert orc.tree64(v) == math.fsum(v)


def test_tree64_pairing_order(orc):
    v = np.ldexp((gen.stream(4, 64) >> np.uint64(11)).astype(np.float64), -(gen.stream(5, 64) % np.uint64(90)).astype(int))
    v *= np.where(gen.stream(6, 64) & np.uint64(1), 1.0, -1.0)
    assert orc.tree64(v) == ind.tree_pairwise_halving(v)
    seq = 0.0
    for t in v:
        seq += float(t)
    adjacent = [float(t) for t in v]
    while len(adjacent) > 1:
        adjacent = [adjacent[2 * i] + adjacent[2 * i + 1] for i in range(len(adjacent) // 2)]
    assert orc.tree64(v) != seq or orc.tree64(v) != adjacent[0]


# ---------------------------------------------------------------- shape contract
def test_lane_shape_contract(orc):
    q, s, x = gen.make_linear(1, 256, 128, 1)
    sf = gen.f16_bits_to_f32(s[0])
    with pytest.raises(ValueError):
        orc.dot_row_lane_group(q[0][:-1], [8, 8], sf, x[0], 128)  # |qrow| != k/8
    with pytest.raises(ValueError):
        orc.dot_row_lane_group(q[0], [8], sf, x[0], 128)  # |zrow| != k/group
    with pytest.raises(ValueError):
        orc.dot_row_lane_group(q[0], [8] * 16, np.ones(16, np.float32), x[0], 16)  # group < 32
    with pytest.raises(ValueError):
        orc.dot_row_lane_group(q[0], [8] * 2, sf, x[0], 96)  # k % group


# ---------------------------------------------------------------- gemm
def test_gemm_lane_threads_and_sampling_agree(orc):
    n, k, g, t = 24, 512, 128, 3
    q, s, x = gen.make_linear(n, k, g, t)
    a = orc.gemm_lane(x, t, q, s, n, k, g, threads=1)
    b = orc.gemm_lane(x, t, q, s, n, k, g, threads=5)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    rows = np.array([0, 5, 23, 7], np.uint32)
    toks = np.array([2, 0, 1, 1], np.uint32)
    smp = orc.gemm_lane_sample(x, q, s, k, g, rows, toks)
    assert np.array_equal(smp.view(np.uint32), a[toks, rows].view(np.uint32))
    for o in (0, 23):
        want = orc.dot_row_lane_group(q[o], [8] * (k // g), gen.f16_bits_to_f32(s[o]), x[1], g)
        assert bits(a[1, o]) == bits(want)


# ---------------------------------------------------------------- routing
def test_routing_known_answers(orc):
    for r in GOLD["routing"]:
        idx, w = orc.moe_topk(r["logits"], r["k"])
        assert list(idx) == r["idx"]
        assert abs(float(w.sum()) - r["sum"]) < 1e-6
        assert abs(float(w[0] / w[1]) - r["ratio"]) < 1e-4
        assert w[0] >= w[1]


def test_routing_matches_numpy_softmax_topk(orc):
    lg = gen.normal_f32(21, (16, 128))
    for row in lg:
        idx, w = orc.moe_topk(row, 8)
        p = np.exp(row.astype(np.float64) - row.max())
        p /= p.sum()
        order = sorted(range(128), key=lambda e: (-p[e], e))[:8]
        assert list(idx) == order
        assert np.allclose(w, p[order] / p[order].sum(), rtol=1e-5)
