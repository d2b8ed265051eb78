"""Writes tests/golden/lane_vectors.json: known-answer data for the W4A16 numeric contract.

Sources of the expected values (nothing here executes or reads the reference):
  * known-answer pairs written out in the reference's own tests — they are data (input, expected output):
      crates/core/src/quant/lane.rs:140-145               half -> f32
      crates/server/src/probes/w4a16/gpu.rs:966-982        f32 -> half edge list
      crates/core/src/matmul/cpu.rs:227-271                dequant rows (word pattern + scales -> closed form)
      crates/core/src/qwen35/stages/moe.rs:135-155         routing
      crates/core/src/quant/lane.rs:185-193                all nibbles 8 => 0.0
  * the two seeded lane tests (lane.rs:98-138 and :147-183): the xorshift64 input generator is spelled out in the
    test text, so the inputs are regenerated here from the stated seeds; the expected output is what THREE separate
    implementations agree on bit-for-bit (C oracle, numpy float32 lanes, Python-double emulation), and for the first
    test it must also satisfy the reference's own assertion (relative distance < 1e-6 from the f64 scalar sum).
  * extra seeded rows at the layer shapes of the benchmark (k = 5120 g128, k = 768 g32), same three-way agreement.

Run from the repo root:  python tests/golden/make_golden.py
"""
import json
import os
import struct
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from llm170_amd import gen  # noqa: E402
from oracle import oracle  # noqa: E402
from tests import independent as ind  # noqa: E402


def f32(v):
    return struct.unpack("<f", struct.pack("<f", v))[0]


def f32_bits(v):
    return struct.unpack("<I", struct.pack("<f", float(v)))[0]


def three_way(qrow, zrow, srow_f32, x, group):
    c_parts = oracle.lane_parts(qrow, zrow, srow_f32, x, group)
    np_parts = ind.lane_numpy(qrow, zrow, srow_f32, x, group)
    py_parts = np.array(ind.lane_python_double(qrow, zrow, srow_f32, x, group))
    assert np.array_equal(c_parts, np_parts), "C oracle vs numpy lanes"
    assert np.array_equal(c_parts, py_parts), "C oracle vs python-double lanes"
    c_out = oracle.dot_row_lane_group(qrow, zrow, srow_f32, x, group)
    tree = np.float32(ind.tree_pairwise_halving(np_parts))
    assert f32_bits(c_out) == f32_bits(tree), "tree64"
    return c_parts, c_out


def lane_test_1():
    """Inputs of w4a16_lane_matches_scalar (lane.rs:98-123)."""
    k = 256
    r = ind.xorshift64(0x9E3779B9)
    q = [next(r) & 0xFFFFFFFF for _ in range(k // 8)]
    z = [next(r) % 16 for _ in range(k // 128)]
    s = [ind.test_to_f16(f32(0.25 + f32(f32(float(next(r) % 100)) / 400.0))) for _ in range(k // 128)]
    x = [ind.test_to_f16(f32(f32(float(next(r) % 2000) / 1000.0) - 1.0)) for _ in range(k)]
    return k, q, z, s, x


def lane_test_2():
    """Inputs of w4a16_lane_g32_bf16_scale (lane.rs:147-167): bf16-truncated scales, group 32."""
    k = 256
    r = ind.xorshift64(0x12345678)
    q = [next(r) & 0xFFFFFFFF for _ in range(k // 8)]
    z = [next(r) % 16 for _ in range(k // 32)]
    s = [f32_bits(f32(0.25 + f32(f32(float(next(r) % 100)) / 400.0))) >> 16 for _ in range(k // 32)]
    x = [ind.test_to_f16(f32(f32(float(next(r) % 2000) / 1000.0) - 1.0)) for _ in range(k)]
    return k, q, z, s, x


def main():
    out = {}
    out["half_to_f32"] = [[0x3C00, f32_bits(1.0)], [0x3800, f32_bits(0.5)], [0xC000, f32_bits(-2.0)]]
    out["f32_to_f16_edges"] = [
        [f32_bits(1.0), 0x3C00], [f32_bits(-2.0), 0xC000], [f32_bits(0.0), 0x0000], [0x80000000, 0x8000],
        [f32_bits(65504.0), 0x7BFF], [f32_bits(65520.0), 0x7C00], [0x7F800000, 0x7C00], [0xFF800000, 0xFC00],
        [0x7FC00000, 0x7E00], [f32_bits(1e-8), 0x0000], [f32_bits(5.9604645e-8), 0x0001],
        [f32_bits(2050.0), 0x6801],
    ]
    out["f32_to_f16_equal_pairs"] = [[f32_bits(2049.0), f32_bits(2048.0)]]

    # cpu.rs:227-248: every word = sum_j j<<4j, scales 1.0 then 0.5 -> out[i] = ((i%8)-8)*sc
    word_up = sum((j & 0xF) << (4 * j) for j in range(8))
    word_dn = sum(((7 - j) & 0xF) << (4 * j) for j in range(8))
    out["dequant_rows"] = [
        {"k": 256, "group": 128, "scale_bf16": 0, "q": [word_up] * 32, "s": [0x3C00, 0x3800],
         "expect": [float(((i % 8) - 8) * (1.0 if i < 128 else 0.5)) for i in range(256)]},
        {"k": 64, "group": 32, "scale_bf16": 1, "q": [word_dn] * 8, "s": [0x3F80, 0x3F80],
         "expect": [float((7 - (i % 8)) - 8) for i in range(64)]},
    ]
    out["routing"] = [
        {"logits": [2.0, 1.0, 0.5, -1.0], "k": 2, "idx": [0, 1], "ratio": float(np.e), "sum": 1.0},
        {"logits": [1.0, 1.0, 1.0], "k": 2, "idx": [0, 1], "ratio": 1.0, "sum": 1.0},
    ]
    out["center"] = {"k": 128, "q": [0x88888888] * 16, "z": [8], "s": [gen.f32_to_f16_bits(0.5).item()],
                     "x": [0x3C00] * 128, "expect_bits": 0}

    k, q, z, s, x = lane_test_1()
    sf = [oracle.half_to_f32(h) for h in s]
    parts, got = three_way(q, z, sf, x, 128)
    want = 0.0
    for i in range(k):
        w = f32(float(ind.nibble(q, i) - z[i // 128]) * sf[i // 128])
        want += f32(w * ind.half_bits_to_float(x[i]))
    rel = abs(float(got) - want) / max(abs(want), 1e-9)
    assert rel < 1e-6, rel  # the reference test's own assertion (lane.rs:133-137)
    assert f32_bits(oracle.dot_row_lane(q, z, s, x)) == f32_bits(got)
    out["lane_test_g128_f16"] = {"k": k, "group": 128, "q": q, "z": z, "s_f16": s, "x": x,
                                 "scalar_f64_sum": want, "expect_bits": f32_bits(got),
                                 "lane_bits": [f32_bits(p) for p in parts]}

    k, q, z, s, x = lane_test_2()
    sf = [oracle.bf16_to_f32(h) for h in s]
    parts, got = three_way(q, z, sf, x, 32)
    out["lane_test_g32_bf16"] = {"k": k, "group": 32, "q": q, "z": z, "s_bf16": s, "x": x,
                                 "expect_bits": f32_bits(got), "lane_bits": [f32_bits(p) for p in parts]}

    rows = []
    for (n, k, group) in [(4, 5120, 128), (4, 768, 32), (2, 2048, 32), (2, 17408, 128)]:
        qm, sm, xm = gen.make_linear(n, k, group, 2)
        for o in range(n):
            sf = gen.f16_bits_to_f32(sm[o])
            z8 = [8] * (k // group)
            for ti in range(2):
                _, got = three_way(qm[o], z8, sf, xm[ti], group)
                rows.append({"n": n, "k": k, "group": group, "row": o, "tok": ti, "expect_bits": f32_bits(got)})
    out["seeded_rows"] = {"generator": "llm170_amd.gen.make_linear(n, k, group, 2) with default seed", "rows": rows}

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lane_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
