"""Launch plans of the decode and prefill paths as pure functions (w4a16_plan_decode, w4a16_plan_prefill): no GPU.

The prefill planner is a price model with constants fitted to measurements; the table of those measurements that is
kept under profiles/ names, per layer shape, the (tile, k slices) that measured fastest.  This test feeds the planner
the same shapes and requires its choice to be that winner or a row the table shows within 3 % of it (the same plan's
time moves by 2-3 % between boxes, so closer rows trade places from one sweep to the next), so that a change to the
kernel or the constants that moves a plan shows up here."""
import os
import re

import pytest

from llm170_amd import ffi, ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SWEEP = os.path.join(ROOT, "profiles", "prefill_plan_sweep.md")


def sweep_rows():
    """Rows `| n | k | t | tile | slices | us |` of the committed sweep table."""
    rows = []
    for ln in open(SWEEP):
        m = re.match(r"^\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*([0-9.]+)\s*\|", ln)
        if m:
            rows.append(tuple(int(m.group(i)) for i in range(1, 6)) + (float(m.group(6)),))
    return rows


def test_prefill_plan_is_the_sweeps_winner_at_the_layer_shapes():
    rows = sweep_rows()
    shapes = sorted(set(r[:3] for r in rows))
    assert {(34816, 5120, 512), (34816, 5120, 1024), (34816, 5120, 4096), (5120, 17408, 512), (5120, 17408, 1024),
            (5120, 17408, 4096)} <= set(shapes)
    for (n, k, t) in shapes:
        cand = {(r[3], r[4]): r[5] for r in rows if r[:3] == (n, k, t)}
        best = min(cand.values())
        p = ops.plan_prefill(t, n, k, cu_count=256)
        pick = (p["tile_rows"], p["k_slices"])
        assert pick in cand, ("the sweep has no row for the planner's choice", n, k, t, pick)
        assert cand[pick] <= 1.03 * best, (n, k, t, pick, cand[pick], best)


def test_prefill_plan_super_tiles_cover_the_grid_and_pins_are_honoured():
    for (t, n, k) in [(4096, 34816, 5120), (1280, 5120, 17408), (100, 7168, 5120), (65, 256, 512)]:
        p = ops.plan_prefill(t, n, k)
        tiles_m, tiles_n = -(-t // p["tile_rows"]), -(-n // 256)
        sm, sn = -(-tiles_m // p["super_m"]), -(-tiles_n // p["super_n"])
        assert p["supers"] == sm * sn and 1 <= p["super_m"] <= 8 and p["super_n"] in (1, 2, 4, 8)
        assert p["k_slices"] == 1 or p["k_slices"] <= (k // 128) // 4
    assert ops.plan_prefill(4096, 34816, 5120, tile_rows=64)["tile_rows"] == 64
    assert ops.plan_prefill(4096, 34816, 5120, tile_rows=96)["tile_rows"] == 96
    assert ops.plan_prefill(4096, 34816, 5120, k_slices=-1)["k_slices"] == 1
    assert ops.plan_prefill(512, 5120, 17408, k_slices=4)["k_slices"] == 4
    with pytest.raises(ops.W4a16Error):
        ops.plan_prefill(512, 5120, 17408, tile_rows=100)


def test_decode_plan_at_the_layer_shapes():
    """The shapes the launch-shape sweeps settled on (27B dense layer, group 128, 256 CUs)."""
    gate_up, down, qkv, o = (34816, 5120), (5120, 17408), (7168, 5120), (5120, 5120)
    want = {  # (n, k, t) -> (rows per wave, waves, k slices)
        gate_up + (1,): (16, 4, 1), gate_up + (4,): (32, 4, 1), gate_up + (16,): (64, 4, 1),
        down + (1,): (32, 4, 8), down + (4,): (32, 4, 8), down + (8,): (64, 4, 8), down + (16,): (64, 4, 8),
        qkv + (4,): (32, 8, 1), o + (4,): (32, 8, 1),
    }
    for (n, k, t), (rows, waves, nks) in want.items():
        p = ops.plan_decode(n, k, 128, t)
        assert (p["rows_per_wave"], p["waves_per_block"], p["k_slices"]) == (rows, waves, nks), (n, k, t, p)
        assert p["lds_bytes"] <= 160 * 1024


def test_decode_plan_shrinks_to_fit_the_lds():
    """Group 32 with a long unsplit k: the staged scales of four row blocks per wave would pass 160 KiB (n = 16384,
    k = 53248, t = 8: 4 waves x 104 k tiles x 4 groups x 4 row blocks x 32 B = 213 KiB).  The plan halves the rows per
    wave instead of refusing the shape; the gated kernel (two row blocks by construction) cuts k into slices."""
    p = ops.plan_decode(16384, 53248, 32, 8)
    assert p["lds_bytes"] <= 160 * 1024 and p["rows_per_wave"] in (16, 32), p
    p = ops.plan_decode(16384, 53248, 128, 8)
    assert p["rows_per_wave"] == 64, "group 128 needs a quarter of that and keeps four row blocks"
    p = ops.plan_decode(16384, 106496, 32, 8, glu=True)
    assert p["lds_bytes"] <= 160 * 1024 and p["k_slices"] >= 2, p
    # nothing fits: a k range that even one row block per wave and eight slices cannot stage
    with pytest.raises(ops.W4a16Error) as e:
        ops.plan_decode(64, 128 * 20000, 32, 1)
    assert e.value.code == ffi.ERR_SHAPE and "LDS" in str(e.value)
    for bad in [(0, 128, 128, 1), (64, 100, 128, 1), (64, 128, 64, 1), (64, 128, 128, 17)]:
        with pytest.raises(ops.W4a16Error):
            ops.plan_decode(*bad)
