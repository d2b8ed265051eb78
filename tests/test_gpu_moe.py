"""GPU parity tests of the MoE expert FFN (grouped / ragged W4A16 GEMM) through the C ABI against the CPU oracle."""
import numpy as np
import pytest

from llm170_amd import gen, ops
from llm170_amd import parity

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def dec():
    d = ops.W4a16Dec()
    yield d
    d.cc.close()


def _f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


def _bf16_scales(s):
    return (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)


SMALL = dict(E=8, h=256, n_ff=128, k=2)


@pytest.fixture(scope="module")
def small_experts(dec):
    out = {}
    for group in (32, 128):
        for bf in (False, True):
            q13, s13, q2, s2 = gen.make_experts(SMALL["E"], SMALL["h"], SMALL["n_ff"], group, seed=gen.GATE_SEED + group)
            if bf:
                s13, s2 = _bf16_scales(s13), _bf16_scales(s2)
            name = "small_g%d_%s" % (group, "bf16" if bf else "f16")
            dec.upload_experts(name, q13, s13, q2, s2, SMALL["E"], SMALL["h"], SMALL["n_ff"], group, bf)
            out[(group, bf)] = (name, q13, s13, q2, s2)
    return out


# ------------------------------------------------------------------ arena re-layout, bit exact
def test_experts_arena_dequant_bit_exact(dec, orc, small_experts):
    for (group, bf), (name, q13, s13, q2, s2) in small_experts.items():
        for e in (0, 3, SMALL["E"] - 1):
            got = dec.experts_dequant(name, 0, e)
            want = orc.dequant_matrix(q13[e], s13[e], 2 * SMALL["n_ff"], SMALL["h"], group, bf)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (group, bf, e, "w13")
            got = dec.experts_dequant(name, 1, e)
            want = orc.dequant_matrix(q2[e], s2[e], SMALL["h"], SMALL["n_ff"], group, bf)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (group, bf, e, "w2")


# ------------------------------------------------------------------ routing on the device
@pytest.mark.parametrize("t,n_exp,k", [(1, 128, 8), (4, 128, 8), (512, 128, 8), (7, 8, 2), (33, 200, 5), (3, 1024, 64)])
def test_route_matches_host_rule(dec, orc, t, n_exp, k):
    say("route", t, n_exp, k)
    lg = gen.router_logits(t, n_exp)
    cc = dec.cc
    pl, pi, pw = cc.to_device(lg), cc.alloc(t * k * 4), cc.alloc(t * k * 4)
    dec.moe_route(pl, t, n_exp, k, pi, pw)
    idx, w = cc.d2h(pi, (t, k), np.int32), cc.d2h(pw, (t, k), np.float32)
    for p in (pl, pi, pw):
        cc.free(p)
    oi, ow = orc.moe_topk_batch(lg, k)
    assert np.array_equal(idx, oi)
    assert np.allclose(w, ow, rtol=2e-6, atol=0)
    assert np.allclose(w.sum(1), 1.0, atol=1e-6)


def test_route_ties_go_to_lower_index(dec):
    cc = dec.cc
    lg = np.ones((2, 130), np.float32)
    lg[1, 70] = 2.0
    pl, pi, pw = cc.to_device(lg), cc.alloc(2 * 4 * 4), cc.alloc(2 * 4 * 4)
    dec.moe_route(pl, 2, 130, 4, pi, pw)
    idx = cc.d2h(pi, (2, 4), np.int32)
    for p in (pl, pi, pw):
        cc.free(p)
    assert idx[0].tolist() == [0, 1, 2, 3] and idx[1].tolist() == [70, 0, 1, 2]


# ------------------------------------------------------------------ align on the device
@pytest.mark.parametrize("ns,n_exp,block", [(8, 128, 4), (32, 128, 4), (128, 128, 16), (4096, 128, 48), (4096, 128, 32),
                                            (4096, 128, 64), (1000, 7, 64), (130, 1024, 16), (1, 1, 4), (777, 33, 16),
                                            (20000, 128, 64), (9000, 1000, 16)])
def test_align_matches_oracle(dec, orc, ns, n_exp, block):
    say("align", ns, n_exp, block)
    rng = np.random.default_rng(ns * 7 + n_exp)
    idx = rng.integers(0, n_exp, ns).astype(np.int32)
    if ns == 4096:
        idx[:64] = 5  # one step of one wave entirely on one expert
    cc = dec.cc
    cap_s, cap_e = ns + n_exp * block, ns // block + n_exp + 1
    pi, ps, pe, pn = cc.to_device(idx), cc.alloc(cap_s * 4), cc.alloc(cap_e * 4), cc.alloc(8)
    dec.moe_align(pi, ns, n_exp, block, ps, pe, pn)
    n_post, hit = cc.d2h(pn, (2,), np.int32)
    s, e = cc.d2h(ps, (cap_s,), np.int32), cc.d2h(pe, (cap_e,), np.int32)
    for p in (pi, ps, pe, pn):
        cc.free(p)
    ws, we, wn = orc.moe_align(idx, n_exp, block)
    assert n_post == wn and hit == np.unique(idx).size
    assert np.array_equal(s[:wn], ws) and np.array_equal(e[:wn // block], we)


# ------------------------------------------------------------------ the FFN, stage by stage and end to end
def _run_ffn(dec, name, x, idx, wt, t, k, h, gelu=False):
    cc = dec.cc
    px, pi, pw, py = cc.to_device(x), cc.to_device(idx), cc.to_device(wt), cc.alloc(t * h * 4)
    dec.moe_ffn(name, px, pi, pw, t, k, py, gelu=gelu)
    y = cc.d2h(py, (t, h), np.float32)
    ns = t * k
    spec = dec.experts_spec(name)
    act, blk = dec.moe_scratch(3, np.uint16)
    c2 = None if blk == 1 else dec.moe_scratch(4, np.uint16)[0].reshape(ns, h)  # direct mode keeps c2 in registers
    for p in (px, pi, pw, py):
        cc.free(p)
    return y, act.reshape(ns, spec["n_ff"]), c2, blk


def _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, what, threads=8, gelu=False):
    t, k = idx.shape
    full = orc.moe_ffn(x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, threads=threads, gelu=gelu)
    if gelu:
        fn = lambda g1, u1: 0.5 * g1 * (1.0 + np.tanh(0.7978846 * (g1 + 0.044715 * g1 ** 3))) * u1
    else:
        fn = lambda g1, u1: g1 / (1.0 + np.exp(-g1)) * u1
    # stage 1: act against the oracle's act.  The device's gate/up sums differ from the lane order by f32 rounding
    # (about 1e-6 absolute here), so a few round to the neighbouring f16 before the activation, and a sum that
    # cancelled to almost nothing moves by many of its own tiny f16 steps.  Tolerance: the device value must lie
    # inside the envelope of silu(g')*u' over g', u' within ONE f16 step of the oracle's gate/up — the step taken at
    # a magnitude clamped from below as in llm170_amd/parity.py — widened by 1.5 f16 steps of the
    # result (final rounding, exp implementation); and nearly all elements must be identical.
    g0 = full["c13"][:, :n_ff].view(np.float16).astype(np.float64)
    u0 = full["c13"][:, n_ff:].view(np.float16).astype(np.float64)
    rms = float(np.sqrt(np.mean(np.concatenate([g0.ravel(), u0.ravel()]) ** 2)))
    dg = parity.f16_ulp(np.maximum(np.abs(g0), rms / parity.CLAMP_DIV))
    du = parity.f16_ulp(np.maximum(np.abs(u0), rms / parity.CLAMP_DIV))
    lo = np.full(g0.shape, np.inf)
    hi = np.full(g0.shape, -np.inf)
    for gs in (-1.0, 0.0, 1.0):
        for us in (-1.0, 0.0, 1.0):
            g1, u1 = g0 + gs * dg, u0 + us * du
            v = fn(g1, u1)
            lo, hi = np.minimum(lo, v), np.maximum(hi, v)
    a = _f16(act).astype(np.float64)
    pad = 1.5 * parity.f16_ulp(np.maximum(np.abs(lo), np.abs(hi)))
    bad = (a < lo - pad) | (a > hi + pad)
    assert not bad.any(), (what, "act outside the one-step envelope", int(bad.sum()))
    same = float(np.mean(act == full["act"]))
    assert same > 0.97, (what, "act identical fraction", same)
    # stage 2: c2 from the device's own act, against the oracle run on that same act
    st2 = orc.moe_ffn(x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, threads=threads, act_in=act, gelu=gelu)
    if c2 is not None:
        m2 = parity.assert_close(_f16(c2), _f16(st2["c2"]), what + " c2")
        # stage 3: the slot-order f32 sum of the device's c2 is exact arithmetic on f16 inputs -> bit for bit
        y3 = orc.moe_topk_sum_f16(c2, t, h, k)
        assert np.array_equal(y.view(np.uint32), y3.view(np.uint32)), what + " sum"
    else:
        # direct mode: down projection, weight, f16 rounding and sum are one launch; y against the oracle's y from the
        # device's own act.  Each of the k terms may round to the neighbouring f16 (the f32 sums differ in their last
        # bits), which moves y by one f16 step of that term; the f32 additions themselves are exact here.
        c2r = _f16(st2["c2"]).astype(np.float64).reshape(t, k, h)
        bound = parity.f16_ulp(c2r).sum(axis=1) + 1e-7
        dy = np.abs(y.astype(np.float64) - st2["y"].astype(np.float64))
        assert np.all(dy <= bound), (what, "y from act", float((dy / bound).max()))
        assert np.mean(y == st2["y"]) > 0.97, (what, "y identical fraction", float(np.mean(y == st2["y"])))
        m2 = parity.compare(y, st2["y"])
    # end to end against the oracle's independent run
    m = parity.compare(y, full["y"])
    assert m["rel_l2"] <= parity.REL_L2_TOL, (what, m)
    return same, m2, m


@pytest.mark.parametrize("group,bf", [(32, False), (32, True), (128, False), (128, True)])
@pytest.mark.parametrize("t", [1, 3, 4, 9, 16, 40, 70, 200])
def test_moe_ffn_small(dec, orc, small_experts, group, bf, t):
    say("moe_ffn small", group, bf, t)
    name, q13, s13, q2, s2 = small_experts[(group, bf)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    x = gen.normal_f16(1000 + t, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=t), k)
    y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
    _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, "small g%d bf%d t%d blk%d" % (group, bf, t, blk))


@pytest.mark.parametrize("group,bf", [(32, False), (128, True)])
@pytest.mark.parametrize("t", [1, 4, 9, 40, 200])
def test_moe_ffn_gelu(dec, orc, small_experts, group, bf, t):
    """The gelu flag of marlin_moe_ffn_dev: tanh-form gelu on the gate instead of silu, every regime of the FFN."""
    say("moe_ffn gelu", group, bf, t)
    name, q13, s13, q2, s2 = small_experts[(group, bf)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    x = gen.normal_f16(3000 + t, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=50 + t), k)
    y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h, gelu=True)
    _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, "gelu g%d bf%d t%d blk%d" % (group, bf, t, blk),
               gelu=True)
    # and it is not silu
    y_s, act_s, _, _ = _run_ffn(dec, name, x, idx, wt, t, k, h)
    assert np.mean(act != act_s) > 0.5
    from llm170_amd import ffi
    with pytest.raises(ops.W4a16Error):  # an activation that does not exist
        ffi.check(dec.cc.lib.w4a16_moe_ffn_act(dec.cc.h, name.encode(), 1, 1, 1, 1, k, 1, 7))


@pytest.mark.parametrize("block,waves", [(1, 0), (1, 2), (4, 1), (4, 2), (16, 1), (16, 4), (32, 4), (48, 8), (64, 4)])
def test_moe_ffn_launch_shapes_agree(dec, orc, small_experts, block, waves):
    """Every segment size and wave count computes the same FFN (t small enough for the 4-slot segments)."""
    say("moe shapes", block, waves)
    name, q13, s13, q2, s2 = small_experts[(32, False)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    t = 4 if block <= 4 else 13 if block == 16 else 90
    x = gen.normal_f16(77, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=3), k)
    dec.set_moe_shape(block, waves)
    try:
        y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
    finally:
        dec.set_moe_shape(0, 0)
    assert blk == block
    _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, 32, False, "shape blk%d w%d" % (block, waves))


@pytest.mark.parametrize("group,bf", [(32, False), (128, True)])
def test_moe_ffn_partly_filled_segments(dec, orc, small_experts, group, bf):
    """Runs of 1, 16, 17, 32, 33, 48, 49 and 64 slots: with 64-slot segments every count of 16-slot blocks that hold a
    slot occurs, and a workgroup multiplies only those.  Against the oracle, and bit for bit the same act, c2 and y with
    32-, 48- and 64-slot segments (a slot's sums do not depend on the block it falls into)."""
    name, q13, s13, q2, s2 = small_experts[(group, bf)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    runs = [1, 16, 17, 32, 33, 48, 49, 64]
    assert len(runs) == E and sum(runs) % k == 0
    slots = np.concatenate([np.full(r, e, np.int32) for e, r in enumerate(runs)])
    t = slots.size // k
    # token i takes slots i and i + t of the list: two different experts per token, every run length as listed
    idx = np.stack([slots[:t], slots[t:]], axis=1).astype(np.int32)
    assert np.all(idx[:, 0] != idx[:, 1]) and [int((idx == e).sum()) for e in range(E)] == runs
    wt = (0.2 + 0.6 * gen.uniform01(9, t * k)).astype(np.float32).reshape(t, k)
    x = gen.normal_f16(4242, (t, h))
    got = {}
    for block in (64, 48, 32):
        say("moe partly filled", group, bf, block)
        dec.set_moe_shape(block, 4)
        try:
            y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
        finally:
            dec.set_moe_shape(0, 0)
        assert blk == block
        got[block] = (y, act, c2)
    _check_ffn(orc, *got[64], x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, "partly filled g%d" % group)
    for block in (48, 32):
        for a, b, what in zip(got[64], got[block], ("y", "act", "c2")):
            assert np.array_equal(a.view(np.uint32 if a.dtype == np.float32 else np.uint16),
                                  b.view(np.uint32 if b.dtype == np.float32 else np.uint16)), (block, what)


def test_moe_ffn_unused_experts_and_hot_expert(dec, orc, small_experts):
    """Routing that leaves experts empty and sends every token to one expert (runs longer than one segment)."""
    name, q13, s13, q2, s2 = small_experts[(32, False)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    t = 100
    x = gen.normal_f16(5, (t, h))
    idx = np.empty((t, k), np.int32)
    idx[:, 0] = 6
    idx[:, 1] = np.arange(t) % 2  # experts 2..5, 7 never chosen
    wt = np.full((t, k), 0.5, np.float32)
    y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
    _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, 32, False, "hot expert")


# ------------------------------------------------------------------ the 35B-A3B layer shape: 128 experts, top-8
@pytest.fixture(scope="module")
def full_experts(dec):
    E, h, n_ff, g = 128, 2048, 768, 32
    q13, s13, q2, s2 = gen.make_experts(E, h, n_ff, g)
    dec.upload_experts("a3b", q13, s13, q2, s2, E, h, n_ff, g, False)
    return "a3b", q13, s13, q2, s2


@pytest.mark.parametrize("t", [1, 4, 512])
def test_moe_ffn_full_shape(dec, orc, full_experts, t):
    say("moe_ffn full", t)
    name, q13, s13, q2, s2 = full_experts
    E, h, n_ff, k = 128, 2048, 768, 8
    x = gen.normal_f16(4242 + t, (t, h))
    lg = gen.router_logits(t, E)
    cc = dec.cc
    pl, pi, pw = cc.to_device(lg), cc.alloc(t * k * 4), cc.alloc(t * k * 4)
    dec.moe_route(pl, t, E, k, pi, pw)
    idx, wt = cc.d2h(pi, (t, k), np.int32), cc.d2h(pw, (t, k), np.float32)
    for p in (pl, pi, pw):
        cc.free(p)
    assert np.array_equal(idx, ops.moe_topk(lg, k)[0])
    y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
    same, m2, m = _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, 32, False, "a3b t%d" % t, threads=16)
    say("  blk", blk, "act identical", same, "c2", m2["rel_l2"], m2["max_ulp"], "y rel_l2", m["rel_l2"])


# ------------------------------------------------------------------ the MFMA-tiled grouped kernels (long runs per expert)
@pytest.mark.parametrize("group,bf", [(32, False), (32, True), (128, False), (128, True)])
@pytest.mark.parametrize("t", [5, 40, 200, 333])
def test_moe_ffn_tiled_small(dec, orc, small_experts, group, bf, t):
    """The 64-slot-segment x 256-column kernels on 32x32x16 tiles, forced at sizes where most segments are ragged:
    same stage-by-stage checks as the streaming kernels."""
    say("moe_ffn tiled small", group, bf, t)
    name, q13, s13, q2, s2 = small_experts[(group, bf)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    x = gen.normal_f16(1500 + t, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=20 + t), k)
    dec.set_moe_tiled(1)
    try:
        y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
        assert blk == 64 and dec.cc.last_launch_symbol() == "w4a16_moe_topk_sum_f16"
        _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, "tiled g%d bf%d t%d" % (group, bf, t))
        if t == 200:
            y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h, gelu=True)
            _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, "tiled gelu", gelu=True)
            # a hot expert (runs of several segments) and experts nobody chose
            idx2 = np.empty((t, k), np.int32)
            idx2[:, 0] = 6
            idx2[:, 1] = np.arange(t) % 2
            wt2 = np.full((t, k), 0.5, np.float32)
            y, act, c2, blk = _run_ffn(dec, name, x, idx2, wt2, t, k, h)
            _check_ffn(orc, y, act, c2, x, idx2, wt2, q13, s13, q2, s2, h, n_ff, group, bf, "tiled hot expert")
    finally:
        dec.set_moe_tiled(0)


def test_moe_ffn_tiled_full_shape(dec, orc, full_experts):
    """T = 2048 at the 35B-A3B layer shape: a mean run of 128 slots per expert, where AUTO picks the tiled kernels; and
    never does below the threshold or with a forced segment size."""
    name, q13, s13, q2, s2 = full_experts
    E, h, n_ff, k, t = 128, 2048, 768, 8, 2048
    say("moe_ffn tiled full", t)
    x = gen.normal_f16(4242 + t, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E), k)
    y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, t, k, h)
    assert blk == 64
    same, m2, m = _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, 32, False, "a3b tiled t%d" % t, threads=16)
    say("  act identical", same, "c2", m2["rel_l2"], m2["max_ulp"], "y rel_l2", m["rel_l2"])
    dec.set_moe_tiled(-1)
    try:
        y2, act2, c22, blk2 = _run_ffn(dec, name, x, idx, wt, t, k, h)
    finally:
        dec.set_moe_tiled(0)
    m3 = parity.compare(y, y2)
    say("  tiled vs streaming rel_l2", m3["rel_l2"], "act identical", float(np.mean(act == act2)))
    assert m3["rel_l2"] < 1e-4 and np.mean(act == act2) > 0.97
    with pytest.raises(ops.W4a16Error):
        dec.set_moe_tiled(2)


@pytest.mark.parametrize("group,bf", [(32, True), (128, False)])
def test_moe_irregular_scales_stay_off_the_tiled_kernels(dec, orc, group, bf):
    """Experts with a zero scale (and, for bf16, a scale of about 1e-38) at a size where AUTO would pick the MFMA-tiled
    grouped kernels: those carry sum / s_cur as a running unit and would produce NaN; the upload marks the arenas
    irregular, AUTO stays on the streaming kernels (same results as with the tiled kernels switched off, checked
    against the oracle) and a forced tiled launch is refused."""
    E, h, n_ff, k, t = 4, 256, 128, 2, 256  # mean run per expert 128 >= 96: AUTO would go tiled
    q13, s13, q2, s2 = gen.make_experts(E, h, n_ff, group, seed=gen.GATE_SEED + 7 * group)
    if bf:
        s13, s2 = _bf16_scales(s13), _bf16_scales(s2)
    x = gen.normal_f16(77, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=5), k)
    dec.upload_experts("regular", q13, s13, q2, s2, E, h, n_ff, group, bf)
    y0, _, _, blk0 = _run_ffn(dec, "regular", x, idx, wt, t, k, h)
    assert blk0 == 64, "the regular arenas take the tiled kernels at this size"
    s13 = s13.copy()
    s2 = s2.copy()
    s13[1, 5, 0] = 0            # a zero scale in expert 1, gate row 5, first group
    s2[2, 9, 1 if n_ff // group > 1 else 0] = 0x0001 if bf else 0  # bf16: 9e-41, far below 2^-60; f16: another zero
    if bf:
        s13[3, 40, 1] = 0x0080  # bf16 1.18e-38 (the smallest normal)
    dec.upload_experts("irregular", q13, s13, q2, s2, E, h, n_ff, group, bf)
    y, act, c2, blk = _run_ffn(dec, "irregular", x, idx, wt, t, k, h)
    assert np.all(np.isfinite(y)), "NaN or Inf from an irregular scale"
    dec.set_moe_tiled(-1)
    try:
        y_stream, act_s, c2_s, blk_s = _run_ffn(dec, "irregular", x, idx, wt, t, k, h)
    finally:
        dec.set_moe_tiled(0)
    assert blk == blk_s and np.array_equal(y.view(np.uint32), y_stream.view(np.uint32)), "AUTO = streaming kernels"
    _check_ffn(orc, y, act, c2, x, idx, wt, q13, s13, q2, s2, h, n_ff, group, bf, "irregular scales g%d bf%d" % (group, bf))
    dec.set_moe_tiled(1)
    try:
        with pytest.raises(ops.W4a16Error) as e:
            _run_ffn(dec, "irregular", x, idx, wt, t, k, h)
        assert "scale" in str(e.value)
    finally:
        dec.set_moe_tiled(0)


def test_moe_errors(dec, small_experts):
    name = small_experts[(32, False)][0]
    with pytest.raises(ops.W4a16Error):
        dec.moe_ffn("nope", 1, 1, 1, 1, 2, 1)
    with pytest.raises(ops.W4a16Error):
        dec.moe_ffn(name, 0, 1, 1, 1, 2, 1)
    with pytest.raises(ops.W4a16Error):
        dec.moe_ffn(name, 1, 1, 1, 1, 99, 1)
    with pytest.raises(ops.W4a16Error):
        dec.upload_experts("bad", np.zeros(4, np.uint32), np.zeros(4, np.uint16), np.zeros(4, np.uint32),
                           np.zeros(4, np.uint16), 2, 256, 128, 32, False)
    with pytest.raises(ops.W4a16Error):
        dec.set_moe_shape(5, 0)


def test_moe_direct_and_aligned_modes_agree(dec, orc, small_experts):
    """t <= 15 runs without the alignment pass by default; forcing the aligned path gives the same act bit for bit and
    a y that differs at most by f16 rounding flips of single c2 terms."""
    name, q13, s13, q2, s2 = small_experts[(32, False)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    for t in (1, 2, 4, 7, 15):
        x = gen.normal_f16(500 + t, (t, h))
        idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=40 + t), k)
        y_d, act_d, c2_d, blk_d = _run_ffn(dec, name, x, idx, wt, t, k, h)
        assert blk_d == 1 and c2_d is None
        dec.set_moe_shape(4, 0)
        try:
            y_a, act_a, c2_a, blk_a = _run_ffn(dec, name, x, idx, wt, t, k, h)
        finally:
            dec.set_moe_shape(0, 0)
        assert blk_a == 4 and np.array_equal(act_d, act_a)
        parity.assert_close(y_d, y_a, "direct vs aligned t%d" % t)


def test_moe_direct_mode_out_of_range_expert_contributes_zero(dec, orc, small_experts):
    name, q13, s13, q2, s2 = small_experts[(32, False)]
    E, h, n_ff, k = SMALL["E"], SMALL["h"], SMALL["n_ff"], SMALL["k"]
    x = gen.normal_f16(77, (2, h))
    idx = np.array([[1, 99], [3, 2]], np.int32)  # expert 99 does not exist
    wt = np.full((2, k), 0.5, np.float32)
    y, act, c2, blk = _run_ffn(dec, name, x, idx, wt, 2, k, h)
    ok_idx = np.array([[1, 1], [3, 2]], np.int32)
    ok_wt = np.array([[0.5, 0.0], [0.5, 0.5]], np.float32)
    ref = orc.moe_ffn(x, ok_idx, ok_wt, q13, s13, q2, s2, h, n_ff, 32, False)
    assert parity.compare(y, ref["y"])["rel_l2"] < 1e-3
