"""Closed-form and exact-value checks of the fast kernels at full layer sizes, through the C ABI.

Two kinds of evidence that need no tolerance argument:
  * operands on which every partial sum is exactly representable in f32 (power-of-two scales, small-integer
    activations): any summation order gives the same bits, so every kernel must equal the plain matrix product bit
    for bit — the reference's own self-checks work this way (w4a16_dec/probe.rs:1291-1426 decode_selfcheck,
    crates/server/src/probes/w4a16/gpu/bench.rs:77-166 run_marlin_selfcheck);
  * on random operands, the compensated f64 dot (crates/core/src/quant/exact.rs:27-53) as the yardstick: the kernels
    are as close to the exact value as the lane-order reference itself is.
"""
import numpy as np
import pytest

from llm170_amd import gen, ops, parity

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def dec():
    d = ops.W4a16Dec()
    yield d
    d.cc.close()


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _device_forward(dec, name, x, t, path, out_f16=False):
    spec = dec.lin_spec(name)
    xd = dec.cc.to_device(np.ascontiguousarray(x[:t]))
    yd = dec.cc.alloc(t * spec["n"] * (2 if out_f16 else 4))
    try:
        dec.lin_forward(name, xd, yd, t, out_f16=out_f16, path=path)
        return dec.cc.d2h(yd, (t, spec["n"]), np.uint16 if out_f16 else np.float32)
    finally:
        dec.cc.free(xd)
        dec.cc.free(yd)


# ------------------------------------------------------------------ exactly summable operands
def pow2_linear(n, k, group, t, seed, e_lo=5, e_hi=8, x_max=2):
    """Weights: seeded nibbles.  Scales: 2^-e, e uniform in e_lo..e_hi per (row, group).  x: integers in
    -x_max..x_max.  Every product is a multiple of 2^-e_hi and the sum of their magnitudes over a row stays below
    2^24 such units (asserted), so every partial sum in any order is exact in f32."""
    q = gen.weights_q(seed, n, k)
    e = (gen.stream(seed + 1, n * (k // group)) % np.uint64(e_hi - e_lo + 1)).astype(np.int64) + e_lo
    s = np.ldexp(np.float32(1.0), -e).astype(np.float16).view(np.uint16).reshape(n, k // group)
    xi = (gen.stream(seed + 2, t * k) % np.uint64(2 * x_max + 1)).astype(np.int64) - x_max
    x = xi.astype(np.float16).view(np.uint16).reshape(t, k)
    assert k * 8 * x_max * (1 << (e_hi - e_lo)) < (1 << 24)
    return q, s, x


def pow2_expect(q, s, x, n, k, group):
    """The matrix product in plain f32 (exact on these operands, whatever order the BLAS takes)."""
    w = (gen.unpack_nibbles(q, k).astype(np.float32)) * np.repeat(s.view(np.float16).astype(np.float32), group, axis=1)
    return x.view(np.float16).astype(np.float32) @ w.T


@pytest.mark.parametrize("n,k,t,what", [
    (34816, 5120, 1024, "prefill"), (5120, 17408, 512, "prefill"), (5120, 17408, 1024, "prefill"),
    (34816, 5120, 64, "stream"), (5120, 17408, 48, "stream"),
    (34816, 5120, 16, "decode"), (5120, 17408, 4, "decode"), (5120, 17408, 1, "decode"),
])
def test_power_of_two_operands_give_the_exact_product(dec, n, k, t, what):
    say("pow2", what, n, k, t)
    group = 128
    q, s, x = pow2_linear(n, k, group, t, seed=900 + t)
    want = pow2_expect(q, s, x, n, k, group)
    dec.upload_lin_g("p2", q, s, n, k, group, False)
    if what == "prefill":
        runs = []
        try:
            for tile in (64, 96, 128):
                for ks in (-1, 0, 2):  # unsplit, automatic, two k slices
                    dec.set_prefill_tile(tile)
                    dec.set_prefill_ksplit(ks)
                    runs.append(("tile %d ksplit %d" % (tile, ks), _device_forward(dec, "p2", x, t, ops.PATH_PREFILL)))
        finally:
            dec.set_prefill_tile(0)
            dec.set_prefill_ksplit(0)
    elif what == "stream":
        runs = [("auto", _device_forward(dec, "p2", x, t, ops.PATH_STREAM))]
        try:
            for ks in (-1, 3):
                dec.set_decode_ksplit(ks)
                runs.append(("ksplit %d" % ks, _device_forward(dec, "p2", x, t, ops.PATH_STREAM)))
        finally:
            dec.set_decode_ksplit(0)
    else:
        runs = [("auto", _device_forward(dec, "p2", x, t, ops.PATH_DECODE))]
        try:
            for ks in (-1, 5):
                dec.set_decode_ksplit(ks)
                runs.append(("ksplit %d" % ks, _device_forward(dec, "p2", x, t, ops.PATH_DECODE)))
        finally:
            dec.set_decode_ksplit(0)
    for label, got in runs:
        bad = np.argwhere(_bits(got) != _bits(want))
        assert bad.size == 0, "%s %s: %d outputs differ, first at %s: %r vs %r" % (
            what, label, len(bad), bad[0], got[tuple(bad[0])], want[tuple(bad[0])])


def test_power_of_two_operands_group_32(dec):
    """The group-32 builds of the three kernels (one expert's gate|up shape, dense)."""
    n, k, group = 1536, 2048, 32
    for t, path in ((300, ops.PATH_PREFILL), (40, ops.PATH_STREAM), (7, ops.PATH_DECODE)):
        q, s, x = pow2_linear(n, k, group, t, seed=70 + t)
        dec.upload_lin_g("p2g32", q, s, n, k, group, False)
        got = _device_forward(dec, "p2g32", x, t, path)
        assert np.array_equal(_bits(got), _bits(pow2_expect(q, s, x, n, k, group))), (t, path)


# ------------------------------------------------------------------ MoE expert FFN, closed form end to end
def test_moe_ffn_exact_operands_full_shape(dec):
    """128 experts, top-8, hidden 2048, n_ff 768, group 32, T = 512 (grouped GEMMs, streaming and MFMA-tiled), 64 and 4 (direct mode), on
    operands that make every stage exactly computable on the host:
      x[token] = c * (+1, -1, +1, ...), c = 1 or 2 by token; gate rows +7, -7, +7, ... with scale 2^-9: gate = 28 c, where silu(g) = g in
      f32 (exp(-28) < 2^-25), so act = f16(f16(gate) * f16(up)); up = power-of-two scales times integer sums (exact);
      down: power-of-two scales times act, every partial sum exact in any order (the bound is asserted on the data);
      c2 = f16(f32(wt) * sum), y = f32 sum of a token's c2 in slot order."""
    E, h, n_ff, g, k = 128, 2048, 768, 32, 8
    q13 = gen.weights_q(501, E * 2 * n_ff, h).reshape(E, 2 * n_ff, h // 8)
    q13[:, :n_ff, :] = 0x1F1F1F1F  # gate weights +7 at even k, -7 at odd k
    e13 = (gen.stream(502, E * 2 * n_ff * (h // g)) % np.uint64(2)).astype(np.int64).reshape(E, 2 * n_ff, h // g) + 6
    e13[:, :n_ff, :] = 9
    s13 = np.ldexp(np.float32(1.0), -e13).astype(np.float16).view(np.uint16)
    q2 = gen.weights_q(503, E * h, n_ff).reshape(E, h, n_ff // 8)
    e2 = (gen.stream(504, E * h * (n_ff // g)) % np.uint64(2)).astype(np.int64).reshape(E, h, n_ff // g) + 4
    s2 = np.ldexp(np.float32(1.0), -e2).astype(np.float16).view(np.uint16)
    dec.upload_experts("p2moe", q13, s13, q2, s2, E, h, n_ff, g, False)
    stage = {}
    alt = np.where(np.arange(h) % 2 == 0, 1.0, -1.0).astype(np.float32)

    def expert(e, c):
        """act f16 [n_ff] and the down projection f32 [h] of expert e on the row c * (+1, -1, ...)."""
        if (e, c) not in stage:
            w13 = gen.unpack_nibbles(q13[e], h).astype(np.float32) * np.repeat(s13[e].view(np.float16).astype(np.float32), g, axis=1)
            w2 = gen.unpack_nibbles(q2[e], n_ff).astype(np.float32) * np.repeat(s2[e].view(np.float16).astype(np.float32), g, axis=1)
            gu = w13 @ (c * alt)  # exact: integers times powers of two
            gate, up = gu[:n_ff].astype(np.float16), gu[n_ff:].astype(np.float16)
            assert np.all(gate == np.float16(28.0 * c))
            act = (gate.astype(np.float32) * up.astype(np.float32)).astype(np.float16)
            af = act.astype(np.float64)
            # act is a multiple of 2^-5 c^2, the down weights of 2^-5: sum of |terms| below 2^24 units, so every
            # partial sum of the down projection is exact in f32 in any order
            assert float(np.max(np.abs(w2.astype(np.float64)) @ np.abs(af))) / (2.0 ** -10 * c * c) < float(1 << 24)
            stage[(e, c)] = (act.view(np.uint16), (w2.astype(np.float64) @ af).astype(np.float32))
        return stage[(e, c)]

    cc = dec.cc
    for t, tiled in ((512, False), (512, True), (64, False), (4, False)):  # tiled: the 32x32x16 grouped kernels
        say("moe exact", t, "tiled" if tiled else "")
        cs = (gen.stream(77 + t, t) % np.uint64(2)).astype(np.int64) + 1
        x = (alt[None, :] * cs[:, None]).astype(np.float16).view(np.uint16)
        idx, wt = ops.moe_topk(gen.router_logits(t, E, seed=900 + t), k)
        px, pi, pw, py = cc.to_device(x), cc.to_device(idx), cc.to_device(wt), cc.alloc(t * h * 4)
        dec.set_moe_tiled(1 if tiled else 0)
        try:
            dec.moe_ffn("p2moe", px, pi, pw, t, k, py)
        finally:
            dec.set_moe_tiled(0)
        y = cc.d2h(py, (t, h), np.float32)
        act, blk = dec.moe_scratch(3, np.uint16)
        assert not tiled or blk == 64
        act = act.reshape(t * k, n_ff)
        c2 = None if blk == 1 else dec.moe_scratch(4, np.uint16)[0].reshape(t * k, h)
        for p_ in (px, pi, pw, py):
            cc.free(p_)
        want_y = np.zeros((t, h), np.float32)
        for tok in range(t):
            for c in range(k):
                j = tok * k + c
                a, d = expert(int(idx[tok, c]), int(cs[tok]))
                assert np.array_equal(act[j], a), ("act", t, tok, c)
                c2j = (np.float32(wt[tok, c]) * d).astype(np.float16)
                if c2 is not None:
                    assert np.array_equal(c2[j], c2j.view(np.uint16)), ("c2", t, tok, c)
                want_y[tok] += c2j.astype(np.float32)
        assert np.array_equal(_bits(y), _bits(want_y)), ("y", t)


# ------------------------------------------------------------------ the compensated f64 dot as the yardstick
@pytest.mark.parametrize("n,k,t,path", [
    (34816, 5120, 1, ops.PATH_DECODE), (5120, 17408, 1, ops.PATH_DECODE), (5120, 17408, 4, ops.PATH_DECODE),
    (34816, 5120, 4096, ops.PATH_PREFILL), (5120, 17408, 1024, ops.PATH_PREFILL), (34816, 5120, 48, ops.PATH_STREAM),
])
def test_kernels_are_as_close_to_exact_as_the_reference(dec, orc, n, k, t, path):
    """Every output at M = 1 (a seeded sample of 8192 beyond), f32 out: the kernel's and the lane-order reference's
    distances from the compensated f64 dot, absolute and in strict f16 ulp of the exact value.  The outputs that miss
    the strict 4-ulp rule against the reference are the ones where the reference itself is that far from exact."""
    say("exact yardstick", n, k, t, path)
    group = 128
    q, s, x = gen.make_linear(n, k, group, t, seed=7)
    dec.upload_lin_g("ex", q, s, n, k, group, False)
    got = _device_forward(dec, "ex", x, t, path)
    if t == 1:
        rows, toks = np.arange(n, dtype=np.uint32), np.zeros(n, np.uint32)
    else:
        rows = (gen.stream(31, 8192) % np.uint64(n)).astype(np.uint32)
        toks = (gen.stream(32, 8192) % np.uint64(t)).astype(np.uint32)
    lane = orc.gemm_lane_sample(x, q, s, k, group, rows, toks)
    exact = orc.exact_dot_sample(x, q, s, k, group, rows, toks)
    ev = parity.exact_evidence(got[toks, rows], lane, exact)
    m = parity.assert_close(got[toks, rows], lane, "exact yardstick n%d k%d t%d" % (n, k, t))
    say("   ", ev)
    say("   ", {a: m[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "strict_fail", "clamped")})
    assert ev["ok"], ev
