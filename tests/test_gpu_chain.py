"""GPU parity tests of the layer chain (linears of a dense decoder layer run back to back with their glue) through
the C ABI against the CPU oracle."""
import numpy as np
import pytest

from llm170_amd import ffi, gen, ops
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


# ------------------------------------------------------------------ device generator == host generator
@pytest.mark.parametrize("n,k,group", [(48, 256, 128), (7168, 5120, 128), (100, 768, 32)])
def test_synth_linear_equals_host_generator(dec, n, k, group):
    sq, ss = gen.shape_seed(n, k, tensor=7), gen.shape_seed(n, k, tensor=8)
    dec.upload_lin_synth("syn", n, k, group, sq, ss)
    q, s = dec.untile("syn")
    assert np.array_equal(q, gen.weights_q(sq, n, k))
    assert np.array_equal(s, gen.scales_f16(ss, n, k, group))


def test_synth_errors(dec):
    with pytest.raises(ops.W4a16Error):
        dec.upload_lin_synth("bad", 16, 256, 128, 1, 2, lo=0.0, hi=0.02)
    with pytest.raises(ops.W4a16Error):
        dec.upload_lin_synth("bad", 16, 200, 128, 1, 2)


# ------------------------------------------------------------------ glue kernels
@pytest.mark.parametrize("t,ld,ncols", [(1, 5120, 5120), (4, 7168, 5120), (16, 300, 257), (3, 64, 1)])
def test_rms_rescale_bit_exact(dec, orc, t, ld, ncols):
    rng = np.random.default_rng(t * 1000 + ld)
    v = (rng.standard_normal((t, ld)) * rng.uniform(0.01, 300, (t, 1))).astype(np.float32)
    cc = dec.cc
    pv, po = cc.to_device(v), cc.alloc(t * ncols * 2)
    dec.rms_rescale_f16(pv, ld, ncols, t, po)
    got = cc.d2h(po, (t, ncols), np.uint16)
    cc.free(pv)
    cc.free(po)
    assert np.array_equal(got, orc.rms_rescale_f16(v, ncols))


@pytest.mark.parametrize("t,n_ff", [(1, 17408), (4, 17408), (5, 33)])
def test_silu_mul_close(dec, orc, t, n_ff):
    rng = np.random.default_rng(t + n_ff)
    gu = (rng.standard_normal((t, 2 * n_ff)) * 6).astype(np.float32)
    cc = dec.cc
    pg, po = cc.to_device(gu), cc.alloc(t * n_ff * 2)
    dec.silu_mul_f16(pg, n_ff, t, po)
    got = cc.d2h(po, (t, n_ff), np.uint16)
    cc.free(pg)
    cc.free(po)
    want = orc.silu_mul_f16_rows(gu)
    # exp is evaluated by different libraries: results may differ in the last f32 bit before the f16 rounding
    a, b = _f16(got).astype(np.float64), _f16(want).astype(np.float64)
    assert np.all(np.abs(a - b) <= parity.f16_ulp(b))
    assert np.mean(got == want) > 0.995


# ------------------------------------------------------------------ gate|up with the SiLU*up epilogue
@pytest.mark.parametrize("n,k,group,bf16", [(1024, 256, 128, False), (2048, 512, 32, False), (1024, 256, 128, True),
                                            (34816, 5120, 128, False)])
@pytest.mark.parametrize("t", [1, 3, 4, 7, 16])
def test_fused_glu_equals_linear_then_silu_mul(dec, orc, n, k, group, bf16, t):
    """The fused kernel gives the bits of the two-launch sequence at the same launch shape, and both stay within one
    f16 step of the oracle's silu_mul of the lane GEMM."""
    q, s, x = gen.make_linear(n, k, group, t, seed=71)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("glu", q, s, n, k, group, bf16)
    cc = dec.cc
    px, pg, pa, pb = cc.to_device(x), cc.alloc(t * n * 4), cc.alloc(t * (n // 2) * 2), cc.alloc(t * (n // 2) * 2)
    dec.set_decode_shape(32, 4 if t > 8 or n >= 16384 else 8)  # the launch shape the fused kernel picks
    try:
        dec.lin_forward("glu", px, pg, t, path=ops.PATH_DECODE)
    finally:
        dec.set_decode_shape(0, 0)
    dec.silu_mul_f16(pg, n // 2, t, pa)
    dec.lin_forward_glu("glu", px, pb, t)
    two, one = cc.d2h(pa, (t, n // 2), np.uint16), cc.d2h(pb, (t, n // 2), np.uint16)
    for p in (px, pg, pa, pb):
        cc.free(p)
    assert np.array_equal(one, two)
    if n <= 4096:
        want = orc.silu_mul_f16_rows(orc.gemm_lane(x, t, q, s, n, k, group, bf16, 8))
        got = one
    else:
        # layer shape: a seeded sample of 4096 (token, column) pairs, gate and up rows through the lane oracle
        cols = (gen.stream(91, 4096) % np.uint64(n // 2)).astype(np.uint32)
        toks = (gen.stream(92, 4096) % np.uint64(t)).astype(np.uint32)
        gate = orc.gemm_lane_sample(x, q, s, k, group, cols, toks, bf16)
        up = orc.gemm_lane_sample(x, q, s, k, group, cols + np.uint32(n // 2), toks, bf16)
        want = orc.silu_mul_f16_rows(np.stack([gate, up], axis=1).reshape(-1, 2))[:, 0]
        got = one[toks, cols]
    a, b = _f16(got).astype(np.float64), _f16(want).astype(np.float64)
    rms = float(np.sqrt(np.mean(b * b)))
    assert np.all(np.abs(a - b) <= 2 * parity.f16_ulp(np.maximum(np.abs(b), rms / parity.CLAMP_DIV)))
    assert np.mean(got == want) > 0.97


@pytest.mark.parametrize("n,k,group,bf16,t", [
    (34816, 5120, 128, False, 64), (34816, 5120, 128, False, 512), (34816, 5120, 128, False, 4096),
    (34816, 5120, 128, False, 17), (34816, 5120, 128, False, 1000),
    (1024, 2048, 32, True, 40), (1024, 2048, 32, True, 300), (5120, 17408, 128, False, 512), (2080, 512, 128, False, 130)])
def test_fused_glu_beyond_the_decode_regime(dec, orc, n, k, group, bf16, t):
    """w4a16_lin_forward_glu at 17..64 rows (weight-streaming kernel) and above (MFMA tiles, both block tiles, split-K
    on the narrow shape, ragged last tiles): the bits of the plain launch on the same path followed by the
    element-wise kernel (the reference's prefill chain runs exactly that pair, w4a16_dec/prefill.rs:148-207 +
    assets/ew.cu:9-32), and a seeded sample against the oracle's silu_mul of the lane GEMM."""
    say("glu beyond decode", n, k, group, bf16, t)
    q, s, x = gen.make_linear(n, k, group, t, seed=73)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("glu", q, s, n, k, group, bf16)
    cc = dec.cc
    px, pg, pa, pb = cc.to_device(x), cc.alloc(t * n * 4), cc.alloc(t * (n // 2) * 2), cc.alloc(t * (n // 2) * 2)
    path = ops.PATH_STREAM if t <= 64 else ops.PATH_PREFILL
    if t <= 64:
        dec.set_decode_ksplit(-1)  # the gated streaming kernel never splits over k: same summation order for the pair
    try:
        dec.lin_forward("glu", px, pg, t, path=path)
    finally:
        dec.set_decode_ksplit(0)
    want_sym = cc.last_launch_symbol()
    dec.silu_mul_f16(pg, n // 2, t, pa)
    dec.lin_forward_glu("glu", px, pb, t)
    got_sym = cc.last_launch_symbol()
    say("   plain:", want_sym, "gated:", got_sym)
    two, one = cc.d2h(pa, (t, n // 2), np.uint16), cc.d2h(pb, (t, n // 2), np.uint16)
    if t > 64 and "splitk" not in want_sym:
        assert got_sym.endswith("_glu") and got_sym[:-4] == want_sym
    assert np.array_equal(one, two)
    # gelu on the same launch shape
    dec.act_mul_f16(pg, n // 2, t, pa, gelu=True)
    dec.lin_forward_glu("glu", px, pb, t, gelu=True)
    assert np.array_equal(cc.d2h(pb, (t, n // 2), np.uint16), cc.d2h(pa, (t, n // 2), np.uint16))
    for p in (px, pg, pa, pb):
        cc.free(p)
    cols = (gen.stream(93, 3000) % np.uint64(n // 2)).astype(np.uint32)
    toks = (gen.stream(94, 3000) % np.uint64(t)).astype(np.uint32)
    gate = orc.gemm_lane_sample(x, q, s, k, group, cols, toks, bf16)
    up = orc.gemm_lane_sample(x, q, s, k, group, cols + np.uint32(n // 2), toks, bf16)
    want = orc.silu_mul_f16_rows(np.stack([gate, up], axis=1).reshape(-1, 2))[:, 0]
    got = one[toks, cols]
    a, b = _f16(got).astype(np.float64), _f16(want).astype(np.float64)
    rms = float(np.sqrt(np.mean(b * b)))
    assert np.all(np.abs(a - b) <= 2 * parity.f16_ulp(np.maximum(np.abs(b), rms / parity.CLAMP_DIV)))
    assert np.mean(got == want) > 0.97


@pytest.mark.parametrize("n,k,group,t", [(1024, 256, 128, 1), (2048, 512, 32, 5), (1024, 256, 128, 16),
                                         (34816, 5120, 128, 4)])
def test_fused_glu_gelu(dec, orc, n, k, group, t):
    """The gelu choice (ew_gelu beside ew): elementwise launch against the oracle, fused kernel bit-identical to linear +
    elementwise launch, and different from the silu result."""
    q, s, x = gen.make_linear(n, k, group, t, seed=72)
    dec.upload_lin_g("glu", q, s, n, k, group, False)
    cc = dec.cc
    px, pg, pa, pb = cc.to_device(x), cc.alloc(t * n * 4), cc.alloc(t * (n // 2) * 2), cc.alloc(t * (n // 2) * 2)
    dec.set_decode_shape(32, 4 if t > 8 or n >= 16384 else 8)
    try:
        dec.lin_forward("glu", px, pg, t, path=ops.PATH_DECODE)
    finally:
        dec.set_decode_shape(0, 0)
    dec.act_mul_f16(pg, n // 2, t, pa, gelu=True)
    dec.lin_forward_glu("glu", px, pb, t, gelu=True)
    gu = cc.d2h(pg, (t, n), np.float32)
    two, one = cc.d2h(pa, (t, n // 2), np.uint16), cc.d2h(pb, (t, n // 2), np.uint16)
    dec.lin_forward_glu("glu", px, pb, t)
    silu = cc.d2h(pb, (t, n // 2), np.uint16)
    for p in (px, pg, pa, pb):
        cc.free(p)
    assert np.array_equal(one, two)
    assert np.mean(one != silu) > 0.5
    want = orc.gelu_mul_f16_rows(gu)  # the device's own f32 GEMM result through the oracle's elementwise step
    a, b = _f16(two).astype(np.float64), _f16(want).astype(np.float64)
    assert np.all(np.abs(a - b) <= parity.f16_ulp(b))  # tanhf from two libraries: last f32 bit ahead of the rounding
    assert np.mean(two == want) > 0.99
    with pytest.raises(ops.W4a16Error):  # an activation that does not exist
        ffi.check(dec.cc.lib.w4a16_act_mul_f16(dec.cc.h, 1, 8, 1, 1, 7))
    with pytest.raises(ops.W4a16Error):
        ffi.check(dec.cc.lib.w4a16_lin_forward_glu_act(dec.cc.h, b"glu", 1, 1, 1, 7))


def test_fused_glu_errors(dec):
    dec.upload_lin_synth("glu_odd", 48, 256, 128, 1, 2)  # n = 48: halves are not whole row blocks
    with pytest.raises(ops.W4a16Error):
        dec.lin_forward_glu("glu_odd", 1, 1, 1)
    with pytest.raises(ops.W4a16Error):
        dec.lin_forward_glu("glu_odd", 1, 1, 17)  # the same contract beyond the decode regime (refused before any launch)
    dec.upload_lin_synth("glu_ok", 64, 256, 128, 1, 2)
    with pytest.raises(ops.W4a16Error):
        dec.lin_forward_glu("glu_ok", 1, 1, 0)
    with pytest.raises(ops.W4a16Error):
        dec.lin_forward_glu("glu_ok", 0, 1, 17)  # null operand


# ------------------------------------------------------------------ the chain
def _host_lins(seeds, prefix, layer, shapes, group):
    out = []
    for role in ops.W4a16Dec.CHAIN_ROLES:
        n, k = shapes[role]
        sq, ss = seeds["%s.%d.%s" % (prefix, layer, role)]
        out.append((gen.weights_q(sq, n, k), gen.scales_f16(ss, n, k, group), n, k))
    return out


def _chain_stagewise(dec, orc, prefix, seeds, shapes, group, layers, t, x, threads):
    """Run the layers one stage at a time through the C ABI; every GEMM is checked against the lane oracle on the
    device's own input of that stage, the RMS glue bit for bit, the activation glue to one f16 step."""
    cc = dec.cc
    hidden, n_ff = shapes["attn_output"][0], shapes["ffn_down"][1]
    cur = x
    for l in range(layers):
        lins = _host_lins(seeds, prefix, l, shapes, group)
        names = ["%s.%d.%s" % (prefix, l, r) for r in ops.W4a16Dec.CHAIN_ROLES]

        def gemm(i, xin):
            got = dec.gemv_host(names[i], xin, t=t)
            q, s, n, k = lins[i]
            want = orc.gemm_lane(xin, t, q, s, n, k, group, False, threads)
            parity.assert_close(got, want, "layer %d %s" % (l, names[i]))
            return got

        def rms(v, ncols):
            pv, po = cc.to_device(v), cc.alloc(t * ncols * 2)
            dec.rms_rescale_f16(pv, v.shape[1], ncols, t, po)
            got = cc.d2h(po, (t, ncols), np.uint16)
            cc.free(pv)
            cc.free(po)
            assert np.array_equal(got, orc.rms_rescale_f16(v, ncols)), "layer %d rms" % l
            return got

        a = rms(gemm(0, cur), hidden)
        b = rms(gemm(1, a), hidden)
        gu = gemm(2, b)
        pg, po = cc.to_device(gu), cc.alloc(t * n_ff * 2)
        dec.silu_mul_f16(pg, n_ff, t, po)
        c = cc.d2h(po, (t, n_ff), np.uint16)
        cc.free(pg)
        cc.free(po)
        cw = orc.silu_mul_f16_rows(gu)
        assert np.all(np.abs(_f16(c).astype(np.float64) - _f16(cw)) <= parity.f16_ulp(_f16(cw))), "layer %d act" % l
        cur = rms(gemm(3, c), hidden)
    return cur


def _chain_oracle(orc, prefix, seeds, shapes, group, layers, x, threads):
    cur = x
    for l in range(layers):
        cur = orc.chain_layer(cur, _host_lins(seeds, prefix, l, shapes, group), group, threads)["x"]
    return cur


@pytest.mark.parametrize("t", [1, 4, 16])
def test_chain_small_many_layers(dec, orc, t):
    """24 small layers: stage-wise parity, the one-call chain equals the staged run bit for bit, and the end-to-end
    result stays close to the oracle's independent run."""
    say("chain small", t)
    hidden, n_qkv, n_ff, group, layers = 256, 384, 512, 128, 24
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("small", layers, hidden, n_qkv, n_ff, group)
    x = gen.normal_f16(31 + t, (t, hidden))
    staged = _chain_stagewise(dec, orc, "small", seeds, shapes, group, layers, t, x, 4)
    cc = dec.cc
    px, py = cc.to_device(x), cc.alloc(t * hidden * 2)
    dec.chain_forward("small", 0, layers, px, t, py)
    got = cc.d2h(py, (t, hidden), np.uint16)
    assert np.array_equal(got, staged)
    # two half chains compose to the whole
    dec.chain_forward("small", 0, 10, px, t, py)
    dec.chain_forward("small", 10, layers - 10, py, t, py)
    assert np.array_equal(cc.d2h(py, (t, hidden), np.uint16), staged)
    want = _chain_oracle(orc, "small", seeds, shapes, group, layers, x, 4)
    m = parity.compare(_f16(got), _f16(want))
    say("  end to end rel_l2", m["rel_l2"], "identical", float(np.mean(got == want)))
    assert m["rel_l2"] < 2e-2  # rounding flips of f16 intermediates accumulate over 96 linears
    ms, _ = dec.bench_chain("small", layers, px, t, py, reps=3, warmup=1, use_graph=True)
    assert np.array_equal(cc.d2h(py, (t, hidden), np.uint16), staged)  # graph replays give the same bits
    cc.free(px)
    cc.free(py)


@pytest.mark.parametrize("t", [40, 200])
def test_chain_prefill_regime(dec, orc, t):
    """The chain at prefill row counts (reference: chain_t_sel / forward_prefill, w4a16_dec/prefill.rs:81-207,
    graphs.rs:368): 40 rows run the weight-streaming kernels, 200 the MFMA tiles; gate|up carries the SiLU*up epilogue
    in both.  Stage-wise parity against the oracle, the one-call chain equal to the staged run bit for bit, and the
    end-to-end result close to the oracle's independent run."""
    say("chain prefill regime", t)
    hidden, n_qkv, n_ff, group, layers = 256, 384, 512, 128, 6
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("pfc", layers, hidden, n_qkv, n_ff, group)
    x = gen.normal_f16(57 + t, (t, hidden))
    cc = dec.cc
    # the gated streaming kernel never splits over k; the staged run's plain gate|up launch must sum in the same order
    dec.set_decode_ksplit(-1)
    try:
        staged = _chain_stagewise(dec, orc, "pfc", seeds, shapes, group, layers, t, x, 8)
        px, py = cc.to_device(x), cc.alloc(t * hidden * 2)
        dec.chain_forward("pfc", 0, layers, px, t, py)
        got = cc.d2h(py, (t, hidden), np.uint16)
    finally:
        dec.set_decode_ksplit(0)
    assert np.array_equal(got, staged)
    want = _chain_oracle(orc, "pfc", seeds, shapes, group, layers, x, 8)
    m = parity.compare(_f16(got), _f16(want))
    say("  end to end rel_l2", m["rel_l2"], "identical", float(np.mean(got == want)))
    assert m["rel_l2"] < 1e-2
    cc.free(px)
    cc.free(py)


def test_chain_27b_layer_shapes(dec, orc):
    """Two layers at the 27B-dense shapes (QKV 5120x7168, O 5120x5120, gate+up 5120x34816, down 17408x5120), M = 4."""
    hidden, n_qkv, n_ff, group, layers, t = 5120, 7168, 17408, 128, 2, 4
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("d27", layers, hidden, n_qkv, n_ff, group)
    x = gen.normal_f16(4, (t, hidden))
    say("chain 27b staged")
    staged = _chain_stagewise(dec, orc, "d27", seeds, shapes, group, layers, t, x, 16)
    cc = dec.cc
    px, py = cc.to_device(x), cc.alloc(t * hidden * 2)
    dec.chain_forward("d27", 0, layers, px, t, py)
    got = cc.d2h(py, (t, hidden), np.uint16)
    cc.free(px)
    cc.free(py)
    assert np.array_equal(got, staged)


def test_chain_errors(dec):
    with pytest.raises(ops.W4a16Error):
        dec.chain_forward("nochain", 0, 1, 1, 1, 1)
    dec.upload_lin_synth("brk.0.attn_qkv", 64, 128, 128, 1, 2)
    dec.upload_lin_synth("brk.0.attn_output", 128, 128, 128, 1, 2)
    dec.upload_lin_synth("brk.0.ffn_gate_up", 256, 128, 128, 1, 2)
    dec.upload_lin_synth("brk.0.ffn_down", 128, 128, 128, 1, 2)
    with pytest.raises(ops.W4a16Error):  # qkv narrower than hidden
        dec.chain_forward("brk", 0, 1, 1, 1, 1)


# ------------------------------------------------------------------ normalisation deferred across a linear
@pytest.mark.parametrize("t,group", [(1, 128), (4, 128), (6, 128), (16, 128), (3, 32)])
def test_deferred_norm_linear(dec, orc, t, group):
    """y = s * (W x) with s from the producer's partial sums, x a column slice of a wider matrix, and the launch's own
    partial sums over the first stat_rows outputs — for every launch shape; bits repeat from run to run."""
    n, k, ldx, stat_rows, in_cols, n_in = 400, 1024, 1536, 300, 777, 7
    q, s, _ = gen.make_linear(n, k, group, 1, seed=21 + t)
    dec.upload_lin_g("dn", q, s, n, k, group, False)
    xw = gen.normal_f16(5 + t, (t, ldx))
    x = np.ascontiguousarray(xw[:, :k])
    rng = np.random.default_rng(t)
    prev = (rng.standard_normal((n_in, 16)) ** 2 * 100).astype(np.float32)
    s_in = (1.0 / np.sqrt(prev.astype(np.float64).sum(0)[:t] / in_cols + 1e-6)).astype(np.float32)
    lane = orc.gemm_lane(x, t, q, s, n, k, group, False, 4)
    want = (s_in[:, None] * lane).astype(np.float32)
    cc = dec.cc
    cap = ((n + 15) // 16) * 64
    px, pp, py, ps = cc.to_device(xw), cc.to_device(prev), cc.alloc(t * n * 4), cc.alloc(cap)
    try:
        for rows, waves in ((0, 0), (16, 4), (32, 8), (64, 2), (16, 1)):
            say("deferred norm", t, group, rows, waves)
            dec.set_decode_shape(rows, waves)
            cc.memset0(ps, cap)
            n_out = dec.lin_forward_deferred_norm("dn", px, t, py, ldx=ldx, stats_in=pp, n_stats_in=n_in, in_cols=in_cols,
                                                  stats_out=ps, stat_rows=stat_rows)
            y = cc.d2h(py, (t, n), np.float32)
            st = cc.d2h(ps, (n_out, 16), np.float32)
            parity.assert_close(y, want, "deferred norm t%d rows%d waves%d" % (t, rows, waves))
            assert 1 <= n_out <= (n + 15) // 16
            got_ss = st.astype(np.float64).sum(0)[:t]
            want_ss = (y[:, :stat_rows].astype(np.float64) ** 2).sum(1)  # the launch's own outputs
            assert np.all(np.abs(got_ss / want_ss - 1.0) < 1e-5)
            # f16 output: the scaled f32 value rounded once
            n2 = dec.lin_forward_deferred_norm("dn", px, t, py, out_f16=True, ldx=ldx, stats_in=pp, n_stats_in=n_in,
                                               in_cols=in_cols, stats_out=ps, stat_rows=stat_rows)
            y16 = cc.d2h(py, (t, n), np.uint16)
            assert n2 == n_out and np.array_equal(y16, gen.f32_to_f16_bits(y))
            assert np.array_equal(cc.d2h(ps, (n_out, 16), np.float32)[:, :t], st[:, :t])  # same bits every run
        dec.set_decode_shape(0, 0)
        # split over k across workgroups: the workgroup that adds the slices applies the factor and leaves the sums
        dec.set_decode_ksplit(2)
        cc.memset0(ps, cap)
        n_out = dec.lin_forward_deferred_norm("dn", px, t, py, ldx=ldx, stats_in=pp, n_stats_in=n_in, in_cols=in_cols,
                                              stats_out=ps, stat_rows=stat_rows)
        y = cc.d2h(py, (t, n), np.float32)
        parity.assert_close(y, want, "deferred norm t%d, two k slices" % t)
        got_ss = cc.d2h(ps, (n_out, 16), np.float32).astype(np.float64).sum(0)[:t]
        assert np.all(np.abs(got_ss / (y[:, :stat_rows].astype(np.float64) ** 2).sum(1) - 1.0) < 1e-5)
        dec.set_decode_ksplit(0)
        # without statistics either way it is the plain decode launch
        dec.lin_forward_deferred_norm("dn", px, t, py, ldx=ldx)
        plain = dec.gemv_host("dn", x, t=t, path=ops.PATH_DECODE)
        assert np.array_equal(cc.d2h(py, (t, n), np.float32).view(np.uint32), plain.view(np.uint32))
    finally:
        dec.set_decode_shape(0, 0)
        dec.set_decode_ksplit(0)
        for p_ in (px, pp, py, ps):
            cc.free(p_)


def test_deferred_norm_many_partial_sums_and_glu(dec, orc):
    """More partial sums than one staging pass holds (8 x 64 entries), and the gated projection: the factor reaches
    gate and up before silu(g) * u."""
    n, k, t, n_in, in_cols = 512, 512, 5, 700, 4096
    q, s, x = gen.make_linear(n, k, 128, t, seed=77)
    dec.upload_lin_g("dg", q, s, n, k, 128, False)
    prev = (np.random.default_rng(9).standard_normal((n_in, 16)) ** 2).astype(np.float32)
    s_in = (1.0 / np.sqrt(prev.astype(np.float64).sum(0)[:t] / in_cols + 1e-6)).astype(np.float32)
    gu = (s_in[:, None] * orc.gemm_lane(x, t, q, s, n, k, 128, False, 4)).astype(np.float32)
    cc = dec.cc
    px, pp, py, pc = cc.to_device(x), cc.to_device(prev), cc.alloc(t * n * 4), cc.alloc(t * (n // 2) * 2)
    try:
        dec.lin_forward_deferred_norm("dg", px, t, py, stats_in=pp, n_stats_in=n_in, in_cols=in_cols)
        parity.assert_close(cc.d2h(py, (t, n), np.float32), gu, "deferred norm, 700 partial sums")
        dec.lin_forward_glu_deferred_norm("dg", px, t, pc, stats_in=pp, n_stats_in=n_in, in_cols=in_cols)
        c = cc.d2h(pc, (t, n // 2), np.uint16)
        cw = orc.silu_mul_f16_rows(gu)
        assert np.all(np.abs(_f16(c).astype(np.float64) - _f16(cw)) <= parity.f16_ulp(_f16(cw)))
        with pytest.raises(ops.W4a16Error):  # x rows closer together than k
            dec.lin_forward_deferred_norm("dg", px, t, py, ldx=k - 8)
        with pytest.raises(ops.W4a16Error):  # statistics without their count
            dec.lin_forward_deferred_norm("dg", px, t, py, stats_in=pp, n_stats_in=0, in_cols=in_cols)
    finally:
        for p_ in (px, pp, py, pc):
            cc.free(p_)


@pytest.mark.parametrize("t,n,k,group,ksplit", [(40, 400, 1024, 128, -1), (300, 400, 1024, 128, -1), (130, 2048, 4096, 128, 0),
                                                (130, 2048, 4096, 128, 4), (100, 320, 512, 32, -1), (600, 5120, 5120, 128, 0)])
def test_deferred_norm_linear_beyond_the_decode_regime(dec, orc, t, n, k, group, ksplit):
    """The same options on the MFMA-tiled kernel (t > 16): row factor from partial sums laid out [entries][ld], x a column
    slice of a wider matrix, residual stream, statistics of the output (whole k range: one entry per 64 columns; split
    over k: one per 1024-column chunk, applied by the finish kernel), norm weight, power-of-two hand-over factors."""
    say("deferred norm prefill", t, n, k, group, ksplit)
    ldx, in_cols, n_in = k + 512, 777, 37
    stat_rows = n - 100
    q, s, _ = gen.make_linear(n, k, group, 1, seed=121 + t)
    dec.upload_lin_g("dnp", q, s, n, k, group, False)
    xw = gen.normal_f16(15 + t, (t, ldx))
    x = np.ascontiguousarray(xw[:, :k])
    rng = np.random.default_rng(t)
    ld = (t + 3) // 4 * 4
    prev = np.zeros((n_in, ld), np.float32)
    prev[:, :t] = (rng.standard_normal((n_in, t)) ** 2 * 100).astype(np.float32)
    s_in = (1.0 / np.sqrt(prev.astype(np.float64).sum(0)[:t] / in_cols + 1e-6)).astype(np.float32)
    if n * t <= 1 << 18:
        lane = orc.gemm_lane(x, t, q, s, n, k, group, False, 16)
    else:
        cc_ = dec.cc
        pxx, pyy = cc_.to_device(x), cc_.alloc(t * n * 4)
        dec.lin_forward("dnp", pxx, pyy, t, path=ops.PATH_LANE)
        lane = cc_.d2h(pyy, (t, n), np.float32)
        cc_.free(pxx)
        cc_.free(pyy)
    resid0 = (rng.standard_normal((t, n)) * 0.5).astype(np.float32)
    nw = (1.0 + 0.3 * rng.standard_normal(n)).astype(np.float32)
    cc = dec.cc
    cap = ((n + 63) // 64) * ld * 4
    px, pp, py, ps = cc.to_device(xw), cc.to_device(prev), cc.alloc(t * n * 4), cc.alloc(cap)
    pr, pw = cc.to_device(resid0), cc.to_device(nw)
    dec.set_prefill_ksplit(ksplit)
    try:
        # factor + statistics
        cc.memset0(ps, cap)
        n_out = dec.lin_forward_deferred_norm("dnp", px, t, py, ldx=ldx, stats_in=pp, n_stats_in=n_in, in_cols=in_cols,
                                              stats_out=ps, stat_rows=stat_rows)
        say("   ", cc.last_launch_symbol(), "entries", n_out)
        y = cc.d2h(py, (t, n), np.float32)
        want = (s_in[:, None] * lane).astype(np.float32)
        parity.assert_close(y, want, "deferred norm prefill t%d" % t)
        st = cc.d2h(ps, (n_out, ld), np.float32)
        got_ss = st.astype(np.float64).sum(0)[:t]
        want_ss = (y[:, :stat_rows].astype(np.float64) ** 2).sum(1)
        assert np.all(np.abs(got_ss / want_ss - 1.0) < 1e-5)
        # f16 out = the f32 value rounded once; the statistics repeat bit for bit
        n2 = dec.lin_forward_deferred_norm("dnp", px, t, py, out_f16=True, ldx=ldx, stats_in=pp, n_stats_in=n_in,
                                           in_cols=in_cols, stats_out=ps, stat_rows=stat_rows)
        assert n2 == n_out and np.array_equal(cc.d2h(py, (t, n), np.uint16), gen.f32_to_f16_bits(y))
        assert np.array_equal(cc.d2h(ps, (n_out, ld), np.float32)[:, :t], st[:, :t])
        # residual stream + norm weight + hand-over factors: v = resid + s_in * 2^3 * (W x); y = f16(v * nw * 2^-2)
        dec.lin_forward_deferred_norm("dnp", px, t, py, out_f16=True, ldx=ldx, stats_in=pp, n_stats_in=n_in, in_cols=in_cols,
                                      stats_out=ps, stat_rows=stat_rows, resid=pr, nw=pw, in_exp=3, out_exp=2)
        v = cc.d2h(pr, (t, n), np.float32)
        v_want = resid0 + (s_in[:, None] * np.float32(8.0)) * lane
        parity.assert_close(v, v_want.astype(np.float32), "residual stream prefill t%d" % t)
        y16 = cc.d2h(py, (t, n), np.uint16)
        assert np.array_equal(y16, gen.f32_to_f16_bits((v * nw[None, :]).astype(np.float32) * np.float32(0.25)))
        got_ss = cc.d2h(ps, (n_out, ld), np.float32).astype(np.float64).sum(0)[:t]
        assert np.all(np.abs(got_ss / (v[:, :stat_rows].astype(np.float64) ** 2).sum(1) - 1.0) < 1e-5)
        # without any option it is the plain prefill launch
        dec.lin_forward_deferred_norm("dnp", px, t, py, ldx=ldx)
        plain = dec.gemv_host("dnp", x, t=t, path=ops.PATH_PREFILL)
        assert np.array_equal(cc.d2h(py, (t, n), np.float32).view(np.uint32), plain.view(np.uint32))
    finally:
        dec.set_prefill_ksplit(0)
        for p_ in (px, pp, py, ps, pr, pw):
            cc.free(p_)


@pytest.mark.parametrize("t", [40, 300])
def test_deferred_norm_glu_beyond_the_decode_regime(dec, orc, t):
    """The gated projection at t > 16: the factor (with its power of two) reaches gate and up before act(g) * u, the
    result leaves times 2^-out_exp."""
    n, k, n_in, in_cols = 1024, 512, 70, 4096
    q, s, x = gen.make_linear(n, k, 128, t, seed=177)
    dec.upload_lin_g("dgp", q, s, n, k, 128, False)
    ld = (t + 3) // 4 * 4
    prev = np.zeros((n_in, ld), np.float32)
    prev[:, :t] = (np.random.default_rng(9).standard_normal((n_in, t)) ** 2).astype(np.float32)
    s_in = (1.0 / np.sqrt(prev.astype(np.float64).sum(0)[:t] / in_cols + 1e-6)).astype(np.float32)
    gu = ((s_in[:, None] * np.float32(4.0)) * orc.gemm_lane(x, t, q, s, n, k, 128, False, 8)).astype(np.float32)
    cc = dec.cc
    px, pp, pc = cc.to_device(x), cc.to_device(prev), cc.alloc(t * (n // 2) * 2)
    try:
        dec.lin_forward_glu_deferred_norm("dgp", px, t, pc, stats_in=pp, n_stats_in=n_in, in_cols=in_cols, in_exp=2, out_exp=1)
        assert dec.cc.last_launch_symbol().endswith("_glu")
        c = _f16(cc.d2h(pc, (t, n // 2), np.uint16)).astype(np.float64) * 2.0
        cw = _f16(orc.silu_mul_f16_rows(gu)).astype(np.float64)
        rms = float(np.sqrt(np.mean(cw * cw)))
        assert np.all(np.abs(c - cw) <= 2 * parity.f16_ulp(np.maximum(np.abs(cw), rms / parity.CLAMP_DIV)))
    finally:
        for p_ in (px, pp, pc):
            cc.free(p_)


@pytest.mark.parametrize("t", [40, 200])
def test_fused_chain_prefill_regime(dec, orc, t):
    """w4a16_chain_forward_fused beyond 16 rows (four launches per layer on the MFMA-tiled kernels, split over k where
    the planner says so): against the oracle's fused statement, against the un-fused chain, deterministic."""
    say("fused chain prefill regime", t)
    hidden, n_qkv, n_ff, group, layers = 1024, 1536, 2048, 128, 4
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("fpf", layers, hidden, n_qkv, n_ff, group)
    x = gen.normal_f16(61 + t, (t, hidden))
    cc = dec.cc
    px, py, pz = cc.to_device(x), cc.alloc(t * hidden * 2), cc.alloc(t * hidden * 2)
    try:
        dec.chain_forward_fused("fpf", 0, layers, px, t, py)
        got = cc.d2h(py, (t, hidden), np.uint16)
        assert np.all(np.isfinite(_f16(got)))
        want = _fused_oracle(orc, "fpf", seeds, shapes, group, layers, x, 8)
        m = parity.compare(_f16(got), _f16(want))
        say("  fused vs oracle rel_l2", m["rel_l2"])
        assert m["rel_l2"] < 1e-2
        dec.chain_forward("fpf", 0, layers, px, t, pz)
        m2 = parity.compare(_f16(got), _f16(cc.d2h(pz, (t, hidden), np.uint16)))
        say("  fused vs unfused rel_l2", m2["rel_l2"])
        assert m2["rel_l2"] < 1e-2
        dec.chain_forward_fused("fpf", 0, layers, px, t, py)
        assert np.array_equal(cc.d2h(py, (t, hidden), np.uint16), got)
    finally:
        for p_ in (px, py, pz):
            cc.free(p_)


@pytest.mark.parametrize("t", [1, 4, 11])
def test_deferred_norm_with_residual_and_norm_weight(dec, orc, t):
    """Two linears with a norm_resid between them (x += ab; xn = x * inv * nw; y = W2 xn16, kernels/mod.rs:11-54),
    as two launches: the first adds its output to the residual stream, leaves the statistics of the sum and emits
    f16(v * nw); the second multiplies by 1/rms(v).  Residual stream and statistics against the oracle of the first
    linear; the final result against the reference sequence (oracle linears around the oracle's norm_resid)."""
    hidden, n2, k1, group = 640, 272, 512, 128
    q1, s1, x = gen.make_linear(hidden, k1, group, t, seed=300 + t)
    q2, s2, _ = gen.make_linear(n2, hidden, group, 1, seed=310 + t)
    dec.upload_lin_g("nr1", q1, s1, hidden, k1, group, False)
    dec.upload_lin_g("nr2", q2, s2, n2, hidden, group, False)
    rng = np.random.default_rng(40 + t)
    resid0 = (rng.standard_normal((t, hidden)) * 3).astype(np.float32)
    nw = (1.0 + 0.3 * rng.standard_normal(hidden)).astype(np.float32)
    # reference sequence
    ab = orc.gemm_lane(x, t, q1, s1, hidden, k1, group, False, 4)
    ref_x, _, _, ref_xn16 = orc.norm_resid(resid0, nw, ab)
    want = orc.gemm_lane(ref_xn16, t, q2, s2, n2, hidden, group, False, 4)
    cc = dec.cc
    cap = ((hidden + 15) // 16) * 64
    px, pr, pw = cc.to_device(x), cc.to_device(resid0), cc.to_device(nw)
    pa, ps, py = cc.alloc(t * hidden * 2), cc.alloc(cap), cc.alloc(t * n2 * 4)
    try:
        cc.memset0(ps, cap)  # token columns >= t are never written
        n_st = dec.lin_forward_deferred_norm("nr1", px, t, pa, out_f16=True, stats_out=ps, stat_rows=hidden, resid=pr, nw=pw)
        v = cc.d2h(pr, (t, hidden), np.float32)
        parity.assert_close(v, ref_x, "residual stream t%d" % t)
        a16 = cc.d2h(pa, (t, hidden), np.uint16)
        assert np.array_equal(a16, gen.f32_to_f16_bits((v * nw[None, :]).astype(np.float32)))  # one f32 product, one rounding
        ss = cc.d2h(ps, (n_st, 16), np.float32).astype(np.float64).sum(0)[:t]
        assert np.all(np.abs(ss / (v.astype(np.float64) ** 2).sum(1) - 1.0) < 1e-5)
        dec.lin_forward_deferred_norm("nr2", pa, t, py, stats_in=ps, n_stats_in=n_st, in_cols=hidden)
        got = cc.d2h(py, (t, n2), np.float32)
        m = parity.compare(got, want)
        say("  norm_resid deferred t", t, "rel_l2", m["rel_l2"])
        assert m["rel_l2"] < 1e-3  # the f16 rounding of the activations falls before the 1/rms factor instead of after
        with pytest.raises(ops.W4a16Error):  # the gated projection takes neither
            dec.lin_forward_glu_deferred_norm("nr1", px, t, pa, stats_in=ps, n_stats_in=0, in_cols=hidden)
    finally:
        for p_ in (px, pr, pw, pa, ps, py):
            cc.free(p_)


def test_deferred_norm_residual_outlier_needs_and_gets_a_scaled_handover(dec, orc):
    """A residual stream with elements around 1e5 (times a norm weight): norm_resid normalises in f32 first and stays
    finite; the un-scaled f16 hand-over carries Inf, the hand-over with out_exp = 3 / in_exp = 3 gives the reference
    sequence's result."""
    t, hidden, n2, k1, group = 4, 640, 272, 512, 128
    q1, s1, x = gen.make_linear(hidden, k1, group, t, seed=331)
    q2, s2, _ = gen.make_linear(n2, hidden, group, 1, seed=332)
    dec.upload_lin_g("no1", q1, s1, hidden, k1, group, False)
    dec.upload_lin_g("no2", q2, s2, n2, hidden, group, False)
    rng = np.random.default_rng(77)
    resid0 = (rng.standard_normal((t, hidden)) * 3).astype(np.float32)
    resid0[:, 5] = np.float32(1.0e5)
    resid0[1, 77] = np.float32(-2.3e5)
    nw = (1.0 + 0.3 * rng.standard_normal(hidden)).astype(np.float32)
    nw[5] = np.float32(1.5)
    ab = orc.gemm_lane(x, t, q1, s1, hidden, k1, group, False, 4)
    _, _, _, ref_xn16 = orc.norm_resid(resid0, nw, ab)
    want = orc.gemm_lane(ref_xn16, t, q2, s2, n2, hidden, group, False, 4)
    assert np.all(np.isfinite(want))
    cc = dec.cc
    cap = ((hidden + 15) // 16) * 64
    px, pw = cc.to_device(x), cc.to_device(nw)
    pa, ps, py = cc.alloc(t * hidden * 2), cc.alloc(cap), cc.alloc(t * n2 * 4)
    try:
        for e, finite in ((0, False), (3, True)):
            pr = cc.to_device(resid0)
            cc.memset0(ps, cap)
            n_st = dec.lin_forward_deferred_norm("no1", px, t, pa, out_f16=True, stats_out=ps, stat_rows=hidden, resid=pr,
                                                 nw=pw, in_exp=0, out_exp=e)
            a = _f16(cc.d2h(pa, (t, hidden), np.uint16))
            assert bool(np.all(np.isfinite(a))) == finite
            dec.lin_forward_deferred_norm("no2", pa, t, py, stats_in=ps, n_stats_in=n_st, in_cols=hidden, in_exp=e, out_exp=0)
            got = cc.d2h(py, (t, n2), np.float32)
            cc.free(pr)
            if finite:
                m = parity.compare(got, want)
                say("  outlier residual, scaled hand-over: rel_l2", m["rel_l2"])
                assert m["rel_l2"] < 1e-3
            else:
                assert not np.all(np.isfinite(got))
    finally:
        for p_ in (px, pw, pa, ps, py):
            cc.free(p_)


def _fused_oracle(orc, prefix, seeds, shapes, group, layers, x, threads):
    cur, sc = x, np.ones(x.shape[0], np.float32)
    for l in range(layers):
        st = orc.chain_layer_fused(cur, sc, _host_lins(seeds, prefix, l, shapes, group), group, threads)
        cur, sc = st["x"], st["s"]
    return orc.rms_rescale_f16(st["v4"], shapes["attn_output"][0])


@pytest.mark.parametrize("t", [1, 4, 13])
def test_fused_chain_small_many_layers(dec, orc, t):
    """24 small layers with the normalisations deferred across the linears: close to the oracle's statement of the
    same chain and to the chain that keeps the normalisation launches; graph replays repeat the eager bits."""
    say("fused chain small", t)
    hidden, n_qkv, n_ff, group, layers = 256, 384, 512, 128, 24
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("fsmall", layers, hidden, n_qkv, n_ff, group)
    x = gen.normal_f16(131 + t, (t, hidden))
    cc = dec.cc
    px, py, pz = cc.to_device(x), cc.alloc(t * hidden * 2), cc.alloc(t * hidden * 2)
    try:
        dec.chain_forward_fused("fsmall", 0, layers, px, t, py)
        got = cc.d2h(py, (t, hidden), np.uint16)
        want = _fused_oracle(orc, "fsmall", seeds, shapes, group, layers, x, 4)
        m = parity.compare(_f16(got), _f16(want))
        say("  fused vs oracle rel_l2", m["rel_l2"])
        assert m["rel_l2"] < 2e-2  # rounding flips of f16 intermediates accumulate over 96 linears
        dec.chain_forward("fsmall", 0, layers, px, t, pz)
        m2 = parity.compare(_f16(got), _f16(cc.d2h(pz, (t, hidden), np.uint16)))
        say("  fused vs unfused rel_l2", m2["rel_l2"])
        assert m2["rel_l2"] < 2e-2
        for _ in range(2):
            dec.chain_forward_fused("fsmall", 0, layers, px, t, py)
            assert np.array_equal(cc.d2h(py, (t, hidden), np.uint16), got)  # deterministic
        dec.bench_chain("fsmall", layers, px, t, py, reps=3, warmup=1, use_graph=True, fused=True)
        assert np.array_equal(cc.d2h(py, (t, hidden), np.uint16), got)  # graph replays give the same bits
    finally:
        for p_ in (px, py, pz):
            cc.free(p_)


def test_fused_chain_27b_layer_shapes(dec, orc):
    """Two layers at the 27B-dense shapes, M = 4: stage by stage against the oracle's fused statement on the device's
    own inputs would repeat test_deferred_norm_linear; here the end-to-end result against the oracle."""
    hidden, n_qkv, n_ff, group, layers, t = 5120, 7168, 17408, 128, 2, 4
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("f27", layers, hidden, n_qkv, n_ff, group)
    x = gen.normal_f16(4, (t, hidden))
    cc = dec.cc
    px, py = cc.to_device(x), cc.alloc(t * hidden * 2)
    say("fused chain 27b")
    dec.chain_forward_fused("f27", 0, layers, px, t, py)
    got = cc.d2h(py, (t, hidden), np.uint16)
    cc.free(px)
    cc.free(py)
    want = _fused_oracle(orc, "f27", seeds, shapes, group, layers, x, 16)
    m = parity.compare(_f16(got), _f16(want))
    say("  rel_l2", m["rel_l2"], "identical", float(np.mean(got == want)))
    assert m["rel_l2"] < 3e-3


# ------------------------------------------------------------------ hand-overs with a power-of-two factor
@pytest.mark.parametrize("n,k,group,bf16", [(512, 1024, 128, False), (200, 256, 32, True), (5120, 17408, 128, False)])
def test_row_norm_max_matches_numpy(dec, orc, n, k, group, bf16):
    """max_r sqrt(sum_c ((nib-8)*scale)^2) against float64 over the oracle's dequantised weights; a second request
    returns the kept value."""
    say("row norm", n, k, group, bf16)
    q, s, _ = gen.make_linear(n, k, group, 1, seed=61)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("rn", q, s, n, k, group, bf16)
    w = orc.dequant_matrix(q, s, n, k, group, scale_bf16=bf16).astype(np.float64)
    want = float(np.max(np.sqrt(np.sum(w * w, axis=1))))
    got = dec.row_norm_max("rn")
    assert abs(got - want) <= 2e-5 * want, (got, want)
    assert dec.row_norm_max("rn") == got


def _pow2(bits16, e):
    """f16 bit patterns times 2^e, exact (the caller keeps the values inside the normal range)."""
    return gen.f32_to_f16_bits(np.ldexp(gen.f16_bits_to_f32(bits16), e).astype(np.float32))


@pytest.mark.parametrize("e", [-3, 4])
@pytest.mark.parametrize("t", [1, 4, 11])
def test_scaled_handover_is_exact(dec, e, t):
    """A power-of-two factor on a hand-over changes nothing but the exponent: the producer's f16 output with out_exp = e
    is its un-scaled output times 2^-e bit for bit (statistics unchanged), and a consumer given x * 2^-e with in_exp = e
    returns the bits it returns for x — plain and gated, with and without input statistics."""
    say("scaled hand-over", e, t)
    cc = dec.cc
    n1, k1, n2 = 1024, 512, 512
    q1, s1, x = gen.make_linear(n1, k1, 128, t, seed=71)
    q2, s2, _ = gen.make_linear(n2, n1, 128, 1, seed=72)
    dec.upload_lin_g("sh1", q1, s1, n1, k1, 128, False)
    dec.upload_lin_g("sh2", q2, s2, n2, n1, 128, False)
    px = cc.to_device(x)
    pa, pb = cc.alloc(t * n1 * 2), cc.alloc(t * n1 * 2)
    sa, sb = cc.alloc((n1 // 16) * 64), cc.alloc((n1 // 16) * 64)
    py, pz, pg, ph = cc.alloc(t * n2 * 4), cc.alloc(t * n2 * 4), cc.alloc(t * (n2 // 2) * 2), cc.alloc(t * (n2 // 2) * 2)
    try:
        na = dec.lin_forward_deferred_norm("sh1", px, t, pa, out_f16=True, stats_out=sa, stat_rows=n1)
        nb = dec.lin_forward_deferred_norm("sh1", px, t, pb, out_f16=True, stats_out=sb, stat_rows=n1, in_exp=0, out_exp=e)
        a, b = cc.d2h(pa, (t, n1), np.uint16), cc.d2h(pb, (t, n1), np.uint16)
        assert na == nb and np.array_equal(cc.d2h(sa, (na, 16), np.uint32)[:, :t], cc.d2h(sb, (nb, 16), np.uint32)[:, :t])
        av = np.abs(gen.f16_bits_to_f32(a))
        normal = (np.ldexp(av, -e) >= 6.2e-5) & (av >= 6.2e-5)  # f16 subnormals round on a different grid
        assert normal.mean() > 0.99
        assert np.array_equal(_pow2(a, -e)[normal], b[normal])
        # consumer: the scaled activations with in_exp = e against the un-scaled ones, statistics in both
        cc.h2d(pb, _pow2(a, -e))  # exact copies, subnormal elements included in neither comparison
        a_clean = np.where(normal, a, 0).astype(np.uint16)
        cc.h2d(pa, a_clean)
        cc.h2d(pb, _pow2(a_clean, -e))
        for stats in (0, sa):
            kw = dict(stats_in=stats, n_stats_in=na if stats else 0, in_cols=n1 if stats else 0)
            dec.lin_forward_deferred_norm("sh2", pa, t, py, **kw)
            dec.lin_forward_deferred_norm("sh2", pb, t, pz, in_exp=e, out_exp=0, **kw)
            assert np.array_equal(cc.d2h(py, (t, n2), np.uint32), cc.d2h(pz, (t, n2), np.uint32))
            dec.lin_forward_glu_deferred_norm("sh2", pa, t, pg, **kw)
            dec.lin_forward_glu_deferred_norm("sh2", pb, t, ph, in_exp=e, out_exp=0, **kw)
            g0 = cc.d2h(pg, (t, n2 // 2), np.uint16)
            assert np.array_equal(g0, cc.d2h(ph, (t, n2 // 2), np.uint16))
            dec.lin_forward_glu_deferred_norm("sh2", pb, t, ph, in_exp=e, out_exp=e, **kw)
            gv = np.abs(gen.f16_bits_to_f32(g0))
            ok = (np.ldexp(gv, -e) >= 6.2e-5) & (gv >= 6.2e-5) & (np.ldexp(gv, -e) < 6.0e4)
            assert np.array_equal(_pow2(g0, -e)[ok], cc.d2h(ph, (t, n2 // 2), np.uint16)[ok]) and ok.mean() > 0.9
        with pytest.raises(ops.W4a16Error):
            dec.lin_forward_deferred_norm("sh2", pa, t, py, in_exp=121, out_exp=0)
    finally:
        for p_ in (px, pa, pb, sa, sb, py, pz, pg, ph):
            cc.free(p_)


@pytest.mark.parametrize("rows", [2, 65])
def test_scaled_handover_error_bound_with_a_large_exponent(dec, rows):
    """A hand-over factor far larger than the values need (out_exp = 9 on outputs of magnitude ~1): elements below
    2^(out_exp - 14) leave as f16 subnormals.  Against the f32 output of the same launch shape the handed-over value times
    2^out_exp is within half an f16 step of a normal value or 2^(out_exp - 25) of a subnormal one, the bound the header
    states — in the decode kernel (2 rows) and in the MFMA-tiled one (65 rows)."""
    say("scaled hand-over bound", rows)
    cc = dec.cc
    n1, k1, e = 1024, 512, 9
    q1, s1, x = gen.make_linear(n1, k1, 128, rows, seed=81)
    dec.upload_lin_g("shb", q1, s1, n1, k1, 128, False)
    px, pf, ph = cc.to_device(x), cc.alloc(rows * n1 * 4), cc.alloc(rows * n1 * 2)
    try:
        dec.lin_forward_deferred_norm("shb", px, rows, pf, out_f16=False, in_exp=0, out_exp=0)
        dec.lin_forward_deferred_norm("shb", px, rows, ph, out_f16=True, in_exp=0, out_exp=e)
        v = cc.d2h(pf, (rows, n1), np.float32).astype(np.float64)
        got = np.ldexp(gen.f16_bits_to_f32(cc.d2h(ph, (rows, n1), np.uint16)).astype(np.float64), e)
        small = np.abs(v) < 2.0 ** (e - 14)
        assert small.mean() > 0.01 and (~small).mean() > 0.5  # both kinds occur
        bound = np.where(small, 2.0 ** (e - 25), np.abs(v) * 2.0 ** -11)
        assert np.all(np.abs(got - v) <= bound * 1.0000001), float((np.abs(got - v) / bound).max())
    finally:
        for p_ in (px, pf, ph):
            cc.free(p_)


def test_fused_chain_keeps_large_outputs_in_range(dec, orc):
    """Weights thirty times larger than the other chains': the down projection's output passes 65504, so an un-scaled
    f16 hand-over would carry Inf across the layer boundary.  The chain with the normalisations deferred stays finite
    and agrees with the chain that normalises in f32 first."""
    hidden, n_qkv, n_ff, group, layers, t = 256, 384, 512, 128, 3, 4
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    seeds = dec.upload_chain_synth("fbig", layers, hidden, n_qkv, n_ff, group, lo=0.06, hi=0.6)
    x = gen.normal_f16(77, (t, hidden))
    lins0 = []
    for role in ops.W4a16Dec.CHAIN_ROLES:
        n, k = shapes[role]
        sq, ss = seeds["fbig.0.%s" % role]
        lins0.append((gen.weights_q(sq, n, k), gen.scales_f16(ss, n, k, group, 0.06, 0.6), n, k))
    v4 = orc.chain_layer_fused(x, np.ones(t, np.float32), lins0, group, 4)["v4"]
    say("fused chain, large weights: max |v4| of layer 0 =", float(np.max(np.abs(v4))))
    assert np.max(np.abs(v4)) > 65504.0
    cc = dec.cc
    px, py, pz = cc.to_device(x), cc.alloc(t * hidden * 2), cc.alloc(t * hidden * 2)
    try:
        dec.chain_forward_fused("fbig", 0, layers, px, t, py)
        dec.chain_forward("fbig", 0, layers, px, t, pz)
        got, want = _f16(cc.d2h(py, (t, hidden), np.uint16)), _f16(cc.d2h(pz, (t, hidden), np.uint16))
        assert np.all(np.isfinite(got)) and np.all(np.isfinite(want))
        m = parity.compare(got, want)
        say("  fused vs unfused rel_l2", m["rel_l2"])
        assert m["rel_l2"] < 2e-2
    finally:
        for p_ in (px, py, pz):
            cc.free(p_)


# ------------------------------------------------------------------ norm_resid (assets/norm.cu:4-48, 97-148)
@pytest.mark.parametrize("t,hidden,w_off", [(1, 5120, 0), (4, 5120, 5120), (7, 2048, 0), (3, 1000, 24), (2, 8192, 0),
                                            (5, 64, 0)])
@pytest.mark.parametrize("copies", ["both", "f16 only", "none"])
def test_norm_resid_bit_exact(dec, orc, t, hidden, w_off, copies):
    print("norm_resid", t, hidden, w_off, copies, flush=True)
    cc = dec.cc
    x = gen.normal_f32(300 + hidden, (t, hidden)) * np.float32(3.0)
    ab = gen.normal_f32(301 + hidden, (t, hidden))
    nw = (np.float32(1.0) + gen.normal_f32(302 + hidden, (w_off + hidden,)) * np.float32(0.1)).astype(np.float32)
    want_x, want_xn, want_xn32, want_xn16 = orc.norm_resid(x, nw, ab, w_off)
    px, pw, pa = cc.to_device(x), cc.to_device(nw), cc.to_device(ab)
    pn, p32, p16 = cc.alloc(t * hidden * 4), cc.alloc(t * hidden * 4), cc.alloc(t * hidden * 2)
    dec.norm_resid(px, pw, pa, pn, t, hidden, w_off, xn32_dev=p32 if copies == "both" else 0,
                   xn16_dev=0 if copies == "none" else p16)
    got_x, got_xn = cc.d2h(px, (t, hidden), np.float32), cc.d2h(pn, (t, hidden), np.float32)
    assert np.array_equal(got_x.view(np.uint32), want_x.view(np.uint32))
    assert np.array_equal(got_xn.view(np.uint32), want_xn.view(np.uint32))
    if copies != "none":
        assert np.array_equal(cc.d2h(p16, (t, hidden), np.uint16), want_xn16)
    if copies == "both":
        assert np.array_equal(cc.d2h(p32, (t, hidden), np.float32).view(np.uint32), want_xn32.view(np.uint32))
    for p in (px, pw, pa, pn, p32, p16):
        cc.free(p)


def test_norm_resid_feeds_the_linear(dec, orc):
    """The f16 copy is the A operand of the next linear: norm_resid -> decode GEMV against the oracle's lane GEMM of
    the oracle's f16 copy."""
    t, hidden, n = 4, 2048, 512
    cc = dec.cc
    x = gen.normal_f32(11, (t, hidden))
    ab = gen.normal_f32(12, (t, hidden))
    nw = np.ones(hidden, np.float32)
    q, s, _ = gen.make_linear(n, hidden, 128, 1, seed=13)
    dec.upload_lin_g("after_norm", q, s, n, hidden, 128, False)
    _, _, _, x16 = orc.norm_resid(x, nw, ab, 0)
    want = orc.gemm_lane(x16, t, q, s, n, hidden, 128, threads=4)
    px, pw, pa = cc.to_device(x), cc.to_device(nw), cc.to_device(ab)
    pn, p16, py = cc.alloc(t * hidden * 4), cc.alloc(t * hidden * 2), cc.alloc(t * n * 4)
    dec.norm_resid(px, pw, pa, pn, t, hidden, xn16_dev=p16)
    dec.lin_forward("after_norm", p16, py, t, path=ops.PATH_DECODE)
    parity.assert_close(cc.d2h(py, (t, n), np.float32), want, "norm_resid -> decode")
    for p in (px, pw, pa, pn, p16, py):
        cc.free(p)


def test_norm_resid_errors(dec):
    with pytest.raises(ops.W4a16Error):
        dec.norm_resid(1, 1, 1, 1, 1, 8193)
    with pytest.raises(ops.W4a16Error):
        dec.norm_resid(0, 1, 1, 1, 1, 1024)
    with pytest.raises(ops.W4a16Error):
        dec.norm_resid(1, 1, 1, 1, 0, 1024)
