"""CPU checks of the MoE pieces: the oracle's stage functions against independent statements of the same rules, and
the host routing function of the library against the oracle and the reference's known answers."""
import math

import numpy as np
import pytest

from llm170_amd import gen, ops


def _f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


# ---------------------------------------------------------------- act: f16(silu(g) * u)
def test_oracle_act_against_float64(orc):
    rng = np.random.default_rng(5)
    g = (rng.standard_normal(4096) * 4).astype(np.float16)
    u = (rng.standard_normal(4096) * 4).astype(np.float16)
    c13 = np.concatenate([g.view(np.uint16), u.view(np.uint16)])[None, :]
    got = _f16(orc.moe_act_silu_f16(c13, 1, 4096)).ravel()
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64
    # one f16 rounding of an f32 result that itself carries a few f32 roundings
    step = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(got - want) <= 0.51 * step + 1e-7)
    # a dropped factor, a wrong sign in the exponent or gate/up swapped would all miss by far more than a step
    swapped = u64 / (1.0 + np.exp(-u64)) * g64
    assert np.mean(np.abs(got - swapped) > step) > 0.9


def test_oracle_act_special_cases(orc):
    h = lambda v: int(np.float16(v).view(np.uint16))
    def act(g, u):
        return float(_f16(orc.moe_act_silu_f16(np.array([[h(g), h(u)]], np.uint16), 1, 1))[0, 0])
    assert act(0.0, 3.0) == 0.0
    assert act(2.5, 0.0) == 0.0
    assert act(30.0, 2.0) == 60.0          # silu(g) -> g for large g
    assert act(-30.0, 2.0) == pytest.approx(0.0, abs=1e-7)  # silu(g) -> 0 for very negative g
    assert act(1.0, 1.0) == float(np.float16(1.0 / (1.0 + math.exp(-1.0))))


def test_oracle_act_layout(orc):
    # gate in columns 0..n_ff, up in n_ff..2 n_ff, row-major over slots
    ns, n_ff = 3, 4
    c13 = np.zeros((ns, 2 * n_ff), np.float16)
    c13[:, :n_ff] = 30.0                       # silu(30) == 30 in f32 to f16 accuracy
    c13[:, n_ff:] = np.arange(ns * n_ff).reshape(ns, n_ff) / 8.0
    got = _f16(orc.moe_act_silu_f16(c13.view(np.uint16), ns, n_ff))
    assert np.array_equal(got, 30.0 * np.arange(ns * n_ff).reshape(ns, n_ff) / 8.0)


def test_oracle_gelu_act(orc):
    """f16(gelu_tanh(g) * u): float64 evaluation of the same formula within one f16 step; close to the erf form of
    gelu; special cases; gate and up are not interchangeable."""
    rng = np.random.default_rng(15)
    g = (rng.standard_normal(4096) * 3).astype(np.float16)
    u = (rng.standard_normal(4096) * 3).astype(np.float16)
    c13 = np.concatenate([g.view(np.uint16), u.view(np.uint16)])[None, :]
    got = _f16(orc.moe_act_gelu_f16(c13, 1, 4096)).ravel()
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = 0.5 * g64 * (1.0 + np.tanh(0.7978846 * (g64 + 0.044715 * g64 ** 3))) * u64
    step = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(got - want) <= 0.51 * step + 1e-6)
    erf_form = 0.5 * g64 * (1.0 + np.array([math.erf(v / math.sqrt(2.0)) for v in g64])) * u64
    assert np.max(np.abs(want - erf_form) / (np.abs(u64) + 1e-9)) < 2e-3  # the tanh form approximates gelu
    swapped = 0.5 * u64 * (1.0 + np.tanh(0.7978846 * (u64 + 0.044715 * u64 ** 3))) * g64
    assert np.mean(np.abs(got - swapped) > step) > 0.9
    silu = g64 / (1.0 + np.exp(-g64)) * u64
    assert np.mean(np.abs(got - silu) > step) > 0.9  # and it is not the silu kernel
    h = lambda v: int(np.float16(v).view(np.uint16))
    act = lambda gg, uu: float(_f16(orc.moe_act_gelu_f16(np.array([[h(gg), h(uu)]], np.uint16), 1, 1))[0, 0])
    assert act(0.0, 3.0) == 0.0 and act(2.5, 0.0) == 0.0
    assert act(10.0, 2.0) == 20.0                      # gelu(g) -> g
    assert act(-10.0, 2.0) == pytest.approx(0.0, abs=1e-7)  # gelu(g) -> 0
    assert act(1.0, 1.0) == float(np.float16(0.5 * (1.0 + math.tanh(0.7978846 * 1.044715))))


# ---------------------------------------------------------------- top-k sum
def test_oracle_topk_sum(orc):
    rng = np.random.default_rng(7)
    t, h, k = 5, 24, 8
    c2 = rng.standard_normal((t * k, h)).astype(np.float16)
    got = orc.moe_topk_sum_f16(c2.view(np.uint16), t, h, k)
    want = np.zeros((t, h), np.float32)
    for kk in range(k):  # slot order, one f32 rounding per addition
        want = (want + c2.reshape(t, k, h)[:, kk, :].astype(np.float32)).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # exactly summable inputs: order cannot matter, the result is the integer sum
    ci = rng.integers(-64, 64, (t * k, h)).astype(np.float16)
    got = orc.moe_topk_sum_f16(ci.view(np.uint16), t, h, k)
    assert np.array_equal(got, ci.astype(np.float64).reshape(t, k, h).sum(1))


# ---------------------------------------------------------------- align
def _align_numpy(idx, n_exp, block):
    idx = np.asarray(idx).ravel()
    ns = idx.size
    order = np.argsort(idx, kind="stable")
    sorted_ids, expert_ids = [], []
    for e in range(n_exp):
        run = order[idx[order] == e].tolist()
        pad = (-len(run)) % block
        sorted_ids += run + [ns] * pad
        expert_ids += [e] * ((len(run) + pad) // block)
    return np.array(sorted_ids, np.int32), np.array(expert_ids, np.int32)


def test_oracle_align_hand_case(orc):
    # 2 tokens x top-3 over 4 experts: slots 0..5 -> experts
    idx = [2, 0, 3, 0, 2, 1]
    s, e, n_post = orc.moe_align(idx, 4, 2)
    assert s.tolist() == [1, 3, 5, 6, 0, 4, 2, 6]
    assert e.tolist() == [0, 1, 2, 3]
    assert n_post == 8


@pytest.mark.parametrize("ns,n_exp,block", [(8, 128, 4), (32, 128, 4), (32, 128, 16), (4096, 128, 48), (4096, 128, 32),
                                            (1000, 7, 64), (130, 1024, 16), (1, 1, 4)])
def test_oracle_align_against_numpy(orc, ns, n_exp, block):
    rng = np.random.default_rng(ns + n_exp)
    idx = rng.integers(0, n_exp, ns).astype(np.int32)
    s, e, n_post = orc.moe_align(idx, n_exp, block)
    ws, we = _align_numpy(idx, n_exp, block)
    assert n_post == ws.size and np.array_equal(s, ws) and np.array_equal(e, we)


# ---------------------------------------------------------------- host routing of the library
def test_host_topk_known_answers():
    # qwen35/stages/moe.rs:135-155: [2,1,.5,-1], k=2 -> (0,1), weight ratio e, sum 1; ties [1,1,1] -> (0,1)
    idx, w = ops.moe_topk(np.array([2.0, 1.0, 0.5, -1.0], np.float32), 2)
    assert idx.tolist() == [[0, 1]]
    assert abs(w[0, 0] / w[0, 1] - math.e) < 1e-5 and abs(w.sum() - 1.0) < 1e-6
    idx, w = ops.moe_topk(np.array([1.0, 1.0, 1.0], np.float32), 2)
    assert idx.tolist() == [[0, 1]] and np.allclose(w, 0.5)


def test_host_topk_matches_oracle(orc):
    lg = gen.router_logits(64, 128)
    idx, w = ops.moe_topk(lg, 8)
    oi, ow = orc.moe_topk_batch(lg, 8)
    assert np.array_equal(idx, oi)
    assert np.array_equal(w.view(np.uint32), ow.view(np.uint32))
    # independent statement: float64 softmax, descending order, ties to the lower index
    p = np.exp(lg.astype(np.float64) - lg.max(1, keepdims=True))
    want = np.argsort(-p, axis=1, kind="stable")[:, :8]
    assert np.array_equal(idx, want)
    sel = np.take_along_axis(p, want, 1)
    assert np.allclose(w, sel / sel.sum(1, keepdims=True), rtol=1e-5)


def test_host_topk_errors():
    with pytest.raises(ops.W4a16Error):
        ops.moe_topk(np.zeros((1, 4), np.float32), 5)


def test_oracle_moe_ffn_against_float64(orc):
    """The composed oracle (lane GEMMs + act + weighted sum) against a float64 dequantised evaluation."""
    E, h, n_ff, g, t, k = 4, 128, 128, 32, 3, 2
    q13, s13, q2, s2 = gen.make_experts(E, h, n_ff, g)
    x = gen.normal_f16(99, (t, h))
    idx, wt = ops.moe_topk(gen.router_logits(t, E), k)
    out = orc.moe_ffn(x, idx, wt, q13, s13, q2, s2, h, n_ff, g)
    xf = _f16(x)
    want = np.zeros((t, h))
    for ti in range(t):
        for kk in range(k):
            e = idx[ti, kk]
            w13 = orc.dequant_matrix(q13[e], s13[e], 2 * n_ff, h, g).astype(np.float64)
            w2 = orc.dequant_matrix(q2[e], s2[e], h, n_ff, g).astype(np.float64)
            c = w13 @ xf[ti]
            a = c[:n_ff] / (1.0 + np.exp(-c[:n_ff])) * c[n_ff:]
            want[ti] += wt[ti, kk] * (w2 @ a)
    err = np.linalg.norm(out["y"] - want) / np.linalg.norm(want)
    assert err < 2e-3  # three f16 roundings of intermediates
