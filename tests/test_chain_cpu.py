"""CPU checks of the layer-chain glue in the oracle against independent statements of the same rules."""
import numpy as np

from llm170_amd import gen


def _f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float64)


def _step(v):
    return np.maximum(np.abs(v), 2.0 ** -14) * 2.0 ** -10


def test_rms_rescale_against_float64(orc):
    rng = np.random.default_rng(3)
    v = (rng.standard_normal((5, 5120)) * rng.uniform(0.1, 50, (5, 1))).astype(np.float32)
    got = _f16(orc.rms_rescale_f16(v, 5120))
    v64 = v.astype(np.float64)
    want = v64 / np.sqrt(np.mean(v64 * v64, axis=1, keepdims=True) + 1e-6)
    assert np.all(np.abs(got - want) <= 0.51 * _step(want) + 1e-9)
    same = np.mean(got == want.astype(np.float32).astype(np.float16).astype(np.float64))
    assert same > 0.999
    assert np.allclose(np.mean(got * got, axis=1), 1.0, atol=2e-3)
    # dividing by the mean |v| or forgetting the square root would be off by far more than a step
    wrong = v64 / np.mean(v64 * v64, axis=1, keepdims=True)
    assert np.mean(np.abs(got - wrong) > _step(want)) > 0.9


def test_rms_rescale_column_slice_and_constant_rows(orc):
    v = np.zeros((3, 700), np.float32)
    v[:, :300] = np.array([[2.0], [-0.5], [1e-4]], np.float32)
    v[:, 300:] = 1e6  # columns past ncols must not enter the mean
    got = _f16(orc.rms_rescale_f16(v, 300))
    assert got.shape == (3, 300)
    assert np.all(got[0] == 1.0) and np.all(got[1] == -1.0)
    # tiny rows: the 1e-6 floor dominates: 1e-4 / sqrt(1e-8 + 1e-6)
    assert np.allclose(got[2], 1e-4 / np.sqrt(1e-8 + 1e-6), rtol=1e-3)


def test_rms_rescale_power_of_two_invariance(orc):
    rng = np.random.default_rng(4)
    v = (rng.standard_normal((2, 1024)) * 8).astype(np.float32)
    a = orc.rms_rescale_f16(v, 1024)
    b = orc.rms_rescale_f16(v * np.float32(4.0), 1024)  # exact scaling; eps is negligible at this magnitude
    assert np.mean(a == b) > 0.999


def test_silu_mul_rows_against_float64(orc):
    rng = np.random.default_rng(6)
    gu = (rng.standard_normal((3, 2 * 512)) * 5).astype(np.float32)
    got = _f16(orc.silu_mul_f16_rows(gu))
    g, u = gu[:, :512].astype(np.float64), gu[:, 512:].astype(np.float64)
    want = g / (1.0 + np.exp(-g)) * u
    assert np.all(np.abs(got - want) <= 0.51 * _step(want) + 1e-7)
    swapped = u / (1.0 + np.exp(-u)) * g
    assert np.mean(np.abs(got - swapped) > _step(want)) > 0.9


def test_gelu_mul_rows_against_float64(orc):
    rng = np.random.default_rng(16)
    gu = (rng.standard_normal((3, 2 * 512)) * 3).astype(np.float32)
    got = _f16(orc.gelu_mul_f16_rows(gu))
    g, u = gu[:, :512].astype(np.float64), gu[:, 512:].astype(np.float64)

    def gelu(v):
        return 0.5 * v * (1.0 + np.tanh(0.7978846 * (v + 0.044715 * v ** 3)))

    want = gelu(g) * u
    # 1 + tanhf cancels in f32 for a gate below about -4 (the reference's arithmetic too): an absolute 1e-6 covers it
    assert np.all(np.abs(got - want) <= 0.51 * _step(want) + 1e-6)
    swapped = gelu(u) * g
    assert np.mean(np.abs(got - swapped) > _step(want)) > 0.8
    # against the erf form of gelu the tanh form stays within 1e-3 absolute per unit of up
    from math import erf
    exact = np.vectorize(lambda v: 0.5 * v * (1.0 + erf(v / np.sqrt(2.0))))(g) * u
    assert np.max(np.abs(want - exact) / (np.abs(u) + 1e-9)) < 1e-3


def test_chain_layer_against_float64(orc):
    hidden, n_qkv, n_ff, g, t = 256, 384, 512, 128, 3
    shapes = [(n_qkv, hidden), (hidden, hidden), (2 * n_ff, hidden), (hidden, n_ff)]
    lins = []
    for i, (n, k) in enumerate(shapes):
        q = gen.weights_q(gen.shape_seed(n, k, tensor=50 + i), n, k)
        s = gen.scales_f16(gen.shape_seed(n, k, tensor=60 + i), n, k, g)
        lins.append((q, s, n, k))
    x = gen.normal_f16(17, (t, hidden))
    st = orc.chain_layer(x, lins, g)
    w = [orc.dequant_matrix(q, s, n, k, g).astype(np.float64) for (q, s, n, k) in lins]
    rms = lambda v: v / np.sqrt(np.mean(v * v, axis=1, keepdims=True) + 1e-6)
    a = rms((_f16(x) @ w[0].T)[:, :hidden])
    b = rms(a @ w[1].T)
    gu = b @ w[2].T
    c = gu[:, :n_ff] / (1.0 + np.exp(-gu[:, :n_ff])) * gu[:, n_ff:]
    want = rms(c @ w[3].T)
    got = _f16(st["x"])
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 3e-3  # four f16 roundings of intermediates


def test_rms_inv_against_float64_and_rms_rescale(orc):
    rng = np.random.default_rng(8)
    v = (rng.standard_normal((4, 700)) * rng.uniform(0.05, 30, (4, 1))).astype(np.float32)
    v[:, 500:] = 1e5  # columns past ncols stay out of the mean
    inv = orc.rms_inv(v, 500)
    v64 = v[:, :500].astype(np.float64)
    want = 1.0 / np.sqrt(np.mean(v64 * v64, axis=1) + 1e-6)
    assert inv.dtype == np.float32 and np.allclose(inv, want, rtol=1e-6)
    # it is the factor rms_rescale_f16 applies: f16(v * inv) agrees with it to a rounding flip
    a = _f16(orc.rms_rescale_f16(v, 500))
    b = (v[:, :500] * inv[:, None]).astype(np.float32).astype(np.float16).astype(np.float64)
    assert np.mean(a == b) > 0.999 and np.all(np.abs(a - b) <= _step(a))
    # a constant row of 3s: mean square 9
    assert np.allclose(orc.rms_inv(np.full((1, 64), 3.0, np.float32), 64), 1.0 / 3.0, rtol=1e-6)


def test_chain_layer_fused_against_float64_and_unfused(orc):
    """The deferred statement is the same function of x as chain_layer: the factor of a stage's input commutes with the
    linear.  Checked against float64 and against the unfused oracle, with an un-normalised input and its factor."""
    hidden, n_qkv, n_ff, g, t = 256, 384, 512, 128, 3
    shapes = [(n_qkv, hidden), (hidden, hidden), (2 * n_ff, hidden), (hidden, n_ff)]
    lins = []
    for i, (n, k) in enumerate(shapes):
        q = gen.weights_q(gen.shape_seed(n, k, tensor=50 + i), n, k)
        s = gen.scales_f16(gen.shape_seed(n, k, tensor=60 + i), n, k, g)
        lins.append((q, s, n, k))
    rng = np.random.default_rng(2)
    v0 = (rng.standard_normal((t, hidden)) * np.array([[0.3], [5.0], [40.0]])).astype(np.float32)  # un-normalised rows
    x_un = orc.f32_to_f16_array(v0).reshape(t, hidden)
    s0 = orc.rms_inv(v0, hidden)
    st = orc.chain_layer_fused(x_un, s0, lins, g)
    w = [orc.dequant_matrix(q, s, n, k, g).astype(np.float64) for (q, s, n, k) in lins]
    rms = lambda v: v / np.sqrt(np.mean(v * v, axis=1, keepdims=True) + 1e-6)
    a = rms((rms(v0.astype(np.float64)) @ w[0].T)[:, :hidden])
    b = rms(a @ w[1].T)
    gu = b @ w[2].T
    c = gu[:, :n_ff] / (1.0 + np.exp(-gu[:, :n_ff])) * gu[:, n_ff:]
    want = rms(c @ w[3].T)
    got = st["v4"].astype(np.float64) * st["s"].astype(np.float64)[:, None]
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 3e-3
    # each stage's activations carry the scale of a normalised input (about 4 here), not of x
    assert np.all(np.abs(np.sqrt(np.mean(st["v1"].astype(np.float64) ** 2, axis=1)) / np.sqrt(np.mean((rms(v0.astype(np.float64)) @ w[0].T)[:, :hidden] ** 2, axis=1)) - 1) < 1e-2)
    # against the unfused oracle fed the normalised input
    x_n = orc.rms_rescale_f16(v0, hidden)
    un = _f16(orc.chain_layer(x_n, lins, g)["x"])
    assert np.linalg.norm(un - want) / np.linalg.norm(want) < 3e-3
    fused_x = _f16(orc.rms_rescale_f16(st["v4"], hidden))
    assert np.linalg.norm(fused_x - un) / np.linalg.norm(un) < 5e-3
    # forgetting the factor of the input changes v1 by far more than rounding
    wrong = orc.chain_layer_fused(x_un, np.ones(t, np.float32), lins, g)
    assert np.linalg.norm(wrong["v1"] - st["v1"]) / np.linalg.norm(st["v1"]) > 0.5
