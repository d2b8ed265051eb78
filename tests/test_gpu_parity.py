"""GPU parity tests: the HIP path through the C ABI against the CPU oracle.  Run on the MI355X box with -m gpu."""
import numpy as np
import pytest

from llm170_amd import ffi, gen, ops
from llm170_amd import parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dec():
    d = ops.W4a16Dec()
    yield d
    d.cc.close()


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ bit-exact gate (reference: gates.rs:4-180)
@pytest.mark.parametrize("n,k,group,bf16", [
    (8, 5120, 128, False), (8, 17408, 128, False), (8, 4096, 128, False), (4, 7168, 128, False),
    (8, 2048, 32, True), (8, 768, 32, True), (8, 2048, 32, False), (5, 256, 128, True), (3, 64, 32, False),
])
@pytest.mark.parametrize("t", [1, 4, 8, 16, 19])
def test_lane_twin_bit_exact_gate(dec, orc, n, k, group, bf16, t):
    say("gate", n, k, group, bf16, t)
    q, s, _ = gen.make_linear(n, k, group, 1)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    x = gen.gate_x(n, k, t)
    got = ops.Gptq4(dec.cc).gemm(x, t, q, s, n, k, group, bf16).reshape(t, n)
    want = orc.gemm_lane(x, t, q, s, n, k, group, scale_bf16=bf16)
    assert np.array_equal(_bits(got), _bits(want))


def test_lane_twin_reference_test_vectors(dec):
    import json
    import os
    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "lane_vectors.json")))
    # zero point is fixed at 8 on the device path, so only z == 8 vectors apply: the centre vector and seeded rows
    c = gold["center"]
    got = ops.Gptq4(dec.cc).gemv(c["x"], c["q"], c["s"], 1, c["k"], 128, False)
    assert _bits(got)[0] == c["expect_bits"]
    cache = {}
    for r in gold["seeded_rows"]["rows"]:
        key = (r["n"], r["k"], r["group"])
        if key not in cache:
            q, s, x = gen.make_linear(r["n"], r["k"], r["group"], 2)
            cache[key] = ops.Gptq4(dec.cc).gemm(x, 2, q, s, r["n"], r["k"], r["group"], False).reshape(2, r["n"])
        assert _bits(cache[key][r["tok"], r["row"]]) == r["expect_bits"]


# ------------------------------------------------------------------ dequant bit-exact, re-layout round trip
def test_dequant_exhaustive_nibbles_times_finite_scales(dec, orc):
    n, k, g = 512, 16384, 128  # n * k/g = 65536 scale slots: every f16 pattern once
    say("dequant exhaustive")
    q = gen.weights_q(77, n, k)
    q[:, ::16] = 0x76543210  # make sure all 16 nibble values meet every scale
    q[:, 1::16] = 0xFEDCBA98
    s = np.arange(65536, dtype=np.uint32).astype(np.uint16).reshape(n, k // g)
    s = np.where((s & 0x7C00) == 0x7C00, (s & 0x83FF) | 0x3000, s).astype(np.uint16)  # Inf/NaN -> finite
    dec.upload_lin_g("exh", q, s, n, k, g, False)
    want = orc.dequant_matrix(q, s, n, k, g)
    assert np.array_equal(_bits(dec.dequant("exh", from_tiled=True)), _bits(want))
    assert np.array_equal(_bits(dec.dequant("exh", from_tiled=False)), _bits(want))
    q2, s2 = dec.untile("exh")
    assert np.array_equal(q2, q) and np.array_equal(s2, s)


@pytest.mark.parametrize("n,k,g,bf16", [(48, 768, 32, False), (40, 256, 32, True), (24, 384, 128, True), (19, 256, 128, False)])
def test_dequant_and_roundtrip_small(dec, orc, n, k, g, bf16):
    q, s, _ = gen.make_linear(n, k, g, 1, seed=5)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("small", q, s, n, k, g, bf16)
    want = orc.dequant_matrix(q, s, n, k, g, scale_bf16=bf16)
    assert np.array_equal(_bits(dec.dequant("small", True)), _bits(want))
    assert np.array_equal(_bits(dec.dequant("small", False)), _bits(want))
    q2, s2 = dec.untile("small")
    assert np.array_equal(q2, q) and np.array_equal(s2, s)


# ------------------------------------------------------------------ decode regime vs oracle
DECODE_SHAPES = [
    (4096, 4096, 128),    # config 0
    (34816, 5120, 128),   # gate+up
    (5120, 17408, 128),   # down
    (7168, 5120, 128),    # QKV
    (1536, 2048, 32),     # MoE gate+up (one expert)
    (2048, 768, 32),      # MoE down
    (80, 128, 128), (16, 256, 32), (24, 384, 128),  # tiny / ragged row-block counts
]


@pytest.mark.parametrize("n,k,group", DECODE_SHAPES)
def test_decode_matches_oracle(dec, orc, n, k, group):
    q, s, x = gen.make_linear(n, k, group, 16)
    dec.upload_lin_g("lin", q, s, n, k, group, False)
    for t in (1, 4, 16, 3):
        say("decode", n, k, group, t)
        want = orc.gemm_lane(x[:t], t, q, s, n, k, group, threads=16)
        got = dec.gemv_host("lin", x[:t], t=t, path=ops.PATH_DECODE)
        m = parity.assert_close(got, want, "decode f32 n%d k%d g%d t%d" % (n, k, group, t))
        say("   ", {a: m[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")})
        got16 = dec.gemv_host("lin", x[:t], t=t, out_f16=True, path=ops.PATH_DECODE)
        # f16 output = one rounding of the f32 result
        assert np.array_equal(got16, gen.f32_to_f16_bits(got))
        # device twin agrees with the CPU oracle at full size, so it can stand in for it where the CPU is too slow
        twin = dec.gemv_host("lin", x[:t], t=t, path=ops.PATH_LANE)
        assert np.array_equal(_bits(twin), _bits(want))


@pytest.mark.parametrize("rows,waves", [(16, 1), (16, 8), (32, 3), (64, 7), (64, 8), (32, 1), (16, 5)])
def test_decode_launch_shapes_agree(dec, orc, rows, waves):
    n, k, group = 208, 2560, 128  # 13 row blocks: not a multiple of 2 or 4
    q, s, x = gen.make_linear(n, k, group, 16, seed=3)
    dec.upload_lin_g("shape", q, s, n, k, group, False)
    want = orc.gemm_lane(x, 16, q, s, n, k, group, threads=8)
    try:
        dec.set_decode_shape(rows, waves)
        got = dec.gemv_host("shape", x, t=16, path=ops.PATH_DECODE)
    finally:
        dec.set_decode_shape(0, 0)
    parity.assert_close(got, want, "decode shape %d/%d" % (rows, waves))


@pytest.mark.parametrize("nks", [2, 3, 8])
def test_decode_split_k_across_workgroups(dec, orc, nks):
    """k slices across workgroups: one launch, the last workgroup of a row-block group adds the slices in slice
    order, so the result is the same on every run; the automatic choice is covered by the 17408 x 5120 shape above."""
    n, k, group = 208, 2560, 128  # 13 row blocks, 20 k tiles
    q, s, x = gen.make_linear(n, k, group, 16, seed=5)
    dec.upload_lin_g("ks", q, s, n, k, group, False)
    want = orc.gemm_lane(x, 16, q, s, n, k, group, threads=8)
    try:
        dec.set_decode_ksplit(nks)
        for t in (1, 4, 8, 16):
            say("decode ksplit", nks, t)
            got = dec.gemv_host("ks", x[:t], t=t, path=ops.PATH_DECODE)
            parity.assert_close(got, want[:t], "decode ksplit %d t%d" % (nks, t))
            for _ in range(3):
                assert np.array_equal(_bits(got), _bits(dec.gemv_host("ks", x[:t], t=t, path=ops.PATH_DECODE)))
        # launch shapes and split together, and the tickets are back at zero for an unsplit launch afterwards
        dec.set_decode_shape(16, 3)
        parity.assert_close(dec.gemv_host("ks", x[:4], t=4, path=ops.PATH_DECODE), want[:4], "decode ksplit rb1")
    finally:
        dec.set_decode_ksplit(0)
        dec.set_decode_shape(0, 0)
    parity.assert_close(dec.gemv_host("ks", x[:4], t=4, path=ops.PATH_DECODE), want[:4], "decode after ksplit")
    with pytest.raises(ops.W4a16Error):
        dec.set_decode_ksplit(9)


def test_decode_split_k_with_an_empty_slice(dec, orc):
    """9 k tiles in 4 slices of 3 (tiles per slice are rounded up): the fourth slice is empty and adds zeros; waves
    beyond a slice's tiles stream nothing."""
    n, k, group = 80, 1152, 128
    q, s, x = gen.make_linear(n, k, group, 4, seed=15)
    dec.upload_lin_g("ks9", q, s, n, k, group, False)
    want = orc.gemm_lane(x, 4, q, s, n, k, group, threads=8)
    try:
        dec.set_decode_ksplit(4)
        for waves in (0, 2, 8):
            dec.set_decode_shape(0, waves)
            for t in (1, 4):
                say("decode empty slice", waves, t)
                parity.assert_close(dec.gemv_host("ks9", x[:t], t=t, path=ops.PATH_DECODE), want[:t],
                                    "decode empty slice waves %d t%d" % (waves, t))
    finally:
        dec.set_decode_ksplit(0)
        dec.set_decode_shape(0, 0)


def test_decode_bf16_scales(dec, orc):
    n, k, group = 256, 2048, 32
    q, s, x = gen.make_linear(n, k, group, 4, seed=8)
    s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("bf", q, s, n, k, group, True)
    want = orc.gemm_lane(x, 4, q, s, n, k, group, scale_bf16=True, threads=8)
    parity.assert_close(dec.gemv_host("bf", x, t=4, path=ops.PATH_DECODE), want, "decode bf16")


def test_decode_closed_forms_full_size(dec):
    """Size-independent checks at the full gate+up shape: unit scales and unit activations give the exact integer
    row sums (every partial sum is an integer below 2^24), and doubling x doubles y exactly."""
    n, k, group = 34816, 5120, 128
    q = gen.weights_q(12, n, k)
    ones = np.full((n, k // group), 0x3C00, np.uint16)
    dec.upload_lin_g("cf", q, ones, n, k, group, False)
    x = np.full((1, k), 0x3C00, np.uint16)
    got = dec.gemv_host("cf", x, t=1, path=ops.PATH_DECODE)
    want = gen.unpack_nibbles(q, k).astype(np.int64).sum(axis=1)
    assert np.array_equal(got[0].astype(np.int64), want) and np.array_equal(got[0], want.astype(np.float32))
    _, s, xr = gen.make_linear(n, k, group, 2)
    dec.upload_lin_g("cf", q, s, n, k, group, False)
    x2 = gen.f32_to_f16_bits(gen.f16_bits_to_f32(xr) * np.float32(2.0))
    a = dec.gemv_host("cf", xr, t=2, path=ops.PATH_DECODE)
    b = dec.gemv_host("cf", x2, t=2, path=ops.PATH_DECODE)
    assert np.array_equal(_bits(b), _bits(a * np.float32(2.0)))


# ------------------------------------------------------------------ contract / error behaviour
def test_error_paths(dec):
    q, s, x = gen.make_linear(16, 256, 128, 1)
    with pytest.raises(ops.W4a16Error) as e:
        dec.upload_lin_g("bad", q, s[:, :1], 16, 256, 128, False)
    assert e.value.code == ffi.ERR_SHAPE
    with pytest.raises(ops.W4a16Error) as e:
        dec.upload_lin_g("bad", q, s, 16, 256, 64, False)
    assert e.value.code == ffi.ERR_UNSUPPORTED
    with pytest.raises(ops.W4a16Error) as e:
        dec.gemv_host("never-registered", x)
    assert e.value.code == ffi.ERR_NOT_FOUND and "never-registered" in str(e.value)
    dec.upload_lin_g("ok", q, s, 16, 256, 128, False)
    with pytest.raises(ops.W4a16Error) as e:
        dec.gemv_host("ok", np.zeros((17, 256), np.uint16), t=17, path=ops.PATH_DECODE)
    assert e.value.code == ffi.ERR_SHAPE
    with pytest.raises(ops.W4a16Error) as e:
        dec.cc.function("w4a16_no_such_kernel")
    assert e.value.code == ffi.ERR_SYMBOL and "w4a16_no_such_kernel" in str(e.value)
    with pytest.raises(ops.W4a16Error):
        ops.Gptq4(dec.cc).gemm(x, 1, q, s, 16, 257, 128, False)
    # k not a multiple of 128 (group 32): no tiled copy, AUTO falls back to the bit-exact kernel
    q, s, x = gen.make_linear(8, 96, 32, 2)
    dec.upload_lin_g("odd", q, s, 8, 96, 32, False)
    assert not dec.lin_spec("odd")["tiled"]
    assert dec.gemv_host("odd", x, t=2).shape == (2, 8)
    before = dec.cc.allocated_bytes()
    dec.upload_lin_g("odd", q, s, 8, 96, 32, False)  # re-registration frees the old buffers
    assert dec.cc.allocated_bytes() == before
    dec.upload_lin_g("ok", *gen.make_linear(16, 256, 128, 1)[:2], 16, 256, 128, False)
    dec.drop_raw("ok")
    assert dec.lin_spec("ok") == {"n": 16, "k": 256, "group": 128, "scale_bf16": False, "tiled": True, "raw": False}
    with pytest.raises(ops.W4a16Error):
        dec.gemv_host("ok", np.zeros((1, 256), np.uint16), path=ops.PATH_LANE)


# ------------------------------------------------------------------ prefill regime (MFMA GEMM)
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


@pytest.mark.parametrize("n,k,group,t,bf16", [
    (256, 256, 128, 256, False), (272, 384, 128, 70, False), (48, 128, 128, 17, False), (1000, 512, 128, 300, False),
    (512, 256, 32, 100, False), (1536, 2048, 32, 33, False), (2048, 768, 32, 512, False), (320, 256, 128, 64, True),
    (4096, 4096, 128, 128, False),
])
def test_prefill_matches_oracle(dec, orc, n, k, group, t, bf16):
    say("prefill", n, k, group, t, bf16)
    q, s, x = gen.make_linear(n, k, group, t, seed=21)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("pf", q, s, n, k, group, bf16)
    want = orc.gemm_lane(x, t, q, s, n, k, group, scale_bf16=bf16, threads=16)
    got = _device_forward(dec, "pf", x, t, ops.PATH_PREFILL)
    m = parity.assert_close(got, want, "prefill n%d k%d g%d t%d" % (n, k, group, t))
    say("   ", {a: m[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")})
    got16 = _device_forward(dec, "pf", x, t, ops.PATH_PREFILL, out_f16=True)
    assert np.array_equal(got16, gen.f32_to_f16_bits(got))
    auto = _device_forward(dec, "pf", x, t, ops.PATH_AUTO)
    if t > 64:
        assert np.array_equal(_bits(auto), _bits(got))  # more than 64 rows route to the prefill kernel
    else:
        stream = _device_forward(dec, "pf", x, t, ops.PATH_STREAM)
        assert np.array_equal(_bits(auto), _bits(stream))  # 17..64 rows route to the streaming kernel
        parity.assert_close(stream, want, "stream n%d k%d g%d t%d" % (n, k, group, t))


@pytest.mark.parametrize("n,k,group,bf16", [(416, 1024, 128, False), (1536, 2048, 32, False), (200, 256, 128, True),
                                            (5120, 5120, 128, False)])
@pytest.mark.parametrize("t", [17, 32, 33, 48, 64, 100])
def test_stream_path_matches_oracle(dec, orc, n, k, group, bf16, t):
    """A few dozen rows: the grouped kernel run on the dense linear as its one expert (x shared through LDS, segments
    of up to 64 rows, k slices across workgroups when the output is narrow).  f32 and f16 outputs, any t."""
    say("stream", n, k, group, bf16, t)
    q, s, x = gen.make_linear(n, k, group, t, seed=61)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    dec.upload_lin_g("st", q, s, n, k, group, bf16)
    if n * t <= 1 << 18:
        want = orc.gemm_lane(x, t, q, s, n, k, group, scale_bf16=bf16, threads=16)
    else:
        want = _device_forward(dec, "st", x, t, ops.PATH_LANE)  # the bit-exact device twin of the oracle
    got = _device_forward(dec, "st", x, t, ops.PATH_STREAM)
    m = parity.assert_close(got, want, "stream n%d k%d g%d t%d" % (n, k, group, t))
    say("   ", {a: m[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")})
    assert np.array_equal(_device_forward(dec, "st", x, t, ops.PATH_STREAM, out_f16=True), gen.f32_to_f16_bits(got))
    assert np.array_equal(_bits(got), _bits(_device_forward(dec, "st", x, t, ops.PATH_STREAM)))  # same bits every run
    try:
        for ks in (-1, 2, 5):
            dec.set_decode_ksplit(ks)
            parity.assert_close(_device_forward(dec, "st", x, t, ops.PATH_STREAM), want, "stream ksplit %d" % ks)
    finally:
        dec.set_decode_ksplit(0)


@pytest.mark.parametrize("n,k,group,t", [(272, 384, 128, 70), (1000, 512, 128, 300), (512, 256, 32, 100), (2048, 2048, 128, 129)])
def test_prefill_block_tiles_agree(dec, orc, n, k, group, t):
    """64-, 96- and 128-row block tiles: every output element sees the same sequence of MFMAs and rescales, so the
    three give the same bits (unsplit), and all meet the contract against the oracle."""
    say("prefill tiles", n, k, group, t)
    q, s, x = gen.make_linear(n, k, group, t, seed=27)
    dec.upload_lin_g("pft", q, s, n, k, group, False)
    if n * t <= 1 << 18:
        want = orc.gemm_lane(x, t, q, s, n, k, group, threads=16)
    else:
        want = _device_forward(dec, "pft", x, t, ops.PATH_LANE)
    out = {}
    try:
        dec.set_prefill_ksplit(-1)
        for rows in (64, 96, 128):
            dec.set_prefill_tile(rows)
            out[rows] = _device_forward(dec, "pft", x, t, ops.PATH_PREFILL)
            parity.assert_close(out[rows], want, "prefill tile %d" % rows)
            assert np.array_equal(_device_forward(dec, "pft", x, t, ops.PATH_PREFILL, out_f16=True),
                                  gen.f32_to_f16_bits(out[rows]))
        dec.set_prefill_ksplit(2)
        for rows in (64, 96):
            dec.set_prefill_tile(rows)
            parity.assert_close(_device_forward(dec, "pft", x, t, ops.PATH_PREFILL), want, "prefill tile %d split" % rows)
    finally:
        dec.set_prefill_tile(0)
        dec.set_prefill_ksplit(0)
    assert np.array_equal(_bits(out[64]), _bits(out[128])) and np.array_equal(_bits(out[96]), _bits(out[128]))
    with pytest.raises(ops.W4a16Error):
        dec.set_prefill_tile(100)


@pytest.mark.parametrize("n,k,t", [(34816, 5120, 512), (5120, 17408, 512), (34816, 5120, 4096), (34816, 5120, 1024),
                                   (5120, 17408, 1024), (5120, 17408, 4096), (34816, 5120, 1000)])
def test_prefill_full_shapes_against_device_twin_and_sampled_oracle(dec, orc, n, k, t):
    """Layer shapes: every output against the bit-exact device twin (itself pinned to the CPU oracle above and on a
    seeded sample here), because the CPU needs ~1e12 scalar MACs for the full matrix.  The shapes cover both block
    tiles, ragged last tiles (t = 1000) and the automatic k slices of the narrow output."""
    say("prefill full", n, k, t)
    group = 128
    q, s, x = gen.make_linear(n, k, group, t, seed=5)
    dec.upload_lin_g("pfull", q, s, n, k, group, False)
    got = _device_forward(dec, "pfull", x, t, ops.PATH_PREFILL)
    twin = _device_forward(dec, "pfull", x, t, ops.PATH_LANE)
    rows = (gen.stream(1, 3000) % np.uint64(n)).astype(np.uint32)
    toks = (gen.stream(2, 3000) % np.uint64(t)).astype(np.uint32)
    smp = orc.gemm_lane_sample(x, q, s, k, group, rows, toks)
    assert np.array_equal(_bits(twin[toks, rows]), _bits(smp))
    m = parity.assert_close(got, twin, "prefill full n%d k%d t%d" % (n, k, t))
    say("   ", {a: m[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")})
    # the same launch again (same bits) and with the k slices switched off
    again = _device_forward(dec, "pfull", x, t, ops.PATH_PREFILL)
    assert np.array_equal(_bits(again), _bits(got))
    dec.set_prefill_ksplit(-1)
    try:
        whole = _device_forward(dec, "pfull", x, t, ops.PATH_PREFILL)
    finally:
        dec.set_prefill_ksplit(0)
    parity.assert_close(whole, twin, "prefill full unsplit n%d k%d t%d" % (n, k, t))
    parity.assert_close(got, whole, "prefill full split vs unsplit n%d k%d t%d" % (n, k, t))


@pytest.mark.parametrize("n,k,group,t,ksplit", [(512, 4096, 128, 100, 2), (512, 4096, 128, 100, 3), (512, 4096, 128, 100, 8),
                                                (300, 2048, 32, 48, 4), (5120, 17408, 128, 512, 0)])
def test_prefill_split_k(dec, orc, n, k, group, t, ksplit):
    """Split-K (forced, or chosen automatically for the narrow down projection at t = 512): partial sums in f32 added
    in slice order; same contract against the lane oracle, and close to the unsplit result."""
    say("prefill split-k", n, k, group, t, ksplit)
    q, s, x = gen.make_linear(n, k, group, t, seed=33)
    dec.upload_lin_g("pks", q, s, n, k, group, False)
    dec.set_prefill_ksplit(-1)
    try:
        whole = _device_forward(dec, "pks", x, t, ops.PATH_PREFILL)
        dec.set_prefill_ksplit(ksplit)
        got = _device_forward(dec, "pks", x, t, ops.PATH_PREFILL)
        got16 = _device_forward(dec, "pks", x, t, ops.PATH_PREFILL, out_f16=True)
    finally:
        dec.set_prefill_ksplit(0)
    assert np.array_equal(got16, gen.f32_to_f16_bits(got))
    if n * t <= 1 << 18:
        want = orc.gemm_lane(x, t, q, s, n, k, group, threads=16)
    else:
        want = _device_forward(dec, "pks", x, t, ops.PATH_LANE)  # the bit-exact device twin of the oracle
    parity.assert_close(got, want, "split-k %d" % ksplit)
    parity.assert_close(got, whole, "split-k %d vs unsplit" % ksplit)
    if ksplit != 0:
        assert not np.array_equal(_bits(got), _bits(whole))  # a different summation order: the split really happened


def test_prefill_refuses_irregular_scales_and_auto_falls_back(dec, orc):
    n, k, group, t = 64, 256, 128, 40
    q, s, x = gen.make_linear(n, k, group, t, seed=9)
    s[3, 1] = 0  # a zero scale: the running-unit rescale of the MFMA kernel would divide by it
    dec.upload_lin_g("irr", q, s, n, k, group, False)
    with pytest.raises(ops.W4a16Error) as e:
        _device_forward(dec, "irr", x, t, ops.PATH_PREFILL)
    assert e.value.code == ffi.ERR_UNSUPPORTED
    want = orc.gemm_lane(x, t, q, s, n, k, group, threads=8)
    parity.assert_close(_device_forward(dec, "irr", x, t, ops.PATH_AUTO), want, "auto fallback")
    x_long = np.concatenate([x, x, x, x, x])[:170]  # beyond 64 rows the fallback is the streaming kernel as well
    parity.assert_close(_device_forward(dec, "irr", x_long, 170, ops.PATH_AUTO),
                        orc.gemm_lane(x_long, 170, q, s, n, k, group, threads=8), "auto fallback, 170 rows")


def test_bf16_scales_of_extreme_range_take_the_streaming_path(dec, orc):
    """A bf16 row whose scales span the f32 range (1.0 next to 1e-38, and a subnormal): the running-unit rescale of
    the MFMA kernel would overflow, so such a linear is refused there and AUTO serves it with the streaming kernel;
    the result is finite and meets the contract like any other."""
    n, k, group, t = 64, 512, 128, 100
    q, s, x = gen.make_linear(n, k, group, t, seed=10)
    s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    s[5] = [0x3F80, 0x006D, 0x3F80, 0x006D]   # 1.0, 1e-38, 1.0, 1e-38
    s[9, 2] = 0x0001                          # a bf16 subnormal
    s[11] = [0x5F00, 0x1E80, 0x5F00, 0x1E80]   # 2^63 next to 2^-66
    dec.upload_lin_g("wild", q, s, n, k, group, True)
    with pytest.raises(ops.W4a16Error) as e:
        _device_forward(dec, "wild", x, t, ops.PATH_PREFILL)
    assert e.value.code == ffi.ERR_UNSUPPORTED
    got = _device_forward(dec, "wild", x, t, ops.PATH_AUTO)
    assert np.all(np.isfinite(got))
    want = orc.gemm_lane(x, t, q, s, n, k, group, scale_bf16=True, threads=8)
    # rows 5, 9 and 11 have their own magnitudes: compare them and the ordinary rows separately
    special = np.zeros(n, bool)
    special[[5, 9, 11]] = True
    parity.assert_close(got[:, ~special], want[:, ~special], "wild scales, ordinary rows")
    for r in (5, 9, 11):
        assert np.allclose(got[:, r], want[:, r], rtol=1e-4, atol=0), r
    # one notch inside the bound the MFMA kernel still serves the linear
    s2 = s.copy()
    s2[5] = [0x3F80, 0x2180, 0x3F80, 0x2180]  # 1.0 next to 2^-60
    s2[9, 2] = 0x3F80
    s2[11] = [0x5D00, 0x2180, 0x5D00, 0x2180]  # 2^59 next to 2^-60
    dec.upload_lin_g("tame", q, s2, n, k, group, True)
    got2 = _device_forward(dec, "tame", x, t, ops.PATH_PREFILL)
    want2 = orc.gemm_lane(x, t, q, s2, n, k, group, scale_bf16=True, threads=8)
    assert np.all(np.isfinite(got2))
    parity.assert_close(got2[:, ~special], want2[:, ~special], "tame scales, ordinary rows")
    for r in (5, 11):
        assert np.allclose(got2[:, r], want2[:, r], rtol=1e-4, atol=0), r
