"""GPU check of the checkpoint reader: a model directory in the reference's on-disk format is read, registered through
the C ABI and served by the decode and prefill kernels; results against the CPU oracle on the tensors that were written."""
import numpy as np
import pytest

from llm170_amd import ckpt, gen, ops
from tests import ckpt_fixture as fx
from llm170_amd import parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("group,bf16,shards", [(128, False, 1), (32, True, 2)])
def test_model_dir_to_device(tmp_path, orc, group, bf16, shards):
    print("ckpt", group, bf16, shards, flush=True)
    d = str(tmp_path / "model")
    lins = [("model.layers.0.self_attn.qkv_proj", 192, 512), ("model.layers.0.mlp.down_proj", 128, 1024),
            ("model.layers.1.self_attn.o_proj", 80, 256)]
    want = fx.write_model(d, lins, group=group, bf16=bf16, shards=shards, index=shards > 1)
    m = ckpt.W4a16Model(d)
    dec = ops.W4a16Dec()
    try:
        assert m.upload_all(dec) == sorted(b for b, _, _ in lins)
        for base, n, k in lins:
            spec = dec.lin_spec(base)
            assert (spec["n"], spec["k"], spec["group"], spec["scale_bf16"]) == (n, k, group, bf16)
            q, s = want[base]
            x = gen.normal_f16(gen.shape_seed(n, k, 5, 3), (4, k))
            ref = orc.gemm_lane(x, 4, q, s, n, k, group, scale_bf16=bf16, threads=4)
            twin = dec.gemv_host(base, x, t=4, path=ops.PATH_LANE)
            assert np.array_equal(twin.view(np.uint32), np.ascontiguousarray(ref, np.float32).view(np.uint32))
            parity.assert_close(dec.gemv_host(base, x, t=4, path=ops.PATH_DECODE), ref, "ckpt decode " + base)
            parity.assert_close(dec.gemv_host(base, x[:1], t=1, path=ops.PATH_DECODE), ref[:1], "ckpt gemv " + base)
    finally:
        dec.cc.close()
        m.close()


def test_group_64_is_refused_by_the_device_path(tmp_path):
    """The reference's config check admits g64 (w4a16.rs:233); the kernels serve g128 and g32, and say so."""
    d = str(tmp_path / "g64")
    fx.write_model(d, [("a", 16, 128)], group=64)
    m = ckpt.W4a16Model(d)
    dec = ops.W4a16Dec()
    try:
        with pytest.raises(ops.W4a16Error):
            m.upload_all(dec)
    finally:
        dec.cc.close()
        m.close()


def test_fused_projections_from_a_checkpoint(tmp_path, orc):
    """q/k/v and gate/up are separate tensors in a checkpoint; fused on the device they are served by one launch, the
    gate|up pair by the kernel with the SiLU*up epilogue."""
    print("ckpt fuse", flush=True)
    d = str(tmp_path / "model")
    hidden, nq, nkv, nff = 512, 320, 72, 256  # nkv is not a multiple of 16: the fused rows are re-tiled, not pasted
    lins = [("l.q_proj", nq, hidden), ("l.k_proj", nkv, hidden), ("l.v_proj", nkv, hidden), ("l.gate_proj", nff, hidden),
            ("l.up_proj", nff, hidden)]
    want = fx.write_model(d, lins, group=128)
    m = ckpt.W4a16Model(d)
    dec = ops.W4a16Dec()
    cc = dec.cc
    try:
        m.upload_fused(dec, "l.qkv", ["l.q_proj", "l.k_proj", "l.v_proj"])
        m.upload_fused(dec, "l.gate_up", ["l.gate_proj", "l.up_proj"])
        spec = dec.lin_spec("l.qkv")
        assert (spec["n"], spec["k"]) == (nq + 2 * nkv, hidden)
        with pytest.raises(ops.W4a16Error):
            dec.lin_spec("l.qkv.__part0")  # the parts are gone
        t = 4
        x = gen.normal_f16(77, (t, hidden))
        got = dec.gemv_host("l.qkv", x, t=t, path=ops.PATH_LANE)
        ref = np.concatenate([orc.gemm_lane(x, t, want[b][0], want[b][1], n, hidden, 128, threads=4)
                              for b, n in (("l.q_proj", nq), ("l.k_proj", nkv), ("l.v_proj", nkv))], axis=1)
        assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(ref, np.float32).view(np.uint32))
        parity.assert_close(dec.gemv_host("l.qkv", x, t=t, path=ops.PATH_DECODE), ref, "fused qkv decode")
        # gate|up through the fused kernel against the oracle's silu_mul of the two lane GEMMs
        px, py = cc.to_device(x), cc.alloc(t * nff * 2)
        dec.lin_forward_glu("l.gate_up", px, py, t)
        act = cc.d2h(py, (t, nff), np.uint16)
        gu = np.concatenate([orc.gemm_lane(x, t, want[b][0], want[b][1], nff, hidden, 128, threads=4)
                             for b in ("l.gate_proj", "l.up_proj")], axis=1)
        ref_act = orc.silu_mul_f16_rows(gu)
        a, b = gen.f16_bits_to_f32(act).astype(np.float64), gen.f16_bits_to_f32(ref_act).astype(np.float64)
        rms = float(np.sqrt(np.mean(b * b)))
        assert np.all(np.abs(a - b) <= 2 * parity.f16_ulp(np.maximum(np.abs(b), rms / parity.CLAMP_DIV)))
        assert np.mean(act == ref_act) > 0.97
    finally:
        cc.close()
        m.close()


def test_lin_fuse_contract():
    print("fuse contract", flush=True)
    dec = ops.W4a16Dec()
    try:
        qa, sa, _ = gen.make_linear(32, 256, 128, 1, seed=1)
        qb, sb, _ = gen.make_linear(48, 256, 128, 1, seed=2)
        qc, sc, _ = gen.make_linear(16, 512, 128, 1, seed=3)
        dec.upload_lin_g("a", qa, sa, 32, 256, 128, False)
        dec.upload_lin_g("b", qb, sb, 48, 256, 128, False)
        dec.upload_lin_g("c", qc, sc, 16, 512, 128, False)
        with pytest.raises(ops.W4a16Error):
            dec.lin_fuse("ab", ["a", "c"])       # k differs
        with pytest.raises(ops.W4a16Error):
            dec.lin_fuse("ab", ["a", "missing"])
        with pytest.raises(ops.W4a16Error):
            dec.lin_fuse("a", ["a", "b"])        # a part under the fused name
        with pytest.raises(ops.W4a16Error):
            dec.lin_fuse("ab", ["a", "a"])
        dec.lin_fuse("ab", ["a", "b"])           # parts kept
        assert dec.lin_spec("a")["n"] == 32 and dec.lin_spec("ab")["n"] == 80
        # the fused operands round-trip through the tiled layout as the concatenation
        q, s = dec.untile("ab")
        assert np.array_equal(q, np.concatenate([qa, qb])) and np.array_equal(s, np.concatenate([sa, sb]))
    finally:
        dec.cc.close()
