"""GPU check of the checkpoint reader: a model directory in the reference's on-disk format is read, registered through
the C ABI and served by the decode and prefill kernels; results against the CPU oracle on the tensors that were written."""
import numpy as np
import pytest

from llm170_amd import ckpt, gen, ops
from tests import ckpt_fixture as fx
from tests import parity

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
