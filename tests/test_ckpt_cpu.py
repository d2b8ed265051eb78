"""CPU checks of the checkpoint reader against the reference's on-disk contract (st.rs, w4a16.rs)."""
import json
import os
import struct

import numpy as np
import pytest

from llm170_amd import ckpt
from tests import ckpt_fixture as fx


def _raw(path, hdr, data):
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hdr)))
        f.write(hdr.encode())
        f.write(b"\0" * data)


def test_rejects_inverted_offsets(tmp_path):  # st.rs:390-400
    p = str(tmp_path / "inv.safetensors")
    _raw(p, '{"a":{"dtype":"F32","shape":[4],"data_offsets":[16,8]}}', 32)
    with pytest.raises(ckpt.StError):
        ckpt.StArchive(p)


def test_rejects_size_mismatch(tmp_path):  # st.rs:402-412
    p = str(tmp_path / "sz.safetensors")
    _raw(p, '{"a":{"dtype":"F32","shape":[4],"data_offsets":[0,8]}}', 32)
    with pytest.raises(ckpt.StError):
        ckpt.StArchive(p)


@pytest.mark.parametrize("hdr", ['[1,2]', '{"a":{"dtype":"Q9","shape":[1],"data_offsets":[0,1]}}',
                                 '{"a":{"dtype":"F32","shape":[1],"data_offsets":[0,4,8]}}', '{"a":{"shape":[1]}}',
                                 '{"a":{"dtype":"F32","shape":[-1],"data_offsets":[0,4]}}', 'not json'])
def test_rejects_bad_headers(tmp_path, hdr):
    p = str(tmp_path / "bad.safetensors")
    _raw(p, hdr, 16)
    with pytest.raises(ckpt.StError):
        ckpt.StArchive(p)


def test_rejects_bad_header_length(tmp_path):
    p = str(tmp_path / "len.safetensors")
    open(p, "wb").write(struct.pack("<Q", 0))
    with pytest.raises(ckpt.StError):
        ckpt.StArchive(p)
    open(p, "wb").write(struct.pack("<Q", 1 << 31) + b"{}")
    with pytest.raises(ckpt.StError):
        ckpt.StArchive(p)


def test_tensor_range_beyond_file(tmp_path):
    p = str(tmp_path / "short.safetensors")
    _raw(p, '{"a":{"dtype":"F32","shape":[4],"data_offsets":[0,16]}}', 8)
    ar = ckpt.StArchive(p)
    with pytest.raises(ckpt.StError):
        ar.tensor("a")


@pytest.mark.parametrize("shards,index,sidecar,bf16,group", [(1, False, True, False, 128), (3, True, True, False, 128),
                                                             (2, False, False, True, 32)])
def test_model_round_trip(tmp_path, shards, index, sidecar, bf16, group):
    d = str(tmp_path / "m")
    lins = [("blk.0.attn_qkv", 48, 256), ("blk.0.ffn_down", 32, 512), ("blk.1.attn_qkv", 16, 128)]
    want = fx.write_model(d, lins, group=group, bf16=bf16, shards=shards, sidecar=sidecar, index=index)
    m = ckpt.W4a16Model(d)
    assert m.group == group and len(m.ar.shard_paths()) == shards
    assert m.lin_shapes() == sorted(lins)
    for base, n, k in lins:
        q, s, nn, kk, bf = m.lin_operands(base)
        assert (nn, kk, bf) == (n, k, bf16)
        assert q.dtype == np.uint32 and np.array_equal(q, want[base][0]) and np.array_equal(s, want[base][1])
    m.close()


def test_index_naming_a_missing_tensor(tmp_path):
    d = str(tmp_path / "m")
    fx.write_model(d, [("a", 16, 128)], index=True)
    idx = json.load(open(os.path.join(d, "model.safetensors.index.json")))
    idx["weight_map"]["ghost.weight"] = "model.safetensors"
    json.dump(idx, open(os.path.join(d, "model.safetensors.index.json"), "w"))
    with pytest.raises(ckpt.StError):
        ckpt.W4a16Model(d)


def _quant(**kw):
    q = json.loads(json.dumps(fx.QUANT))
    q.update(kw)
    return q


def test_quant_config_contract():
    assert ckpt.check_quant(fx.QUANT) == 128
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.check_quant(_quant(quant_method="gptq"))
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.check_quant(_quant(format="int-quantized"))
    two = _quant()
    two["config_groups"]["group_1"] = two["config_groups"]["group_0"]
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.check_quant(two)
    for key, val in (("num_bits", 8), ("symmetric", False), ("group_size", 256)):
        bad = _quant()
        bad["config_groups"]["group_0"]["weights"][key] = val
        with pytest.raises(ckpt.W4a16CkptError):
            ckpt.check_quant(bad)
    g64 = _quant()
    g64["config_groups"]["group_0"]["weights"]["group_size"] = 64
    assert ckpt.check_quant(g64) == 64
    # format may sit in the config group instead of the top level
    inner = _quant()
    del inner["format"]
    inner["config_groups"]["group_0"]["format"] = "pack-quantized"
    assert ckpt.check_quant(inner) == 128


def test_triple_contract_violations(tmp_path):
    def model(mutate):
        d = str(tmp_path / ("m%d" % len(os.listdir(tmp_path))))
        os.makedirs(d)
        json.dump(fx.QUANT, open(os.path.join(d, "quantization_config.json"), "w"))
        t, _, _ = fx.linear_tensors("a", 16, 256, 128)
        mutate(t)
        fx.write_safetensors(os.path.join(d, "model.safetensors"), t)
        return d

    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.W4a16Model(model(lambda t: t.pop("a.weight_scale")))
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.W4a16Model(model(lambda t: t.pop("a.weight_shape")))
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.W4a16Model(model(lambda t: t.__setitem__("a.weight_packed", ("F32", [16, 32], t["a.weight_packed"][2]))))
    with pytest.raises(ckpt.W4a16CkptError):  # scale rows do not match
        ckpt.W4a16Model(model(lambda t: t.__setitem__("a.weight_scale", ("F16", [8, 4], t["a.weight_scale"][2]))))
    def only_dense(t):
        t.clear()
        t["x"] = ("F32", [1], bytes(4))

    with pytest.raises(ckpt.W4a16CkptError):  # no quantised tensor at all
        ckpt.W4a16Model(model(only_dense))
    d = model(lambda t: t.__setitem__("a.weight_shape", ("I64", [2], struct.pack("<qq", 16, 999))))
    m = ckpt.W4a16Model(d)
    with pytest.raises(ckpt.W4a16CkptError):  # declared shape disagrees with the packed tensor
        m.lin_operands("a")


def test_missing_config(tmp_path):
    d = str(tmp_path / "m")
    os.makedirs(d)
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.W4a16Model(d)
    json.dump({"model_type": "x"}, open(os.path.join(d, "config.json"), "w"))
    with pytest.raises(ckpt.W4a16CkptError):
        ckpt.W4a16Model(d)
