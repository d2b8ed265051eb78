"""Writes small synthetic compressed-tensors W4A16 checkpoints in the reference's on-disk format (the format its own
fixture script scripts/gen_tiny_w4a16.py:44-75 produces: 8-byte little-endian header length, JSON header, tensor
bytes; <base>.weight_packed I32 [n][k/8], .weight_scale F16/BF16 [n][k/g], .weight_shape I64 [2])."""
import json
import os
import struct

import numpy as np

from llm170_amd import gen

QUANT = {"quant_method": "compressed-tensors", "format": "pack-quantized",
         "config_groups": {"group_0": {"weights": {"num_bits": 4, "group_size": 128, "symmetric": True, "type": "int"},
                                       "targets": ["Linear"]}}}


def write_safetensors(path, tensors, metadata=True):
    """tensors: {name: (dtype string, shape list, bytes)}.  The archive layout (u64 header length, JSON header whose
    entries give each tensor's byte range in the data section, then the data section) is the container's definition;
    tensors are laid out in name order, each range derived from the running sizes."""
    order = sorted(tensors)
    ends = np.cumsum([len(tensors[name][2]) for name in order]).tolist()
    starts = [0] + ends[:-1]
    header = {"__metadata__": {"format": "pt"}} if metadata else {}
    for name, lo, hi in zip(order, starts, ends):
        dtype, shape, _ = tensors[name]
        header[name] = {"dtype": dtype, "shape": [int(d) for d in shape], "data_offsets": [int(lo), int(hi)]}
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    with open(path, "wb") as out:
        out.write(len(text).to_bytes(8, "little"))
        out.write(text)
        for name in order:
            out.write(tensors[name][2])


def linear_tensors(base, n, k, group, bf16=False, seed=1):
    q = gen.weights_q(gen.shape_seed(n, k, seed, 1), n, k)
    s = gen.scales_f16(gen.shape_seed(n, k, seed, 2), n, k, group)
    if bf16:
        s = (gen.f16_bits_to_f32(s).view(np.uint32) >> 16).astype(np.uint16)
    t = {base + ".weight_packed": ("I32", [n, k // 8], q.tobytes()),
         base + ".weight_scale": ("BF16" if bf16 else "F16", [n, k // group], s.tobytes()),
         base + ".weight_shape": ("I64", [2], struct.pack("<qq", n, k))}
    return t, q, s


def write_model(d, lins, group=128, bf16=False, shards=1, sidecar=True, index=False):
    """lins: [(base, n, k)].  Returns {base: (q, s)}."""
    os.makedirs(d, exist_ok=True)
    quant = json.loads(json.dumps(QUANT))
    quant["config_groups"]["group_0"]["weights"]["group_size"] = group
    if sidecar:
        json.dump(quant, open(os.path.join(d, "quantization_config.json"), "w"))
    else:
        json.dump({"model_type": "tiny", "quantization_config": quant}, open(os.path.join(d, "config.json"), "w"))
    per_shard = [dict() for _ in range(shards)]
    ops, weight_map = {}, {}
    for i, (base, n, k) in enumerate(lins):
        t, q, s = linear_tensors(base, n, k, group, bf16, seed=10 + i)
        ops[base] = (q, s)
        per_shard[i % shards].update(t)
        per_shard[i % shards]["model.norm_%d.weight" % i] = ("F32", [4], np.ones(4, np.float32).tobytes())
    for si, t in enumerate(per_shard):
        fname = "model.safetensors" if shards == 1 else "model-%05d-of-%05d.safetensors" % (si + 1, shards)
        write_safetensors(os.path.join(d, fname), t)
        for name in t:
            weight_map[name] = fname
    if index:
        json.dump({"metadata": {}, "weight_map": weight_map}, open(os.path.join(d, "model.safetensors.index.json"), "w"))
    return ops
