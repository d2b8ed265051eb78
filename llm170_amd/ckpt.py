"""Reader of W4A16 compressed-tensors checkpoints for the linear path (host side; no device code).

Mirrors the reference's on-disk contract so that the tensors a real checkpoint holds can be registered with
W4a16Dec.upload_lin_g without conversion:

  StArchive    <- crates/core/src/st.rs:105-360      safetensors file or sharded directory, header validation
  W4a16Model   <- crates/core/src/w4a16.rs:99-300    quantisation config check, discovery of the
                                                     <base>.weight_packed / .weight_scale / .weight_shape triples

Tensor data is memory-mapped and handed out as numpy views; nothing is executed from the files (JSON headers only).
"""
import json
import mmap
import os

import numpy as np


class StError(ValueError):
    """Malformed safetensors header or archive (reference: StError::BadHeader)."""


class W4a16CkptError(ValueError):
    """Checkpoint is not a W4A16 compressed-tensors model this path serves (reference: W4a16Error)."""


# dtype name -> (numpy dtype of the raw storage, bytes per element)   st.rs:49-86
ST_DTYPES = {"F16": (np.uint16, 2), "BF16": (np.uint16, 2), "F32": (np.float32, 4), "I16": (np.int16, 2),
             "I32": (np.int32, 4), "I64": (np.int64, 8), "U8": (np.uint8, 1), "F8_E4M3": (np.uint8, 1)}


class StEntry:
    __slots__ = ("dtype", "shape", "begin", "end", "shard")

    def __init__(self, dtype, shape, begin, end, shard):
        self.dtype, self.shape, self.begin, self.end, self.shard = dtype, shape, begin, end, shard

    def nbytes(self):
        return self.end - self.begin


class StArchive:
    """One .safetensors file, or a directory with model*.safetensors shards and an optional
    model.safetensors.index.json (st.rs:115-211)."""

    def __init__(self, path):
        self.shards = []   # (path, data_base, data_len)
        self.entries = {}
        self._maps = {}
        if os.path.isdir(path):
            self._open_dir(path)
        else:
            for name, e in self._parse_shard(path, 0).items():
                self.entries[name] = e

    def _open_dir(self, d):
        idx_path = os.path.join(d, "model.safetensors.index.json")
        weight_map = None
        if os.path.exists(idx_path):
            try:
                v = json.load(open(idx_path), object_pairs_hook=_no_duplicates)
            except ValueError as e:
                raise StError("index.json: %s" % e)
            weight_map = v.get("weight_map") if isinstance(v, dict) else None
            if not isinstance(weight_map, dict):
                raise StError("index.json: weight_map missing")
            for name, f in weight_map.items():
                if not isinstance(f, str):
                    raise StError("weight_map value not a string")
            shard_names = sorted(set(weight_map.values()))
        else:
            shard_names = sorted(f for f in os.listdir(d) if f.endswith(".safetensors") and f.startswith("model"))
            if not shard_names:
                raise StError("no model*.safetensors in %s" % d)
        for si, fname in enumerate(shard_names):
            shard_entries = self._parse_shard(os.path.join(d, fname), si)
            if weight_map is not None:
                for name, f in weight_map.items():
                    if f == fname and name in shard_entries:
                        self.entries[name] = shard_entries[name]
            else:
                self.entries.update(shard_entries)
        if weight_map is not None:
            missing = sorted(n for n in weight_map if n not in self.entries)
            if missing:
                raise StError("index.json: %d tensors not in any shard header %r" % (len(missing), missing[:4]))

    def _parse_shard(self, path, shard):
        with open(path, "rb") as f:
            lenb = f.read(8)
            if len(lenb) != 8:
                raise StError("%s: truncated header length" % path)
            hlen = int.from_bytes(lenb, "little")
            if hlen == 0 or hlen > (1 << 30):
                raise StError("%s: header len %d" % (path, hlen))
            hb = f.read(hlen)
            if len(hb) != hlen:
                raise StError("%s: truncated header" % path)
            data_base = 8 + hlen
            data_len = max(0, os.fstat(f.fileno()).st_size - data_base)
        try:
            obj = json.loads(hb.decode("utf-8"), object_pairs_hook=_no_duplicates)
        except (ValueError, UnicodeDecodeError) as e:
            raise StError("%s: %s" % (path, e))
        if not isinstance(obj, dict):
            raise StError("header not an object")
        out = {}
        for name, tv in obj.items():
            if name == "__metadata__":
                continue
            if not isinstance(tv, dict) or not isinstance(tv.get("dtype"), str):
                raise StError("%s: dtype" % name)
            if tv["dtype"] not in ST_DTYPES:
                raise StError("unknown dtype %s" % tv["dtype"])
            shape, offs = tv.get("shape"), tv.get("data_offsets")
            if not _is_uint_list(shape):
                raise StError("%s: shape" % name)
            if not _is_uint_list(offs):
                raise StError("%s: data_offsets" % name)
            if len(offs) != 2:
                raise StError("%s: offsets len" % name)
            numel = 1
            for s in shape:
                numel *= s
            expect = numel * ST_DTYPES[tv["dtype"]][1]
            if expect >= 1 << 64:
                raise StError("%s: numel overflow" % name)
            if offs[1] < offs[0]:
                raise StError("%s: data_offsets inverted %d..%d" % (name, offs[0], offs[1]))
            if offs[1] - offs[0] != expect:
                raise StError("%s: bytes %d != numel %d x %d" % (name, offs[1] - offs[0], numel, ST_DTYPES[tv["dtype"]][1]))
            out[name] = StEntry(tv["dtype"], list(shape), offs[0], offs[1], shard)
        self.shards.append((path, data_base, data_len))
        return out

    def entry(self, name):
        return self.entries.get(name)

    def shard_paths(self):
        return [p for p, _, _ in self.shards]

    def tensor(self, name):
        """numpy view of the tensor's bytes in its storage dtype and shape (memory-mapped, read-only)."""
        e = self.entries.get(name)
        if e is None:
            raise KeyError(name)
        path, base, data_len = self.shards[e.shard]
        if e.end > data_len:
            raise StError("%s: data range %d..%d beyond the shard's %d data bytes" % (name, e.begin, e.end, data_len))
        mm = self._maps.get(e.shard)
        if mm is None:
            with open(path, "rb") as f:
                mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
            self._maps[e.shard] = mm
        dt = ST_DTYPES[e.dtype][0]
        return np.frombuffer(mm, dtype=dt, count=(e.end - e.begin) // np.dtype(dt).itemsize,
                             offset=base + e.begin).reshape(e.shape)

    def close(self):
        for mm in self._maps.values():
            try:
                mm.close()
            except BufferError:  # a numpy view is still alive
                pass
        self._maps = {}


def _no_duplicates(pairs):
    out = {}
    for k, v in pairs:
        if k in out:
            raise ValueError("duplicate key %s" % k)
        out[k] = v
    return out


def _is_uint_list(v):
    return isinstance(v, list) and all(isinstance(x, int) and not isinstance(x, bool) and x >= 0 for x in v)


def check_quant(cfg):
    """quantization_config contract (w4a16.rs:193-238): compressed-tensors, a single config group, pack-quantized,
    4-bit symmetric weights, group size 32 / 64 / 128.  Returns the group size."""
    if not isinstance(cfg, dict):
        raise W4a16CkptError("quantization_config is not an object")
    method = cfg.get("quant_method", "")
    if method != "compressed-tensors":
        raise W4a16CkptError("quant_method=%r" % (method,))
    cgs = cfg.get("config_groups")
    if not isinstance(cgs, dict):
        raise W4a16CkptError("config_groups missing")
    if len(cgs) != 1:
        raise W4a16CkptError("config_groups has %d entries - a single scheme is supported" % len(cgs))
    g0 = next(iter(cgs.values()))
    fmt = g0.get("format") if isinstance(g0.get("format"), str) else cfg.get("format", "")
    if fmt != "pack-quantized":
        raise W4a16CkptError("format=%r" % (fmt,))
    w = g0.get("weights")
    if not isinstance(w, dict):
        raise W4a16CkptError("group_0.weights missing")
    bits, group, sym = int(w.get("num_bits") or 0), int(w.get("group_size") or 0), bool(w.get("symmetric", False))
    if bits != 4 or not sym:
        raise W4a16CkptError("bits=%d sym=%s - int4 symmetric only" % (bits, sym))
    if group not in (32, 64, 128):
        raise W4a16CkptError("group=%d - g32/g64/g128 only" % group)
    return group


class W4a16Model:
    """A checkpoint directory: quantisation config + the W4A16 linears it holds (w4a16.rs:107-190)."""

    def __init__(self, d):
        self.dir = d
        cfg = None
        for f in ("quantization_config.json", "quant_config.json"):
            p = os.path.join(d, f)
            if os.path.exists(p):
                cfg = _load_json(p)
                break
        if cfg is None:
            p = os.path.join(d, "config.json")
            if not os.path.exists(p):
                raise W4a16CkptError("config.json: missing")
            whole = _load_json(p)
            cfg = whole.get("quantization_config") if isinstance(whole, dict) else None
            if cfg is None:
                raise W4a16CkptError("quantization_config missing (neither sidecar nor embedded)")
        self.group = check_quant(cfg)
        self.ar = StArchive(d)
        self.lins = {}
        for name in self.ar.entries:
            if not name.endswith(".weight_packed"):
                continue
            base = name[:-len(".weight_packed")]
            pk, sc, shp = self.ar.entry(name), self.ar.entry(base + ".weight_scale"), self.ar.entry(base + ".weight_shape")
            if sc is None:
                raise W4a16CkptError("%s: weight_scale missing" % base)
            if shp is None:
                raise W4a16CkptError("%s: weight_shape missing" % base)
            if pk.dtype != "I32":
                raise W4a16CkptError("%s: packed %s" % (base, pk.dtype))
            if sc.dtype not in ("F16", "BF16"):
                raise W4a16CkptError("%s: scale %s" % (base, sc.dtype))
            if shp.dtype != "I64":
                raise W4a16CkptError("%s: shape %s" % (base, shp.dtype))
            if len(pk.shape) != 2 or len(sc.shape) != 2 or shp.shape != [2]:
                raise W4a16CkptError("%s: rank contract violated packed=%r scale=%r shape=%r" % (base, pk.shape, sc.shape, shp.shape))
            n, k = pk.shape[0], pk.shape[1] * 8
            if k % self.group != 0 or n == 0:
                raise W4a16CkptError("%s: n=%d k=%d - not aligned to g%d" % (base, n, k, self.group))
            if sc.shape != [n, k // self.group]:
                raise W4a16CkptError("%s: scale %r != [%d, %d]" % (base, sc.shape, n, k // self.group))
            self.lins[base] = (n, k)
        if not self.lins:
            raise W4a16CkptError("no weight_packed tensor - not a W4A16 checkpoint")

    def lin_shapes(self):
        return sorted((b, n, k) for b, (n, k) in self.lins.items())

    def scale_is_bf16(self, base):
        return self.ar.entry(base + ".weight_scale").dtype == "BF16"

    def lin_operands(self, base):
        """(q u32 [n][k/8], s u16 [n][k/g], n, k, scale_bf16) in the operand format the kernels take; the declared
        weight_shape must agree with the packed shape."""
        n, k = self.lins[base]
        shp = self.ar.tensor(base + ".weight_shape")
        if int(shp[0]) != n or int(shp[1]) != k:
            raise W4a16CkptError("%s: weight_shape %r != packed [%d, %d]" % (base, shp.tolist(), n, k))
        q = self.ar.tensor(base + ".weight_packed").view(np.uint32)
        s = self.ar.tensor(base + ".weight_scale")
        return q, s, n, k, self.scale_is_bf16(base)

    def upload_all(self, dec, names=None):
        """Register every (or the named) linear with a W4a16Dec under its checkpoint name."""
        done = []
        for base, n, k in self.lin_shapes():
            if names is not None and base not in names:
                continue
            q, s, n, k, bf = self.lin_operands(base)
            dec.upload_lin_g(base, q, s, n, k, self.group, bf)
            done.append(base)
        return done

    def upload_fused(self, dec, name, bases):
        """Register the linears `bases` (which share their input: q/k/v, gate/up) as ONE linear `name`, rows in the
        order given; the parts are uploaded, fused on the device and dropped."""
        tmp = []
        for i, base in enumerate(bases):
            q, s, n, k, bf = self.lin_operands(base)
            part = "%s.__part%d" % (name, i)
            dec.upload_lin_g(part, q, s, n, k, self.group, bf)
            tmp.append(part)
        dec.lin_fuse(name, tmp, drop_parts=True)

    def close(self):
        self.ar.close()


def _load_json(p):
    try:
        return json.load(open(p))
    except ValueError as e:
        raise W4a16CkptError("%s: %s" % (os.path.basename(p), e))
