"""ctypes binding of the CPU oracle (oracle/lane_oracle.c).

TEST INFRASTRUCTURE ONLY: importable from tests/, from __graft_entry__.smoke() and from bench.py's cpu_baseline
leg.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblane_oracle.so")


def build(force=False):
    """Compile the C restatement with the flags the numeric contract needs (no FMA contraction)."""
    src = os.path.join(_HERE, "lane_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liblane_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        u16p, u32p, f32p, f64p, u8p = (C.POINTER(C.c_uint16), C.POINTER(C.c_uint32), C.POINTER(C.c_float),
                                       C.POINTER(C.c_double), C.POINTER(C.c_uint8))
        sz = C.c_size_t
        L.orc_half_to_f32.argtypes, L.orc_half_to_f32.restype = [C.c_uint16], C.c_float
        L.orc_half_to_f32_bits.argtypes, L.orc_half_to_f32_bits.restype = [C.c_uint16], C.c_uint32
        L.orc_bf16_to_f32.argtypes, L.orc_bf16_to_f32.restype = [C.c_uint16], C.c_float
        L.orc_f32_to_f16.argtypes, L.orc_f32_to_f16.restype = [C.c_float], C.c_uint16
        L.orc_tree64.argtypes, L.orc_tree64.restype = [f64p], C.c_double
        L.orc_lane_parts.argtypes = [u32p, sz, u32p, sz, f32p, u16p, sz, sz, f64p]
        L.orc_lane_parts.restype = C.c_int
        L.orc_dot_row_lane_group.argtypes = [u32p, sz, u32p, sz, f32p, u16p, sz, sz, f32p]
        L.orc_dot_row_lane_group.restype = C.c_int
        L.orc_dot_row_lane.argtypes = [u32p, sz, u32p, sz, u16p, sz, u16p, sz, f32p]
        L.orc_dot_row_lane.restype = C.c_int
        L.orc_dequant_row_split.argtypes = [u8p, u8p, sz, sz, sz, C.c_int, f32p]
        L.orc_dequant_row_split.restype = None
        L.orc_exact_dot.argtypes, L.orc_exact_dot.restype = [u8p, u8p, f32p, sz, sz, C.c_int], C.c_double
        L.orc_gemm_lane.argtypes = [u16p, sz, u32p, u16p, sz, sz, sz, C.c_int, f32p, C.c_int]
        L.orc_gemm_lane.restype = C.c_int
        L.orc_gemm_lane_sample.argtypes = [u16p, u32p, u16p, sz, sz, C.c_int, u32p, u32p, sz, f32p]
        L.orc_gemm_lane_sample.restype = C.c_int
        L.orc_exact_dot_sample.argtypes = [u16p, u32p, u16p, sz, sz, C.c_int, u32p, u32p, sz, f64p]
        L.orc_exact_dot_sample.restype = C.c_int
        L.orc_moe_topk.argtypes, L.orc_moe_topk.restype = [f32p, sz, sz, u32p, f32p], None
        L.orc_silu_mul_f16.argtypes, L.orc_silu_mul_f16.restype = [C.c_float, C.c_float], C.c_uint16
        L.orc_f32_to_f16_array.argtypes, L.orc_f32_to_f16_array.restype = [f32p, sz, u16p], None
        L.orc_rms_rescale_f16.argtypes, L.orc_rms_rescale_f16.restype = [f32p, sz, sz, sz, u16p], None
        L.orc_silu_mul_f16_rows.argtypes, L.orc_silu_mul_f16_rows.restype = [f32p, sz, sz, u16p], None
        L.orc_gelu_mul_f16_rows.argtypes, L.orc_gelu_mul_f16_rows.restype = [f32p, sz, sz, u16p], None
        L.orc_norm_resid.argtypes, L.orc_norm_resid.restype = [f32p, f32p, f32p, f32p, f32p, u16p, sz, sz, sz], None
        i32p = C.POINTER(C.c_int32)
        L.orc_moe_act_silu_f16.argtypes, L.orc_moe_act_silu_f16.restype = [u16p, sz, sz, u16p], None
        L.orc_moe_act_gelu_f16.argtypes, L.orc_moe_act_gelu_f16.restype = [u16p, sz, sz, u16p], None
        L.orc_moe_topk_sum_f16.argtypes, L.orc_moe_topk_sum_f16.restype = [u16p, sz, sz, sz, f32p], None
        L.orc_moe_align.argtypes, L.orc_moe_align.restype = [i32p, sz, sz, sz, i32p, i32p], sz
        _lib = L
    return _lib


def _p(a, ty):
    return a.ctypes.data_as(C.POINTER(ty))


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def half_to_f32(h):
    return float(lib().orc_half_to_f32(int(h)))


def bf16_to_f32(h):
    return float(lib().orc_bf16_to_f32(int(h)))


def f32_to_f16(v):
    return int(lib().orc_f32_to_f16(float(np.float32(v))))


def half_to_f32_bits_all():
    """f32 bit patterns of half_to_f32 for all 65536 halves."""
    L = lib()
    return np.fromiter((L.orc_half_to_f32_bits(h) for h in range(65536)), dtype=np.uint32, count=65536)


def f32_to_f16_array(v):
    v = _c(v, np.float32).ravel()
    out = np.empty(v.size, np.uint16)
    lib().orc_f32_to_f16_array(_p(v, C.c_float), v.size, _p(out, C.c_uint16))
    return out


def tree64(v):
    v = _c(v, np.float64)
    assert v.shape == (64,)
    return float(lib().orc_tree64(_p(v, C.c_double)))


def lane_parts(qrow, zrow, srow_f32, x, group):
    qrow, zrow, srow_f32, x = _c(qrow, np.uint32), _c(zrow, np.uint32), _c(srow_f32, np.float32), _c(x, np.uint16)
    out = np.empty(64, np.float64)
    rc = lib().orc_lane_parts(_p(qrow, C.c_uint32), qrow.size, _p(zrow, C.c_uint32), zrow.size,
                              _p(srow_f32, C.c_float), _p(x, C.c_uint16), x.size, group, _p(out, C.c_double))
    if rc != 0:
        raise ValueError("lane_parts: shape contract (lane.rs:50-55) violated")
    return out


def dot_row_lane_group(qrow, zrow, srow_f32, x, group):
    qrow, zrow, srow_f32, x = _c(qrow, np.uint32), _c(zrow, np.uint32), _c(srow_f32, np.float32), _c(x, np.uint16)
    out = C.c_float()
    rc = lib().orc_dot_row_lane_group(_p(qrow, C.c_uint32), qrow.size, _p(zrow, C.c_uint32), zrow.size,
                                      _p(srow_f32, C.c_float), _p(x, C.c_uint16), x.size, group, C.byref(out))
    if rc != 0:
        raise ValueError("dot_row_lane_group: shape contract (lane.rs:50-55) violated")
    return np.float32(out.value)


def dot_row_lane(qrow, zrow, srow_f16, x):
    qrow, zrow, srow_f16, x = _c(qrow, np.uint32), _c(zrow, np.uint32), _c(srow_f16, np.uint16), _c(x, np.uint16)
    out = C.c_float()
    rc = lib().orc_dot_row_lane(_p(qrow, C.c_uint32), qrow.size, _p(zrow, C.c_uint32), zrow.size,
                                _p(srow_f16, C.c_uint16), srow_f16.size, _p(x, C.c_uint16), x.size, C.byref(out))
    if rc != 0:
        raise ValueError("dot_row_lane: shape contract (lane.rs:26-28) violated")
    return np.float32(out.value)


def dequant_row_split(q_bytes, s_bytes, row, k, group, scale_bf16):
    q_bytes, s_bytes = _c(q_bytes, np.uint8), _c(s_bytes, np.uint8)
    out = np.empty(k, np.float32)
    lib().orc_dequant_row_split(_p(q_bytes, C.c_uint8), _p(s_bytes, C.c_uint8), row, k, group, int(scale_bf16),
                                _p(out, C.c_float))
    return out


def dequant_matrix(q, s, n, k, group, scale_bf16=False):
    """All rows of orc_dequant_row_split: f32 [n][k]."""
    qb = _c(q, np.uint32).view(np.uint8).ravel()
    sb = _c(s, np.uint16).view(np.uint8).ravel()
    out = np.empty((n, k), np.float32)
    L = lib()
    for r in range(n):
        L.orc_dequant_row_split(_p(qb, C.c_uint8), _p(sb, C.c_uint8), r, k, group, int(scale_bf16),
                                out[r].ctypes.data_as(C.POINTER(C.c_float)))
    return out


def exact_dot(qrow_bytes, srow_bytes, x_f32, k, group, scale_bf16):
    qrow_bytes, srow_bytes, x_f32 = _c(qrow_bytes, np.uint8), _c(srow_bytes, np.uint8), _c(x_f32, np.float32)
    return float(lib().orc_exact_dot(_p(qrow_bytes, C.c_uint8), _p(srow_bytes, C.c_uint8), _p(x_f32, C.c_float), k,
                                     group, int(scale_bf16)))


def gemm_lane(x, t, q, s, n, k, group, scale_bf16=False, threads=1):
    """out[t][n] f32 exactly as the parity gate's expectation (gates.rs:113-132)."""
    x, q, s = _c(x, np.uint16).ravel(), _c(q, np.uint32).ravel(), _c(s, np.uint16).ravel()
    assert x.size == t * k and q.size == n * (k // 8) and s.size == n * (k // group)
    out = np.empty((t, n), np.float32)
    rc = lib().orc_gemm_lane(_p(x, C.c_uint16), t, _p(q, C.c_uint32), _p(s, C.c_uint16), n, k, group,
                             int(scale_bf16), _p(out, C.c_float), int(threads))
    if rc != 0:
        raise ValueError("gemm_lane: shape contract violated")
    return out


def gemm_lane_sample(x, q, s, k, group, rows, toks, scale_bf16=False):
    x, q, s = _c(x, np.uint16).ravel(), _c(q, np.uint32).ravel(), _c(s, np.uint16).ravel()
    rows, toks = _c(rows, np.uint32), _c(toks, np.uint32)
    out = np.empty(rows.size, np.float32)
    rc = lib().orc_gemm_lane_sample(_p(x, C.c_uint16), _p(q, C.c_uint32), _p(s, C.c_uint16), k, group,
                                    int(scale_bf16), _p(rows, C.c_uint32), _p(toks, C.c_uint32), rows.size,
                                    _p(out, C.c_float))
    if rc != 0:
        raise ValueError("gemm_lane_sample: shape contract violated")
    return out


def exact_dot_sample(x, q, s, k, group, rows, toks, scale_bf16=False):
    """f64 [count]: the compensated f64 dot (quant/exact.rs:27-53) of row rows[j] with x row toks[j]."""
    x, q, s = _c(x, np.uint16).ravel(), _c(q, np.uint32).ravel(), _c(s, np.uint16).ravel()
    rows, toks = _c(rows, np.uint32), _c(toks, np.uint32)
    out = np.empty(rows.size, np.float64)
    rc = lib().orc_exact_dot_sample(_p(x, C.c_uint16), _p(q, C.c_uint32), _p(s, C.c_uint16), k, group,
                                    int(scale_bf16), _p(rows, C.c_uint32), _p(toks, C.c_uint32), rows.size,
                                    _p(out, C.c_double))
    if rc != 0:
        raise ValueError("exact_dot_sample: shape contract violated")
    return out


def moe_topk(logits, k):
    logits = _c(logits, np.float32)
    kk = min(k, logits.size)
    idx = np.empty(kk, np.uint32)
    w = np.empty(kk, np.float32)
    lib().orc_moe_topk(_p(logits, C.c_float), logits.size, k, _p(idx, C.c_uint32), _p(w, C.c_float))
    return idx, w


def silu_mul_f16(g, u):
    return int(lib().orc_silu_mul_f16(float(np.float32(g)), float(np.float32(u))))


def moe_act_silu_f16(c13, ns, n_ff):
    """f16 bits [ns][2*n_ff] (gate | up) -> f16 bits [ns][n_ff]."""
    c13 = _c(c13, np.uint16).reshape(ns, 2 * n_ff)
    act = np.empty((ns, n_ff), np.uint16)
    lib().orc_moe_act_silu_f16(_p(c13, C.c_uint16), ns, n_ff, _p(act, C.c_uint16))
    return act


def moe_act_gelu_f16(c13, ns, n_ff):
    """w4a16_moe_act_gelu_f16 (assets/moe.cu:1635-1647): f16 bits [ns][2*n_ff] -> f16 bits [ns][n_ff]."""
    c13 = _c(c13, np.uint16).reshape(ns, 2 * n_ff)
    act = np.empty((ns, n_ff), np.uint16)
    lib().orc_moe_act_gelu_f16(_p(c13, C.c_uint16), ns, n_ff, _p(act, C.c_uint16))
    return act


def moe_topk_sum_f16(c2, t, h, top_k):
    c2 = _c(c2, np.uint16).reshape(t * top_k, h)
    out = np.empty((t, h), np.float32)
    lib().orc_moe_topk_sum_f16(_p(c2, C.c_uint16), t, h, top_k, _p(out, C.c_float))
    return out


def moe_align(idx, n_exp, block):
    """-> (sorted_ids int32 [num_post], expert_ids int32 [num_post/block], num_post)."""
    idx = _c(idx, np.int32).ravel()
    ns = idx.size
    sorted_ids = np.empty(ns + n_exp * block, np.int32)
    expert_ids = np.empty(ns // block + n_exp + 1, np.int32)
    n_post = lib().orc_moe_align(_p(idx, C.c_int32), ns, n_exp, block, _p(sorted_ids, C.c_int32),
                                 _p(expert_ids, C.c_int32))
    return sorted_ids[:n_post].copy(), expert_ids[:n_post // block].copy(), int(n_post)


def moe_topk_batch(logits, k):
    logits = _c(logits, np.float32)
    t = logits.shape[0]
    idx = np.empty((t, k), np.int32)
    w = np.empty((t, k), np.float32)
    for i in range(t):
        a, b = moe_topk(logits[i], k)
        idx[i], w[i] = a.astype(np.int32), b
    return idx, w


def moe_ffn(x, idx, wt, q13, s13, q2, s2, h, n_ff, group, scale_bf16=False, threads=1, act_in=None, gelu=False):
    """The routed-expert FFN of the reference's device path (kernels/marlin_moe.rs:290-422) with every GEMM done by
    the lane contract: per slot j (token j // top_k, expert idx[j])
        c13 = f16(lane(W13[e], x[token]));  act = f16(silu(gate) * up)   (gelu: the tanh form of gelu instead of silu)
        c2  = f16(wt[j] * lane(W2[e], act));  y[token] = sum_k c2 in slot order (f32).
    x: f16 bits [t][h]; idx int32 [t][top_k]; wt f32 [t][top_k]; q13 u32 [E][2*n_ff][h/8] ...
    act_in (f16 bits [ns][n_ff]) replaces the first stage's result when given (stage-wise checks).
    Returns dict(c13, act, c2, y)."""
    x = _c(x, np.uint16).reshape(-1, h)
    t, top_k = idx.shape
    ns = t * top_k
    flat = _c(idx, np.int32).ravel()
    wflat = _c(wt, np.float32).ravel()
    c13 = np.zeros((ns, 2 * n_ff), np.uint16)
    c2 = np.zeros((ns, h), np.uint16)
    act = np.zeros((ns, n_ff), np.uint16) if act_in is None else _c(act_in, np.uint16).reshape(ns, n_ff).copy()
    order = np.argsort(flat, kind="stable")
    bounds = np.flatnonzero(np.diff(flat[order], prepend=-1, append=1 << 30))
    for b0, b1 in zip(bounds[:-1], bounds[1:]):
        slots = order[b0:b1]
        e = int(flat[slots[0]])
        if act_in is None:
            xs = x[slots // top_k]
            y13 = gemm_lane(xs, len(slots), q13[e], s13[e], 2 * n_ff, h, group, scale_bf16, threads)
            c13[slots] = f32_to_f16_array(y13).reshape(len(slots), 2 * n_ff)
            act[slots] = (moe_act_gelu_f16 if gelu else moe_act_silu_f16)(c13[slots], len(slots), n_ff)
        y2 = gemm_lane(act[slots], len(slots), q2[e], s2[e], h, n_ff, group, scale_bf16, threads)
        y2 = (y2 * wflat[slots][:, None]).astype(np.float32)
        c2[slots] = f32_to_f16_array(y2).reshape(len(slots), h)
    y = moe_topk_sum_f16(c2, t, h, top_k)
    return {"c13": c13, "act": act, "c2": c2, "y": y}


def rms_rescale_f16(v, ncols):
    """v f32 [t][ld] -> f16 bits [t][ncols] over the first ncols columns of every row."""
    v = _c(v, np.float32)
    t, ld = v.shape
    out = np.empty((t, ncols), np.uint16)
    lib().orc_rms_rescale_f16(_p(v, C.c_float), ld, ncols, t, _p(out, C.c_uint16))
    return out


def norm_resid(x, nw, ab, w_off=0):
    """norm_resid (assets/norm.cu:4-48): returns (x + ab, xn f32, xn32 f32, xn16 f16 bits), each [t][hidden]."""
    x = np.array(x, np.float32, order="C")  # copy: updated in place
    ab, nw = _c(ab, np.float32), _c(nw, np.float32)
    t, hidden = x.shape
    assert ab.shape == x.shape and nw.size >= w_off + hidden
    xn, xn32, xn16 = np.empty_like(x), np.empty_like(x), np.empty(x.shape, np.uint16)
    lib().orc_norm_resid(_p(x, C.c_float), _p(nw, C.c_float), _p(ab, C.c_float), _p(xn, C.c_float), _p(xn32, C.c_float),
                         _p(xn16, C.c_uint16), t, w_off, hidden)
    return x, xn, xn32, xn16


def silu_mul_f16_rows(gu):
    gu = _c(gu, np.float32)
    t, two = gu.shape
    out = np.empty((t, two // 2), np.uint16)
    lib().orc_silu_mul_f16_rows(_p(gu, C.c_float), two // 2, t, _p(out, C.c_uint16))
    return out


def gelu_mul_f16_rows(gu):
    """ew_gelu (assets/ew.cu:34-57): f32 [t][2*n_ff] = (gate | up) -> f16 bits [t][n_ff]."""
    gu = _c(gu, np.float32)
    t, two = gu.shape
    out = np.empty((t, two // 2), np.uint16)
    lib().orc_gelu_mul_f16_rows(_p(gu, C.c_float), two // 2, t, _p(out, C.c_uint16))
    return out


def chain_layer(x, lins, group=128, threads=1):
    """One decoder layer of linears with its glue (the build's statement of chain_device_body, chains.rs:195-304):
    lins = [(q, s, n, k)] for attn_qkv, attn_output, ffn_gate_up, ffn_down; x f16 bits [t][hidden].
    Returns the stage outputs {qkv, a, o, b, gu, c, d, x}."""
    x = _c(x, np.uint16)
    t, hidden = x.shape
    (q0, s0, n0, k0), (q1, s1, n1, k1), (q2, s2, n2, k2), (q3, s3, n3, k3) = lins
    st = {}
    st["qkv"] = gemm_lane(x, t, q0, s0, n0, k0, group, False, threads)
    st["a"] = rms_rescale_f16(st["qkv"], hidden)
    st["o"] = gemm_lane(st["a"], t, q1, s1, n1, k1, group, False, threads)
    st["b"] = rms_rescale_f16(st["o"], hidden)
    st["gu"] = gemm_lane(st["b"], t, q2, s2, n2, k2, group, False, threads)
    st["c"] = silu_mul_f16_rows(st["gu"])
    st["d"] = gemm_lane(st["c"], t, q3, s3, n3, k3, group, False, threads)
    st["x"] = rms_rescale_f16(st["d"], hidden)
    return st


def rms_inv(v, ncols):
    """Per row: f32(1 / sqrt(mean(v[:, :ncols]^2) + 1e-6)), the mean taken in f64 (the factor rms_rescale_f16 applies)."""
    v64 = _c(v, np.float32)[:, :ncols].astype(np.float64)
    return (1.0 / np.sqrt(np.mean(v64 * v64, axis=1) + 1e-6)).astype(np.float32)


def chain_layer_fused(x, s_in, lins, group=128, threads=1):
    """chain_layer with each normalisation applied after the linear that follows it: x f16 bits [t][hidden] travel
    un-normalised, s_in f32 [t] is the factor they still lack (ones for a normalised input).  Every product is one f32
    rounding.  Returns the stage values {v1, a, v2, b, gu, c, v4, x, s}: x = f16(v4), s = rms_inv(v4)."""
    x = _c(x, np.uint16)
    t, hidden = x.shape
    s_in = _c(s_in, np.float32).reshape(t, 1)
    (q0, s0, n0, k0), (q1, s1, n1, k1), (q2, s2, n2, k2), (q3, s3, n3, k3) = lins
    st = {}
    st["v1"] = (s_in * gemm_lane(x, t, q0, s0, n0, k0, group, False, threads)[:, :hidden]).astype(np.float32)
    st["a"] = f32_to_f16_array(st["v1"]).reshape(t, -1)
    st["v2"] = (rms_inv(st["v1"], hidden).reshape(t, 1) * gemm_lane(st["a"], t, q1, s1, n1, k1, group, False, threads)).astype(np.float32)
    st["b"] = f32_to_f16_array(st["v2"]).reshape(t, -1)
    st["gu"] = (rms_inv(st["v2"], hidden).reshape(t, 1) * gemm_lane(st["b"], t, q2, s2, n2, k2, group, False, threads)).astype(np.float32)
    st["c"] = silu_mul_f16_rows(st["gu"])
    st["v4"] = gemm_lane(st["c"], t, q3, s3, n3, k3, group, False, threads)
    st["x"] = f32_to_f16_array(st["v4"]).reshape(t, -1)
    st["s"] = rms_inv(st["v4"], hidden)
    return st
