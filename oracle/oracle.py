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
        L.orc_moe_topk.argtypes, L.orc_moe_topk.restype = [f32p, sz, sz, u32p, f32p], None
        L.orc_silu_mul_f16.argtypes, L.orc_silu_mul_f16.restype = [C.c_float, C.c_float], C.c_uint16
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
    L = lib()
    return np.fromiter((L.orc_f32_to_f16(float(x)) for x in v), dtype=np.uint16, count=v.size)


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


def moe_topk(logits, k):
    logits = _c(logits, np.float32)
    kk = min(k, logits.size)
    idx = np.empty(kk, np.uint32)
    w = np.empty(kk, np.float32)
    lib().orc_moe_topk(_p(logits, C.c_float), logits.size, k, _p(idx, C.c_uint32), _p(w, C.c_float))
    return idx, w


def silu_mul_f16(g, u):
    return int(lib().orc_silu_mul_f16(float(np.float32(g)), float(np.float32(u))))
