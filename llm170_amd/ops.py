"""Host-side mirror of the reference's operator interface for the W4A16 linear path, over the C ABI.

  Ctx       <- CudaCtx                      crates/backend-gpu/src/rawcuda/ctx/mod.rs:62-77
  Gptq4     <- Gptq4 (gemv / gemm)          crates/backend-gpu/src/rawcuda/gptq4.rs:72-190
  W4a16Dec  <- W4a16Dec linear entry points crates/backend-gpu/src/rawcuda/w4a16_dec/upload.rs:4-65,
                                            w4a16_dec/kernels/mod.rs:121-144
               MoE entry points             w4a16_dec/upload.rs:1116-1235, w4a16_dec/mod.rs:168-185,
                                            w4a16_dec/kernels/marlin_moe.rs:290-422

Same names, argument meaning and error behaviour (errors surface as W4a16Error carrying the library's message).
numpy arrays stand in for the Rust slices; device pointers are plain ints.
"""
import ctypes as C

import numpy as np

from . import ffi
from .ffi import ACT_GELU_TANH, ACT_SILU, PATH_AUTO, PATH_DECODE, PATH_LANE, PATH_PREFILL, PATH_STREAM, W4a16Error  # noqa: F401


def plan_decode(n, k, group, t, cu_count=256, glu=False):
    """Launch plan of the decode path for a linear of this shape (no context, no GPU): dict of rows_per_wave,
    waves_per_block, k_slices, lds_bytes."""
    rows, waves, nks, lds = C.c_int(), C.c_int(), C.c_int(), C.c_size_t()
    ffi.check(ffi.load().w4a16_plan_decode(n, k, group, t, cu_count, int(bool(glu)), C.byref(rows), C.byref(waves),
                                           C.byref(nks), C.byref(lds)))
    return {"rows_per_wave": rows.value, "waves_per_block": waves.value, "k_slices": nks.value, "lds_bytes": lds.value}


def plan_prefill(t, n, k, cu_count=256, tile_rows=0, k_slices=0, group=128):
    """Launch plan of the prefill path (no context, no GPU): dict of tile_rows, k_slices, super_m, super_n, supers,
    price_us."""
    out = (C.c_size_t * 5)()
    us = C.c_double()
    ffi.check(ffi.load().w4a16_plan_prefill(t, n, k, group, cu_count, tile_rows, k_slices, out, C.byref(us)))
    return {"tile_rows": out[0], "k_slices": out[1], "super_m": out[2], "super_n": out[3], "supers": out[4],
            "price_us": us.value}


def check_shapes(t, qlen, slen, xlen, n, k, group):
    """gptq4.rs:31-58.  Raises W4a16Error(ERR_SHAPE) on violation."""
    ffi.check(ffi.load().w4a16_check_shapes(t, qlen, slen, xlen, n, k, group))


def kernel_sym(group, scale_bf16):
    """gptq4.rs:60-70."""
    r = ffi.load().w4a16_kernel_sym(int(group), int(bool(scale_bf16)))
    if r is None:
        ffi.check(ffi.ERR_UNSUPPORTED)
    return r.decode()


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


class Event:
    def __init__(self, ctx):
        self.ctx = ctx
        h = C.c_void_p()
        ffi.check(ctx.lib.w4a16_event_create(ctx.h, C.byref(h)))
        self.h = h

    def record(self):
        ffi.check(self.ctx.lib.w4a16_event_record(self.ctx.h, self.h))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        ffi.check(self.ctx.lib.w4a16_event_elapsed_ms(self.ctx.h, self.h, stop.h, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self.h:
            self.ctx.lib.w4a16_event_destroy(self.ctx.h, self.h)
            self.h = None


class Graph:
    """A captured sequence of launches (GraphEntry of the reference: exec + handle)."""

    def __init__(self, ctx, handle):
        self.ctx, self.h = ctx, handle

    def launch(self):
        ffi.check(self.ctx.lib.w4a16_graph_launch(self.ctx.h, self.h))

    @property
    def nodes(self):
        return self.ctx.lib.w4a16_graph_nodes(self.h)

    def destroy(self):
        if self.h and self.ctx.h:
            self.ctx.lib.w4a16_graph_destroy(self.ctx.h, self.h)
        self.h = None


class Ctx:
    """Device context: launch stream, loaded gfx950 code objects, tracked allocations."""

    def __init__(self, device=0, asset_dir=None):
        self.lib = ffi.load()
        h = C.c_void_p()
        ffi.check(self.lib.w4a16_ctx_create(device, asset_dir.encode() if asset_dir else None, C.byref(h)))
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            self.lib.w4a16_ctx_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- CudaCtx::alloc / free / h2d / d2h / d2d / sync
    def alloc(self, nbytes):
        p = C.c_uint64()
        ffi.check(self.lib.w4a16_alloc(self.h, nbytes, C.byref(p)))
        return p.value

    def free(self, dptr):
        ffi.check(self.lib.w4a16_free(self.h, dptr))

    def h2d(self, dptr, arr):
        arr = np.ascontiguousarray(arr)
        ffi.check(self.lib.w4a16_h2d(self.h, dptr, _ptr(arr), arr.nbytes))

    def d2h(self, dptr, shape, dtype):
        out = np.empty(shape, dtype)
        ffi.check(self.lib.w4a16_d2h(self.h, _ptr(out), dptr, out.nbytes))
        return out

    def d2d(self, dst, src, nbytes):
        ffi.check(self.lib.w4a16_d2d(self.h, dst, src, nbytes))

    def memset0(self, dptr, nbytes):
        ffi.check(self.lib.w4a16_memset0(self.h, dptr, nbytes))

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.alloc(arr.nbytes)
        self.h2d(p, arr)
        return p

    def sync(self):
        ffi.check(self.lib.w4a16_sync(self.h))

    def allocated_bytes(self):
        return self.lib.w4a16_allocated_bytes(self.h)

    def has_symbol(self, name):
        return self.lib.w4a16_has_symbol(self.h, name.encode()) == 0

    def function(self, name):
        """CudaCtx::function: raises for an unknown symbol, naming it."""
        ffi.check(self.lib.w4a16_has_symbol(self.h, name.encode()))
        return name

    def launch(self, symbol, gx, gy, block, args, shmem=0):
        """CudaCtx::launch: args is a list of ctypes scalars (kept alive for the call)."""
        arr = (C.c_void_p * len(args))(*[C.cast(C.byref(a), C.c_void_p) for a in args])
        ffi.check(self.lib.w4a16_launch(self.h, symbol.encode(), gx, gy, block, shmem, arr))

    def event(self):
        return Event(self)

    def last_launch_symbol(self):
        return self.lib.w4a16_last_launch_symbol(self.h).decode()

    def module_load(self, key, image, symbols):
        """CudaCtx::load_fatbin: a gfx950 code object image and the symbols to resolve from it."""
        arr = (C.c_char_p * len(symbols))(*[s.encode() for s in symbols])
        ffi.check(self.lib.w4a16_module_load(self.h, key.encode(), image, len(image), arr, len(symbols)))

    # ---- CudaCtx::capture_begin / capture_end + graph_instantiate + graph_upload (ctx/graph.rs:4-85)
    def capture_begin(self):
        ffi.check(self.lib.w4a16_capture_begin(self.h))

    def capture_end(self):
        g = C.c_void_p()
        ffi.check(self.lib.w4a16_capture_end(self.h, C.byref(g)))
        return Graph(self, g)


class Gptq4:
    """Standalone operator on the bit-exact kernel (upload, launch, download per call)."""

    def __init__(self, ctx=None):
        self.cc = ctx or Ctx()

    def gemv(self, x, q, s, n, k, group, scale_bf16):
        return self.gemm(x, 1, q, s, n, k, group, scale_bf16)

    def gemm(self, x, t, q, s, n, k, group, scale_bf16):
        x = np.ascontiguousarray(x, np.uint16).ravel()
        q = np.ascontiguousarray(q, np.uint32).ravel()
        s = np.ascontiguousarray(s, np.uint16).ravel()
        check_shapes(t, q.size, s.size, x.size, n, k, group)
        kernel_sym(group, scale_bf16)
        out = np.empty((t, n), np.float32)
        ffi.check(self.cc.lib.w4a16_gemm_host(self.cc.h, _ptr(x), t, _ptr(q), _ptr(s), n, k, group,
                                              int(bool(scale_bf16)), _ptr(out)))
        return out.ravel()


class W4a16Dec:
    """Resident linears by name and the regime dispatch."""

    def __init__(self, ctx=None):
        self.cc = ctx or Ctx()

    def upload_lin(self, name, q, s, n, k):
        return self.upload_lin_g(name, q, s, n, k, 128, False)

    def upload_lin_g(self, name, q, s, n, k, group, scale_bf16):
        q = np.ascontiguousarray(q)
        s = np.ascontiguousarray(s)
        ffi.check(self.cc.lib.w4a16_upload_lin(self.cc.h, name.encode(), _ptr(q), q.nbytes, _ptr(s), s.nbytes, n, k,
                                               group, int(bool(scale_bf16))))

    def lin_fuse(self, name, parts, drop_parts=False):
        """One linear from several that share x (rows concatenated in the order given)."""
        arr = (C.c_char_p * len(parts))(*[p.encode() for p in parts])
        ffi.check(self.cc.lib.w4a16_lin_fuse(self.cc.h, name.encode(), arr, len(parts), int(bool(drop_parts))))

    def lin_forward_multi(self, name, x_dev, outs_dev, t, out_f16=False):
        """gemv_multi_t_dev (w4a16_dec/kernels/gemv.rs:270-300): one decode launch over a fused linear, one output per
        part."""
        arr = (C.c_uint64 * len(outs_dev))(*outs_dev)
        ffi.check(self.cc.lib.w4a16_lin_forward_multi(self.cc.h, name.encode(), x_dev, arr, len(outs_dev), t, int(bool(out_f16))))

    def lin_spec(self, name):
        n, k, g = C.c_size_t(), C.c_size_t(), C.c_size_t()
        bf, tiled, raw = C.c_int(), C.c_int(), C.c_int()
        ffi.check(self.cc.lib.w4a16_lin_info(self.cc.h, name.encode(), C.byref(n), C.byref(k), C.byref(g), C.byref(bf),
                                             C.byref(tiled), C.byref(raw)))
        return {"n": n.value, "k": k.value, "group": g.value, "scale_bf16": bool(bf.value),
                "tiled": bool(tiled.value), "raw": bool(raw.value)}

    def drop_raw(self, name):
        ffi.check(self.cc.lib.w4a16_lin_drop_raw(self.cc.h, name.encode()))

    def lin_forward(self, name, x_dev, dst_dev, t, out_f16=False, path=PATH_AUTO):
        ffi.check(self.cc.lib.w4a16_lin_forward(self.cc.h, name.encode(), x_dev, dst_dev, t, int(out_f16), path))

    def lin_forward_noalloc(self, name, x_dev, dst_dev, t, out_f16=False):
        """lin_forward (decode regime) with the split-K workspace in the library's fixed device array: no allocation."""
        ffi.check(self.cc.lib.w4a16_lin_forward_noalloc(self.cc.h, name.encode(), x_dev, dst_dev, t, int(out_f16)))

    def lin_forward_glu(self, name, x_dev, y_f16_dev, t, gelu=False):
        """Fused gate|up projection with the act(gate)*up epilogue (silu, or the tanh form of gelu): y f16 [t][n/2]."""
        if gelu:
            ffi.check(self.cc.lib.w4a16_lin_forward_glu_act(self.cc.h, name.encode(), x_dev, y_f16_dev, t,
                                                            ffi.ACT_GELU_TANH))
        else:
            ffi.check(self.cc.lib.w4a16_lin_forward_glu(self.cc.h, name.encode(), x_dev, y_f16_dev, t))

    def lin_forward_deferred_norm(self, name, x_dev, t, y_dev, out_f16=False, ldx=0, stats_in=0, n_stats_in=0, in_cols=0,
                                  stats_out=0, stat_rows=0, resid=0, nw=0, in_exp=None, out_exp=None):
        """y = s * (W x) with s = 1/rms of the input from its producer's partial sums; returns the number of partial
        sums this launch wrote to stats_out (0 without one).  in_exp / out_exp: x holds its true values times
        2^-in_exp, y receives its true values times 2^-out_exp (the _scaled entry point; None, None = the plain one)."""
        n_out = C.c_size_t(0)
        if in_exp is None and out_exp is None:
            ffi.check(self.cc.lib.w4a16_lin_forward_deferred_norm(self.cc.h, name.encode(), x_dev, ldx, t, stats_in,
                                                                  n_stats_in, in_cols, y_dev, int(out_f16), stats_out,
                                                                  stat_rows, C.byref(n_out), resid, nw))
        else:
            ffi.check(self.cc.lib.w4a16_lin_forward_deferred_norm_scaled(
                self.cc.h, name.encode(), x_dev, ldx, t, stats_in, n_stats_in, in_cols, in_exp or 0, y_dev, int(out_f16),
                out_exp or 0, stats_out, stat_rows, C.byref(n_out), resid, nw))
        return n_out.value

    def lin_forward_glu_deferred_norm(self, name, x_dev, t, y_f16_dev, ldx=0, stats_in=0, n_stats_in=0, in_cols=0,
                                      gelu=False, in_exp=None, out_exp=None):
        act = ffi.ACT_GELU_TANH if gelu else ffi.ACT_SILU
        if in_exp is None and out_exp is None:
            ffi.check(self.cc.lib.w4a16_lin_forward_glu_deferred_norm(self.cc.h, name.encode(), x_dev, ldx, t, stats_in,
                                                                      n_stats_in, in_cols, y_f16_dev, act))
        else:
            ffi.check(self.cc.lib.w4a16_lin_forward_glu_deferred_norm_scaled(
                self.cc.h, name.encode(), x_dev, ldx, t, stats_in, n_stats_in, in_cols, in_exp or 0, y_f16_dev,
                out_exp or 0, act))

    def row_norm_max(self, name):
        """Largest row norm of the linear's dequantised weights (f32, device arithmetic)."""
        v = C.c_float(0)
        ffi.check(self.cc.lib.w4a16_lin_row_norm_max(self.cc.h, name.encode(), C.byref(v)))
        return v.value

    def gemv_host(self, name, x, t=1, out_f16=False, path=PATH_AUTO):
        """Host operands in, host result out: y [t][n] (f32, or f16 bit patterns when out_f16)."""
        spec = self.lin_spec(name)
        x = np.ascontiguousarray(x, np.uint16).ravel()
        if x.size != t * spec["k"]:
            raise W4a16Error(ffi.ERR_SHAPE, "gemv_host %s: x has %d halves, want t*k = %d" % (name, x.size, t * spec["k"]))
        y = np.empty((t, spec["n"]), np.uint16 if out_f16 else np.float32)
        ffi.check(self.cc.lib.w4a16_lin_forward_host(self.cc.h, name.encode(), _ptr(x), _ptr(y), t, int(out_f16), path))
        return y

    def dequant(self, name, from_tiled=True):
        spec = self.lin_spec(name)
        nbytes = spec["n"] * spec["k"] * 4
        p = self.cc.alloc(nbytes)
        try:
            ffi.check(self.cc.lib.w4a16_dequant_dump(self.cc.h, name.encode(), int(from_tiled), p))
            return self.cc.d2h(p, (spec["n"], spec["k"]), np.float32)
        finally:
            self.cc.free(p)

    def untile(self, name):
        spec = self.lin_spec(name)
        n, k, g = spec["n"], spec["k"], spec["group"]
        pq, ps = self.cc.alloc(n * (k // 8) * 4), self.cc.alloc(n * (k // g) * 2)
        try:
            ffi.check(self.cc.lib.w4a16_lin_untile(self.cc.h, name.encode(), pq, ps))
            return self.cc.d2h(pq, (n, k // 8), np.uint32), self.cc.d2h(ps, (n, k // g), np.uint16)
        finally:
            self.cc.free(pq)
            self.cc.free(ps)

    def set_decode_shape(self, rows_per_wave=0, waves_per_block=0):
        ffi.check(self.cc.lib.w4a16_set_decode_shape(self.cc.h, rows_per_wave, waves_per_block))

    def set_prefill_tile(self, rows=0):
        """0 = automatic, 64 or 128 rows per block tile of the prefill kernel."""
        ffi.check(self.cc.lib.w4a16_set_prefill_tile(self.cc.h, rows))

    def set_decode_ksplit(self, ksplit=0):
        """0 = automatic, -1 = never, n = exactly n k slices across workgroups."""
        ffi.check(self.cc.lib.w4a16_set_decode_ksplit(self.cc.h, ksplit))

    def set_prefill_ksplit(self, ksplit=0):
        ffi.check(self.cc.lib.w4a16_set_prefill_ksplit(self.cc.h, ksplit))

    def bench_forward(self, names, x_dev, y_dev, t, reps, warmup=1, out_f16=False, path=PATH_AUTO):
        """run_bench_gemv / run_bench_gemm (probes/w4a16/gpu/bench.rs:366-433): returns (ms by events, ms wall) for
        `reps` back-to-back launches rotating over `names`."""
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        ms, wall = C.c_float(), C.c_double()
        ffi.check(self.cc.lib.w4a16_bench_forward(self.cc.h, arr, len(names), x_dev, y_dev, t, int(out_f16), path, warmup,
                                                  reps, C.byref(ms), C.byref(wall)))
        return ms.value, wall.value

    # ---- MoE expert FFN
    def upload_experts(self, name, q13, s13, q2, s2, n_experts, h, n_ff, group=32, scale_bf16=False):
        """build_marlin_moe_arenas (upload.rs:1116-1235).  q13 u32 [E][2*n_ff][h/8] (gate rows then up rows),
        s13 u16 [E][2*n_ff][h/group], q2 u32 [E][h][n_ff/8], s2 u16 [E][h][n_ff/group]."""
        arrs = [np.ascontiguousarray(a) for a in (q13, s13, q2, s2)]
        ffi.check(self.cc.lib.w4a16_upload_experts(self.cc.h, name.encode(), n_experts, _ptr(arrs[0]), arrs[0].nbytes,
                                                   _ptr(arrs[1]), arrs[1].nbytes, _ptr(arrs[2]), arrs[2].nbytes,
                                                   _ptr(arrs[3]), arrs[3].nbytes, h, n_ff, group, int(bool(scale_bf16))))

    def experts_spec(self, name):
        e, h, f, g = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_size_t()
        bf = C.c_int()
        ffi.check(self.cc.lib.w4a16_experts_info(self.cc.h, name.encode(), C.byref(e), C.byref(h), C.byref(f),
                                                 C.byref(g), C.byref(bf)))
        return {"n_experts": e.value, "h": h.value, "n_ff": f.value, "group": g.value, "scale_bf16": bool(bf.value)}

    def experts_dequant(self, name, which, expert):
        spec = self.experts_spec(name)
        n, k = (2 * spec["n_ff"], spec["h"]) if which == 0 else (spec["h"], spec["n_ff"])
        p = self.cc.alloc(n * k * 4)
        try:
            ffi.check(self.cc.lib.w4a16_experts_dequant_dump(self.cc.h, name.encode(), which, expert, p))
            return self.cc.d2h(p, (n, k), np.float32)
        finally:
            self.cc.free(p)

    def moe_route(self, logits_dev, t, n_exp, top_k, idx_dev, wt_dev):
        """w4a16_moe_topk_t (assets/moe.cu:686-759) on resident logits."""
        ffi.check(self.cc.lib.w4a16_moe_route(self.cc.h, logits_dev, t, n_exp, top_k, idx_dev, wt_dev))

    def moe_align(self, idx_dev, ns, n_exp, block, sorted_dev, expert_ids_dev, num_post_dev):
        ffi.check(self.cc.lib.w4a16_moe_align(self.cc.h, idx_dev, ns, n_exp, block, sorted_dev, expert_ids_dev,
                                              num_post_dev))

    def moe_ffn(self, name, x_dev, idx_dev, wt_dev, t, top_k, y_dev, gelu=False):
        """marlin_moe_ffn_dev (kernels/marlin_moe.rs:290-422); gelu = its flag of the same name."""
        if gelu:
            ffi.check(self.cc.lib.w4a16_moe_ffn_act(self.cc.h, name.encode(), x_dev, idx_dev, wt_dev, t, top_k, y_dev, ACT_GELU_TANH))
        else:
            ffi.check(self.cc.lib.w4a16_moe_ffn(self.cc.h, name.encode(), x_dev, idx_dev, wt_dev, t, top_k, y_dev))

    def moe_scratch(self, which, dtype):
        """Scratch buffer of the last moe_ffn call as a flat numpy array, plus the segment size used."""
        p, nb, blk = C.c_uint64(), C.c_size_t(), C.c_size_t()
        ffi.check(self.cc.lib.w4a16_moe_scratch(self.cc.h, which, C.byref(p), C.byref(nb), C.byref(blk)))
        return self.cc.d2h(p.value, (nb.value // np.dtype(dtype).itemsize,), dtype), blk.value

    def set_moe_shape(self, block=0, waves=0):
        ffi.check(self.cc.lib.w4a16_set_moe_shape(self.cc.h, block, waves))

    def set_moe_tiled(self, mode=0):
        """MFMA-tiled grouped kernels for the expert FFN: 0 = automatic (long runs per expert), -1 = never, 1 = always."""
        ffi.check(self.cc.lib.w4a16_set_moe_tiled(self.cc.h, mode))

    def bench_moe(self, names, x_dev, idx_dev, wt_dev, t, top_k, y_dev, reps, warmup=1):
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        ms, wall = C.c_float(), C.c_double()
        ffi.check(self.cc.lib.w4a16_bench_moe(self.cc.h, arr, len(names), x_dev, idx_dev, wt_dev, t, top_k, y_dev,
                                              warmup, reps, C.byref(ms), C.byref(wall)))
        return ms.value, wall.value

    # ---- layer chain
    CHAIN_ROLES = ("attn_qkv", "attn_output", "ffn_gate_up", "ffn_down")

    def upload_lin_synth(self, name, n, k, group, seed_q, seed_s, lo=0.002, hi=0.02):
        """A linear generated on the device from the SplitMix64 streams gen.weights_q(seed_q, n, k) and
        gen.scales_f16(seed_s, n, k, group, lo, hi)."""
        ffi.check(self.cc.lib.w4a16_upload_lin_synth(self.cc.h, name.encode(), n, k, group, seed_q, seed_s, lo, hi))

    def upload_chain_synth(self, prefix, n_layers, hidden, n_qkv, n_ff, group=128, seed=None, lo=0.002, hi=0.02):
        """Register n_layers synthetic decoder layers "<prefix>.<l>.<role>" with independent weights; returns the
        (seed_q, seed_s) pairs used, keyed by linear name."""
        from . import gen
        seed = gen.GATE_SEED if seed is None else seed
        shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
                  "ffn_down": (hidden, n_ff)}
        seeds = {}
        for l in range(n_layers):
            for r, role in enumerate(self.CHAIN_ROLES):
                n, k = shapes[role]
                sq, ss = gen.shape_seed(n, k, seed, 100 + 8 * l + 2 * r), gen.shape_seed(n, k, seed, 101 + 8 * l + 2 * r)
                name = "%s.%d.%s" % (prefix, l, role)
                self.upload_lin_synth(name, n, k, group, sq, ss, lo, hi)
                seeds[name] = (sq, ss)
        return seeds

    def rms_rescale_f16(self, v_dev, ld, ncols, t, out_dev):
        ffi.check(self.cc.lib.w4a16_rms_rescale_f16(self.cc.h, v_dev, ld, ncols, t, out_dev))

    def norm_resid(self, x_dev, nw_dev, ab_dev, xn_dev, t, hidden, w_off=0, xn32_dev=0, xn16_dev=0):
        """x <- x + ab; xn = x * inv_rms * nw[w_off:]; optional f16-rounded copies (0 = skip)."""
        ffi.check(self.cc.lib.w4a16_norm_resid(self.cc.h, x_dev, nw_dev, ab_dev, xn_dev, xn32_dev, xn16_dev, t, w_off,
                                               hidden))

    def silu_mul_f16(self, gu_dev, n_ff, t, out_dev):
        ffi.check(self.cc.lib.w4a16_silu_mul_f16(self.cc.h, gu_dev, n_ff, t, out_dev))

    def act_mul_f16(self, gu_dev, n_ff, t, out_dev, gelu=False):
        ffi.check(self.cc.lib.w4a16_act_mul_f16(self.cc.h, gu_dev, n_ff, t, out_dev,
                                                ffi.ACT_GELU_TANH if gelu else ffi.ACT_SILU))

    def chain_forward(self, prefix, layer0, n_layers, x_dev, t, y_dev):
        """chain_device_body (w4a16_dec/chains.rs:195-304) reduced to its linears and glue."""
        ffi.check(self.cc.lib.w4a16_chain_forward(self.cc.h, prefix.encode(), layer0, n_layers, x_dev, t, y_dev))

    def chain_forward_fused(self, prefix, layer0, n_layers, x_dev, t, y_dev):
        """The chain with its normalisations deferred across the linears: four launches per layer, t <= 16."""
        ffi.check(self.cc.lib.w4a16_chain_forward_fused(self.cc.h, prefix.encode(), layer0, n_layers, x_dev, t, y_dev))

    def chain_graph(self, prefix, layer0, n_layers, x_dev, t, y_dev, fused=False):
        """ensure_graph (w4a16_dec/graphs.rs:41-134): one chain step captured for replay."""
        g = C.c_void_p()
        ffi.check(self.cc.lib.w4a16_chain_graph_create(self.cc.h, prefix.encode(), layer0, n_layers, x_dev, t, y_dev,
                                                       int(fused), C.byref(g)))
        return Graph(self.cc, g)

    def bench_chain(self, prefix, n_layers, x_dev, t, y_dev, reps, warmup=1, use_graph=False, fused=False):
        ms, wall = C.c_float(), C.c_double()
        ffi.check(self.cc.lib.w4a16_bench_chain(self.cc.h, prefix.encode(), n_layers, x_dev, t, y_dev, warmup, reps,
                                                int(use_graph), int(fused), C.byref(ms), C.byref(wall)))
        return ms.value, wall.value


def moe_topk(logits, top_k):
    """moe_topk (w4a16_dec/mod.rs:168-185) on the host: logits f32 [t][n_exp] -> (idx int32 [t][top_k], w f32)."""
    logits = np.ascontiguousarray(logits, np.float32)
    if logits.ndim == 1:
        logits = logits[None, :]
    t, n_exp = logits.shape
    idx = np.empty((t, top_k), np.int32)
    w = np.empty((t, top_k), np.float32)
    ffi.check(ffi.load().w4a16_moe_topk_host(_ptr(logits), t, n_exp, top_k, _ptr(idx), _ptr(w)))
    return idx, w
