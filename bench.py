#!/usr/bin/env python3
"""Benchmark of the W4A16 linear path on one MI355X.

Headline workload (one "step" = one pass of the hot path over one batch): the decode GEMV of the fused gate+up
projection of the 27B dense layer, M=1, K=5120, N=34816, group 128, f16 activations in, f16 out with f32
accumulation.  Operands are resident in HBM before the timed region.  Each step uses the next of several distinct
weight copies whose total size exceeds L2 + the 256 MB last-level cache, so every step streams its weights from HBM.

Prints ONE JSON line.  `value` is algorithmic bytes per step / time per step (GB/s):
    bytes(M,K,N,g) = N*K/2 (int4 weights) + 2*N*K/g (f16 scales) + 2*M*K (x) + 2*M*N (y)
`roofline` prices the same kernel against the 8 TB/s HBM peak; `cpu_baseline` times the CPU oracle (lane-order
restatement of the reference's CPU contract) on the box's host cores.
"""
import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense f16 MFMA, published


def algorithmic_bytes(m, k, n, g):
    return n * k // 2 + 2 * n * k // g + 2 * m * k + 2 * m * n


def make_copies(dec, gen, n, k, g, copies, prefix):
    names = []
    first = None
    for c in range(copies):
        sq, ss = gen.shape_seed(n, k, tensor=1) + 977 * c, gen.shape_seed(n, k, tensor=2) + 977 * c
        name = "%s.%d" % (prefix, c)
        if c == 0:  # the copy the oracle checks is generated on the host; the others, same streams, on the device
            first = (gen.weights_q(sq, n, k), gen.scales_f16(ss, n, k, g))
            dec.upload_lin_g(name, first[0], first[1], n, k, g, False)
        else:
            dec.upload_lin_synth(name, n, k, g, sq, ss)
        dec.drop_raw(name)
        names.append(name)
    return names, first


def kernel_source_hash(kernel):
    """sha256 (16 hex digits) over the source file a kernel is built from and the header all kernels share."""
    csrc = os.path.join(ROOT, "llm170_amd", "csrc")
    src = ("bench/probes.hip" if kernel in PROBE_SYMS else "kernels/decode.hip" if kernel.startswith("w4a16_decode")
           else "kernels/prefill.hip" if kernel.startswith("w4a16_prefill") else None)
    if src is None:
        return None
    h = hashlib.sha256()
    for f in (src, "kernels/w4a16_common.hpp"):
        with open(os.path.join(csrc, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` from the committed counter summary profiles/pmc_traffic.txt (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE, scaled by the plain-copy calibration): (bytes, provenance) — a recorded figure, not a
    measurement of this run.  The summary records the hash of the kernel's source at the time of the counter runs;
    (None, reason) when it has no line for the kernel this run dispatched or when that source has changed since."""
    path = os.path.join(ROOT, "profiles", "pmc_traffic.txt")
    if not os.path.exists(path):
        return None, "no profiles/pmc_traffic.txt"
    recorded, value = None, None
    for ln in open(path):
        f = ln.split()
        if len(f) >= 3 and f[0] == kernel and f[1] == "kernel_source_hash":
            recorded = f[2]
        if len(f) >= 3 and f[0] == kernel and f[1] == "traffic_bytes_per_launch":
            value = int(float(f[2]))
    if value is None:
        return None, "profiles/pmc_traffic.txt has no record for %s" % kernel
    now = kernel_source_hash(kernel)
    if recorded != now:
        return None, "profiles/pmc_traffic.txt: %s was recorded at kernel source %s, the source is now %s" % (kernel, recorded, now)
    return value, "profiles/pmc_traffic.txt, kernel %s, recorded at kernel source %s" % (kernel, recorded)


PROBE_SYMS = ["w4a16_copy_u4", "w4a16_read_u4", "w4a16_mfma_peak_f16"]


def load_probes(cc):
    """The measurement kernels are not product assets: their code object is loaded here through w4a16_module_load."""
    if not cc.has_symbol(PROBE_SYMS[0]):
        image = open(os.path.join(ROOT, "llm170_amd", "assets", "bench_probes.hsaco"), "rb").read()
        cc.module_load("bench_probes", image, PROBE_SYMS)


def chip_probes(cc, nbytes, copies):
    """What the chip sustains with nothing but the bounding resource in use (context for the roofline fractions, which
    stay priced against the published peaks): a read-only stream over buffers of the headline linear's size, rotated
    like its weight copies, launch after launch as in the timed region; the same stream as one long launch; and a loop
    of v_mfma_f32_32x32x16_f16 on independent accumulators."""
    import ctypes as C
    load_probes(cc)
    n16 = (nbytes + 15) // 16
    buf = cc.alloc(n16 * 16 * copies)
    cc.memset0(buf, n16 * 16 * copies)
    sink = cc.alloc(256)
    e0, e1 = cc.event(), cc.event()

    def read_run(blocks, reps, span, rotate):
        for timed in (False, True):
            e0.record()
            for r in range(reps):
                src = buf + (r % copies) * n16 * 16 if rotate else buf
                cc.launch("w4a16_read_u4", blocks, 1, 256, [C.c_uint64(src), C.c_size_t(span), C.c_uint64(sink)])
            e1.record()
            cc.sync()
        return e0.elapsed_ms(e1) / reps

    per_launch = min(read_run(b, 400, n16, True) for b in (2048, 4096, 8192))
    one_long = min(read_run(b, 4, n16 * copies, False) for b in (2048, 4096, 8192))
    iters, blocks = 4096, 1024
    for timed in (False, True):
        e0.record()
        for r in range(8):
            cc.launch("w4a16_mfma_peak_f16", blocks, 1, 256, [C.c_uint64(sink), C.c_int(iters)])
        e1.record()
        cc.sync()
    mfma_ms = e0.elapsed_ms(e1) / 8
    e0.destroy()
    e1.destroy()
    cc.free(buf)
    cc.free(sink)
    return {"read_only_GBps_per_launch_same_bytes": round(n16 * 16 / per_launch / 1e6, 1),
            "read_only_us_per_launch_same_bytes": round(per_launch * 1e3, 2),
            "read_only_GBps_one_long_launch": round(n16 * 16 * copies / one_long / 1e6, 1),
            "mfma_f16_loop_TFLOPs": round(blocks * 4 * iters * 4 * 32768 / mfma_ms / 1e9, 1)}


def time_forward(dec, names, xd, yd, t, steps, warmup, path, out_f16=True):
    ms, wall = dec.bench_forward(names, xd, yd, t, steps, warmup=warmup, out_f16=out_f16, path=path)
    return ms / steps, wall / steps


ROUNDS = 5  # every leg is timed as this many rounds of its K launches; the median round is reported, min and max beside it


def spread(samples, scale=1.0, digits=3):
    v = sorted(samples)
    return {"median": round(v[len(v) // 2] * scale, digits), "min": round(v[0] * scale, digits),
            "max": round(v[-1] * scale, digits), "rounds": len(v)}


def time_rounds(dec, names, xd, yd, t, steps, warmup, path, out_f16=True, rounds=ROUNDS):
    """`rounds` timed regions of exactly `steps` launches each (HIP events on the launch stream), `warmup` untimed
    launches before each; returns (median ms per launch, all samples, wall ms per launch of the median round)."""
    got = [time_forward(dec, names, xd, yd, t, steps, warmup, path, out_f16) for _ in range(rounds)]
    got.sort()
    med = got[len(got) // 2]
    return med[0], [g[0] for g in got], med[1]


def bench_moe(dec, gen, ops, args):
    """MoE expert FFN of the 35B-A3B layer shape: 128 experts, top-8, hidden 2048, n_ff 768, group 32; routing from
    seeded N(0,1) router logits (ragged per-expert row counts).  Bytes = distinct experts hit x (weights + scales of
    both projections) + activations in and out of every stage."""
    cc = dec.cc
    E, h, n_ff, g, k = 128, 2048, 768, 32, 8
    q13, s13, q2, s2 = gen.make_experts(E, h, n_ff, g)
    names = []
    for c in range(3):  # 3 x 340 MB of experts rotated: beyond L2 + last-level cache
        dec.upload_experts("experts.%d" % c, q13, s13, q2, s2, E, h, n_ff, g, False)
        names.append("experts.%d" % c)
    per_expert = (2 * n_ff * h // 2 + 2 * n_ff * (h // g) * 2) + (h * n_ff // 2 + h * (n_ff // g) * 2)
    out = []
    for t in (1, 4, 64, 512):
        x = gen.normal_f16(1 + t, (t, h))
        lg = cc.to_device(gen.router_logits(t, E))
        px, pi, pw, py = cc.to_device(x), cc.alloc(t * k * 4), cc.alloc(t * k * 4), cc.alloc(t * h * 4)
        dec.moe_route(lg, t, E, k, pi, pw)
        hit = int(np.unique(cc.d2h(pi, (t * k,), np.int32)).size)
        ns = t * k
        nbytes = hit * per_expert + t * h * 2 + 2 * ns * n_ff * 2 + 2 * ns * h * 2 + t * h * 4
        flops = 2.0 * ns * (2 * n_ff * h + h * n_ff)
        reps = max(20, args.steps // (2 if t <= 4 else 8))
        dec.bench_moe(names, px, pi, pw, t, k, py, 2000 if t <= 4 else 300, warmup=0)  # settle clocks, untimed
        samples = [dec.bench_moe(names, px, pi, pw, t, k, py, reps, warmup=10)[0] * 1e3 / reps for _ in range(ROUNDS)]
        us = sorted(samples)[len(samples) // 2]
        out.append({"T": t, "experts_hit": hit, "us_per_ffn": round(us, 2), "us_spread": spread(samples, 1.0, 2),
                    "GBps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                    "TFLOPs": round(flops / us / 1e6, 1), "mfma_frac": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4)})
        for p_ in (lg, px, pi, pw, py):
            cc.free(p_)
    return out


def bench_chain(dec, gen, ops, args):
    """64 dense decoder layers of linears at M = 4 (QKV 5120->7168, O 5120->5120, gate+up 5120->34816, down
    17408->5120, group 128) with the RMS-rescale / SiLU*up glue, independent device-generated weights (10.9 GB).
    Two statements of the same chain are timed, eager and as graph replays: w4a16_chain_forward (seven launches per
    layer: every activation is normalised in f32 by a launch of its own before it is rounded to f16) and
    w4a16_chain_forward_fused (four launches per layer: the normalisations deferred across the linears, hand-overs with
    power-of-two factors).  A variant counts only if its output is finite, of unit mean square and the same bits from
    graph replays as from eager passes; the configuration's figure is the faster valid one."""
    cc = dec.cc
    layers, hidden, n_qkv, n_ff, g, t = 64, 5120, 7168, 17408, 128, 4
    dec.upload_chain_synth("c4", layers, hidden, n_qkv, n_ff, g)
    shapes = {"attn_qkv": (n_qkv, hidden), "attn_output": (hidden, hidden), "ffn_gate_up": (2 * n_ff, hidden),
              "ffn_down": (hidden, n_ff)}
    for l in range(layers):
        for role in ops.W4a16Dec.CHAIN_ROLES:
            dec.row_norm_max("c4.%d.%s" % (l, role))  # needs nothing but the tiled copy; kept with the linear
            dec.drop_raw("c4.%d.%s" % (l, role))
    px, py = cc.to_device(gen.normal_f16(404, (t, hidden))), cc.alloc(t * hidden * 2)
    reps = max(3, args.steps // 80)
    total = sum(algorithmic_bytes(t, kk, nn, g) for (nn, kk) in shapes.values()) * layers

    def variant(fused):
        def timed(use_graph):
            return [dec.bench_chain("c4", layers, px, t, py, reps, warmup=1, use_graph=use_graph, fused=fused)[0] / reps
                    for _ in range(ROUNDS)]
        eager = timed(False)
        y_eager = cc.d2h(py, (t, hidden), np.uint16)
        v = gen.f16_bits_to_f32(y_eager).astype(np.float64)
        finite = bool(np.all(np.isfinite(v)))
        unit_ms = bool(finite and np.allclose(np.mean(v * v, axis=1), 1.0, atol=2e-3))
        if args.no_graph:  # eager passes only (a tracer that cannot follow graph replays)
            graph, same = eager, None
        else:
            graph = timed(True)
            same = bool(np.array_equal(cc.d2h(py, (t, hidden), np.uint16), y_eager))
        best = min(sorted(eager)[ROUNDS // 2], sorted(graph)[ROUNDS // 2])
        return {"launches_per_layer": 4 if fused else 7, "ms_per_pass_eager": spread(eager, 1.0, 4),
                "ms_per_pass_graph": spread(graph, 1.0, 4), "ms_per_pass": round(best, 4),
                "output_finite": finite, "output_unit_mean_square": unit_ms, "graph_equals_eager_bits": same,
                "valid": bool(finite and unit_ms and same is not False)}

    kept, deferred = variant(False), variant(True)
    valid = [v for v in (kept, deferred) if v["valid"]]
    if not valid:
        raise RuntimeError("chain: no valid variant: %r / %r" % (kept, deferred))
    fig = min(valid, key=lambda v: v["ms_per_pass"])
    best = fig["ms_per_pass"]
    per_gemm = []
    xw, yw = cc.alloc(t * n_ff * 2), cc.alloc(t * 2 * n_ff * 4)
    cc.memset0(xw, t * n_ff * 2)
    for role in ops.W4a16Dec.CHAIN_ROLES:
        nn, kk = shapes[role]
        names = ["c4.%d.%s" % (l, role) for l in range(layers)]
        ms, samples, _ = time_rounds(dec, names, xw, yw, t, 256, 64, ops.PATH_AUTO, out_f16=False)
        b = algorithmic_bytes(t, kk, nn, g) + 2 * t * nn  # f32 output
        per_gemm.append({"linear": role, "K": kk, "N": nn, "us": round(ms * 1e3, 2), "us_spread": spread(samples, 1e3, 2),
                         "GBps": round(b / (ms * 1e-3) / 1e9, 1)})
    for p_ in (px, py, xw, yw):
        cc.free(p_)
    # the same layers in the prefill regime (reference: chain_t_sel / forward_prefill, w4a16_dec/prefill.rs:81-207):
    # 8 layers at M = 1024, the chain with its normalisation launches (gate|up carries SiLU*up in its epilogue) and
    # the chain with the normalisations deferred across the MFMA-tiled linears
    tp, lp = 1024, 8
    pxp, pyp = cc.to_device(gen.normal_f16(405, (tp, hidden))), cc.alloc(tp * hidden * 2)
    prefill_chain = {"layers": lp, "M": tp}
    for fused in (False, True):
        smp = [dec.bench_chain("c4", lp, pxp, tp, pyp, 3, warmup=1, use_graph=False, fused=fused)[0] / 3 for _ in range(ROUNDS)]
        vv = gen.f16_bits_to_f32(cc.d2h(pyp, (tp, hidden), np.uint16)).astype(np.float64)
        ok = bool(np.all(np.isfinite(vv)) and np.allclose(np.mean(vv * vv, axis=1), 1.0, atol=2e-3))
        prefill_chain["normalisations_deferred" if fused else "normalisation_launches_kept"] = {
            "ms_per_layer": round(sorted(smp)[ROUNDS // 2] / lp, 4), "ms_per_pass": spread(smp, 1.0, 4),
            "output_finite_unit_mean_square": ok}
    flops_layer = 2.0 * tp * sum(nn * kk for (nn, kk) in shapes.values())
    best_layer = min(v["ms_per_layer"] for v in prefill_chain.values() if isinstance(v, dict) and v["output_finite_unit_mean_square"])
    prefill_chain["TFLOPs_end_to_end"] = round(flops_layer / (best_layer * 1e-3) / 1e12, 1)
    cc.free(pxp)
    cc.free(pyp)
    return {"layers": layers, "M": t, "launches_per_layer": fig["launches_per_layer"], "ms_per_pass": best,
            "prefill_regime": prefill_chain,
            "us_per_token": round(best * 1e3 / t, 2), "GBps_end_to_end": round(total / (best * 1e-3) / 1e9, 1),
            "hbm_frac_end_to_end": round(total / (best * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "normalisation_launches_kept": kept, "normalisations_deferred": deferred, "per_gemm": per_gemm}


PLAN_SWEEP_SHAPES = [(34816, 5120), (5120, 17408)]
PLAN_SWEEP_T = (512, 1024, 4096)


def plan_sweep(out_path):
    """Times every (block tile, k slices) the prefill planner can choose at the layer shapes of the benchmark and writes
    the table the planner test reads (profiles/prefill_plan_sweep.md): per shape every candidate's time, the fastest, and
    what the planner picks with everything automatic."""
    from llm170_amd import gen, ops
    from llm170_amd import build as pkg_build
    pkg_build.ensure_built()
    dec = ops.W4a16Dec()
    cc = dec.cc
    g = 128
    lines = ["# Prefill launch plans: every (tile, k slices) timed at the layer shapes", "",
             "Command: `python bench.py --plan-sweep profiles/prefill_plan_sweep.md` (one MI355X; source hash %s)." % pkg_build.built_hash(),
             "Each entry: best of 3 timed regions of 12 launches after 3 warm-up launches, HIP events on the launch stream,",
             "f16 output, two to four weight copies rotated.  `plan` marks what `w4a16_plan_prefill` picks with every",
             "setting automatic; `best` the fastest row of the shape.  tests/test_plan_cpu.py requires the planner's",
             "pick to be a row within 3 % of the best: the same plan's time moves by 2-3 % from one box to the next",
             "(5120 x 17408 at t = 4096: 64 rows unsplit / 128 rows in two slices measured 622 / 626 us on the box the",
             "constants were fitted on and 621 / 606 us on another), so closer rows trade places between sweeps.", "",
             "| n | k | t | tile rows | k slices | us | note |", "|---|---|---|---|---|---|---|"]
    for (n, k) in PLAN_SWEEP_SHAPES:
        names, _ = make_copies(dec, gen, n, k, g, 2 if n > 8192 else 4, "ps%d_%d" % (n, k))
        xd = cc.to_device(gen.normal_f16(3, (max(PLAN_SWEEP_T), k)))
        yd = cc.alloc(max(PLAN_SWEEP_T) * n * 2)
        time_forward(dec, names, xd, yd, max(PLAN_SWEEP_T), 30, 0, ops.PATH_PREFILL)
        for t in PLAN_SWEEP_T:
            rows = []
            for tile in (64, 96, 128):
                for ks in (1, 2, 3, 4, 6, 8):
                    if ks > 1 and ks > (k // 128) // 4:
                        continue
                    dec.set_prefill_tile(tile)
                    dec.set_prefill_ksplit(-1 if ks == 1 else ks)
                    us = min(time_forward(dec, names, xd, yd, t, 12, 3, ops.PATH_PREFILL, out_f16=True)[0] for _ in range(3)) * 1e3
                    rows.append((tile, ks, us))
            dec.set_prefill_tile(0)
            dec.set_prefill_ksplit(0)
            plan = ops.plan_prefill(t, n, k, cu_count=256)
            best = min(r[2] for r in rows)
            for tile, ks, us in rows:
                note = " ".join(w for w, on in (("best", us == best), ("plan", (tile, ks) == (plan["tile_rows"], plan["k_slices"]))) if on)
                lines.append("| %d | %d | %d | %d | %d | %.2f | %s |" % (n, k, t, tile, ks, us, note))
            print("plan sweep", n, k, t, "best %.2f us" % best, "plan", plan["tile_rows"], plan["k_slices"], flush=True)
        cc.free(xd)
        cc.free(yd)
    with open(out_path, "w") as fh:
        fh.write("\n".join(lines) + "\n")
    cc.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--copies", type=int, default=8, help="distinct weight copies rotated through (cold HBM)")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="time the layer chain with eager launches only")
    ap.add_argument("--plan-sweep", metavar="PATH", help="time every prefill launch plan at the layer shapes and write the table to PATH, nothing else")
    ap.add_argument("--prefill-down-only", action="store_true",
                    help="only the calibration copy and the M=4096 prefill of the down projection (K=17408, N=5120): the "
                         "leg a counter run needs to attribute traffic to that launch alone")
    args = ap.parse_args()
    if args.plan_sweep:
        plan_sweep(args.plan_sweep)
        return
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the W4A16 linear path has no collective); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from llm170_amd import gen, ops, parity
    from llm170_amd import build as pkg_build
    pkg_build.ensure_built()
    dec = ops.W4a16Dec()
    cc = dec.cc
    load_probes(cc)

    # profiler calibration: one plain copy of exactly 256 MiB read + 256 MiB written
    import ctypes as C
    cal_bytes = 256 << 20
    ca, cb = cc.alloc(cal_bytes), cc.alloc(cal_bytes)
    cc.memset0(ca, cal_bytes)
    cc.launch("w4a16_copy_u4", 4096, 1, 256, [C.c_uint64(ca), C.c_uint64(cb), C.c_size_t(cal_bytes // 16)])
    cc.sync()
    cc.free(ca)
    cc.free(cb)

    if args.prefill_down_only:
        k2, n2, g, mp = 17408, 5120, 128, 4096
        names2, _ = make_copies(dec, gen, n2, k2, g, 4, "down")
        xp2 = cc.to_device(gen.normal_f16(gen.shape_seed(n2, k2, tensor=4), (mp, k2)))
        yp2 = cc.alloc(mp * n2 * 2)
        psteps = max(10, args.steps // 8)
        time_forward(dec, names2, xp2, yp2, mp, 40, 0, ops.PATH_PREFILL)
        ms_m, smp, _ = time_rounds(dec, names2, xp2, yp2, mp, psteps, 5, ops.PATH_PREFILL)
        tf = 2.0 * mp * n2 * k2 / (ms_m * 1e-3) / 1e12
        print(json.dumps({"workload": "prefill GEMM M=4096 K=17408 N=5120 g128", "ms_per_launch": round(ms_m, 4),
                          "ms_spread": spread(smp, 1.0, 4), "TFLOPs": round(tf, 1), "mfma_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                          "kernel": cc.last_launch_symbol(), "source_hash": pkg_build.built_hash()}))
        return

    # ---------------------------------------------------------------- headline: decode GEMV, M=1, gate+up
    m, k, n, g = 1, 5120, 34816, 128
    names, (q0, s0) = make_copies(dec, gen, n, k, g, args.copies, "gate_up")
    x = gen.normal_f16(gen.shape_seed(n, k, tensor=3), (16, k))
    xd = cc.to_device(x)
    yd = cc.alloc(16 * n * 4)

    # the card's clocks take tens of milliseconds of load to settle: an untimed run of the same launches first, so the
    # W warm-up and K timed steps below see the steady state.  The step time reported is the median of ROUNDS timed
    # regions of exactly K steps each (W untimed steps before each); min and max are in `extra`.
    time_forward(dec, names, xd, yd, m, 3000, 0, ops.PATH_DECODE)
    ms_step, step_samples, wall_step = time_rounds(dec, names, xd, yd, m, args.steps, args.warmup, ops.PATH_DECODE)
    decode_kernel = cc.last_launch_symbol()
    nbytes = algorithmic_bytes(m, k, n, g)
    gbps = nbytes / (ms_step * 1e-3) / 1e9
    warm_ms, _, _ = time_rounds(dec, names[:1], xd, yd, m, args.steps, args.warmup, ops.PATH_DECODE)

    # parity of what was just timed, against the CPU oracle (checker only), with the compensated f64 dot beside it
    from oracle import oracle
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    y16 = dec.gemv_host(names[0], x[:1], t=1, out_f16=True, path=ops.PATH_DECODE)
    y32 = dec.gemv_host(names[0], x[:1], t=1, path=ops.PATH_DECODE)
    y_ref = oracle.gemm_lane(x[:1], 1, q0, s0, n, k, g, threads=cores)
    par = parity.assert_close(gen.f16_bits_to_f32(y16), gen.f16_bits_to_f32(gen.f32_to_f16_bits(y_ref)), "headline f16 out")
    par_f32 = parity.assert_close(y32, y_ref, "headline f32 out")
    all_rows = np.arange(n, dtype=np.uint32)
    ev = parity.exact_evidence(y32[0], y_ref[0], oracle.exact_dot_sample(x, q0, s0, k, g, all_rows, np.zeros(n, np.uint32)))
    if not ev["ok"]:
        raise RuntimeError("headline: the kernel is further from the exact dot than the reference allows: %r" % (ev,))

    cpu = None
    if not args.no_cpu:
        reps, t_cpu = 0, 0.0
        t_begin = time.perf_counter()
        while t_cpu < 2.0 and reps < 64:  # ~2 s wall on all cores = tens of core-seconds of scalar work
            oracle.gemm_lane(x[:1], 1, q0, s0, n, k, g, threads=cores)
            reps += 1
            t_cpu = time.perf_counter() - t_begin
        cpu = {"value": round(nbytes * reps / t_cpu / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": "%d full passes of the same M=1 K=5120 N=34816 GEMV (all %d rows), rows split over %d "
                         "threads, %.2f s wall" % (reps, n, cores, t_cpu)}

    keys = ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "strict_fail", "clamped")
    extra = {"source_hash": pkg_build.built_hash(),
             "ms_per_step_spread": spread(step_samples, 1.0, 6),
             "warm_single_copy_GBps": round(nbytes / (warm_ms * 1e-3) / 1e9, 1),
             "weight_only_GBps": round((n * k / 2) / (ms_step * 1e-3) / 1e9, 1),
             "wall_ms_per_step": round(wall_step, 5),
             "parity_f16_out": {a: par[a] for a in keys},
             "parity_f32_out": {a: par_f32[a] for a in keys},
             "parity_vs_exact_f64_dot": {a: ev[a] for a in ("kernel_rms_err", "lane_rms_err", "kernel_max_err", "lane_max_err",
                                                            "kernel_max_strict_ulp", "lane_max_strict_ulp",
                                                            "kernel_beyond_4ulp", "lane_beyond_4ulp")},
             "peaks": {"hbm_GBps": HBM_PEAK_GBPS, "mfma_f16_TFLOPs": MFMA_F16_PEAK_TFLOPS}}
    if not args.no_extra:
        extra["chip_probes"] = chip_probes(cc, nbytes, args.copies)

    # ---------------------------------------------------------------- prefill GEMM, M=4096 (second half of the metric)
    mp = 4096
    xp = gen.normal_f16(gen.shape_seed(n, k, tensor=4), (mp, k))
    xpd = cc.to_device(xp)
    ypd = cc.alloc(mp * n * 2)
    psteps = max(10, args.steps // 8)
    time_forward(dec, names, xpd, ypd, mp, 40, 0, ops.PATH_PREFILL)  # settle clocks, untimed
    pf_ms, pf_samples, _ = time_rounds(dec, names, xpd, ypd, mp, psteps, 5, ops.PATH_PREFILL)
    prefill_kernel = cc.last_launch_symbol()
    pf_flops = 2.0 * mp * n * k
    pf_tf = pf_flops / (pf_ms * 1e-3) / 1e12
    # parity of the prefill result: a seeded sample of outputs against the CPU oracle
    rows = (gen.stream(11, 2048) % np.uint64(n)).astype(np.uint32)
    toks = (gen.stream(12, 2048) % np.uint64(mp)).astype(np.uint32)
    dec.lin_forward(names[0], xpd, ypd, mp, out_f16=True, path=ops.PATH_PREFILL)
    yp = cc.d2h(ypd, (mp, n), np.uint16)
    ref_s = oracle.gemm_lane_sample(xp, q0, s0, k, g, rows, toks)
    par_pf = parity.assert_close(gen.f16_bits_to_f32(yp[toks, rows]), gen.f16_bits_to_f32(gen.f32_to_f16_bits(ref_s)),
                                 "prefill f16 out, sample")
    extra["parity_prefill_f16_sample2048"] = {a: par_pf[a] for a in keys}
    extra["prefill_ms_spread"] = spread(pf_samples, 1.0, 4)
    if not args.no_extra:
        # every one of the 4096 x 34816 outputs of the launch just timed against the bit-exact device twin of the lane
        # order (itself pinned to the CPU oracle on the sample above): the full-shape strict-failure count
        ytw = cc.alloc(mp * n * 4)
        dec.upload_lin_g("gate_up.twin", q0, s0, n, k, g, False)  # the timed copies dropped their as-given operands
        dec.lin_forward("gate_up.twin", xpd, ytw, mp, out_f16=False, path=ops.PATH_LANE)
        twin = cc.d2h(ytw, (mp, n), np.float32)
        cc.free(ytw)
        if not np.array_equal(twin[toks, rows].view(np.uint32), ref_s.view(np.uint32)):
            raise RuntimeError("prefill: the device twin of the lane order differs from the CPU oracle on the sample")
        par_full = parity.assert_close(gen.f16_bits_to_f32(yp), gen.f16_bits_to_f32(gen.f32_to_f16_bits(twin)),
                                       "prefill f16 out, all outputs against the device twin")
        extra["parity_prefill_f16_full_vs_device_twin"] = dict({a: par_full[a] for a in keys}, outputs=int(mp) * int(n))
        del twin
        # the same GEMM with the SiLU*up epilogue (f16 [M][N/2] out): what the prefill chain runs for gate|up
        yg = cc.alloc(mp * (n // 2) * 2)
        e0, e1 = cc.event(), cc.event()
        glu_samples = []
        for r in range(ROUNDS):
            for i in range(5):
                dec.lin_forward_glu(names[i % len(names)], xpd, yg, mp)
            e0.record()
            for i in range(psteps):
                dec.lin_forward_glu(names[(5 + i) % len(names)], xpd, yg, mp)
            e1.record()
            cc.sync()
            glu_samples.append(e0.elapsed_ms(e1) / psteps)
        glu_kernel = cc.last_launch_symbol()
        glu_ms = sorted(glu_samples)[ROUNDS // 2]
        # same bits as the plain launch followed by the element-wise kernel (checked on the first copy)
        y32 = cc.alloc(mp * n * 4)
        ya = cc.alloc(mp * (n // 2) * 2)
        dec.lin_forward(names[0], xpd, y32, mp, out_f16=False, path=ops.PATH_PREFILL)
        dec.silu_mul_f16(y32, n // 2, mp, ya)
        dec.lin_forward_glu(names[0], xpd, yg, mp)
        glu_same = bool(np.array_equal(cc.d2h(ya, (mp, n // 2), np.uint16), cc.d2h(yg, (mp, n // 2), np.uint16)))
        if not glu_same:
            raise RuntimeError("prefill: the gated launch differs from linear + silu_mul")
        # what the fusion replaces: the element-wise launch over the f32 [M][N] intermediate
        ew_samples = []
        for r in range(ROUNDS):
            e0.record()
            for i in range(psteps):
                dec.silu_mul_f16(y32, n // 2, mp, ya)
            e1.record()
            cc.sync()
            ew_samples.append(e0.elapsed_ms(e1) / psteps)
        ew_ms = sorted(ew_samples)[ROUNDS // 2]
        for p_ in (y32, ya, yg):
            cc.free(p_)
        glu_tf = pf_flops / (glu_ms * 1e-3) / 1e12
        extra["prefill_gate_up_silu_fused"] = {
            "workload": "prefill GEMM M=4096 K=5120 N=34816 g128 with SiLU*up in the epilogue, f16 [M][N/2] out",
            "ms": round(glu_ms, 4), "ms_spread": spread(glu_samples, 1.0, 4), "TFLOPs": round(glu_tf, 1),
            "mfma_frac": round(glu_tf / MFMA_F16_PEAK_TFLOPS, 4), "kernel": glu_kernel,
            "equals_linear_then_silu_mul_bits": glu_same,
            "plain_launch_ms": round(pf_ms, 4), "separate_silu_mul_launch_ms": round(ew_ms, 4),
            "two_launch_sequence_ms": round(pf_ms + ew_ms, 4)}
    cc.free(xpd)
    cc.free(ypd)

    if not args.no_extra:
        table = []
        settle = 1500  # untimed launches before every table entry, as for the headline (the prefill leg in between
                       # leaves the card in another clock state)

        def decode_row(nm, xdev, mm, kk, nn, shape):
            time_forward(dec, nm, xdev, yd, mm, settle, 0, ops.PATH_DECODE)
            ms_m, smp, _ = time_rounds(dec, nm, xdev, yd, mm, args.steps, args.warmup, ops.PATH_DECODE)
            b = algorithmic_bytes(mm, kk, nn, g)
            return {"shape": shape, "M": mm, "us": round(ms_m * 1e3, 2), "us_spread": spread(smp, 1e3, 2),
                    "GBps": round(b / (ms_m * 1e-3) / 1e9, 1), "hbm_frac": round(b / (ms_m * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "kernel": cc.last_launch_symbol()}

        for mm in (4, 16):
            table.append(decode_row(names, xd, mm, k, n, "gate_up K5120 N34816 g128"))
        k2, n2 = 17408, 5120
        names2, _ = make_copies(dec, gen, n2, k2, g, args.copies * 2, "down")
        x2d = cc.to_device(gen.normal_f16(gen.shape_seed(n2, k2, tensor=3), (16, k2)))
        for mm in (1, 4, 16):
            table.append(decode_row(names2, x2d, mm, k2, n2, "down K17408 N5120 g128"))
        extra["decode_table"] = table
        ptable = []
        xp2 = cc.to_device(gen.normal_f16(gen.shape_seed(n2, k2, tensor=4), (mp, k2)))
        yp2 = cc.alloc(mp * max(n, n2) * 2)
        xp1 = cc.to_device(xp)
        for (nm, kk, nn, xdev, shape) in ((names, k, n, xp1, "gate_up K5120 N34816 g128"),
                                          (names2, k2, n2, xp2, "down K17408 N5120 g128")):
            for mm in (512, 1024, 4096):
                time_forward(dec, nm, xdev, yp2, mm, 20, 0, ops.PATH_PREFILL)
                ms_m, smp, _ = time_rounds(dec, nm, xdev, yp2, mm, psteps, 5, ops.PATH_PREFILL)
                tf = 2.0 * mm * nn * kk / (ms_m * 1e-3) / 1e12
                ptable.append({"shape": shape, "M": mm, "ms": round(ms_m, 4), "ms_spread": spread(smp, 1.0, 4),
                               "TFLOPs": round(tf, 1), "mfma_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                               "kernel": cc.last_launch_symbol()})
        extra["prefill_table"] = ptable
        down4096 = [r for r in ptable if r["shape"].startswith("down") and r["M"] == 4096][0]
        for p_ in (xp2, yp2, xp1, x2d):
            cc.free(p_)
        extra["moe_table"] = bench_moe(dec, gen, ops, args)
        extra["chain"] = bench_chain(dec, gen, ops, args)

    traffic, traffic_src = measured_traffic(decode_kernel)
    pf_traffic, pf_traffic_src = measured_traffic(prefill_kernel)
    line = {
        "metric": "W4A16 GEMM: decode GB/s (M=1) & prefill TFLOP/s (M=4096) vs MI355X peak",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int4 weights x f16 activations, f32 accumulate, f16 out",
        "data": "synthetic (SplitMix64-seeded: int4 uniform -8..7, f16 scales U[0.002,0.02), f16 N(0,1) x)",
        "config": {"workload": "decode GEMV M=1 K=5120 N=34816 g128 (27B dense gate+up), cold HBM: %d weight copies "
                               "rotated; median of %d timed regions of %d steps" % (args.copies, ROUNDS, args.steps),
                   "M": m, "K": k, "N": n, "group": g},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_src,
                     "kernel": decode_kernel, "algorithmic_bytes_per_launch": nbytes},
        "roofline_prefill": {"bound": "mfma", "achieved": round(pf_tf, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                             "unit": "TFLOP/s", "frac": round(pf_tf / MFMA_F16_PEAK_TFLOPS, 4),
                             "traffic": pf_traffic, "traffic_source": pf_traffic_src,
                             "kernel": prefill_kernel, "workload": "prefill GEMM M=4096 K=5120 N=34816 g128",
                             "ms_per_launch": round(pf_ms, 4), "algorithmic_flops_per_launch": pf_flops},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    if not args.no_extra:
        pf2_traffic, pf2_src = measured_traffic(down4096["kernel"])
        line["roofline_prefill_down"] = {
            "bound": "mfma", "achieved": down4096["TFLOPs"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": down4096["mfma_frac"], "traffic": pf2_traffic, "traffic_source": pf2_src, "kernel": down4096["kernel"],
            "workload": "prefill GEMM M=4096 K=17408 N=5120 g128", "ms_per_launch": down4096["ms"],
            "algorithmic_flops_per_launch": 2.0 * 4096 * 5120 * 17408}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
