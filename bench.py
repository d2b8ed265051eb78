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
        q = gen.weights_q(gen.shape_seed(n, k, tensor=1) + 977 * c, n, k)
        s = gen.scales_f16(gen.shape_seed(n, k, tensor=2) + 977 * c, n, k, g)
        name = "%s.%d" % (prefix, c)
        dec.upload_lin_g(name, q, s, n, k, g, False)
        dec.drop_raw(name)
        names.append(name)
        if c == 0:
            first = (q, s)
    return names, first


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by the plain-copy
    calibration), as recorded in the committed summary profiles/pmc_traffic.txt; None if no record."""
    path = os.path.join(ROOT, "profiles", "pmc_traffic.txt")
    if not os.path.exists(path):
        return None
    for ln in open(path):
        f = ln.split()
        if len(f) >= 3 and f[0] == kernel and f[1] == "traffic_bytes_per_launch":
            return int(float(f[2]))
    return None


def time_forward(dec, names, xd, yd, t, steps, warmup, path, out_f16=True):
    ms, wall = dec.bench_forward(names, xd, yd, t, steps, warmup=warmup, out_f16=out_f16, path=path)
    return ms / steps, wall / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--copies", type=int, default=8, help="distinct weight copies rotated through (cold HBM)")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the W4A16 linear path has no collective); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from llm170_amd import gen, ops
    dec = ops.W4a16Dec()
    cc = dec.cc

    # profiler calibration: one plain copy of exactly 256 MiB read + 256 MiB written
    import ctypes as C
    cal_bytes = 256 << 20
    ca, cb = cc.alloc(cal_bytes), cc.alloc(cal_bytes)
    cc.memset0(ca, cal_bytes)
    cc.launch("w4a16_copy_u4", 4096, 1, 256, [C.c_uint64(ca), C.c_uint64(cb), C.c_size_t(cal_bytes // 16)])
    cc.sync()
    cc.free(ca)
    cc.free(cb)

    # ---------------------------------------------------------------- headline: decode GEMV, M=1, gate+up
    m, k, n, g = 1, 5120, 34816, 128
    names, (q0, s0) = make_copies(dec, gen, n, k, g, args.copies, "gate_up")
    x = gen.normal_f16(gen.shape_seed(n, k, tensor=3), (16, k))
    xd = cc.to_device(x)
    yd = cc.alloc(16 * n * 4)

    ms_step, wall_step = time_forward(dec, names, xd, yd, m, args.steps, args.warmup, ops.PATH_DECODE)
    nbytes = algorithmic_bytes(m, k, n, g)
    gbps = nbytes / (ms_step * 1e-3) / 1e9
    warm_ms, _ = time_forward(dec, names[:1], xd, yd, m, args.steps, args.warmup, ops.PATH_DECODE)

    # parity of what was just timed, against the CPU oracle (checker only)
    from oracle import oracle
    from tests import parity
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    y16 = dec.gemv_host(names[0], x[:1], t=1, out_f16=True, path=ops.PATH_DECODE)
    t0 = time.perf_counter()
    y_ref = oracle.gemm_lane(x[:1], 1, q0, s0, n, k, g, threads=cores)
    par = parity.compare(gen.f16_bits_to_f32(y16), gen.f16_bits_to_f32(gen.f32_to_f16_bits(y_ref)))
    par_f32 = parity.compare(dec.gemv_host(names[0], x[:1], t=1, path=ops.PATH_DECODE), y_ref)

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

    extra = {"warm_single_copy_GBps": round(nbytes / (warm_ms * 1e-3) / 1e9, 1),
             "weight_only_GBps": round((n * k / 2) / (ms_step * 1e-3) / 1e9, 1),
             "wall_ms_per_step": round(wall_step, 5),
             "parity_f16_out": {a: par[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")},
             "parity_f32_out": {a: par_f32[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")},
             "peaks": {"hbm_GBps": HBM_PEAK_GBPS, "mfma_f16_TFLOPs": MFMA_F16_PEAK_TFLOPS}}

    # ---------------------------------------------------------------- prefill GEMM, M=4096 (second half of the metric)
    mp = 4096
    xp = gen.normal_f16(gen.shape_seed(n, k, tensor=4), (mp, k))
    xpd = cc.to_device(xp)
    ypd = cc.alloc(mp * n * 2)
    psteps = max(5, args.steps // 20)
    pf_ms, _ = time_forward(dec, names, xpd, ypd, mp, psteps, 3, ops.PATH_PREFILL)
    pf_flops = 2.0 * mp * n * k
    pf_tf = pf_flops / (pf_ms * 1e-3) / 1e12
    # parity of the prefill result: a seeded sample of outputs against the CPU oracle
    rows = (gen.stream(11, 2048) % np.uint64(n)).astype(np.uint32)
    toks = (gen.stream(12, 2048) % np.uint64(mp)).astype(np.uint32)
    dec.lin_forward(names[0], xpd, ypd, mp, out_f16=True, path=ops.PATH_PREFILL)
    yp = cc.d2h(ypd, (mp, n), np.uint16)
    ref_s = oracle.gemm_lane_sample(xp, q0, s0, k, g, rows, toks)
    par_pf = parity.compare(gen.f16_bits_to_f32(yp[toks, rows]), gen.f16_bits_to_f32(gen.f32_to_f16_bits(ref_s)))
    cc.free(xpd)
    cc.free(ypd)
    extra["parity_prefill_f16_sample2048"] = {a: par_pf[a] for a in ("rel_l2", "max_ulp", "max_ulp_strict", "strict_pass_frac", "clamped")}

    if not args.no_extra:
        table = []
        for mm in (4, 16):
            ms_m, _ = time_forward(dec, names, xd, yd, mm, args.steps, args.warmup, ops.PATH_DECODE)
            b = algorithmic_bytes(mm, k, n, g)
            table.append({"shape": "gate_up K5120 N34816 g128", "M": mm, "us": round(ms_m * 1e3, 2),
                          "GBps": round(b / (ms_m * 1e-3) / 1e9, 1), "hbm_frac": round(b / (ms_m * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        k2, n2 = 17408, 5120
        names2, _ = make_copies(dec, gen, n2, k2, g, args.copies * 2, "down")
        x2d = cc.to_device(gen.normal_f16(gen.shape_seed(n2, k2, tensor=3), (16, k2)))
        for mm in (1, 4, 16):
            ms_m, _ = time_forward(dec, names2, x2d, yd, mm, args.steps, args.warmup, ops.PATH_DECODE)
            b = algorithmic_bytes(mm, k2, n2, g)
            table.append({"shape": "down K17408 N5120 g128", "M": mm, "us": round(ms_m * 1e3, 2),
                          "GBps": round(b / (ms_m * 1e-3) / 1e9, 1), "hbm_frac": round(b / (ms_m * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        extra["decode_table"] = table
        ptable = []
        xp2 = cc.to_device(gen.normal_f16(gen.shape_seed(n2, k2, tensor=4), (mp, k2)))
        yp2 = cc.alloc(mp * max(n, n2) * 2)
        xp1 = cc.to_device(xp)
        for (nm, kk, nn, xdev, shape) in ((names, k, n, xp1, "gate_up K5120 N34816 g128"),
                                          (names2, k2, n2, xp2, "down K17408 N5120 g128")):
            for mm in (512, 1024, 4096):
                ms_m, _ = time_forward(dec, nm, xdev, yp2, mm, psteps, 3, ops.PATH_PREFILL)
                tf = 2.0 * mm * nn * kk / (ms_m * 1e-3) / 1e12
                ptable.append({"shape": shape, "M": mm, "ms": round(ms_m, 4), "TFLOPs": round(tf, 1),
                               "mfma_frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)})
        extra["prefill_table"] = ptable

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
                               "rotated" % args.copies, "M": m, "K": k, "N": n, "group": g},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": measured_traffic("w4a16_decode_g128_f16_rb2_x1"),
                     "kernel": "w4a16_decode_g128_f16_rb2_x1", "algorithmic_bytes_per_launch": nbytes},
        "roofline_prefill": {"bound": "mfma", "achieved": round(pf_tf, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                             "unit": "TFLOP/s", "frac": round(pf_tf / MFMA_F16_PEAK_TFLOPS, 4),
                             "traffic": measured_traffic("w4a16_prefill_g128_f16"),
                             "kernel": "w4a16_prefill_g128_f16", "workload": "prefill GEMM M=4096 K=5120 N=34816 g128",
                             "ms_per_launch": round(pf_ms, 4), "algorithmic_flops_per_launch": pf_flops},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
