#!/usr/bin/env python3
"""Benchmark of the BCQ LUT matvec on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg1]

Default (cfg1, the headline): a step is one matvec of m=1, k=n=12288, q=3, g=128, fp16
activations, no offset, with the packed weight already resident in HBM.  Consecutive steps use
different weight copies (R copies, R * packed bytes > 4 x the 256 MiB last-level cache), so every
step streams its weight from HBM and not from cache.  The K timed steps are issued back to back,
ONE KERNEL LAUNCH PER MATVEC (the protocol of the reference's own caller, a loop of lutGEMM::matmul
calls, tests/opt/fp16/int3_col_wise_matmul_fp16.cu:120-133), and bracketed by HIP events on the
launch stream: that is `value`, `ms_per_step` and `roofline.frac`.  The same steps as independent
matvecs sharing launches (lutgemm_matvec_many) are reported beside it (`fused_independent`, and
`roofline.frac_fused_independent`).

Prints ONE JSON line: value = packed-weight GB/s (higher is better), plus us per matvec, the
roofline block for the matvec kernel, the dense fp16 GEMV comparator, the single-copy ("hot")
figure and the CPU baseline (the reference's CPU path restated in oracle/, timed on this box's
host cores: the whole cfg0 matvec and a bounded slice of cfg1).

Other workloads, same protocol, one JSON line each (no CPU / dense legs):
  --config cfg0 | cfg2        single shapes
  --config cfg3               k=n=7168, q in 1..4 x g in {32,64,128,k}: 16 points
  --config cfg4 [--m M] [--graph]
                              q=2 g=128 decoder layer: QKV, out, FC1, FC2 matvecs back to back,
                              m activation rows; --graph replays the chain from a captured HIP graph
  --config dequant            dense fp16 weight from the packed tiles (lutgemm_dequantize), both
                              orientations, cfg1 and cfg2 weights
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "lut-gemm_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
LLC_BYTES = 256 << 20  # last-level (memory-side) cache
METRIC = "µs/matvec + weight-GB/s (% HBM peak), n=k=12288 q=3 g=128 m=1 fp16"
# HBM bytes per launch of lut_matvec_kernel<3,false,1> on cfg1 with the launch plan 8 wavefronts x 5
# k-splits, from the rocprofv3 counter runs summarised in profiles/lut_matvec_kernel_cfg1.md
# (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 per dispatch, the factors a plain copy kernel of known
# size reads on the same counters): 64.01 MB read + 0.61 MB written.  Quoted only when the run
# uses that plan; any other launch shape reports null.
CFG1_PROFILED_PLAN = (8, 5)
CFG1_PROFILED_TRAFFIC_BYTES_PER_LAUNCH = 64.63e6


def event_time_ms(torch, fn, stream):
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record(stream)
    fn()
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop)


def cpu_matvec(oracle, w, x16, slice_n, omp):
    """dequantize_cpu then the fp32 triple-loop matmul (the reference's CPU path) on the first
    slice_n outputs; returns (seconds, y, threads)."""
    import numpy as np
    bW = np.ascontiguousarray(w["bW"][:, :, :slice_n])
    alpha = np.ascontiguousarray(w["alpha"].astype(np.float16)[:, :, :slice_n])
    t0 = time.perf_counter()
    if omp:
        fW, threads = oracle.dequantize_cpu_omp(bW, alpha)
        y, _ = oracle.matmul_cpu_omp(x16, fW)
    else:
        fW, threads = oracle.dequantize_cpu(bW, alpha), 1
        y = oracle.matmul_cpu(x16, fW)
    return time.perf_counter() - t0, y, int(threads)


def cpu_baseline(synth, cfg, x16, w, truth, slice_n=12288):
    """The reference's CPU path restated in oracle/, single-threaded as the reference is, on the
    first `slice_n` outputs of the cfg1 workload; then the same loops with OpenMP over the host
    cores; then the whole cfg0 matvec (the reference's CPU-runnable configuration) both ways."""
    import numpy as np
    from oracle import oracle
    k, n = cfg["k"], cfg["n"]
    serial_s, y, _ = cpu_matvec(oracle, w, x16, slice_n, omp=False)
    omp_s, _, threads = cpu_matvec(oracle, w, x16, slice_n, omp=True)
    scale = n / float(slice_n)
    b_w = (k * slice_n * cfg["q"] // 8) + (k // cfg["g"]) * cfg["q"] * slice_n * 2
    c0 = synth.CONFIGS["cfg0"]
    w0 = synth.make_weight(c0["k"], c0["n"], c0["q"], c0["g"], seed=0)
    x0 = synth.make_x(1, c0["k"], seed=0)
    b_w0, _ = synth.algorithmic_bytes(c0["k"], c0["n"], c0["q"], c0["g"], False, 1)
    s0, y0, _ = cpu_matvec(oracle, w0, x0, c0["n"], omp=False)
    o0, _, _ = cpu_matvec(oracle, w0, x0, c0["n"], omp=True)
    t0 = oracle.matvec_f64(w0["bW"], w0["alpha"].astype(np.float16), None, x0)
    return {
        "value": b_w / serial_s / 1e9,
        "unit": "GB/s (packed-weight bytes)",
        "cores": 1,
        "kind": "port",
        "sample": "cfg1 outputs 0..%d of %d (%.1f%% of one matvec): dequantize_cpu + matmul_cpu, %.2f s" % (
            slice_n - 1, n, 100.0 / scale, serial_s),
        "us_per_matvec_extrapolated": serial_s * scale * 1e6,
        "openmp": {"cores": threads, "value": b_w / omp_s / 1e9,
                   "us_per_matvec_extrapolated": omp_s * scale * 1e6},
        "max_abs_vs_truth": float(np.abs(y[0].astype(np.float64) - truth[0, :y.shape[1]]).max()),
        "cfg0_whole_matvec": {"us_per_matvec": s0 * 1e6, "value": b_w0 / s0 / 1e9,
                              "openmp_us_per_matvec": o0 * 1e6, "openmp_value": b_w0 / o0 / 1e9,
                              "max_abs_vs_truth": float(np.abs(y0.astype(np.float64) - t0).max())},
        "checksum": float(np.abs(y).sum()),
    }


PARITY_FAILURES = []   # filled by parity_record; a non-empty list makes the run exit with status 1


def parity_record(oracle, y16, truth, n_chk, label=""):
    """Error statistics of an fp16 result against the float64 truth, and the verdict of the
    path's tolerance (oracle.tolerance_violation); a violation is remembered for the exit status."""
    mean_abs, max_abs, rel_l2 = oracle.error_stats(y16, truth)
    bad = oracle.tolerance_violation(y16, truth)
    if bad is not None:
        PARITY_FAILURES.append("%s%s" % (label + ": " if label else "", bad))
    return {"truth": "fp64 accumulation over fp16-rounded inputs (oracle)", "outputs_checked": n_chk,
            "mean_abs": mean_abs, "max_abs": max_abs, "rel_l2": rel_l2,
            "tolerance": "|y-y*| <= %g ulp_fp16(|y*|) + %g and rel L2 <= %g" % (oracle.ULPS, oracle.ABS_TOL, oracle.REL_L2_TOL),
            "within_tolerance": bad is None, "violation": bad}


class Point:
    """One weight shape on the device: R rotating copies, an autotuned plan, buffers."""

    def __init__(self, lutgemm, synth, torch, dev, k, n, q, g, rtn, m, seed, stream_handle, copies=None,
                 rotation_bytes=4 * LLC_BYTES, plan=None):
        self.k, self.n, self.q, self.g, self.m = k, n, q, g, m
        self.w = synth.make_weight(k, n, q, g, rtn=rtn, seed=seed)
        self.has_offset = self.w["q_bias"] is not None
        self.b_w, self.b_total = synth.algorithmic_bytes(k, n, q, g, self.has_offset, m)
        if copies is None:
            copies = min(200, max(2, int(math.ceil(rotation_bytes / float(self.b_w))) + 1))
        self.copies = copies
        first = lutgemm.BCQWeight(self.w["bW"], self.w["alpha"], k, n, q, k // g, self.w["q_bias"])
        if plan:
            first.set_plan(plan[0], plan[1])
        else:
            first.autotune(stream_handle)  # measured once (untimed launches); clones keep the plan
        self.weights = [first] + [first.clone() for _ in range(copies - 1)]
        self.x16 = synth.make_x(m, k, seed=seed)
        self.xd = torch.from_numpy(self.x16).to(dev)
        self.yd = torch.zeros((copies, m, n), dtype=torch.float16, device=dev)
        self.plan = first.plan()
        self.plan_m = first.plan(m)

    def items(self, count, rotate=True, offset=0):
        out = []
        for i in range(count):
            c = ((i + offset) % self.copies) if rotate else 0
            out.append((self.weights[c], self.xd.data_ptr(), self.yd[c].data_ptr(), self.m))
        return out

    def parity(self, max_outputs=None):
        """Error statistics of copy 0's last output against the fp64 oracle (checker only)."""
        import numpy as np
        from oracle import oracle
        n_chk = self.n if max_outputs is None else min(self.n, max_outputs)
        z = self.w["q_bias"].astype(np.float16)[:, :n_chk] if self.has_offset else None
        truth = oracle.matvec_f64(np.ascontiguousarray(self.w["bW"][:, :, :n_chk]),
                                  np.ascontiguousarray(self.w["alpha"].astype(np.float16)[:, :, :n_chk]),
                                  np.ascontiguousarray(z) if z is not None else None, self.x16)
        y = self.yd[0].cpu().numpy()[:, :n_chk]
        return parity_record(oracle, y, truth, n_chk), truth

    def close(self):
        for wgt in self.weights:
            wgt.close()


PREWARM_MS = 100.0  # the device reaches its sustained clocks only after some tens of ms under load
BURSTS = 15         # the --steps burst is timed this many times back to back; the median is reported


def prewarm(torch, launch, min_ms=PREWARM_MS):
    """Keep the device busy with `launch` (a burst of the workload's own launches) for min_ms."""
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        launch()
        launch()
        torch.cuda.synchronize()


def time_bursts(torch, stream, launches):
    """Each callable in `launches` issues one burst; all bursts are issued back to back, each
    bracketed by HIP events on the launch stream.  Returns the burst times in ms."""
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in launches]
    for (e0, e1), fn in zip(ev, launches):
        e0.record(stream)
        fn()
        e1.record(stream)
    torch.cuda.synchronize()
    return [e0.elapsed_time(e1) for e0, e1 in ev]


def median(v):
    v = sorted(v)
    n = len(v)
    return v[n // 2] if n % 2 else 0.5 * (v[n // 2 - 1] + v[n // 2])


def time_point(lutgemm, torch, stream, pt, steps, warmup):
    """us per step with one launch per matvec (rotating copies and single copy): `warmup` untimed
    steps, then (whatever `warmup` is) PREWARM_MS of launches so that the clocks are up, then
    BURSTS bursts of exactly `steps` steps; the median burst counts.  The rotation over the weight
    copies continues from burst to burst, so no burst finds its weights in the memory-side cache.
    pt.fused_us: the same bursts through lutgemm_matvec_many, which puts up to 32 independent
    matvecs (here: different weight copies) into one launch."""
    sh = stream.cuda_stream
    lutgemm.MatvecSequence(pt.items(max(1, warmup))).launch(sh, fused=False)
    torch.cuda.synchronize()
    seqs = [lutgemm.MatvecSequence(pt.items(steps, offset=b * steps)) for b in range(BURSTS)]
    hot = lutgemm.MatvecSequence(pt.items(steps, rotate=False))
    prewarm(torch, lambda: seqs[0].launch(sh, fused=False))
    ms = time_bursts(torch, stream, [(lambda q=q: q.launch(sh, fused=False)) for q in seqs])
    ms_hot = time_bursts(torch, stream, [lambda: hot.launch(sh, fused=False)] * BURSTS)
    ms_fused = time_bursts(torch, stream, [(lambda q=q: q.launch(sh, fused=True)) for q in seqs])
    pt.burst_us = [t * 1e3 / steps for t in ms]
    pt.fused_burst_us = [t * 1e3 / steps for t in ms_fused]
    pt.fused_us = median(ms_fused) * 1e3 / steps
    return median(ms) * 1e3 / steps, median(ms_hot) * 1e3 / steps


def point_record(pt, us, us_hot):
    return {"k": pt.k, "n": pt.n, "q": pt.q, "g": pt.g, "m": pt.m, "offset": pt.has_offset,
            "us_per_matvec": us, "weight_GBps": pt.b_w / us / 1e3, "pct_hbm_peak": pt.b_w / us / 1e3 / HBM_PEAK_GBS * 100,
            "fused_independent_us_per_matvec": pt.fused_us,
            "fused_independent_pct_hbm_peak": pt.b_w / pt.fused_us / 1e3 / HBM_PEAK_GBS * 100,
            "hot_us_per_matvec": us_hot, "packed_weight_bytes": pt.b_w, "weight_copies_rotated": pt.copies,
            "plan": pt.plan_m, "plan_of_one_row_launches": pt.plan}


def base_line(args, metric, value, us, workload, extra_config=None):
    cfg = {"workload": workload}
    cfg.update(extra_config or {})
    return {
        "metric": metric, "value": value, "unit": "GB/s (packed-weight bytes / matvec time)",
        "us_per_matvec": us, "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "dtype_detail": "fp16 activations, scales and outputs; fp32 tables and accumulation",
        "data": "synthetic (seeded; Bernoulli signs, |N(0,0.02)| scales, N(0,1) fp16 activations)",
        "config": cfg,
    }


MAX_FUSED = 32   # independent matvecs lutgemm_matvec_many puts into one launch


def run_single(args, lutgemm, synth, torch, dev, stream, name):
    cfg = synth.CONFIGS[name]
    k, n, q, g = cfg["k"], cfg["n"], cfg["q"], cfg["g"]
    pt = Point(lutgemm, synth, torch, dev, k, n, q, g, cfg["rtn"], 1, 1, stream.cuda_stream,
               copies=args.copies if name == "cfg1" else None, plan=args.plan)
    us, us_hot = time_point(lutgemm, torch, stream, pt, args.steps, args.warmup)
    us_fused = pt.fused_us
    weight_gbs = pt.b_w / (us * 1e-6) / 1e9
    achieved = pt.b_total / (us * 1e-6) / 1e9
    parity, truth = pt.parity(None if name != "cfg2" else 4096)

    metric = METRIC if name == "cfg1" else "µs/matvec + weight-GB/s (%% HBM peak), k=%d n=%d q=%d g=%d m=1 fp16" % (k, n, q, g)
    workload = "%s: BCQ matvec m=1 k=%d n=%d q=%d g=%d %s" % (
        name, k, n, q, g, "RTN codes as BCQ with offset" if cfg["rtn"] else "no offset")
    units = min(args.steps, MAX_FUSED, pt.copies)
    line = base_line(args, metric, weight_gbs, us, workload,
                     {"weight_copies_rotated": pt.copies, "packed_weight_bytes": pt.b_w,
                      "launch": "one kernel launch per matvec (lutgemm_matvec_each), %d launches back to back per timed burst, "
                                "every launch on its own copy of the weight: what a chain of matvecs that depend on each other "
                                "sees, and the protocol of the reference's caller" % args.steps,
                      "plan": pt.plan})
    line["ms_per_step"] = us / 1e3
    tag = "%d,%s,1" % (q, "true" if pt.has_offset else "false")
    profiled = name == "cfg1" and (pt.plan["waves"], pt.plan["k_splits"]) == CFG1_PROFILED_PLAN
    line["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": achieved / HBM_PEAK_GBS,
                        "traffic": CFG1_PROFILED_TRAFFIC_BYTES_PER_LAUNCH if profiled else None,
                        "traffic_source": (
                            "not measured in this run: rocprofv3 --pmc FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 per dispatch of this "
                            "kernel with this launch plan, from profiles/lut_matvec_kernel_cfg1.md" if profiled else
                            "null: no counter run on record for this kernel with this launch plan (profiles/)"),
                        "kernel": "lut_matvec_kernel<%s>" % tag, "matvecs_per_launch": 1,
                        "algorithmic_bytes_per_launch": pt.b_total, "avg_launch_us": us,
                        "us_per_matvec_bursts": pt.burst_us,
                        "value_is": "back_to_back",
                        "frac_back_to_back": achieved / HBM_PEAK_GBS, "us_back_to_back": us,
                        "frac_fused_independent": pt.b_total / us_fused / 1e3 / HBM_PEAK_GBS,
                        "us_fused_independent": us_fused,
                        "hot_single_copy_us_per_matvec": us_hot}
    line["fused_independent"] = {
        "what": "the same bursts as INDEPENDENT matvecs through lutgemm_matvec_many, which puts up to %d of them (own weight "
                "copy each) into one kernel launch; not what dependent matvecs get" % MAX_FUSED,
        "kernel": "lut_matvec_multi_kernel<%s>" % tag, "matvecs_per_launch": units,
        "us_per_matvec": us_fused, "weight_GBps": pt.b_w / us_fused / 1e3,
        "roofline_frac": pt.b_total / us_fused / 1e3 / HBM_PEAK_GBS,
        "algorithmic_bytes_per_launch": pt.b_total * units, "avg_launch_us": us_fused * units,
        "us_per_matvec_bursts": pt.fused_burst_us}
    us_each = us
    # the device's pure-read time for the same tiles, same grid, same rotation over the copies,
    # timed like the matvec (clocks warmed, median of BURSTS bursts)
    reads = max(1, args.steps)
    orders = [[pt.weights[(b * reads + i) % pt.copies] for i in range(reads)] for b in range(BURSTS)]
    prewarm(torch, lambda: lutgemm.read_probe(orders[0], stream.cuda_stream))
    rms = time_bursts(torch, stream, [(lambda o=o: lutgemm.read_probe(o, stream.cuda_stream)) for o in orders])
    read_us = median(rms) * 1e3 / reads
    tile_bytes = sum(lutgemm.packed_sizes(k, n, q, k // g, pt.has_offset))  # packed tiles incl. padding
    line["pure_read_same_tiles"] = {
        "what": "one launch per weight that only reads the tiles (same grid, same loads in flight): the floor of a single launch",
        "us": read_us, "bytes": tile_bytes, "GBps": tile_bytes / read_us / 1e3, "matvec_time_over_read_time": us_each / read_us}
    line["roofline"]["read_floor_us_single_launch"] = read_us
    if name == "cfg1":
        import numpy as np
        from oracle import oracle
        ref_y = oracle.ref_kernel_fp16(pt.w["bW"][:, :, :1024], pt.w["alpha"].astype(np.float16)[:, :, :1024], None, pt.x16[0])
        ref_err = oracle.error_stats(ref_y, truth[0, :1024])
        parity["emulated_reference_kernel_first_1024_outputs"] = {
            "mean_abs": ref_err[0], "max_abs": ref_err[1], "rel_l2": ref_err[2]}
    line["parity"] = parity

    if args.copy_calibration:
        copy_calibration(torch, dev)

    if name == "cfg1":
        # what the box gives an ordinary device-to-device copy of 1 GiB, timed like everything else
        src = torch.empty(512 * 1024 * 1024, dtype=torch.float16, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        prewarm(torch, lambda: dst.copy_(src))
        cms = median(time_bursts(torch, stream, [lambda: dst.copy_(src)] * BURSTS))
        line["measured_device_copy"] = {
            "what": "torch device-to-device copy of 1 GiB on the same box (1 GiB read + 1 GiB written)",
            "us": cms * 1e3, "GBps_read_plus_written": 2.0 * src.numel() * 2 / (cms * 1e-3) / 1e9}
        del src, dst

    dense = None
    if name == "cfg1" and not args.no_dense:
        # dense fp16 GEMV of the same shape through the vendor library (rocBLAS/hipBLASLt via torch)
        nd = 5  # 5 x 302 MB > 4 x last-level cache
        Wd = [torch.randn((n, k), dtype=torch.float16, device=dev) * 0.03 for _ in range(nd)]
        xv = pt.xd[0]
        outs = torch.empty((nd, n), dtype=torch.float16, device=dev)
        reps = 50

        def warm_dense():
            for i in range(10):
                torch.mv(Wd[i % nd], xv, out=outs[i % nd])
        prewarm(torch, warm_dense)

        def run_dense():
            for i in range(reps):
                torch.mv(Wd[i % nd], xv, out=outs[i % nd])
        dms = event_time_ms(torch, run_dense, stream)
        dense_us = dms * 1e3 / reps
        dense = {"kind": "torch.mv fp16 (rocBLAS/hipBLASLt)", "us_per_matvec": dense_us,
                 "bytes": 2 * k * n + 2 * k + 2 * n,
                 "GBps": (2 * k * n + 2 * k + 2 * n) / (dense_us * 1e-6) / 1e9,
                 "lut_speedup": dense_us / us, "lut_speedup_fused_independent": dense_us / us_fused}
        # the same product through this library's plain streaming kernel (bandwidth-bound comparator)
        sh = stream.cuda_stream
        for i in range(10):
            lutgemm.dense_gemv(Wd[i % nd].data_ptr(), xv.data_ptr(), outs[i % nd].data_ptr(), k, n, sh)
        torch.cuda.synchronize()
        agree = bool(torch.allclose(outs[9 % nd].float(), torch.mv(Wd[9 % nd], xv).float(), rtol=2e-2, atol=2e-2))

        def run_plain():
            for i in range(reps):
                lutgemm.dense_gemv(Wd[i % nd].data_ptr(), xv.data_ptr(), outs[i % nd].data_ptr(), k, n, sh)
        pus = event_time_ms(torch, run_plain, stream) * 1e3 / reps
        dense["handwritten_streaming_gemv"] = {"us_per_matvec": pus, "GBps": dense["bytes"] / pus / 1e3,
                                                "lut_speedup": pus / us, "lut_speedup_fused_independent": pus / us_fused,
                                                "agrees_with_library": agree}
        del Wd
    line["dense_fp16_gemv"] = dense
    line["cpu_baseline"] = None
    if name == "cfg1" and not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(synth, cfg, pt.x16, pt.w, truth)
    pt.close()
    return line


def copy_calibration(torch, dev):
    """Five launches of an ordinary elementwise kernel of known size (reads 256 MiB, writes 256 MiB):
    what FETCH_SIZE and WRITE_SIZE read for it gives the factor between the counters and bytes."""
    src = torch.empty(128 * 1024 * 1024, dtype=torch.float16, device=dev).fill_(1.0)  # 256 MiB
    dst = torch.empty_like(src)
    for _ in range(5):
        torch.mul(src, 1.0, out=dst)
    torch.cuda.synchronize()
    del src, dst


def run_cfg3(args, lutgemm, synth, torch, dev, stream):
    points = []
    tot_bytes = tot_us = tot_fused = 0.0
    worst = 0.0
    todo = [c for c in synth.CFG3_POINTS if args.point is None or (c["q"], c["g"]) == args.point]
    if not todo:
        sys.exit("bench.py: --point %s is not one of the cfg3 points" % (args.point,))
    for c in todo:
        pt = Point(lutgemm, synth, torch, dev, c["k"], c["n"], c["q"], c["g"], False, 1, c["q"] * 10000 + c["g"],
                   stream.cuda_stream)
        us, us_hot = time_point(lutgemm, torch, stream, pt, args.steps, args.warmup)
        rec = point_record(pt, us, us_hot)
        rec["parity"], _ = pt.parity(2048)
        worst = max(worst, rec["parity"]["max_abs"])
        points.append(rec)
        tot_bytes += pt.b_w
        tot_us += us
        tot_fused += pt.fused_us
        pt.close()
    value = tot_bytes / tot_us / 1e3
    fused = tot_bytes / tot_fused / 1e3
    line = base_line(args, "weight-GB/s over the k=n=7168 sweep (q 1..4 x g 32,64,128,k), m=1 fp16", value,
                     tot_us / len(points), "cfg3: %d BCQ matvecs k=n=7168, q in 1..4, g in {32,64,128,7168}" % len(points),
                     {"points": len(points),
                      "launch": "per point, bursts with one kernel launch per matvec (one weight copy each), back to back"})
    line["ms_per_step"] = tot_us / 1e3
    line["points"] = points
    line["fused_independent"] = {"weight_GBps": fused, "us_sum": tot_fused, "frac_hbm_peak": fused / HBM_PEAK_GBS,
                                 "what": "the same bursts as independent matvecs through lutgemm_matvec_many"}
    line["parity"] = {"worst_max_abs": worst, "outputs_checked_per_point": 2048}
    line["roofline"] = {"bound": "hbm", "achieved": value, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": value / HBM_PEAK_GBS, "traffic": None, "kernel": "lut_matvec_kernel<q,false,gsub>",
                        "value_is": "back_to_back", "frac_back_to_back": value / HBM_PEAK_GBS,
                        "frac_fused_independent": fused / HBM_PEAK_GBS,
                        "note": "aggregate packed-weight bytes / summed time over the %d points" % len(points)}
    line["cpu_baseline"] = None
    return line


def run_cfg4(args, lutgemm, synth, torch, dev, stream):
    """One decoder layer's four matvecs back to back (q=2, g=128): a step is the chain."""
    m = args.m
    sh = stream.cuda_stream
    names = ["qkv", "out", "fc1", "fc2"]
    pts = {}
    step_bytes = sum(synth.algorithmic_bytes(L["k"], L["n"], 2, 128, False, m)[0] for L in synth.CFG4_LAYERS.values())
    copies = max(2, int(math.ceil(4.0 * LLC_BYTES / step_bytes)) + 1)  # every launch misses the cache
    for i, nm in enumerate(names):
        L = synth.CFG4_LAYERS[nm]
        pts[nm] = Point(lutgemm, synth, torch, dev, L["k"], L["n"], 2, 128, False, m, 400 + i, sh, copies=copies)
    layers = []
    for nm in names:
        us, us_hot = time_point(lutgemm, torch, stream, pts[nm], args.steps, args.warmup)
        rec = point_record(pts[nm], us, us_hot)
        rec["layer"] = nm
        rec["parity"], _ = pts[nm].parity(2048)
        layers.append(rec)

    def chain_items(steps):
        out = []
        for s in range(steps):
            for nm in names:
                out.extend(pts[nm].items(1, offset=s))
        return out

    # a decoder's projections depend on each other: one launch per matvec, in order
    lutgemm.MatvecSequence(chain_items(max(1, args.warmup))).launch(sh, fused=False)
    torch.cuda.synchronize()
    timed = lutgemm.MatvecSequence(chain_items(args.steps))
    prewarm(torch, lambda: timed.launch(sh, fused=False))
    ms = median(time_bursts(torch, stream, [lambda: timed.launch(sh, fused=False)] * 7))
    chain_us = ms * 1e3 / args.steps
    graph = None
    if args.graph:
        # the same chain replayed from a captured HIP graph: one graph = `copies` steps, so that the
        # rotation over weight copies is part of the graph; replays are checked against the eager result
        eager = [pts[nm].yd.clone() for nm in names]
        g = torch.cuda.CUDAGraph()
        seq = lutgemm.MatvecSequence(chain_items(copies))
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            seq.launch(side.cuda_stream, fused=False)  # warm-up on the capture stream
            side.synchronize()
            with torch.cuda.graph(g, stream=side):
                seq.launch(torch.cuda.current_stream().cuda_stream, fused=False)
        stream.wait_stream(side)
        torch.cuda.synchronize()
        reps = max(1, args.steps // copies)
        same = True
        for _ in range(3):
            for nm in names:
                pts[nm].yd.zero_()
            g.replay()
            torch.cuda.synchronize()
            same = same and all(torch.equal(pts[nm].yd, e) for nm, e in zip(names, eager))

        def replay():
            for _ in range(reps):
                g.replay()
        # timed like the eager chain: clocks brought up with the workload itself, median of seven bursts
        prewarm(torch, replay)
        gms = median(time_bursts(torch, stream, [replay] * 7))
        graph = {"us_per_layer_step": gms * 1e3 / (reps * copies), "steps_per_graph": copies,
                 "replays_per_burst": reps, "replays_equal_eager": bool(same)}
    if args.copy_calibration:
        copy_calibration(torch, dev)
    value = step_bytes / chain_us / 1e3
    line = base_line(args, "µs per decoder layer (QKV+out+FC1+FC2 matvecs) + weight-GB/s, q=2 g=128 m=%d fp16" % m,
                     value, chain_us / 4.0, "cfg4: OPT-175B decoder layer matvecs q=2 g=128 m=%d" % m,
                     {"weight_copies_rotated": copies, "packed_weight_bytes_per_step": step_bytes})
    line["ms_per_step"] = chain_us / 1e3
    line["us_per_layer_step"] = chain_us
    line["sum_of_separately_timed_layers_us"] = sum(r["us_per_matvec"] for r in layers)
    line["layers"] = layers
    line["hip_graph"] = graph
    line["roofline"] = {"bound": "hbm", "achieved": value, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": value / HBM_PEAK_GBS, "traffic": None,
                        "kernel": "lut_matvec_kernel<2,false,1>" if m == 1 else "lut_matvec2_kernel<2,false,1>",
                        "note": "packed-weight bytes of the four layers / time of the chain"}
    line["cpu_baseline"] = None
    for p in pts.values():
        p.close()
    return line


def run_dequant(args, lutgemm, synth, torch, dev, stream):
    """Dense fp16 weight from the packed tiles (the route of batches too large for the LUT
    kernels): a step is one dequantisation of the cfg1 weight; both orientations and the cfg2
    weight are reported beside it.  Bytes = packed tiles read + 2 k n written."""
    import numpy as np
    from oracle import oracle
    sh = stream.cuda_stream
    reps = max(1, min(args.steps, 100))
    shapes = []
    for name in ("cfg1", "cfg2"):
        c = synth.CONFIGS[name]
        k, n, q, g = c["k"], c["n"], c["q"], c["g"]
        w = synth.make_weight(k, n, q, g, rtn=c["rtn"], seed=1)
        W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
        # two outputs alternate so that a launch does not rewrite lines still in the cache
        outs = [torch.empty((k * n,), dtype=torch.float16, device=dev) for _ in range(2)]
        rec = {"workload": name, "k": k, "n": n, "q": q, "g": g, "offset": w["q_bias"] is not None}
        for transposed in (True, False):
            for i in range(max(4, min(args.warmup, 50))):
                W.dequantize(outs[i % 2].data_ptr(), transposed, sh)
            torch.cuda.synchronize()

            def run():
                for i in range(reps):
                    W.dequantize(outs[i % 2].data_ptr(), transposed, sh)
            us = event_time_ms(torch, run, stream) * 1e3 / reps
            nbytes = 2 * k * n + W.weight_bytes()
            rec["W[n][k]" if transposed else "W[k][n]"] = {"us": us, "GBps": nbytes / us / 1e3, "bytes": nbytes}
        # parity of the last result (W[k][n]) on the first 256 outputs against the oracle's dense weight
        got = outs[(reps - 1) % 2].view(k, n)[:, :256].cpu().numpy().astype(np.float64)
        z = w["q_bias"].astype(np.float16)[:, :256] if w["q_bias"] is not None else None
        dense = oracle.dense_weight_f64(np.ascontiguousarray(w["bW"][:, :, :256]),
                                        np.ascontiguousarray(w["alpha"].astype(np.float16)[:, :, :256]),
                                        np.ascontiguousarray(z) if z is not None else None)
        exact = bool(np.all(np.abs(got - dense) <= 2.0 ** -11 * np.abs(dense) + 2.0 ** -24))
        rec["parity"] = {"outputs_checked": 256, "within_half_ulp_fp16": exact}
        if not exact:
            PARITY_FAILURES.append("dequantize %s: more than half an fp16 ulp from the dense weight" % name)
        shapes.append(rec)
        W.close()
        del outs
    if args.copy_calibration:
        copy_calibration(torch, dev)
    head = shapes[0]["W[n][k]"]
    line = base_line(args, "GB/s of dequantisation to dense fp16 (packed tiles read + 2kn written), cfg1 weight, W[n][k]",
                     head["GBps"], head["us"], "dequantize: cfg1 weight k=n=12288 q=3 g=128 to fp16 W[n][k]", {})
    line["unit"] = "GB/s (bytes read + written / time)"
    line["steps"] = reps
    line["ms_per_step"] = head["us"] / 1e3
    line["shapes"] = shapes
    line["roofline"] = {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": head["GBps"] / HBM_PEAK_GBS, "traffic": None, "kernel": "dequantize_kernel<3,false,1>",
                        "algorithmic_bytes_per_launch": head["bytes"], "avg_launch_us": head["us"]}
    line["cpu_baseline"] = None
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=2000,
                    help="untimed steps first (the device reaches its sustained clocks only after some ms of load)")
    ap.add_argument("--config", default="cfg1", choices=["cfg0", "cfg1", "cfg2", "cfg3", "cfg4", "dequant"])
    ap.add_argument("--m", type=int, default=1, help="activation rows (cfg4 only)")
    ap.add_argument("--graph", action="store_true", help="cfg4: also replay the chain from a captured HIP graph")
    ap.add_argument("--copies", type=int, default=33, help="cfg1: distinct weight copies rotated through")
    ap.add_argument("--plan", default=None,
                    help="cfg0/1/2: WAVES,KSPLITS launch plan instead of the measured choice (profiling runs)")
    ap.add_argument("--point", default=None, help="cfg3: only the point Q,G of the sweep (profiling runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense fp16 GEMV comparator")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (known traffic) for scaling rocprof byte counters")
    args = ap.parse_args()
    if args.plan:
        args.plan = tuple(int(v) for v in args.plan.split(","))
    if args.point:
        args.point = tuple(int(v) for v in args.point.split(","))
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (got --gpus %d); a matvec shards by output "
                 "columns, no multi-GPU path is built" % args.gpus)

    import torch

    import lutgemm
    from lutgemm import synth

    lutgemm.load()  # no fallback: fails loudly if the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream()

    if args.config == "cfg3":
        line = run_cfg3(args, lutgemm, synth, torch, dev, stream)
    elif args.config == "cfg4":
        line = run_cfg4(args, lutgemm, synth, torch, dev, stream)
    elif args.config == "dequant":
        line = run_dequant(args, lutgemm, synth, torch, dev, stream)
    else:
        line = run_single(args, lutgemm, synth, torch, dev, stream, args.config)
    print(json.dumps(line), flush=True)
    if PARITY_FAILURES:
        sys.exit("bench.py: result outside the tolerance of the path: " + "; ".join(PARITY_FAILURES))


if __name__ == "__main__":
    main()
