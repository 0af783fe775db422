#!/usr/bin/env python3
"""Benchmark of the BCQ LUT matvec on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one matvec of the headline configuration (cfg1: m=1, k=n=12288, q=3, g=128, fp16
activations, no offset) with the packed weight already resident in HBM.  Consecutive steps use
different weight copies (R copies, R * packed bytes > 4 x the 256 MiB last-level cache), so every
step streams its weight from HBM and not from cache.  The K timed steps are issued back to back
with one C-ABI call and bracketed by HIP events on the launch stream.

Prints ONE JSON line: value = packed-weight GB/s (higher is better), plus us per matvec, the
roofline block for the matvec kernel, the dense fp16 GEMV comparator, the single-copy ("hot")
figure and the CPU baseline (the reference's CPU path restated in oracle/, timed on this box's
host cores on a bounded slice of the same workload).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "lut-gemm_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
METRIC = "µs/matvec + weight-GB/s (% HBM peak), n=k=12288 q=3 g=128 m=1 fp16"


def event_time_ms(torch, fn, stream):
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record(stream)
    fn()
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop)


def cpu_baseline(cfg, x16, w, slice_n=12288):
    """The reference's CPU path (dequantize_cpu then the float triple-loop matmul), restated in
    oracle/, single-threaded as the reference is, on the first `slice_n` outputs of the workload;
    then the same loops with OpenMP over all host cores."""
    import numpy as np
    from oracle import oracle
    k, n = cfg["k"], cfg["n"]
    bW = np.ascontiguousarray(w["bW"][:, :, :slice_n])
    alpha = np.ascontiguousarray(w["alpha"].astype(np.float16)[:, :, :slice_n])
    t0 = time.perf_counter()
    fW = oracle.dequantize_cpu(bW, alpha)
    y = oracle.matmul_cpu(x16, fW)
    t1 = time.perf_counter()
    fW2, threads = oracle.dequantize_cpu_omp(bW, alpha)
    y2, _ = oracle.matmul_cpu_omp(x16, fW2)
    t2 = time.perf_counter()
    scale = n / float(slice_n)
    b_w = (k * slice_n * cfg["q"] // 8) + (k // cfg["g"]) * cfg["q"] * slice_n * 2
    serial_s = t1 - t0
    omp_s = t2 - t1
    return {
        "value": b_w / serial_s / 1e9,
        "unit": "GB/s (packed-weight bytes)",
        "cores": 1,
        "kind": "port",
        "sample": "cfg1 outputs 0..%d of %d (%.1f%% of one matvec): dequantize_cpu + matmul_cpu, %.2f s" % (
            slice_n - 1, n, 100.0 / scale, serial_s),
        "us_per_matvec_extrapolated": serial_s * scale * 1e6,
        "openmp": {"cores": int(threads), "value": b_w / omp_s / 1e9,
                   "us_per_matvec_extrapolated": omp_s * scale * 1e6},
        "checksum": float(np.abs(y).sum()),
    }, y


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--copies", type=int, default=17, help="distinct weight copies rotated through")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense fp16 GEMV comparator")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (known traffic) for scaling rocprof byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (got --gpus %d); the path shards by output "
                 "columns, see DESIGN.md" % args.gpus)

    import numpy as np
    import torch

    import lutgemm
    from lutgemm import synth

    lutgemm.load()  # no fallback: fails loudly if the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream

    cfg = synth.CONFIGS["cfg1"]
    k, n, q, g = cfg["k"], cfg["n"], cfg["q"], cfg["g"]
    b_w, b_total = synth.algorithmic_bytes(k, n, q, g, False, 1)
    w = synth.make_weight(k, n, q, g, seed=1)
    x16 = synth.make_x(1, k, seed=1)

    copies = max(1, args.copies)
    weights = [lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, None) for _ in range(copies)]
    xd = torch.from_numpy(x16).to(dev)
    yd = torch.zeros((copies, n), dtype=torch.float16, device=dev)
    # launch plan: measured once on the first copy (a few untimed launches), same plan for all
    plan = weights[0].autotune(sh)
    for wgt in weights[1:]:
        wgt.set_plan(plan["waves"], plan["k_splits"])

    def sequence(count, rotate=True):
        return lutgemm.MatvecSequence(
            [(weights[(i % copies) if rotate else 0], xd.data_ptr(), yd[(i % copies) if rotate else 0].data_ptr(), 1)
             for i in range(count)])

    warm = sequence(max(1, args.warmup))
    timed = sequence(args.steps)
    hot = sequence(args.steps, rotate=False)

    warm.launch(sh)
    torch.cuda.synchronize()
    ms = event_time_ms(torch, lambda: timed.launch(sh), stream)
    torch.cuda.synchronize()
    ms_hot = event_time_ms(torch, lambda: hot.launch(sh), stream)
    torch.cuda.synchronize()

    us = ms * 1e3 / args.steps
    us_hot = ms_hot * 1e3 / args.steps
    weight_gbs = b_w / (us * 1e-6) / 1e9
    achieved = b_total / (us * 1e-6) / 1e9

    # parity of what was just timed, against the double-precision oracle (checker only)
    from oracle import oracle
    truth = oracle.matvec_f64(w["bW"], w["alpha"].astype(np.float16), None, x16)
    y = yd[0].cpu().numpy()
    mean_abs, max_abs, rel_l2 = oracle.error_stats(y, truth)
    ref_y = oracle.ref_kernel_fp16(w["bW"][:, :, :1024], w["alpha"].astype(np.float16)[:, :, :1024], None, x16[0])
    ref_err = oracle.error_stats(ref_y, truth[0, :1024])

    if args.copy_calibration:
        src = torch.empty(128 * 1024 * 1024, dtype=torch.float16, device=dev).fill_(1.0)  # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.mul(src, 1.0, out=dst)  # an ordinary elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    dense = None
    if not args.no_dense:
        # dense fp16 GEMV of the same shape through the vendor library (rocBLAS/hipBLASLt via torch)
        nd = 5  # 5 x 302 MB > 4 x last-level cache
        Wd = [torch.randn((n, k), dtype=torch.float16, device=dev) * 0.03 for _ in range(nd)]
        xv = xd[0]
        outs = torch.empty((nd, n), dtype=torch.float16, device=dev)
        for i in range(10):
            torch.mv(Wd[i % nd], xv, out=outs[i % nd])
        torch.cuda.synchronize()
        reps = 50

        def run_dense():
            for i in range(reps):
                torch.mv(Wd[i % nd], xv, out=outs[i % nd])
        dms = event_time_ms(torch, run_dense, stream)
        dense_us = dms * 1e3 / reps
        dense = {"kind": "torch.mv fp16 (rocBLAS/hipBLASLt)", "us_per_matvec": dense_us,
                 "bytes": 2 * k * n + 2 * k + 2 * n,
                 "GBps": (2 * k * n + 2 * k + 2 * n) / (dense_us * 1e-6) / 1e9,
                 "lut_speedup": dense_us / us}
        del Wd

    cpu = None
    if not args.no_cpu:
        cpu, ycpu = cpu_baseline(cfg, x16, w)
        cpu["max_abs_vs_truth"] = float(np.abs(ycpu[0].astype(np.float64) - truth[0, :ycpu.shape[1]]).max())

    line = {
        "metric": METRIC,
        "value": weight_gbs,
        "unit": "GB/s (packed-weight bytes / matvec time)",
        "us_per_matvec": us,
        "pct_hbm_peak": 100.0 * weight_gbs / HBM_PEAK_GBS,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16 in/out, fp32 accumulate",
        "data": "synthetic (seeded; Bernoulli signs, |N(0,0.02)| scales, N(0,1) fp16 activations)",
        "config": {"workload": "cfg1: BCQ matvec m=1 k=12288 n=12288 q=3 g=128 no offset",
                   "weight_copies_rotated": copies, "packed_weight_bytes": b_w,
                   "plan": weights[0].plan()},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "lut_matvec_kernel<3,false,1>", "algorithmic_bytes_per_launch": b_total,
                     "avg_launch_us": us},
        "hot_single_copy": {"us_per_matvec": us_hot, "weight_GBps": b_w / (us_hot * 1e-6) / 1e9},
        "parity": {"truth": "fp64 accumulation over fp16-rounded inputs (oracle)",
                   "mean_abs": mean_abs, "max_abs": max_abs, "rel_l2": rel_l2,
                   "emulated_reference_kernel_first_1024_outputs": {
                       "mean_abs": ref_err[0], "max_abs": ref_err[1], "rel_l2": ref_err[2]}},
        "dense_fp16_gemv": dense,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
