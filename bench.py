#!/usr/bin/env python3
"""Benchmark of the Lloyd iteration on one MI355X.

    python bench.py [--gpus 1] [--steps 20] [--warmup 100] [--config 2]

A "step" is one full k-means iteration (assignment + update + divide) over the whole
synthetic data set of the chosen benchmark configuration (default: the headline, N = 2,097,152,
d = 32, k = 1024, fp32, seeded Gaussian mixture, initial centroids = first k points), with the points
and the initial centroids already resident in HBM when the clock starts -- the reference's protocol
(k-means.cpp:155-169: wall clock around run(), transfers excluded). Prints ONE JSON line.

Legs:
  1. warm-up: the configuration's own run (20 iterations from the initial centroids at the headline) repeated until
     --warmup iterations are done, each followed by a state reset: the first 50 or so iterations after an idle period
     run up to 15 % slower than the following ones;
  2. the timed region: K iterations back to back on the library's stream, one sync on each side,
     wall clock -> value / ms_per_step; every kernel is launched call by call (--graph: the first iteration call by
     call, the others as replays of a recorded pair of iterations, a HIP graph);
  3. the same K iterations again with the library's per-kernel events on (kmx_set_profiling) and events
     around the assignment / update calls -> the split, the dominant kernel's average duration, roofline;
  4. cpu_baseline: the reference's serial k-means (oracle/_ref build of the reference's own serial.hpp if it
     travelled with the tree, else the C restatement in oracle/) timed on ONE host core over a bounded
     sample of the same workload and scaled to the full N.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_TFLOPS = 157.3   # MI355X fp32 (vector or matrix), dense
PEAK_BF16_TFLOPS = 2500.0  # MI355X bf16 matrix, dense
PEAK_FP64_TFLOPS = 78.6    # MI355X fp64 (vector or matrix), dense
VARIANT_NAMES = {0: "base", 1: "lds_fma", 2: "mfma", 4: "mfma_bf16x3"}
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# published full-iteration time for the headline shape on the reference's best hardware (V100 SXM2)
PUBLISHED_MS = {2: 25.45}  # results/README.md:20 of the reference
# HBM bytes per launch of the dominant kernels from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, scaled by
# the readings for a device copy of known size: read from the table rows `| traffic | <config> | <assign|update> | <bytes> |`
# of this file if it travelled with the tree; null otherwise (a run cannot count its own HBM bytes)
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.md")


def measured_traffic(config):
    out = {}
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 4 and cells[0] == "traffic" and cells[1] == str(config):
                    out[cells[2]] = float(cells[3])
    except OSError:
        pass
    return out


def cpu_baseline(km, spec, n_sample, data, means0):
    """One serial Lloyd iteration on one core over the first n_sample points; scaled to N."""
    from oracle import binding as orc  # the checker is only timed here, never used by the measured path
    dim, k = spec.dim, spec.k
    sample = np.ascontiguousarray(data[: n_sample * dim])
    if orc.ref_lib() is not None:
        kind = "reference"
        t0 = time.perf_counter()
        orc.ref_kmeans(sample, means0, dim, k, n_sample, 1)
        dt = time.perf_counter() - t0
    else:
        kind = "port"
        t0 = time.perf_counter()
        orc.kmeans(sample, means0, dim, k, n_sample, 1, threads=1, fast=False)
        dt = time.perf_counter() - t0
    scaled_ms = dt * 1e3 * (int(spec.n) / n_sample)
    out = {
        "value": round(scaled_ms, 1), "unit": "ms/iteration", "cores": 1, "kind": kind,
        "sample": "1 iteration over the first %d of %d points x all %d centroids took %.2f s on 1 core; scaled by N/sample"
                  % (n_sample, int(spec.n), k, dt),
    }
    # the same iteration with the restatement's OpenMP mode (results bit-identical to one thread): what the host cores
    # of this box deliver together; the reference itself has no multi-threaded CPU path
    cores = int(os.environ.get("OMP_NUM_THREADS") or 0) or min(os.cpu_count() or 1, 16)
    if cores > 1:
        t0 = time.perf_counter()
        orc.kmeans(sample, means0, dim, k, n_sample, 1, threads=cores, fast=False)
        dt_all = time.perf_counter() - t0
        out["all_cores"] = {"value": round(dt_all * 1e3 * (int(spec.n) / n_sample), 1), "unit": "ms/iteration", "cores": cores,
                            "kind": "port", "sample": "same sample, %d OpenMP threads: %.2f s" % (cores, dt_all)}
    return out


def warm_up(alg, args, spec, means0, **run_args):
    """The untimed iterations: the configuration's own run (its iteration count, from the initial centroids) as often
    as --warmup asks for, so that the timed run starts from the same state on a device at its working clocks (the
    first 50 or so iterations after an idle period run up to 15 % slower)."""
    left = args.warmup
    while left > 0:
        it = min(left, max(1, int(spec.iterations)))
        alg.run(iters=it, **run_args)
        alg.reset(means0)
        left -= it


def fused_main(km, args, spec, data, means0):
    """--fused: the same protocol around HipFusedKMeansAlgorithm (mirror of CudaFusedKMeansAlgorithm, cuda.hpp:116-233)."""
    n, dim, k = int(spec.n), spec.dim, spec.k
    alg = km.HipFusedKMeansAlgorithm()
    alg.initialize(dim, k, n, args.steps, data, means0)
    warm_up(alg, args, spec, means0)
    km.sync()
    t0 = time.perf_counter()
    alg.run(iters=args.steps)
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    assert int(alg.getClusterSizes().sum()) == n, "cluster counts do not sum to N"
    km.set_profiling(True)
    k_ms = 0.0
    left_over = 0
    for _ in range(args.steps):
        alg.iteration()
        k_ms += km.last_kernel_ms(0)
        left_over += km.last_rechecked()
    km.set_profiling(False)
    k_ms /= args.steps
    alg.cleanup()
    one_pass = k <= 32 and dim <= 32
    read_bytes = 4.0 * (n * dim + 2 * k * dim + k) if one_pass else 4.0 * (2 * n * dim + 2 * n + 2 * k * dim + k)
    out = {
        "metric": "ms per fused k-means iteration, benchmark configuration %d" % args.config,
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "benchmark configuration %d: N=%d d=%d k=%d, fused iteration (%s)"
                               % (args.config, n, dim, k, "single pass over the points" if one_pass else "assignment + update behind one call"),
                   "layout": "aos"},
        "points_centroids_dims_per_s": round(float(n) * k * dim / (ms_per_step * 1e-3), 0),
        "rechecked_points_per_iteration": round(left_over / args.steps, 1),
    }
    if one_pass:
        gbs = read_bytes / (k_ms * 1e-3) / 1e9
        out["roofline"] = {"kernel": "fused single-pass kernel", "bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                           "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None,
                           "algorithmic_bytes": read_bytes, "avg_kernel_ms": round(k_ms, 4)}
    print(json.dumps(out))


def double_main(km, args, spec, data, means0):
    """--double: the same protocol on doubles (kmx_assign_f64 / kmx_update_f64, the reference's --double instantiation).
    The points are the configuration's floats widened to doubles with full mantissas."""
    import numpy as np
    n, dim, k = int(spec.n), spec.dim, spec.k
    data, means0 = km.widen_points(data), km.widen_points(means0)
    alg = km.HipKMeansAlgorithm(dtype=np.float64)
    alg.initialize(dim, k, n, args.steps, data, means0)
    warm_up(alg, args, spec, means0)
    km.sync()
    t0 = time.perf_counter()
    alg.run(iters=args.steps)
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    assert int(alg.getClusterSizes().sum()) == n, "cluster counts do not sum to N"
    alg.reset(means0)
    km.set_profiling(True)
    k_assign = k_update = 0.0
    for _ in range(args.steps):
        nxt = alg.iteration()
        alg.update_step(nxt)
        k_assign += km.last_kernel_ms(0)
        k_update += km.last_kernel_ms(1)
    km.set_profiling(False)
    k_assign /= args.steps; k_update /= args.steps
    alg.cleanup()
    ran_variant = km.last_assign_variant()
    algorithmic = 2.0 * n * k * dim / (k_assign * 1e-3) / 1e12
    update_bytes = 8.0 * (n * dim + k * dim) + 4.0 * (n + k)
    update_gbs = update_bytes / (k_update * 1e-3) / 1e9
    if ran_variant == km.ASSIGN_MFMA_BF16X3:
        roofline = {"kernel": "ranking sweep on float copies (split-bf16 MFMA)", "bound": "mfma", "achieved": round(algorithmic, 1),
                    "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(algorithmic / PEAK_BF16_TFLOPS, 4), "traffic": None,
                    "flops_counted": "algorithmic: 2 N k d per launch"}
    elif k >= 64:
        roofline = {"kernel": "ranking sweep on float copies", "bound": "mfma", "achieved": round(algorithmic, 2), "peak": PEAK_FP32_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(algorithmic / PEAK_FP32_TFLOPS, 4), "traffic": None}
    else:
        gbs = 4.0 * (n * dim + n + k * dim) / (k_assign * 1e-3) / 1e9
        roofline = {"kernel": "ranking sweep on float copies", "bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None}
    roofline["avg_kernel_ms"] = round(k_assign, 4)
    out = {
        "metric": "ms per k-means iteration (assign+update) in double precision, benchmark configuration %d" % args.config,
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64 (points ranked by the float sweep on rounded copies; every point it cannot certify is decided by the serial "
                 "double arithmetic; sums in f64)", "data": "synthetic",
        "config": {"workload": "benchmark configuration %d: N=%d d=%d k=%d in doubles, initial centroids = first k points, seed %d"
                               % (args.config, n, dim, k, spec.seed), "layout": "aos",
                   "assignment_kernel": VARIANT_NAMES.get(ran_variant, str(ran_variant))},
        "points_centroids_dims_per_s": round(float(n) * k * dim / (ms_per_step * 1e-3), 0),
        "roofline": roofline,
        "roofline_update": {"kernel": "update accumulation (fp64 atomics)", "bound": "hbm", "achieved": round(update_gbs, 1),
                            "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(update_gbs / PEAK_HBM_GBS, 4), "traffic": None,
                            "algorithmic_bytes": update_bytes, "avg_kernel_ms": round(k_update, 4)},
    }
    print(json.dumps(out))


def single_pass_report(km, args, spec, alg, means0, ms_per_step, data):
    """The default pair of kernels went through kmx_iteration_f32's single pass (k <= 32, dim <= 32): one kernel reads every
    point once, assigns it, accumulates it and writes its assignment. There is no assignment / update split to report; the
    dominant kernel is that one, bound by HBM."""
    n, dim, k = int(spec.n), spec.dim, spec.k
    alg.reset(means0)
    km.set_profiling(True)
    k_ms, rechecked = 0.0, 0
    for _ in range(args.steps):
        alg.step()
        k_ms += km.last_kernel_ms(0)
        rechecked += km.last_rechecked()
    km.set_profiling(False)
    k_ms /= args.steps
    alg.cleanup()
    traffic = measured_traffic(args.config)
    algorithmic = 4.0 * (n * dim + n + 2 * k * dim + k)     # points in, assignment out, centroids in and out, counts
    gbs = algorithmic / (k_ms * 1e-3) / 1e9
    out = {
        "metric": "ms per k-means iteration (assign+update), benchmark configuration %d" % args.config,
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "benchmark configuration %d: N=%d d=%d k=%d, %s, initial centroids = first k points, seed %d"
                               % (args.config, n, dim, k, "Gaussian mixture" if spec.kind != 1 else "uniform", spec.seed),
                   "layout": "aos", "assignment": "hip_best", "update": "atomic_shm",
                   "launch": "one kmx_iteration_f32 call per iteration: a single pass over the points"},
        "assign_ms": None, "update_ms": None,
        "points_centroids_dims_per_s": round(float(n) * k * dim / (ms_per_step * 1e-3), 0),
        "rechecked_points_per_iteration": round(rechecked / args.steps, 1),
        "roofline": {"kernel": "single-pass iteration kernel (ranking and sums on the matrix cores, the next batch of rows in flight)",
                     "bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                     "traffic": traffic.get("iteration"), "algorithmic_bytes": algorithmic, "avg_kernel_ms": round(k_ms, 4)},
    }
    if not args.no_cpu_baseline:
        per_point_s = 0.45e-9 * k * dim
        n_sample = args.cpu_sample or int(min(n, max(1024, 12.0 / per_point_s)))
        out["cpu_baseline"] = cpu_baseline(km, spec, n_sample, data, means0)
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed iterations before the timed ones, run as repetitions of the configuration's own run")
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (2 = headline)")
    ap.add_argument("--cpu-sample", type=int, default=0, help="points in the CPU baseline sample (0 = about 12 s of work)")
    ap.add_argument("--assign-variant", default="best", choices=["base", "lds_fma", "mfma", "mfma_bf16x3", "best"])
    ap.add_argument("--update-variant", default="atomic_shm", choices=["atomic_point", "atomic_fine", "atomic_shm", "serial_order"],
                    help="serial_order: sums in the order of the reference's serial loop (whole runs bit-identical to it); "
                         "its roofline_update covers all kernels of the variant (sort + sums)")
    ap.add_argument("--fused", action="store_true",
                    help="time the fused iteration (kmx_fused_f32: one call per iteration, no assignment vector; a single "
                         "pass over the points where k <= 32) instead of assignment + update")
    ap.add_argument("--double", action="store_true",
                    help="time the iteration on doubles (kmx_assign_f64 / kmx_update_f64) instead of floats")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="replay a recorded pair of iterations (HIP graph) instead of launching every kernel of the timed "
                         "iterations one by one (measured: no gain on this runtime, 0.042 vs 0.035 ms at configuration 1)")
    ap.add_argument("--two-level", type=int, default=1, choices=[0, 1, 2],
                    help="the split-bf16 sweep in two levels: 0 never, 1 where it pays (default), 2 wherever the kernels allow it")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="one device-to-device copy of the point array before the timed region (a copy kernel of known "
                         "size, to scale FETCH_SIZE / WRITE_SIZE counter readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus %d is not supported" % args.gpus)

    km = importlib.import_module("cuda-kmeans_amd")
    if not (os.path.exists(km.HIP_LIB_PATH) and os.path.exists(km.HOST_LIB_PATH)):
        km.build(force=False)
    if km.device_count() == 0:
        sys.exit("bench.py: no HIP device visible")
    km.set_two_level_sweep(args.two_level)
    spec = km.baseline_config(args.config)
    n, dim, k = int(spec.n), spec.dim, spec.k
    data = km.generate_points(spec)
    means0 = km.first_k_means(spec)

    assign_variant = {"base": km.ASSIGN_BASE, "lds_fma": km.ASSIGN_LDS_FMA, "mfma": km.ASSIGN_MFMA, "mfma_bf16x3": km.ASSIGN_MFMA_BF16X3,
                      "best": km.ASSIGN_BEST}[args.assign_variant]
    update_variant = {"atomic_point": km.UPDATE_ATOMIC_POINT, "atomic_fine": km.UPDATE_ATOMIC_FINE,
                      "atomic_shm": km.UPDATE_ATOMIC_SHM, "serial_order": km.UPDATE_SERIAL_ORDER}[args.update_variant]
    if args.fused:
        return fused_main(km, args, spec, data, means0)
    if args.double:
        return double_main(km, args, spec, data, means0)
    alg = km.HipKMeansAlgorithm(assign_variant, update_variant)
    alg.initialize(dim, k, n, args.steps, data, means0)

    if args.calibrate_copy:
        scratch = km.DeviceBuffer(alg.cu_data.nbytes)
        km.check(km.hip_lib().kmx_d2d(scratch.ptr, alg.cu_data.ptr, alg.cu_data.nbytes))
        km.sync()
        scratch.free()

    # 1. warm-up
    warm_up(alg, args, spec, means0, use_graph=args.graph)

    # 2. timed region
    km.sync()
    t0 = time.perf_counter()
    alg.run(iters=args.steps, use_graph=args.graph)   # ends with one device sync
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / args.steps
    counts = alg.getClusterSizes()
    assert int(counts.sum()) == n, "cluster counts do not sum to N"

    if alg.one_call() and km.last_iteration_passes() == 1:
        return single_pass_report(km, args, spec, alg, means0, ms_per_step, data)

    # 3. instrumented repeat of the same iterations
    alg.reset(means0)
    km.set_profiling(True)
    ev = [km.Event() for _ in range(3)]
    t_assign = t_update = k_assign = k_update = 0.0
    rechecked = 0
    for _ in range(args.steps):
        ev[0].record()
        nxt = alg.iteration()
        ev[1].record()
        alg.update_step(nxt)
        ev[2].record()
        t_assign += ev[0].elapsed_ms(ev[1])
        t_update += ev[1].elapsed_ms(ev[2])
        k_assign += km.last_kernel_ms(0)
        k_update += km.last_kernel_ms(1)
        rechecked += km.last_rechecked()
    ran_variant = km.last_assign_variant()
    km.set_profiling(False)
    t_assign /= args.steps; t_update /= args.steps; k_assign /= args.steps; k_update /= args.steps
    alg.cleanup()

    flop = 2.0 * n * k * dim                                      # one multiply-add per point x centroid x dim
    update_bytes = 4.0 * (n * dim + n + k * dim + k)              # points + assignment in, sums + counts out
    assign_bytes = 4.0 * (n * dim + n + k * dim)
    assign_tflops = flop / (k_assign * 1e-3) / 1e12
    update_gbs = update_bytes / (k_update * 1e-3) / 1e9
    assign_gbs = assign_bytes / (k_assign * 1e-3) / 1e9
    # the dominant kernel is the assignment sweep; it is compute-bound unless k is tiny (flop/byte = k/2)
    if k >= 64 and ran_variant == km.ASSIGN_MFMA_BF16X3:
        # The sweep runs on the bf16 matrix pipeline: the fraction is the ALGORITHMIC work (one multiply-add per point x
        # centroid x dim) against that pipeline's peak. Each algorithmic multiply-add is executed as three bf16 products
        # (split operands); the executed rate is reported beside it, not as the roofline fraction.
        roofline = {"kernel": "assignment sweep (split-bf16 MFMA)", "bound": "mfma", "achieved": round(assign_tflops, 1),
                    "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(assign_tflops / PEAK_BF16_TFLOPS, 4),
                    "traffic": None, "flops_counted": "algorithmic: 2 N k d per launch",
                    "frac_of_fp32_peak": round(assign_tflops / PEAK_FP32_TFLOPS, 4)}
        if args.two_level == 0 and dim > 4:
            # one level: every algorithmic multiply-add is executed as three bf16 products (split operands)
            roofline.update({"executed_tflops": round(3.0 * assign_tflops, 1), "executed_frac": round(3.0 * assign_tflops / PEAK_BF16_TFLOPS, 4),
                             "executed_note": "3 bf16 products per point x centroid x dim on the bf16 matrix pipeline"})
        else:
            roofline["executed_note"] = ("two levels where they pay: one bf16 product per point x centroid x dim for every point, three more "
                                         "for the points the first level cannot settle; packed rows (dim <= 4): one instruction per tile")
    elif k >= 64:
        roofline = {"kernel": "assignment sweep", "bound": "mfma", "achieved": round(assign_tflops, 2),
                    "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s", "frac": round(assign_tflops / PEAK_FP32_TFLOPS, 4),
                    "traffic": None}
    else:
        roofline = {"kernel": "assignment sweep", "bound": "hbm", "achieved": round(assign_gbs, 1),
                    "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(assign_gbs / PEAK_HBM_GBS, 4), "traffic": None}
    traffic = measured_traffic(args.config) if (args.assign_variant, args.update_variant) == ("best", "atomic_shm") else {}
    roofline["traffic"] = traffic.get("assign")
    roofline["traffic_source"] = "profiles/hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this command)" if traffic else None
    roofline["algorithmic_bytes"] = assign_bytes
    roofline["avg_kernel_ms"] = round(k_assign, 4)
    roofline_update = {"kernel": "update accumulation", "bound": "hbm", "achieved": round(update_gbs, 1),
                       "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(update_gbs / PEAK_HBM_GBS, 4),
                       "traffic": traffic.get("update"), "algorithmic_bytes": update_bytes,
                       "avg_kernel_ms": round(k_update, 4)}

    out = {
        "metric": "ms per k-means iteration (assign+update) at N=2M,d=32,k=1024; % roofline" if args.config == 2
                  else "ms per k-means iteration (assign+update), benchmark configuration %d" % args.config,
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": round(ms_per_step / PUBLISHED_MS[args.config], 4) if args.config in PUBLISHED_MS else None,
        "baseline_note": "published: 25.45 ms on V100 SXM2 for this shape (reference results/README.md:20); lower is better"
                         if args.config in PUBLISHED_MS else None,
        "dtype": "f32 (sweep on bf16x3 split operands, f32 accumulate; exact f32 re-evaluation of uncertified points)"
                 if ran_variant == km.ASSIGN_MFMA_BF16X3 else "f32",
        "data": "synthetic",
        "config": {"workload": "benchmark configuration %d: N=%d d=%d k=%d, %s, initial centroids = first k points, seed %d"
                               % (args.config, n, dim, k, "Gaussian mixture" if spec.kind != 1 else "uniform", spec.seed),
                   "layout": "aos", "assignment": "hip_" + args.assign_variant,
                   "assignment_kernel": VARIANT_NAMES.get(ran_variant, str(ran_variant)), "update": args.update_variant,
                   "two_level_sweep": {0: "never", 1: "where it pays", 2: "wherever the kernels allow it"}[args.two_level],
                   "launch": "call by call" if not args.graph or args.steps < 3 else "first iteration call by call, then a recorded pair of iterations replayed (HIP graph)"},
        "assign_ms": round(t_assign, 4), "update_ms": round(t_update, 4),
        "points_centroids_dims_per_s": round(float(n) * k * dim / (ms_per_step * 1e-3), 0),
        "rechecked_points_per_iteration": round(rechecked / args.steps, 1),
        "roofline": roofline, "roofline_update": roofline_update,
    }

    if not args.no_cpu_baseline:
        per_point_s = 0.45e-9 * k * dim        # measured cost of the serial loop per point
        n_sample = args.cpu_sample or int(min(n, max(1024, 12.0 / per_point_s)))
        out["cpu_baseline"] = cpu_baseline(km, spec, n_sample, data, means0)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
