#!/usr/bin/env python3
"""Benchmark of the walk path: one "step" = one pass of the walk kernel over the whole query batch.

Default workload = the headline configuration: DeepWalk, length 80, one query per vertex, on the
symmetrised R-MAT scale-24 graph (edge factor 16, a/b/c/d = .57/.19/.19/.05, weights U[1,100)).
Inputs (CSR, start vertices, path matrix) are resident in HBM before the timed region starts.

Prints ONE JSON line with the walk-steps/s of the whole job, the HBM roofline of the walk path
(algorithmic bytes of one pass / device time of that pass, measured with HIP events on the launch
stream) and the CPU oracle timed on the host cores of the same box over a bounded prefix of the same
queries.  With hub parking (the default for large batches) one pass is a short pipeline of launches --
fw_walk_zprs, then per round fw_hub_scan + fw_hub_batch + fw_walk_zprs -- and the HIP events bracket the whole
pipeline, host-side round trips included.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]
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

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

# name -> generator / walk settings of the five benchmark configurations; "headline" is the one the metric is quoted on.
WORKLOADS = {
    "deepwalk_rmat24_sym": dict(scale=24, sym=True, app="deepwalk", depth=80, queries="all", labels=0),
    "deepwalk_rmat22": dict(scale=22, sym=False, app="deepwalk", depth=80, queries="all", labels=0),
    "ppr_rmat22": dict(scale=22, sym=False, app="ppr", depth=80, queries="all", labels=0),
    "node2vec_rmat24_sym": dict(scale=24, sym=True, app="node2vec", depth=80, queries="all", labels=0),
    "metapath_rmat26": dict(scale=26, sym=False, app="metapath", depth=5, queries=10_000_000, labels=5),
}
HEADLINE = "deepwalk_rmat24_sym"

# HBM-side bytes of one pass (all launches of the walk pipeline) from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs, each scaled by what the same counter reads for the 1 GiB copy kernel (profiles/).
# None for workloads that have not been measured.
MEASURED_TRAFFIC_BYTES = {"deepwalk_rmat24_sym": 5.73e11, "node2vec_rmat24_sym": 5.24e13}


def algorithmic_bytes(app, steps, sampled_edges, queries, probe_terms=0):
    """Bytes the algorithm has to touch: bias array once per visited neighbour + per-step and per-query words.

    DeepWalk / PPR / MetaPath: 4*D + 16*S + 16*Q; node2vec: 8*D + 24*S + 16*Q (binary-search probes are
    reported separately and not included).
    """
    if app == "node2vec":
        return 8 * sampled_edges + 24 * steps + 16 * queries
    return 4 * sampled_edges + 16 * steps + 16 * queries


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--scale", type=int, default=0, help="override the R-MAT scale (smaller boxes / quick checks)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the CPU baseline sample")
    ap.add_argument("--hub-threshold", type=int, default=-1)
    ap.add_argument("--wg-threads", type=int, default=0)
    ap.add_argument("--park-threshold", type=int, default=0, help="0 = library default, -1 = hub parking off")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run the plain copy kernel on 1 GiB (what rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE are "
                         "scaled against)")
    args = ap.parse_args()

    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; the walk path shards by replicating the CSR and splitting "
                 "the queries (no collectives), and no multi-GPU figure is produced.  Run with --gpus 1.")

    fw = importlib.import_module("flowwalker-artifact_amd")
    if fw.device_count() < 1:
        sys.exit("bench.py: no HIP device visible; the walk engine has no CPU fallback")

    wl = dict(WORKLOADS[args.workload])
    if args.scale:
        wl["scale"] = args.scale
    app_id = {"deepwalk": fw.APP_DEEPWALK, "ppr": fw.APP_PPR, "node2vec": fw.APP_NODE2VEC,
              "metapath": fw.APP_METAPATH}[wl["app"]]

    t0 = time.time()
    g = fw.Graph.rmat(wl["scale"], 16, 0.57, 0.19, 0.19, symmetrise=wl["sym"], w_lo=1.0, w_hi=100.0,
                      n_labels=wl["labels"], make_weights=wl["app"] != "metapath", seed=1)
    fw.check(fw.lib().fw_dev_sync())
    gen_s = time.time() - t0

    if wl["queries"] == "all":
        starts = np.arange(g.V, dtype=np.int32)
    else:
        starts = np.random.RandomState(12345).randint(0, g.V, size=int(wl["queries"])).astype(np.int32)
    n = len(starts)
    params = fw.default_params(app=app_id, max_depth=wl["depth"] + 1, seed=1)
    if args.hub_threshold >= 0:
        params.hub_threshold = args.hub_threshold
    if args.wg_threads:
        params.wg_threads = args.wg_threads
    params.park_threshold = args.park_threshold
    d_starts = fw.DeviceBuffer.from_numpy(starts)
    d_paths = fw.DeviceBuffer(n * params.max_depth * 4)

    if args.calibration_copy:
        src, dst = fw.DeviceBuffer(1 << 30), fw.DeviceBuffer(1 << 30)
        fw.check(fw.lib().fw_dev_fill_i32(src.ptr, 7, (1 << 30) // 4))
        fw.check(fw.lib().fw_dev_copy(dst.ptr, src.ptr, 1 << 30))  # fw_copy_u32x4_kernel: reads 1 GiB, writes 1 GiB
        src.free()
        dst.free()

    for _ in range(args.warmup):
        g.walk_device(params, d_starts, n, d_paths)

    fw.check(fw.lib().fw_dev_sync())
    t0 = time.perf_counter()
    kernel_ms = []
    last = None
    for _ in range(args.steps):
        last = g.walk_device(params, d_starts, n, d_paths)  # synchronous: returns after the kernel finished
        kernel_ms.append(last.kernel_ms)
    fw.check(fw.lib().fw_dev_sync())
    wall = time.perf_counter() - t0

    steps_per_pass = last.steps
    ms_per_step = wall * 1e3 / args.steps
    value = steps_per_pass * args.steps / wall
    avg_kernel_ms = float(np.mean(kernel_ms))
    alg_bytes = algorithmic_bytes(wl["app"], last.steps, last.sampled_edges, n)
    achieved = alg_bytes / (avg_kernel_ms * 1e-3) / 1e9

    out = {
        "metric": "walk steps/sec (1 GPU) + % of HBM roofline; R-MAT s24 DeepWalk len 80",
        "value": value,
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "%s: R-MAT scale %d ef 16 %s, %s, %d queries, length %d" % (
                args.workload, wl["scale"], "symmetrised" if wl["sym"] else "directed", wl["app"], n, wl["depth"]),
            "vertices": g.V, "csr_entries": g.E, "queries": n,
            "walk_steps_per_pass": int(last.steps), "sampled_edges_per_pass": int(last.sampled_edges),
            "wg_threads": params.wg_threads, "hub_threshold": params.hub_threshold,
            "park_threshold": params.park_threshold, "launches_per_pass": last.launches, "grid": last.grid,
            "graph_gen_s": round(gen_s, 2),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            # measured with the library defaults only: any override makes it another run
            "traffic": MEASURED_TRAFFIC_BYTES.get(
                args.workload if not args.scale and args.park_threshold == 0 and args.hub_threshold < 0
                and args.wg_threads == 0 and (last.launches > 1 or wl["app"] == "node2vec") else None),
            "kernel": "fw_walk_zprs" if last.launches == 1 else "fw_walk_zprs + fw_hub_batch pipeline",
            "kernel_ms": avg_kernel_ms,
            "algorithmic_bytes": int(alg_bytes),
        },
    }
    if out["roofline"]["traffic"] is not None:
        # what the memory actually moved per pass, as a rate over the same device time: with hub parking a list is
        # read once per batch of walkers, so `achieved` (bytes every walker would read alone) exceeds the peak and
        # measures reuse; this pair is the pipeline's real HBM rate
        out["roofline"]["traffic_achieved"] = out["roofline"]["traffic"] / (avg_kernel_ms * 1e-3) / 1e9
        out["roofline"]["traffic_frac"] = out["roofline"]["traffic_achieved"] / HBM_PEAK_GBS
    if last.launches > 1:
        # per-kernel view of the last pass: each kernel's own HIP-event time and the algorithmic bytes of the steps
        # it took (what every walker would have to read on its own; fw_hub_batch reads a hub list once per batch
        # of up to 64 walkers, so its figure measures reuse, not DRAM speed)
        walk_b = algorithmic_bytes(wl["app"], last.steps - last.hub_steps, last.sampled_edges - last.hub_sampled_edges, n)
        hub_b = algorithmic_bytes(wl["app"], last.hub_steps, last.hub_sampled_edges, 0)
        out["roofline"]["kernels"] = [
            {"kernel": "fw_walk_zprs", "total_ms": last.walk_kernel_ms, "algorithmic_bytes": int(walk_b),
             "achieved": walk_b / (last.walk_kernel_ms * 1e-3) / 1e9, "steps": int(last.steps - last.hub_steps)},
            {"kernel": "fw_hub_scan + fw_hub_batch", "total_ms": last.hub_kernel_ms, "algorithmic_bytes": int(hub_b),
             "achieved": hub_b / (last.hub_kernel_ms * 1e-3) / 1e9, "steps": int(last.hub_steps)},
        ]

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(fw, g, params, starts, args.cpu_seconds)

    g.destroy()
    print(json.dumps(out))


def cpu_baseline(fw, g, params, starts, target_s):
    """Times the CPU oracle (the checker, used here only as the reported baseline) on a prefix of the queries."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import fw_oracle_binding as orc

    labels = params.app == fw.APP_METAPATH
    xadj, adj, w, lab = g.download(weights=not labels, labels=labels)
    og = orc.Graph(xadj, adj, w, lab)
    op = orc.from_walk_params(params)
    cores = orc.lib().fw_oracle_num_threads()
    # pilot to size the sample so that the timed run takes about target_s
    pilot = min(len(starts), 4096)
    t = time.perf_counter()
    _, s0, _ = orc.walk(og, op, starts[:pilot])
    dt = max(time.perf_counter() - t, 1e-4)
    m = int(min(len(starts), max(pilot, pilot * target_s / dt)))
    t = time.perf_counter()
    _, steps, _ = orc.walk(og, op, starts[:m])
    dt = time.perf_counter() - t
    return {
        "value": steps / dt, "unit": "steps/s", "cores": int(cores), "kind": "port",
        "sample": "first %d of %d queries of the same workload, %d steps in %.1f s, OpenMP schedule(dynamic)" % (
            m, len(starts), steps, dt),
    }


if __name__ == "__main__":
    main()
