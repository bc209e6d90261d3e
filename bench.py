#!/usr/bin/env python3
"""Benchmark of the walk path: one "step" = one pass of the walk kernel over the whole query batch.

Default workload = the headline configuration: DeepWalk, length 80, one query per vertex, on the
symmetrised R-MAT scale-24 graph (edge factor 16, a/b/c/d = .57/.19/.19/.05, weights U[1,100)).
Inputs (CSR, start vertices, path matrix) are resident in HBM before the timed region starts.

Prints ONE JSON line with the walk-steps/s of the whole job, the HBM roofline of the walk path on three
stated bases (what the kernels of one pass ask of the memory, modelled from the run's counters; the
useful part of it; the algorithmic bytes every walker would read alone -- all over the device time of
that pass, measured with HIP events on the launch stream), the profiler's measured traffic for the same
workload when the summary under profiles/ was taken on these sources, one line per benchmark
configuration measured after the timed region (`configs`) and the CPU oracle timed on the host cores
of the same box over a bounded prefix of the same queries.  With hub parking (the default for large batches) one pass is a short pipeline of launches --
fw_walk_zprs, then per round fw_hub_scan + fw_hub_batch + fw_walk_zprs -- and the HIP events bracket the whole
pipeline, host-side round trips included.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-configs]
"""
import argparse
import ctypes as C
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
CONFIG_OF = {"deepwalk_rmat22": "C2", "ppr_rmat22": "C3", "node2vec_rmat24_sym": "C4", "metapath_rmat26": "C5",
             "deepwalk_rmat24_sym": "C4 graph, DeepWalk (headline)"}

# The profiler's view of a pass (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters read for
# the 1 GiB copy kernel) lives in the summary under profiles/, in a line
#   traffic_bytes_per_pass workload=<name> fetched=<B> written=<B> total=<B> sources=<sha of the kernel sources>
# which is read at run time; the line says on which sources it was taken, and the JSON says whether those are the
# sources of this run.
PROFILE_OF = {
    "deepwalk_rmat24_sym": "profiles/walk_pipeline_deepwalk_rmat24sym_pmc.txt",
    "node2vec_rmat24_sym": "profiles/walk_pipeline_node2vec_rmat24sym_pmc.txt",
}


def profiled_traffic(workload, sources_sha):
    """(total bytes, fields) of the traffic line for `workload` in its profile summary, or None."""
    path = PROFILE_OF.get(workload)
    if not path or not os.path.exists(os.path.join(ROOT, path)):
        return None
    for line in open(os.path.join(ROOT, path)):
        parts = line.split()
        if parts[:1] != ["traffic_bytes_per_pass"]:
            continue
        kv = dict(x.split("=", 1) for x in parts[1:] if "=" in x)
        if kv.get("workload") != workload:
            continue
        return {"traffic": float(kv["total"]), "traffic_fetched": float(kv["fetched"]),
                "traffic_written": float(kv["written"]), "traffic_source": path,
                "traffic_sources_sha": kv.get("sources"), "traffic_taken_on_these_sources": kv.get("sources") == sources_sha}
    return None


def algorithmic_bytes(app, steps, sampled_edges, queries):
    """Bytes every walker would have to touch on its own: the bias array once per visited neighbour + per-step and
    per-query words.  DeepWalk / PPR / MetaPath: 4*D + 16*S + 16*Q; node2vec: 8*D + 24*S + 16*Q (binary-search
    probes not included)."""
    if app == "node2vec":
        return 8 * sampled_edges + 24 * steps + 16 * queries
    return 4 * sampled_edges + 16 * steps + 16 * queries


def roofline_of(app, st, n, kernel_ms):
    """HBM roofline of one pass on three bases, all over the same device time.
    * `achieved` / `frac`: what the kernels asked of the memory, MODELLED from the run's own counters
      (fw_walk_stats: lists as often as they were actually streamed + 128 bytes per scattered read + 32 bytes per
      scattered store + the records streamed; `breakdown` has the parts).  Bounded by 1.
    * `useful_frac`: the part of it an implementation cannot avoid once lists are shared: the list bytes streamed
      + 16 bytes per step + 16 bytes per query.
    * `algorithmic_rate` / `algorithmic_frac`: the bytes every walker would read on its own (4*D + 16*S + 16*Q; node2vec
      as the reference evaluates it, 8*D + 24*S + 16*Q) over the same time.  With hub parking a list is read once per
      batch of walkers, so this exceeds the peak; `reuse_factor` = algorithmic / modelled says by how much lists were
      shared.  Without parking (roofline.no_parking) it is the fraction of the roofline the walk kernel reaches."""
    alg = algorithmic_bytes(app, st.steps, st.sampled_edges, n)
    req = int(st.requested_bytes)
    sec = kernel_ms * 1e-3
    useful = int(st.list_bytes) + 16 * int(st.steps) + 16 * n
    return {
        "bound": "hbm", "achieved": req / sec / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": req / sec / 1e9 / HBM_PEAK_GBS, "kernel_ms": kernel_ms,
        "bytes_basis": "modelled from the run's counters (lists as streamed + 128 B per scattered read + 32 B per "
                       "scattered store + records)",
        "requested_bytes": req,
        "breakdown": {"list_bytes": int(st.list_bytes), "scattered_read_bytes": 128 * int(st.scattered_reads),
                      "scattered_write_bytes": 32 * int(st.scattered_writes), "record_bytes": int(st.record_bytes)},
        "useful_bytes": useful, "useful_frac": useful / sec / 1e9 / HBM_PEAK_GBS,
        "algorithmic_bytes": int(alg), "algorithmic_rate": alg / sec / 1e9,
        "algorithmic_frac": alg / sec / 1e9 / HBM_PEAK_GBS, "reuse_factor": alg / req if req else None,
    }


def make_graph(fw, wl):
    return fw.Graph.rmat(wl["scale"], 16, 0.57, 0.19, 0.19, symmetrise=wl["sym"], w_lo=1.0, w_hi=100.0,
                         n_labels=wl["labels"], make_weights=wl["app"] != "metapath", seed=1)


def starts_of(g, wl):
    if wl["queries"] == "all":
        return np.arange(g.V, dtype=np.int32)
    return np.random.RandomState(12345).randint(0, g.V, size=int(wl["queries"])).astype(np.int32)


def app_id_of(fw, name):
    return {"deepwalk": fw.APP_DEEPWALK, "ppr": fw.APP_PPR, "node2vec": fw.APP_NODE2VEC,
            "metapath": fw.APP_METAPATH}[name]


def one_config(fw, g, name, wl, passes, warmup, **overrides):
    """`passes` passes of one configuration with the library defaults, device-resident inputs; a line of configs[]."""
    starts = starts_of(g, wl)
    n = len(starts)
    params = fw.default_params(app=app_id_of(fw, wl["app"]), max_depth=wl["depth"] + 1, seed=1, **overrides)
    d_starts = fw.DeviceBuffer.from_numpy(starts)
    d_paths = fw.DeviceBuffer(n * params.max_depth * 4)
    try:
        for _ in range(warmup):
            g.walk_device(params, d_starts, n, d_paths)
        ms, st = [], None
        for _ in range(passes):
            st = g.walk_device(params, d_starts, n, d_paths)
            ms.append(st.kernel_ms)
    finally:
        d_starts.free()
        d_paths.free()
    kernel_ms = float(np.mean(ms))
    r = roofline_of(wl["app"], st, n, kernel_ms)
    return {
        "config": CONFIG_OF.get(name, name), "workload": name, "app": wl["app"], "vertices": g.V, "csr_entries": g.E,
        "queries": n, "walk_steps_per_pass": int(st.steps), "passes": passes, "device_ms_per_pass": kernel_ms,
        "steps_per_s": st.steps / (kernel_ms * 1e-3), "launches_per_pass": st.launches,
        "frac": r["frac"], "achieved_GBs": r["achieved"], "bytes_basis": r["bytes_basis"],
        "useful_frac": r["useful_frac"], "algorithmic_frac": r["algorithmic_frac"],
        "algorithmic_rate_GBs": r["algorithmic_rate"], "reuse_factor": r["reuse_factor"],
    }


def config1(fw):
    """C1: directed uniform-random graph, 7,115 vertices, 103,689 distinct edges (no self-loops), weights U[1,5),
    seed 1; 100 seeded uniform starts, length 80."""
    rng = np.random.RandomState(1)
    V, E = 7115, 103689
    keys = np.empty(0, dtype=np.int64)
    while len(keys) < E:
        s = rng.randint(0, V, size=2 * E).astype(np.int64)
        d = rng.randint(0, V, size=2 * E).astype(np.int64)
        keys = np.unique(np.concatenate([keys, (s * V + d)[s != d]]))
    keys = np.sort(rng.choice(keys, size=E, replace=False))
    xadj = np.zeros(V + 1, dtype=np.uint32)
    np.cumsum(np.bincount(keys // V, minlength=V), out=xadj[1:])
    g = fw.Graph.from_csr(xadj, (keys % V).astype(np.int32), (1.0 + 4.0 * rng.random_sample(E)).astype(np.float32))
    try:
        wl = dict(app="deepwalk", depth=80, queries=100)
        starts = rng.randint(0, V, size=100).astype(np.int32)
        params = fw.default_params(app=fw.APP_DEEPWALK, max_depth=81, seed=1)
        g.walk(params, starts)
        ms, st = [], None
        for _ in range(5):
            _, st = g.walk(params, starts)
            ms.append(st.kernel_ms)
        kernel_ms = float(np.mean(ms))
        r = roofline_of("deepwalk", st, 100, kernel_ms)
        return {"config": "C1", "workload": "deepwalk_uniform_7115", "app": "deepwalk", "vertices": V, "csr_entries": E,
                "queries": 100, "walk_steps_per_pass": int(st.steps), "passes": 5, "device_ms_per_pass": kernel_ms,
                "steps_per_s": st.steps / (kernel_ms * 1e-3), "launches_per_pass": st.launches, "frac": r["frac"],
                "achieved_GBs": r["achieved"], "bytes_basis": r["bytes_basis"],
                "useful_frac": r["useful_frac"], "algorithmic_frac": r["algorithmic_frac"],
                "algorithmic_rate_GBs": r["algorithmic_rate"], "reuse_factor": r["reuse_factor"],
                "note": "100 walks of 80 dependent steps: a latency measurement, not a bandwidth one"}
    finally:
        g.destroy()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--scale", type=int, default=0, help="override the R-MAT scale (smaller boxes / quick checks)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip what follows the timed region: the report of the other configurations and the extra "
                         "pass that splits the time over the kernels")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target duration of the CPU baseline sample")
    ap.add_argument("--p", type=float, default=0.0, help="node2vec return parameter (0 = the library default 2.0)")
    ap.add_argument("--q", type=float, default=0.0, help="node2vec in-out parameter (0 = the library default 0.5)")
    ap.add_argument("--hub-threshold", type=int, default=-1)
    ap.add_argument("--wg-threads", type=int, default=0)
    ap.add_argument("--park-threshold", type=int, default=0, help="0 = library default, -1 = hub parking off")
    ap.add_argument("--sampler", default="native", choices=["native", "ref_zprs", "ref_dprs"],
                    help="native = this engine's sampler; ref_zprs / ref_dprs = the reference's own samplers and round "
                         "structure restated for 64-lane waves (ablation baseline, hub_threshold 1024 unless given)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run the plain copy kernel on 1 GiB (what rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE are "
                         "scaled against)")
    ap.add_argument("--calibration-random", action="store_true",
                    help="also measure the memory's rate of scattered accesses over 4 GiB (64-byte line reads, 4-byte "
                         "and 16-byte stores) and report it as calibration.random_access")
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
    defaults = (not args.scale and args.park_threshold == 0 and args.hub_threshold < 0 and args.wg_threads == 0
                and args.sampler == "native" and args.p == 0.0 and args.q == 0.0)

    t0 = time.time()
    g = make_graph(fw, wl)
    fw.check(fw.lib().fw_dev_sync())
    gen_s = time.time() - t0

    starts = starts_of(g, wl)
    n = len(starts)
    params = fw.default_params(app=app_id_of(fw, wl["app"]), max_depth=wl["depth"] + 1, seed=1)
    if args.hub_threshold >= 0:
        params.hub_threshold = args.hub_threshold
    if args.wg_threads:
        params.wg_threads = args.wg_threads
    params.park_threshold = args.park_threshold
    if args.p > 0.0:
        params.p = args.p
    if args.q > 0.0:
        params.q = args.q
    if args.sampler != "native":
        params.sampler = fw.SAMPLER_REF_ZPRS if args.sampler == "ref_zprs" else fw.SAMPLER_REF_DPRS
        if args.hub_threshold < 0:
            params.hub_threshold = 1024  # THRESHOLD of the reference (include/walker.cuh:29)
    d_starts = fw.DeviceBuffer.from_numpy(starts)
    d_paths = fw.DeviceBuffer(n * params.max_depth * 4)

    if args.calibration_copy:
        src, dst = fw.DeviceBuffer(1 << 30), fw.DeviceBuffer(1 << 30)
        fw.check(fw.lib().fw_dev_fill_i32(src.ptr, 7, (1 << 30) // 4))
        fw.check(fw.lib().fw_dev_copy(dst.ptr, src.ptr, 1 << 30))  # fw_copy_u32x4_kernel: reads 1 GiB, writes 1 GiB
        src.free()
        dst.free()

    random_access = None
    if args.calibration_random:
        buf = fw.DeviceBuffer(4 << 30)
        fw.check(fw.lib().fw_dev_fill_i32(buf.ptr, 0, (4 << 30) // 4))
        random_access = {"buffer_GiB": 4}
        for name, mode in (("line_reads_per_s", 0), ("stores_4B_per_s", 1), ("stores_16B_per_s", 3),
                           ("loads_per_s_two_halves_of_one_128B_block", 4), ("loads_per_s_two_128B_blocks", 5)):
            rate = C.c_double(0.0)
            fw.check(fw.lib().fw_dev_random_access_rate(buf.ptr, 4 << 30, mode, C.byref(rate)))
            random_access[name] = rate.value
        buf.free()

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
    split = None
    if last.launches > 1 and not args.no_configs:
        # per-kernel view: one more pass, outside the timed region, with an event pair around every launch (the timed
        # passes do without: an event costs the stream about 5 us, and a pass is some 150 launches)
        params.time_kernels = 1
        split = g.walk_device(params, d_starts, n, d_paths)
        params.time_kernels = 0
    d_starts.free()
    d_paths.free()

    steps_per_pass = last.steps
    ms_per_step = wall * 1e3 / args.steps
    value = steps_per_pass * args.steps / wall
    avg_kernel_ms = float(np.mean(kernel_ms))
    roofline = roofline_of(wl["app"], last, n, avg_kernel_ms)
    roofline["kernel"] = ("fw_walk_ref" if args.sampler != "native" else
                          "fw_walk_zprs" if last.launches == 1 else "fw_walk_zprs + fw_hub_scan + fw_hub_batch + fw_hub_quad pipeline")
    # the profiler's view of the same workload (library defaults only: any override makes it another run)
    sources_sha = fw.sources_sha()
    prof = profiled_traffic(args.workload, sources_sha) if defaults and last.launches > 1 else None
    roofline["traffic"] = None
    if prof:
        roofline.update(prof)
        roofline["traffic_frac"] = prof["traffic"] / (avg_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
    if split is not None:
        roofline["kernels"] = [
            {"kernel": "fw_walk_zprs", "total_ms": split.walk_kernel_ms, "steps": int(split.steps - split.hub_steps)},
            {"kernel": "fw_hub_scan + fw_hub_batch + fw_hub_quad", "total_ms": split.hub_kernel_ms, "steps": int(split.hub_steps)},
        ]
        roofline["kernels_pass_ms"] = split.kernel_ms

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
            "park_threshold": params.park_threshold, "sampler": args.sampler, "launches_per_pass": last.launches,
            "p": params.p, "q": params.q,
            "grid": last.grid,
            "graph_gen_s": round(gen_s, 2), "sources_sha": sources_sha,
        },
        "roofline": roofline,
    }
    if random_access is not None:
        # the modelled requests of a pass: lists in 128-byte blocks, one request per scattered read or store
        random_access["pipeline_requests_per_s"] = (
            (last.list_bytes + last.record_bytes) / 128.0 + last.scattered_reads + last.scattered_writes) / (avg_kernel_ms * 1e-3)
        out["calibration"] = {"random_access": random_access}

    if not args.no_configs and defaults and args.workload == HEADLINE:
        # after the timed region: the headline without hub parking (every walker reads its lists itself, one launch:
        # the walk kernel against the roofline on the bytes it touches) and one line per benchmark configuration
        nop = one_config(fw, g, HEADLINE, wl, passes=1, warmup=0, park_threshold=-1)
        # one launch in which every walker reads its own lists: the walk kernel against the roofline on the algorithmic
        # bytes 4*D + 16*S + 16*Q
        nop["modelled_frac"] = nop["frac"]
        nop["frac"] = nop["algorithmic_frac"]
        nop["achieved_GBs"] = nop["algorithmic_rate_GBs"]
        nop["bytes_basis"] = "algorithmic (4*D + 16*S + 16*Q)"
        out["roofline"]["no_parking"] = nop
        configs = [config1(fw)]
        configs.append(one_config(fw, g, "node2vec_rmat24_sym", WORKLOADS["node2vec_rmat24_sym"], passes=3, warmup=1))
        # node2vec's two-stage step (propose by weight, accept by the node2vec factor) costs trials in proportion to
        # max(1, q) where most proposals are not adjacent to the previous vertex (and nothing for a small p: the return
        # edge's excess is a component of its own); the reference's one-pass sampler costs the same at every (p, q).
        # Two points away from the benchmark's, one pass each.
        n2v_points = []
        for pp, qq in ((4.0, 0.25), (0.25, 4.0)):
            c = one_config(fw, g, "node2vec_rmat24_sym", WORKLOADS["node2vec_rmat24_sym"], passes=1, warmup=0, p=pp, q=qq)
            c["config"] = "C4 at p = %g, q = %g" % (pp, qq)
            c["p"], c["q"] = pp, qq
            n2v_points.append(c)
        cpu = None if args.no_cpu else cpu_baseline(fw, g, params, starts, args.cpu_seconds)
        g.destroy()
        g22 = make_graph(fw, WORKLOADS["deepwalk_rmat22"])
        try:
            configs.insert(1, one_config(fw, g22, "deepwalk_rmat22", WORKLOADS["deepwalk_rmat22"], passes=3, warmup=1))
            configs.insert(2, one_config(fw, g22, "ppr_rmat22", WORKLOADS["ppr_rmat22"], passes=3, warmup=1))
        finally:
            g22.destroy()
        g26 = make_graph(fw, WORKLOADS["metapath_rmat26"])
        try:
            configs.append(one_config(fw, g26, "metapath_rmat26", WORKLOADS["metapath_rmat26"], passes=3, warmup=1))
        finally:
            g26.destroy()
        configs.append({
            "config": CONFIG_OF[HEADLINE], "workload": HEADLINE, "app": wl["app"], "vertices": out["config"]["vertices"],
            "csr_entries": out["config"]["csr_entries"], "queries": n, "walk_steps_per_pass": int(last.steps),
            "passes": args.steps, "device_ms_per_pass": avg_kernel_ms, "steps_per_s": last.steps / (avg_kernel_ms * 1e-3),
            "launches_per_pass": last.launches, "frac": roofline["frac"], "achieved_GBs": roofline["achieved"],
            "bytes_basis": roofline["bytes_basis"], "useful_frac": roofline["useful_frac"],
            "algorithmic_frac": roofline["algorithmic_frac"], "algorithmic_rate_GBs": roofline["algorithmic_rate"],
            "reuse_factor": roofline["reuse_factor"]})
        out["configs"] = configs
        out["node2vec_other_parameters"] = n2v_points
        if cpu is not None:
            out["cpu_baseline"] = cpu
    else:
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline(fw, g, params, starts, args.cpu_seconds)
        g.destroy()
    print(json.dumps(out))


def cpu_baseline(fw, g, params, starts, target_s):
    """Times the CPU oracle (the checker, used here only as the reported baseline) on a prefix of the queries: one
    warm-up run, then the best of three timed runs, wall clock around the walk only (the graph is in host memory);
    the prefix is sized so that the three runs together take about target_s."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import fw_oracle_binding as orc

    labels = params.app == fw.APP_METAPATH
    xadj, adj, w, lab = g.download(weights=not labels, labels=labels)
    og = orc.Graph(xadj, adj, w, lab)
    op = orc.from_walk_params(params)
    cores = orc.lib().fw_oracle_num_threads()
    # warm-up, which also sizes the sample
    pilot = min(len(starts), 4096)
    t = time.perf_counter()
    orc.walk(og, op, starts[:pilot])
    dt = max(time.perf_counter() - t, 1e-4)
    m = int(min(len(starts), max(pilot, pilot * (target_s / 3.0) / dt)))
    best, steps = None, 0
    for _ in range(3):
        t = time.perf_counter()
        _, steps, _ = orc.walk(og, op, starts[:m])
        dt = time.perf_counter() - t
        best = dt if best is None or dt < best else best
    return {
        "value": steps / best, "unit": "steps/s", "cores": int(cores), "kind": "port",
        "sample": "first %d of %d queries of the same workload, %d steps: one warm-up, best of 3 runs %.2f s, OpenMP "
                  "schedule(dynamic)" % (m, len(starts), steps, best),
    }


if __name__ == "__main__":
    main()
