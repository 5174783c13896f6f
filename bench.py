#!/usr/bin/env python3
"""Benchmark of the ANN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mix-1m-768]

A step is one batch of 10,000 vectors taken through the beam search of the
graph build (closest_vectors) against the current graph.  Whatever K is, the
timed region is the COMPLETE build - every batch of every optimisation loop,
with prune and the per-loop self-recall - run with the library's profiling
hooks off; `value` is N / its wall time.  `steps` / `ms_per_step` describe the
first K steps of that build (K = 0: all of them).  Warm-up steps run on a
throw-away 50,000-vector build and never touch the timed one.

After the build:
  * roofline pass: the first K batches of the state every optimisation loop
    started from are run again with the hooks ON (HIP events around the
    launches on the launch stream, fetched rows counted on the device); the
    per-loop averages are combined with the timed build's launch counts;
  * measured ceilings of the box: a 1 GiB device copy, and the library's own
    gathered-distance kernel over a 4.3 GiB and a 120 MiB table with ids in
    memory order and with uniformly random ids;
  * search leg: exact kNN on MFMA tiles for ground truth, then a sweep of the
    search-queue length; QPS (median of 5 runs timed with HIP events on the
    launch stream) is reported at the shortest queue reaching recall@10 >= 0.95,
    for the parity loop (the reference's batch-wide stop) and for the per-query
    early exit; `--tuned` adds a sweep over the other search settings;
  * CPU leg: the CPU oracle (a port of the reference algorithm, op for op) on
    the 4,096 x 128 workload - all cores: whole build + 256-query search;
    one thread: one 512-row batch + the search - beside the GPU on the same
    workload, and a 768-row sample of the benchmark workload itself.
ONE short JSON line (under 3 KB: the headline, `roofline`, `cpu_baseline`,
`search`, `exact_knn`) goes to stdout, last.  Everything else measured on the
way (per-setting sweeps, per-loop tables, launch counts per phase) is written to
the file `--detail` names, if one is given.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "vectorlink-gpu_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E bandwidth
MFMA_FP32_PEAK = 157.3  # MI355X published dense fp32 matrix TFLOP/s

PROFILE_DIR = os.path.join(ROOT, "profiles")
LINE_LIMIT = 3072       # the one JSON line on stdout stays below this many bytes


def traffic_from_profiles(workload):
    """Bytes moved past L2 per launch of the beam-search step, per optimisation-loop state, read from the committed
    rocprofv3 --pmc summary of this same command (profiles/beam_step_kernel_<workload>_by_phase.txt: FETCH_SIZE and
    WRITE_SIZE in KiB per dispatch, each scaled by what the counter reads for the 1 GiB copy).  NOT measured in this
    run; None when no summary for the workload is committed."""
    path = os.path.join(PROFILE_DIR, f"beam_step_kernel_{workload}_by_phase.txt")
    if not os.path.exists(path):
        return None, None
    fetch_factor = write_factor = None
    section = None
    per_loop = {}
    with open(path) as f:
        for line in f:
            if line.startswith("## FETCH_SIZE"):
                section = "fetch"
            elif line.startswith("## WRITE_SIZE"):
                section = "write"
            m = re.search(r"# calibration: .*-> factor ([0-9.]+)", line)
            if m and section == "fetch":
                fetch_factor = float(m.group(1))
            elif m and section == "write":
                write_factor = float(m.group(1))
            m = re.match(r"roofline pass, state of loop (\d+): FETCH_SIZE ([0-9.]+), WRITE_SIZE ([0-9.]+)", line)
            if m:
                per_loop[int(m.group(1))] = (float(m.group(2)), float(m.group(3)))
    if fetch_factor is None or write_factor is None or not per_loop:
        return None, None
    out = [(per_loop[k][0] * fetch_factor + per_loop[k][1] * write_factor) * 1024.0 for k in sorted(per_loop)]
    return out, os.path.relpath(path, ROOT)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def profile_read(nv, reset=True, enable=1):
    out = (ctypes.c_double * 9)()
    nv.lib().vl_beam_profile(enable, 1 if reset else 0, out)
    keys = ("expand_ms", "merge_ms", "expand_launches", "merge_launches", "evals", "rows", "iterations", "wanted",
            "sketched")
    return dict(zip(keys, list(out)))


def step_roofline(prof, dim, batch_rows):
    """Algorithmic bytes of the beam-search step from the hook counters: 4*dim + 12 per candidate row actually
    fetched and evaluated, a sketch row, its tail and the id (16*ceil(dim/16) + 8 + 4) per candidate looked at through the
    8-bit sketch, plus the query row (4*dim) once per (row, iteration)."""
    launches = max(prof["expand_launches"], 1.0)
    per_eval = 4 * dim + 12
    per_sketch = 16 * ((dim + 15) // 16) + 8 + 4
    q_loads = prof["iterations"] * batch_rows * 4.0 * dim
    algo = prof["evals"] * per_eval + prof["sketched"] * per_sketch + q_loads
    secs = prof["expand_ms"] / 1e3
    gbs = algo / secs / 1e9 if secs > 0 else 0.0
    ref_equiv = (prof["wanted"] * per_eval + q_loads) / secs / 1e9 if secs > 0 else 0.0
    wanted = max(prof["wanted"], 1.0)
    return dict(launches=int(prof["expand_launches"]), avg_launch_ms=prof["expand_ms"] / launches,
                algorithmic_bytes_per_launch=algo / launches, achieved_gbs=gbs, frac=gbs / HBM_PEAK_GBS,
                reference_equivalent_gbs=ref_equiv,
                candidate_rows_fetched=prof["evals"] / wanted,
                candidates_through_the_sketch=prof["sketched"] / wanted,
                distances_served_from_cache=(1.0 - prof["evals"] / wanted) if prof["sketched"] == 0 else None)


def gather_ceilings(torch, dev, dim):
    """The library's own gathered-distance kernel (one distance = one row of 4*dim bytes fetched, an id read, a
    distance written) on a table far beyond the 256 MB memory-side cache (4.3 GiB) and on one inside it (120 MiB),
    with ids in memory order and with uniformly random ids: what this box delivers to that access pattern, best of 3."""
    from vectorlink_gpu.kernels import gather_distances

    width = 64
    out = {}
    for (label, rows) in (("4.3GiB", int(4.3 * 2**30) // (4 * dim)), ("120MiB", 120 * 2**20 // (4 * dim))):
        table = torch.empty((rows, dim), dtype=torch.float32, device=dev).normal_()
        n_q = min(max(rows // width, 16384), 65536)
        queries = table[:n_q].contiguous()
        g = torch.Generator(device="cpu").manual_seed(5)
        order = (torch.arange(n_q * width, dtype=torch.int64) % rows).to(torch.int32).view(n_q, width)
        rand = torch.randint(0, rows, (n_q, width), generator=g, dtype=torch.int32)
        for (kind, ids) in (("sequential", order.to(dev)), ("random", rand.to(dev))):
            res = torch.empty((n_q, width), dtype=torch.float32, device=dev)
            gather_distances(queries, table, ids, res)
            torch.cuda.synchronize()
            best = None
            for _ in range(3):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                gather_distances(queries, table, ids, res)
                b.record()
                torch.cuda.synchronize()
                ms = a.elapsed_time(b)
                best = ms if best is None or ms < best else best
            out[f"{kind}_{label}"] = n_q * width * (4.0 * dim + 12) / (best / 1e3) / 1e9
        del table, queries
    return out


def measured_copy_gbs(torch, dev):
    """Bandwidth of a plain 1 GiB device-to-device copy (read + write = 2 GiB moved), best of 5."""
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    best = None
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        dst.copy_(src)
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b)
        best = ms if best is None or ms < best else best
    del src, dst
    return 2.0 * (1 << 30) / (best / 1e3) / 1e9


class Phases:
    """Beam-search launches per phase of this run, in order, so that a profiler's list of beam-search step
    dispatches (beam_step_*, beam_window_*) can be cut into the same phases."""

    def __init__(self):
        from vectorlink_gpu import _native as nv

        self.count = nv.lib().vl_beam_launches
        self.rows, self.last = [], self.count()

    def mark(self, name):
        now = self.count()
        self.rows.append(dict(phase=name, beam_step_launches=now - self.last))
        self.last = now


def recall_at(found, truth):
    hits = (found.unsqueeze(2) == truth.unsqueeze(1)).any(dim=2).sum().item()
    return hits / truth.numel()


def cpu_leg(torch, dev, base_c3, cfg_c3, cpu_rows, gpu_c3_batch):
    """The CPU oracle as the reported CPU baseline (test infrastructure, timed here as the checker's own speed)."""
    from oracle import oracle as orc
    from vectorlink_gpu import ANN, synthetic

    cores = os.cpu_count() or 1
    threads = min(16, cores)
    out = dict(unit="vectors/s", kind="port", cpu_count=cores)

    # ---- the 4,096 x 128 workload, whole: build (all cores), 256-query top-10 search ----
    base, queries, w = synthetic.make("iid-4k-128")
    cfg = dict(orc.DEFAULT_CONFIG)
    cfg.update(synthetic.ann_kwargs(w))
    v, q = base.numpy(), queries.numpy()
    n = v.shape[0]
    orc.set_threads(threads)
    t0 = time.time()
    trace = []
    (ob, od) = orc.generate_ann(v, cfg, trace=trace)
    t_build = time.time() - t0
    t0 = time.time()
    res = orc.search(v, ob, q, cfg)
    t_search = time.time() - t0
    (truth, _) = orc.knn_exact(q, v, 10)
    import numpy as np

    cpu_recall = float(np.mean([len(set(res.indices[i, :10]) & set(truth[i])) / 10.0 for i in range(q.shape[0])]))
    all_core = dict(threads=threads, build_seconds=t_build, build_vectors_per_s=n / t_build,
                    optimisation_loops_run=len({t[0] for t in trace}), search_seconds=t_search,
                    search_qps=q.shape[0] / t_search, recall_at_10=cpu_recall)
    # ---- one thread: one batch of 512 rows of the first loop, and the search ----
    orc.set_threads(1)
    rows = 512
    ql = cfg["beam_size"] * cfg["beam_queue_factor"]
    b0 = orc.generate_circulant_beams(n, orc.primes(ql))
    d0 = orc.gather_distances(v[:rows], v, b0[:rows])
    oq = orc.Queue(rows, ql, ql + ql * cfg["parallel_visit_count"])
    oq.insert(b0[:rows], d0)
    t0 = time.time()
    orc.closest_vectors(v[:rows], oq, v, b0, cfg, orc.excluding_self(0, rows))
    t_rows = time.time() - t0
    t0 = time.time()
    orc.search(v, ob, q, cfg)
    t_search1 = time.time() - t0
    single = dict(threads=1, build_rows_per_s_first_loop=rows / t_rows,
                  build_sample=f"rows [0,{rows}) of the first optimisation loop in {t_rows:.1f} s (a loop takes "
                               f"every row through the same search; this build ran {all_core['optimisation_loops_run']} loop(s))",
                  search_seconds=t_search1, search_qps=q.shape[0] / t_search1)
    orc.set_threads(threads)
    # ---- the GPU on the same workload ----
    vd, qd = base.to(dev), queries.to(dev)
    kw = synthetic.ann_kwargs(w)
    ANN(vd, **kw)  # warm the shapes
    torch.cuda.synchronize()
    t0 = time.time()
    ann = ANN(vd, **kw)
    torch.cuda.synchronize()
    g_build = time.time() - t0
    ann.search(qd)
    torch.cuda.synchronize()
    t0 = time.time()
    gres = ann.search(qd)
    torch.cuda.synchronize()
    g_search = time.time() - t0
    same = bool(np.array_equal(ann.beams.cpu().numpy(), ob)
                and np.array_equal(gres.indices[:, :res.length].cpu().numpy(), res.indices[:, :res.length]))
    gpu = dict(build_seconds=g_build, build_vectors_per_s=n / g_build, search_seconds=g_search,
               search_qps=q.shape[0] / g_search, graph_and_search_ids_equal_the_cpu=same)
    out.update(value=all_core["build_vectors_per_s"], cores=threads,
               sample=f"iid-4k-128 whole (4,096 x 128, degree 32, queue 64; build + 256-query top-10 search) on "
                      f"{threads} of {cores} host cores: build {t_build:.1f} s, search {t_search:.2f} s",
               all_core=all_core, single_thread=single, gpu_same_workload=gpu)

    # ---- a sample of the benchmark workload itself: rows [0, cpu_rows) of the first loop ----
    if base_c3 is not None and cpu_rows > 0:
        v3 = base_c3.numpy()
        n3 = v3.shape[0]
        ql3 = cfg_c3["beam_size"] * cfg_c3["beam_queue_factor"]
        b3 = orc.generate_circulant_beams(n3, orc.primes(ql3))
        d3 = orc.gather_distances(v3[:cpu_rows], v3, b3[:cpu_rows])
        q3 = orc.Queue(cpu_rows, ql3, ql3 + ql3 * cfg_c3["parallel_visit_count"])
        q3.insert(b3[:cpu_rows], d3)
        t0 = time.time()
        iters = orc.closest_vectors(v3[:cpu_rows], q3, v3, b3, cfg_c3, orc.excluding_self(0, cpu_rows))
        dt = time.time() - t0
        (gi, gd) = gpu_c3_batch(cpu_rows)
        ok = bool((q3.indices[:, :ql3] == gi).all() and (q3.distances[:, :ql3] == gd).all())
        out["benchmark_workload_sample"] = dict(
            threads=threads, rows=cpu_rows, iterations=int(iters), seconds=dt, rows_per_s_first_loop=cpu_rows / dt,
            sample=f"rows [0,{cpu_rows}) of the benchmark workload against the initial circulant graph",
            ids_and_distances_match_gpu=ok)
    return out


def _r(x, digits=4):
    """Numbers of the printed line carry a few significant digits only."""
    if isinstance(x, float):
        return float(f"{x:.{digits}g}")
    return x


def _pick(d, keys, digits=4):
    return {k: _r(d[k], digits) for k in keys if d is not None and k in d and d[k] is not None}


def headline(result):
    """The ONE line for stdout, from everything a run measured: the contract's keys, `roofline`, `cpu_baseline`,
    `search`, `exact_knn`, a few figures each - never a sweep.  Stays under LINE_LIMIT bytes whatever `result` holds."""
    line = {k: _r(result[k], 6) for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                          "higher_is_better", "scaling", "vs_baseline", "dtype", "data") if k in result}
    line["config"] = _pick(result.get("config", {}), ("workload", "n", "dim", "degree", "build_queue", "batch_size",
                                                      "optimization_loops", "parallel_visit_count", "prune",
                                                      "concurrent_batches", "queries", "search_seeding"))
    line.update(_pick(result, ("build_seconds", "build_steps")))
    rf = result.get("roofline")
    if rf is not None:
        out = {k: rf.get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
        out = {k: _r(v) for k, v in out.items()}
        out["kernel"] = "beam_step"
        out["scope"] = "algorithmic bytes / published HBM peak; served beyond L2"
        out.update(_pick(rf, ("avg_launch_ms", "algorithmic_bytes_per_launch", "launches_in_timed_build",
                              "copy_gbs_measured")))
        if rf.get("in_timed_build"):
            out["in_timed_build"] = _pick(rf["in_timed_build"], ("achieved", "frac", "batches_in_flight"), 3)
        if rf.get("gather_gbs_measured"):
            out["gather_gbs_measured"] = {k: _r(v, 3) for k, v in rf["gather_gbs_measured"].items()}
        out["per_loop"] = [_pick(r, ("loop", "avg_launch_ms", "algorithmic_bytes_per_launch", "frac",
                                     "traffic_over_algorithmic", "build_launches_of_this_loop"), 3)
                           for r in rf.get("per_loop", [])][:4]
        line["roofline"] = out
    search_keys = ("seeding", "stop", "queue", "qps", "qps_min", "qps_max", "runs", "recall_at_10", "reached_0_95")
    short_keys = ("seeding", "stop", "queue", "qps", "recall_at_10")
    for name in ("search", "search_full_rank_seeds", "search_per_query_stop", "search_reference_seeding"):
        if name in result:
            line[name] = _pick(result[name], search_keys if name == "search" else short_keys)
    sr = (result.get("search") or {}).get("roofline")
    if sr:
        line["search"]["iterations"] = _pick(sr["iterations"], ("launches", "avg_launch_ms", "frac"), 3)
        line["search"]["seeding_tiles"] = _pick(sr["seeding_tiles"], ("seconds", "tflops", "frac"), 3)
    tuned = result.get("search_tuned")
    if tuned:
        keys = short_keys + ("entry_points", "seed_dims", "parallel_visit_count", "speculative_readahead")
        line["search_tuned"] = dict(settings_tried=len(tuned.get("tried", [])), best=_pick(tuned.get("best"), keys),
                                    best_with_the_reference_stop=_pick(tuned.get("best_with_the_reference_stop"), keys))
    if "exact_knn" in result:
        line["exact_knn"] = _pick(result["exact_knn"], ("bound", "seconds", "tflops", "peak_tflops", "frac"))
    cb = result.get("cpu_baseline")
    if cb is not None:
        out = {k: _r(cb.get(k)) for k in ("value", "unit", "cores", "kind")}
        out["sample"] = str(cb.get("sample", ""))[:200]
        if "all_core" in cb:
            out["search_qps"] = _r(cb["all_core"].get("search_qps"))
        if "gpu_same_workload" in cb:
            out["gpu_same_workload"] = _pick(cb["gpu_same_workload"], ("build_vectors_per_s", "search_qps",
                                                                       "graph_and_search_ids_equal_the_cpu"))
        if "benchmark_workload_sample" in cb:
            out["benchmark_workload_sample"] = _pick(cb["benchmark_workload_sample"],
                                                     ("rows", "seconds", "rows_per_s_first_loop",
                                                      "ids_and_distances_match_gpu"))
        line["cpu_baseline"] = out
    text = json.dumps(line)
    if len(text) >= LINE_LIMIT:   # never happens with the keys above; if it ever does, the optional parts go first
        for k in ("search_reference_seeding", "search_full_rank_seeds", "search_per_query_stop", "search_tuned"):
            line.pop(k, None)
            if len(json.dumps(line)) < LINE_LIMIT:
                break
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20,
                    help="batch steps that `ms_per_step` describes and that the roofline pass replays per loop "
                         "(0 = all); the build itself always runs whole")
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="mix-1m-768")
    ap.add_argument("--n", type=int, default=None, help="override the number of vectors")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-search", action="store_true", help="skip the search leg")
    ap.add_argument("--tuned", action="store_true",
                    help="also sweep the other search settings (entry points, columns ranked, nodes visited per "
                         "iteration, progress-check cadence, stop): a few hundred searches; off by default")
    ap.add_argument("--no-tuned", action="store_true", help="accepted for older command lines; the sweep is off by default")
    ap.add_argument("--search-runs", type=int, default=5, help="timed runs per search setting (the median is reported)")
    ap.add_argument("--seed-dims", type=int, default=-1,
                    help="the dense seeding of the search leg ranks its 32,768 entry points by their first this many "
                         "columns (0 = all; seeds only have to land near the query); the all-column figure is reported "
                         "beside it as search_full_rank_seeds.  Default: 64 for rows of 512 columns or more, else 128 "
                         "(measured at 1M x 768, reference stop, recall@10 0.9994 throughout: 128 columns 1.69, "
                         "96 1.74, 64 1.81, 48 1.82 M QPS, 32 columns 1.86 M at 0.9988; at 1M x 128 all 128 columns "
                         "beat 64: 1.47 against 1.07 M QPS)")
    ap.add_argument("--seeds", type=int, default=-1,
                    help="nearest entry points a query of the search leg starts from (0 = as many as its queue holds, "
                         "16 at most).  Default: 4 for rows of 512 columns or more, else 0.  Measured with the "
                         "reference stop at 1M x 768, recall@10 0.9994 throughout: 10 seeds 1.80, 8 1.84, 4 1.90, "
                         "2 1.92, 1 seed 1.97 M QPS; at 1M x 128 (recall@10 0.83 either way) 10 seeds 1.47, 4 seeds "
                         "1.05 M QPS: there a batch waits longer for its slowest query when it starts from fewer")
    ap.add_argument("--queues", default="10,16,32,64,96,128,192,256",
                    help="search-queue lengths swept in this order (the sweep stops at the first that reaches recall@10 0.95)")
    ap.add_argument("--no-reference-seeding", action="store_true",
                    help="skip the search sweep with the reference's circulant seeds")
    ap.add_argument("--detail", default=None,
                    help="write everything measured (sweeps, per-loop tables, launches per phase) to this JSON file")
    ap.add_argument("--knn-only", action="store_true",
                    help="only the dense MFMA tiles on this workload's vectors (exact kNN of the queries, and the "
                         "seeding pass over 32,768 entry points); prints their figures as the JSON line")
    ap.add_argument("--cpu-rows", type=int, default=768)
    ap.add_argument("--loops", type=int, default=3, help="optimisation loops of the build (the reference's default is 3)")
    ap.add_argument("--concurrent-batches", type=int, default=3,
                    help="batches of an optimisation loop kept in flight by the timed build (streams / host threads)")
    ap.add_argument("--no-sketch", action="store_true",
                    help="build without the 8-bit sketch of the vectors (every candidate row of the first loop is "
                         "fetched whole, as before the sketch existed; the graph is the same)")
    ap.add_argument("--prune", choices=["reference", "rank", "none"], default="reference",
                    help="reference = prune_ between loops as the reference does (default); rank = detour-count "
                         "cut with reverse edges at the end (an addition); none = no pruning")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch

    from vectorlink_gpu import _native as nv
    from vectorlink_gpu import synthetic
    from vectorlink_gpu.ann import ANN, GraphBuild
    from vectorlink_gpu.kernels import knn_exact

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    nv.lib()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")

    t0 = time.time()
    base, queries, w = synthetic.make(args.workload, n=args.n)
    n, dim = base.shape
    log(f"[bench] workload {args.workload}: {n} x {dim}, generated in {time.time() - t0:.1f} s")
    kwargs = synthetic.ann_kwargs(w)
    cfg = dict(prune={"reference": True, "rank": "rank", "none": False}[args.prune], parallel_visit_count=4,
               visit_queue_factor=3, exclude_factor=5, optimization_loops=args.loops, batch_size=10_000,
               speculative_readahead=5, **kwargs)
    if args.no_sketch:
        cfg["sketch"] = False
    vectors = base.to(dev)
    qdev = queries.to(dev)
    torch.cuda.synchronize()

    if args.knn_only:
        out = {"metric": "dense distance tiles (fp32 MFMA), TFLOP/s", "unit": "TFLOP/s", "n_gpus": 1,
               "higher_is_better": True, "dtype": "f32", "data": "synthetic",
               "config": {"workload": args.workload, "n": n, "dim": dim, "queries": int(qdev.shape[0])}}
        from vectorlink_gpu.ann import entry_point_ids
        entries = vectors[entry_point_ids(n, 32_768, dev).long()].contiguous()
        for (name, table, k) in (("exact_knn", vectors, 10), ("seeding_tiles", entries, 16)):
            knn_exact(qdev, table, k)
            torch.cuda.synchronize()
            reps = max(1, args.steps // 4)
            t0 = time.time()
            for _ in range(reps):
                knn_exact(qdev, table, k)
            torch.cuda.synchronize()
            dt = (time.time() - t0) / reps
            flops = 2.0 * qdev.shape[0] * table.shape[0] * dim
            out[name] = dict(bound="mfma", vectors=int(table.shape[0]), k=k, seconds=dt, tflops=flops / dt / 1e12,
                             peak_tflops=MFMA_FP32_PEAK, frac=flops / dt / 1e12 / MFMA_FP32_PEAK, calls=reps + 1)
        out["value"] = out["exact_knn"]["tflops"]
        out["roofline"] = dict(bound="mfma", achieved=out["exact_knn"]["tflops"], peak=MFMA_FP32_PEAK, unit="TFLOP/s",
                               frac=out["exact_knn"]["frac"], traffic=None)
        print(json.dumps(out))
        return

    phases = Phases()
    # warm-up: a small separate build (kernels loaded, allocator primed)
    if args.warmup > 0:
        wb = GraphBuild(vectors[:50_000].contiguous(), cfg)
        for i, _ in enumerate(wb.steps()):
            if i + 1 >= args.warmup:
                break
        torch.cuda.synchronize()
        del wb
    phases.mark("warm-up")

    copy_gbs = measured_copy_gbs(torch, dev)
    gather_gbs = gather_ceilings(torch, dev, dim)
    log(f"[bench] 1 GiB device copy: {copy_gbs:.0f} GB/s; gathered distances (GB/s): "
        + ", ".join(f"{k} {v:.0f}" for k, v in gather_gbs.items()))

    # ---- the timed build: whole, hooks off ----
    profile_read(nv, reset=True, enable=0)
    torch.cuda.synchronize()
    t_start = time.time()
    build = GraphBuild(vectors, cfg, keep_history=True, concurrent_batches=args.concurrent_batches)
    total_steps = build.batches_per_loop() * cfg["optimization_loops"]
    k_steps = args.steps if 0 < args.steps < total_steps else total_steps
    done = 0
    t_first_k = None
    t_said = t_start
    in_loop = 0
    for (loop, start, end, iters) in build.steps():
        if loop != in_loop:
            phases.mark(f"build loop {in_loop} (with its self-recall search)")
            in_loop = loop
        done += 1
        if done == k_steps:
            t_first_k = time.time() - t_start   # closest_vectors returns after a stream synchronisation
        if time.time() - t_said > 30.0:   # a long build keeps talking
            t_said = time.time()
            log(f"[bench] build: step {done} of {total_steps}, loop {loop}, {t_said - t_start:.0f} s")
    phases.mark(f"build loop {in_loop} (with its self-recall search)")
    (beams, dists) = build.result()
    torch.cuda.synchronize()
    t_build = time.time() - t_start
    if t_first_k is None:
        (k_steps, t_first_k) = (done, t_build)
    value = n / t_build
    log(f"[bench] build: {done} steps in {t_build:.1f} s -> {value:.0f} vectors/s; seconds per loop: "
        + ", ".join(f"{st['seconds']:.1f}" for st in build.stats))

    # ---- roofline pass: the first batches of every loop's starting state again, hooks on ----
    batch_rows = min(cfg["batch_size"], n)
    replay = min(k_steps, build.batches_per_loop())
    per_loop = []
    for li, tables in enumerate(build.history):
        profile_read(nv, reset=True, enable=1)
        # one launch at a time under the events; the first loop starts from the circulant graph, as in the build
        rb = GraphBuild(vectors, cfg, initial=tables if li > 0 else None, concurrent_batches=1)
        for i, _ in enumerate(rb.steps()):
            if i + 1 >= replay:
                break
        torch.cuda.synchronize()
        r = step_roofline(profile_read(nv, reset=True, enable=0), dim, batch_rows)
        phases.mark(f"roofline pass, state of loop {li}")
        r.update(loop=li, replayed_batches=replay, build_launches_of_this_loop=int(build.stats[li]["iterations"]),
                 build_seconds_of_this_loop=build.stats[li]["seconds"])
        per_loop.append(r)
        del rb
    weights = [r["build_launches_of_this_loop"] for r in per_loop]
    w_time = sum(wt * r["avg_launch_ms"] for wt, r in zip(weights, per_loop))
    w_bytes = sum(wt * r["algorithmic_bytes_per_launch"] for wt, r in zip(weights, per_loop))
    w_launch = max(sum(weights), 1)
    achieved = w_bytes / (w_time / 1e3) / 1e9 if w_time > 0 else 0.0
    (per_loop_traffic, traffic_file) = traffic_from_profiles(args.workload)
    traffic = traffic_detail = None
    if per_loop_traffic and len(per_loop_traffic) >= len(per_loop) and args.n is None:
        traffic = sum(wt * tb for wt, tb in zip(weights, per_loop_traffic)) / w_launch
        for tb, r in zip(per_loop_traffic, per_loop):
            r["traffic_bytes_per_launch"] = tb
            r["traffic_over_algorithmic"] = tb / max(r["algorithmic_bytes_per_launch"], 1.0)
            # where the counter shows fewer bytes leaving L2 than the algorithm asks for, part of them are L2 hits:
            # the HBM-side rate is the counter's bytes over the launch time
            r["frac_of_peak_by_counter_bytes"] = tb / (r["avg_launch_ms"] / 1e3) / 1e9 / HBM_PEAK_GBS
        traffic_detail = dict(
            source=f"{traffic_file} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, committed); "
                   "not measured in this run",
            bytes_per_launch_by_loop=per_loop_traffic[:len(per_loop)])
    roofline = dict(
        bound="hbm",
        kernel="beam_step_kernel (one beam-search iteration: gathered cosine distances + queue merge per row)",
        achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS,
        frac_scope="algorithmic bytes over the published HBM peak; the bytes are served by the path beyond L2 "
                   "(memory-side cache + HBM), see gather_gbs_measured for what that path delivers on this box",
        traffic=traffic, traffic_detail=traffic_detail,
        copy_gbs_measured=copy_gbs, frac_of_measured_copy=achieved / copy_gbs if copy_gbs > 0 else None,
        gather_gbs_measured=gather_gbs,
        avg_launch_ms=w_time / w_launch, algorithmic_bytes_per_launch=w_bytes / w_launch,
        launches_in_timed_build=int(sum(weights)),
        # the same bytes over the wall time of the timed build's loops (everything a loop does included): with
        # several batches in flight one batch's launch runs on the compute units that the last workgroups of
        # another's leave idle, which a launch timed alone cannot show
        in_timed_build=dict(achieved=w_bytes / max(sum(st["seconds"] for st in build.stats[:len(per_loop)]), 1e-9) / 1e9,
                            frac=w_bytes / max(sum(st["seconds"] for st in build.stats[:len(per_loop)]), 1e-9) / 1e9
                                 / HBM_PEAK_GBS,
                            batches_in_flight=args.concurrent_batches),
        method=f"hooks are off in the timed build; the first {replay} batches of the tables each optimisation loop "
               "started from were run again with HIP events around the launches (on the launch stream) and the fetched "
               "rows counted on the device; per-loop averages below, combined here with the timed build's launch counts",
        per_loop=per_loop)
    log(f"[bench] roofline: {achieved:.0f} GB/s = {achieved / HBM_PEAK_GBS:.3f} of peak; per loop: "
        + ", ".join(f"{r['avg_launch_ms']:.3f} ms {r['frac']:.3f}" for r in per_loop))

    result = {
        "metric": "build vecs/s + search QPS @recall@10=0.95, 1M×768 fp32, 1 MI355X",
        "value": value, "unit": "vectors/s", "n_gpus": 1, "steps": k_steps, "warmup": args.warmup,
        "ms_per_step": t_first_k * 1e3 / max(k_steps, 1), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "n": n, "dim": dim, "degree": cfg["beam_size"],
                   "build_queue": cfg["beam_size"] * cfg["beam_queue_factor"], "batch_size": cfg["batch_size"],
                   "optimization_loops": cfg["optimization_loops"], "parallel_visit_count": 4,
                   "prune": args.prune, "build_seeding": "circulant (reference)",
                   "concurrent_batches": args.concurrent_batches,
                   "sketch": "8-bit sketch of the vectors decides which candidate rows the first loop fetches; "
                             "graph bit-identical" if build.sketch is not None else "none",
                   "sketch_bytes": int(build.sketch.numel()) if build.sketch is not None else 0,
                   "search_seeding": "dense, 32768 entry points", "queries": int(queries.shape[0])},
        "partial": False, "build_seconds": t_build, "build_steps": done,
        "steps_note": f"value = n / build_seconds over all {done} steps (hooks off); steps and ms_per_step describe "
                      f"the first {k_steps} of them",
        "loops": build.stats, "roofline": roofline,
    }

    if not args.no_search:
        ann = ANN(vectors, beams=beams, distances=dists, **{k: v for k, v in cfg.items()})
        knn_exact(qdev[:256].contiguous(), vectors, 10)
        torch.cuda.synchronize()
        t0 = time.time()
        (truth, _) = knn_exact(qdev, vectors, 10)
        torch.cuda.synchronize()
        t_knn = time.time() - t0
        flops = 2.0 * qdev.shape[0] * n * dim
        result["exact_knn"] = dict(seconds=t_knn, tflops=flops / t_knn / 1e12, peak_tflops=MFMA_FP32_PEAK,
                                   frac=flops / t_knn / 1e12 / MFMA_FP32_PEAK, bound="mfma")
        log(f"[bench] exact kNN: {t_knn:.3f} s = {result['exact_knn']['tflops']:.1f} TFLOP/s")

        def one_search(qs, seeding, mode, runs=args.search_runs):
            """Median of `runs` whole searches of all queries, each between two HIP events on the launch stream
            (the search's own progress checks synchronise the host in between, as in any use of it)."""
            ann.search(qdev[:256].contiguous(), queue_size=qs, seeding=seeding, stop=mode)  # warm this shape
            torch.cuda.synchronize()
            times = []
            for _ in range(runs):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                res = ann.search(qdev, queue_size=qs, seeding=seeding, stop=mode)
                b.record()
                torch.cuda.synchronize()
                times.append(a.elapsed_time(b) / 1e3)
            times.sort()
            nq = qdev.shape[0]
            return dict(queue=qs, qps=nq / times[len(times) // 2], qps_min=nq / times[-1], qps_max=nq / times[0],
                        runs=runs, recall_at_10=recall_at(res.indices[:, :10], truth))

        def sweep_search(seeding, mode):
            sweep, chosen = [], None
            for qs in [int(x) for x in args.queues.split(",")]:
                sweep.append(one_search(qs, seeding, mode))
                if chosen is None and sweep[-1]["recall_at_10"] >= 0.95:
                    chosen = sweep[-1]
                    break   # the shortest queue that reaches the target is the one reported
            best = chosen or max(sweep, key=lambda r: r["recall_at_10"])
            log(f"[bench] search: {seeding} seeds, {mode} stop: " + "; ".join(
                f"queue {r['queue']} {r['qps'] / 1e3:.0f}k QPS recall {r['recall_at_10']:.4f}" for r in sweep))
            return dict(seeding=seeding, stop=mode, sweep=sweep, reached_0_95=chosen is not None, **best)

        # query-dependent seeds from dense MFMA tiles over 32,768 entry points (what reaches the recall target);
        # "batch" = the reference's stop (the whole batch runs until no row changed), bit-exact against the oracle
        wanted_seeds = args.seeds if args.seeds >= 0 else (4 if dim >= 512 else 0)
        ann.dense_seeds = wanted_seeds if wanted_seeds > 0 else None
        wanted_dims = args.seed_dims if args.seed_dims >= 0 else (64 if dim >= 512 else 128)
        seed_dims = wanted_dims if 0 < wanted_dims < dim else None
        if seed_dims is not None:
            result["search_full_rank_seeds"] = sweep_search("dense", "batch")
            ann.seed_dims, ann._entry = seed_dims, None
        result["config"]["search_seeding"] = ("dense, 32768 entry points"
                                              + (f" ranked by their first {seed_dims} columns" if seed_dims else "")
                                              + (f", {ann.dense_seeds} seeds per query" if ann.dense_seeds else ""))
        result["search"] = sweep_search("dense", "batch")
        # rows that are quiet stop expanding on their own (an addition; not bit-exact against the reference)
        result["search_per_query_stop"] = sweep_search("dense", "per_query")
        # the reference's query-independent circulant seeds, for comparison
        if not args.no_reference_seeding:
            result["search_reference_seeding"] = sweep_search("circulant", "batch")
        # roofline of the search iterations and of the seeding tiles at the reported queue length
        qs = result["search"]["queue"]
        profile_read(nv, reset=True, enable=1)
        ann.search(qdev, queue_size=qs, seeding="dense")
        torch.cuda.synchronize()
        sr = step_roofline(profile_read(nv, reset=True, enable=0), dim, qdev.shape[0])
        (entry_ids, entry_vectors) = ann._entry_tables()
        ranked_by = qdev if entry_vectors.shape[1] == dim else qdev[:, :entry_vectors.shape[1]].contiguous()
        k_seed = min(ann.dense_seeds or 16, 16, qs)  # what dense_search_queue asks of the tiles
        knn_exact(ranked_by, entry_vectors, k_seed)
        torch.cuda.synchronize()
        t0 = time.time()
        knn_exact(ranked_by, entry_vectors, k_seed)
        torch.cuda.synchronize()
        t_seed = time.time() - t0
        seed_flops = 2.0 * qdev.shape[0] * entry_vectors.shape[0] * entry_vectors.shape[1]
        result["search"]["roofline"] = dict(
            iterations=dict(bound="hbm", queue=qs, **sr),
            seeding_tiles=dict(bound="mfma", seconds=t_seed, tflops=seed_flops / t_seed / 1e12,
                               frac=seed_flops / t_seed / 1e12 / MFMA_FP32_PEAK,
                               entry_points=int(entry_vectors.shape[0])))
        # the same graph searched with other settings of the additions (entry points of the dense seeding, queue
        # length, how often progress is checked, which stop): the fastest of them that still reaches recall@10 >= 0.95
        tuned = []
        keep = (ann.entry_points, ann.configuration["speculative_readahead"], ann.seed_dims,
                ann.configuration["parallel_visit_count"])
        seen_settings = set()
        for entry_points in (32_768, 16_384, 8_192) if args.tuned else ():
            for seed_dims in (None, 256 if dim > 256 else None, 128 if dim > 128 else None):
                if (entry_points, seed_dims) in seen_settings:
                    continue
                seen_settings.add((entry_points, seed_dims))
                for visit in (2, 3, 4):
                    for readahead in (1, 2, 5):
                        for qs in (10, 16):
                            for mode in ("batch", "per_query"):
                                ann.entry_points, ann.seed_dims, ann._entry = entry_points, seed_dims, None
                                ann.configuration["speculative_readahead"] = readahead
                                ann.configuration["parallel_visit_count"] = visit
                                r = one_search(qs, "dense", mode, runs=3)
                                r.update(entry_points=entry_points, seed_dims=seed_dims, parallel_visit_count=visit,
                                         speculative_readahead=readahead, stop=mode)
                                tuned.append(r)
            log(f"[bench] search sweep: {len(tuned)} settings tried")
        ok = [r for r in tuned if r["recall_at_10"] >= 0.95]
        winners = dict(best=max(ok, key=lambda r: r["qps"]) if ok else None,
                       best_with_the_reference_stop=max((r for r in ok if r["stop"] == "batch"),
                                                        key=lambda r: r["qps"], default=None))
        for w_ in winners.values():
            if w_ is None or "iterations_roofline" in w_:
                continue
            # the winner once more with the hooks on: what its iterations fetch and how fast
            ann.entry_points, ann.seed_dims, ann._entry = w_["entry_points"], w_["seed_dims"], None
            ann.configuration["speculative_readahead"] = w_["speculative_readahead"]
            ann.configuration["parallel_visit_count"] = w_["parallel_visit_count"]
            profile_read(nv, reset=True, enable=1)
            ann.search(qdev, queue_size=w_["queue"], seeding="dense", stop=w_["stop"])
            torch.cuda.synchronize()
            w_["iterations_roofline"] = dict(bound="hbm", **step_roofline(profile_read(nv, reset=True, enable=0), dim,
                                                                          qdev.shape[0]))
        (ann.entry_points, ann.configuration["speculative_readahead"], ann.seed_dims,
         ann.configuration["parallel_visit_count"]) = keep
        ann._entry = None
        if args.tuned:
            result["search_tuned"] = dict(tried=tuned, **winners)
            log(f"[bench] search (tuned): {winners['best']}")
        phases.mark("search leg")

    if not args.no_cpu:
        def gpu_c3_batch(n_rows):
            from vectorlink_gpu.ann import closest_vectors, excluding_self
            from vectorlink_gpu.queue import Queue

            ql = cfg["beam_size"] * cfg["beam_queue_factor"]
            (b0, d0) = build.history[0]
            gq = Queue(n_rows, ql, ql + ql * cfg["parallel_visit_count"], device=dev)
            gq.insert(b0[:n_rows], d0[:n_rows])
            closest_vectors(vectors[:n_rows], gq, vectors, b0, cfg, excluding_self(0, n_rows, device=dev))
            return gq.indices[:, :ql].cpu().numpy(), gq.distances[:, :ql].cpu().numpy()

        try:
            result["cpu_baseline"] = cpu_leg(torch, dev, base, cfg, min(args.cpu_rows, n), gpu_c3_batch)
        except Exception as e:  # the CPU leg must never take the GPU numbers down with it
            result["cpu_baseline"] = dict(value=None, unit="vectors/s", cores=0, kind="port", sample=f"failed: {e!r}")

    phases.mark("CPU leg (the GPU's side of its comparisons)")
    result["beam_step_launches_by_phase"] = phases.rows
    if args.detail:
        os.makedirs(os.path.dirname(os.path.abspath(args.detail)), exist_ok=True)
        with open(args.detail, "w") as f:
            json.dump(result, f, indent=1)
    print(json.dumps(headline(result)), flush=True)


if __name__ == "__main__":
    main()
