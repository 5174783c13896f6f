"""bench.py's command line without a GPU: more than one GPU is refused with a message that says why."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def _fake_result(n_tried):
    """A result dict shaped like the one bench.main() collects, with a tuning sweep of n_tried settings in it."""
    one = dict(queue=10, qps=911234.5678, qps_min=880000.1234, qps_max=930000.5678, runs=5, recall_at_10=0.99941234,
               entry_points=32768, seed_dims=128, parallel_visit_count=3, speculative_readahead=1, stop="per_query")
    per_loop = [dict(loop=i, avg_launch_ms=0.61234567, algorithmic_bytes_per_launch=3.77e9, frac=0.771234567,
                     achieved_gbs=6170.123456, launches=4900, reference_equivalent_gbs=23456.789,
                     candidate_rows_fetched=0.0581234, candidates_through_the_sketch=0.7241234,
                     traffic_bytes_per_launch=4.18e9, traffic_over_algorithmic=1.1087654,
                     frac_of_peak_by_counter_bytes=0.85123456, build_launches_of_this_loop=24500,
                     build_seconds_of_this_loop=14.5, replayed_batches=20) for i in range(3)]
    sweep = dict(one, seeding="dense", stop="batch", sweep=[dict(one) for _ in range(8)], reached_0_95=True)
    return {
        "metric": "build vecs/s + search QPS @recall@10=0.95, 1M×768 fp32, 1 MI355X", "value": 42718.123456789,
        "unit": "vectors/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 158.7123456, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "mix-1m-768", "n": 1000000, "dim": 768, "degree": 64, "build_queue": 128,
                   "batch_size": 10000, "optimization_loops": 3, "parallel_visit_count": 4, "prune": "reference",
                   "sketch": "x" * 300, "queries": 10000},
        "build_seconds": 23.41, "build_steps": 300, "steps_note": "y" * 400, "loops": [dict(seconds=1.0)] * 3,
        "roofline": dict(bound="hbm", kernel="k" * 200, achieved=4690.123, peak=8000.0, unit="GB/s", frac=0.586265,
                         traffic=2.94e9, traffic_detail=dict(source="s" * 300), copy_gbs_measured=5025.4,
                         gather_gbs_measured={"sequential_4.3GiB": 5123.4, "random_4.3GiB": 5800.1,
                                              "sequential_120MiB": 6900.7, "random_120MiB": 7000.2},
                         avg_launch_ms=0.5123, algorithmic_bytes_per_launch=2.4e9, launches_in_timed_build=47815,
                         method="m" * 500, per_loop=per_loop),
        "exact_knn": dict(seconds=0.126, tflops=121.9, peak_tflops=157.3, frac=0.775, bound="mfma"),
        "search": dict(sweep, roofline=dict(iterations=dict(bound="hbm", launches=25, avg_launch_ms=0.211, frac=0.35),
                                            seeding_tiles=dict(bound="mfma", seconds=0.0046, tflops=108.0, frac=0.69))),
        "search_per_query_stop": dict(sweep, stop="per_query"),
        "search_reference_seeding": dict(sweep, seeding="circulant"),
        "search_tuned": dict(tried=[dict(one) for _ in range(n_tried)], best=dict(one),
                             best_with_the_reference_stop=dict(one, stop="batch")),
        "cpu_baseline": dict(value=457.3, unit="vectors/s", cores=16, kind="port", sample="z" * 1000,
                             all_core=dict(search_qps=774.2), single_thread=dict(threads=1),
                             gpu_same_workload=dict(build_vectors_per_s=327000.0, search_qps=96000.0,
                                                    graph_and_search_ids_equal_the_cpu=True),
                             benchmark_workload_sample=dict(rows=768, seconds=8.5, rows_per_s_first_loop=90.0,
                                                            ids_and_distances_match_gpu=True, sample="w" * 300)),
        "beam_step_launches_by_phase": [dict(phase="p" * 40, beam_step_launches=1)] * 12,
    }


def test_the_printed_line_stays_short_whatever_was_swept():
    """The one line on stdout must survive a capture of a few KB: a 324-setting sweep in the collected result
    leaves it under 3 KB with the contract's keys at the top level."""
    import json

    sys.path.insert(0, ROOT)
    import bench

    line = bench.headline(_fake_result(324))
    text = json.dumps(line)
    assert len(text) < 3072, len(text)
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "search", "exact_knn"):
        assert key in back, key
    assert back["config"]["workload"] == "mix-1m-768" and back["dtype"] == "f32"
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in back["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in back["cpu_baseline"], key
    assert back["search_tuned"]["settings_tried"] == 324 and "tried" not in back["search_tuned"]
    assert "sweep" not in back["search"] and back["search"]["runs"] == 5


def test_traffic_is_read_from_the_committed_profile():
    sys.path.insert(0, ROOT)
    import bench

    (per_loop, source) = bench.traffic_from_profiles("mix-1m-768")
    assert source == os.path.join("profiles", "beam_step_kernel_mix-1m-768_by_phase.txt")
    assert len(per_loop) == 3 and all(1e8 < b < 1e11 for b in per_loop)
    assert bench.traffic_from_profiles("no-such-workload") == (None, None)
