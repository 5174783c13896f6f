"""Writes tests/golden/ann_small.npz: a seeded small workload and what the CPU oracle
answers for it (graph, search queues, pruned table, optimised graph).

    python tests/golden/make_golden.py

The reference ships no tests, fixtures or golden vectors, and it was never imported here
(it needs Numba and a CUDA device at import time); these vectors come from the oracle, whose
functions are pinned by the known-answer and brute-force tests in tests/test_oracle_*.py.
The fixture guards against drift: a CPU test re-derives it from the oracle, a GPU test
compares the HIP path with it without needing the oracle at all.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as orc  # noqa: E402

CONFIG = dict(orc.DEFAULT_CONFIG)
CONFIG.update(beam_size=8, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=300, optimization_loops=2)


def inputs():
    rng = np.random.default_rng(2024)
    centres = rng.standard_normal((12, 20)).astype(np.float32)
    v = centres[rng.integers(0, 12, 700)] + 0.3 * rng.standard_normal((700, 20)).astype(np.float32)
    v = (v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    q = centres[rng.integers(0, 12, 40)] + 0.3 * rng.standard_normal((40, 20)).astype(np.float32)
    q = (q / np.linalg.norm(q, axis=1, keepdims=True)).astype(np.float32)
    return v, q


def outputs(v, q):
    beams, dists = orc.generate_ann(v, CONFIG)
    queue = orc.search(v, beams, q, CONFIG)
    ql = CONFIG["beam_size"] * CONFIG["beam_queue_factor"]
    wide = orc.generate_circulant_beams(v.shape[0], orc.primes(ql))
    wide_d = orc.calculate_distances(v, wide)
    wide, wide_d = orc.queue_sort(wide, wide_d)
    pruned, pruned_d = orc.prune_(wide, wide_d)
    return dict(beams=beams, distances=dists, search_ids=queue.indices[:, :queue.length],
                search_distances=queue.distances[:, :queue.length], wide=wide, wide_distances=wide_d,
                pruned=pruned, pruned_distances=pruned_d, optimized=orc.optimize_graph(wide, CONFIG["beam_size"]))


if __name__ == "__main__":
    v, q = inputs()
    np.savez_compressed(os.path.join(HERE, "ann_small.npz"), vectors=v, queries=q, **outputs(v, q))
    print("wrote", os.path.join(HERE, "ann_small.npz"))
