"""Pins for the oracle's beam search and build drivers (CPU only): the C loop
against the statement-by-statement Python loop, invariants, and brute force on
graphs small enough to reason about."""
import numpy as np
import pytest

from oracle import oracle as orc

M = orc.MAXINT
F = orc.MAXFLOAT


def unit(rng, n, d):
    v = rng.standard_normal((n, d)).astype(np.float32)
    return v / np.linalg.norm(v, axis=1, keepdims=True)


def cfg(**kw):
    c = dict(orc.DEFAULT_CONFIG)
    c.update(kw)
    return c


def build_queue(v, beams, d, start, end, ql, pv):
    q = orc.Queue(end - start, ql, ql + ql * pv)
    q.insert(beams[start:end], d[start:end])
    return q


@pytest.mark.parametrize("n,dim,beam,bqf,pv,vqf,ef,ra", [
    (64, 8, 4, 2, 2, 3, 5, 5),
    (200, 16, 6, 3, 4, 3, 5, 5),
    (150, 12, 5, 2, 3, 2, 1, 2),   # tiny visited list: exhausts and stops feeding
    (90, 10, 2, 2, 4, 1, 2, 3),    # visit queue shorter than the visit count
])
def test_c_loop_equals_python_loop(n, dim, beam, bqf, pv, vqf, ef, ra):
    rng = np.random.default_rng(n)
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, visit_queue_factor=vqf,
            exclude_factor=ef, speculative_readahead=ra)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    qa = build_queue(v, beams, d, 10, n - 5, ql, pv)
    qb = build_queue(v, beams, d, 10, n - 5, ql, pv)
    ex = orc.excluding_self(10, n - 5)
    ta = orc.closest_vectors(v[10:n - 5], qa, v, beams, c, ex)
    tb = orc.closest_vectors_py(v[10:n - 5], qb, v, beams, c, ex)
    assert ta == tb and ta % ra == 0
    assert np.array_equal(qa.indices, qb.indices)
    assert np.array_equal(qa.distances.view(np.uint32), qb.distances.view(np.uint32))
    # queue prefix: sorted by (distance, id), distinct ids, never the row itself
    for r in range(qa.indices.shape[0]):
        ids = qa.indices[r, :ql]
        dd = qa.distances[r, :ql]
        real = ids != M
        assert (np.diff(dd) >= 0).all()
        assert len(set(ids[real].tolist())) == real.sum()
        assert (10 + r) not in ids.tolist()
        # every stored distance belongs to its id
        for i, x in zip(ids[real], dd[real]):
            assert x == orc.distance(v[i], v[10 + r])


def test_search_improves_monotonically():
    rng = np.random.default_rng(11)
    n, dim = 300, 16
    v = unit(rng, n, dim)
    c = cfg(beam_size=6, beam_queue_factor=2, speculative_readahead=1)
    ql = 12
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    q = build_queue(v, beams, d, 0, n, ql, 4)
    before = q.distances[:, :ql].copy()
    orc.closest_vectors(v, q, v, beams, c, orc.excluding_self(0, n))
    assert (q.distances[:, :ql] <= before).all()
    assert (q.distances[:, :ql] < before).any()


def test_complete_graph_finds_exact_neighbours():
    # every node lists every other node: one expansion of any node sees everything
    rng = np.random.default_rng(12)
    n, dim, k = 24, 6, 5
    v = unit(rng, n, dim)
    beams = np.stack([np.array([j for j in range(n) if j != i]) for i in range(n)]).astype(np.int32)
    c = cfg(beam_size=n - 1, recall_search_queue_factor=1, parallel_visit_count=1, visit_queue_factor=1)
    qv = unit(rng, 7, dim)
    res = orc.search(v, beams, qv, c, queue_size=k)
    want, wd = orc.knn_exact(qv, v, k)
    assert np.array_equal(res.indices[:, :k], want)
    assert np.allclose(res.distances[:, :k], wd, rtol=1e-5, atol=1e-6)


def test_layered_search_ends_on_the_last_layer():
    # a layered search is one search per neighbour table; with the complete graph as the last
    # layer every row must find itself whatever the coarse layers did, and one layer alone
    # equals a plain search
    rng = np.random.default_rng(15)
    n, dim = 40, 5
    v = unit(rng, n, dim)
    coarse = orc.generate_circulant_beams(n, orc.primes(6))
    full = np.stack([np.array([j for j in range(n) if j != i]) for i in range(n)]).astype(np.int32)
    # the queue's spare capacity is sized from the configured beam size: layers may be narrower, not wider
    c = cfg(beam_size=n - 1, recall_search_queue_factor=1, parallel_visit_count=2, visit_queue_factor=1)
    assert orc.hnsw_calculate_recall(v, [coarse, full], c) == (n, 1.0)
    a = orc.initial_queue(v, c)
    orc.search_layers([coarse], v, a, v, c)
    b = orc.initial_queue(v, c)
    orc.closest_vectors(v, b, v, coarse, c, None)
    assert np.array_equal(a.indices, b.indices) and np.array_equal(a.distances, b.distances)
    assert orc.hnsw_calculate_recall(v, [coarse], c) == orc.ann_calculate_recall(v, coarse, c)


def test_knn_exact_against_numpy():
    rng = np.random.default_rng(13)
    v = unit(rng, 500, 20)
    q = unit(rng, 9, 20)
    ids, d = orc.knn_exact(q, v, 10)
    full = np.clip((1 - q.astype(np.float64) @ v.astype(np.float64).T) / 2, 0, 1)
    want = np.argsort(full, axis=1, kind="stable")[:, :10]
    assert np.array_equal(ids, want)
    assert np.allclose(d, np.take_along_axis(full, want, 1))


def recall_at_k(found, truth):
    hits = sum(len(set(f.tolist()) & set(t.tolist())) for f, t in zip(found, truth))
    return hits / truth.size


def test_generate_ann_end_to_end():
    rng = np.random.default_rng(14)
    n, dim = 1500, 24
    v = unit(rng, n, dim)
    c = cfg(beam_size=12, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=400, optimization_loops=2)
    trace = []
    beams, d = orc.generate_ann(v, c, trace=trace)
    assert beams.shape == (n, 12) and d.shape == (n, 12)
    assert len(trace) >= 4 and all(t % 5 == 0 for _, _, t in trace)
    real = beams != M
    assert real[:, 0].all()
    rows = np.repeat(np.arange(n), 12).reshape(n, 12)
    assert (beams[real] != rows[real]).all()       # no self edges
    want = orc.calculate_distances(v, np.where(real, beams, 0).astype(np.int32))
    assert np.array_equal(d[real], want[real])     # returned distances belong to the ids
    # graph quality: its lists overlap the exact neighbours, and search on it finds them
    truth, _ = orc.knn_exact(v[:200], v, 11)
    assert recall_at_k(beams[:200, :10], truth[:, 1:]) > 0.6
    qv = unit(rng, 100, dim)
    res = orc.search(v, beams, qv, c)
    t10, _ = orc.knn_exact(qv, v, 10)
    assert recall_at_k(res.indices[:, :10], t10) > 0.9
    found, rec = orc.ann_calculate_recall(v, beams, c, sample=v[:300])
    assert rec > 0.95


def test_generate_ann_stale_distance_mode_differs_only_after_loop_zero():
    rng = np.random.default_rng(15)
    v = unit(rng, 400, 12)
    c = cfg(beam_size=6, beam_queue_factor=2, batch_size=400, optimization_loops=1, prune=False)
    b1, d1 = orc.generate_ann(v, c)
    b2, d2 = orc.generate_ann(v, c, stale_distances=True)
    assert np.array_equal(b1, b2)          # one loop: same graph
    assert not np.array_equal(d1, d2)      # but the reference hands back the circulant distances
    init = orc.calculate_distances(v, orc.generate_circulant_beams(400, orc.primes(12)))
    assert np.array_equal(d2, init[:, :6])
