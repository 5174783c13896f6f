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


def test_knn_exact_l2_against_numpy():
    """Rows of unequal length: the squared-distance order differs from the cosine order."""
    rng = np.random.default_rng(14)
    v = (rng.standard_normal((500, 20)) * rng.uniform(0.5, 2, (500, 1))).astype(np.float32)
    q = (rng.standard_normal((9, 20)) * rng.uniform(0.5, 2, (9, 1))).astype(np.float32)
    with orc.metric("l2"):
        ids, d = orc.knn_exact(q, v, 10)
    cos_ids, _ = orc.knn_exact(q, v, 10)
    full = ((q[:, None, :].astype(np.float64) - v[None, :, :].astype(np.float64)) ** 2).sum(2)
    want = np.argsort(full, axis=1, kind="stable")[:, :10]
    assert np.array_equal(ids, want) and not np.array_equal(ids, cos_ids)
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


# ---- a beam search small enough to follow by hand ---------------------------------------------
# One query q = [1.0] over one-dimensional "vectors" x_i = 1 - 2*delta_i, so that the distance of
# node i is (1 - x_i) / 2 = delta_i exactly (sixteenths: no rounding anywhere).  Node i lists
# [i+1, i+2] mod n and lies at delta_i = (n - i) / 16: every hop moves closer.  Configuration:
# width 2, one visit per iteration, visit queue of 2 slots (+2 spare), visited list of 4 columns,
# progress checked every iteration; search queue of 2 slots (+2 spare) seeded with nodes 0 and 1.
#
# n = 12, derived statement by statement from ann.py:66-91, queue.py:37-61,87-95, utils.py:61-82:
#  it 1  pop 1    candidates 2,3    search [3,2|1,0]    visited [1]        visit [3,2|0,-]
#  it 2  pop 3    candidates 4,5    search [5,4|3,2]    visited [1,3]      visit [5,4|2,-]   (0 is overwritten)
#  it 3  pop 5    candidates 6,7    search [7,6|5,4]    visited [1,3,5]    visit [7,6|4,-]
#  it 4  pop 7    candidates 8,9    search [9,8|7,6]    visited [1,3,5,7]  visit [9,8|6,-]
#  it 5  pop 9    candidates 10,11  search [11,10|9,8]  no free column: add_new_to_seen_ returns None,
#                                                       the visit queue is not fed and stays [-,8|6,-]
#  it 6  pop -    (slot 0 was emptied by the pop of it 5 and nothing re-sorted the row: node 8 is never
#                 visited)  no candidates, search prefix unchanged -> the loop ends.  T = 6.
# n = 8: the visited list fills at it 4 ([1,3,5,7]); it 4 pops 7, candidates 0,1 leave the prefix
#  [7,6] unchanged -> T = 4.  With node 6 excluded from the search queue (it still enters the visit
#  queue, which only excludes visited nodes): it 3 gives search [7,5|4,-], it 4 changes nothing -> [7,5].
def chain(n):
    delta = np.array([(n - i) / 16.0 for i in range(n)], dtype=np.float32)
    v = (1.0 - 2.0 * delta).reshape(n, 1).astype(np.float32)
    beams = np.array([[(i + 1) % n, (i + 2) % n] for i in range(n)], dtype=np.int32)
    c = cfg(beam_size=2, parallel_visit_count=1, visit_queue_factor=1, exclude_factor=2, speculative_readahead=1)
    q = orc.Queue(1, 2, 4)
    q.insert(np.array([[0, 1]], dtype=np.int32), np.array([[delta[0], delta[1]]], dtype=np.float32))
    return v, beams, c, q, delta


@pytest.mark.parametrize("loop", [orc.closest_vectors, orc.closest_vectors_py])
def test_hand_enumerated_trace(loop):
    one = np.ones((1, 1), dtype=np.float32)
    v, beams, c, q, delta = chain(12)
    assert loop(one, q, v, beams, c, None) == 6
    assert q.indices[0, :2].tolist() == [11, 10]
    assert q.distances[0, :2].tolist() == [1 / 16, 2 / 16]
    v, beams, c, q, delta = chain(8)
    assert loop(one, q, v, beams, c, None) == 4
    assert q.indices[0, :2].tolist() == [7, 6] and q.distances[0, :2].tolist() == [1 / 16, 2 / 16]
    v, beams, c, q, delta = chain(8)
    assert loop(one, q, v, beams, c, np.array([[6]], dtype=np.int32)) == 4
    assert q.indices[0, :2].tolist() == [7, 5] and q.distances[0, :2].tolist() == [1 / 16, 3 / 16]


def test_hand_enumerated_trace_per_query_stop():
    # the per-query model on the same chains, patience = speculative_readahead = 1.  n = 12: iterations
    # 1-5 each change the search queue; at it 5 the visited list has no free column, the row is
    # finished: T = 5, same answer.  n = 8: it 4 leaves the prefix [7,6] unchanged -> finished, T = 4.
    # With patience 2 (progress checked every second iteration) on n = 8: it 4 is the first quiet
    # iteration, it 5 pops 6 (candidates 7 and 0 change nothing) and the visited list is full: T = 6,
    # the first check at which the row is finished.
    one = np.ones((1, 1), dtype=np.float32)
    v, beams, c, q, delta = chain(12)
    assert orc.closest_vectors_per_query(one, q, v, beams, c, None) == 5
    assert q.indices[0, :2].tolist() == [11, 10]
    v, beams, c, q, delta = chain(8)
    assert orc.closest_vectors_per_query(one, q, v, beams, c, None) == 4
    assert q.indices[0, :2].tolist() == [7, 6]
    v, beams, c, q, delta = chain(8)
    c["speculative_readahead"] = 2
    assert orc.closest_vectors_per_query(one, q, v, beams, c, None) == 6
    assert q.indices[0, :2].tolist() == [7, 6]


def test_per_query_stop_rows_are_independent_and_no_worse_than_their_seeds():
    # with a visited list that never fills, a row's result under the per-query stop depends on that row
    # alone: the batch equals its rows searched one at a time; on a complete graph it is exact kNN
    rng = np.random.default_rng(21)
    n, dim = 400, 12
    v = unit(rng, n, dim)
    c = cfg(beam_size=6, beam_queue_factor=2, exclude_factor=40, speculative_readahead=3)
    ql = 12
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    rows = slice(30, 70)
    q = build_queue(v, beams, d, rows.start, rows.stop, ql, 4)
    before = q.distances[:, :ql].copy()
    t = orc.closest_vectors_per_query(v[rows], q, v, beams, c, orc.excluding_self(rows.start, rows.stop))
    assert t % 3 == 0 and (q.distances[:, :ql] <= before).all()
    for r in range(rows.start, rows.stop, 7):
        one = build_queue(v, beams, d, r, r + 1, ql, 4)
        orc.closest_vectors_per_query(v[r:r + 1], one, v, beams, c, orc.excluding_self(r, r + 1))
        assert np.array_equal(one.indices[0, :ql], q.indices[r - rows.start, :ql])
    full = np.stack([np.array([j for j in range(24) if j != i]) for i in range(24)]).astype(np.int32)
    cc = cfg(beam_size=23, recall_search_queue_factor=1, parallel_visit_count=1, visit_queue_factor=1)
    qv = unit(rng, 5, dim)
    res = orc.search(v[:24], full, qv, cc, queue_size=4, stop="per_query")
    want, _ = orc.knn_exact(qv, v[:24], 4)
    assert np.array_equal(res.indices[:, :4], want)
