"""The rule by which a beam-search row drops candidates it only knows bounds of (csrc/beam.hip, `refine`),
checked on the CPU against the oracle's reference-faithful queues: the loop of closest_vectors is run once as
the reference runs it and once with every candidate that the rule drops replaced by the empty pair before
both queue inserts; the queues must come out identical however loose the bounds are.  No GPU needed: this
pins the rule itself, the GPU tests pin its implementation."""
import numpy as np
import pytest

from oracle import oracle as orc

M, F = orc.MAXINT, orc.MAXFLOAT


def bounds_for(ids, d, slack, seed):
    """lo <= d <= hi with a gap of up to `slack` each side that depends on the id (as a sketch row's does) and,
    a little, on the slot: copies of one id may carry different bounds (fresh from the sketch, or decoded from
    the cache and a step wider)."""
    h = (ids.astype(np.int64) * 2654435761 + seed) % 1000003
    widen = 1.0 + 0.05 * (np.arange(ids.shape[0]) % 3)
    below = (h % 997) / 997.0 * slack * widen
    above = ((h // 997) % 991) / 991.0 * slack * widen
    lo = np.maximum(d - below, 0).astype(np.float32)
    hi = np.minimum(d + above, 1).astype(np.float32)
    lo[ids == M] = F
    hi[ids == M] = F
    return lo, hi


def drop_by_rule(ids, d, lo, hi, ws_d, wv_d, seen, vt):
    """What the kernel keeps of one row's candidates: keep[i] is False for a candidate that it drops.
    seen: the row's visited list after this iteration's update, or None when it has no free column.
    First round: candidates that may be below a queue's last slot, and the vt distinct unvisited candidates
    with the smallest upper bounds among those certainly above the visit queue's last live slot; the largest
    exact distance of the latter is the threshold of the second round."""
    real = ids != M
    need = real & ~(lo > ws_d)
    if seen is not None:
        unseen = real & ~np.isin(ids, seen[seen != M])
        need |= unseen & ~(lo > wv_d)
        rest = unseen & (lo > wv_d)
        first = []   # vt distinct ids, smallest (hi, id) first; every copy of a chosen id goes with it
        for (_, cid) in sorted((float(hi[i]), int(ids[i])) for i in np.flatnonzero(rest)):
            if cid not in first and len(first) < vt:
                first.append(cid)
        if len(first) < vt:
            need |= rest
        else:
            winners = rest & np.isin(ids, first)
            tv = d[winners].max()
            need |= winners | (rest & ~(lo > tv))
    return need


def run(q, v, beams, cfg, queue, exclude, slack, seed):
    """closest_vectors (ann.py:38-93) statement by statement; slack None = as the reference, else with the
    dropped candidates emptied.  Returns the iteration count and how many candidates were dropped."""
    width = beams.shape[1]
    vt = cfg["parallel_visit_count"]
    b = queue.size()[0]
    vl = cfg["visit_queue_factor"] * cfg["beam_size"]
    visit_queue = orc.Queue(b, vl, vl + width * vt)
    visit_queue.initialize_from_queue(queue)
    seen = np.full((b, cfg["exclude_factor"] * vl), M, dtype=np.int32)
    take = min(vl, vt)
    progressing, count, dropped, asked = True, 0, 0, 0
    while progressing:
        count += 1
        checking = count % cfg["speculative_readahead"] == 0
        visit = visit_queue.pop_n_ids(vt)
        idx, d = orc.search_from_seeds(q, visit, beams, v)
        ws = queue.distances[:, queue.length - 1].copy()
        wv = visit_queue.distances[:, vl - 1].copy() if vl > take else np.full(b, -1.0, dtype=np.float32)
        new_seen = orc.add_new_to_seen_(seen, visit) if seen is not None else None
        if slack is not None:
            idx, d = idx.copy(), d.copy()
            for r in range(b):
                lo, hi = bounds_for(idx[r], d[r], slack, seed)
                keep = drop_by_rule(idx[r], d[r], lo, hi, ws[r], wv[r], None if new_seen is None else new_seen[r], take)
                gone = (idx[r] != M) & ~keep
                dropped += int(gone.sum())
                asked += int((idx[r] != M).sum())
                idx[r, gone] = M
                d[r, gone] = F
        did = queue.insert(idx, d, exclude=exclude, output_update=checking)
        seen = new_seen
        if seen is not None:
            visit_queue.insert(idx, d, exclude=seen)
        if checking:
            progressing = bool(did.any())
    return count, dropped, asked


CASES = [
    # n, dim, beam, bqf, pv, vqf, ef, ra, rows
    (300, 8, 4, 2, 2, 3, 5, 5, 40),
    (500, 16, 8, 2, 4, 3, 5, 5, 30),
    (400, 12, 5, 2, 3, 2, 1, 2, 40),   # a visited list that runs full
    (200, 10, 2, 2, 4, 1, 2, 3, 30),   # visit queue shorter than the visit count
    (600, 24, 6, 3, 1, 3, 5, 5, 25),   # one visit per iteration
    (350, 6, 3, 2, 9, 4, 2, 4, 20),
]


@pytest.mark.parametrize("n,dim,beam,bqf,pv,vqf,ef,ra,rows", CASES)
@pytest.mark.parametrize("slack", [0.0, 0.002, 0.02, 0.2, 2.0])
def test_dropping_by_bounds_never_changes_a_queue(n, dim, beam, bqf, pv, vqf, ef, ra, rows, slack):
    rng = np.random.default_rng(n * 31 + dim)
    v = rng.standard_normal((n, dim)).astype(np.float32)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    v[7] = v[3]   # duplicate rows: equal distances, ties ordered by id
    cfg = dict(orc.DEFAULT_CONFIG)
    cfg.update(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, visit_queue_factor=vqf,
               exclude_factor=ef, speculative_readahead=ra)
    ql = beam * bqf
    table = orc.generate_circulant_beams(n, orc.primes(ql))
    table[rng.random(table.shape) < 0.03] = M
    table[:, 1] = table[:, 0]   # the same id twice in every neighbour list
    d0 = orc.calculate_distances(v, table)
    excl = orc.excluding_self(0, rows)

    def fresh():
        q = orc.Queue(rows, ql, ql + ql * pv)
        q.insert(table[:rows], d0[:rows])
        return q

    want = fresh()
    (t_want, _, _) = run(v[:rows], v, table, cfg, want, excl, None, 0)
    assert t_want == orc.closest_vectors(v[:rows], fresh(), v, table, cfg, excl)   # the model is the oracle's loop
    got = fresh()
    (t_got, dropped, asked) = run(v[:rows], v, table, cfg, got, excl, slack, 12345)
    assert t_got == t_want
    assert np.array_equal(got.indices[:, :ql], want.indices[:, :ql])
    assert np.array_equal(got.distances[:, :ql].view(np.uint32), want.distances[:, :ql].view(np.uint32))
    if slack <= 0.02:
        assert dropped > 0.2 * asked   # tight bounds do drop candidates: the rule is not vacuous
