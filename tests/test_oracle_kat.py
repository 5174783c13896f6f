"""Pins for the CPU oracle: known answers derived by hand from the reference's
source, closed forms, and brute force with independent Python code.  No GPU."""
import hashlib
import itertools

import numpy as np
import pytest

from oracle import oracle as orc

M = orc.MAXINT
F = orc.MAXFLOAT


# ---------------------------------------------------------------- constants
def test_sentinels():
    assert M == 2**31 - 1
    assert np.float32(3.4028e37).view(np.uint32) == 0x7DCCCC6F
    assert F.view(np.uint32) == 0x7DCCCC6F


def test_primes_table():
    p = orc.all_primes()
    assert len(p) == 965
    # SHA-256 of the comma-joined decimal entries of constants.py:10-980
    digest = hashlib.sha256(",".join(str(int(x)) for x in p).encode()).hexdigest()
    assert digest == "8429c680ef173757588a246e49760e8a81060d2c436d6435265f80bc9a4a8f50"
    assert p[0] == 10000349 and p[63] == 10001347 and p[127] == 10002323
    assert p[583] == 10009729 and p[584] == 1009007 and p[658] == 1009997
    assert list(p[659:664]) == [1, 2, 59063, 79193, 3] and p[964] == 1999
    assert list(orc.primes(4)) == [10000349, 10000357, 10000363, 10000379]


# ---------------------------------------------------------------- circulants
def test_circulant_kat():
    p4 = orc.primes(4)
    got = orc.generate_circulant_beams(10, p4)
    want = [[9, 7, 3, 9], [0, 8, 4, 0], [1, 9, 5, 1], [2, 0, 6, 2], [3, 1, 7, 3],
            [4, 2, 8, 4], [5, 3, 9, 5], [6, 4, 0, 6], [7, 5, 1, 7], [8, 6, 2, 8]]
    assert got.tolist() == want
    g7 = orc.generate_circulant_beams(7, p4)
    assert g7[0].tolist() == [2, 3, 2, 4] and g7[3].tolist() == [5, 6, 5, 0]
    assert orc.generate_queue_circulants(2, 1000, p4).tolist() == [[349, 357, 363, 379], [350, 358, 364, 380]]


@pytest.mark.parametrize("n,k", [(100, 8), (4096, 64), (1000, 72), (977, 700)])
def test_circulant_closed_form(n, k):
    p = orc.primes(k).astype(np.int64)
    got = orc.generate_circulant_beams(n, orc.primes(k))
    want = np.sort(np.arange(n)[:, None] + p[None, :], axis=1) % n
    assert np.array_equal(got, want)
    # row i+1 = row i + 1 (mod n)
    assert np.array_equal(got[1:], (got[:-1] + 1) % n)
    q = orc.generate_queue_circulants(17, n, orc.primes(k))
    assert np.array_equal(q, np.sort(np.arange(17)[:, None] + p[None, :], axis=1) % n)


# ---------------------------------------------------------------- distance
def test_distance_special_cases():
    assert orc.distance_from_cos(1.0) == 0.0
    assert orc.distance_from_cos(0.0) == 0.5
    assert orc.distance_from_cos(-1.0) == 1.0
    assert orc.distance_from_cos(0.5) == 0.25
    assert orc.distance_from_cos(1.0000001) == 0.0
    assert orc.distance_from_cos(-1.5) == 1.0
    e0 = np.zeros(8, np.float32); e0[0] = 1
    e1 = np.zeros(8, np.float32); e1[1] = 1
    assert orc.distance(e0, e0) == 0.0
    assert orc.distance(e0, e1) == 0.5
    assert orc.distance(e0, -e0) == 1.0


@pytest.mark.parametrize("dim", [1, 3, 4, 5, 63, 64, 128, 255, 256, 257, 384, 768, 1000, 1024, 1536, 2049, 6144])
def test_distance_against_float64(dim):
    rng = np.random.default_rng(dim)
    for _ in range(20):
        a = rng.standard_normal(dim).astype(np.float32); a /= np.linalg.norm(a)
        b = rng.standard_normal(dim).astype(np.float32); b /= np.linalg.norm(b)
        want = np.clip((1.0 - np.dot(a.astype(np.float64), b.astype(np.float64))) / 2.0, 0, 1)
        got = float(orc.distance(a, b))
        assert abs(got - want) <= 1e-5 * abs(want) + 1e-6
        assert orc.distance(a, b) == orc.distance(b, a)
        # unit vectors: d = |a-b|^2 / 4
        assert abs(got - np.sum((a.astype(np.float64) - b) ** 2) / 4) < 1e-6


@pytest.mark.parametrize("dim", [5, 130, 771, 1030])
def test_dot_every_element_counts(dim):
    # a dropped, doubled or misplaced element changes an exactly representable sum
    for i in range(dim):
        a = np.zeros(dim, np.float32); b = np.zeros(dim, np.float32)
        a[i] = 3.0; b[i] = 0.25
        assert orc.dot(a, b) == np.float32(0.75)
    a = np.arange(1, dim + 1, dtype=np.float32)
    assert orc.dot(a, np.ones(dim, np.float32)) == np.float32(dim * (dim + 1) / 2)
    # pairs (i, j) must multiply element-wise, not crosswise
    b = np.zeros(dim, np.float32); b[dim - 1] = 1
    assert orc.dot(a, b) == np.float32(dim)


# ---------------------------------------------------------------- K6 / K7
def _unit(rng, n, d):
    v = rng.standard_normal((n, d)).astype(np.float32)
    return v / np.linalg.norm(v, axis=1, keepdims=True)


def test_calculate_distances_bruteforce():
    rng = np.random.default_rng(1)
    v = _unit(rng, 50, 24)
    beams = rng.integers(0, 50, (50, 7)).astype(np.int32)
    beams[3, 2] = M
    out = orc.calculate_distances(v, beams)
    for r, c in itertools.product(range(50), range(7)):
        if beams[r, c] == M:
            assert out[r, c] == F
        else:
            want = np.clip((1 - float(np.dot(v[r].astype(np.float64), v[beams[r, c]]))) / 2, 0, 1)
            assert abs(out[r, c] - want) < 1e-6


def test_search_from_seeds_bruteforce():
    rng = np.random.default_rng(2)
    n, d, w, b, nv = 40, 16, 5, 6, 3
    v = _unit(rng, n, d)
    q = _unit(rng, b, d)
    beams = rng.integers(0, n, (n, w)).astype(np.int32)
    beams[7, 1] = M
    visit = rng.integers(0, n, (b, nv)).astype(np.int32)
    visit[0, 1] = M
    visit[1, 0] = 7
    idx, dist = orc.search_from_seeds(q, visit, beams, v)
    assert idx.shape == (b, nv * w)
    for r, s, k in itertools.product(range(b), range(nv), range(w)):
        slot = s * w + k  # kernels.py:241,253
        if visit[r, s] == M or beams[visit[r, s], k] == M:
            assert idx[r, slot] == M and dist[r, slot] == F
        else:
            nb = beams[visit[r, s], k]
            assert idx[r, slot] == nb
            want = np.clip((1 - float(np.dot(q[r].astype(np.float64), v[nb]))) / 2, 0, 1)
            assert abs(dist[r, slot] - want) < 1e-6
    # same pair, same bits, whichever entry point computed it
    cd = orc.calculate_distances(v, beams)
    i2, d2 = orc.search_from_seeds(v, np.arange(n, dtype=np.int32).reshape(-1, 1), beams, v)
    assert np.array_equal(d2.view(np.uint32), cd.view(np.uint32))


# ---------------------------------------------------------------- sort / dedup
def model_queue_sort(ids, d):
    """Independent model of queue.py:15-18 on one row: order by (distance, id),
    drop the later of two neighbouring slots with the same id, pad."""
    pairs = sorted(zip([float(x) for x in d], [int(x) for x in ids]))
    kept = [p for i, p in enumerate(pairs) if i == 0 or pairs[i - 1][1] != p[1]]
    kept = [p for p in kept if p[1] != M] + [(float(F), M)] * 0
    out_ids = [p[1] for p in kept] + [M] * (len(ids) - len(kept))
    out_d = [np.float32(p[0]) for p in kept] + [F] * (len(ids) - len(kept))
    return out_ids, out_d


def test_mark_punch_invariant():
    rng = np.random.default_rng(3)
    ids = np.sort(rng.integers(0, 12, (30, 40)).astype(np.int32), axis=1)
    ids[:, 35:] = M
    d = rng.random((30, 40)).astype(np.float32)
    a, b = ids.copy(), d.copy()
    orc.dedup_tensor_pair_(a, b)
    c = ids.copy()
    orc.dedup_tensor_(c)
    assert np.array_equal(a, c)
    for r in range(30):
        for q in range(40):
            first_of_run = q == 0 or ids[r, q - 1] != ids[r, q]
            if first_of_run and ids[r, q] != M:
                assert a[r, q] == ids[r, q] and b[r, q] == d[r, q]
            else:
                assert a[r, q] == M and b[r, q] == F


def test_queue_sort_against_model():
    rng = np.random.default_rng(4)
    for trial in range(200):
        cap = int(rng.integers(2, 50))
        ids = rng.integers(0, 15, cap).astype(np.int32)
        # distances from a small set -> many ties; same id may carry different distances
        d = (rng.integers(0, 6, cap) / 8.0).astype(np.float32)
        sent = rng.random(cap) < 0.2
        ids[sent] = M
        d[sent] = F
        gi, gd = orc.queue_sort(ids[None, :], d[None, :])
        wi, wd = model_queue_sort(ids, d)
        assert gi[0].tolist() == wi, (trial, ids, d)
        assert gd[0].tolist() == wd


def test_queue_sort_deterministic_distances_is_sorted_set():
    # when an id always carries the same distance the result is sorted(set(pairs))
    rng = np.random.default_rng(5)
    table = rng.random(64).astype(np.float32)
    table[10:20] = table[10]  # ties between different ids
    ids = rng.integers(0, 64, (40, 96)).astype(np.int32)
    d = table[ids]
    gi, gd = orc.queue_sort(ids, d)
    for r in range(40):
        want = sorted(set(zip(d[r].tolist(), ids[r].tolist())))
        k = len(want)
        assert gi[r, :k].tolist() == [w[1] for w in want]
        assert gd[r, :k].tolist() == [w[0] for w in want]
        assert (gi[r, k:] == M).all() and (gd[r, k:] == F).all()


def test_index_by_tensor():
    rng = np.random.default_rng(6)
    a = rng.integers(0, 1000, (9, 13)).astype(np.int32)
    b = np.stack([rng.permutation(13) for _ in range(9)])
    assert np.array_equal(orc.index_by_tensor(a, b), np.take_along_axis(a, b, axis=1))


def test_punchout_excluded_rule():
    ids = np.array([[1, 2, 3, 4, 5, M]], dtype=np.int32)
    d = np.array([[.1, .2, .3, .4, .5, F]], dtype=np.float32)
    excl = np.array([[2, 4, M, 5]], dtype=np.int32)  # scan stops at the first MAXINT: 5 survives
    orc.punchout_excluded_(ids, d, excl)
    assert ids.tolist() == [[1, M, 3, M, 5, M]]
    assert d[0, 1] == F and d[0, 3] == F and d[0, 4] == np.float32(.5)


# ---------------------------------------------------------------- Queue
def test_queue_kat():
    q = orc.Queue(1, 4, 8)
    q.insert(np.array([[5, 3, 5, 9]]), np.array([[.3, .1, .3, .2]], np.float32))
    assert q.indices.tolist() == [[3, 9, 5, M, M, M, M, M]]
    assert q.distances[0, :3].tolist() == [np.float32(.1), np.float32(.2), np.float32(.3)]
    assert (q.distances[0, 3:] == F).all()
    mask = q.insert(np.array([[7, 3, 2, M]]), np.array([[.05, .1, .2, F]], np.float32),
                    exclude=np.array([[2, M]], np.int32), output_update=True)
    assert q.indices.tolist() == [[7, 3, 9, 5, M, M, M, M]]
    assert q.distances[0, :4].tolist() == [np.float32(x) for x in (.05, .1, .2, .3)]
    assert mask.tolist() == [[True, True, True, True]]
    popped = q.pop_n_ids(2)
    assert popped.tolist() == [[7, 3]]
    assert q.indices.tolist() == [[M, M, 9, 5, M, M, M, M]]
    assert q.distances[0, 2:4].tolist() == [np.float32(.2), np.float32(.3)] and q.distances[0, 0] == F


def test_queue_tie_break_and_tail():
    q = orc.Queue(1, 2, 6)
    q.insert(np.array([[8, 2]]), np.array([[.5, .5]], np.float32))
    assert q.indices[0, :2].tolist() == [2, 8]
    # capacity - length (4) exceeds the insert width (2): slots [length+m, cap) survive
    q.insert(np.array([[1, 3]]), np.array([[.1, .3]], np.float32))
    assert q.indices[0].tolist() == [1, 3, 2, 8, M, M]
    q.insert(np.array([[4, 5]]), np.array([[.2, .9]], np.float32))
    # before sort: [1,3 | 4,5 | M,M]  ->  (2,.5),(8,.5) were overwritten
    assert q.indices[0].tolist() == [1, 4, 3, 5, M, M]


def test_queue_initialize_from_queue():
    a = orc.Queue(2, 3, 5)
    a.insert(np.array([[1, 2], [4, 5]]), np.array([[.3, .2], [.1, .2]], np.float32))
    b = orc.Queue(2, 1, 4)
    b.initialize_from_queue(a)
    assert b.indices.tolist() == [[2, M, M, M], [4, M, M, M]]


# ---------------------------------------------------------------- prune
def test_prune_kat():
    beams = np.array([[1, 2], [2, 0], [1, 0]], np.int32)
    d = np.array([[.1, .3], [.05, .1], [.05, .3]], np.float32)
    ob, od = orc.prune_(beams, d)
    assert ob.tolist() == [[1, M], [2, 0], [1, 0]]
    assert od[0].tolist() == [np.float32(.1), F]
    assert np.array_equal(od[1:], d[1:])


def model_prune(beams, d):
    n, w = beams.shape
    ob, od = beams.copy(), d.copy()
    for x in range(n):
        for j in range(w):
            y = beams[x, j]
            if y == M:
                continue
            z = beams[y, 0]
            if z == M:
                continue
            hits = [i for i in range(w) if beams[x, i] == z]
            if not hits:
                continue
            i = hits[-1]
            if d[x, i] > d[x, j] and d[x, i] > d[y, 0]:
                ob[x, i] = M
                od[x, i] = F
    for x in range(n):
        order = sorted(range(w), key=lambda i: (od[x, i], i))
        ob[x] = ob[x, order]
        od[x] = od[x, order]
    return ob, od


def test_prune_against_model():
    rng = np.random.default_rng(7)
    n, w, dim = 60, 6, 8
    v = _unit(rng, n, dim)
    beams = np.stack([rng.choice(n, w, replace=False) for _ in range(n)]).astype(np.int32)
    beams[5, 3] = M
    d = orc.calculate_distances(v, beams)
    beams, d = orc.queue_sort(beams, d)
    ob, od = orc.prune_(beams, d)
    wb, wd = model_prune(beams, d)
    assert np.array_equal(ob, wb) and np.array_equal(od, wd)
    assert (ob[:, 0] == beams[:, 0]).all()  # slot 0 of a sorted row is never pruned
    assert (ob != beams).any()


# ---------------------------------------------------------------- visited list
def test_seen_add():
    seen = np.full((2, 6), M, np.int32)
    r = orc.add_new_to_seen_(seen, np.array([[5, 3], [7, M]], np.int32))
    assert r is seen and seen.tolist() == [[3, 5, M, M, M, M], [7, M, M, M, M, M]]
    # first free column is global: column 2 (row 0 holds two ids)
    orc.add_new_to_seen_(seen, np.array([[4, 5], [1, 2]], np.int32))
    assert seen.tolist() == [[3, 4, 5, M, M, M], [1, 2, 7, M, M, M]]  # the repeated 5 collapses
    orc.add_new_to_seen_(seen, np.array([[9, 8], [M, M]], np.int32))
    assert seen.tolist() == [[3, 4, 5, 8, 9, M], [1, 2, 7, M, M, M]]
    # one free column left: only the first visited id is recorded
    orc.add_new_to_seen_(seen, np.array([[11, 12], [13, 14]], np.int32))
    assert seen.tolist() == [[3, 4, 5, 8, 9, 11], [1, 2, 7, 13, M, M]]
    # no column is free in every row any more -> None
    assert orc.add_new_to_seen_(seen, np.array([[20, 21], [22, 23]], np.int32)) is None
    assert seen.tolist() == [[3, 4, 5, 8, 9, 11], [1, 2, 7, 13, M, M]]


# ---------------------------------------------------------------- rank prune / reverse merge (additions)
def model_rank_prune(beams, degree):
    n, w = beams.shape
    out = np.full((n, degree), M, np.int32)
    for x in range(n):
        scored = []
        for j in range(w):
            y = beams[x, j]
            if y == M:
                continue
            c = sum(1 for i in range(j) if beams[x, i] != M and y in beams[beams[x, i], :j].tolist())
            scored.append((c, j, y))
        scored.sort()
        for o, (_, _, y) in enumerate(scored[:degree]):
            out[x, o] = y
    return out


def model_reverse_merge(pruned, keep, rev_from):
    n, d = pruned.shape
    rev = {y: [] for y in range(n)}
    for k, x in sorted((k, x) for x in range(n) for k in range(rev_from)):
        y = pruned[x, k]
        if y != M:
            rev[int(y)].append((k, x))
    out = np.full((n, d), M, np.int32)
    for x in range(n):
        row = [int(y) for y in pruned[x, :keep] if y != M]
        for _, r in sorted(rev[x])[:d - keep]:
            if r != x and r not in row and len(row) < d:
                row.append(r)
        for y in pruned[x, keep:]:
            if y != M and int(y) not in row and len(row) < d:
                row.append(int(y))
        out[x, :len(row)] = row
    return out


def test_rank_prune_kat():
    # 0 lists [1,2,3]; 1 lists 2 first: the edge 0->2 (slot 1) has the detour 0->1->2 (slot 0 of row 1 < 1)
    beams = np.array([[1, 2, 3], [2, 0, 3], [3, 0, 1], [0, 1, 2]], np.int32)
    got = orc.rank_prune(beams, 3)
    # row 0: 1 (no slot before it), 2 (detour via 1), 3 (via 1? row 1[:2]=[2,0] no; via 2: row 2[:2]=[3,0] yes)
    assert got[0].tolist() == [1, 2, 3]
    beams = np.array([[1, 2, 3], [3, 2, 0], [0, 1, 3], [0, 1, 2]], np.int32)
    # row 0: 2 has no detour (row 1[:1]=[3]); 3 has one (row 1[:2] holds 3) -> order unchanged, counts [0,0,1]
    assert orc.rank_prune(beams, 2)[0].tolist() == [1, 2]
    beams = np.array([[1, 3, 2], [3, 2, 0], [0, 1, 3], [0, 1, 2]], np.int32)
    # row 0: slot1=3 detour via 1 (row 1[:1]=[3]) -> count 1; slot2=2: via 1 (row1[:2] has 2) -> 1, via 3 (row3[:2]=[0,1]) no
    assert orc.rank_prune(beams, 3)[0].tolist() == [1, 3, 2]
    beams = np.array([[1, 3, 2], [0, 2, 3], [0, 1, 3], [0, 1, 2]], np.int32)
    # row 0: 3 -> none (row1[:1]=[0]); 2 -> via 1 (row1[:2]=[0,2]) -> counts [0,0,1]
    assert orc.rank_prune(beams, 3)[0].tolist() == [1, 3, 2]
    beams = np.array([[1, 2, 3], [3, 0, 2], [0, 1, 3], [0, 1, 2]], np.int32)
    # row 0: 2 -> none (row1[:1]=[3]); 3 -> via 1 (row1[:2]=[3,0]) -> counts [0,0,1]; with M holes
    beams[0, 1] = M
    assert orc.rank_prune(beams, 3)[0].tolist() == [1, 3, M]


def test_rank_prune_and_reverse_merge_against_models():
    rng = np.random.default_rng(30)
    for n, w, d in [(40, 8, 4), (60, 12, 6), (25, 6, 6)]:
        beams = np.stack([rng.choice([j for j in range(n) if j != i], w, replace=False) for i in range(n)]).astype(np.int32)
        beams[rng.random((n, w)) < 0.08] = M
        beams = np.stack([np.concatenate([r[r != M], r[r == M]]) for r in beams])  # empties last, as after a sort
        got = orc.rank_prune(beams, d)
        assert np.array_equal(got, model_rank_prune(beams, d))
        for keep, rev_from in [(d // 2, d // 2), (1, d), (d, 2)]:
            merged = orc.reverse_merge(got, keep, rev_from)
            assert np.array_equal(merged, model_reverse_merge(got, keep, rev_from))
            for x in range(n):
                real = merged[x][merged[x] != M]
                assert len(set(real.tolist())) == len(real) and x not in real.tolist()
                assert merged[x, :keep].tolist()[:int((got[x, :keep] != M).sum())] == got[x, :keep][got[x, :keep] != M].tolist()


# ---------------------------------------------------------------- squared L2 (an addition: not in the reference)
def test_l2_known_answers():
    a = np.array([3, 0, -1, 2, 5], np.float32)
    b = np.ones(5, np.float32)
    assert orc.l2(a, b) == 26.0 and orc.l2(b, a) == 26.0          # 4 + 1 + 4 + 1 + 16
    assert orc.l2(a, a) == 0.0
    e0 = np.zeros(8, np.float32); e0[0] = 1
    e1 = np.zeros(8, np.float32); e1[1] = 1
    assert orc.l2(e0, e1) == 2.0 and orc.l2(e0, -e0) == 4.0        # orthogonal, antipodal unit vectors
    big = np.full(4, 100.0, np.float32)
    assert orc.l2(big, -big) == 160000.0                           # no clamp to [0, 1]


@pytest.mark.parametrize("dim", [1, 3, 4, 5, 63, 64, 128, 255, 257, 384, 768, 1030, 1536, 2049])
def test_l2_against_float64_and_cosine(dim):
    rng = np.random.default_rng(900 + dim)
    for _ in range(10):
        a = rng.standard_normal(dim).astype(np.float32)
        b = rng.standard_normal(dim).astype(np.float32) * 3
        want = np.sum((a.astype(np.float64) - b.astype(np.float64)) ** 2)
        assert abs(float(orc.l2(a, b)) - want) <= 1e-5 * want
        assert orc.l2(a, b) == orc.l2(b, a)
        # on unit rows |a - b|^2 = 2 - 2<a, b> = 4 x the cosine distance
        a /= np.linalg.norm(a); b /= np.linalg.norm(b)
        assert abs(float(orc.l2(a, b)) - 4 * float(orc.distance(a, b))) < 2e-6


@pytest.mark.parametrize("dim", [5, 130, 771])
def test_l2_every_element_counts(dim):
    # a dropped, doubled or misplaced element, or a difference taken crosswise, changes an exact sum
    for i in range(dim):
        a = np.zeros(dim, np.float32); b = np.zeros(dim, np.float32)
        a[i] = 3.0; b[i] = 0.5
        assert orc.l2(a, b) == np.float32(6.25)
    a = np.arange(1, dim + 1, dtype=np.float32)
    assert orc.l2(a, np.zeros(dim, np.float32)) == np.float32(dim * (dim + 1) * (2 * dim + 1) / 6)
    assert orc.l2(a, a - 2) == np.float32(4 * dim)


def test_l2_metric_switch_reaches_the_drivers_and_is_restored():
    rng = np.random.default_rng(5)
    v = rng.standard_normal((60, 12)).astype(np.float32)
    ids = rng.integers(0, 60, (60, 5)).astype(np.int32)
    ids[4, 1] = M
    cos = orc.calculate_distances(v, ids)
    with orc.metric("l2"):
        out = orc.calculate_distances(v, ids)
        for r, c in itertools.product(range(60), range(5)):
            if ids[r, c] == M:
                assert out[r, c] == F
            else:
                assert out[r, c] == orc.l2(v[ids[r, c]], v[r])
        # a complete graph searched by L2 returns the exact L2 neighbours (not the cosine ones: rows differ in length)
        full = np.stack([np.array([j for j in range(24) if j != i]) for i in range(24)]).astype(np.int32)
        c = dict(orc.DEFAULT_CONFIG, beam_size=23, recall_search_queue_factor=1, parallel_visit_count=1,
                 visit_queue_factor=1)
        q = rng.standard_normal((6, 12)).astype(np.float32)
        res = orc.search(v[:24], full, q, c, queue_size=4)
        d2 = ((q[:, None, :].astype(np.float64) - v[None, :24, :]) ** 2).sum(2)
        assert np.array_equal(res.indices[:, :4], np.argsort(d2, axis=1, kind="stable")[:, :4])
    assert np.array_equal(orc.calculate_distances(v, ids), cos)
