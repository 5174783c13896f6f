"""GPU parity: every libvlgpu entry point (reached through the vectorlink_gpu
Python surface, i.e. through the C ABI) against the CPU oracle on the same
seeded inputs.  ids must match exactly; distances are compared bit for bit
because the kernels and the oracle share one documented summation order (the
contract is rtol 1e-5 / atol 1e-6; bit equality is the stronger statement)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

M = orc.MAXINT
F = orc.MAXFLOAT
DEV = "cuda"


def unit(rng, n, d):
    v = rng.standard_normal((n, d)).astype(np.float32)
    return v / np.linalg.norm(v, axis=1, keepdims=True)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    return t.detach().cpu().numpy()


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def cfg(**kw):
    c = dict(orc.DEFAULT_CONFIG)
    c.update(kw)
    return c


def say(msg):
    print(msg, flush=True)


# ---------------------------------------------------------------- distances
@pytest.mark.parametrize("dim", [4, 20, 64, 100, 128, 130, 256, 384, 768, 1024, 1536, 2048, 2052, 3000])
def test_gather_distances_bit_exact(dim):
    say(f"gather_distances dim={dim}")
    from vectorlink_gpu.kernels import calculate_distances, gather_distances

    rng = np.random.default_rng(dim)
    n, w = 300, 37
    v = unit(rng, n, dim)
    beams = rng.integers(0, n, (n, w)).astype(np.int32)
    beams[rng.random((n, w)) < 0.1] = M
    want = orc.calculate_distances(v, beams)
    got = host(calculate_distances(dev(v), dev(beams)))
    assert np.array_equal(bits(got), bits(want))
    # against float64, the contract's tolerance
    safe = np.where(beams == M, 0, beams)
    ref = np.clip((1 - np.einsum("nd,nwd->nw", v.astype(np.float64), v[safe].astype(np.float64))) / 2, 0, 1)
    real = beams != M
    assert np.allclose(got[real], ref[real], rtol=1e-5, atol=1e-6)
    assert (got[~real] == F).all()
    # separate query tensor, ids out of range read as empty
    q = unit(rng, 50, dim)
    ids = rng.integers(0, n, (50, 9)).astype(np.int32)
    ids[0, 0] = n + 5
    ids[1, 1] = -3
    got2 = host(gather_distances(dev(q), dev(v), dev(ids)))
    for r in range(50):
        for c in range(9):
            if 0 <= ids[r, c] < n:
                assert got2[r, c] == orc.distance(v[ids[r, c]], q[r])
            else:
                assert got2[r, c] == F


@pytest.mark.parametrize("dim,w,nv", [(128, 64, 4), (768, 128, 4), (96, 24, 3), (1536, 48, 2), (50, 7, 5)])
def test_search_from_seeds(dim, w, nv):
    say(f"search_from_seeds dim={dim} w={w} nv={nv}")
    from vectorlink_gpu.kernels import search_from_seeds

    rng = np.random.default_rng(dim + w)
    n, b = 500, 70
    v = unit(rng, n, dim)
    q = unit(rng, b, dim)
    beams = rng.integers(0, n, (n, w)).astype(np.int32)
    beams[rng.random((n, w)) < 0.05] = M
    visit = rng.integers(0, n, (b, nv)).astype(np.int32)
    visit[rng.random((b, nv)) < 0.2] = M
    wi, wd = orc.search_from_seeds(q, visit, beams, v)
    gi, gd = search_from_seeds(dev(q), dev(visit), dev(beams), dev(v))
    assert np.array_equal(host(gi), wi)
    assert np.array_equal(bits(host(gd)), bits(wd))


def test_circulants():
    from vectorlink_gpu.utils import generate_circulant_beams, generate_queue_circulants, primes

    assert np.array_equal(host(primes(965)), orc.all_primes())
    for n, k in [(10, 4), (7, 4), (4096, 64), (1000, 72), (977, 700), (5000, 965)]:
        say(f"circulants n={n} k={k}")
        got = host(generate_circulant_beams(n, primes(k)))
        assert np.array_equal(got, orc.generate_circulant_beams(n, orc.primes(k)))
        got = host(generate_queue_circulants(33, n, primes(k)))
        assert np.array_equal(got, orc.generate_queue_circulants(33, n, orc.primes(k)))


# ---------------------------------------------------------------- id-list kernels
def random_rows(rng, rows, cols, n_ids, n_dist, p_sent=0.15):
    ids = rng.integers(0, n_ids, (rows, cols)).astype(np.int32)
    d = (rng.integers(0, n_dist, (rows, cols)) / np.float32(n_dist)).astype(np.float32)
    s = rng.random((rows, cols)) < p_sent
    ids[s] = M
    d[s] = F
    return ids, d


@pytest.mark.parametrize("cols", [1, 2, 3, 8, 63, 64, 65, 320, 352, 640, 704, 1000, 1024, 2500, 4096])
def test_sorts_and_dedup(cols):
    say(f"sort/dedup cols={cols}")
    from vectorlink_gpu import kernels as K
    from vectorlink_gpu.utils import index_sort, queue_sort

    rng = np.random.default_rng(cols)
    rows = 40
    ids, d = random_rows(rng, rows, cols, max(3, cols // 3), 7)
    wi, wd = orc.index_sort(ids, d)
    gi, gd = index_sort(dev(ids), dev(d))
    assert np.array_equal(host(gi), wi) and np.array_equal(bits(host(gd)), bits(wd))

    wi, wd = orc.queue_sort(ids, d)
    gi, gd = queue_sort(dev(ids), dev(d))
    assert np.array_equal(host(gi), wi) and np.array_equal(bits(host(gd)), bits(wd))

    # punchout_duplicates_ on rows ordered by id (neighbouring duplicates)
    sid = np.sort(ids, axis=1)
    wi, wd = orc.punchout_duplicates_(sid, d)
    ti, td = dev(sid), dev(d)
    K.punchout_duplicates_(ti, td)
    assert np.array_equal(host(ti), wi) and np.array_equal(bits(host(td)), bits(wd))

    a, b = sid.copy(), d.copy()
    orc.dedup_tensor_pair_(a, b)
    ti, td = dev(sid), dev(d)
    K.dedup_tensor_pair_(ti, td)
    assert np.array_equal(host(ti), a) and np.array_equal(bits(host(td)), bits(b))
    c = sid.copy()
    orc.dedup_tensor_(c)
    ti = dev(sid)
    K.dedup_tensor_(ti)
    assert np.array_equal(host(ti), c)


def test_queue_sort_odd_distances():
    # distances outside [0,1]: negative, beyond MAXFLOAT, infinities; -0.0 comes back as +0.0
    from vectorlink_gpu.utils import queue_sort

    ids = np.array([[4, 9, 2, 7, M, 5, 5, 3, 8]], np.int32)
    d = np.array([[-1.5, np.inf, 3.0e38, 0.0, F, 1e-30, 1e-30, -0.0, F]], np.float32)
    wi, wd = orc.queue_sort(ids, d)
    gi, gd = queue_sort(dev(ids), dev(d))
    assert np.array_equal(host(gi), wi)
    assert np.array_equal(host(gd), wd)  # value equality: -0.0 == +0.0


def test_punchout_excluded_strided_view():
    from vectorlink_gpu.kernels import punchout_excluded_

    rng = np.random.default_rng(5)
    rows, cap, length, m, e = 30, 50, 12, 30, 9
    ids, d = random_rows(rng, rows, cap, 25, 5)
    excl = rng.integers(0, 25, (rows, e)).astype(np.int32)
    excl[rng.random((rows, e)) < 0.2] = M
    wi, wd = ids.copy(), d.copy()
    ti, td = np.ascontiguousarray(wi[:, length:length + m]), np.ascontiguousarray(wd[:, length:length + m])
    orc.punchout_excluded_(ti, td, excl)
    wi[:, length:length + m], wd[:, length:length + m] = ti, td
    gi, gd = dev(ids), dev(d)
    punchout_excluded_(gi.narrow(1, length, m), gd.narrow(1, length, m), dev(excl))
    assert np.array_equal(host(gi), wi) and np.array_equal(bits(host(gd)), bits(wd))
    assert (wi != ids).any()


def test_index_by_tensor():
    from vectorlink_gpu.kernels import index_by_tensor

    rng = np.random.default_rng(6)
    a = rng.integers(0, 1000, (19, 77)).astype(np.int32)
    b = np.stack([rng.permutation(77) for _ in range(19)])
    assert np.array_equal(host(index_by_tensor(dev(a), dev(b))), np.take_along_axis(a, b, axis=1))
    f = rng.random((19, 77)).astype(np.float32)
    assert np.array_equal(host(index_by_tensor(dev(f), dev(b))), np.take_along_axis(f, b, axis=1))


# ---------------------------------------------------------------- Queue
def test_queue_kat():
    from vectorlink_gpu import Queue

    q = Queue(1, 4, 8)
    q.insert(dev(np.array([[5, 3, 5, 9]], np.int32)), dev(np.array([[.3, .1, .3, .2]], np.float32)))
    assert host(q.indices).tolist() == [[3, 9, 5, M, M, M, M, M]]
    mask = q.insert(dev(np.array([[7, 3, 2, M]], np.int32)), dev(np.array([[.05, .1, .2, F]], np.float32)),
                    exclude=dev(np.array([[2, M]], np.int32)), output_update=True)
    assert host(q.indices).tolist() == [[7, 3, 9, 5, M, M, M, M]]
    assert host(q.distances)[0, :4].tolist() == [np.float32(x) for x in (.05, .1, .2, .3)]
    assert host(mask).tolist() == [[True, True, True, True]]
    assert host(q.pop_n_ids(2)).tolist() == [[7, 3]]
    assert host(q.indices).tolist() == [[M, M, 9, 5, M, M, M, M]]
    assert host(q.distances)[0, 0] == F


@pytest.mark.parametrize("length,m,cap,e", [(4, 6, 10, 0), (64, 256, 320, 1), (96, 256, 352, 480), (128, 512, 640, 1),
                                           (192, 512, 704, 960), (20, 30, 64, 7), (64, 128, 320, 3)])
def test_queue_insert_pop_sequence(length, m, cap, e):
    say(f"queue sequence length={length} m={m} cap={cap} excl={e}")
    from vectorlink_gpu import Queue

    rng = np.random.default_rng(length * 7 + m)
    rows = 25
    table = rng.random(400).astype(np.float32)  # an id always carries the same distance
    table[100:140] = table[100]
    oq = orc.Queue(rows, length, cap)
    gq = Queue(rows, length, cap)
    for step in range(6):
        ids = rng.integers(0, 400, (rows, m)).astype(np.int32)
        d = table[ids]
        s = rng.random((rows, m)) < 0.1
        ids[s], d[s] = M, F
        ex = None
        if e:
            ex = rng.integers(0, 400, (rows, e)).astype(np.int32)
            ex.sort(axis=1)
            ex[:, e // 2 + 1:] = M
        upd = step % 2 == 1
        wm = oq.insert(ids, d, exclude=ex, output_update=upd)
        gm = gq.insert(dev(ids), dev(d), exclude=None if ex is None else dev(ex), output_update=upd)
        assert np.array_equal(host(gq.indices), oq.indices), step
        assert np.array_equal(bits(host(gq.distances)), bits(oq.distances))
        if upd:
            assert np.array_equal(host(gm), wm)
        if step == 3:
            assert np.array_equal(host(gq.pop_n_ids(3)), oq.pop_n_ids(3))
            assert np.array_equal(host(gq.indices), oq.indices)


def test_seen_add_sequence():
    from vectorlink_gpu.utils import add_new_to_seen_

    rng = np.random.default_rng(8)
    rows, cols, nv = 20, 22, 4
    so = np.full((rows, cols), M, np.int32)
    sg = dev(so)
    alive_o, alive_g = so, sg
    for step in range(30):
        visit = rng.integers(0, 600, (rows, nv)).astype(np.int32)
        visit[rng.random((rows, nv)) < 0.2] = M
        alive_o = orc.add_new_to_seen_(so, visit)
        alive_g = add_new_to_seen_(sg, dev(visit))
        assert (alive_o is None) == (alive_g is None), step
        assert np.array_equal(host(sg), so), step
        if alive_o is None:
            break
    assert alive_o is None  # the list did fill up


# ---------------------------------------------------------------- prune
def test_prune():
    from vectorlink_gpu.kernels import prune_

    b = np.array([[1, 2], [2, 0], [1, 0]], np.int32)
    d = np.array([[.1, .3], [.05, .1], [.05, .3]], np.float32)
    gb, gd = prune_(dev(b), dev(d))
    assert host(gb).tolist() == [[1, M], [2, 0], [1, 0]]
    assert host(gd)[0].tolist() == [np.float32(.1), F]
    rng = np.random.default_rng(9)
    for n, w, dim in [(200, 6, 8), (3000, 64, 16), (1500, 128, 8), (500, 24, 12)]:
        say(f"prune n={n} w={w}")
        v = unit(rng, n, dim)
        beams = np.stack([rng.choice(n, w, replace=False) for _ in range(n)]).astype(np.int32)
        beams[rng.random((n, w)) < 0.03] = M
        dd = orc.calculate_distances(v, beams)
        beams, dd = orc.queue_sort(beams, dd)
        wb, wd = orc.prune_(beams, dd)
        gb, gd = prune_(dev(beams), dev(dd))
        assert np.array_equal(host(gb), wb) and np.array_equal(bits(host(gd)), bits(wd))
        assert (wb != beams).any()


# ---------------------------------------------------------------- beam search
BEAM_CASES = [
    # n, dim, beam, bqf, pv, vqf, ef, ra
    (64, 8, 4, 2, 2, 3, 5, 5),
    (600, 32, 8, 2, 4, 3, 5, 5),
    (500, 128, 32, 2, 4, 3, 5, 5),
    (300, 12, 5, 2, 3, 2, 1, 2),   # small visited list: fills up, the visit queue stops being fed
    (200, 10, 2, 2, 4, 1, 2, 3),   # visit queue shorter than the visit count
    (400, 768, 16, 2, 4, 3, 5, 5),
    (500, 1536, 24, 3, 4, 3, 5, 5),  # the reference's default configuration at its default dimension
    (900, 384, 48, 2, 4, 3, 5, 5),   # degree 48, queue 96: candidate rows of 384 slots (not a power of two)
    (700, 20, 6, 2, 1, 3, 5, 5),     # one visit per iteration
    (700, 20, 3, 2, 9, 4, 2, 4),     # more visits than a power of two
]


@pytest.mark.parametrize("n,dim,beam,bqf,pv,vqf,ef,ra", BEAM_CASES)
@pytest.mark.parametrize("fused", [True, False, "windows"])
def test_closest_vectors_build_step(n, dim, beam, bqf, pv, vqf, ef, ra, fused):
    """fused: one launch per iteration (the default); False: the loop statement by statement on the
    single-purpose kernels; "windows": the iterations between two progress checks in one launch."""
    say(f"closest_vectors n={n} dim={dim} beam={beam} fused={fused}")
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_WINDOWS, closest_vectors, closest_vectors_stepwise, excluding_self

    rng = np.random.default_rng(n + dim)
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, visit_queue_factor=vqf,
            exclude_factor=ef, speculative_readahead=ra)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    lo, hi = 3, n - 2
    oq = orc.Queue(hi - lo, ql, ql + ql * pv)
    oq.insert(beams[lo:hi], d[lo:hi])
    t_want = orc.closest_vectors(v[lo:hi], oq, v, beams, c, orc.excluding_self(lo, hi))

    gv, gb = dev(v), dev(beams)
    gq = Queue(hi - lo, ql, ql + ql * pv)
    gq.insert(gb[lo:hi], dev(d)[lo:hi])
    if fused == "windows":
        t_got = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi), flags=BEAM_WINDOWS)
    else:
        fn = closest_vectors if fused else closest_vectors_stepwise
        t_got = fn(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi))
    assert t_got == t_want
    assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
    assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))


@pytest.mark.parametrize("windows", [False, True])
@pytest.mark.parametrize("ra,ef,vqf", [(5, 2, 2), (1, 1, 2), (2, 3, 1), (3, 1, 3)])
def test_closest_vectors_many_rows_short_visited_list(ra, ef, vqf, windows):
    """Thousands of rows per launch with a visited list that fills up after a few iterations:
    the batch-wide state (first free column, changed flags) is read and raised by
    workgroups that are in different phases of the same launch."""
    say(f"closest_vectors 30000 rows, readahead={ra} exclude_factor={ef} windows={windows}")
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_WINDOWS, closest_vectors, excluding_self

    rng = np.random.default_rng(77 + ra)
    n, dim, beam, bqf, pv = 30000, 8, 4, 2, 4
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, visit_queue_factor=vqf,
            exclude_factor=ef, speculative_readahead=ra)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    oq = orc.Queue(n, ql, ql + ql * pv)
    oq.insert(beams, d)
    t_want = orc.closest_vectors(v, oq, v, beams, c, orc.excluding_self(0, n))
    gv, gb = dev(v), dev(beams)
    for attempt in range(3):  # the interleaving of workgroups differs from run to run
        gq = Queue(n, ql, ql + ql * pv)
        gq.insert(gb, dev(d))
        t_got = closest_vectors(gv, gq, gv, gb, c, excluding_self(0, n), flags=BEAM_WINDOWS if windows else 0)
        assert t_got == t_want
        assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
        assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))


@pytest.mark.parametrize("ra", [2, 3, 5, 8])
def test_windows_with_rows_that_start_late_in_a_launch(ra):
    """Several iterations per launch on a batch of more workgroups than the GPU holds at once (3,500 rows
    of 128 threads): rows that start after others of the same launch have finished must not see what those
    wrote for the launch after it (the largest visited-list fill, whose slot is the one an iteration reads
    for "the lists were full an iteration ago" when the launch spans 2, 5, 8, ... iterations)."""
    say(f"windows of {ra} iterations, 3500 rows")
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_WINDOWS, closest_vectors, excluding_self

    rng = np.random.default_rng(4242)
    n, dim, beam, bqf, pv = 6000, 32, 8, 2, 4
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, speculative_readahead=ra)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    lo, hi = 2500, 6000
    oq = orc.Queue(hi - lo, ql, ql + ql * pv)
    oq.insert(beams[lo:hi], d[lo:hi])
    t_want = orc.closest_vectors(v[lo:hi], oq, v, beams, c, orc.excluding_self(lo, hi))
    gv, gb = dev(v), dev(beams)
    gq = Queue(hi - lo, ql, ql + ql * pv)
    gq.insert(gb[lo:hi], dev(d)[lo:hi])
    t_got = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi), flags=BEAM_WINDOWS)
    assert t_got == t_want
    assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
    assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))


@pytest.mark.parametrize("dim,sketch", [(32, False), (64, False), (256, True)])
def test_neighbour_lists_that_share_ids(dim, sketch):
    """A ring graph (node i lists i+1 ... i+W): the four nodes a row visits in one iteration list mostly the
    same ids.  Only one copy of an id is evaluated per iteration - the counters show it, with the distance
    cache off so that nothing else answers a repeat - and the queues equal the oracle's, which evaluates
    every copy as the reference does (kernels.py:238-255)."""
    say(f"neighbour lists that share ids, dim={dim} sketch={sketch}")
    import ctypes

    from vectorlink_gpu import Queue
    from vectorlink_gpu import _native as nv
    from vectorlink_gpu.ann import BEAM_NO_CACHE, closest_vectors, excluding_self
    from vectorlink_gpu.kernels import build_sketch

    rng = np.random.default_rng(99 + dim)
    n, beam, bqf, pv = 3000, 8, 2, 4
    # rows that change slowly along the ring, so that a search walks along it and keeps visiting neighbours
    steps = rng.standard_normal((n, dim)).astype(np.float32) * 0.05
    v = np.cumsum(steps, axis=0) + rng.standard_normal(dim).astype(np.float32)
    v = (v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv)
    ql = beam * bqf
    ring = ((np.arange(n, dtype=np.int64)[:, None] + np.arange(1, ql + 1)[None, :]) % n).astype(np.int32)
    d = orc.calculate_distances(v, ring)
    lo, hi = 100, 1300
    oq = orc.Queue(hi - lo, ql, ql + ql * pv)
    oq.insert(ring[lo:hi], d[lo:hi])
    t_want = orc.closest_vectors(v[lo:hi], oq, v, ring, c, orc.excluding_self(lo, hi))
    gv, gb = dev(v), dev(ring)
    gq = Queue(hi - lo, ql, ql + ql * pv)
    gq.insert(gb[lo:hi], dev(d)[lo:hi])
    out = (ctypes.c_double * 9)()
    nv.lib().vl_beam_profile(1, 1, out)
    try:
        t_got = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi), flags=BEAM_NO_CACHE,
                                sketch=build_sketch(gv) if sketch else None)
    finally:
        nv.lib().vl_beam_profile(0, 1, out)
    (fetched, wanted, sketched) = (out[4], out[7], out[8])
    say(f"  iterations {t_got}, candidates {wanted:.0f}, through the sketch {sketched:.0f}, rows fetched {fetched:.0f}")
    assert t_got == t_want
    assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
    assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))
    # four overlapping lists of 16 hold at most 19 + ... distinct ids of 64: well under half are looked at
    assert 0 < fetched < 0.6 * wanted and sketched < 0.6 * wanted
    assert (sketched > 0) == sketch


def test_generate_ann_and_search_against_oracle():
    say("generate_ann + search, n=1500")
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(14)
    n, dim = 1500, 24
    v = unit(rng, n, dim)
    kw = dict(beam_size=12, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=400, optimization_loops=2)
    c = cfg(**kw)
    wb, wd = orc.generate_ann(v, c)
    ann = ANN(dev(v), **kw)
    assert np.array_equal(host(ann.beams), wb)
    assert np.array_equal(bits(host(ann.distances)), bits(wd))
    qv = unit(rng, 100, dim)
    res = ann.search(dev(qv))
    want = orc.search(v, wb, qv, c)
    L = want.length
    assert np.array_equal(host(res.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(res.distances)[:, :L]), bits(want.distances[:, :L]))
    assert ann.recall(300) == orc.ann_calculate_recall(v, wb, c, sample=v[:300])
    # a longer search queue than configured
    res = ann.search(dev(qv), queue_size=40)
    want = orc.search(v, wb, qv, c, queue_size=40)
    assert np.array_equal(host(res.indices)[:, :40], want.indices[:, :40])
    # resume from a stored graph (ann.py:391-396)
    again = ANN(dev(v), beams=ann.beams, **kw)
    assert np.array_equal(bits(host(again.distances)), bits(wd))


def test_layered_search_against_oracle():
    say("search_layers / hnsw_calculate_recall")
    from vectorlink_gpu.ann import ann_recall_test, hnsw_calculate_recall, initial_queue, search_layers

    rng = np.random.default_rng(16)
    n, dim = 1200, 16
    v = unit(rng, n, dim)
    c = cfg(beam_size=8, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=500, optimization_loops=2)
    fine, _ = orc.generate_ann(v, c)
    coarse = orc.generate_circulant_beams(n, orc.primes(5))          # a narrower table as the first layer
    want = orc.initial_queue(v[:300], c)
    orc.search_layers([coarse, fine], v[:300], want, v, c)
    got = initial_queue(dev(v[:300]), c)
    search_layers([dev(coarse), dev(fine)], dev(v[:300]), got, dev(v), c)
    L = want.length
    assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L]))
    assert hnsw_calculate_recall(dev(v), [dev(coarse), dev(fine)], c, sample=dev(v[:300]), verbose=False) == \
        orc.hnsw_calculate_recall(v, [coarse, fine], c, sample=v[:300])
    assert ann_recall_test(dev(v), c) == orc.ann_calculate_recall(v, fine, c, sample=v)


def test_generate_ann_stale_distance_mode():
    from vectorlink_gpu.ann import generate_ann

    rng = np.random.default_rng(15)
    v = unit(rng, 400, 12)
    c = cfg(beam_size=6, beam_queue_factor=2, batch_size=150, optimization_loops=2, prune=True)
    wb, wd = orc.generate_ann(v, c, stale_distances=True)
    gb, gd = generate_ann(dev(v), c, stale_distances=True)
    assert np.array_equal(host(gb), wb) and np.array_equal(bits(host(gd)), bits(wd))


# ---------------------------------------------------------------- exact kNN tiles
@pytest.mark.parametrize("n,dim,nq,k", [(5000, 128, 300, 10), (3000, 768, 129, 10), (1000, 20, 7, 16), (700, 36, 260, 1),
                                        (130, 8, 5, 10), (20000, 64, 64, 10),
                                        # odd numbers of 32-float stages, ragged last stages, every list length
                                        (4000, 96, 200, 4), (2500, 160, 130, 8), (6000, 100, 50, 12), (300, 32, 1, 16),
                                        (50000, 32, 1000, 10), (90, 4, 3, 2)])
def test_knn_exact(n, dim, nq, k):
    say(f"knn_exact n={n} dim={dim} nq={nq} k={k}")
    from vectorlink_gpu.kernels import knn_exact

    rng = np.random.default_rng(n + dim)
    v = unit(rng, n, dim)
    q = unit(rng, nq, dim)
    q[0] = v[17]  # an exact hit at distance 0
    wi, wd = orc.knn_exact(q, v, k)
    gi, gd = knn_exact(dev(q), dev(v), k)
    gi, gd = host(gi), host(gd)
    assert np.allclose(gd, wd, rtol=1e-5, atol=1e-6)
    assert gi[0, 0] == 17
    assert (np.diff(gd, axis=1) >= 0).all()
    # ids agree except where two distances are closer than float32 MFMA rounding can order
    mism = gi != wi
    assert mism.mean() < 0.01
    for r, c in zip(*np.nonzero(mism)):
        d_true = (1 - float(np.dot(q[r].astype(np.float64), v[gi[r, c]]))) / 2
        assert abs(d_true - wd[r, c]) < 2e-6
    for r in range(nq):
        assert len(set(gi[r].tolist())) == k


# ---------------------------------------------------------------- dense seeding (addition)
def test_dense_seeded_search():
    say("dense seeded search")
    from vectorlink_gpu import ANN
    from vectorlink_gpu.ann import entry_point_ids

    rng = np.random.default_rng(21)
    n, dim, nq = 3000, 32, 90
    centres = unit(rng, 30, dim)
    v = centres[rng.integers(0, 30, n)] + 0.05 * rng.standard_normal((n, dim)).astype(np.float32)
    v = (v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    q = centres[rng.integers(0, 30, nq)] + 0.05 * rng.standard_normal((nq, dim)).astype(np.float32)
    q = (q / np.linalg.norm(q, axis=1, keepdims=True)).astype(np.float32)
    kw = dict(beam_size=12, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=1000, optimization_loops=2)
    c = cfg(**kw)
    ann = ANN(dev(v), seeding="dense", entry_points=500, **kw)
    eids = host(entry_point_ids(n, 500))
    assert np.array_equal(eids, (np.arange(500, dtype=np.int64) * n) // 500)
    res = ann.search(dev(q))
    L = res.length
    gi = host(res.indices)
    # the seeds the GPU picked = the 16 nearest entry points (exact, up to float32 near-ties)
    wi, wd = orc.knn_exact(q, v[eids], 16)
    seeds_want = eids[wi]
    # replay on the oracle from the oracle's seeds: identical answer unless a near-tie changed the seed set
    oq = orc.Queue(nq, L, res.indices.shape[1])
    oq.insert(seeds_want.astype(np.int32), orc.gather_distances(q, v, seeds_want.astype(np.int32)))
    orc.closest_vectors(q, oq, v, host(ann.beams), c, None)
    same = (gi[:, :L] == oq.indices[:, :L]).all(axis=1)
    assert same.mean() > 0.97
    assert np.array_equal(bits(host(res.distances)[same, :L]), bits(oq.distances[same, :L]))
    # and it finds the true neighbours where circulant seeding cannot
    t10, _ = orc.knn_exact(q, v, 10)
    rec_dense = np.mean([len(set(a) & set(b)) / 10 for a, b in zip(gi[:, :10].tolist(), t10.tolist())])
    rec_circ = ann.recall_at_k(dev(q), 10, seeding="circulant")
    assert rec_dense > 0.9 and rec_dense == pytest.approx(ann.recall_at_k(dev(q), 10), abs=0.02)
    assert rec_dense >= rec_circ


# ---------------------------------------------------------------- rank-based graph optimisation (addition)
@pytest.mark.parametrize("n,w,d", [(40, 8, 4), (300, 12, 6), (1000, 64, 32), (700, 128, 64), (200, 6, 6), (50, 5, 1)])
def test_optimize_graph(n, w, d):
    say(f"optimize_graph n={n} w={w} d={d}")
    from vectorlink_gpu.kernels import optimize_graph

    rng = np.random.default_rng(n + w)
    beams = np.stack([rng.choice([j for j in range(n) if j != i], w, replace=False) for i in range(n)]).astype(np.int32)
    beams[rng.random((n, w)) < 0.05] = M
    beams = np.stack([np.concatenate([r[r != M], r[r == M]]) for r in beams])
    want = orc.optimize_graph(beams, d)
    got = host(optimize_graph(dev(beams), d))
    assert np.array_equal(got, want)


def test_optimize_graph_with_hubs():
    """Rows that thousands of others point at from their first slots: the reverse pass keeps only the first few
    sources of a row in (slot, source) order and must find them among more edges than it sorts at a time,
    whatever order the edges were scattered in."""
    say("optimize_graph with hubs")
    from vectorlink_gpu.kernels import optimize_graph

    rng = np.random.default_rng(8)
    n, w, d = 6000, 12, 8
    beams = np.stack([rng.choice(n, size=w, replace=False) for _ in range(n)]).astype(np.int32)
    beams[:, 0] = 7                      # every row points at row 7 from slot 0 ...
    beams[::2, 1] = 11                   # ... half of them at row 11 from slot 1 ...
    beams[rng.random(n) < 0.3, 2] = 7    # ... and some at row 7 again from slot 2 (an id twice in a row)
    beams[7, 0], beams[11, 1] = 8, 12
    want = orc.optimize_graph(beams, d)
    for _ in range(3):                   # the scatter's order differs from run to run; the result must not
        got = host(optimize_graph(dev(beams), d))
        assert np.array_equal(got, want)


def test_rank_pruned_build():
    say("build with prune='rank'")
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(31)
    n, dim = 1200, 16
    v = unit(rng, n, dim)
    kw = dict(beam_size=8, beam_queue_factor=3, recall_search_queue_factor=2, batch_size=500, optimization_loops=2)
    ann = ANN(dev(v), prune="rank", **kw)
    # the oracle's version of the same pipeline: loops without pruning at full width, then optimize_graph
    c = cfg(prune=False, **kw)
    beams = orc.generate_circulant_beams(n, orc.primes(24))
    d = orc.calculate_distances(v, beams)
    for _ in range(2):
        nb, nd = np.empty_like(beams), np.empty_like(d)
        for s in range(0, n, 500):
            e = min(s + 500, n)
            q = orc.Queue(e - s, 24, 24 + 24 * 4)
            q.insert(beams[s:e], d[s:e])
            orc.closest_vectors(v[s:e], q, v, beams, c, orc.excluding_self(s, e))
            nb[s:e], nd[s:e] = q.indices[:, :24], q.distances[:, :24]
        beams, d = nb, nd
        _, rec = orc.ann_calculate_recall(v, np.ascontiguousarray(beams[:, :8]), c, sample=v[:1000])
        if rec == 1.0:
            break
    want = orc.optimize_graph(beams, 8)
    assert np.array_equal(host(ann.beams), want)
    real = want != M
    wd = orc.calculate_distances(v, np.where(real, want, 0).astype(np.int32))
    assert np.array_equal(bits(host(ann.distances)[real]), bits(wd[real]))


def test_exact_duplicate_rows_tie_break_by_id():
    """Exact duplicate vectors (as in the 20M x 384 workload's 2 % duplicates) give exactly equal
    distances; every queue must then order by id, as the oracle does."""
    say("duplicate rows: ties broken by id")
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(41)
    n, dim = 1600, 24
    v = unit(rng, n, dim)
    dup = rng.choice(n, 400, replace=False)
    v[dup] = v[rng.integers(0, n, 400)]            # a quarter of the rows are copies of other rows
    kw = dict(beam_size=10, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=600, optimization_loops=2)
    c = cfg(**kw)
    wb, wd = orc.generate_ann(v, c)
    ann = ANN(dev(v), **kw)
    assert np.array_equal(host(ann.beams), wb)
    assert np.array_equal(bits(host(ann.distances)), bits(wd))
    ties = (np.diff(wd, axis=1) == 0) & (wb[:, 1:] != M)
    assert ties.sum() > 100                          # the case is really exercised
    assert (wb[:, 1:][ties] > wb[:, :-1][ties]).all()
    qv = v[rng.integers(0, n, 64)]
    res = ann.search(dev(qv))
    want = orc.search(v, wb, qv, c)
    L = want.length
    assert np.array_equal(host(res.indices)[:, :L], want.indices[:, :L])


def test_closest_vectors_seeded_configuration_sweep():
    """Forty seeded configurations (sizes, dimensions that are not multiples of 4, queue
    shapes with and without slack, exclusion lists of several columns, search- and
    build-shaped calls) through the fused loop against the oracle."""
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_NO_CACHE, closest_vectors
    from vectorlink_gpu.kernels import build_sketch

    master = np.random.default_rng(2025)
    for case in range(40):
        n = int(master.integers(40, 1500))
        dim = int(master.choice([1, 3, 4, 7, 16, 33, 64, 100, 128, 130, 257, 300]))
        beam = int(master.integers(1, 20))
        width = int(master.choice([beam, beam * int(master.integers(1, 4))]))   # neighbour table columns
        pv = int(master.integers(1, 7))
        vqf = int(master.integers(1, 4))
        ef = int(master.integers(1, 6))
        ra = int(master.integers(1, 7))
        b = int(master.integers(1, min(n, 400)))
        length = int(master.integers(1, 50))
        take = min(vqf * beam, pv)
        cap = length + max(take * width, min(length, n)) + int(master.choice([0, 0, 5, 40]))
        excl_cols = int(master.choice([0, 1, 3]))
        say(f"sweep {case}: n={n} dim={dim} beam={beam} width={width} pv={pv} vqf={vqf} ef={ef} ra={ra} rows={b} "
            f"length={length} cap={cap} excl={excl_cols}")
        rng = np.random.default_rng(1000 + case)
        v = unit(rng, n, dim)
        q = unit(rng, b, dim)
        c = cfg(beam_size=beam, parallel_visit_count=pv, visit_queue_factor=vqf, exclude_factor=ef,
                speculative_readahead=ra)
        table = np.stack([rng.choice(n, width, replace=width > n) for _ in range(n)]).astype(np.int32)
        table[rng.random((n, width)) < 0.05] = M
        seeds = np.stack([rng.choice(n, min(length, n), replace=False) for _ in range(b)]).astype(np.int32)
        sd = orc.gather_distances(q, v, seeds)
        ex = None
        if excl_cols:
            ex = rng.integers(0, n, (b, excl_cols)).astype(np.int32)
            if excl_cols == 3:
                ex[rng.random(b) < 0.5, 1] = M          # lists that end early
        oq = orc.Queue(b, length, cap)
        oq.insert(seeds, sd)
        t_want = orc.closest_vectors(q, oq, v, table, c, ex)
        gq = Queue(b, length, cap)
        gq.insert(dev(seeds), dev(sd))
        t_got = closest_vectors(dev(q), gq, dev(v), dev(table), c, None if ex is None else dev(ex))
        assert t_got == t_want, case
        assert np.array_equal(host(gq.indices)[:, :length], oq.indices[:, :length]), case
        assert np.array_equal(bits(host(gq.distances)[:, :length]), bits(oq.distances[:, :length])), case
        if dim % 4 == 0:
            # the same call through the 8-bit sketch of the vectors, with and without the distance cache
            sk = build_sketch(dev(v))
            for flags in (0, BEAM_NO_CACHE):
                gq = Queue(b, length, cap)
                gq.insert(dev(seeds), dev(sd))
                t_got = closest_vectors(dev(q), gq, dev(v), dev(table), c, None if ex is None else dev(ex), flags=flags,
                                        sketch=sk)
                assert t_got == t_want, (case, flags)
                assert np.array_equal(host(gq.indices)[:, :length], oq.indices[:, :length]), (case, flags)
                assert np.array_equal(bits(host(gq.distances)[:, :length]), bits(oq.distances[:, :length])), (case, flags)


def test_command_line_driver_and_parameter_sweep(tmp_path):
    say("main.py: parse, main, grid_search")
    import importlib.util
    import json
    import os

    from vectorlink_gpu.utils import generate_random_vectors

    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("vl_main", os.path.join(here, "vectorlink-gpu_amd", "main.py"))
    cli = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(cli)
    options = cli.parse(["-c", "1500", "-d", "16", "-n", "8", "-b", "500", "-l", "2", "-P"])
    assert options["vector_count"] == 1500 and options["prune"] is True and options["recall_search_queue_factor"] == 6
    data = generate_random_vectors(number_of_vectors=1500, dimensions=16)
    report = cli.main(data, options)
    assert report["vector_count"] == 1500 and 0.0 <= report["recall"] <= 1.0 and report["total_time"] > 0
    runs = cli.grid_search(vector_count=600, vector_dimension=8, log_dir=str(tmp_path))
    logs = sorted(os.listdir(tmp_path))
    assert runs == 48 and len(logs) == 48
    one = json.load(open(os.path.join(tmp_path, logs[0])))
    assert one["vector_count"] == 600 and "recall" in one


def test_caller_with_a_cuda_default_device():
    """The reference's ANN switches torch's default device to the GPU (ann.py:373-375); a caller who
    has done the same must still get CPU-seeded workloads and a working build."""
    say("workload generator and build under torch.set_default_device('cuda')")
    from vectorlink_gpu import ANN, synthetic

    before = torch.get_default_device()
    try:
        torch.set_default_device("cuda")
        base, q, w = synthetic.make("zipf-20m-384", n=3000, queries=16, centres=8)
        assert base.device.type == "cpu" and q.device.type == "cpu"
        again, _, _ = synthetic.make("zipf-20m-384", n=3000, queries=16, centres=8)
        ann = ANN(base, beam_size=8, beam_queue_factor=2, batch_size=1000, optimization_loops=1)
        res = ann.search(q)
    finally:
        torch.set_default_device(before)
    assert torch.equal(base, again)
    assert ann.beams.shape == (3000, 8) and res.indices.shape[0] == 16


def test_two_host_threads_on_two_streams():
    """Two beam searches in flight at once, one host thread and one stream each: each call owns the
    scratch memory of its (device, stream), so both must equal the oracle, as must two threads that
    share the default stream (serialised by the workspace lock)."""
    say("closest_vectors from two host threads")
    import threading

    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import closest_vectors, excluding_self

    rng = np.random.default_rng(4242)
    n, dim, beam, bqf, pv = 6000, 32, 8, 2, 4
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    parts = [(0, 2500), (2500, 6000)]
    want = []
    for (lo, hi) in parts:
        oq = orc.Queue(hi - lo, ql, ql + ql * pv)
        oq.insert(beams[lo:hi], d[lo:hi])
        t = orc.closest_vectors(v[lo:hi], oq, v, beams, c, orc.excluding_self(lo, hi))
        want.append((t, oq))
    gv, gb, gd = dev(v), dev(beams), dev(d)
    torch.cuda.synchronize()

    for own_stream in (True, False):
        got = [None, None]
        errors = []

        def work(i):
            try:
                (lo, hi) = parts[i]
                stream = torch.cuda.Stream() if own_stream else torch.cuda.current_stream()
                with torch.cuda.stream(stream):
                    gq = Queue(hi - lo, ql, ql + ql * pv)
                    gq.insert(gb[lo:hi], gd[lo:hi])
                    t = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi))
                    stream.synchronize()
                got[i] = (t, host(gq.indices), host(gq.distances))
            except Exception as e:  # surfaces in the main thread below
                errors.append(e)

        threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
        for th in threads:
            th.start()
        for th in threads:
            th.join(timeout=120)
        assert not any(th.is_alive() for th in threads), "a beam search did not return"
        assert not errors, errors
        for i in range(2):
            (t_want, oq) = want[i]
            assert got[i][0] == t_want
            assert np.array_equal(got[i][1][:, :ql], oq.indices[:, :ql])
            assert np.array_equal(bits(got[i][2][:, :ql]), bits(oq.distances[:, :ql]))


def test_hand_enumerated_chain_on_the_gpu():
    """The twelve-node chain of tests/test_oracle_search.py, whose trace is written out by hand there:
    six iterations, nodes 11 and 10 at 1/16 and 2/16; eight nodes with node 6 excluded: four, nodes 7 and 5."""
    say("hand-enumerated chain")
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_PER_QUERY_STOP, BEAM_SORT_MERGE, closest_vectors

    c = cfg(beam_size=2, parallel_visit_count=1, visit_queue_factor=1, exclude_factor=2, speculative_readahead=1)
    for (n, excl, flags, t_want, ids_want, d_want) in [
            (12, None, 0, 6, [11, 10], [1 / 16, 2 / 16]), (12, None, BEAM_SORT_MERGE, 6, [11, 10], [1 / 16, 2 / 16]),
            (8, None, 0, 4, [7, 6], [1 / 16, 2 / 16]), (8, [[6]], 0, 4, [7, 5], [1 / 16, 3 / 16]),
            (12, None, BEAM_PER_QUERY_STOP, 5, [11, 10], [1 / 16, 2 / 16]),
            (8, None, BEAM_PER_QUERY_STOP, 4, [7, 6], [1 / 16, 2 / 16])]:
        delta = np.array([(n - i) / 16.0 for i in range(n)], dtype=np.float32)
        v = (1.0 - 2.0 * delta).reshape(n, 1).astype(np.float32)
        table = np.array([[(i + 1) % n, (i + 2) % n] for i in range(n)], dtype=np.int32)
        q = Queue(1, 2, 4)
        q.insert(dev(np.array([[0, 1]], dtype=np.int32)), dev(np.array([[delta[0], delta[1]]], dtype=np.float32)))
        ex = None if excl is None else dev(np.array(excl, dtype=np.int32))
        t = closest_vectors(dev(np.ones((1, 1), dtype=np.float32)), q, dev(v), dev(table), c, ex, flags=flags)
        assert t == t_want, (n, excl, flags)
        assert host(q.indices)[0, :2].tolist() == ids_want and host(q.distances)[0, :2].tolist() == d_want


@pytest.mark.parametrize("windows", [False, True])
@pytest.mark.parametrize("n,dim,beam,bqf,pv,vqf,ef,ra", BEAM_CASES)
def test_per_query_stop_against_its_model(n, dim, beam, bqf, pv, vqf, ef, ra, windows):
    """VL_BEAM_PER_QUERY_STOP against the CPU model that defines it (oracle.closest_vectors_per_query):
    same iteration count, ids and distance bits, on a build step with self exclusion; also with several
    iterations per launch."""
    say(f"per-query stop n={n} dim={dim} beam={beam} windows={windows}")
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_PER_QUERY_STOP, BEAM_WINDOWS, closest_vectors, excluding_self

    rng = np.random.default_rng(1000 + n + dim)
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, visit_queue_factor=vqf,
            exclude_factor=ef, speculative_readahead=ra)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    lo, hi = 3, n - 2
    oq = orc.Queue(hi - lo, ql, ql + ql * pv)
    oq.insert(beams[lo:hi], d[lo:hi])
    t_want = orc.closest_vectors_per_query(v[lo:hi], oq, v, beams, c, orc.excluding_self(lo, hi))
    gv, gb = dev(v), dev(beams)
    gq = Queue(hi - lo, ql, ql + ql * pv)
    gq.insert(gb[lo:hi], dev(d)[lo:hi])
    t_got = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi),
                            flags=BEAM_PER_QUERY_STOP | (BEAM_WINDOWS if windows else 0))
    assert t_got == t_want
    assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
    assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))


def test_per_query_stop_search_quality_and_cost():
    """ANN.search(stop="per_query") equals its model on a built graph, needs no more iterations than the
    reference's batch-wide stop needs, and loses little recall against it."""
    say("per-query stop: search on a built graph")
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(31)
    n, dim = 6000, 48
    v = unit(rng, n, dim)
    qv = unit(rng, 500, dim)
    kw = dict(beam_size=16, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=2000, optimization_loops=2)
    ann = ANN(dev(v), **kw)
    c = cfg(**kw)
    wb = host(ann.beams)
    want = orc.search(v, wb, qv, c, stop="per_query")
    got = ann.search(dev(qv), stop="per_query")
    L = want.length
    assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L]))
    full = ann.search(dev(qv))
    truth, _ = orc.knn_exact(qv, v, 10)

    def recall(ids):
        return np.mean([len(set(a[:10].tolist()) & set(t.tolist())) / 10 for a, t in zip(ids, truth)])

    (r_own, r_batch) = (recall(host(got.indices)), recall(host(full.indices)))
    say(f"  recall@10 per-query stop {r_own:.4f}, batch-wide stop {r_batch:.4f}")
    assert r_own > r_batch - 0.10   # iid rows, query-independent seeds: the hardest case for an early stop


# ---------------------------------------------------------------- squared L2 (an addition: not in the reference)
@pytest.mark.parametrize("dim", [1, 7, 64, 128, 130, 384, 768, 1030, 1536, 2500])
def test_l2_gather_distances_bit_exact(dim):
    say(f"L2 gather dim={dim}")
    from vectorlink_gpu.kernels import gather_distances, search_from_seeds

    rng = np.random.default_rng(70 + dim)
    n, rows, w = 300, 37, 21
    v = (rng.standard_normal((n, dim)) * rng.uniform(0.5, 3.0, (n, 1))).astype(np.float32)   # rows of any length
    q = rng.standard_normal((rows, dim)).astype(np.float32)
    ids = rng.integers(0, n, (rows, w)).astype(np.int32)
    ids[2, 3] = M
    with orc.metric("l2"):
        want = orc.gather_distances(q, v, ids)
        visit = rng.integers(0, n, (rows, 3)).astype(np.int32)
        table = rng.integers(0, n, (n, 6)).astype(np.int32)
        (wi, wd) = orc.search_from_seeds(q, visit, table, v)
    got = gather_distances(dev(q), dev(v), dev(ids), metric="l2")
    assert np.array_equal(bits(host(got)), bits(want))
    ref = ((q[:, None, :].astype(np.float64) - v[np.where(ids == M, 0, ids)]) ** 2).sum(2)
    ok = ids != M
    assert np.allclose(host(got)[ok], ref[ok], rtol=1e-5)
    (gi, gd) = search_from_seeds(dev(q), dev(visit), dev(table), dev(v), metric="l2")
    assert np.array_equal(host(gi), wi) and np.array_equal(bits(host(gd)), bits(wd))


def test_l2_build_and_search_against_oracle():
    """ANN(metric="l2") on rows of unequal length: graph, distances and search queues equal the oracle's
    under its L2 switch."""
    say("L2 build + search")
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(91)
    n, dim = 3000, 40
    v = (rng.standard_normal((n, dim)) * rng.uniform(0.7, 1.5, (n, 1))).astype(np.float32)
    qv = rng.standard_normal((100, dim)).astype(np.float32)
    kw = dict(beam_size=12, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=1100, optimization_loops=2)
    c = cfg(**kw)
    ann = ANN(dev(v), metric="l2", **kw)
    got = ann.search(dev(qv))
    with orc.metric("l2"):
        (wb, wd) = orc.generate_ann(v, c)
        want = orc.search(v, wb, qv, c)
    assert np.array_equal(host(ann.beams), wb) and np.array_equal(bits(host(ann.distances)), bits(wd))
    L = want.length
    assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L]))
    # the answers are near the exact L2 neighbours
    d2 = ((qv[:, None, :].astype(np.float64) - v[None, :, :]) ** 2).sum(2)
    truth = np.argsort(d2, axis=1)[:, :10]
    rec = np.mean([len(set(a[:10].tolist()) & set(t.tolist())) / 10 for a, t in zip(host(got.indices), truth)])
    assert rec > 0.8
    # dense seeding and recall@k follow the metric: the seeds are the nearest entry points by L2
    dense = ann.search(dev(qv), seeding="dense")
    found = host(dense.indices)[:, :10]
    rec_dense = np.mean([len(set(a.tolist()) & set(t.tolist())) / 10 for a, t in zip(found, truth)])
    assert rec_dense > 0.8
    assert abs(ann.recall_at_k(dev(qv), 10, seeding="dense") - rec_dense) < 1e-9


@pytest.mark.parametrize("n,dim,nq,k", [(5000, 128, 300, 10), (3000, 768, 129, 10), (1000, 20, 7, 16), (700, 36, 260, 1),
                                        (6000, 100, 50, 12), (90, 4, 3, 2), (20000, 64, 64, 10)])
def test_knn_exact_l2(n, dim, nq, k):
    """Rows of unequal length, so the L2 order differs from the cosine order; truth is a float64
    brute force that subtracts first."""
    say(f"knn_exact L2 n={n} dim={dim} nq={nq} k={k}")
    from vectorlink_gpu.kernels import knn_exact

    rng = np.random.default_rng(3 * n + dim)
    v = (rng.standard_normal((n, dim)) * rng.uniform(0.5, 2.0, (n, 1))).astype(np.float32)
    q = (rng.standard_normal((nq, dim)) * rng.uniform(0.5, 2.0, (nq, 1))).astype(np.float32)
    q[0] = v[17]  # an exact hit
    with orc.metric("l2"):
        wi, wd = orc.knn_exact(q, v, k)
    d2 = ((q[:, None, :].astype(np.float64) - v[None, :, :].astype(np.float64)) ** 2).sum(2) if n * nq * dim < 3e8 else None
    if d2 is not None:  # the oracle against numpy
        order = np.argsort(d2, axis=1, kind="stable")[:, :k]
        assert np.array_equal(order, wi)
    ci, _ = knn_exact(dev(q), dev(v), k)
    gi, gd = knn_exact(dev(q), dev(v), k, metric="l2")
    gi, gd = host(gi), host(gd)
    assert not np.array_equal(host(ci), gi)  # the metric matters on these rows
    # |q|^2 + |v|^2 - 2 q.v carries the rounding of the squared lengths
    scale = (q.astype(np.float64) ** 2).sum(1)[:, None] + (v.astype(np.float64) ** 2).sum(1).max()
    tol = 4e-6 * scale
    assert (np.abs(gd - wd) <= tol).all()
    assert gi[0, 0] == 17
    assert (np.diff(gd, axis=1) >= 0).all()
    mism = gi != wi
    assert mism.mean() < 0.02
    for r, c in zip(*np.nonzero(mism)):
        d_true = ((q[r].astype(np.float64) - v[gi[r, c]]) ** 2).sum()
        assert abs(d_true - wd[r, c]) <= 2 * tol[r, 0]
    for r in range(nq):
        assert len(set(gi[r].tolist())) == k


def test_self_recall_with_a_sample_that_is_not_the_head_of_the_vectors():
    """ann_calculate_recall seeds row i with ids over the SAMPLE and distances between sample rows
    (ann.py:196-208), then searches `vectors`: for a sample taken from the middle an id carries two
    distances.  The Python layer then picks the whole-row-sort form of the loop; same answer as the oracle."""
    say("self-recall over a middle slice")
    from vectorlink_gpu.ann import ann_calculate_recall

    rng = np.random.default_rng(57)
    n, dim = 1200, 24
    v = unit(rng, n, dim)
    c = cfg(beam_size=8, beam_queue_factor=2, recall_search_queue_factor=2)
    table = orc.generate_circulant_beams(n, orc.primes(8))
    for (lo, hi) in ((0, 300), (500, 800)):
        want = orc.ann_calculate_recall(v, table, c, sample=v[lo:hi])
        got = ann_calculate_recall(dev(v), dev(table), c, sample=dev(v)[lo:hi])
        assert tuple(got) == tuple(want), (lo, hi)


def test_dedup_sort():
    """utils.dedup_sort (utils.py:85-89): sort, punch out neighbouring duplicates, sort: each row ends up as its
    distinct ids in ascending order followed by empty ids."""
    say("dedup_sort")
    from vectorlink_gpu.utils import dedup_sort

    rng = np.random.default_rng(58)
    rows = rng.integers(0, 40, (50, 33)).astype(np.int32)
    rows[3, :5] = M
    got = host(dedup_sort(dev(rows)))
    for r in range(rows.shape[0]):
        distinct = sorted(set(int(x) for x in rows[r] if x != M))
        assert got[r].tolist() == distinct + [M] * (rows.shape[1] - len(distinct))


def test_build_does_not_depend_on_the_batches_in_flight():
    """GraphBuild keeps several batches of a loop in flight on streams of their own; one, two and three give
    the same graph, the oracle's."""
    say("build with 1, 2, 3 batches in flight")
    from vectorlink_gpu.ann import generate_ann

    rng = np.random.default_rng(61)
    n, dim = 4000, 20
    v = unit(rng, n, dim)
    c = cfg(beam_size=8, beam_queue_factor=2, batch_size=700, optimization_loops=2)
    (wb, wd) = orc.generate_ann(v, c)
    for lanes in (1, 2, 3):
        (gb, gd) = generate_ann(dev(v), c, concurrent_batches=lanes)
        assert np.array_equal(host(gb), wb), lanes
        assert np.array_equal(bits(host(gd)), bits(wd)), lanes


def test_dense_seeding_ranked_by_leading_columns():
    """ANN(seed_dims=k) ranks the entry points by their first k columns only; the queue still holds full
    distances (those of the gathered-distance kernel) and the search still finds the neighbours."""
    say("dense seeding on leading columns")
    from vectorlink_gpu import ANN
    from vectorlink_gpu.kernels import gather_distances

    rng = np.random.default_rng(77)
    n, dim = 5000, 64
    v = unit(rng, n, dim)
    qv = unit(rng, 200, dim)
    kw = dict(beam_size=16, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=2500, optimization_loops=2)
    full = ANN(dev(v), seeding="dense", entry_points=512, **kw)
    part = ANN(dev(v), beams=full.beams, distances=full.distances, seeding="dense", entry_points=512, seed_dims=16, **kw)
    a, b = full.search(dev(qv)), part.search(dev(qv))
    L = b.length
    ids = b.indices[:, :L].contiguous()
    real = ids != M
    want = gather_distances(dev(qv), dev(v), torch.where(real, ids, torch.zeros_like(ids)))
    assert torch.equal(want[real], b.distances[:, :L][real])
    truth, _ = orc.knn_exact(qv, v, 10)

    def recall(q):
        return np.mean([len(set(x[:10].tolist()) & set(t.tolist())) / 10 for x, t in zip(host(q.indices), truth)])

    say(f"  recall@10 all columns {recall(a):.3f}, 16 of 64 columns {recall(b):.3f}")
    assert recall(b) > recall(a) - 0.05

    # ANN(dense_seeds=k): a query starts from its k nearest entry points only - the oracle's loop from that very
    # queue gives the same rows
    few = ANN(dev(v), beams=full.beams, distances=full.distances, seeding="dense", entry_points=512, dense_seeds=3, **kw)
    from vectorlink_gpu.ann import dense_search_queue
    (entry_ids, entry_vectors) = few._entry_tables()
    start = dense_search_queue(dev(v), dev(qv), few.configuration, entry_ids, entry_vectors, None, 3)
    L = start.length
    assert ((start.indices[:, :L] != M).sum(dim=1) == 3).all()
    oq = orc.Queue(len(qv), L, start.indices.size(1))
    oq.insert(host(start.indices)[:, :3], host(start.distances)[:, :3])
    c = cfg(**kw)
    t_want = orc.closest_vectors(qv, oq, v, host(full.beams), c, None)
    got = few.search(dev(qv))
    assert np.array_equal(host(got.indices)[:, :L], oq.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(oq.distances[:, :L]))
    say(f"  3 seeds per query: {t_want} iterations, recall@10 {recall(got):.3f}")
    assert recall(got) > recall(a) - 0.05


def test_queues_beyond_64_kib_of_lds():
    """Degree 256 with a build queue of 512: 2048 candidates per iteration, a visit queue of 768 and a visited
    list of 3840 ids need about 90 KB of LDS per row, more than a kernel gets by default; the fused step, the
    two-launch form and the queue kernels ask for it."""
    say("queues that need more than 64 KiB of LDS")
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import BEAM_TWO_LAUNCHES, closest_vectors, excluding_self

    rng = np.random.default_rng(333)
    n, dim, beam, bqf, pv = 1300, 8, 256, 2, 4
    v = unit(rng, n, dim)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv)
    ql = beam * bqf
    table = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, table)
    lo, hi = 100, 148
    oq = orc.Queue(hi - lo, ql, ql + ql * pv)
    oq.insert(table[lo:hi], d[lo:hi])
    t_want = orc.closest_vectors(v[lo:hi], oq, v, table, c, orc.excluding_self(lo, hi))
    gv, gb = dev(v), dev(table)
    for flags in (0, BEAM_TWO_LAUNCHES):
        gq = Queue(hi - lo, ql, ql + ql * pv)
        gq.insert(gb[lo:hi], dev(d)[lo:hi])
        t_got = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi), flags=flags)
        assert t_got == t_want, flags
        assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql]), flags
        assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql])), flags


# ---------------------------------------------------------------- 8-bit sketch
@pytest.mark.parametrize("dim", [4, 20, 64, 100, 128, 384, 768, 1000, 1536, 2048])
def test_sketch_rows_bound_every_dot_product(dim):
    """build_sketch: the bytes are the row rounded to 8 bits under the row's own scale, and the tail's two
    bounds hold against float64 - the 2-norm of what the rounding moved, and the row's 2-norm.  Then, for
    random queries, |<q, v> - scale * <q, u>| <= ||q|| * bound, which is what the search relies on."""
    say(f"sketch rows dim={dim}")
    from vectorlink_gpu.kernels import build_sketch, sketch_parts, sketch_row_bytes

    rng = np.random.default_rng(dim)
    n = 300
    v = unit(rng, n, dim)
    v[1] = 0.0                               # an all-zero row
    v[2] *= 37.5                             # not a unit row
    v[3, ::2] = 0.0
    v[4] = np.float32(1e-30) * v[4]          # tiny
    if dim > 4:
        v[5, 3] = np.nan                     # promises nothing
        v[6, 1] = np.inf
    rb = sketch_row_bytes(dim)
    pad = 16 * ((dim + 15) // 16)
    assert rb == pad + 8
    sk = build_sketch(dev(v))
    assert tuple(sk.shape) == (n, rb)
    (data, scale, resid, norm) = (host(x) for x in sketch_parts(sk))
    assert data.shape == (n, pad) and np.all(data[:, dim:] == 0)
    u = data[:, :dim].astype(np.float64)
    scale, resid, norm = scale.astype(np.float64), resid.astype(np.float64), norm.astype(np.float64)
    bad = ~np.isfinite(v).all(axis=1)
    assert np.all(np.isinf(resid[bad])) and np.all(np.isinf(norm[bad]))
    ok = ~bad
    v64 = v[ok].astype(np.float64)
    assert np.all(np.abs(u[ok]) <= 127)
    moved = np.linalg.norm(v64 - scale[ok, None] * u[ok], axis=1)
    assert np.all(resid[ok] >= moved)
    assert np.all(norm[ok] >= np.linalg.norm(v64, axis=1))
    # tight: rounding moves an element by at most half a step, and the bounds are within 0.3 % of the truth (they
    # are kept as halves, rounded up: 0.1 % at most, and never below the smallest half, 6e-8)
    assert np.all(moved <= 0.5 * scale[ok] * np.sqrt(dim) * (1 + 1e-6) + 1e-30)
    assert np.all(resid[ok] <= moved * 1.003 + 6e-8) and np.all(norm[ok] <= np.linalg.norm(v64, axis=1) * 1.003 + 6e-8)
    mx = np.abs(v64).max(axis=1)
    assert np.allclose(scale[ok], mx / 127.0, rtol=1e-6, atol=0)
    q = unit(rng, 50, dim).astype(np.float64)
    exact = q @ v64.T
    approx = (q @ u[ok].T) * scale[ok][None, :]
    assert np.all(np.abs(exact - approx) <= np.linalg.norm(q, axis=1)[:, None] * resid[ok][None, :] + 1e-12)


SKETCH_CASES = [
    # n, dim, beam, bqf, pv, vqf, ef, ra
    (700, 16, 4, 2, 2, 3, 5, 5),       # one chunk per sketch row
    (900, 64, 8, 2, 4, 3, 5, 5),
    (1200, 100, 8, 2, 4, 3, 5, 5),     # a last chunk that is only partly data
    (2000, 128, 32, 2, 4, 3, 5, 5),    # the 128-column benchmark shape
    (1500, 256, 16, 2, 4, 3, 5, 5),
    (1500, 384, 48, 2, 4, 3, 5, 5),
    (1200, 512, 16, 2, 4, 3, 5, 5),
    (2000, 768, 64, 2, 4, 3, 5, 5),    # the 768-column benchmark shape
    (1200, 1024, 16, 2, 4, 3, 5, 5),
    (800, 1280, 8, 2, 3, 3, 5, 2),
    (1200, 1536, 24, 3, 4, 3, 5, 5),
    (600, 1792, 8, 2, 4, 2, 2, 3),     # a visited list that runs full
    (600, 2048, 8, 2, 9, 4, 2, 4),
    (500, 2052, 8, 2, 4, 3, 5, 5),     # beyond the sketch's sizes: ignored
    (500, 130, 8, 2, 4, 3, 5, 5),      # rows that are not 16-byte aligned: ignored
]


@pytest.mark.parametrize("n,dim,beam,bqf,pv,vqf,ef,ra", SKETCH_CASES)
@pytest.mark.parametrize("cache", [False, True, "windows"])
def test_closest_vectors_with_sketch(n, dim, beam, bqf, pv, vqf, ef, ra, cache):
    """The loop with the 8-bit sketch against the oracle: same iteration count, ids and distance bits, without
    the distance cache, with it (a probe then finds exact distances and bounds), and with cache, sketch and
    several iterations per launch (the LDS table in front of the cache).  Every row starts out looking through
    the sketch from its second iteration; the profiling counters show that it was really used."""
    say(f"closest_vectors with sketch n={n} dim={dim} beam={beam} cache={cache}")
    import ctypes

    from vectorlink_gpu import Queue
    from vectorlink_gpu import _native as nv
    from vectorlink_gpu.ann import BEAM_NO_CACHE, BEAM_WINDOWS, closest_vectors, excluding_self
    from vectorlink_gpu.kernels import build_sketch

    rng = np.random.default_rng(n + dim)
    v = unit(rng, n, dim)
    if dim >= 64:
        v[5] = v[9]            # exact duplicate rows: ties ordered by id
        v[11] *= 1.5           # a row that is not of unit length
        v[13] *= 1e6           # ... and one longer than the sketch's tail can say (bounds of infinity: always fetched)
    c = cfg(beam_size=beam, beam_queue_factor=bqf, parallel_visit_count=pv, visit_queue_factor=vqf,
            exclude_factor=ef, speculative_readahead=ra)
    ql = beam * bqf
    beams = orc.generate_circulant_beams(n, orc.primes(ql))
    d = orc.calculate_distances(v, beams)
    lo, hi = 0, min(n, 600)
    oq = orc.Queue(hi - lo, ql, ql + ql * pv)
    oq.insert(beams[lo:hi], d[lo:hi])
    t_want = orc.closest_vectors(v[lo:hi], oq, v, beams, c, orc.excluding_self(lo, hi))

    gv, gb = dev(v), dev(beams)
    sk = build_sketch(gv)
    gq = Queue(hi - lo, ql, ql + ql * pv)
    gq.insert(gb[lo:hi], dev(d)[lo:hi])
    out = (ctypes.c_double * 9)()
    nv.lib().vl_beam_profile(1, 1, out)
    try:
        flags = {False: BEAM_NO_CACHE, True: 0, "windows": BEAM_WINDOWS}[cache]
        t_got = closest_vectors(gv[lo:hi], gq, gv, gb, c, excluding_self(lo, hi), flags=flags, sketch=sk)
    finally:
        nv.lib().vl_beam_profile(0, 1, out)
    (fetched, wanted, sketched) = (out[4], out[7], out[8])
    say(f"  iterations {t_got}, candidates {wanted:.0f}, through the sketch {sketched:.0f}, rows fetched {fetched:.0f}")
    assert t_got == t_want
    assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
    assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))
    if dim % 4 == 0 and dim <= 2048:
        # every row starts with the sketch; rows that end up fetching more than half of their candidates
        # anyway (these small iid tables put many within the sketch's error of the queues' ends) give it up
        assert 0 < sketched <= wanted
    else:
        assert sketched == 0


def test_build_with_and_without_the_sketch():
    """ANN builds the sketch for rows of 1 KiB and more and searches the initial circulant graph through it
    (no distance cache in that loop); sketch=False builds as before.  Both give the oracle's graph."""
    say("build with and without the sketch, n=3000 dim=256")
    from vectorlink_gpu import ANN
    from vectorlink_gpu.ann import GraphBuild

    rng = np.random.default_rng(256)
    n, dim = 3000, 256
    centres = rng.standard_normal((30, dim)).astype(np.float32)
    v = centres[rng.integers(0, 30, n)] + 0.15 * rng.standard_normal((n, dim)).astype(np.float32)
    v = (v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    kw = dict(beam_size=16, beam_queue_factor=2, batch_size=800, optimization_loops=2)
    (wb, wd) = orc.generate_ann(v, cfg(**kw))
    gv = dev(v)
    assert GraphBuild(gv, cfg(**kw)).sketch is not None and GraphBuild(gv, cfg(sketch=False, **kw)).sketch is None
    for sketch in (True, False):
        ann = ANN(gv, sketch=sketch, **kw)
        assert np.array_equal(host(ann.beams), wb), sketch
        assert np.array_equal(bits(host(ann.distances)), bits(wd)), sketch


@pytest.mark.parametrize("dim", [4, 64, 100, 128, 256, 384, 512, 768, 1024, 1536, 2048])
def test_sketch_bounds_hold_for_the_exact_kernel(dim):
    """vl_sketch_bounds (the code the beam-search step runs on its candidates): lo <= d <= hi for the float32
    distance the exact kernel returns, on random pairs and on the pairs that stress the bound - a query along
    what the rounding moved (the Cauchy-Schwarz worst case, both signs), a query equal or opposite to the row,
    a query with one huge and many tiny elements (coarse steps of its own rounding), rows that are not of unit
    length (one longer than a half can say: its bounds are the widest), rows of zeros, tiny rows, NaN.  And the
    bounds are worth something: on unit rows hi - lo stays
    within 2.3 x ||q|| x (what the rounding moved)."""
    say(f"sketch bounds dim={dim}")
    from vectorlink_gpu.kernels import build_sketch, gather_distances, sketch_bounds, sketch_parts

    rng = np.random.default_rng(1000 + dim)
    n, nq, m = 600, 96, 200
    v = unit(rng, n, dim)
    v[1] = 0.0
    v[2] *= 6.5
    v[4] = np.float32(1e-30) * v[4]
    v[5] *= 0.01
    v[7] *= 1e6                                                              # longer than the largest half: bounds of infinity
    sk = build_sketch(dev(v))
    (data, scale, _, _) = (host(x) for x in sketch_parts(sk))
    u = data[:, :dim].astype(np.float64)
    moved = v.astype(np.float64) - scale[:, None].astype(np.float64) * u    # what the rounding moved, per row
    q = unit(rng, nq, dim)
    ids = rng.integers(0, n, (nq, m)).astype(np.int32)
    ids[:, 0] = np.arange(nq) + 10
    for r in range(0, 24):                                                   # along / against the moved part
        e = moved[ids[r, 0]]
        if np.linalg.norm(e) > 0:
            q[r] = (e / np.linalg.norm(e) * (1 if r % 2 else -1)).astype(np.float32)
    for r in range(24, 36):
        q[r] = v[ids[r, 0]] * (1 if r % 2 else -1)                           # the row itself / its opposite
    for r in range(36, 48):
        q[r] = (rng.standard_normal(dim) * 1e-3).astype(np.float32)
        q[r, r % dim] = 1.0                                                  # one big element: coarse steps
    q[48] *= 3.0                                                             # queries that are not unit length
    q[49] = 0.0
    q[50] = np.float32(1e-32) * q[50]
    ids[:, 5] = M
    ids[:, 6] = n + 7                                                        # out of range
    (lo, hi) = sketch_bounds(dev(q), sk, dev(ids))
    d = host(gather_distances(dev(q), dev(v), dev(np.where(ids >= n, M, ids).astype(np.int32))))
    lo, hi = host(lo), host(hi)
    empty = (ids == M) | (ids >= n)
    assert np.all(lo[empty] == np.float32(F)) and np.all(hi[empty] == np.float32(F))
    real = ~empty
    assert np.all(lo[real] <= d[real]) and np.all(d[real] <= hi[real])
    # not vacuous: on unit queries and unit rows the gap is about 2 eps = ||q|| x moved (in distance units: / 2 x 2)
    rows = np.arange(51, nq)
    cols = np.arange(7, m)
    sub = ids[np.ix_(rows, cols)]
    unit_rows = np.isin(sub, [1, 2, 4, 5, 7], invert=True)
    gap = (hi - lo)[np.ix_(rows, cols)][unit_rows]
    want = np.linalg.norm(moved[sub[unit_rows]], axis=1)
    assert np.all(gap <= 2.3 * want * 0.5 * 2 + 1e-5) and np.all(gap > 0)
    # a query with a NaN: nothing is promised, and nothing wrong is claimed (lo <= hi or a NaN)
    q[0, 0] = np.nan
    (lo2, hi2) = sketch_bounds(dev(q[:1]), sk, dev(ids[:1]))
    lo2, hi2 = host(lo2)[0][real[0]], host(hi2)[0][real[0]]
    assert np.all(np.isnan(lo2) | np.isnan(hi2) | ((lo2 == 0) & (hi2 == 1)))


def test_search_with_the_sketch_equals_the_oracle():
    """ANN.search(sketch=True): the same queues as the oracle's search, under both seedings and both stops."""
    say("search with the sketch, n=2500 dim=256")
    from vectorlink_gpu import ANN

    rng = np.random.default_rng(99)
    n, dim, nq = 2500, 256, 200
    centres = rng.standard_normal((25, dim)).astype(np.float32)
    v = centres[rng.integers(0, 25, n)] + 0.15 * rng.standard_normal((n, dim)).astype(np.float32)
    v = (v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    q = centres[rng.integers(0, 25, nq)] + 0.15 * rng.standard_normal((nq, dim)).astype(np.float32)
    q = (q / np.linalg.norm(q, axis=1, keepdims=True)).astype(np.float32)
    kw = dict(beam_size=16, beam_queue_factor=2, batch_size=900, optimization_loops=2)
    c = cfg(**kw)
    (wb, _) = orc.generate_ann(v, c)
    ann = ANN(dev(v), **kw)
    assert np.array_equal(host(ann.beams), wb)
    for stop in ("batch", "per_query"):
        want = orc.search(v, wb, q, c, stop=stop)
        L = want.length
        for use in (True, False):
            got = ann.search(dev(q), stop=stop, sketch=use)
            assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L]), (stop, use)
            assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L])), (stop, use)
    # dense seeds: no oracle for the seeding tiles' choice, so the two paths are compared with each other
    a = ann.search(dev(q), seeding="dense", sketch=True)
    b = ann.search(dev(q), seeding="dense", sketch=False)
    assert torch.equal(a.indices[:, :a.length], b.indices[:, :b.length])
    assert torch.equal(a.distances[:, :a.length].view(torch.int32), b.distances[:, :b.length].view(torch.int32))
