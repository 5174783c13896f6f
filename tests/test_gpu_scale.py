"""GPU checks at the full sizes of the benchmark workloads (1M x 128 and
1M x 768), through properties that do not need the CPU oracle to run at that
scale: ordering, membership, distances recomputed from ids, float64 samples,
round trips, determinism - plus a small batch at full scale replayed on the
oracle for exact ids."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

M = orc.MAXINT
DEV = "cuda"


def say(msg):
    print(msg, flush=True)


@pytest.fixture(scope="module")
def mix128():
    from vectorlink_gpu import synthetic

    base, q, w = synthetic.make("mix-1m-128")
    return base, q, w


def test_build_1m_x_128_properties(mix128):
    say("full build 1M x 128")
    from vectorlink_gpu import ANN, synthetic
    from vectorlink_gpu.kernels import gather_distances, knn_exact

    base, q, w = mix128
    v = base.to(DEV)
    ann = ANN(v, **synthetic.ann_kwargs(w))
    n, deg = ann.beams.shape
    assert (n, deg) == (1_000_000, 32) and ann.distances.shape == (n, deg)
    ids, d = ann.beams, ann.distances
    real = ids != M
    assert bool(real[:, 0].all())
    assert bool(((ids >= 0) & (ids < n))[real].all())
    rows = torch.arange(n, device=DEV, dtype=torch.int32).unsqueeze(1).expand(n, deg)
    assert not bool((ids == rows)[real].any())                       # no self edges
    assert bool((d[:, 1:] >= d[:, :-1]).all())                        # rows ordered by distance
    srt = ids.sort(dim=1).values
    assert not bool(((srt[:, 1:] == srt[:, :-1]) & (srt[:, 1:] != M)).any())  # distinct ids per row
    assert bool((d[~real] == torch.tensor(3.4028e37, device=DEV)).all())
    # the distances are the distances of the ids: recomputed bit for bit, and against float64 on a sample
    again = gather_distances(v, v, ids)
    assert torch.equal(again, d)
    sample = torch.randint(0, n, (512,), generator=torch.Generator(device="cpu").manual_seed(0), device="cpu")
    vs = base[sample].double()
    nb = base[ids[sample.to(DEV)].cpu().long()].double()              # [512, deg, dim]
    ref = ((1 - (vs.unsqueeze(1) * nb).sum(2)) / 2).clamp(0, 1)
    assert torch.allclose(d[sample.to(DEV)].cpu().double(), ref, rtol=1e-5, atol=1e-6)
    # graph quality and search
    t11, _ = knn_exact(v[:1024].contiguous(), v, 11)
    hits = (ids[:1024, :, None] == t11[:, None, 1:11]).any(dim=1).sum().item()
    assert hits / (1024 * 10) > 0.7
    qd = q[:2000].to(DEV)
    r1 = ann.search(qd, seeding="dense")
    r2 = ann.search(qd, seeding="dense")
    assert torch.equal(r1.indices[:, :r1.length], r2.indices[:, :r2.length])      # deterministic
    assert bool((r1.distances[:, 1:r1.length] >= r1.distances[:, :r1.length - 1]).all())
    truth, td = knn_exact(qd, v, 10)
    found = r1.indices[:, :10]
    recall = (found.unsqueeze(2) == truth.unsqueeze(1)).any(dim=2).sum().item() / truth.numel()
    assert recall > 0.75
    # what search returns are real distances of real ids
    fd = gather_distances(qd, v, found.contiguous())
    assert torch.equal(fd, r1.distances[:, :10])
    # resume from the stored graph (ann.py:391-396): same distances, same answers
    again = ANN(v, beams=ann.beams, **synthetic.ann_kwargs(w))
    assert torch.equal(again.distances, d)
    r3 = again.search(qd, seeding="dense")
    assert torch.equal(r3.indices[:, :r3.length], r1.indices[:, :r1.length])


def test_build_1m_x_768_properties():
    """The headline workload built whole (1M x 768, degree 64, queue 128, three loops with the reference's
    prune, through cache + sketch): what can be checked without the oracle at that size."""
    say("full build 1M x 768")
    from vectorlink_gpu import ANN, synthetic
    from vectorlink_gpu.kernels import gather_distances, knn_exact

    base, q, w = synthetic.make("mix-1m-768")
    v = base.to(DEV)
    ann = ANN(v, **synthetic.ann_kwargs(w))
    n, deg = ann.beams.shape
    assert (n, deg) == (1_000_000, 64) and ann.distances.shape == (n, deg)
    ids, d = ann.beams, ann.distances
    real = ids != M
    assert bool(real[:, 0].all())
    assert bool(((ids >= 0) & (ids < n))[real].all())
    rows = torch.arange(n, device=DEV, dtype=torch.int32).unsqueeze(1).expand(n, deg)
    assert not bool((ids == rows)[real].any())                       # no self edges
    assert bool((d[:, 1:] >= d[:, :-1]).all())                        # rows ordered by distance
    srt = ids.sort(dim=1).values
    assert not bool(((srt[:, 1:] == srt[:, :-1]) & (srt[:, 1:] != M)).any())  # distinct ids per row
    assert bool((d[~real] == torch.tensor(3.4028e37, device=DEV)).all())
    del srt, rows
    # the distances are the distances of the ids: recomputed bit for bit, and against float64 on a sample
    again = gather_distances(v, v, ids)
    assert torch.equal(again, d)
    del again
    sample = torch.randint(0, n, (256,), generator=torch.Generator(device="cpu").manual_seed(0), device="cpu")
    vs = base[sample].double()
    nb = base[ids[sample.to(DEV)].cpu().long().clamp(max=n - 1)].double()     # [256, deg, dim]
    ref = ((1 - (vs.unsqueeze(1) * nb).sum(2)) / 2).clamp(0, 1)
    ok = real[sample.to(DEV)].cpu()
    assert torch.allclose(d[sample.to(DEV)].cpu().double()[ok], ref[ok], rtol=1e-5, atol=1e-6)
    # graph quality: most of a row's exact 10 nearest neighbours are among its 64
    t11, _ = knn_exact(v[:1024].contiguous(), v, 11)
    hits = (ids[:1024, :, None] == t11[:, None, 1:11]).any(dim=1).sum().item()
    say(f"  exact 10-NN among the 64 neighbours: {hits / (1024 * 10):.3f}")
    assert hits / (1024 * 10) > 0.85
    # search: deterministic, ordered, real distances of real ids, recall@10 at the quoted level
    qd = q[:2000].to(DEV)
    r1 = ann.search(qd, seeding="dense")
    r2 = ann.search(qd, seeding="dense")
    assert torch.equal(r1.indices[:, :r1.length], r2.indices[:, :r2.length])
    assert bool((r1.distances[:, 1:r1.length] >= r1.distances[:, :r1.length - 1]).all())
    truth, td = knn_exact(qd, v, 10)
    found = r1.indices[:, :10]
    recall = (found.unsqueeze(2) == truth.unsqueeze(1)).any(dim=2).sum().item() / truth.numel()
    say(f"  recall@10 with dense seeds: {recall:.4f}")
    assert recall >= 0.95
    fd = gather_distances(qd, v, found.contiguous())
    assert torch.equal(fd, r1.distances[:, :10])


def test_1m_x_768_distances_knn_and_one_batch_on_the_oracle():
    say("1M x 768: distances, exact kNN, one small batch against the oracle")
    from vectorlink_gpu import synthetic
    from vectorlink_gpu.ann import closest_vectors, excluding_self
    from vectorlink_gpu.kernels import calculate_distances, knn_exact
    from vectorlink_gpu.queue import Queue
    from vectorlink_gpu.utils import generate_circulant_beams, primes

    base, q, w = synthetic.make("mix-1m-768")
    n, dim = base.shape
    v = base.to(DEV)
    ql = w["beam_size"] * w["beam_queue_factor"]
    beams = generate_circulant_beams(n, primes(ql))
    d = calculate_distances(v, beams)
    assert bool(((d >= 0) & (d <= 1)).all())
    # closed form of the circulant table and float64 distances on a sample of rows
    sample = torch.tensor([0, 1, 777_777, n - 1], device="cpu")
    p = torch.from_numpy(orc.primes(ql).astype(np.int64))
    want_ids = (sample.unsqueeze(1) + p.unsqueeze(0)) % n
    assert torch.equal(beams[sample.to(DEV)].cpu().long(), want_ids)
    ref = ((1 - (base[sample].double().unsqueeze(1) * base[want_ids].double()).sum(2)) / 2).clamp(0, 1)
    assert torch.allclose(d[sample.to(DEV)].cpu().double(), ref, rtol=1e-5, atol=1e-6)
    # symmetry d(a, b) == d(b, a), bit for bit, through the two operand roles
    a, b = 12_345, int(want_ids[0, 5])
    from vectorlink_gpu.kernels import gather_distances
    dab = gather_distances(v[a:a + 1].contiguous(), v, torch.tensor([[b]], dtype=torch.int32, device=DEV))
    dba = gather_distances(v[b:b + 1].contiguous(), v, torch.tensor([[a]], dtype=torch.int32, device=DEV))
    assert torch.equal(dab, dba)
    # exact kNN against a float64 brute force for a few queries
    qd = q[:8].to(DEV)
    gi, gd = knn_exact(qd, v, 10)
    full = ((1 - q[:8].double() @ base.double().t()) / 2).clamp(0, 1)
    wd, wi = full.topk(10, dim=1, largest=False)
    assert torch.allclose(gd.cpu().double(), wd, rtol=1e-5, atol=1e-6)
    assert (gi.cpu().long() == wi).float().mean() > 0.95
    # one batch of 24 rows of the first optimisation loop, replayed on the CPU oracle: exact ids and distances
    rows = 24
    cfg = dict(orc.DEFAULT_CONFIG)
    cfg.update(synthetic.ann_kwargs(w))
    gq = Queue(rows, ql, ql + ql * 4)
    gq.insert(beams[:rows], d[:rows])
    t_gpu = closest_vectors(v[:rows], gq, v, beams, cfg, excluding_self(0, rows))
    vn = base.numpy()
    ob = orc.generate_circulant_beams(n, orc.primes(ql))
    oq = orc.Queue(rows, ql, ql + ql * 4)
    oq.insert(ob[:rows], orc.gather_distances(vn[:rows], vn, ob[:rows]))
    t_cpu = orc.closest_vectors(vn[:rows], oq, vn, ob, cfg, orc.excluding_self(0, rows))
    assert t_gpu == t_cpu
    assert np.array_equal(gq.indices[:, :ql].cpu().numpy(), oq.indices[:, :ql])
    assert np.array_equal(gq.distances[:, :ql].cpu().numpy().view(np.uint32), oq.distances[:, :ql].view(np.uint32))


def test_offsets_beyond_2_to_31_elements():
    """N x D above 2^31 elements (the shape class of the 20M x 384 and 10M x 1536 workloads):
    every row offset must be computed in 64 bits."""
    say("2.2M x 1024: 64-bit offsets")
    from vectorlink_gpu.ann import closest_vectors, excluding_self
    from vectorlink_gpu.kernels import calculate_distances, gather_distances, knn_exact
    from vectorlink_gpu.queue import Queue
    from vectorlink_gpu.utils import generate_circulant_beams, primes

    n, dim = 2_200_000, 1024
    assert n * dim > 2**31
    g = torch.Generator(device=DEV).manual_seed(5)
    v = torch.empty((n, dim), dtype=torch.float32, device=DEV)
    for s in range(0, n, 200_000):
        e = min(n, s + 200_000)
        v[s:e] = torch.nn.functional.normalize(torch.randn((e - s, dim), generator=g, device=DEV), dim=1)
    hi = n - 4096
    # gathered distances between rows at the far end, against float64 on the device
    rows = torch.arange(hi, hi + 512, device=DEV)
    ids = torch.randint(hi, n, (512, 33), generator=g, device=DEV).to(torch.int32)
    got = gather_distances(v[hi:hi + 512], v, ids)
    ref = ((1 - (v[rows].double().unsqueeze(1) * v[ids.long()].double()).sum(2)) / 2).clamp(0, 1)
    assert torch.allclose(got.double(), ref, rtol=1e-5, atol=1e-6)
    # exact kNN: a query that is a copy of a far row must come back first at distance ~0
    q = v[torch.tensor([n - 1, n - 77, 5], device=DEV)].contiguous()
    ki, kd = knn_exact(q, v, 4)
    assert ki[:, 0].tolist() == [n - 1, n - 77, 5] and float(kd[:, 0].max()) < 1e-6
    full = ((1 - q.double() @ v[hi:].double().t()) / 2).clamp(0, 1)   # the far block alone bounds the answer
    assert bool((kd[:, 1].double() <= full.topk(2, dim=1, largest=False).values[:, 1] + 1e-6).all())
    # one beam-search batch over the last rows: ordered, self excluded, distances belong to the ids
    cfg = dict(orc.DEFAULT_CONFIG)
    cfg.update(beam_size=16, beam_queue_factor=2)
    ql = 32
    beams = generate_circulant_beams(n, primes(ql))
    d = calculate_distances(v, beams)
    s0, e0 = n - 1000, n
    gq = Queue(e0 - s0, ql, ql + ql * 4)
    gq.insert(beams[s0:e0], d[s0:e0])
    t = closest_vectors(v[s0:e0], gq, v, beams, cfg, excluding_self(s0, e0))
    assert t > 0 and t % 5 == 0
    qi, qd = gq.indices[:, :ql], gq.distances[:, :ql]
    assert bool((qd[:, 1:] >= qd[:, :-1]).all()) and bool((qi != M).all())
    own = torch.arange(s0, e0, device=DEV, dtype=torch.int32).unsqueeze(1)
    assert not bool((qi == own).any())
    assert torch.equal(gather_distances(v[s0:e0], v, qi.contiguous()), qd)
    assert bool((qd[:, 0] <= d[s0:e0].min(dim=1).values).all())       # never worse than the seeds


def test_three_forms_of_the_loop_agree_at_scale(mix128):
    """One batch of 10,000 rows at 1M x 128 through the fused step, the two-launch form and
    the full-sort merge: same iteration count, same queues, bit for bit."""
    say("fused vs two launches vs sort merge, 10000 rows of 1M x 128")
    from vectorlink_gpu import synthetic
    from vectorlink_gpu.ann import BEAM_SORT_MERGE, BEAM_TWO_LAUNCHES, closest_vectors, excluding_self
    from vectorlink_gpu.kernels import calculate_distances
    from vectorlink_gpu.queue import Queue
    from vectorlink_gpu.utils import generate_circulant_beams, primes

    base, q, w = mix128
    v = base.to(DEV)
    n = v.shape[0]
    cfg = dict(orc.DEFAULT_CONFIG)
    cfg.update(synthetic.ann_kwargs(w))
    ql = cfg["beam_size"] * cfg["beam_queue_factor"]
    beams = generate_circulant_beams(n, primes(ql))
    d = calculate_distances(v, beams)
    s0, e0 = 500_000, 510_000
    results = []
    for flags in (0, BEAM_TWO_LAUNCHES, BEAM_SORT_MERGE, 0):
        gq = Queue(e0 - s0, ql, ql + ql * 4)
        gq.insert(beams[s0:e0], d[s0:e0])
        t = closest_vectors(v[s0:e0], gq, v, beams, cfg, excluding_self(s0, e0), flags=flags)
        results.append((t, gq.indices[:, :ql].clone(), gq.distances[:, :ql].clone()))
    for (t, ids, dist) in results[1:]:
        assert t == results[0][0]
        assert torch.equal(ids, results[0][1]) and torch.equal(dist, results[0][2])


def test_10m_x_1536_scale():
    """The shape of the largest workload this library is sized for (10M x 1536 fp32 = 61 GB resident): the initial
    distance table, one beam-search batch at each end of the id range and exact kNN."""
    say("10M x 1536 (61 GB)")
    free, _ = torch.cuda.mem_get_info()
    if free < 100 * 2**30:
        pytest.skip("needs 100 GB of free device memory")
    from vectorlink_gpu.ann import closest_vectors, excluding_self
    from vectorlink_gpu.kernels import calculate_distances, gather_distances, knn_exact
    from vectorlink_gpu.queue import Queue
    from vectorlink_gpu.utils import generate_circulant_beams, primes

    n, dim, beam = 10_000_000, 1536, 64
    g = torch.Generator(device=DEV).manual_seed(4)
    v = torch.empty((n, dim), dtype=torch.float32, device=DEV)
    for s in range(0, n, 250_000):
        e = min(n, s + 250_000)
        v[s:e] = torch.nn.functional.normalize(torch.randn((e - s, dim), generator=g, device=DEV), dim=1)
    cfg = dict(orc.DEFAULT_CONFIG)
    cfg.update(beam_size=beam, beam_queue_factor=2)
    ql = 2 * beam
    beams = generate_circulant_beams(n, primes(ql))
    d = calculate_distances(v, beams)
    rows = torch.tensor([0, 4_999_999, n - 1], device=DEV)
    ref = ((1 - (v[rows].double().unsqueeze(1) * v[beams[rows].long()].double()).sum(2)) / 2).clamp(0, 1)
    assert torch.allclose(d[rows].double(), ref, rtol=1e-5, atol=1e-6)
    for s0 in (0, n - 2000):
        gq = Queue(2000, ql, ql + ql * 4)
        gq.insert(beams[s0:s0 + 2000], d[s0:s0 + 2000])
        t = closest_vectors(v[s0:s0 + 2000], gq, v, beams, cfg, excluding_self(s0, s0 + 2000))
        qi, qd = gq.indices[:, :ql], gq.distances[:, :ql]
        assert t % 5 == 0 and bool((qd[:, 1:] >= qd[:, :-1]).all()) and bool((qi != M).all())
        assert torch.equal(gather_distances(v[s0:s0 + 2000], v, qi.contiguous()), qd)
        assert bool((qd[:, 0] <= d[s0:s0 + 2000].min(dim=1).values).all())
    q = v[torch.tensor([7, n // 2, n - 3], device=DEV)].contiguous()
    ki, kd = knn_exact(q, v, 5)
    assert ki[:, 0].tolist() == [7, n // 2, n - 3] and float(kd[:, 0].max()) < 1e-6


def test_tables_with_more_rows_than_one_launch_holds():
    """17.5M rows: one workgroup per row at 256 threads would need more than 2^32 threads in
    one launch, which the hardware queue does not take whole. Every whole-table entry point
    must cover all rows (checked at both ends of the table and across the seams between launches)."""
    say("17.5M-row tables: gather, sorts, dedup, prune, queue insert")
    from vectorlink_gpu.kernels import (dedup_tensor_, gather_distances, index_sort_, knn_exact, optimize_graph, prune_,
                                        queue_sort_)
    from vectorlink_gpu.queue import Queue

    n, dim, w = 17_500_000, 4, 4
    assert n * 256 > 2**32
    g = torch.Generator(device=DEV).manual_seed(11)
    v = torch.nn.functional.normalize(torch.randn((n, dim), generator=g, device=DEV), dim=1)
    ids = torch.randint(0, n, (n, w), generator=g, device=DEV).to(torch.int32)
    # rows looked at closely: both ends and every seam between launches of 2^21 workgroups
    step = 1 << 21
    probe = torch.cat([torch.arange(0, 2000, device=DEV), torch.arange(n - 2000, n, device=DEV)]
                      + [torch.arange(s - 500, s + 500, device=DEV) for s in range(step, n, step)])

    d = gather_distances(v, v, ids)
    ref = ((1 - (v[probe].double().unsqueeze(1) * v[ids[probe].long()].double()).sum(2)) / 2).clamp(0, 1)
    assert torch.allclose(d[probe].double(), ref, rtol=1e-5, atol=1e-6)
    hv, hi, hd = v.cpu().numpy(), ids.cpu().numpy(), d.cpu().numpy()
    pr = probe.cpu().numpy()
    assert np.array_equal(orc.gather_distances(hv[pr], hv, hi[pr]).view(np.uint32), hd[pr].view(np.uint32))

    # prune over the whole table against the oracle, every row
    say("  prune")
    gb, gd = prune_(ids.clone(), d.clone())
    wb, wd = orc.prune_(hi, hd)
    assert np.array_equal(gb.cpu().numpy(), wb) and np.array_equal(gd.cpu().numpy().view(np.uint32), wd.view(np.uint32))
    del gb, gd, wb, wd

    # row sorts against torch.sort (random distances: no ties)
    say("  sorts")
    si, sd = ids.clone(), d.clone()
    index_sort_(si, sd)                                   # by (distance, id)
    order = torch.sort(d, dim=1, stable=True)
    ties = (order.values[:, 1:] == order.values[:, :-1]).any(dim=1)
    assert torch.equal(sd, order.values) and torch.equal(si[~ties], torch.gather(ids, 1, order.indices)[~ties])
    by_id = torch.sort(ids, dim=1).values
    si = by_id.clone()
    dedup_tensor_(si)
    dup = torch.zeros_like(by_id, dtype=torch.bool)
    dup[:, 1:] = by_id[:, 1:] == by_id[:, :-1]
    assert torch.equal(si, torch.where(dup, torch.full_like(si, M), by_id))
    qi, qd = ids.clone(), d.clone()
    queue_sort_(qi, qd)
    assert bool((qd[:, 1:] >= qd[:, :-1]).all())
    assert torch.equal(gather_distances(v, v, torch.where(qi == M, torch.zeros_like(qi), qi))[qi != M], qd[qi != M])
    del si, sd, qi, qd, order, dup, by_id, ties

    # queue insert into empty queues: the row-wise best `length` distinct candidates in order
    say("  queue insert")
    q = Queue(n, 2, 2 + w)
    q.insert(ids, d)
    got_i, got_d = q.indices[probe, :2].cpu().numpy(), q.distances[probe, :2].cpu().numpy()
    oq = orc.Queue(len(pr), 2, 2 + w)
    oq.insert(hi[pr], hd[pr])
    assert np.array_equal(got_i, oq.indices[:, :2]) and np.array_equal(got_d.view(np.uint32), oq.distances[:, :2].view(np.uint32))
    assert bool((q.distances[:, 0] == d.min(dim=1).values).all())
    del q

    # rank pruning + reverse edges over more rows than one launch
    say("  optimize_graph, exact kNN")
    m = 2_300_000
    table = torch.randint(0, m, (m, 6), generator=g, device=DEV).to(torch.int32)
    got = optimize_graph(table, 4)
    assert np.array_equal(got.cpu().numpy(), orc.optimize_graph(table.cpu().numpy(), 4))
    # exact kNN with more queries than one launch of the merge kernel
    small = v[:300].contiguous()
    ki, kd = knn_exact(v[:m].contiguous(), small, 2)
    tail = slice(m - 3000, m)
    full = ((1 - v[:m][tail].double() @ small.double().t()) / 2).clamp(0, 1)
    best = full.topk(2, dim=1, largest=False)
    assert torch.allclose(kd[tail].double(), best.values, rtol=1e-5, atol=1e-6)
    clear = (best.values[:, 1] - best.values[:, 0]) > 1e-5
    assert torch.equal(ki[tail][clear, 0].long(), best.indices[clear, 0])
    assert bool((ki[:300, 0] == torch.arange(300, device=DEV)).all())


@pytest.mark.parametrize("workload,n", [("mix-1m-768", 300_000), ("zipf-20m-384", 400_000), ("mix-10m-1536", 150_000)])
def test_sketch_and_plain_paths_agree_at_scale(workload, n):
    """Two independent code paths over the same inputs at the benchmark row sizes: batches of 10,000 rows against
    the circulant graph and against the graph one optimisation loop leaves, searched (a) as before the sketch
    existed, (b) through the sketch alone, (c) with cache and sketch together.  Same iteration count, ids and
    distance bits; the counters show that (b) and (c) did fetch fewer rows."""
    say(f"sketch and plain paths, {workload} cut to {n}")
    import ctypes

    from vectorlink_gpu import Queue, synthetic
    from vectorlink_gpu import _native as nv
    from vectorlink_gpu.ann import BEAM_NO_CACHE, GraphBuild, closest_vectors, excluding_self
    from vectorlink_gpu.kernels import build_sketch

    base, _, w = synthetic.make(workload, n=n)
    kw = synthetic.ann_kwargs(w)
    c = dict(orc.DEFAULT_CONFIG)
    c.update(kw)
    c.update(optimization_loops=1, batch_size=10_000)
    v = base.to(DEV)
    build = GraphBuild(v, c, keep_history=True)
    for _ in build.steps():
        pass
    ql = c["beam_size"] * c["beam_queue_factor"]
    sk = build_sketch(v)
    rows = 10_000
    for state, (tb, td) in enumerate([build.history[0], (build.beams, build.distances)]):
        results = []
        for name, flags, sketch in (("plain", 0, None), ("sketch", BEAM_NO_CACHE, sk), ("cache+sketch", 0, sk)):
            q = Queue(rows, ql, ql + ql * c["parallel_visit_count"], device=DEV)
            q.insert(tb[n - rows:], td[n - rows:])
            out = (ctypes.c_double * 9)()
            nv.lib().vl_beam_profile(1, 1, out)
            try:
                t = closest_vectors(v[n - rows:], q, v, tb, c, excluding_self(n - rows, n, device=DEV), flags=flags,
                                    sketch=sketch)
            finally:
                nv.lib().vl_beam_profile(0, 1, out)
            say(f"  state {state} {name}: {t} iterations, rows fetched {out[4]:.0f}, through the sketch {out[8]:.0f}")
            results.append((t, q.indices[:, :ql].clone(), q.distances[:, :ql].clone(), out[4], out[8]))
        (t0, i0, d0, fetched0, _) = results[0]
        for (t, i, d, fetched, sketched) in results[1:]:
            assert t == t0
            assert torch.equal(i, i0)
            assert torch.equal(d.view(torch.int32), d0.view(torch.int32))
            assert sketched > 0
        if state == 0:
            assert results[1][3] < 0.5 * fetched0 and results[2][3] < 0.5 * fetched0
        # 24 rows of the same state through cache + sketch, replayed on the CPU oracle: exact ids and distances
        # (state 1 is what 45 % of a build's launches run on: a pruned table with empty slots, distances carried)
        few = 24
        q = Queue(few, ql, ql + ql * c["parallel_visit_count"], device=DEV)
        q.insert(tb[n - few:], td[n - few:])
        t_gpu = closest_vectors(v[n - few:], q, v, tb, c, excluding_self(n - few, n, device=DEV), sketch=sk)
        vn, tbn, tdn = base.numpy(), tb.cpu().numpy(), td.cpu().numpy()
        oq = orc.Queue(few, ql, ql + ql * c["parallel_visit_count"])
        oq.insert(tbn[n - few:], tdn[n - few:])
        t_cpu = orc.closest_vectors(vn[n - few:], oq, vn, tbn, c, orc.excluding_self(n - few, n))
        say(f"  state {state}: {few} rows on the oracle, {t_cpu} iterations")
        assert t_gpu == t_cpu
        assert np.array_equal(q.indices[:, :ql].cpu().numpy(), oq.indices[:, :ql])
        assert np.array_equal(q.distances[:, :ql].cpu().numpy().view(np.uint32), oq.distances[:, :ql].view(np.uint32))
        if state == 1:
            assert (tbn == M).any()
