"""The benchmark workloads themselves, as their generator makes them, against the CPU oracle:
the 4,096 x 128 workload whole (build, search, recall), the Zipf workload with exact duplicate
rows at a cut size, the 1536-dimensional mixture at a cut size beyond 2^31 elements, and the
two 1M-row mixtures through oracle replays on the graph the GPU built."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

M = orc.MAXINT
DEV = "cuda"


def say(msg):
    print(msg, flush=True)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def host(t):
    return t.detach().cpu().numpy()


def config_of(w, **kw):
    from vectorlink_gpu import synthetic

    c = dict(orc.DEFAULT_CONFIG)
    c.update(synthetic.ann_kwargs(w))
    c.update(kw)
    return c


def recall_at_10(found, truth):
    return float(np.mean([len(set(f[:10].tolist()) & set(t[:10].tolist())) / 10.0 for f, t in zip(found, truth)]))


def test_iid_4k_128_whole_against_the_oracle():
    """4,096 x 128 iid unit vectors, degree 32, queue 64, 256 queries, top-10: the whole build and the whole
    search on the oracle and on the GPU; graph, distances and search queues must be equal, recall@10 the same."""
    say("iid-4k-128: whole build + search on the oracle")
    from vectorlink_gpu import ANN, synthetic

    base, queries, w = synthetic.make("iid-4k-128")
    assert base.shape == (4096, 128) and queries.shape == (256, 128)
    c = config_of(w)
    assert c["beam_size"] == 32 and c["beam_size"] * c["beam_queue_factor"] == 64
    v, q = base.numpy(), queries.numpy()
    (wb, wd) = orc.generate_ann(v, c)
    want = orc.search(v, wb, q, c)
    ann = ANN(base.to(DEV), **synthetic.ann_kwargs(w))
    got = ann.search(queries.to(DEV))
    assert np.array_equal(host(ann.beams), wb)
    assert np.array_equal(bits(host(ann.distances)), bits(wd))
    L = want.length
    assert L == 64
    assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L]))
    (truth, _) = orc.knn_exact(q, v, 10)
    r_gpu, r_cpu = recall_at_10(host(got.indices), truth), recall_at_10(want.indices, truth)
    say(f"  recall@10 gpu {r_gpu:.4f} oracle {r_cpu:.4f}")
    assert abs(r_gpu - r_cpu) <= 0.005 and r_gpu > 0.9
    # self-recall@1 (ann.py:456-464) and the MFMA ground truth agree with the oracle's float64 one
    assert ann.recall()[1] == orc.ann_calculate_recall(v, wb, c, sample=v[:1000])[1]
    assert abs(ann.recall_at_k(queries.to(DEV), 10) - r_cpu) <= 0.005


def test_zipf_384_cut_with_duplicate_rows_against_the_oracle():
    """zipf-20m-384's generator at 200,000 rows: Zipf cluster sizes and 2 % exact duplicate rows.  One build
    batch made of duplicated rows, their originals and ordinary rows, and a search whose queries include
    duplicated rows (so that both copies tie at the same distance), on the oracle."""
    say("zipf-20m-384 cut to 200k: one build batch + search on the oracle")
    from vectorlink_gpu import ANN, Queue, synthetic
    from vectorlink_gpu.ann import closest_vectors
    from vectorlink_gpu.kernels import calculate_distances
    from vectorlink_gpu.utils import generate_circulant_beams, primes

    n = 200_000
    base, queries, w = synthetic.make("zipf-20m-384", n=n, queries=256)
    assert base.shape == (n, 384)
    v = base.numpy()
    # the generator's duplicates: rows that are bit-equal to an earlier or later row
    (_, first, counts) = np.unique(v.view(np.uint32)[:, :8], axis=0, return_index=True, return_counts=True)
    assert (counts > 1).sum() > 0.015 * n, "the cut has no duplicate rows"
    key = {}
    groups = []
    for i, row in enumerate(v.view(np.uint32)[:, :8]):
        k = row.tobytes()
        if k in key:
            groups.append((key[k], i))
        else:
            key[k] = i
    pairs = [(a, b) for (a, b) in groups if np.array_equal(v[a], v[b])][:64]
    assert len(pairs) == 64
    c = config_of(w)
    assert c["beam_size"] == 48 and c["beam_size"] * c["beam_queue_factor"] == 96
    ql = 96
    vd = base.to(DEV)
    beams = generate_circulant_beams(n, primes(ql))
    d = calculate_distances(vd, beams)
    rows = np.array(sorted({a for a, _ in pairs} | {b for _, b in pairs} | set(range(1000, 1128))), dtype=np.int64)
    rt = torch.from_numpy(rows).to(DEV)
    gq = Queue(len(rows), ql, ql + ql * 4)
    gq.insert(beams[rt], d[rt])
    excl = rt.to(torch.int32).unsqueeze(1).contiguous()
    t_gpu = closest_vectors(vd[rt].contiguous(), gq, vd, beams, c, excl)
    ob = host(beams)
    oq = orc.Queue(len(rows), ql, ql + ql * 4)
    oq.insert(ob[rows], orc.gather_distances(v[rows], v, ob[rows]))
    t_cpu = orc.closest_vectors(v[rows], oq, v, ob, c, rows.astype(np.int32).reshape(-1, 1))
    assert t_gpu == t_cpu
    assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
    assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))

    # search on a graph built by the GPU over the first 40,000 rows (duplicates included)
    say("  build 40k x 384 and search with duplicated rows as queries")
    m = 40_000
    sub = np.ascontiguousarray(v[:m])
    ann = ANN(vd[:m].contiguous(), **synthetic.ann_kwargs(w))
    dup_q = [b for (a, b) in groups if b < m and np.array_equal(v[a], v[b])][:128]
    assert len(dup_q) >= 64
    qn = np.concatenate([sub[dup_q], queries.numpy()[:128]])
    want = orc.search(sub, host(ann.beams), qn, c)
    got = ann.search(torch.from_numpy(qn).to(DEV))
    L = want.length
    assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L]))
    # ties are really there: neighbouring slots at one distance with different ids, ordered by id
    wi, wdist = want.indices[:, :L], want.distances[:, :L]
    tie = (wdist[:, 1:] == wdist[:, :-1]) & (wi[:, 1:] != M)
    assert tie.sum() >= 32, "no tied distances among the results"
    assert (wi[:, 1:][tie] > wi[:, :-1][tie]).all()
    # dense seeds (query-dependent entry points) give the same queues as the oracle seeded with the same ids
    r1 = ann.search(torch.from_numpy(qn).to(DEV), seeding="dense")
    assert bool((r1.distances[:, 1:L] >= r1.distances[:, :L - 1]).all())


def test_mix_1536_cut_beyond_2_to_31_elements_against_the_oracle():
    """mix-10m-1536's generator (8,192 centres, sigma 0.2) at 1.5M rows = 2.3e9 floats: a build batch at each
    end of the table and a dense-seeded search, on the oracle."""
    say("mix-10m-1536 cut to 1.5M: build batches + search on the oracle")
    from vectorlink_gpu import ANN, Queue, synthetic
    from vectorlink_gpu.ann import closest_vectors, excluding_self
    from vectorlink_gpu.kernels import calculate_distances, knn_exact
    from vectorlink_gpu.utils import generate_circulant_beams, primes

    n = 1_500_000
    base, queries, w = synthetic.make("mix-10m-1536", n=n, queries=64)
    assert base.shape == (n, 1536) and n * 1536 > 2**31
    c = config_of(w)
    assert c["beam_size"] == 64
    ql = 128
    v = base.numpy()
    vd = base.to(DEV)
    beams = generate_circulant_beams(n, primes(ql))
    d = calculate_distances(vd, beams)
    ob = orc.generate_circulant_beams(n, orc.primes(ql))
    for s0 in (0, n - 16):
        rows = 16
        gq = Queue(rows, ql, ql + ql * 4)
        gq.insert(beams[s0:s0 + rows], d[s0:s0 + rows])
        t_gpu = closest_vectors(vd[s0:s0 + rows], gq, vd, beams, c, excluding_self(s0, s0 + rows))
        oq = orc.Queue(rows, ql, ql + ql * 4)
        oq.insert(ob[s0:s0 + rows], orc.gather_distances(v[s0:s0 + rows], v, ob[s0:s0 + rows]))
        t_cpu = orc.closest_vectors(v[s0:s0 + rows], oq, v, ob, c, orc.excluding_self(s0, s0 + rows))
        assert t_gpu == t_cpu
        assert np.array_equal(host(gq.indices)[:, :ql], oq.indices[:, :ql])
        assert np.array_equal(bits(host(gq.distances)[:, :ql]), bits(oq.distances[:, :ql]))
    # exact kNN of the held-out mixture queries against float64 on the host
    qd = queries.to(DEV)
    (gi, gd) = knn_exact(qd, vd, 10)
    full = ((1 - queries[:8].double() @ base.double().t()) / 2).clamp(0, 1)
    (wdist, wi) = full.topk(10, dim=1, largest=False)
    assert torch.allclose(gd[:8].cpu().double(), wdist, rtol=1e-5, atol=1e-6)
    assert (gi[:8].cpu().long() == wi).float().mean() > 0.95


def test_mix_1m_128_search_on_the_built_graph_against_the_oracle():
    """mix-1m-128 whole on the GPU (three loops, prune), then 256 held-out queries searched on that graph by
    the oracle and by the GPU: equal queues."""
    say("mix-1m-128: GPU build, oracle search replay")
    from vectorlink_gpu import ANN, synthetic

    base, queries, w = synthetic.make("mix-1m-128")
    c = config_of(w)
    ann = ANN(base.to(DEV), **synthetic.ann_kwargs(w))
    qn = queries.numpy()[:256]
    want = orc.search(base.numpy(), host(ann.beams), qn, c)
    got = ann.search(queries[:256].to(DEV))
    L = want.length
    assert np.array_equal(host(got.indices)[:, :L], want.indices[:, :L])
    assert np.array_equal(bits(host(got.distances)[:, :L]), bits(want.distances[:, :L]))
    # one batch of the state the second optimisation loop starts from would need the full-width table; the
    # final graph stands in: rows searched as queries with themselves excluded
    from vectorlink_gpu import Queue
    from vectorlink_gpu.ann import closest_vectors, excluding_self

    rows = 48
    s0 = 123_456
    vd = ann.vectors
    gq = Queue(rows, 32, 32 + 32 * 4)
    gq.insert(ann.beams[s0:s0 + rows], ann.distances[s0:s0 + rows])
    t_gpu = closest_vectors(vd[s0:s0 + rows], gq, vd, ann.beams, c, excluding_self(s0, s0 + rows))
    v = base.numpy()
    gb = host(ann.beams)
    oq = orc.Queue(rows, 32, 32 + 32 * 4)
    oq.insert(gb[s0:s0 + rows], host(ann.distances)[s0:s0 + rows])
    t_cpu = orc.closest_vectors(v[s0:s0 + rows], oq, v, gb, c, orc.excluding_self(s0, s0 + rows))
    assert t_gpu == t_cpu
    assert np.array_equal(host(gq.indices)[:, :32], oq.indices[:, :32])
    assert np.array_equal(bits(host(gq.distances)[:, :32]), bits(oq.distances[:, :32]))


def test_multi_loop_build_with_prune_on_clustered_rows_equals_the_oracle():
    """Three optimisation loops with the reference's prune between them on clustered rows (40 clusters of 100
    rows, 256 columns - long enough for the 8-bit sketch, so loops 1 and 2 run through cache + sketch on pruned
    tables with empty slots): the graph, its distances and the self-recall@1 after EVERY loop equal the
    oracle's.  On such rows the self-recall falls once the neighbour lists lie inside their clusters (the
    circulant seeds of the recall search then only reach a row whose cluster a seed falls into); that figure is
    the algorithm's, and this pins it."""
    say("clustered rows, three loops with prune: graph and per-loop self-recall against the oracle")
    from vectorlink_gpu.ann import GraphBuild

    rng = np.random.default_rng(31)
    n, dim, clusters = 4000, 256, 40
    centres = rng.standard_normal((clusters, dim)).astype(np.float32)
    v = centres[rng.integers(0, clusters, n)] + 0.15 * rng.standard_normal((n, dim)).astype(np.float32)
    v = (v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    c = dict(orc.DEFAULT_CONFIG)
    c.update(beam_size=32, beam_queue_factor=2, recall_search_queue_factor=2, batch_size=1500,
             optimization_loops=3, prune=True)
    want_recalls = []
    (wb, wd) = orc.generate_ann(v, c, recalls=want_recalls)
    build = GraphBuild(torch.from_numpy(v).to(DEV), c)
    for _ in build.steps():
        pass
    assert build.sketch is not None
    (gb, gd) = build.result()
    got_recalls = [st["self_recall"] for st in build.stats]
    say(f"  self-recall per loop: gpu {got_recalls} oracle {want_recalls}")
    assert got_recalls == want_recalls and len(got_recalls) >= 2
    assert np.array_equal(host(gb), wb)
    assert np.array_equal(bits(host(gd)), bits(wd))
    assert bool((build.beams == M).any())   # the prune did empty slots of the build-width table
