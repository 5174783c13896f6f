"""Graph build and beam search drivers (reference: vectorlink_gpu/ann.py).

Same names, arguments and control flow as the reference; the device work goes
to libvlgpu.so.  Differences are stated where they occur.
"""
from __future__ import annotations

import ctypes
import threading
import time
from typing import Dict, Optional, Tuple

import torch
from torch import Tensor

from . import _native as nv
from .constants import DEVICE, MAXFLOAT, MAXINT
from .kernels import (build_sketch, calculate_distances, gather_distances, knn_exact, optimize_graph, prune_,
                      search_from_seeds, sketch_row_bytes)
from . import log as _log
from .log import log_time
from .queue import Queue
from .utils import add_new_to_seen_, generate_circulant_beams, generate_queue_circulants, primes


BEAM_TWO_LAUNCHES = 1  # include/vlgpu.h: VL_BEAM_TWO_LAUNCHES
BEAM_SORT_MERGE = 2    # include/vlgpu.h: VL_BEAM_SORT_MERGE
BEAM_PER_QUERY_STOP = 4  # include/vlgpu.h: VL_BEAM_PER_QUERY_STOP (a different loop: every row stops on its own)
BEAM_NO_CACHE = 8  # include/vlgpu.h: VL_BEAM_NO_CACHE (no per-row cache of evaluated distances; same result)
BEAM_USES_SKETCH = 16  # include/vlgpu.h: VL_BEAM_USES_SKETCH (set by closest_vectors when it is given a sketch)
BEAM_WINDOWS = 32  # include/vlgpu.h: VL_BEAM_WINDOWS (several iterations per launch while rows are independent; same result)


def _beam_params(batch: int, dim: int, n_vectors: int, width: int, queue: Queue, config: Dict,
                 excl_cols: int, flags: int = 0) -> nv.BeamParams:
    return nv.BeamParams(
        n_rows=batch, dim=dim, n_vectors=n_vectors, width=width, queue_capacity=queue.indices.size(1),
        queue_length=queue.length, beam_size=config["beam_size"],
        parallel_visit_count=config["parallel_visit_count"], visit_queue_factor=config["visit_queue_factor"],
        exclude_factor=config["exclude_factor"], speculative_readahead=config["speculative_readahead"],
        excl_cols=excl_cols, flags=flags, metric=nv.metric_code(config.get("metric", "cosine")))


class _Workspace:
    """Scratch memory of the beam-search loop for one (device, stream): the loop's control
    block, visit queues, visited lists and distance cache live in it, so two calls must
    never share it while either runs.  The lock serialises host threads that launch on the
    same stream; calls on different streams get different workspaces and may overlap."""

    def __init__(self):
        self.lock = threading.Lock()
        self.tensor: Optional[Tensor] = None

    def reserve(self, nbytes: int, device) -> Tensor:
        if self.tensor is None or self.tensor.numel() < nbytes:
            self.tensor = None  # let the old block go before the larger one is asked for
            self.tensor = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        return self.tensor


_WORKSPACES: Dict[Tuple[str, int], _Workspace] = {}
_WORKSPACES_LOCK = threading.Lock()


def _workspace(device) -> _Workspace:
    """The workspace of torch's current stream on `device` (owned by torch's allocator)."""
    dev = torch.device(device)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    key = (f"cuda:{index}", int(torch.cuda.current_stream(index).cuda_stream))
    with _WORKSPACES_LOCK:
        ws = _WORKSPACES.get(key)
        if ws is None:
            _WORKSPACES[key] = ws = _Workspace()
    return ws


def release_workspaces(streams=None) -> None:
    """Drop the scratch memory kept for beam searches (one block per device and stream, sized by the largest
    batch seen; several GB after a large build) - of the given torch streams only, or of all.  The next search
    on such a stream allocates what it needs again."""
    only = None if streams is None else {int(st.cuda_stream) for st in streams}
    with _WORKSPACES_LOCK:
        for ((_, stream), ws) in _WORKSPACES.items():
            if only is not None and stream not in only:
                continue
            with ws.lock:
                ws.tensor = None


_BUILD_STREAMS: Dict[str, list] = {}


def _build_streams(device, lanes: int) -> list:
    """The side streams every build on `device` shares (each stream owns a beam-search workspace, so builds
    must not create streams of their own every time)."""
    dev = torch.device(device)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    with _WORKSPACES_LOCK:
        streams = _BUILD_STREAMS.setdefault(f"cuda:{index}", [])
        while len(streams) < lanes:
            streams.append(torch.cuda.Stream(device=index))
        return streams[:lanes]


def closest_vectors_stepwise(query_vecs: Tensor, search_queue: Queue, vectors: Tensor, beams: Tensor, config: Dict,
                             exclude: Optional[Tensor] = None) -> int:
    """The loop of ann.py:38-93 statement by statement on the single-purpose
    kernels (one launch and, for the visited list, one host sync per step).
    Same result as closest_vectors; kept for checking the fused loop."""
    (_, beam_size) = beams.size()
    extra_capacity = beam_size * config["parallel_visit_count"]
    (batch_size, _) = search_queue.size()
    visit_queue_len = config["visit_queue_factor"] * config["beam_size"]
    capacity = visit_queue_len + extra_capacity
    device = vectors.device
    visit_queue = Queue(batch_size, visit_queue_len, capacity, device=device)
    visit_queue.initialize_from_queue(search_queue)
    exclude_len = config["exclude_factor"] * visit_queue_len
    seen = torch.full((batch_size, exclude_len), MAXINT, dtype=torch.int32, device=device)

    progressing = True
    count = 0
    while progressing:
        count += 1
        checking_output = (count % config["speculative_readahead"]) == 0
        neighbors_to_visit = visit_queue.pop_n_ids(config["parallel_visit_count"])
        (indexes_of_comparisons, distances_of_comparisons) = search_from_seeds(
            query_vecs, neighbors_to_visit, beams, vectors, config.get("metric", "cosine"))
        did_something = search_queue.insert(indexes_of_comparisons, distances_of_comparisons, exclude=exclude,
                                            output_update=checking_output)
        if seen is not None:
            seen = add_new_to_seen_(seen, neighbors_to_visit)
        if seen is not None:
            visit_queue.insert(indexes_of_comparisons, distances_of_comparisons, exclude=seen)
        if checking_output:
            progressing = bool(torch.any(did_something))
    return count


@log_time
def closest_vectors(query_vecs: Tensor, search_queue: Queue, vectors: Tensor, beams: Tensor, config: Dict,
                    exclude: Optional[Tensor] = None, flags: int = 0, sketch: Optional[Tensor] = None) -> int:
    """reference ann.py:38-93.  Updates search_queue in place; returns the
    number of iterations run (the reference returns True).  Rows are exact on
    [:, :search_queue.length]; the slots beyond are unspecified.  flags picks
    another form of the same loop (BEAM_TWO_LAUNCHES, BEAM_SORT_MERGE) or the
    per-query stop (BEAM_PER_QUERY_STOP: not the reference's loop, which keeps
    every row expanding until the whole batch is quiet, ann.py:90-91).

    The default form relies on what Queue.insert leaves behind: rows ordered by
    (distance, id) with distinct ids, and an id carrying the same distance
    wherever it occurs, i.e. the queue's distances are distances to `vectors`
    rows under this call's query rows.  For a queue in any other state pass
    BEAM_SORT_MERGE, which sorts whole rows like the reference does.

    sketch (an addition): the 8-bit sketch of `vectors` from kernels.build_sketch.
    Rows whose candidates rarely repeat then look at their candidates through the
    sketch first and fetch only the rows that can still enter a queue; the
    result is the same, bit for bit."""
    assert query_vecs.dtype == torch.float32 and vectors.dtype == torch.float32 and beams.dtype == torch.int32
    nv.require_gpu(query_vecs, vectors, beams, search_queue.indices, exclude)
    query_vecs = query_vecs.contiguous()
    assert vectors.is_contiguous() and beams.is_contiguous()
    assert search_queue.indices.is_contiguous() and search_queue.distances.is_contiguous()
    (batch, dim) = query_vecs.size()
    assert search_queue.indices.size(0) == batch and vectors.size(1) == dim and beams.size(0) == vectors.size(0)
    excl = None
    if exclude is not None:
        assert exclude.dtype == torch.int32 and exclude.size(0) == batch
        excl = exclude.contiguous()
    p = _beam_params(batch, dim, vectors.size(0), beams.size(1), search_queue, config,
                     0 if excl is None else excl.size(1), flags | (BEAM_USES_SKETCH if sketch is not None else 0))
    need = nv.check(nv.lib().vl_beam_workspace_bytes(ctypes.byref(p)))
    workspace = _workspace(vectors.device)
    with workspace.lock:
        ws = workspace.reserve(need, vectors.device)
        if sketch is not None:
            assert sketch.dtype == torch.uint8 and sketch.is_contiguous() and sketch.is_cuda
            assert sketch.size() == (vectors.size(0), sketch_row_bytes(dim)), "not a sketch of these vectors"
        iterations = nv.check(nv.lib().vl_closest_vectors_with_sketch(
            ctypes.byref(p), nv.ptr(query_vecs), nv.ptr(vectors), nv.ptr(sketch), nv.ptr(beams),
            nv.ptr(search_queue.indices), nv.ptr(search_queue.distances), nv.ptr(excl), nv.ptr(ws), ws.numel(),
            nv.stream()))
    with _WORKSPACES_LOCK:
        _log.BEAM_ITERATIONS += iterations
    return iterations


def excluding_self(start: int, end: int, queue_length: int = 0, device=DEVICE) -> Tensor:
    """reference ann.py:315-320: one exclusion per row, the row's own id"""
    return torch.arange(start, end, dtype=torch.int32, device=device).unsqueeze(1)


class GraphBuild:
    """generate_ann (reference ann.py:109-193) as a sequence of batch steps, so a
    caller can time or interleave them.  One step = one batch of rows taken
    through closest_vectors against the current graph; the step that ends an
    optimisation loop also prunes and runs the self-recall test.

    The reference seeds every optimisation loop with the distances of the
    initial circulant graph and returns those too (ann.py:145-147,172,190-193),
    so from the second loop on ids and distances no longer belong together.
    Here the distances travel with their ids; stale_distances=True restores the
    reference's behaviour (and then uses the step-by-step loop, because the
    fused loop relies on an id always carrying the same distance)."""

    def __init__(self, vectors: Tensor, config: Dict, stale_distances: bool = False,
                 initial: Optional[Tuple[Tensor, Tensor]] = None, keep_history: bool = False,
                 concurrent_batches: int = 3):
        """initial: (ids, distances) tables of the build-queue width to start from instead of the
        circulant graph (a later optimisation loop's starting state).  keep_history: keep a
        reference to the tables every optimisation loop started from in self.history."""
        self.vectors = vectors
        self.config = config
        self.stale = stale_distances
        self.concurrent = concurrent_batches  # batches of a loop kept in flight (see steps)
        self._streams = None
        (self.num_vecs, _) = vectors.size()
        device = vectors.device
        self.beam_size = config["beam_size"]
        self.queue_length = self.beam_size * config["beam_queue_factor"]
        self.circulant_start = initial is None
        if initial is None:
            neighbor_primes = primes(self.queue_length, device)
            self.beams = generate_circulant_beams(self.num_vecs, neighbor_primes)
            self.beam_distances = calculate_distances(vectors, self.beams, metric=config.get("metric", "cosine"))
        else:
            (self.beams, self.beam_distances) = initial
            assert self.beams.size() == (self.num_vecs, self.queue_length) == self.beam_distances.size()
        self.distances = self.beam_distances
        # 8-bit sketch of the vectors (an addition; config["sketch"] = False turns it off): the first loop's
        # searches sample the table almost at random and keep few of their candidates, which the sketch
        # finds out for a quarter of the traffic.  The graph does not depend on it.
        # Rows below 1 KiB are not worth it: their launches are bound by the merge phase, not by the bytes
        # (measured: -19 % per launch of the first loop at 384 columns, -49 % at 768, +15 % at 128).
        self.sketch = None
        if (config.get("sketch", True) and not stale_distances and config.get("metric", "cosine") == "cosine"
                and 256 <= vectors.size(1) <= 2048 and vectors.size(1) % 4 == 0):
            self.sketch = build_sketch(vectors)
        self.stats: list = []  # one dict per finished optimisation loop
        self.history: Optional[list] = [] if keep_history else None
        self.finished = False

    def batches_per_loop(self) -> int:
        bs = self.config["batch_size"]
        return (self.num_vecs + bs - 1) // bs

    def steps(self):
        """Generator: runs the build, yielding (loop, start, end, iterations) after each batch."""
        config, vectors, device = self.config, self.vectors, self.vectors.device
        ql = self.queue_length
        remaining_capacity = ql * config["parallel_visit_count"]
        batch_size = config["batch_size"]
        search = closest_vectors_stepwise if self.stale else closest_vectors
        for loop in range(0, config["optimization_loops"]):
            loop_start = time.time()
            iterations = 0
            if self.history is not None:
                self.history.append((self.beams, self.beam_distances if self.stale else self.distances))
            next_beams = torch.empty_like(self.beams)
            next_beam_distances = torch.empty_like(self.beam_distances)
            seed_distances = self.beam_distances if self.stale else self.distances

            def run_batch(start: int, stream) -> int:
                end = min(start + batch_size, self.num_vecs)
                with torch.cuda.stream(stream):
                    exclude = excluding_self(start, end, ql, device)
                    queue = Queue(end - start, ql, ql + remaining_capacity, device=device)
                    queue.insert(self.beams.narrow(0, start, end - start), seed_distances.narrow(0, start, end - start))
                    if self.sketch is not None:
                        # the neighbour lists of a circulant graph share little, so a search of it meets few
                        # candidates twice (27 % at 1M x 768): with short sketch rows the cache's probes cost
                        # more than those repeats save, with long ones less (per launch, without and with the
                        # cache: 0.35 and 0.37 ms at 384 columns, 0.73 and 0.64 ms at 768, 1.54 and 1.24 ms at 1536)
                        first = BEAM_NO_CACHE if (loop == 0 and self.circulant_start and vectors.size(1) <= 512) else 0
                        t = search(vectors[start:end], queue, vectors, self.beams, config, exclude, flags=first,
                                   sketch=self.sketch)
                    else:
                        t = search(vectors[start:end], queue, vectors, self.beams, config, exclude)
                    next_beams.narrow(0, start, end - start).copy_(queue.indices.narrow(1, 0, ql))
                    next_beam_distances.narrow(0, start, end - start).copy_(queue.distances.narrow(1, 0, ql))
                    stream.synchronize()
                return t

            # The batches of a loop only read the previous loop's table and write disjoint rows of the next
            # one (ann.py:132-166), so `concurrent` of them are kept in flight, each on a stream and a host
            # thread of its own: while one batch's launch drains, the other's fills the idle compute units.
            # The result does not depend on it.
            starts = list(range(0, self.num_vecs, batch_size))
            lanes = max(1, min(self.concurrent, len(starts)))
            torch.cuda.synchronize(device)  # the tables come from the main stream
            if lanes == 1:
                results = ((start, run_batch(start, torch.cuda.current_stream(device))) for start in starts)
            else:
                results = self._in_flight(run_batch, starts, lanes, device)
            for (start, t) in results:
                end = min(start + batch_size, self.num_vecs)
                iterations += t
                last = end == self.num_vecs
                if last:
                    recall = self._finish_loop(next_beams, next_beam_distances)
                    torch.cuda.synchronize(device)
                    self.stats.append(dict(loop=loop, seconds=time.time() - loop_start, iterations=iterations,
                                           self_recall=recall))
                yield (loop, start, end, t)
            if recall == 1.0:  # ann.py:187
                break
        self.finished = True
        if self._streams is not None:
            # the side streams' beam-search workspaces (one per batch in flight, each with its own distance cache)
            # are only worth keeping while batches run
            release_workspaces(self._streams)

    def _in_flight(self, run_batch, starts, lanes: int, device):
        """Runs run_batch(start, stream) for every start with `lanes` of them in flight, yielding
        (start, result) in the order of `starts`."""
        from concurrent.futures import ThreadPoolExecutor

        self._streams = _build_streams(device, lanes)
        with ThreadPoolExecutor(max_workers=lanes) as pool:
            pending = []
            for k, start in enumerate(starts):
                if len(pending) == lanes:
                    (s0, f0) = pending.pop(0)
                    yield (s0, f0.result())
                # batch k runs on stream k % lanes, free again because batch k - lanes has been waited for
                pending.append((start, pool.submit(run_batch, start, self._streams[k % lanes])))
            for (s0, f0) in pending:
                yield (s0, f0.result())

    def _finish_loop(self, next_beams: Tensor, next_beam_distances: Tensor) -> float:
        if self.config["prune"] is True:  # ann.py:171-177 (prune="rank" thins nothing between loops)
            (self.beams, self.distances) = prune_(next_beams, next_beam_distances)
        else:
            (self.beams, self.distances) = (next_beams, next_beam_distances)
        prefix = min(self.num_vecs, 1000)  # ann.py:179-185
        (_, recall) = ann_calculate_recall(self.vectors, self.beams.narrow_copy(1, 0, self.beam_size), self.config,
                                           sample=self.vectors[:prefix])
        return recall

    def result(self) -> Tuple[Tensor, Tensor]:
        if self.config["prune"] == "rank":
            # addition: cut the full-width table to beam_size by detour count and merge reverse edges
            ids = optimize_graph(self.beams, self.beam_size)
            return (ids, gather_distances(self.vectors, self.vectors, ids, metric=self.config.get("metric", "cosine")))
        out_distances = self.beam_distances if self.stale else self.distances  # ann.py:190-193
        return (self.beams.narrow_copy(1, 0, self.beam_size), out_distances.narrow_copy(1, 0, self.beam_size))


def generate_ann(vectors: Tensor, config: Dict, stale_distances: bool = False,
                 stats: Optional[list] = None, concurrent_batches: int = 3) -> Tuple[Tensor, Tensor]:
    """reference ann.py:109-193 (see GraphBuild).  stats, when given, receives
    one dict per optimisation loop (wall seconds, beam-search iterations summed
    over batches, self-recall)."""
    build = GraphBuild(vectors, config, stale_distances, concurrent_batches=concurrent_batches)
    for _ in build.steps():
        pass
    if stats is not None:
        stats.extend(build.stats)
    return build.result()


def initial_queue(vectors: Tensor, config: Dict) -> Queue:
    """reference ann.py:196-208"""
    queue_size = config["recall_search_queue_factor"] * config["beam_size"]
    (batch_size, _) = vectors.size()
    extra_capacity = max(queue_size, config["parallel_visit_count"] * config["beam_size"])
    queue = Queue(batch_size, queue_size, queue_size + extra_capacity, device=vectors.device)
    p = primes(queue_size, vectors.device)
    initial_queue_indices = generate_circulant_beams(batch_size, p)
    d = calculate_distances(vectors, initial_queue_indices, metric=config.get("metric", "cosine"))
    queue.insert(initial_queue_indices, d)
    return queue


def query_cosine_distances(query_vectors: Tensor, vectors: Tensor, ids: Tensor, metric: str = "cosine") -> Tensor:
    """d[b, j] = clamp((1 - <query[b], vectors[ids[b, j]]>) / 2, 0, 1).

    The reference's version (ann.py:211-214) multiplies [B, D] by a gathered
    [B, Q, D] tensor, which only broadcasts for one query, and leaves out the
    clamp; this one evaluates the seeds with the kernel every other distance
    uses, so a seed found again during the search carries identical bits.
    metric="l2" (an addition) gives squared Euclidean distances instead."""
    return gather_distances(query_vectors, vectors, ids, metric=metric)


def initial_search_queue(vectors: Tensor, query_vectors: Tensor, config: Dict,
                         queue_size: Optional[int] = None) -> Queue:
    """reference ann.py:217-232; queue_size overrides recall_search_queue_factor * beam_size"""
    if queue_size is None:
        queue_size = config["recall_search_queue_factor"] * config["beam_size"]
    (batch_size, _) = query_vectors.size()
    extra_capacity = max(queue_size, config["parallel_visit_count"] * config["beam_size"])
    queue = Queue(batch_size, queue_size, queue_size + extra_capacity, device=vectors.device)
    p = primes(queue_size, vectors.device)
    (vector_count, _) = vectors.size()
    initial_queue_indices = generate_queue_circulants(batch_size, vector_count, p)
    d = query_cosine_distances(query_vectors, vectors, initial_queue_indices, config.get("metric", "cosine"))
    queue.insert(initial_queue_indices, d)
    return queue


DENSE_SEEDS = 16  # seeds per query taken from the entry-point tiles (the exact-kNN kernel keeps 16 per lane)


def entry_point_ids(vector_count: int, entry_points: int, device=DEVICE) -> Tensor:
    """Ids of the entry-point sample: entry_points ids spread evenly over [0, vector_count)."""
    s = min(entry_points, vector_count)
    return ((torch.arange(s, dtype=torch.int64, device=device) * vector_count) // s).to(torch.int32)


def dense_search_queue(vectors: Tensor, query_vectors: Tensor, config: Dict, entry_ids: Tensor,
                       entry_vectors: Tensor, queue_size: Optional[int] = None,
                       seeds: Optional[int] = None) -> Queue:
    # entry_vectors may hold only the first columns of the entry points (ANN.seed_dims): the seeds are
    # then ranked by that part of the dot product, which is enough to land near the query; the distances
    # that enter the queue are always the full ones.
    """Query-dependent seeding (not in the reference, whose seeds (b + p_k) % N ignore
    the query, utils.py:26-32): the seeds of a query are its DENSE_SEEDS nearest
    entry points, found with one dense query x entry-point pass on fp32 MFMA tiles.
    Their distances are then re-evaluated with the gathered-distance kernel so that
    a seed met again during the search carries identical bits.  Same queue shape as
    initial_search_queue (ann.py:217-232); slots beyond the seeds start empty."""
    if queue_size is None:
        queue_size = config["recall_search_queue_factor"] * config["beam_size"]
    (batch_size, _) = query_vectors.size()
    extra_capacity = max(queue_size, config["parallel_visit_count"] * config["beam_size"])
    queue = Queue(batch_size, queue_size, queue_size + extra_capacity, device=vectors.device)
    k = min(seeds or DENSE_SEEDS, DENSE_SEEDS, entry_ids.size(0), queue_size)
    cols = entry_vectors.size(1)
    ranked_by = query_vectors if cols == query_vectors.size(1) else query_vectors[:, :cols].contiguous()
    (local, _) = knn_exact(ranked_by, entry_vectors, k, config.get("metric", "cosine"))
    seeds = entry_ids[local.long()].contiguous()
    d = query_cosine_distances(query_vectors, vectors, seeds, config.get("metric", "cosine"))
    queue.insert(seeds, d)
    return queue


def _flags_for_sample(sample: Tensor, vectors: Tensor) -> int:
    """initial_queue (ann.py:196-208) seeds row i with ids over the SAMPLE and their distances to
    sample rows.  When the sample is the head of `vectors` those are also the distances to
    vectors[id], which is what the loop evaluates, and the default form of the loop applies.  For
    any other sample an id can carry two different distances, which only the form that sorts whole
    rows like the reference treats as the reference does."""
    return 0 if sample.data_ptr() == vectors.data_ptr() else BEAM_SORT_MERGE


def ann_calculate_recall(vectors: Tensor, beams: Tensor, config: Dict, sample: Optional[Tensor] = None,
                         verbose: bool = False):
    """reference ann.py:235-259: share of sample rows whose best hit is themselves"""
    if sample is None:
        sample = vectors
    (sample_size, _) = sample.size()
    queue = initial_queue(sample.contiguous(), config)
    closest_vectors(sample, queue, vectors, beams.contiguous(), config, flags=_flags_for_sample(sample, vectors))
    expected = torch.arange(sample_size, device=vectors.device)
    actual = queue.indices.t()[0]
    found = (expected == actual).sum().item()
    if verbose:
        print(f"found: {found} / {sample_size}")
        print(f"recall: {found / sample_size}")
    return (found, found / sample_size)


def search_layers(layers, query_vecs: Tensor, search_queue: Queue, vectors: Tensor, config: Dict, flags: int = 0):
    """reference ann.py:96-106: one beam search per neighbour table, coarse to fine, each starting
    from the queue the previous one left.  Every table is [N, width] over the ids of `vectors`;
    no ids are excluded, because the queries are vectors, not rows of the index."""
    for layer in layers:
        closest_vectors(query_vecs, search_queue, vectors, layer.contiguous(), config, None, flags=flags)


def hnsw_calculate_recall(vectors: Tensor, hnsw, config: Dict, sample: Optional[Tensor] = None, verbose: bool = True):
    """reference ann.py:262-284: self-recall@1 of a layered search.  (There the expected ids are
    built on the CPU and compared with a device tensor; here they live on the device.)"""
    if sample is None:
        sample = vectors
    (sample_size, _) = sample.size()
    queue = initial_queue(sample.contiguous(), config)
    search_layers(hnsw, sample, queue, vectors, config, flags=_flags_for_sample(sample, vectors))
    expected = torch.arange(sample_size, device=vectors.device)
    found = (expected == queue.indices.t()[0]).sum().item()
    if verbose:
        print(f"found: {found} / {sample_size}")
        print(f"recall: {found / sample_size}")
    return (found, found / sample_size)


def print_timestamp(msg):
    """reference ann.py:297-298"""
    print(msg)


def ann_recall_test(vectors: Tensor, config: Dict):
    """reference ann.py:287-293: build, then self-recall@1 over the first 10,000 rows"""
    (beams, _) = generate_ann(vectors, config)
    print_timestamp("=> ANN generated")
    prefix = min(vectors.size()[0], 10_000)
    return ann_calculate_recall(vectors, beams, config, sample=vectors[:prefix])


class ANN:
    """reference ann.py:356-489"""

    def __init__(
        self,
        vectors: Tensor,
        prune: bool = True,
        beam_size: int = 24,
        parallel_visit_count: int = 4,
        beam_queue_factor: int = 3,
        visit_queue_factor: int = 3,
        exclude_factor: int = 5,
        optimization_loops: int = 3,
        batch_size: int = 10_000,
        recall_search_queue_factor: int = 3,
        speculative_readahead: int = 5,
        beams: Optional[Tensor] = None,
        distances: Optional[Tensor] = None,
        seeding: str = "circulant",
        entry_points: int = 32_768,
        keep_queues: bool = False,
        metric: str = "cosine",
        concurrent_batches: int = 3,
        seed_dims: Optional[int] = None,
        sketch: bool = True,
        dense_seeds: Optional[int] = None,
    ):
        """seeding / entry_points are additions: "circulant" seeds searches as the
        reference does; "dense" seeds them from the nearest of `entry_points`
        evenly spread vectors (see dense_search_queue).  prune also accepts
        "rank": no pruning between loops, and the final cut from the build queue
        width to beam_size is done by detour count with reverse edges merged in
        (kernels.optimize_graph) instead of keeping the first beam_size columns.
        seed_dims (with seeding="dense") ranks the entry points by their first seed_dims
        columns only - a cheaper pass that still lands near the query; None uses all.
        dense_seeds (with seeding="dense") is the number of nearest entry points a query starts from
        (None: as many as the search queue holds, 16 at most); the tile pass keeps shorter lists for fewer.
        concurrent_batches (an addition) is the number of batches of an optimisation loop
        that the build keeps in flight, each on its own stream and host thread; the
        graph does not depend on it.  Three by default: with the stream of the caller that makes
        four, as many as a process has hardware queues by default - a fourth batch shares one
        (measured at 1M x 768: 21.2 / 21.4 / 22.0 / 21.3 / 21.7 s with 2 / 3 / 4 / 6 / 8 in flight,
        the same order at 128 and 384 columns).  metric is an addition too: "cosine" is the reference's distance; "l2" builds
        and searches by squared Euclidean distance (rows need not be unit length);
        dense seeding and recall_at_k follow the metric.  sketch (an addition): the build keeps an
        8-bit copy of rows of 1 KiB and more and lets searches of the initial graph decide from it
        which candidate rows to fetch (kernels.build_sketch); the graph is the same either way."""
        assert prune in (True, False, "rank")
        nv.metric_code(metric)
        assert vectors.dim() == 2 and vectors.dtype == torch.float32
        assert seeding in ("circulant", "dense")
        self.seeding = seeding
        self.entry_points = entry_points
        self.seed_dims = seed_dims
        self.dense_seeds = dense_seeds
        assert dense_seeds is None or dense_seeds >= 1
        assert seed_dims is None or (seed_dims > 0 and seed_dims % 4 == 0), "seed_dims must be a multiple of 4"
        self._entry = None
        self._queues = None
        self._sketch = None   # the 8-bit sketch of the vectors, when the build made one (or a search asked for it)
        (count, dim) = vectors.size()
        self.configuration: Dict = {
            "prune": prune,
            "beam_size": beam_size,
            "parallel_visit_count": parallel_visit_count,
            "beam_queue_factor": beam_queue_factor,
            "visit_queue_factor": visit_queue_factor,
            "exclude_factor": exclude_factor,
            "optimization_loops": optimization_loops,
            "batch_size": batch_size,
            "recall_search_queue_factor": recall_search_queue_factor,
            "speculative_readahead": speculative_readahead,
        }
        if metric != "cosine":
            self.configuration["metric"] = metric
        if not sketch:
            self.configuration["sketch"] = False
        if not vectors.is_cuda:
            vectors = vectors.to(DEVICE)
        self.vectors = vectors.contiguous()
        wall_start = time.time()
        if beams is not None:
            self.beams = beams.to(self.vectors.device).contiguous()
            if distances is None:
                self.distances = calculate_distances(self.vectors, self.beams, metric=metric)
            else:
                self.distances = distances.to(self.vectors.device).contiguous()
        else:
            build = GraphBuild(self.vectors, self.configuration, concurrent_batches=concurrent_batches)
            for _ in build.steps():
                pass
            self.build_stats: list = build.stats
            # the build's sketch (N x (16 * ceil(dim / 16) + 8) bytes) is let go with the build: searches
            # run without one unless they ask (search(sketch=True) makes it again)
            (self.beams, self.distances) = build.result()
            if keep_queues:
                width = build.beams.size(1)
                self._queues = Queue(count, width, width + 1, device=self.vectors.device)
                self._queues.indices[:, :width].copy_(build.beams)
                self._queues.distances[:, :width].copy_(build.distances)
        torch.cuda.synchronize(self.vectors.device)
        wall_end = time.time()
        self.log = self.configuration.copy()
        self.log["total_time"] = wall_end - wall_start
        self.log["vector_count"] = count
        self.log["vector_dimension"] = dim

    @classmethod
    def load_from_dataframe(cls, dataframe, device=DEVICE, **kwargs) -> "ANN":
        """reference ann.py:408-454: `dataframe` has the columns vector_id, embedding and
        beams and optionally distances; rows are taken in vector_id order.  Accepts a
        pyarrow Table or anything with DataFusion's `to_arrow_table()`."""
        import pyarrow as pa
        import pyarrow.compute as pc

        from .datafusion import dataframe_to_tensor

        table = dataframe.to_arrow_table() if hasattr(dataframe, "to_arrow_table") else dataframe
        assert isinstance(table, pa.Table), "expected a pyarrow Table or a DataFusion DataFrame"
        names = table.schema.names
        assert "embedding" in names and "beams" in names
        if "vector_id" in names:
            table = table.take(pc.sort_indices(table, sort_keys=[("vector_id", "ascending")]))
        count = table.num_rows

        def width(name):
            t = table.schema.field(name).type
            if pa.types.is_fixed_size_list(t):
                return t.list_size
            return len(table.column(name)[0]) if count else 0

        vectors = torch.empty((count, width("embedding")), dtype=torch.float32, device=device)
        dataframe_to_tensor(table, vectors, "embedding")
        beams = torch.empty((count, width("beams")), dtype=torch.int32, device=device)
        dataframe_to_tensor(table, beams, "beams")
        distances = None
        if "distances" in names:
            distances = torch.empty((count, beams.size(1)), dtype=torch.float32, device=device)
            dataframe_to_tensor(table, distances, "distances")
        return cls(vectors, beam_size=beams.size(1), beams=beams, distances=distances, **kwargs)

    def to_arrow(self):
        """The index as a pyarrow Table with the columns load_from_dataframe reads."""
        import pyarrow as pa

        from .datafusion import tensor_to_arrow

        return pa.table({
            "vector_id": pa.array(range(self.vectors.size(0)), type=pa.int32()),
            "embedding": tensor_to_arrow(self.vectors),
            "beams": tensor_to_arrow(self.beams),
            "distances": tensor_to_arrow(self.distances),
        })

    def recall(self, sample_size: int = 1000) -> Tuple[float, float]:
        """reference ann.py:456-464"""
        (count, _) = self.vectors.size()
        sample_size = min(sample_size, count)
        sample = self.vectors[0:sample_size]
        return ann_calculate_recall(self.vectors, self.beams, self.configuration, sample)

    def clusters(self):
        """reference ann.py:466-467 is a stub (`pass`); its README says "returns all search
        queues".  Here: the search queues the build ended with, one per vector at the
        build queue width, as a Queue - when the index was built with keep_queues=True;
        otherwise None, like the reference."""
        return self._queues

    def _entry_tables(self):
        if self._entry is None:
            ids = entry_point_ids(self.vectors.size(0), self.entry_points, self.vectors.device)
            rows = self.vectors[ids.long()]
            if self.seed_dims is not None and self.seed_dims < rows.size(1):
                rows = rows[:, :self.seed_dims]
            self._entry = (ids, rows.contiguous())
        return self._entry

    def _search_sketch(self, use: bool) -> Optional[Tensor]:
        """The sketch for a search that asks for one (made now if the build did not make it)."""
        dim = self.vectors.size(1)
        able = (self.configuration.get("sketch", True) and self.configuration.get("metric", "cosine") == "cosine"
                and dim % 4 == 0 and dim <= 2048)
        if not (use and able):
            return None
        if self._sketch is None:
            self._sketch = build_sketch(self.vectors)
        return self._sketch

    def search(self, query: Tensor, queue_size: Optional[int] = None, seeding: Optional[str] = None,
               stop: str = "batch", sketch: bool = False) -> Queue:
        """reference ann.py:469-477: takes a batch of query vectors, returns the
        search Queue; the answer is queue.indices[:, :k] / queue.distances[:, :k].
        queue_size overrides the configured search-queue length, seeding the
        instance's seeding mode.  stop="batch" is the reference's loop (every row
        expands until no row of the batch changed at a progress check);
        stop="per_query" finishes each row on its own after speculative_readahead
        iterations in a row that left its queue unchanged - faster for large
        batches, not the reference's result.  sketch=True (an addition) lets the
        search decide from the 8-bit sketch of the vectors which candidate rows to
        fetch; the result is the same.  Off by default: a search runs on the pruned
        graph, whose candidates are near neighbours the sketch cannot tell apart, so
        its rows give the sketch up after a few iterations (measured: 64 k QPS
        either way at 1M x 1536, 120 k without and 116 k with it at 1M x 768)."""
        assert stop in ("batch", "per_query")
        assert query.dim() == 2 and query.dtype == torch.float32
        if not query.is_cuda:
            query = query.to(self.vectors.device)
        query = query.contiguous()
        seeding = seeding or self.seeding
        assert seeding in ("circulant", "dense")
        if seeding == "dense":
            (entry_ids, entry_vectors) = self._entry_tables()
            search_queue = dense_search_queue(self.vectors, query, self.configuration, entry_ids, entry_vectors,
                                              queue_size, self.dense_seeds)
        else:
            search_queue = initial_search_queue(self.vectors, query, self.configuration, queue_size)
        closest_vectors(query, search_queue, self.vectors, self.beams, self.configuration, None,
                        flags=BEAM_PER_QUERY_STOP if stop == "per_query" else 0, sketch=self._search_sketch(sketch))
        return search_queue

    def recall_at_k(self, query: Tensor, k: int = 10, queue_size: Optional[int] = None,
                    seeding: Optional[str] = None) -> float:
        """Share of the exact k nearest neighbours (brute force on MFMA tiles)
        that search() returns in its first k slots.  Not in the reference,
        whose recall() is self-recall@1."""
        if not query.is_cuda:
            query = query.to(self.vectors.device)
        query = query.contiguous()
        found = self.search(query, queue_size, seeding).indices[:, :k]
        (truth, _) = knn_exact(query, self.vectors, k, self.configuration.get("metric", "cosine"))
        hits = (found.unsqueeze(2) == truth.unsqueeze(1)).any(dim=2).sum().item()
        return hits / truth.numel()

    def dump_logs(self) -> Dict:
        """reference ann.py:479-489 without the nvidia-smi / git shell-outs"""
        out = self.log.copy()
        out["closest_vectors_batch_time"] = _log.CLOSEST_VECTORS_BATCH_TIME
        out["gpu_arch"] = torch.cuda.get_device_name(self.vectors.device)
        (_, recall) = self.recall()
        out["recall"] = recall
        return out
