"""Launchers with the names and signatures of the reference's
vectorlink_gpu/kernels.py; every body is a call into libvlgpu.so (hand-written
HIP for gfx950) on torch's current stream."""
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _native as nv
from .constants import MAXFLOAT, MAXINT
from .log import log_time


def _check_ids(t: Tensor, name: str):
    assert t.dtype == torch.int32, f"{name} must be int32"
    assert t.is_contiguous(), f"{name} must be contiguous"


def _check_f32(t: Tensor, name: str):
    assert t.dtype == torch.float32, f"{name} must be float32"
    assert t.is_contiguous(), f"{name} must be contiguous"


def gather_distances(queries: Tensor, vectors: Tensor, ids: Tensor, out: Optional[Tensor] = None,
                     metric: str = "cosine") -> Tensor:
    """out[r, j] = distance of queries[r] and vectors[ids[r, j]] (MAXFLOAT for MAXINT ids): the reference's
    cosine distance, or with metric="l2" (an addition) the squared Euclidean distance."""
    _check_f32(queries, "queries")
    _check_f32(vectors, "vectors")
    _check_ids(ids, "ids")
    nv.require_gpu(queries, vectors, ids)
    (rows, width) = ids.size()
    assert queries.size(0) == rows and queries.size(1) == vectors.size(1)
    if out is None:
        out = torch.empty((rows, width), dtype=torch.float32, device=ids.device)
    else:
        _check_f32(out, "out")
        assert out.size() == ids.size()
    nv.check(nv.lib().vl_gather_distances_metric(nv.ptr(queries), rows, nv.ptr(vectors), vectors.size(0),
                                                 vectors.size(1), nv.ptr(ids), width, nv.metric_code(metric),
                                                 nv.ptr(out), nv.stream()))
    return out


@log_time
def calculate_distances(vectors: Tensor, beams: Tensor, distances_out: Optional[Tensor] = None,
                        metric: str = "cosine") -> Tensor:
    """reference kernels.py:174-201"""
    _check_f32(vectors, "vectors")
    _check_ids(beams, "beams")
    (vector_count, _) = vectors.size()
    (batches, _) = beams.size()
    assert batches == vector_count  # kernels.py:186
    return gather_distances(vectors, vectors, beams, distances_out, metric)


def search_from_seeds(query_vecs: Tensor, neighbors_to_visit: Tensor, beams: Tensor,
                      vectors: Tensor, metric: str = "cosine") -> Tuple[Tensor, Tensor]:
    """reference kernels.py:260-311"""
    _check_f32(query_vecs, "query_vecs")
    _check_ids(neighbors_to_visit, "neighbors_to_visit")
    _check_ids(beams, "beams")
    _check_f32(vectors, "vectors")
    nv.require_gpu(query_vecs, neighbors_to_visit, beams, vectors)
    (batch_size, visit_length) = neighbors_to_visit.size()
    (node_count, beam_size) = beams.size()
    (vector_count, dim) = vectors.size()
    assert query_vecs.size(0) == batch_size and query_vecs.size(1) == dim
    index_out = torch.empty((batch_size, visit_length * beam_size), dtype=torch.int32, device=vectors.device)
    distance_out = torch.empty((batch_size, visit_length * beam_size), dtype=torch.float32, device=vectors.device)
    nv.check(nv.lib().vl_search_from_seeds_metric(nv.ptr(query_vecs), batch_size, dim, nv.ptr(neighbors_to_visit),
                                                  visit_length, nv.ptr(beams), node_count, beam_size, nv.ptr(vectors),
                                                  vector_count, nv.metric_code(metric), nv.ptr(index_out),
                                                  nv.ptr(distance_out), nv.stream()))
    return (index_out, distance_out)


def dedup_tensor_(ids: Tensor):
    """reference kernels.py:370-380 (in place)"""
    _check_ids(ids, "ids")
    nv.require_gpu(ids)
    nv.check(nv.lib().vl_dedup_ids(nv.ptr(ids), ids.size(0), ids.size(1), nv.stream()))


def dedup_tensor_pair_(ids: Tensor, distances: Tensor):
    """reference kernels.py:383-397 (in place; assumes sorted rows)"""
    _check_ids(ids, "ids")
    _check_f32(distances, "distances")
    assert ids.size() == distances.size()
    nv.require_gpu(ids, distances)
    nv.check(nv.lib().vl_dedup_pairs(nv.ptr(ids), nv.ptr(distances), ids.size(0), ids.size(1), nv.stream()))


def punchout_duplicates_(ids: Tensor, distances: Tensor):
    """reference kernels.py:400-406; works in place and returns the same tensors"""
    _check_ids(ids, "ids")
    _check_f32(distances, "distances")
    assert ids.size() == distances.size()
    nv.require_gpu(ids, distances)
    nv.check(nv.lib().vl_punchout_duplicates(nv.ptr(ids), nv.ptr(distances), ids.size(0), ids.size(1), nv.stream()))
    return (ids, distances)


def prune_(beams: Tensor, distances: Tensor):
    """reference kernels.py:441-468.  Decisions are taken from the tables as
    passed in and the result is returned in new tensors; the inputs are left
    untouched (the reference marks them in place while other blocks read)."""
    _check_ids(beams, "beams")
    _check_f32(distances, "distances")
    assert beams.size() == distances.size()
    nv.require_gpu(beams, distances)
    out_b = torch.empty_like(beams)
    out_d = torch.empty_like(distances)
    nv.check(nv.lib().vl_prune(nv.ptr(beams), nv.ptr(distances), beams.size(0), beams.size(1), nv.ptr(out_b),
                               nv.ptr(out_d), nv.stream()))
    return (out_b, out_d)


def punchout_excluded_(indices: Tensor, distances: Tensor, exclusions: Tensor):
    """reference kernels.py:491-501; indices/distances may be column slices of a wider tensor"""
    assert indices.dtype == torch.int32 and distances.dtype == torch.float32 and exclusions.dtype == torch.int32
    assert indices.dim() == 2 and indices.size() == distances.size()
    assert indices.stride(1) == 1 and distances.stride(1) == 1 and exclusions.stride(1) == 1
    (batch_size, queue_size) = indices.size()
    (batch_size2, exclusion_size) = exclusions.size()
    assert batch_size == batch_size2
    nv.require_gpu(indices, distances, exclusions)
    nv.check(nv.lib().vl_punchout_excluded(nv.ptr(indices), nv.ptr(distances), batch_size, queue_size,
                                           indices.stride(0) if batch_size > 1 else queue_size,
                                           distances.stride(0) if batch_size > 1 else queue_size,
                                           nv.ptr(exclusions), exclusion_size,
                                           exclusions.stride(0) if batch_size > 1 else exclusion_size, nv.stream()))


def index_by_tensor(a: Tensor, b: Tensor) -> Tensor:
    """reference kernels.py:554-559: out[r, c] = a[r, b[r, c]]"""
    assert a.dim() == 2 and a.size() == b.size() and a.element_size() == 4
    nv.require_gpu(a, b)
    a = a.contiguous()
    b = b.contiguous().to(torch.int64)
    out = torch.empty_like(a)
    nv.check(nv.lib().vl_index_by_tensor(nv.ptr(a), nv.ptr(b), nv.ptr(out), a.size(0), a.size(1), nv.stream()))
    return out


def index_sort_(ids: Tensor, distances: Tensor):
    """order rows by (distance, id) in place (reference utils.py:44-53)"""
    _check_ids(ids, "ids")
    _check_f32(distances, "distances")
    nv.require_gpu(ids, distances)
    nv.check(nv.lib().vl_index_sort(nv.ptr(ids), nv.ptr(distances), ids.size(0), ids.size(1), nv.stream()))


def queue_sort_(ids: Tensor, distances: Tensor):
    """reference queue.py:15-18, in place"""
    _check_ids(ids, "ids")
    _check_f32(distances, "distances")
    nv.require_gpu(ids, distances)
    nv.check(nv.lib().vl_queue_sort(nv.ptr(ids), nv.ptr(distances), ids.size(0), ids.size(1), nv.stream()))


def knn_exact(queries: Tensor, vectors: Tensor, k: int, metric: str = "cosine") -> Tuple[Tensor, Tensor]:
    """Exact k nearest neighbours under `metric` on dense fp32 MFMA tiles
    (no counterpart in the reference; ground truth for recall@k).  Returns
    (ids [Q, k] int32, distances [Q, k] float32) ordered by (distance, id)."""
    _check_f32(queries, "queries")
    _check_f32(vectors, "vectors")
    nv.require_gpu(queries, vectors)
    (nq, dim) = queries.size()
    assert vectors.size(1) == dim
    need = nv.check(nv.lib().vl_knn_workspace_bytes(nq, vectors.size(0), dim, k))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=vectors.device)
    ids = torch.empty((nq, k), dtype=torch.int32, device=vectors.device)
    dists = torch.empty((nq, k), dtype=torch.float32, device=vectors.device)
    nv.check(nv.lib().vl_knn_exact_metric(nv.ptr(queries), nq, nv.ptr(vectors), vectors.size(0), dim, k,
                                          nv.metric_code(metric), nv.ptr(ids), nv.ptr(dists), nv.ptr(ws), ws.numel(),
                                          nv.stream()))
    return (ids, dists)


def sketch_row_bytes(dim: int) -> int:
    """Bytes per vector in the 8-bit sketch of [N, dim] vectors: 16 * ceil(dim / 16) of data and 8 of tail."""
    return nv.check(nv.lib().vl_sketch_row_bytes(dim))


def build_sketch(vectors: Tensor) -> Tensor:
    """8-bit sketch of `vectors` (no counterpart in the reference): per vector the
    elements rounded to 8 bits with one scale, and how far the rounding moved the
    vector, which bounds every dot product with it.  One block of
    N * sketch_row_bytes(dim) bytes, shaped [N, sketch_row_bytes(dim)] uint8 for its
    size only: all the data rows come first, then all the tails (sketch_parts takes
    it apart), so a slice of it is not the sketch of a slice of the vectors.
    closest_vectors(..., sketch=...) uses it to decide which candidate rows to
    fetch; no distance it returns comes from the sketch."""
    _check_f32(vectors, "vectors")
    nv.require_gpu(vectors)
    (n, dim) = vectors.size()
    out = torch.empty((n, sketch_row_bytes(dim)), dtype=torch.uint8, device=vectors.device)
    nv.check(nv.lib().vl_sketch_build(nv.ptr(vectors), n, dim, nv.ptr(out), nv.stream()))
    return out


def sketch_parts(sketch: Tensor) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """The parts of a sketch from build_sketch, as views and small copies: the int8 data rows
    [N, 16 * ceil(dim / 16)] (zeros after column dim), and per vector its scale (float32) and the two
    bounds the tail holds as halves, on the 2-norm of what the rounding moved and on the vector's own."""
    (n, row_bytes) = sketch.size()
    data_bytes = row_bytes - 8
    flat = sketch.reshape(-1)
    data = flat[:n * data_bytes].view(torch.int8).reshape(n, data_bytes)
    tails = flat[n * data_bytes:].reshape(n, 8)
    scale = tails[:, :4].contiguous().view(torch.float32).reshape(n)
    bounds = tails[:, 4:].contiguous().view(torch.float16).reshape(n, 2)
    return (data, scale, bounds[:, 0].float(), bounds[:, 1].float())


def sketch_bounds(queries: Tensor, sketch: Tensor, ids: Tensor) -> Tuple[Tensor, Tensor]:
    """(lo, hi) with lo[r, j] <= gather_distances(queries, vectors, ids)[r, j] <= hi[r, j], from the 8-bit sketch
    of `vectors` alone (no counterpart in the reference): what a beam-search row knows of a candidate before it
    decides whether to fetch it."""
    _check_f32(queries, "queries")
    _check_ids(ids, "ids")
    nv.require_gpu(queries, sketch, ids)
    assert sketch.dtype == torch.uint8 and sketch.is_contiguous()
    (rows, m) = ids.size()
    dim = queries.size(1)
    assert queries.size(0) == rows and sketch.size(1) == sketch_row_bytes(dim)
    lo = torch.empty((rows, m), dtype=torch.float32, device=ids.device)
    hi = torch.empty((rows, m), dtype=torch.float32, device=ids.device)
    need = nv.check(nv.lib().vl_sketch_bounds_workspace_bytes(rows, dim))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=ids.device)
    nv.check(nv.lib().vl_sketch_bounds(nv.ptr(queries), rows, dim, nv.ptr(sketch), sketch.size(0), nv.ptr(ids), m,
                                       nv.ptr(lo), nv.ptr(hi), nv.ptr(ws), ws.numel(), nv.stream()))
    return (lo, hi)


def optimize_graph(beams: Tensor, degree: int) -> Tensor:
    """Rank-based graph optimisation (not in the reference): re-order every row of
    `beams` ([N, W], best first, MAXINT = empty) by the number of two-hop detours
    of each edge, cut to `degree`, and merge in reverse edges.  Returns ids
    [N, degree]; see include/vlgpu.h for the exact rule."""
    _check_ids(beams, "beams")
    nv.require_gpu(beams)
    (n, width) = beams.size()
    need = nv.check(nv.lib().vl_optimize_graph_workspace_bytes(n, width, degree))
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=beams.device)
    out = torch.empty((n, degree), dtype=torch.int32, device=beams.device)
    nv.check(nv.lib().vl_optimize_graph(nv.ptr(beams), n, width, degree, nv.ptr(out), nv.ptr(ws), ws.numel(),
                                        nv.stream()))
    return out
