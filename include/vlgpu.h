/*
 * libvlgpu - C ABI of the MI355X (gfx950) kernels behind the vectorlink_gpu
 * Python surface: gathered cosine distances, batched sorted queues, candidate
 * dedup / exclusion, the beam-search loop, detour pruning and exact kNN tiles.
 *
 * The reference has no FFI of its own: its boundary is the set of Python
 * launcher functions in vectorlink_gpu/kernels.py plus the Queue class, all
 * taking torch tensors.  Each entry point below names the launcher or method
 * it stands in for (paths relative to the reference checkout).
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless its name starts with host_;
 *  - matrices are row-major and dense unless a *_stride argument (in
 *    elements) is given; sizes are int64_t;
 *  - ids are int32 with VL_MAXINT as the empty id, distances are float32 with
 *    VL_MAXFLOAT as the empty distance (vectorlink_gpu/constants.py:5-6);
 *    real ids must be below 2^30 (bit 30 is the reference's duplicate flag,
 *    kernels.py:325);
 *  - `stream` is a hipStream_t passed as void*; work is enqueued on it and
 *    the call returns without synchronising unless stated otherwise;
 *  - the library allocates no device memory: scratch comes from the caller
 *    as a workspace whose size the matching *_workspace_bytes call reports;
 *  - threads: every entry point may be called from several host threads at
 *    once (the reference is driven from one thread).  The library's only
 *    shared state is the profiling sums of vl_beam_profile (mutex), the launch
 *    counter of vl_beam_launches (atomic) and the thread-local error text.  A workspace belongs to ONE call at a time: the
 *    beam-search loop keeps its control block, visit queues and visited lists
 *    in it, so two vl_closest_vectors calls in flight need two workspaces;
 *  - return value 0 is success; a negative value is an error whose text
 *    vl_last_error() returns (thread local).  Shapes are validated on the
 *    host before anything is launched.
 */
#ifndef VLGPU_H
#define VLGPU_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VL_MAXINT 2147483647
#define VL_MAXFLOAT 3.4028e37f
#define VL_DUP_FLAG (1 << 30)

#define VL_OK 0
#define VL_ERR_ARG (-1)      /* bad shape / null pointer / unsupported size */
#define VL_ERR_HIP (-2)      /* a HIP runtime call failed */
#define VL_ERR_WORKSPACE (-3) /* workspace too small */
#define VL_ERR_STATE (-4)     /* device-side loop state is inconsistent (a workspace used by two calls at once) */

const char *vl_last_error(void);
int vl_version(void);

/* ---- distances -------------------------------------------------------- */

/* The reference has one metric, the cosine distance of unit rows
 * clamp((1 - <a, b>) / 2, 0, 1) (kernels.py:85-114).  VL_METRIC_L2 is an
 * addition: the squared Euclidean distance sum_j (a_j - b_j)^2, not clamped,
 * accumulated in the same order (for unit rows it equals 4 x the cosine
 * distance up to rounding, so both order neighbours alike). */
#define VL_METRIC_COSINE 0
#define VL_METRIC_L2 1

/* out[r, j] = clamp((1 - <queries[r], vectors[ids[r, j]]>) / 2, 0, 1);
 * VL_MAXFLOAT where ids[r, j] is VL_MAXINT or outside [0, n_vectors).
 * With queries == vectors and ids == beams this is calculate_distances
 * (kernels.py:174-201, kernel 130-171); with circulant seed ids it is the
 * seed-distance step of initial_search_queue (ann.py:228-229). */
int vl_gather_distances(const float *queries, int64_t n_rows,
                        const float *vectors, int64_t n_vectors, int64_t dim,
                        const int32_t *ids, int64_t width,
                        float *out, void *stream);

/* vl_gather_distances with the metric chosen by the caller (VL_METRIC_*). */
int vl_gather_distances_metric(const float *queries, int64_t n_rows,
                               const float *vectors, int64_t n_vectors, int64_t dim,
                               const int32_t *ids, int64_t width, int metric,
                               float *out, void *stream);

/* search_from_seeds (kernels.py:260-311, kernel 204-257): for row b, visit
 * slot s, neighbour slot k: nb = beams[visit[b,s], k];
 * idx_out[b, s*width+k] = nb, dist_out[...] = d(vectors[nb], queries[b]).
 * A VL_MAXINT visit id or neighbour id yields (VL_MAXINT, VL_MAXFLOAT). */
int vl_search_from_seeds(const float *queries, int64_t n_rows, int64_t dim,
                         const int32_t *visit, int64_t n_visit,
                         const int32_t *beams, int64_t n_nodes, int64_t width,
                         const float *vectors, int64_t n_vectors,
                         int32_t *idx_out, float *dist_out, void *stream);

/* vl_search_from_seeds with the metric chosen by the caller (VL_METRIC_*). */
int vl_search_from_seeds_metric(const float *queries, int64_t n_rows, int64_t dim,
                                const int32_t *visit, int64_t n_visit,
                                const int32_t *beams, int64_t n_nodes, int64_t width,
                                const float *vectors, int64_t n_vectors, int metric,
                                int32_t *idx_out, float *dist_out, void *stream);

/* ---- seed graphs ------------------------------------------------------ */

/* generate_circulant_beams / generate_queue_circulants (utils.py:26-41):
 * out[r, k] = sort_k(row0 + r + primes[k]) % modulus. primes: device int32. */
int vl_circulants(int32_t *out, int64_t rows, int64_t row0, int64_t modulus,
                  const int32_t *primes, int64_t n_primes, void *stream);

/* ---- dedup / exclusion / gather helpers ------------------------------- */

/* dedup_tensor_ (kernels.py:370-380): per row, a slot whose id equals its
 * left neighbour's (bit 30 ignored) becomes VL_MAXINT.  In place. */
int vl_dedup_ids(int32_t *ids, int64_t rows, int64_t cols, void *stream);

/* dedup_tensor_pair_ (kernels.py:383-397): same, and the distance of a
 * punched slot becomes VL_MAXFLOAT.  In place. */
int vl_dedup_pairs(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream);

/* punchout_excluded_ (kernels.py:491-501): slots whose id occurs in
 * excl[r, 0:e) before that row's first VL_MAXINT become the empty pair.
 * ids/dists may be strided views (queue.py:47-53 passes the queue tail). */
int vl_punchout_excluded(int32_t *ids, float *dists, int64_t rows, int64_t cols,
                         int64_t ids_stride, int64_t dists_stride,
                         const int32_t *excl, int64_t excl_cols, int64_t excl_stride,
                         void *stream);

/* index_by_tensor (kernels.py:554-559) for 4-byte elements:
 * out[r, c] = a[r, index[r, c]], index is int64 as torch.sort returns it. */
int vl_index_by_tensor(const void *a, const int64_t *index, void *out,
                       int64_t rows, int64_t cols, void *stream);

/* ---- sorted queues (vectorlink_gpu/queue.py) -------------------------- */

/* index_sort (utils.py:44-53): order each row by (distance asc, id asc). */
int vl_index_sort(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream);

/* punchout_duplicates_ (kernels.py:400-406): dedup_pairs, then order by
 * distance keeping the previous order on ties.  In place. */
int vl_punchout_duplicates(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream);

/* queue_sort (queue.py:15-18) = index_sort then punchout_duplicates_. */
int vl_queue_sort(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream);

/* Queue.insert (queue.py:37-61): copy m candidates per row into slots
 * [length, length+m), punch those that occur in the exclusion row (may be
 * NULL), queue_sort the whole row of `capacity` slots.  When changed is not
 * NULL it receives, as bytes, indices[:, :length] != the ids before. */
int vl_queue_insert(int32_t *q_ids, float *q_dists, int64_t rows, int64_t capacity,
                    int64_t length, const int32_t *cand_ids, const float *cand_dists,
                    int64_t m, const int32_t *excl, int64_t excl_cols,
                    uint8_t *changed, void *stream);

/* Queue.pop_n_ids (queue.py:87-95): out[r, 0:take) = ids[r, 0:take); those
 * slots become the empty pair; nothing is re-sorted. */
int vl_queue_pop(int32_t *q_ids, float *q_dists, int64_t rows, int64_t capacity,
                 int64_t take, int32_t *out, void *stream);

/* add_new_to_seen_ (utils.py:61-82): append visit[:, 0:n) at the first
 * column that is empty in every row, then sort + dedup + sort each row.
 * host_status receives 1 (updated) or 0 (no free column: the reference
 * returns None and seen is left as it was).  Synchronises the stream.
 * workspace: 8 bytes. */
int vl_seen_add(int32_t *seen, int64_t rows, int64_t cols,
                const int32_t *visit, int64_t n_visit,
                void *workspace, int *host_status, void *stream);

/* ---- beam search (ann.py:38-93 closest_vectors) ----------------------- */

typedef struct vl_beam_params {
    int64_t n_rows;               /* queries in this batch */
    int64_t dim;
    int64_t n_vectors;
    int64_t width;                /* columns of the neighbour table passed in */
    int64_t queue_capacity;       /* search queue row size */
    int64_t queue_length;         /* search queue .length */
    int64_t beam_size;            /* config["beam_size"] */
    int64_t parallel_visit_count;
    int64_t visit_queue_factor;
    int64_t exclude_factor;
    int64_t speculative_readahead;
    int64_t excl_cols;            /* columns of the exclusion tensor, 0 if none */
    int64_t flags;                /* 0 = default; VL_BEAM_* bits select another form of the same loop */
    int64_t metric;               /* VL_METRIC_COSINE (the reference's) or VL_METRIC_L2 */
} vl_beam_params;

/* Forms of one iteration, all with the same result on [:, :queue_length] for a
 * search queue in the state vl_queue_insert leaves it - rows ordered by
 * (distance, id) with distinct ids - whose distances are the distances of its
 * ids to this call's query rows (an id carries one distance wherever it
 * occurs).  Only SORT_MERGE treats a queue in any other state as the
 * reference does; the other forms are not checked against such input.
 * default        one fused launch (expand + merge phases of a row in one workgroup);
 * TWO_LAUNCHES   expand kernel, then merge kernel;
 * SORT_MERGE     two launches, the merge step sorts whole queue rows (exact for
 *                queue rows in any state, not only in Queue.insert order). */
#define VL_BEAM_TWO_LAUNCHES 1
#define VL_BEAM_SORT_MERGE 2
/* A different loop, not the reference's: PER_QUERY_STOP ends every row on its
 * own.  The reference tests for progress over the whole batch (ann.py:90-91),
 * so every row keeps expanding until the slowest one is quiet.  With this bit a
 * row is finished after speculative_readahead iterations in a row that left
 * the first queue_length ids of its search queue unchanged (or when the visited
 * list has no free column), later iterations skip it, and the loop ends at the
 * first progress check that finds every row finished.  Results differ from the
 * reference's loop (fewer expansions per row); they are defined by, and tested
 * against, the CPU model closest_vectors_per_query of the test oracle.  Fused
 * step only. */
#define VL_BEAM_PER_QUERY_STOP 4
/* Same loop, same result, without the per-row cache of already evaluated
 * (id, distance) pairs: the workspace shrinks by the cache's table and every
 * candidate distance is evaluated when it is asked for. */
#define VL_BEAM_NO_CACHE 8
/* The call brings the 8-bit sketch of the vector table
 * (vl_closest_vectors_with_sketch): the workspace then also holds the call's
 * query rows rounded for it (32 bytes per 16 columns and row). */
#define VL_BEAM_USES_SKETCH 16
/* Same loop, same result, several iterations per launch: the fused step takes
 * a row through the speculative_readahead iterations between two progress
 * checks in ONE launch, with the row's queues and visited list resident in LDS
 * and a small LDS table of the (id, distance) pairs met in them, for as long as
 * no visited list can fill up within them (parallel_visit_count * iteration <=
 * exclude_factor * visit queue length); the stretch after that runs one
 * iteration per launch.  Off by default (it measures slower on an MI355X: the
 * longer kernel runs with fewer wavefronts per SIMD). */
#define VL_BEAM_WINDOWS 32

int64_t vl_beam_workspace_bytes(const vl_beam_params *p);

/* Runs the whole loop of closest_vectors on the search queue in place and
 * returns the number of iterations (a multiple of speculative_readahead) or
 * a negative error.  Synchronises the stream every speculative_readahead
 * iterations to read the batch-wide "any row changed" flag, as the
 * reference does (ann.py:90-91).  Rows of the search queue are exact on
 * [:, :queue_length]; slots beyond are unspecified. */
int64_t vl_closest_vectors(const vl_beam_params *p,
                           const float *queries, const float *vectors,
                           const int32_t *beams,
                           int32_t *q_ids, float *q_dists,
                           const int32_t *exclude,
                           void *workspace, int64_t workspace_bytes,
                           void *stream);

/* ---- 8-bit sketch of the vector table (no counterpart in the reference) --
 *
 * The reference evaluates every candidate distance of an iteration in full
 * (cuda_search_from_seeds_kernel, kernels.py:204-257) although a row keeps a
 * handful of its hundreds of candidates.  The sketch holds every vector rounded
 * to 8 bits per element with one scale per vector (dim int8 values round(v / scale),
 * scale = max |v| / 127, padded with zeros to a multiple of 16) and an 8-byte
 * tail: float scale, then as halves, rounded up, a bound on the 2-norm of what
 * the rounding moved and a bound on the vector's 2-norm.  The table is ONE block:
 * the n_vectors data rows first (16 * ceil(dim / 16) bytes each), then the
 * n_vectors tails - a part of it is not the sketch of a part of the vectors.
 * With it a dot product is known to within
 * ||q|| x that bound (Cauchy-Schwarz) from a quarter of the bytes, by integer
 * arithmetic (the query row is rounded to 15 bits, which the bound accounts for).  vl_closest_vectors_with_sketch uses those bounds ONLY to decide
 * which candidate rows to fetch: a candidate whose lower bound is above the last
 * slot of the search queue and, when it is unvisited, above the last live slot
 * of the visit queue and above the parallel_visit_count-th smallest upper bound
 * beyond it, cannot enter either queue and is dropped; every other candidate is
 * evaluated exactly.  Queues are bit-identical to vl_closest_vectors'. */

/* Bytes per vector in the sketch of vectors of `dim` columns:
 * 16 * ceil(dim / 16) + 8. */
int64_t vl_sketch_row_bytes(int64_t dim);

/* Fills table (n_vectors * vl_sketch_row_bytes(dim) bytes, 16-byte aligned; on a
 * 128-byte boundary its rows cost least) from vectors[n_vectors, dim].  A row holding a NaN or an infinity gets an infinite
 * bound: its candidates are always evaluated exactly. */
int vl_sketch_build(const float *vectors, int64_t n_vectors, int64_t dim,
                    uint8_t *table, void *stream);

/* Bounds of gathered cosine distances from the sketch: for every id
 * lo[r, j] <= d(queries[r], vectors[ids[r, j]]) <= hi[r, j], where d is the very
 * float32 value vl_gather_distances returns (VL_MAXFLOAT twice for an empty or
 * out-of-range id).  The code that the beam-search step runs on its
 * candidates, exposed so that the bound can be checked on its own.  workspace:
 * vl_sketch_bounds_workspace_bytes(n_rows, dim) bytes, 16-byte aligned (the
 * query rows rounded to 15 bits).  dim: a multiple of 4, at most 2048. */
int64_t vl_sketch_bounds_workspace_bytes(int64_t n_rows, int64_t dim);
int vl_sketch_bounds(const float *queries, int64_t n_rows, int64_t dim,
                     const uint8_t *table, int64_t n_vectors,
                     const int32_t *ids, int64_t m, float *lo, float *hi,
                     void *workspace, int64_t workspace_bytes, void *stream);

/* vl_closest_vectors with the sketch of `vectors` (NULL: exactly
 * vl_closest_vectors).  Same arguments, same result, same return value.  The
 * sketch serves the fused step under the cosine metric for 16-byte aligned rows
 * of up to 2048 columns; other calls ignore it.  The distance cache then also
 * remembers candidates that were only bounded, so a repeat costs neither a
 * sketch row nor a vector row.  A row whose bounded candidates mostly need
 * their exact distance after all gives the sketch up for the rest of the call.
 * p->flags must hold VL_BEAM_USES_SKETCH, also in the vl_beam_workspace_bytes
 * call that sized the workspace. */
int64_t vl_closest_vectors_with_sketch(const vl_beam_params *p,
                                       const float *queries, const float *vectors,
                                       const uint8_t *sketch,
                                       const int32_t *beams,
                                       int32_t *q_ids, float *q_dists,
                                       const int32_t *exclude,
                                       void *workspace, int64_t workspace_bytes,
                                       void *stream);

/* vl_closest_vectors for callers that cannot allocate or wait: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  Differences from vl_closest_vectors:
 *  - no workspace argument: the loop's scratch memory (control block, visit
 *    queues, visited lists; the fused step only, without the per-row distance
 *    cache) is a static device array of VL_NOALLOC_SCRATCH_BYTES inside the
 *    library, which every GPU the library runs on holds until the process
 *    ends.  A batch that needs more (about 8 * visit queue length + 4 * visited
 *    list length bytes per row) is refused with VL_ERR_ARG; nothing is
 *    allocated or freed, here or in anything this call uses;
 *  - no host round trips: exactly `iterations` launches are enqueued and the
 *    call returns 0 at once.  When a progress check finds the batch quiet the
 *    remaining launches do nothing, so with iterations >= the count
 *    vl_closest_vectors would return the queues end up bit-identical to its;
 *  - status_out (device, 2 x int32) receives [0] = 1 if the loop ended within
 *    `iterations` (else 0: the queues hold an unfinished search; -1: a row found
 *    more ids in its visited list than the iterations run can have put there,
 *    i.e. the array was written by another call meanwhile - the rows stop and
 *    the queues are not to be used) and [1] = the number of iterations that ran.
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU
 * (two streams, two threads) race; serialise them.  (vl_closest_vectors reports
 * the same condition, a workspace shared by two calls in flight, as
 * VL_ERR_STATE.) */
#define VL_NOALLOC_SCRATCH_BYTES (32 << 20)
int vl_closest_vectors_noalloc(const vl_beam_params *p,
                               const float *queries, const float *vectors,
                               const int32_t *beams,
                               int32_t *q_ids, float *q_dists,
                               const int32_t *exclude,
                               int64_t iterations, int32_t *status_out,
                               void *stream);

/* Per-kernel timing of vl_closest_vectors (no counterpart in the reference,
 * whose log.py:7-17 times whole calls): with enable != 0 every expand / merge
 * launch is bracketed by HIP events on the caller's stream.  out (9 doubles,
 * may be NULL) receives the sums since the last reset: expand ms, merge ms,
 * expand launches, merge launches, candidate rows fetched, query rows,
 * iterations, candidate distances asked for (fetched + served by the per-row
 * cache of already evaluated pairs), candidate rows looked at through the
 * sketch.  The sums are kept under a mutex, so
 * profiled calls from several host threads add up without tearing. */
int vl_beam_profile(int enable, int reset, double *out);

/* Beam-search step launches (one iteration, or one window of iterations, of one
 * batch each) enqueued by this process since the library was loaded, whatever
 * the profiling switch says; lets a caller cut a profiler's dispatch list into
 * the phases of its own run.  No counterpart in the reference. */
int64_t vl_beam_launches(void);

/* ---- pruning (kernels.py:441-468 prune_) ------------------------------ */

/* For every x and slot j: y = beams[x,j], z = beams[y,0]; if z occurs in row
 * x at (last) slot i and d[x,i] > d[x,j] and d[x,i] > d[y,0], slot (x,i)
 * becomes the empty pair; then each row is ordered by distance.  Every
 * decision reads the tables as passed in (the reference mutates in place
 * while other blocks read); results go to the *_out tables. */
int vl_prune(const int32_t *beams, const float *dists, int64_t n, int64_t width,
             int32_t *beams_out, float *dists_out, void *stream);

/* ---- rank-based graph optimisation ------------------------------------- */
/* Detour-count re-ordering of every neighbour row and reverse-edge merge (the
 * CAGRA optimisation).  No counterpart in the reference: its prune is vl_prune
 * above and its reverse-edge collector is commented out (kernels.py:503-550).
 * beams [n, width] holds rows ordered best first with distinct ids, VL_MAXINT
 * for empty slots.  For the edge x->y at slot j a detour is a slot i < j of
 * row x whose node lists y at a slot k < j; slots are re-ordered by (detours,
 * slot) and cut to `degree`.  Then node y collects the sources x of edges
 * x->y found in the first degree/2 slots of the cut rows, ordered by (slot,
 * x), at most degree - degree/2 of them, and the final row of x is its first
 * degree/2 edges, then its reverse edges not yet in the row (never x), then
 * its remaining edges, cut to `degree`, padded with VL_MAXINT.
 * out [n, degree] holds ids only; distances come from vl_gather_distances. */
int64_t vl_optimize_graph_workspace_bytes(int64_t n, int64_t width, int64_t degree);
int vl_optimize_graph(const int32_t *beams, int64_t n, int64_t width, int64_t degree,
                      int32_t *out, void *workspace, int64_t workspace_bytes, void *stream);

/* ---- exact k nearest neighbours on dense fp32 MFMA tiles -------------- */
/* No counterpart in the reference (its recall is self-recall@1 only,
 * ann.py:235-259); used for ground truth recall@k.  ids_out/dists_out are
 * [n_queries, k], ordered by (distance, id).  k <= 16, dim % 4 == 0,
 * pointers 16-byte aligned.  Distances come from MFMA accumulation, so they
 * agree with the gathered-distance kernels to ~1e-7, not bit for bit. */
int64_t vl_knn_workspace_bytes(int64_t n_queries, int64_t n_vectors, int64_t dim, int64_t k);
int vl_knn_exact(const float *queries, int64_t n_queries,
                 const float *vectors, int64_t n_vectors, int64_t dim, int64_t k,
                 int32_t *ids_out, float *dists_out,
                 void *workspace, int64_t workspace_bytes, void *stream);
/* The same under a metric (VL_METRIC_*).  L2 distances are formed as
 * |q|^2 + |v|^2 - 2 q.v from the tiles' dot products and clamped at 0: a
 * distance much smaller than the squared lengths carries their rounding
 * (about 1e-7 of |q|^2 + |v|^2), so near-ties may order differently from the
 * gathered-distance kernels, which subtract first.  The workspace of
 * vl_knn_workspace_bytes serves both metrics. */
int vl_knn_exact_metric(const float *queries, int64_t n_queries,
                        const float *vectors, int64_t n_vectors, int64_t dim, int64_t k,
                        int32_t metric, int32_t *ids_out, float *dists_out,
                        void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* VLGPU_H */
