// Gathered cosine distances for gfx950: the replacement of the reference's
// cuda_distances_kernel (vectorlink_gpu/kernels.py:130-171) and
// cuda_search_from_seeds_kernel (kernels.py:204-257).
//
// The reference launches one thread block per scalar distance.  Here one
// wavefront owns up to 64 candidate ids (one per lane), keeps the query row in
// registers, and streams the candidate rows with 16-byte loads, several rows in
// flight at a time; sentinel candidates are compacted away with a ballot before
// any row is fetched.  HBM traffic is the candidate rows: 4*dim bytes each.
//
// Summation order of one dot product (fixed so that every entry point and the
// CPU oracle produce the same bits): the row is cut into chunks of 4 floats,
// chunk c belongs to partial sum c mod 64, a partial sum takes its elements in
// index order with one fused multiply-add each, and the 64 partial sums are
// folded pairwise at lane distances 32, 16, 8, 4, 2, 1.  Short rows are
// handled by groups of LPR = 16 or 32 lanes, several rows per wavefront: a lane
// then holds the partial sums lig, lig + LPR, ... of its row and folds them
// itself (distances 32 and 16) before the cross-lane folds; partial sums no
// chunk reaches are zeros, so the result is the same.
#include "vl_common.h"
#include "beam_ctrl.h"
#include "dist_device.h"

namespace {

struct ExpandArgs {
    const float *queries;
    const float *vectors;
    const int32_t *ids;    // direct mode: [n_rows, m] candidate ids
    const int32_t *visit;  // visit mode: [n_rows, n_visit] node ids (else null)
    const int32_t *beams;  // visit mode: [n_nodes, width]
    int32_t *idx_out;      // may be null in direct mode
    float *dist_out;
    BeamCtrl *ctrl;        // beam-search loop only (else null): batch-wide loop state
    int iter;              //   iteration number, from 1
    int readahead;         //   speculative_readahead
    int seen_cols;         //   columns of the visited list
    int visit_stride;      // row stride of `visit` in elements
    int count_evals;       //   profiling: add the number of fetched rows to ctrl->evals
    uint64_t *memo;        // optional per-row cache of (id, distance) pairs already evaluated (else null)
    int memo_shift;        //   32 - log2(slots per row)
    int64_t n_rows;
    int64_t n_vectors;
    int64_t n_nodes;
    int dim;
    int nchunks;
    int n_visit;
    int width;
    int m;     // candidates per row
    int cw;    // candidates per wavefront (<= 64)
    int parts; // workgroups per row
    int l2;    // 0: cosine distance (the reference's), 1: squared L2
};

// blockIdx -> (row, part) so that all workgroups of one row, and the same rows
// from one launch to the next, land on the same XCD (workgroups are dealt to
// the 8 XCDs round-robin): the query row and neighbour-table rows then hit
// that XCD's L2.
__device__ __forceinline__ bool map_block(const ExpandArgs &a, int64_t &row, int &part) {
    int64_t bid = blockIdx.x;
    int xcd = (int)(bid & 7);
    int64_t j = bid >> 3;
    row = (j / a.parts) * 8 + xcd;
    part = (int)(j % a.parts);
    return row < a.n_rows;
}

template <int CPL, int LPR, int U, bool GENERIC>
__global__ __launch_bounds__(256) void expand_kernel(ExpandArgs a) {
    int gate = 0;
    if (a.ctrl) {
        gate = beam_gate(a.ctrl, a.iter, a.readahead, a.seen_cols, blockIdx.x == 0 && threadIdx.x == 0);
        if (gate == 2) return;
    }
    int64_t row;
    int part;
    if (!map_block(a, row, part)) return;
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    const int c0 = (part * 4 + wave) * a.cw;
    if (c0 >= a.m) return;
    const int n = min(a.cw, a.m - c0);
    const bool has = lane < n;
    const int slot = c0 + lane;

    int32_t id = VL_MAXINT;
    if (has) {
        if (a.visit) {
            int s = slot / a.width, k = slot - s * a.width;
            int32_t node = gate ? VL_MAXINT : a.visit[row * a.visit_stride + s];
            if (node != VL_MAXINT && (uint32_t)node < (uint64_t)a.n_nodes)
                id = a.beams[(int64_t)node * a.width + k];
        } else {
            id = a.ids[row * a.m + slot];
        }
    }
    bool ok = has && id != VL_MAXINT && id >= 0 && (int64_t)id < a.n_vectors;
    float *out_d = a.dist_out + row * a.m + c0;
    if (has) {
        if (a.idx_out) a.idx_out[row * a.m + slot] = ok ? id : VL_MAXINT;
        if (!ok) out_d[lane] = VL_MAXFLOAT;
    }
    if (a.count_evals) {
        uint64_t wm = __ballot(ok);
        if (lane == 0 && wm) atomicAdd(&a.ctrl->wanted[blockIdx.x & (kBeamStripes - 1)], (unsigned long long)__popcll(wm));
    }
    // A distance evaluated earlier in this search for the same (row, id) is
    // reused: the cached bits are the ones this kernel would produce again.
    uint64_t *memo_row = nullptr;
    if (a.memo) {
        memo_row = a.memo + ((uint64_t)row << (32 - a.memo_shift));
        if (ok) {
            uint64_t e = memo_load(memo_row, a.memo_shift, id);
            if ((int32_t)(uint32_t)e == id) {
                out_d[lane] = __builtin_bit_cast(float, (uint32_t)(e >> 32));
                ok = false;
            }
        }
    }
    if (a.count_evals) {
        uint64_t okm = __ballot(ok);
        if (lane == 0 && okm) atomicAdd(&a.ctrl->evals[blockIdx.x & (kBeamStripes - 1)], (unsigned long long)__popcll(okm));
    }
    const float *q_row = a.queries + row * a.dim;
    if constexpr (GENERIC)
        wave_distances_generic(q_row, a.vectors, a.dim, a.nchunks, id, ok, out_d, memo_row, a.memo_shift, a.l2 != 0);
    else
        wave_distances<CPL, LPR, U>(q_row, a.vectors, a.dim, a.nchunks, id, ok, out_d, memo_row, a.memo_shift, a.l2 != 0);
}

template <int CPL, int LPR, int U>
void launch_fast(const ExpandArgs &a, dim3 grid, hipStream_t st) {
    hipLaunchKernelGGL((expand_kernel<CPL, LPR, U, false>), grid, dim3(256), 0, st, a);
}

// one launch: c.n_rows * c.parts workgroups, rounded up to whole groups of 8 rows
void launch_expand_piece(const ExpandArgs &a, bool aligned, hipStream_t st) {
    const int nchunks = a.nchunks;
    dim3 grid((unsigned)((a.n_rows + 7) / 8 * 8 * a.parts));
    if (!aligned || nchunks > 512) {
        hipLaunchKernelGGL((expand_kernel<1, 64, 1, true>), grid, dim3(256), 0, st, a);
    } else if (nchunks <= 16) launch_fast<1, 16, 8>(a, grid, st);
    else if (nchunks <= 32) launch_fast<2, 16, 4>(a, grid, st);
    else if (nchunks <= 64) launch_fast<1, 64, 8>(a, grid, st);
    else if (nchunks <= 96) launch_fast<3, 32, 4>(a, grid, st);
    else if (nchunks <= 128) launch_fast<2, 64, 8>(a, grid, st);
    else if (nchunks <= 192) launch_fast<3, 64, 4>(a, grid, st);
    else if (nchunks <= 256) launch_fast<4, 64, 4>(a, grid, st);
    else if (nchunks <= 320) launch_fast<5, 64, 2>(a, grid, st);
    else if (nchunks <= 384) launch_fast<6, 64, 2>(a, grid, st);
    else if (nchunks <= 448) launch_fast<7, 64, 2>(a, grid, st);
    else launch_fast<8, 64, 2>(a, grid, st);
}

}  // namespace

// Host-side launcher shared by the C entry points and the beam-search loop.
int vl_launch_expand(const float *queries, int64_t n_rows, const float *vectors, int64_t n_vectors,
                     int64_t dim, const int32_t *ids, const int32_t *visit, int64_t n_visit,
                     const int32_t *beams, int64_t n_nodes, int64_t width, int64_t m,
                     int32_t *idx_out, float *dist_out, BeamCtrl *ctrl, int iter, int readahead,
                     int seen_cols, int64_t visit_stride, int count_evals, uint64_t *memo, int memo_slots,
                     int metric, hipStream_t st) {
    if (n_rows == 0 || m == 0) return VL_OK;
    VL_REQUIRE(metric == VL_METRIC_COSINE || metric == VL_METRIC_L2, "unknown metric %d", metric);
    VL_REQUIRE(dim >= 1 && dim <= (1 << 24), "dim %lld out of range", (long long)dim);
    VL_REQUIRE(m <= (1 << 24), "row of %lld candidates is too wide", (long long)m);
    ExpandArgs a;
    a.queries = queries; a.vectors = vectors; a.ids = ids; a.visit = visit; a.beams = beams;
    a.idx_out = idx_out; a.dist_out = dist_out;
    a.ctrl = ctrl; a.iter = iter; a.readahead = readahead; a.seen_cols = seen_cols;
    a.visit_stride = (int)visit_stride;
    a.l2 = metric == VL_METRIC_L2;
    a.count_evals = ctrl ? count_evals : 0;
    a.memo = memo_slots > 0 ? memo : nullptr;
    a.memo_shift = 32;
    if (a.memo) {
        int lg = 0;
        while ((1 << lg) < memo_slots) ++lg;
        VL_REQUIRE((1 << lg) == memo_slots && lg >= 4 && lg <= 24, "memo slots must be a power of two, 16 or more");
        a.memo_shift = 32 - lg;
    }
    a.n_rows = n_rows; a.n_vectors = n_vectors; a.n_nodes = n_nodes;
    a.dim = (int)dim; a.nchunks = (int)((dim + 3) / 4);
    a.n_visit = (int)n_visit; a.width = (int)width; a.m = (int)m;

    const bool aligned = (dim % 4 == 0) && (((uintptr_t)queries | (uintptr_t)vectors) % 16 == 0);
    const int nchunks = a.nchunks;
    // candidates per wavefront: enough to amortise the query load, few enough
    // that one row's candidates spread over several wavefronts
    a.cw = nchunks <= 64 ? 64 : 32;
    if (m < a.cw * 4) a.cw = (int)((m + 3) / 4 < 8 ? 8 : (m + 3) / 4);
    if (a.cw > 64) a.cw = 64;
    a.parts = (int)((m + 4 * a.cw - 1) / (4 * a.cw));
    // rows per launch: a multiple of 8 (the XCD mapping) whose workgroups stay below kMaxBlocks
    const int64_t rows_per_launch = (kMaxBlocks / a.parts) & ~7ll;
    VL_REQUIRE(rows_per_launch >= 8, "row of %lld candidates is too wide", (long long)m);
    VL_REQUIRE(ctrl == nullptr || n_rows <= rows_per_launch, "a beam-search batch of %lld rows is too large (limit %lld)",
               (long long)n_rows, (long long)rows_per_launch);
    const int64_t memo_row_slots = a.memo ? (1ll << (32 - a.memo_shift)) : 0;
    for (int64_t r0 = 0; r0 < n_rows; r0 += rows_per_launch) {
        ExpandArgs c = a;
        c.n_rows = (n_rows - r0 < rows_per_launch) ? n_rows - r0 : rows_per_launch;
        c.queries = queries + r0 * dim;
        if (ids) c.ids = ids + r0 * m;
        if (visit) c.visit = visit + r0 * visit_stride;
        if (idx_out) c.idx_out = idx_out + r0 * m;
        c.dist_out = dist_out + r0 * m;
        if (c.memo) c.memo = a.memo + r0 * memo_row_slots;
        launch_expand_piece(c, aligned, st);
    }
    VL_LAUNCH_CHECK("expand_kernel");
    return VL_OK;
}

VL_EXPORT int vl_gather_distances_metric(const float *queries, int64_t n_rows, const float *vectors,
                                         int64_t n_vectors, int64_t dim, const int32_t *ids,
                                         int64_t width, int metric, float *out, void *stream) {
    VL_REQUIRE(n_rows >= 0 && width >= 0 && n_vectors >= 0, "negative size");
    if (n_rows == 0 || width == 0) return VL_OK;
    VL_REQUIRE(queries && vectors && ids && out, "null pointer");
    return vl_launch_expand(queries, n_rows, vectors, n_vectors, dim, ids, nullptr, 0, nullptr, 0,
                            width, width, nullptr, out, nullptr, 0, 1, 0, 0, 0, nullptr, 0, metric, (hipStream_t)stream);
}

VL_EXPORT int vl_gather_distances(const float *queries, int64_t n_rows, const float *vectors,
                                  int64_t n_vectors, int64_t dim, const int32_t *ids,
                                  int64_t width, float *out, void *stream) {
    return vl_gather_distances_metric(queries, n_rows, vectors, n_vectors, dim, ids, width, VL_METRIC_COSINE, out, stream);
}

VL_EXPORT int vl_search_from_seeds_metric(const float *queries, int64_t n_rows, int64_t dim,
                                          const int32_t *visit, int64_t n_visit, const int32_t *beams,
                                          int64_t n_nodes, int64_t width, const float *vectors,
                                          int64_t n_vectors, int metric, int32_t *idx_out, float *dist_out,
                                          void *stream) {
    VL_REQUIRE(n_rows >= 0 && n_visit >= 0 && width >= 0, "negative size");
    if (n_rows == 0 || n_visit == 0 || width == 0) return VL_OK;
    VL_REQUIRE(queries && visit && beams && vectors && idx_out && dist_out, "null pointer");
    return vl_launch_expand(queries, n_rows, vectors, n_vectors, dim, nullptr, visit, n_visit, beams,
                            n_nodes, width, n_visit * width, idx_out, dist_out, nullptr, 0, 1, 0, n_visit, 0, nullptr, 0,
                            metric, (hipStream_t)stream);
}

VL_EXPORT int vl_search_from_seeds(const float *queries, int64_t n_rows, int64_t dim,
                                   const int32_t *visit, int64_t n_visit, const int32_t *beams,
                                   int64_t n_nodes, int64_t width, const float *vectors,
                                   int64_t n_vectors, int32_t *idx_out, float *dist_out,
                                   void *stream) {
    return vl_search_from_seeds_metric(queries, n_rows, dim, visit, n_visit, beams, n_nodes, width, vectors, n_vectors,
                                       VL_METRIC_COSINE, idx_out, dist_out, stream);
}
