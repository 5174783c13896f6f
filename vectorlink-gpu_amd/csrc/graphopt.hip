// Rank-based graph optimisation for gfx950: detour-count re-ordering of every
// neighbour row and reverse-edge merge (the CAGRA graph optimisation).  The
// reference has neither: its only pruning is prune_ (kernels.py:409-468) and
// its reverse-edge collector is commented out (kernels.py:503-550, an O(N^2)
// scan).  The exact rule is the one stated in the CPU oracle (orc_rank_prune,
// orc_reverse_merge); this file must produce the same ids.
//
//  rank_prune_kernel     one workgroup per row x: for every 2-hop x -> z -> y
//                        with both hops ranked better than the direct slot of
//                        y in row x, count a detour for that slot; re-order by
//                        (detours, slot), keep `degree`.  W rows of W ids are
//                        read per row (W^2 * 4 bytes, rows gathered).
//  reverse edges         the edges x -> y of the first rev_from slots of every
//                        pruned row, grouped by target: a histogram of the
//                        targets, an exclusive scan of it (three small
//                        kernels), and a scatter of (slot, x) keys into the
//                        targets' segments, in whatever order the atomics hand
//                        out the places of a segment.
//  reverse_merge_kernel  one workgroup per row y: only the first `cap` sources of
//                        y in (slot, x) order are needed, and they are selected
//                        from the segment here (chunks of it sorted in LDS
//                        together with the best so far), so the result does not
//                        depend on the segment's order; then keep | reverse |
//                        rest, without duplicates, cut to `degree`.
#include "rowsort.h"

#include <cstring>

namespace {


__global__ __launch_bounds__(kQueueThreads) void rank_prune_kernel(const int32_t *__restrict__ beams, int64_t n, int W,
                                                                  int P, int degree, int32_t *__restrict__ out,
                                                                  int64_t row0) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);       // (id, slot) ordered by id, later (count, slot)
    int32_t *ids = reinterpret_cast<int32_t *>(keys + P);       // row x
    int32_t *count = ids + W;
    const int64_t x = row0 + blockIdx.x;
    for (int j = threadIdx.x; j < W; j += blockDim.x) {
        ids[j] = beams[x * W + j];
        count[j] = 0;
    }
    __syncthreads();
    for (int j = threadIdx.x; j < P; j += blockDim.x)
        keys[j] = (j < W && ids[j] != VL_MAXINT) ? (((uint64_t)(uint32_t)ids[j] << 32) | (uint32_t)j) : kPadKey;
    block_bitonic_sort(keys, P);
    // every (i, k): z = row[i], y = beams[z, k]; if y sits at slot j of row x with j > i and j > k, z is a detour for j
    const int64_t pairs = (int64_t)W * W;
    for (int64_t t = threadIdx.x; t < pairs; t += blockDim.x) {
        int i = (int)(t / W), k = (int)(t - (int64_t)i * W);
        int32_t z = ids[i];
        if (z == VL_MAXINT || z < 0 || z >= n) continue;
        int32_t y = beams[(int64_t)z * W + k];
        if (y == VL_MAXINT) continue;
        uint64_t want = (uint64_t)(uint32_t)y << 32;
        int lo = 0, hi = P;
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if (keys[mid] < want) lo = mid + 1;
            else hi = mid;
        }
        // a row may hold the same id twice; every slot of it counts, as in the oracle's scan over slots
        for (; lo < P && (keys[lo] >> 32) == (uint32_t)y; ++lo) {
            int j = (int)(uint32_t)keys[lo];
            if (j > i && j > k) atomicAdd(&count[j], 1);
        }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < P; j += blockDim.x)
        keys[j] = (j < W && ids[j] != VL_MAXINT) ? (((uint64_t)(uint32_t)count[j] << 32) | (uint32_t)j) : kPadKey;
    block_bitonic_sort(keys, P);
    for (int o = threadIdx.x; o < degree; o += blockDim.x) {
        uint64_t k = o < P ? keys[o] : kPadKey;
        out[x * degree + o] = (k == kPadKey) ? VL_MAXINT : ids[(uint32_t)k];
    }
}

// An edge of the reverse pass: slot k < rev_from of pruned row x, pointing at a real row y.
__device__ inline bool rev_edge(const int32_t *__restrict__ pruned, int64_t n, int degree, int rev_from, int64_t e,
                                int64_t *x, int *k, int32_t *y) {
    *x = e / rev_from;
    *k = (int)(e - *x * rev_from);
    *y = pruned[*x * degree + *k];
    return *y != VL_MAXINT && *y >= 0 && *y < n;
}

__global__ void rev_zero_kernel(int32_t *__restrict__ a, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) a[i] = 0;
}

// count[y] = edges that point at y
__global__ void rev_count_kernel(const int32_t *__restrict__ pruned, int64_t n, int degree, int rev_from,
                                 int32_t *__restrict__ count) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n * rev_from;
         e += (int64_t)gridDim.x * blockDim.x) {
        int64_t x;
        int k;
        int32_t y;
        if (rev_edge(pruned, n, degree, rev_from, e, &x, &k, &y)) atomicAdd(&count[y], 1);
    }
}

// Exclusive scan of m counts in three steps: every workgroup scans kScanItems of them and reports its total,
// one workgroup scans the totals, every workgroup adds the total of those before it.
constexpr int kScanThreads = 256, kScanPerThread = 8, kScanItems = kScanThreads * kScanPerThread;

__device__ inline int block_exclusive_scan(int mine, int *lds, int *total) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int incl = mine;
    for (int d = 1; d < kWave; d <<= 1) {
        int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) lds[wave] = incl;
    __syncthreads();
    int before = 0, all = 0;
    for (int w = 0; w < (int)(blockDim.x / kWave); ++w) {
        if (w < wave) before += lds[w];
        all += lds[w];
    }
    __syncthreads();
    *total = all;
    return before + incl - mine;
}

__global__ __launch_bounds__(kScanThreads) void scan_blocks_kernel(const int32_t *__restrict__ in, int64_t m,
                                                                  int32_t *__restrict__ out,
                                                                  int32_t *__restrict__ block_total) {
    __shared__ int lds[kScanThreads / kWave];
    const int64_t base = (int64_t)blockIdx.x * kScanItems + (int64_t)threadIdx.x * kScanPerThread;
    int v[kScanPerThread], sum = 0;
#pragma unroll
    for (int j = 0; j < kScanPerThread; ++j) {
        v[j] = base + j < m ? in[base + j] : 0;
        sum += v[j];
    }
    int total;
    int run = block_exclusive_scan(sum, lds, &total);
#pragma unroll
    for (int j = 0; j < kScanPerThread; ++j) {
        if (base + j < m) out[base + j] = run;
        run += v[j];
    }
    if (threadIdx.x == 0) block_total[blockIdx.x] = total;
}

__global__ __launch_bounds__(1024) void scan_totals_kernel(int32_t *__restrict__ block_total, int64_t blocks) {
    __shared__ int lds[1024 / kWave];
    int carry = 0;
    for (int64_t base = 0; base < blocks; base += 1024) {
        const int64_t i = base + threadIdx.x;
        const int v = i < blocks ? block_total[i] : 0;
        int total;
        const int ex = block_exclusive_scan(v, lds, &total);
        if (i < blocks) block_total[i] = carry + ex;
        carry += total;
    }
}

__global__ __launch_bounds__(kScanThreads) void scan_add_kernel(int32_t *__restrict__ out, int64_t m,
                                                               const int32_t *__restrict__ block_total) {
    const int add = block_total[blockIdx.x];
    const int64_t base = (int64_t)blockIdx.x * kScanItems + threadIdx.x;
    for (int j = 0; j < kScanPerThread; ++j) {
        const int64_t i = base + (int64_t)j * kScanThreads;
        if (i < m) out[i] += add;
    }
}

// keys[start[y] ...] receive the (slot << 32 | x) of the edges that point at y; count[y] runs down to 0 as the
// places of y's segment are handed out (from its end: the order inside a segment is whatever the atomics make it)
__global__ void rev_scatter_kernel(const int32_t *__restrict__ pruned, int64_t n, int degree, int rev_from,
                                   const int32_t *__restrict__ start, int32_t *__restrict__ count,
                                   uint64_t *__restrict__ keys) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n * rev_from;
         e += (int64_t)gridDim.x * blockDim.x) {
        int64_t x;
        int k;
        int32_t y;
        if (rev_edge(pruned, n, degree, rev_from, e, &x, &k, &y)) {
            const int place = atomicSub(&count[y], 1) - 1;
            keys[(int64_t)start[y] + place] = ((uint64_t)(uint32_t)k << 32) | (uint32_t)x;
        }
    }
}

constexpr int kRevChunk = 1024;  // keys of a segment sorted at a time, together with the best so far

__global__ __launch_bounds__(kQueueThreads) void reverse_merge_kernel(const int32_t *__restrict__ pruned, int64_t n,
                                                                     int degree, int keep, int cap, int best_slots,
                                                                     const uint64_t *__restrict__ rev_keys,
                                                                     const int32_t *__restrict__ start,
                                                                     int32_t *__restrict__ out, int64_t row0) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *best = reinterpret_cast<uint64_t *>(smem);            // [0, cap): the smallest (slot, x) so far
    int32_t *cand = reinterpret_cast<int32_t *>(best + best_slots);  // keep | reverse | rest
    uint8_t *ok = reinterpret_cast<uint8_t *>(cand + 2 * degree);
    __shared__ int wave_cnt[kQueueWaves];
    const int64_t x = row0 + blockIdx.x;
    const int64_t s = start[x];
    const int64_t seg = (int64_t)start[x + 1] - s;
    const int n_rev = (int)min((int64_t)cap, seg);
    // the first n_rev sources of x in (slot, source) order: chunk after chunk of the segment is sorted together
    // with the best of the chunks before it; what ends up in [0, n_rev) is the same whatever order the segment is in
    for (int64_t done = 0; done < seg; done += kRevChunk) {
        const int len = (int)min((int64_t)kRevChunk, seg - done);
        const int held = done == 0 ? 0 : cap;
        int P = 2;
        while (P < held + len) P <<= 1;
        for (int i = threadIdx.x; i < P; i += blockDim.x) {
            if (i >= held) best[i] = i - held < len ? rev_keys[s + done + (i - held)] : kPadKey;
        }
        block_bitonic_sort(best, P);
        if (seg > kRevChunk) {  // more chunks may follow: everything beyond the best `cap` is forgotten
            for (int i = cap + threadIdx.x; i < P; i += blockDim.x) best[i] = kPadKey;
            for (int i = P + threadIdx.x; i < cap; i += blockDim.x) best[i] = kPadKey;
            __syncthreads();
        }
    }
    const int total = keep + n_rev + (degree - keep);
    for (int p = threadIdx.x; p < total; p += blockDim.x) {
        int32_t v;
        if (p < keep) v = pruned[x * degree + p];
        else if (p < keep + n_rev) v = (int32_t)(uint32_t)best[p - keep];
        else v = pruned[x * degree + keep + (p - keep - n_rev)];
        cand[p] = v;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < total; p += blockDim.x) {
        int32_t v = cand[p];
        bool good = v != VL_MAXINT;
        if (p >= keep) {
            if (p < keep + n_rev && v == (int32_t)x) good = false;
            for (int q = 0; q < p && good; ++q) {
                int32_t u = cand[q];
                // an earlier equal entry that is itself usable (a reverse entry equal to x never is)
                if (u == v && !(q >= keep && q < keep + n_rev && u == (int32_t)x)) good = false;
            }
        }
        ok[p] = good;
    }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int run = 0;
    for (int base = 0; base < total; base += blockDim.x) {
        int p = base + threadIdx.x;
        bool k = p < total && ok[p];
        uint64_t b = __ballot(k);
        if (lane == 0) wave_cnt[wave] = __popcll(b);
        __syncthreads();
        if (k) {
            int dest = run + __popcll(b & ((1ull << lane) - 1));
            for (int w = 0; w < wave; ++w) dest += wave_cnt[w];
            if (dest < degree) out[x * degree + dest] = cand[p];
        }
        for (int w = 0; w < kQueueWaves; ++w) run += wave_cnt[w];
        __syncthreads();
    }
    for (int o = run + threadIdx.x; o < degree; o += blockDim.x) out[x * degree + o] = VL_MAXINT;
}

struct OptPlan {
    int64_t n_edges, scan_blocks;
    int64_t off_pruned, off_keys, off_count, off_start, off_totals, total;
    int rev_from, keep;
};

inline int64_t align256(int64_t x) { return (x + 255) & ~255ll; }

int opt_plan(int64_t n, int64_t width, int64_t degree, OptPlan *p) {
    VL_REQUIRE(n > 0 && n < (1ll << 30), "row count out of range");
    VL_REQUIRE(width >= 1 && width <= 2048, "neighbour rows must have 1..2048 slots");
    VL_REQUIRE(degree >= 1 && degree <= width, "degree must be between 1 and the row width");
    p->keep = (int)(degree / 2);
    p->rev_from = (int)(degree / 2);
    p->n_edges = n * p->rev_from;
    VL_REQUIRE(p->n_edges < (1ll << 31), "too many reverse edges for 32-bit segment offsets");
    p->scan_blocks = (n + 1 + kScanItems - 1) / kScanItems;
    int64_t o = 0;
    p->off_pruned = o; o = align256(o + n * degree * 4);
    p->off_keys = o; o = align256(o + p->n_edges * 8);
    p->off_count = o; o = align256(o + (n + 1) * 4);
    p->off_start = o; o = align256(o + (n + 1) * 4);
    p->off_totals = o; o = align256(o + p->scan_blocks * 4);
    p->total = o;
    return VL_OK;
}

}  // namespace

VL_EXPORT int64_t vl_optimize_graph_workspace_bytes(int64_t n, int64_t width, int64_t degree) {
    OptPlan p;
    int rc = opt_plan(n, width, degree, &p);
    return rc < 0 ? rc : p.total;
}

VL_EXPORT int vl_optimize_graph(const int32_t *beams, int64_t n, int64_t width, int64_t degree,
                                int32_t *out, void *workspace, int64_t workspace_bytes, void *stream) {
    OptPlan p;
    int rc = opt_plan(n, width, degree, &p);
    if (rc < 0) return rc;
    VL_REQUIRE(beams && out && workspace, "null pointer");
    VL_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    if (workspace_bytes < p.total) {
        vl_set_error("workspace of %lld bytes is smaller than the %lld needed", (long long)workspace_bytes,
                     (long long)p.total);
        return VL_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    char *ws = (char *)workspace;
    int32_t *pruned = (int32_t *)(ws + p.off_pruned);
    uint64_t *keys = (uint64_t *)(ws + p.off_keys);
    int32_t *count = (int32_t *)(ws + p.off_count), *start = (int32_t *)(ws + p.off_start);
    int32_t *totals = (int32_t *)(ws + p.off_totals);

    int P = vl_next_pow2(width);
    if (P < 2) P = 2;
    size_t smem = (size_t)P * 8 + (size_t)width * 8;
    for (int64_t row0 = 0; row0 < n; row0 += kMaxBlocks) {
        int64_t rows = n - row0 < kMaxBlocks ? n - row0 : kMaxBlocks;
        hipLaunchKernelGGL(rank_prune_kernel, dim3((unsigned)rows), dim3(kQueueThreads), smem, st, beams, n, (int)width,
                           P, (int)degree, pruned, row0);
    }
    VL_LAUNCH_CHECK("rank_prune_kernel");

    // the reverse edges grouped by target: histogram, exclusive scan, scatter
    hipLaunchKernelGGL(rev_zero_kernel, dim3(vl_grid_for(n + 1, 256)), dim3(256), 0, st, count, n + 1);
    VL_LAUNCH_CHECK("rev_zero_kernel");
    if (p.n_edges > 0) {
        hipLaunchKernelGGL(rev_count_kernel, dim3(vl_grid_for(p.n_edges, 256)), dim3(256), 0, st, pruned, n, (int)degree,
                           p.rev_from, count);
        VL_LAUNCH_CHECK("rev_count_kernel");
    }
    hipLaunchKernelGGL(scan_blocks_kernel, dim3((unsigned)p.scan_blocks), dim3(kScanThreads), 0, st, count, n + 1, start,
                       totals);
    hipLaunchKernelGGL(scan_totals_kernel, dim3(1), dim3(1024), 0, st, totals, p.scan_blocks);
    hipLaunchKernelGGL(scan_add_kernel, dim3((unsigned)p.scan_blocks), dim3(kScanThreads), 0, st, start, n + 1, totals);
    VL_LAUNCH_CHECK("exclusive scan of the edge counts");
    if (p.n_edges > 0) {
        hipLaunchKernelGGL(rev_scatter_kernel, dim3(vl_grid_for(p.n_edges, 256)), dim3(256), 0, st, pruned, n, (int)degree,
                           p.rev_from, start, count, keys);
        VL_LAUNCH_CHECK("rev_scatter_kernel");
    }
    const int cap = (int)(degree - p.keep);
    // the sort of a chunk together with the best so far pads to a power of two (at most 4096 slots: cap <= 1024)
    const int best_slots = vl_next_pow2(cap + kRevChunk);
    const size_t smem2 = (size_t)best_slots * 8 + (size_t)degree * 8 + (size_t)degree * 2 + 16;
    VL_HIP(vl_allow_lds(reverse_merge_kernel, smem2));
    for (int64_t row0 = 0; row0 < n; row0 += kMaxBlocks) {
        int64_t rows = n - row0 < kMaxBlocks ? n - row0 : kMaxBlocks;
        hipLaunchKernelGGL(reverse_merge_kernel, dim3((unsigned)rows), dim3(kQueueThreads), smem2, st, pruned, n,
                           (int)degree, p.keep, cap, best_slots, keys, start, out, row0);
    }
    VL_LAUNCH_CHECK("reverse_merge_kernel");
    return VL_OK;
}
