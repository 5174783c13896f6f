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
//  reverse edges         (y, slot) keys + x values for the first rev_from slots
//                        of every pruned row, one stable radix sort (rocPRIM):
//                        afterwards the sources of each y are contiguous and
//                        ordered by (slot, x).
//  reverse_merge_kernel  one workgroup per row: keep | reverse | rest, without
//                        duplicates, cut to `degree`.
#include "rowsort.h"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace {

constexpr int kSlotBits = 12;  // slots per row < 4096

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

__global__ void rev_keys_kernel(const int32_t *__restrict__ pruned, int64_t n, int degree, int rev_from,
                                uint64_t *__restrict__ keys, int32_t *__restrict__ vals) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n * rev_from;
         e += (int64_t)gridDim.x * blockDim.x) {
        int64_t x = e / rev_from;
        int k = (int)(e - x * rev_from);
        int32_t y = pruned[x * degree + k];
        bool real = y != VL_MAXINT && y >= 0 && y < n;
        keys[e] = real ? (((uint64_t)(uint32_t)y << kSlotBits) | (uint32_t)k) : ((1ull << (30 + kSlotBits)) | 0ull);
        vals[e] = (int32_t)x;
    }
}

// start[y] = first sorted edge whose target is >= y, for y in [0, n]
__global__ void rev_start_kernel(const uint64_t *__restrict__ keys, int64_t n_edges, int64_t n, int64_t *__restrict__ start) {
    for (int64_t y = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; y <= n; y += (int64_t)gridDim.x * blockDim.x) {
        uint64_t want = (uint64_t)y << kSlotBits;
        int64_t lo = 0, hi = n_edges;
        while (lo < hi) {
            int64_t mid = (lo + hi) >> 1;
            if (keys[mid] < want) lo = mid + 1;
            else hi = mid;
        }
        start[y] = lo;
    }
}

__global__ __launch_bounds__(kQueueThreads) void reverse_merge_kernel(const int32_t *__restrict__ pruned, int64_t n,
                                                                     int degree, int keep, int cap,
                                                                     const int32_t *__restrict__ rev_src,
                                                                     const int64_t *__restrict__ start,
                                                                     int32_t *__restrict__ out, int64_t row0) {
    extern __shared__ __align__(16) unsigned char smem[];
    int32_t *cand = reinterpret_cast<int32_t *>(smem);  // keep | reverse | rest
    uint8_t *ok = reinterpret_cast<uint8_t *>(cand + 2 * degree);
    __shared__ int wave_cnt[kQueueWaves];
    const int64_t x = row0 + blockIdx.x;
    const int64_t s = start[x];
    const int n_rev = (int)min((int64_t)cap, start[x + 1] - s);
    const int total = keep + n_rev + (degree - keep);
    for (int p = threadIdx.x; p < total; p += blockDim.x) {
        int32_t v;
        if (p < keep) v = pruned[x * degree + p];
        else if (p < keep + n_rev) v = rev_src[s + (p - keep)];
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
    int64_t n_edges;
    int64_t off_pruned, off_keys_a, off_keys_b, off_vals_a, off_vals_b, off_start, off_temp, total;
    size_t temp_bytes;
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
    VL_REQUIRE(p->n_edges < (1ll << 31), "too many reverse edges for one sort");
    size_t temp = 0;
    if (p->n_edges > 0) {
        hipError_t e = rocprim::radix_sort_pairs(nullptr, temp, (uint64_t *)nullptr, (uint64_t *)nullptr,
                                                 (int32_t *)nullptr, (int32_t *)nullptr, (size_t)p->n_edges, 0,
                                                 31 + kSlotBits, (hipStream_t)0);
        if (e != hipSuccess) {
            vl_set_error("rocprim::radix_sort_pairs (size query) failed: %s", hipGetErrorString(e));
            return VL_ERR_HIP;
        }
    }
    p->temp_bytes = temp;
    int64_t o = 0;
    p->off_pruned = o; o = align256(o + n * degree * 4);
    p->off_keys_a = o; o = align256(o + p->n_edges * 8);
    p->off_keys_b = o; o = align256(o + p->n_edges * 8);
    p->off_vals_a = o; o = align256(o + p->n_edges * 4);
    p->off_vals_b = o; o = align256(o + p->n_edges * 4);
    p->off_start = o; o = align256(o + (n + 1) * 8);
    p->off_temp = o; o = align256(o + (int64_t)temp);
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
    uint64_t *keys_a = (uint64_t *)(ws + p.off_keys_a), *keys_b = (uint64_t *)(ws + p.off_keys_b);
    int32_t *vals_a = (int32_t *)(ws + p.off_vals_a), *vals_b = (int32_t *)(ws + p.off_vals_b);
    int64_t *start = (int64_t *)(ws + p.off_start);

    int P = vl_next_pow2(width);
    if (P < 2) P = 2;
    size_t smem = (size_t)P * 8 + (size_t)width * 8;
    for (int64_t row0 = 0; row0 < n; row0 += kMaxBlocks) {
        int64_t rows = n - row0 < kMaxBlocks ? n - row0 : kMaxBlocks;
        hipLaunchKernelGGL(rank_prune_kernel, dim3((unsigned)rows), dim3(kQueueThreads), smem, st, beams, n, (int)width,
                           P, (int)degree, pruned, row0);
    }
    VL_LAUNCH_CHECK("rank_prune_kernel");

    if (p.n_edges > 0) {
        hipLaunchKernelGGL(rev_keys_kernel, dim3(vl_grid_for(p.n_edges, 256)), dim3(256), 0, st, pruned, n,
                           (int)degree, p.rev_from, keys_a, vals_a);
        VL_LAUNCH_CHECK("rev_keys_kernel");
        size_t temp = p.temp_bytes;
        VL_HIP(rocprim::radix_sort_pairs(ws + p.off_temp, temp, keys_a, keys_b, vals_a, vals_b, (size_t)p.n_edges, 0,
                                         31 + kSlotBits, st));
    }
    hipLaunchKernelGGL(rev_start_kernel, dim3(vl_grid_for(n + 1, 256)), dim3(256), 0, st, keys_b, p.n_edges, n,
                       start);
    VL_LAUNCH_CHECK("rev_start_kernel");
    size_t smem2 = (size_t)degree * 8 + (size_t)degree * 2 + 16;
    for (int64_t row0 = 0; row0 < n; row0 += kMaxBlocks) {
        int64_t rows = n - row0 < kMaxBlocks ? n - row0 : kMaxBlocks;
        hipLaunchKernelGGL(reverse_merge_kernel, dim3((unsigned)rows), dim3(kQueueThreads), smem2, st, pruned, n,
                           (int)degree, p.keep, (int)(degree - p.keep), vals_b, start, out, row0);
    }
    VL_LAUNCH_CHECK("reverse_merge_kernel");
    return VL_OK;
}
