// Detour pruning for gfx950: stands in for prune_kernel / prune_
// (vectorlink_gpu/kernels.py:409-468).
//
// The reference launches a (W,1,1) block per (x, j) whose W threads all do the
// same work with y_link_z = threadIdx.y = 0, and mutates the tables while
// other blocks read them.  Here one workgroup owns row x: it reads the row
// once into LDS, takes every decision from the tables as passed in, and writes
// the pruned, distance-ordered row to separate output tables.  Traffic per
// row: 16*W bytes streamed plus W random 8-byte reads of (beams[y,0], d[y,0]).
#include "rowsort.h"

namespace {

__global__ __launch_bounds__(kQueueThreads) void prune_kernel(const int32_t *beams, const float *dists, int64_t n,
                                                             int W, int P, int32_t *beams_out, float *dists_out,
                                                             int64_t row0) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);
    int32_t *ids = reinterpret_cast<int32_t *>(keys + P);
    float *dd = reinterpret_cast<float *>(ids + P);
    int32_t *mark = reinterpret_cast<int32_t *>(dd + P);
    const int64_t x = row0 + blockIdx.x;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        ids[i] = beams[x * W + i];
        dd[i] = dists[x * W + i];
        mark[i] = 0;
    }
    __syncthreads();
    for (int j = threadIdx.x; j < W; j += blockDim.x) {
        int32_t y = ids[j];
        if (y == VL_MAXINT || y < 0 || y >= n) continue;       // kernels.py:417-418
        int32_t z = beams[(int64_t)y * W];
        if (z == VL_MAXINT) continue;                          // kernels.py:421-422
        int xz = -1;
        for (int i = 0; i < W; ++i)                            // kernels.py:424-427 (last match wins)
            if (ids[i] == z) xz = i;
        if (xz < 0) continue;
        float dxz = dd[xz], dxy = dd[j], dyz = dists[(int64_t)y * W];
        if (dxz > dxy && dxz > dyz) mark[xz] = 1;              // kernels.py:436-438
    }
    __syncthreads();
    // distances.sort() then the ids follow (kernels.py:466-467); ties keep slot order
    for (int i = threadIdx.x; i < P; i += blockDim.x) {
        uint64_t k = kPadKey;
        if (i < W) {
            float d = mark[i] ? VL_MAXFLOAT : dd[i];
            k = ((uint64_t)vl_float_key(d) << 32) | (uint32_t)i;
        }
        keys[i] = k;
    }
    block_bitonic_sort(keys, P);
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        int src = (int)(uint32_t)keys[i];
        beams_out[x * W + i] = mark[src] ? VL_MAXINT : ids[src];
        dists_out[x * W + i] = mark[src] ? VL_MAXFLOAT : vl_key_dist(keys[i]);
    }
}

}  // namespace

VL_EXPORT int vl_prune(const int32_t *beams, const float *dists, int64_t n, int64_t width,
                       int32_t *beams_out, float *dists_out, void *stream) {
    VL_REQUIRE(n >= 0 && width >= 0, "negative size");
    VL_REQUIRE(width <= kMaxRowSlots / 2, "neighbour rows of %lld slots are too wide", (long long)width);
    VL_REQUIRE(n < (1ll << 31), "too many rows");
    if (n == 0 || width == 0) return VL_OK;
    VL_REQUIRE(beams && dists && beams_out && dists_out, "null pointer");
    VL_REQUIRE(beams != beams_out && dists != dists_out, "prune needs separate output tables");
    int P = vl_next_pow2(width);
    if (P < 2) P = 2;
    size_t smem = (size_t)P * (8 + 4 + 4 + 4);
    for (int64_t row0 = 0; row0 < n; row0 += kMaxBlocks) {
        int64_t rows = n - row0 < kMaxBlocks ? n - row0 : kMaxBlocks;
        hipLaunchKernelGGL(prune_kernel, dim3((unsigned)rows), dim3(kQueueThreads), smem, (hipStream_t)stream, beams,
                           dists, n, (int)width, P, beams_out, dists_out, row0);
    }
    VL_LAUNCH_CHECK("prune_kernel");
    return VL_OK;
}
