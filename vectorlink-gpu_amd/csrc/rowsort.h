// Workgroup-level building blocks for the batched sorted queues: an LDS
// bitonic sort on 64-bit (distance, id) keys, the adjacent-duplicate rule of
// the reference's mark/punch-out kernels, and the stable three-way placement
// that stands in for the reference's second sort.
#pragma once
#include "vl_common.h"

constexpr int kQueueThreads = 256;
constexpr int kQueueWaves = kQueueThreads / kWave;
constexpr int kMaxRowSlots = 4096;   // largest row (after padding to a power of two) sorted in LDS

// Ascending bitonic sort of P (power of two) keys in LDS by the whole
// workgroup.  Ends with a barrier.  A compare-exchange step whose partners lie
// 64 or more keys apart goes through LDS with a barrier; the steps below that
// distance stay inside one wavefront's 64 consecutive keys and run in
// registers (cross-lane exchanges, no barrier), all of them between one LDS
// read and one LDS write of the key.
__device__ inline void block_bitonic_sort(uint64_t *keys, int P) {
    __syncthreads();
    for (int k = 2; k <= P; k <<= 1) {
        int j = k >> 1;
        for (; j >= kWave; j >>= 1) {
            for (int t = threadIdx.x; t < (P >> 1); t += blockDim.x) {
                int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
                int p = i | j;
                bool up = (i & k) == 0;
                uint64_t a = keys[i], b = keys[p];
                if ((a > b) == up) {
                    keys[i] = b;
                    keys[p] = a;
                }
            }
            __syncthreads();
        }
        for (int idx = threadIdx.x; idx < P; idx += blockDim.x) {
            uint64_t key = keys[idx];
            const bool up = (idx & k) == 0;
            for (int jj = j; jj > 0; jj >>= 1) {
                const uint64_t other = __shfl_xor((unsigned long long)key, jj);
                const bool take_min = ((idx & jj) == 0) == up;
                key = (take_min == (other < key)) ? other : key;
            }
            keys[idx] = key;
        }
        __syncthreads();
    }
}

__device__ inline bool same_id_ignoring_flag(int32_t a, int32_t b) {
    return (a & ~VL_DUP_FLAG) == (b & ~VL_DUP_FLAG);  // kernels.py:325-330
}

// Scratch for block_place3: per-wave counts of one tile and class totals.
struct PlaceScratch {
    int wave_cnt[kQueueWaves][3];
    int total[3];
};

// keys[0:n) is a row already ordered by (distance, id).  Applies the
// reference's mark + punch-out (a slot whose id equals its left neighbour's
// becomes the empty pair, kernels.py:314-349) followed by its sort by
// distance that keeps the previous order on ties (kernels.py:402-403), and
// writes the resulting row to out_ids/out_d[0:n_out).  The stable sort is
// realised as a three-way placement: kept slots closer than VL_MAXFLOAT stay
// in order, then every punched slot or slot at exactly VL_MAXFLOAT, then
// slots beyond VL_MAXFLOAT.
//
// before/changed (optional): before[0:len) are the ids the row started with;
// changed_bytes[i] = (new id at i != before[i]) for i < len and *any_changed
// is or-ed with 1 when some slot differs.
__device__ inline void block_place3(const uint64_t *keys, int n, int n_out, int32_t *out_ids,
                                    float *out_d, PlaceScratch *ps, const int32_t *before,
                                    int len, uint8_t *changed_bytes, int *any_changed) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint32_t fkey = vl_float_key(VL_MAXFLOAT);
    if (threadIdx.x < 3) ps->total[threadIdx.x] = 0;
    __syncthreads();

    auto classify = [&](int i, int32_t &id, float &d) -> int {
        uint64_t k = keys[i];
        id = vl_key_id(k);
        uint32_t hk = (uint32_t)(k >> 32);
        d = vl_key_float(hk);
        // punched: a duplicate of the left neighbour, or any id carrying bit 30
        // (kernels.py:346-349 tests the bit alone, so an empty id always
        // leaves with the empty distance)
        bool flagged = (id & VL_DUP_FLAG) || (i > 0 && same_id_ignoring_flag(id, vl_key_id(keys[i - 1])));
        if (flagged) {
            id = VL_MAXINT;
            d = VL_MAXFLOAT;
            return 1;
        }
        return hk < fkey ? 0 : (hk == fkey ? 1 : 2);
    };

    // pass 1: class totals
    int cnt[3] = {0, 0, 0};
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        int32_t id;
        float d;
        cnt[classify(i, id, d)]++;
    }
#pragma unroll
    for (int c = 0; c < 3; ++c)
        if (cnt[c]) atomicAdd(&ps->total[c], cnt[c]);
    __syncthreads();
    int run[3] = {0, ps->total[0], ps->total[0] + ps->total[1]};
    __syncthreads();

    // pass 2: stable destinations, tile by tile
    bool diff = false;
    for (int base = 0; base < n; base += blockDim.x) {
        int i = base + threadIdx.x;
        int32_t id = VL_MAXINT;
        float d = VL_MAXFLOAT;
        int c = -1;
        if (i < n) c = classify(i, id, d);
        uint64_t b0 = __ballot(c == 0), b1 = __ballot(c == 1), b2 = __ballot(c == 2);
        if (lane == 0) {
            ps->wave_cnt[wave][0] = __popcll(b0);
            ps->wave_cnt[wave][1] = __popcll(b1);
            ps->wave_cnt[wave][2] = __popcll(b2);
        }
        __syncthreads();
        uint64_t lt = (1ull << lane) - 1;
        if (c >= 0) {
            uint64_t mine = c == 0 ? b0 : (c == 1 ? b1 : b2);
            int dest = run[c] + __popcll(mine & lt);
            for (int w = 0; w < wave; ++w) dest += ps->wave_cnt[w][c];
            if (dest < n_out) {
                out_ids[dest] = id;
                out_d[dest] = d;
                if (before && dest < len) {
                    bool ch = id != before[dest];
                    diff |= ch;
                    if (changed_bytes) changed_bytes[dest] = ch ? 1 : 0;
                }
            }
        }
#pragma unroll
        for (int cc = 0; cc < 3; ++cc)
            for (int w = 0; w < kQueueWaves; ++w) run[cc] += ps->wave_cnt[w][cc];
        __syncthreads();
    }
    if (any_changed && __ballot(diff) && lane == 0) atomicOr(any_changed, 1);
}
