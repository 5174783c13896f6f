// Batched fixed-capacity sorted queues and the small id-list kernels around
// them, for gfx950.  Stands in for vectorlink_gpu/queue.py (Queue.insert /
// pop_n_ids), utils.py (index_sort, add_new_to_seen_, circulant seeds) and the
// mark / punch-out / exclusion kernels of kernels.py:314-406,471-501.
//
// The reference orders a row with three torch sorts, three int64 gathers and
// two elementwise kernels per insert.  Here one workgroup owns one row: the
// row is packed into 64-bit (distance, id) keys in LDS, sorted once with a
// bitonic network, de-duplicated by the reference's neighbour rule and written
// back in its final order.  Traffic per row is one read and one write of the
// row (8 bytes per slot each way).
#include "rowsort.h"

namespace {

enum RowMode { kIndexSort = 0, kQueueSort = 1, kPunchDup = 2, kInsert = 3 };

struct RowArgs {
    int32_t *ids;
    float *dists;
    int64_t rows;
    int64_t row0;   // first row of this launch
    int cols;       // slots per row (queue capacity)
    int P;          // cols padded to a power of two
    // insert only
    int length;
    int m;
    const int32_t *cand_ids;
    const float *cand_d;
    const int32_t *excl;
    int excl_cols;
    uint8_t *changed;  // [rows, length] or null
};

// exclusion rule of punchout_excluded_kernel (kernels.py:478-488): the list
// ends at its first VL_MAXINT
__device__ inline bool excluded_linear(int32_t v, const int32_t *ex, int n_ex) {
    bool hit = false;
    for (int i = 0; i < n_ex; ++i) hit |= (ex[i] == v);
    return hit;
}

template <int MODE>
__global__ __launch_bounds__(kQueueThreads) void queue_row_kernel(RowArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);
    int32_t *aux = reinterpret_cast<int32_t *>(keys + a.P);  // before-ids / payload ids
    int32_t *exl = aux + a.P;                                 // exclusion prefix
    __shared__ PlaceScratch ps;
    __shared__ int n_ex_s;

    const int64_t row = a.row0 + blockIdx.x;
    int32_t *ids = a.ids + row * a.cols;
    float *dd = a.dists + row * a.cols;

    if constexpr (MODE == kInsert) {
        if (threadIdx.x == 0) n_ex_s = a.excl ? a.excl_cols : 0;
        __syncthreads();
        if (a.excl) {
            const int32_t *ex = a.excl + row * a.excl_cols;
            for (int i = threadIdx.x; i < a.excl_cols; i += blockDim.x) {
                int32_t e = ex[i];
                exl[i] = e;
                if (e == VL_MAXINT) atomicMin(&n_ex_s, i);
            }
        }
        for (int i = threadIdx.x; i < a.length; i += blockDim.x) aux[i] = ids[i];
        __syncthreads();
        const int n_ex = n_ex_s;
        for (int i = threadIdx.x; i < a.P; i += blockDim.x) {
            uint64_t k = kPadKey;
            if (i < a.cols) {
                int32_t id;
                float d;
                if (i >= a.length && i < a.length + a.m) {  // queue.py:47-50
                    id = a.cand_ids[row * a.m + (i - a.length)];
                    d = a.cand_d[row * a.m + (i - a.length)];
                    if (n_ex && excluded_linear(id, exl, n_ex)) {  // queue.py:52-53
                        id = VL_MAXINT;
                        d = VL_MAXFLOAT;
                    }
                } else {
                    id = ids[i];
                    d = dd[i];
                }
                k = vl_make_key(id, d);
            }
            keys[i] = k;
        }
    } else if constexpr (MODE == kPunchDup) {
        // mark + punch on the row as it stands (kernels.py:383-397), then a
        // sort by distance that keeps the current order on ties: the key's
        // low word is the slot position, the id rides along in aux.
        for (int i = threadIdx.x; i < a.P; i += blockDim.x) {
            uint64_t k = kPadKey;
            if (i < a.cols) {
                int32_t id = ids[i];
                float d = dd[i];
                if ((id & VL_DUP_FLAG) || (i > 0 && same_id_ignoring_flag(id, ids[i - 1]))) {
                    id = VL_MAXINT;
                    d = VL_MAXFLOAT;
                }
                aux[i] = id;
                k = ((uint64_t)vl_float_key(d) << 32) | (uint32_t)i;
            }
            keys[i] = k;
        }
    } else {
        for (int i = threadIdx.x; i < a.P; i += blockDim.x)
            keys[i] = i < a.cols ? vl_make_key(ids[i], dd[i]) : kPadKey;
    }

    block_bitonic_sort(keys, a.P);

    if constexpr (MODE == kIndexSort) {
        for (int i = threadIdx.x; i < a.cols; i += blockDim.x) {
            ids[i] = vl_key_id(keys[i]);
            dd[i] = vl_key_dist(keys[i]);
        }
    } else if constexpr (MODE == kPunchDup) {
        for (int i = threadIdx.x; i < a.cols; i += blockDim.x) {
            ids[i] = aux[(uint32_t)keys[i]];
            dd[i] = vl_key_dist(keys[i]);
        }
    } else if constexpr (MODE == kQueueSort) {
        block_place3(keys, a.cols, a.cols, ids, dd, &ps, nullptr, 0, nullptr, nullptr);
    } else {
        block_place3(keys, a.cols, a.cols, ids, dd, &ps, aux, a.length,
                     a.changed ? a.changed + row * a.length : nullptr, nullptr);
    }
}

template <int MODE>
int launch_row_kernel(RowArgs a, hipStream_t st) {
    if (a.rows == 0 || a.cols == 0) return VL_OK;
    VL_REQUIRE(a.cols <= kMaxRowSlots, "row of %d slots exceeds the %d that fit the LDS sort", a.cols, kMaxRowSlots);
    VL_REQUIRE(a.excl_cols <= kMaxRowSlots, "exclusion row of %d ids is too long", a.excl_cols);
    VL_REQUIRE(a.rows < (1ll << 31), "too many rows");
    a.P = vl_next_pow2(a.cols);
    if (a.P < 2) a.P = 2;
    size_t smem = (size_t)a.P * 8 + (size_t)a.P * 4 + (size_t)(a.excl_cols > 0 ? a.excl_cols : 0) * 4;
    VL_REQUIRE(smem + 2048 <= kLdsPerCu, "row of %d slots with %d exclusions needs %zu bytes of LDS (a compute unit has %zu)",
               a.cols, a.excl_cols, smem, kLdsPerCu);
    VL_HIP(vl_allow_lds(queue_row_kernel<MODE>, smem));
    for (a.row0 = 0; a.row0 < a.rows; a.row0 += kMaxBlocks) {
        int64_t rows = a.rows - a.row0 < kMaxBlocks ? a.rows - a.row0 : kMaxBlocks;
        hipLaunchKernelGGL((queue_row_kernel<MODE>), dim3((unsigned)rows), dim3(kQueueThreads), smem, st, a);
    }
    VL_LAUNCH_CHECK("queue_row_kernel");
    return VL_OK;
}

// ---- elementwise kernels ---------------------------------------------------
__global__ void mark_kernel(int32_t *ids, int64_t rows, int64_t cols) {
    // slot t only ever writes slot t + 1's flag bit and compares ids without that bit, so slots may go in any order
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < rows * cols; t += (int64_t)gridDim.x * blockDim.x) {
        int64_t q = t % cols;
        if (q + 1 < cols && same_id_ignoring_flag(ids[t], ids[t + 1])) ids[t + 1] |= VL_DUP_FLAG;
    }
}
__global__ void punch_kernel(int32_t *ids, float *d, int64_t n) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x)
        if (ids[t] & VL_DUP_FLAG) {  // kernels.py:346-349 (VL_MAXINT itself carries the bit)
            ids[t] = VL_MAXINT;
            if (d) d[t] = VL_MAXFLOAT;
        }
}
__global__ void excluded_kernel(int32_t *ids, float *d, int64_t rows, int64_t cols, int64_t is,
                                int64_t ds, const int32_t *excl, int64_t ec, int64_t es) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < rows * cols; t += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = t / cols, q = t % cols;
        int32_t v = ids[r * is + q];
        for (int64_t i = 0; i < ec; ++i) {
            int32_t e = excl[r * es + i];
            if (e == VL_MAXINT) break;
            if (e == v) {
                ids[r * is + q] = VL_MAXINT;
                d[r * ds + q] = VL_MAXFLOAT;
                break;
            }
        }
    }
}
__global__ void index_kernel(const uint32_t *a, const int64_t *idx, uint32_t *out, int64_t rows, int64_t cols) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < rows * cols; t += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = t / cols;
        int64_t j = idx[t];
        out[t] = (j >= 0 && j < cols) ? a[r * cols + j] : 0u;
    }
}
__global__ void pop_kernel(int32_t *ids, float *d, int64_t rows, int64_t cap, int64_t take, int32_t *out) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < rows * take; t += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = t / take, q = t % take;
        out[t] = ids[r * cap + q];
        ids[r * cap + q] = VL_MAXINT;
        d[r * cap + q] = VL_MAXFLOAT;
    }
}

// ---- circulant seed rows (utils.py:26-41) ----------------------------------
// sort_k(row + p_k) = row + sort_k(p_k) as long as the sum stays inside int32,
// so each workgroup sorts the prime list once in LDS and then emits rows.
__global__ __launch_bounds__(kQueueThreads) void circulant_kernel(int32_t *out, int64_t rows, int64_t row0,
                                                                 int64_t modulus, const int32_t *primes,
                                                                 int n, int P) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);
    for (int i = threadIdx.x; i < P; i += blockDim.x)
        keys[i] = i < n ? (uint64_t)((uint32_t)primes[i] ^ 0x80000000u) : kPadKey;
    block_bitonic_sort(keys, P);
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x)
        for (int k = threadIdx.x; k < n; k += blockDim.x) {
            int64_t p = (int32_t)((uint32_t)keys[k] ^ 0x80000000u);
            out[r * n + k] = (int32_t)((row0 + r + p) % modulus);
        }
}

// ---- visited list (utils.py:61-89) -----------------------------------------
// first[0] = smallest column that holds VL_MAXINT in every row (cols if none)
__global__ void seen_first_free_kernel(const int32_t *seen, int64_t rows, int64_t cols, int *first) {
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    bool all = true;
    for (int64_t r = 0; r < rows && all; ++r) all = seen[r * cols + c] == VL_MAXINT;
    if (all) atomicMin(first, (int)c);
}
__global__ void set_int_kernel(int *p, int v) { *p = v; }

__global__ __launch_bounds__(kQueueThreads) void seen_add_kernel(int32_t *seen, int64_t rows, int cols, int P,
                                                                const int32_t *visit, int n_visit,
                                                                const int *first_p, int64_t row0) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);
    const int first = *first_p;
    if (first >= cols) return;                                   // utils.py:68-69
    const int n = min(cols - first, n_visit);                    // utils.py:73-75
    if (n == 0) return;
    const int64_t row = row0 + blockIdx.x;
    int32_t *s = seen + row * cols;
    for (int i = threadIdx.x; i < P; i += blockDim.x) {
        uint64_t k = kPadKey;
        if (i < cols) {
            int32_t v = (i >= first && i < first + n) ? visit[row * n_visit + (i - first)] : s[i];
            k = (uint64_t)((uint32_t)v ^ 0x80000000u);           // signed ascending
        }
        keys[i] = k;
    }
    block_bitonic_sort(keys, P);                                 // utils.py:86
    // mark + punch + second sort (utils.py:87-88): first of each run stays, in order
    const int lane = threadIdx.x & (kWave - 1);
    __shared__ int wave_cnt[kQueueWaves];
    int run = 0;
    for (int base = 0; base < cols; base += blockDim.x) {
        int i = base + threadIdx.x;
        bool keep = false;
        int32_t v = VL_MAXINT;
        if (i < cols) {
            v = (int32_t)((uint32_t)keys[i] ^ 0x80000000u);
            int32_t left = i > 0 ? (int32_t)((uint32_t)keys[i - 1] ^ 0x80000000u) : 0;
            keep = !(i > 0 && same_id_ignoring_flag(v, left)) && !(v & VL_DUP_FLAG);
        }
        uint64_t b = __ballot(keep);
        if (lane == 0) wave_cnt[threadIdx.x / kWave] = __popcll(b);
        __syncthreads();
        if (keep) {
            int dest = run + __popcll(b & ((1ull << lane) - 1));
            for (int w = 0; w < (int)(threadIdx.x / kWave); ++w) dest += wave_cnt[w];
            s[dest] = v;
        }
        for (int w = 0; w < kQueueWaves; ++w) run += wave_cnt[w];
        __syncthreads();
    }
    for (int i = run + threadIdx.x; i < cols; i += blockDim.x) s[i] = VL_MAXINT;
}

inline unsigned blocks_for(int64_t n, int per) { return vl_grid_for(n, per); }

}  // namespace

VL_EXPORT int vl_index_sort(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0, "negative size");
    VL_REQUIRE(rows == 0 || cols == 0 || (ids && dists), "null pointer");
    RowArgs a = {};
    a.ids = ids; a.dists = dists; a.rows = rows; a.cols = (int)cols;
    VL_REQUIRE(cols <= kMaxRowSlots, "row too long");
    return launch_row_kernel<kIndexSort>(a, (hipStream_t)stream);
}

VL_EXPORT int vl_queue_sort(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0, "negative size");
    VL_REQUIRE(rows == 0 || cols == 0 || (ids && dists), "null pointer");
    RowArgs a = {};
    a.ids = ids; a.dists = dists; a.rows = rows; a.cols = (int)cols;
    VL_REQUIRE(cols <= kMaxRowSlots, "row too long");
    return launch_row_kernel<kQueueSort>(a, (hipStream_t)stream);
}

VL_EXPORT int vl_punchout_duplicates(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0, "negative size");
    VL_REQUIRE(rows == 0 || cols == 0 || (ids && dists), "null pointer");
    RowArgs a = {};
    a.ids = ids; a.dists = dists; a.rows = rows; a.cols = (int)cols;
    VL_REQUIRE(cols <= kMaxRowSlots, "row too long");
    return launch_row_kernel<kPunchDup>(a, (hipStream_t)stream);
}

VL_EXPORT int vl_queue_insert(int32_t *q_ids, float *q_dists, int64_t rows, int64_t capacity,
                              int64_t length, const int32_t *cand_ids, const float *cand_dists,
                              int64_t m, const int32_t *excl, int64_t excl_cols, uint8_t *changed,
                              void *stream) {
    VL_REQUIRE(rows >= 0 && capacity >= 0 && length >= 0 && m >= 0 && excl_cols >= 0, "negative size");
    VL_REQUIRE(length + m <= capacity, "insert of %lld candidates does not fit: length %lld, capacity %lld",
               (long long)m, (long long)length, (long long)capacity);
    VL_REQUIRE(capacity <= kMaxRowSlots, "queue capacity %lld exceeds %d", (long long)capacity, kMaxRowSlots);
    if (rows == 0) return VL_OK;
    VL_REQUIRE(q_ids && q_dists && (m == 0 || (cand_ids && cand_dists)), "null pointer");
    RowArgs a = {};
    a.ids = q_ids; a.dists = q_dists; a.rows = rows; a.cols = (int)capacity;
    a.length = (int)length; a.m = (int)m; a.cand_ids = cand_ids; a.cand_d = cand_dists;
    a.excl = excl_cols > 0 ? excl : nullptr; a.excl_cols = excl ? (int)excl_cols : 0; a.changed = changed;
    return launch_row_kernel<kInsert>(a, (hipStream_t)stream);
}

VL_EXPORT int vl_queue_pop(int32_t *q_ids, float *q_dists, int64_t rows, int64_t capacity,
                           int64_t take, int32_t *out, void *stream) {
    VL_REQUIRE(rows >= 0 && take >= 0 && take <= capacity, "bad pop size");
    if (rows == 0 || take == 0) return VL_OK;
    VL_REQUIRE(q_ids && q_dists && out, "null pointer");
    hipLaunchKernelGGL(pop_kernel, dim3(blocks_for(rows * take, 256)), dim3(256), 0, (hipStream_t)stream,
                       q_ids, q_dists, rows, capacity, take, out);
    VL_LAUNCH_CHECK("pop_kernel");
    return VL_OK;
}

VL_EXPORT int vl_dedup_ids(int32_t *ids, int64_t rows, int64_t cols, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0, "negative size");
    if (rows == 0 || cols == 0) return VL_OK;
    VL_REQUIRE(ids, "null pointer");
    hipLaunchKernelGGL(mark_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0, (hipStream_t)stream, ids, rows, cols);
    hipLaunchKernelGGL(punch_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0, (hipStream_t)stream, ids,
                       (float *)nullptr, rows * cols);
    VL_LAUNCH_CHECK("mark/punch");
    return VL_OK;
}

VL_EXPORT int vl_dedup_pairs(int32_t *ids, float *dists, int64_t rows, int64_t cols, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0, "negative size");
    if (rows == 0 || cols == 0) return VL_OK;
    VL_REQUIRE(ids && dists, "null pointer");
    hipLaunchKernelGGL(mark_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0, (hipStream_t)stream, ids, rows, cols);
    hipLaunchKernelGGL(punch_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0, (hipStream_t)stream, ids, dists,
                       rows * cols);
    VL_LAUNCH_CHECK("mark/punch");
    return VL_OK;
}

VL_EXPORT int vl_punchout_excluded(int32_t *ids, float *dists, int64_t rows, int64_t cols,
                                   int64_t ids_stride, int64_t dists_stride, const int32_t *excl,
                                   int64_t excl_cols, int64_t excl_stride, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0 && excl_cols >= 0, "negative size");
    VL_REQUIRE(ids_stride >= cols && dists_stride >= cols && excl_stride >= excl_cols, "stride smaller than row");
    if (rows == 0 || cols == 0 || excl_cols == 0) return VL_OK;
    VL_REQUIRE(ids && dists && excl, "null pointer");
    hipLaunchKernelGGL(excluded_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0, (hipStream_t)stream, ids,
                       dists, rows, cols, ids_stride, dists_stride, excl, excl_cols, excl_stride);
    VL_LAUNCH_CHECK("excluded_kernel");
    return VL_OK;
}

VL_EXPORT int vl_index_by_tensor(const void *a, const int64_t *index, void *out, int64_t rows,
                                 int64_t cols, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0, "negative size");
    if (rows == 0 || cols == 0) return VL_OK;
    VL_REQUIRE(a && index && out && a != out, "null or aliased pointer");
    hipLaunchKernelGGL(index_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t *)a, index, (uint32_t *)out, rows, cols);
    VL_LAUNCH_CHECK("index_kernel");
    return VL_OK;
}

VL_EXPORT int vl_circulants(int32_t *out, int64_t rows, int64_t row0, int64_t modulus,
                            const int32_t *primes, int64_t n_primes, void *stream) {
    VL_REQUIRE(rows >= 0 && n_primes >= 0 && row0 >= 0, "negative size");
    VL_REQUIRE(modulus > 0 && modulus <= VL_MAXINT, "modulus out of range");
    VL_REQUIRE(n_primes <= kMaxRowSlots, "too many primes");
    // every prime of the table is below 2^24; keep row + prime inside int32 as the reference's int32 add
    VL_REQUIRE(row0 + rows <= (1ll << 31) - (1ll << 24), "row index too large for int32 seeds");
    if (rows == 0 || n_primes == 0) return VL_OK;
    VL_REQUIRE(out && primes, "null pointer");
    int P = vl_next_pow2(n_primes);
    if (P < 2) P = 2;
    unsigned grid = (unsigned)(rows < 4096 ? rows : 4096);
    hipLaunchKernelGGL(circulant_kernel, dim3(grid), dim3(kQueueThreads), (size_t)P * 8, (hipStream_t)stream, out, rows,
                       row0, modulus, primes, (int)n_primes, P);
    VL_LAUNCH_CHECK("circulant_kernel");
    return VL_OK;
}

VL_EXPORT int vl_seen_add(int32_t *seen, int64_t rows, int64_t cols, const int32_t *visit,
                          int64_t n_visit, void *workspace, int *host_status, void *stream) {
    VL_REQUIRE(rows >= 0 && cols >= 0 && n_visit >= 0, "negative size");
    VL_REQUIRE(cols <= kMaxRowSlots, "visited list of %lld columns exceeds %d", (long long)cols, kMaxRowSlots);
    VL_REQUIRE(host_status && workspace, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (rows == 0 || cols == 0) {
        *host_status = cols == 0 ? 0 : 1;
        return VL_OK;
    }
    VL_REQUIRE(seen && (n_visit == 0 || visit), "null pointer");
    int *first = (int *)workspace;
    hipLaunchKernelGGL(set_int_kernel, dim3(1), dim3(1), 0, st, first, (int)cols);
    hipLaunchKernelGGL(seen_first_free_kernel, dim3(blocks_for(cols, 64)), dim3(64), 0, st, seen, rows, cols, first);
    int P = vl_next_pow2(cols);
    if (P < 2) P = 2;
    for (int64_t row0 = 0; row0 < rows; row0 += kMaxBlocks) {
        int64_t part = rows - row0 < kMaxBlocks ? rows - row0 : kMaxBlocks;
        hipLaunchKernelGGL(seen_add_kernel, dim3((unsigned)part), dim3(kQueueThreads), (size_t)P * 8, st, seen, rows,
                           (int)cols, P, visit, (int)n_visit, first, row0);
    }
    VL_LAUNCH_CHECK("seen_add");
    int h = 0;
    VL_HIP(hipMemcpyAsync(&h, first, sizeof(int), hipMemcpyDeviceToHost, st));
    VL_HIP(hipStreamSynchronize(st));
    *host_status = h < cols ? 1 : 0;
    return VL_OK;
}
