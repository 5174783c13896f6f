// The beam-search loop of closest_vectors (vectorlink_gpu/ann.py:38-93) for
// gfx950.
//
// The reference runs ~50 torch ops / Numba launches and at least two blocking
// host round trips per iteration.  Here an iteration has two phases per query
// row:
//   expand  pop the visit-queue heads, gather their neighbour lists, evaluate
//           the candidate distances (dist_device.h);
//   merge   insert the candidates into the search queue (Queue.insert,
//           queue.py:37-61), record the visited ids (add_new_to_seen_,
//           utils.py:61-82) and refill the visit queue with the candidates
//           not yet visited.
// By default both phases of a row run in one workgroup of ONE launch
// (beam_step_kernel); the two-launch form (expand kernel of dist.hip, then a
// merge kernel) is kept behind a flag.  Batch-wide state (first free
// visited-list column, "any row changed") lives in a device control block;
// the host only reads the changed flag every speculative_readahead
// iterations, the cadence at which the reference tests for progress
// (ann.py:68,90-91).
#include "beam_ctrl.h"
#include "rowsort.h"
#include "dist_device.h"
#include "sketch_device.h"
#include <stddef.h>
#include <stdlib.h>
#include <atomic>
#include <mutex>

int vl_launch_expand(const float *queries, int64_t n_rows, const float *vectors, int64_t n_vectors,
                     int64_t dim, const int32_t *ids, const int32_t *visit, int64_t n_visit,
                     const int32_t *beams, int64_t n_nodes, int64_t width, int64_t m,
                     int32_t *idx_out, float *dist_out, BeamCtrl *ctrl, int iter, int readahead,
                     int seen_cols, int64_t visit_stride, int count_evals, uint64_t *memo, int memo_slots,
                     int metric, hipStream_t st);

int vl_launch_sketch_queries(const float *queries, int64_t n_rows, int64_t dim, uint8_t *out_rows, hipStream_t st);

namespace {

constexpr int kMaxVisit = 64;  // parallel_visit_count handled by one wavefront

// Optional per-kernel timing of the loop (off by default): HIP events around
// every expand and merge launch on the caller's stream, summed per call.
struct BeamProfile {
    int enabled = 0;
    double expand_ms = 0, merge_ms = 0;
    int64_t expand_launches = 0, merge_launches = 0, evals = 0, rows = 0, iterations = 0, wanted = 0, sketched = 0;
};
// The only mutable state of the library besides the thread-local error text.  A call
// sums into a BeamProfile of its own and adds it here once, under the mutex, when it
// returns, so calls on different host threads do not tear each other's sums.
BeamProfile g_prof;
std::mutex g_prof_mutex;
std::atomic<int64_t> g_step_launches{0};  // vl_beam_launches

// HIP events of one profiled call; destroyed on every way out of the call.
struct EventSet {
    hipEvent_t ev[3 * 64];
    int n = 0;
    int create(int count) {
        for (; n < count; ++n) VL_HIP(hipEventCreate(&ev[n]));
        return VL_OK;
    }
    ~EventSet() {
        for (int i = 0; i < n; ++i) (void)hipEventDestroy(ev[i]);
    }
};

struct MergeArgs {
    BeamCtrl *ctrl;
    int iter;
    int readahead;
    int64_t n_rows;
    const int32_t *cand_ids;
    const float *cand_d;
    int m;
    int32_t *q_ids;
    float *q_d;
    int cap, L, Ps;
    const int32_t *excl;
    int excl_cols;
    int32_t *v_ids;
    float *v_d;
    int VL, Vt, Pv, Pc;
    int32_t *seen;
    int32_t *seen_count;
    int E;
    int32_t *row_quiet;  // per-query stop only (else null): iterations in a row that left the row's search queue unchanged
};

__device__ inline bool sorted_contains(const int32_t *a, int n, int32_t v) {
    int lo = 0, hi = n;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (a[mid] < v) lo = mid + 1;
        else hi = mid;
    }
    return lo < n && a[lo] == v;
}
__device__ inline int lower_bound(const int32_t *a, int n, int32_t v) {
    int lo = 0, hi = n;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (a[mid] < v) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

__global__ void beam_memo_clear_kernel(uint64_t *memo, int64_t n) {
    // an empty slot holds id VL_MAXINT, which no probe asks for
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        memo[i] = (uint64_t)(uint32_t)VL_MAXINT;
}

// row_word: what every row starts with in its word of the memo_rate array (StepArgs); sketch_rows: how many rows
// that makes users of the sketch.
__global__ __launch_bounds__(kQueueThreads) void beam_init_kernel(BeamCtrl *ctrl, int64_t n_rows, const int32_t *q_ids,
                                                                 const float *q_d, int cap, int head, int32_t *v_ids,
                                                                 float *v_d, int VL, int32_t *seen_count,
                                                                 int32_t *row_quiet, int32_t *memo_rate, int row_word,
                                                                 int sketch_rows) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t == 0) {
        ctrl->stop = 0;
        ctrl->ended_after = 0;
        ctrl->first[0] = ctrl->first[1] = ctrl->first[2] = 0;
        ctrl->sketch_rows = sketch_rows;
        ctrl->error = 0;
    }
    if (t < 64) ctrl->changed[t] = 0;
    if (t < kBeamStripes) {
        ctrl->evals[t] = 0;
        ctrl->wanted[t] = 0;
        ctrl->sketched[t] = 0;
    }
    if (t < n_rows) {
        seen_count[t] = 0;
        row_quiet[t] = 0;
        memo_rate[t] = row_word;
    }
    if (t < n_rows * VL) {  // Queue.initialize_from_queue, queue.py:30-35
        int64_t r = t / VL;
        int i = (int)(t % VL);
        v_ids[t] = i < head ? q_ids[r * cap + i] : VL_MAXINT;
        v_d[t] = i < head ? q_d[r * cap + i] : VL_MAXFLOAT;
    }
}

__global__ __launch_bounds__(kQueueThreads) void beam_merge_kernel(MergeArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int Pmax = a.Ps > a.Pv ? a.Ps : a.Pv;
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);
    int32_t *before = reinterpret_cast<int32_t *>(keys + Pmax);
    int32_t *seen_a = before + a.L;
    int32_t *seen_b = seen_a + a.E;
    int32_t *exl = seen_b + a.E;
    __shared__ PlaceScratch ps;
    __shared__ int n_ex_s;
    __shared__ int32_t newv[kMaxVisit];
    __shared__ int n_new_s;

    BeamCtrl *c = a.ctrl;
    if (c->stop) return;
    const int t = a.iter;
    const int64_t row = blockIdx.x;
    int cnt = a.seen_count[row];
    int *first_next = &c->first[(t + 1) % 3];
    if (t >= 2 && c->first[(t - 1) % 3] >= a.E) {
        // the visit queue is no longer fed: every candidate of this iteration is
        // empty and no queue changes; keep the running maximum current
        if (threadIdx.x == 0) atomicMax(first_next, cnt);
        return;
    }
    const int first = c->first[t % 3];
    const bool seen_full = first >= a.E;  // add_new_to_seen_ returns None now (utils.py:68-69)
    const bool checking = (t % a.readahead) == 0;

    // ---- search_queue.insert(candidates, exclude) : ann.py:75-80 -----------
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
    int32_t *qi = a.q_ids + row * a.cap;
    float *qd = a.q_d + row * a.cap;
    const int32_t *ci = a.cand_ids + row * a.m;
    const float *cd = a.cand_d + row * a.m;
    for (int i = threadIdx.x; i < a.L; i += blockDim.x) before[i] = qi[i];
    __syncthreads();
    const int n_ex = n_ex_s;
    for (int i = threadIdx.x; i < a.Ps; i += blockDim.x) {
        uint64_t k = kPadKey;
        if (i < a.cap) {
            int32_t id;
            float d;
            if (i >= a.L && i < a.L + a.m) {
                id = ci[i - a.L];
                d = cd[i - a.L];
                bool hit = false;
                for (int e = 0; e < n_ex; ++e) hit |= (exl[e] == id);
                if (hit) {
                    id = VL_MAXINT;
                    d = VL_MAXFLOAT;
                }
            } else {
                id = qi[i];
                d = qd[i];
            }
            k = vl_make_key(id, d);
        }
        keys[i] = k;
    }
    block_bitonic_sort(keys, a.Ps);
    block_place3(keys, a.cap, a.cap, qi, qd, &ps, before, a.L, nullptr,
                 checking ? &c->changed[(t / a.readahead) & 63] : nullptr);

    if (seen_full) {
        if (threadIdx.x == 0) atomicMax(first_next, cnt);
        return;
    }

    // ---- add_new_to_seen_(seen, visited) : utils.py:61-82 -------------------
    // The row is kept sorted, duplicate free and packed at the front, which is
    // what sort + dedup + sort leaves; `cnt` ids are in use.
    int32_t *srow = a.seen + row * a.E;
    const int32_t *vrow_i = a.v_ids + row * a.VL;
    const float *vrow_d = a.v_d + row * a.VL;
    for (int i = threadIdx.x; i < cnt; i += blockDim.x) seen_a[i] = srow[i];
    if (threadIdx.x == 0) n_new_s = 0;
    __syncthreads();
    const int n_add = min(min(a.E - first, a.Vt), a.E - cnt);  // utils.py:73-75 (cnt <= first: rows are packed)
    if (threadIdx.x < kWave) {
        const int j = threadIdx.x;
        int32_t x = j < n_add ? vrow_i[j] : VL_MAXINT;
        bool valid = j < n_add && x != VL_MAXINT && !sorted_contains(seen_a, cnt, x);
        for (int i = 0; i < j && valid; ++i)
            if (vrow_i[i] == x) valid = false;
        uint64_t vm = __ballot(valid);
        // ascending rank among the valid new ids
        int rank = 0;
        for (int i = 0; i < n_add; ++i) {
            int32_t y = vrow_i[i];
            if (((vm >> i) & 1) && y < x) ++rank;
        }
        if (valid) newv[rank] = x;
        if (j == 0) n_new_s = __popcll(vm);
    }
    __syncthreads();
    const int n_new = n_new_s;
    for (int p = threadIdx.x; p < cnt; p += blockDim.x) {
        int32_t v = seen_a[p];
        int shift = 0;
        for (int i = 0; i < n_new; ++i) shift += newv[i] < v;
        seen_b[p + shift] = v;
    }
    if (threadIdx.x < n_new) seen_b[lower_bound(seen_a, cnt, newv[threadIdx.x]) + threadIdx.x] = newv[threadIdx.x];
    __syncthreads();
    cnt += n_new;
    for (int i = threadIdx.x; i < cnt; i += blockDim.x) srow[i] = seen_b[i];
    if (threadIdx.x == 0) {
        a.seen_count[row] = cnt;
        atomicMax(first_next, cnt);
    }

    // ---- visit_queue.insert(candidates, exclude=seen) : ann.py:85-88 --------
    // slots [0, Vt) were popped at the start of this iteration (queue.py:87-95)
    for (int i = threadIdx.x; i < a.Pv; i += blockDim.x) {
        uint64_t k = kPadKey;
        if (i < a.VL + a.m) {
            int32_t id = VL_MAXINT;
            float d = VL_MAXFLOAT;
            if (i >= a.VL) {
                id = ci[i - a.VL];
                d = cd[i - a.VL];
                if (sorted_contains(seen_b, cnt, id)) {
                    id = VL_MAXINT;
                    d = VL_MAXFLOAT;
                }
            } else if (i >= a.Vt) {
                id = vrow_i[i];
                d = vrow_d[i];
            }
            k = vl_make_key(id, d);
        }
        keys[i] = k;
    }
    block_bitonic_sort(keys, a.Pv);
    block_place3(keys, a.VL + a.m, a.VL, a.v_ids + row * a.VL, a.v_d + row * a.VL, &ps, nullptr, 0, nullptr,
                 nullptr);
}

// ---- merge, second form ------------------------------------------------------
// Same result as beam_merge_kernel on [0, length) of the search queue and on the
// visit queue, for queues in the state Queue.insert leaves them (ordered by
// (distance, id), distinct ids) and ids that always carry the same distance -
// both hold for everything closest_vectors is handed by this package.  Instead
// of two full-row sorts, the candidates are sorted once; what is already queued
// (or excluded, or visited) is filtered out with binary searches; the few
// survivors are merged into each sorted queue by rank.
__device__ inline int key_lower_bound(const uint64_t *a, int n, uint64_t k) {
    int lo = 0, hi = n;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (a[mid] < k) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

// Order-preserving compaction of src[0:n) by predicate into dst; returns the
// kept count (uniform).  wave_cnt: kQueueWaves ints of LDS.
template <class Pred>
__device__ inline int block_compact(const uint64_t *src, int n, uint64_t *dst, Pred keep, int *wave_cnt) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    int run = 0;
    for (int base = 0; base < n; base += blockDim.x) {
        int i = base + threadIdx.x;
        bool k = i < n && keep(i);
        uint64_t b = __ballot(k);
        if (lane == 0) wave_cnt[wave] = __popcll(b);
        __syncthreads();
        if (k) {
            int dest = run + __popcll(b & ((1ull << lane) - 1));
            for (int w = 0; w < wave; ++w) dest += wave_cnt[w];
            dst[dest] = src[i];
        }
        for (int w = 0; w < (int)(blockDim.x / kWave); ++w) run += wave_cnt[w];
        __syncthreads();
    }
    return run;
}

// Raise the batch-wide running maximum *slot to at least cnt.  Same-address
// atomics from thousands of workgroups serialise in L2 and were the most
// expensive part of the merge step, so they are kept for the rare case only:
// a row that is at the largest fill any row can have (bound) publishes it with
// a plain store - every such writer stores the same value and no atomicMax of a
// smaller value can lower it - and any row skips the update when a late read
// shows the slot is already there.
__device__ inline void raise_running_max(int *slot, int cnt, int bound) {
    if (__hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= cnt) return;
    if (cnt >= bound) __hip_atomic_store(slot, cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else atomicMax(slot, cnt);
}

// Smallest 32-bit value over a wavefront, in every lane: halves and rows are folded with the swap instructions
// and DPP row shifts that fold_group uses (a lane without a source keeps its own value), a few cycles per
// step where a cross-lane shuffle through the LDS crossbar takes a round trip each.
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t x) {
    {
        uint32_t lo = x, hi = x;
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
        x = lo < hi ? lo : hi;
    }
    {
        uint32_t even = x, odd = x;
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(even), "+v"(odd));
        x = even < odd ? even : odd;
    }
    uint32_t y;
    y = __builtin_amdgcn_update_dpp(x, x, 0x108, 0xf, 0xf, false); x = y < x ? y : x;  // row_shl:8
    y = __builtin_amdgcn_update_dpp(x, x, 0x104, 0xf, 0xf, false); x = y < x ? y : x;  // row_shl:4
    y = __builtin_amdgcn_update_dpp(x, x, 0x102, 0xf, 0xf, false); x = y < x ? y : x;  // row_shl:2
    y = __builtin_amdgcn_update_dpp(x, x, 0x101, 0xf, 0xf, false); x = y < x ? y : x;  // row_shl:1
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)x);
}

// Smallest value over the workgroup of each thread's `mine` (0xFFFFFFFF = none).
// red: 2 * kQueueWaves words of LDS, used alternately so one barrier per call suffices.
__device__ inline uint32_t block_min_u32(uint32_t mine, uint32_t *red, int round) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nw = blockDim.x / kWave;
    mine = wave_min_u32(mine);
    uint32_t *slot = red + (round & 1) * kQueueWaves;
    if (lane == 0) slot[wave] = mine;
    __syncthreads();
    uint32_t m = slot[0];
    for (int w = 1; w < nw; ++w) m = slot[w] < m ? slot[w] : m;
    return m;
}

// A candidate's upper bound (a cosine distance, in [0, 1]) and its slot in one 32-bit key, smallest bound first:
// the bound to 19 bits, rounded down, then the slot (a row has at most kMaxCandidates candidate slots: more would
// not fit the LDS).  Only used to choose which candidates to look at first - any choice is a valid one there - so
// the rounding costs nothing but a slightly different pick among near-equal bounds.  Never 0xFFFFFFFF.
constexpr int kMaxCandidates = 8192;
__device__ __forceinline__ uint32_t bound_slot_key(float hi, int slot) {
    return ((uint32_t)(hi * 524286.0f) << 13) | (uint32_t)slot;
}

// Workgroup-wide scalars shared by the expand and merge phases of a row.
__shared__ int g_n_ex_s;                  // exclusion ids before the row's first empty one
__shared__ int32_t g_visit_s[kMaxVisit];  // the ids popped from the visit queue in this iteration
// The ids the merge phase adds to the visited list (between two of its barriers).  The expand phase and the exact
// rounds of a sketched row, which run before and after that, use the same 256 bytes as the wavefronts' lists of
// candidate lanes (wave_sketch, wave_distances_lds: 64 bytes each) - sixteen 128-thread workgroups of the
// 128-column shape fit a compute unit's LDS with these bytes shared and fifteen without.
__shared__ int32_t g_new_s[kMaxVisit];
static_assert(kMaxVisit * 4 >= 256, "one byte per thread of the largest workgroup");

// What the fused step has read of a row before its merge phase starts.
struct RowState {
    int cnt;    // fill of the row's visited list
    int first;  // first visited-list column that is free in every row
};

// FUSED: the candidates of this row are already in LDS (ids at uk, distances behind them,
// written by the expand phase of the same workgroup), the loop state has been checked, and
// the row's queues, visited list, popped ids and exclusions have been placed in LDS by
// stage_row (the global reads were issued at the start of the kernel).
// refine (fused step only): called once the visited list is current and before the candidates are
// looked at, with the last slots of both queues; it may replace candidate distances that are only known
// as bounds by exact ones and drop candidates that provably cannot enter a queue.
struct NoRefine {
    __device__ __forceinline__ void operator()(const int32_t *, int, bool, uint64_t, uint64_t, uint8_t *, uint64_t *) const {}
};

// RESIDENT (a workgroup that takes its row through several iterations, beam_window_body): the row's queues and
// visited list stay in LDS between iterations.  The merge phase reads them where this says and writes the merged
// queues to the *_out arrays instead of memory; nothing of the row goes to memory here.
struct ResidentRow {
    uint64_t *qa, *qa_out;    // search queue [0, L) as keys
    uint64_t *va, *va_out;    // visit queue, all VL slots (the popped heads first)
    int32_t *seen_a, *seen_b; // visited list before / after this iteration
    int32_t *exl;
    uint8_t *fl;
    int *quiet;               // per-query stop: the row's count of quiet iterations
};
struct MergeResult {
    int cnt;           // fill of the visited list after this iteration
    bool queue_moved;  // RESIDENT: the search queue was written to qa_out (else it is unchanged in qa)
};

// PREFILTERED: the caller has already dropped every candidate that the updated visited list holds.
template <int THREADS, bool FUSED, class Refine = NoRefine, bool RESIDENT = false, bool PREFILTERED = false>
__device__ __forceinline__ MergeResult merge_row(const MergeArgs &a, unsigned char *smem, RowState pre = RowState{0, 0},
                                                 Refine refine = Refine(), const ResidentRow *rr = nullptr) {
    static_assert(FUSED || !RESIDENT, "a resident row is a fused one");
    const int Pc = a.Pc;
    uint64_t *raw = reinterpret_cast<uint64_t *>(smem);  // candidate keys as they arrive
    uint64_t *uk = raw + Pc;                             // the candidates that can matter, then sorted
    uint64_t *cc = raw;                                  // filtered for one merge (raw is no longer needed by then)
    uint64_t *qa = RESIDENT ? rr->qa : uk + Pc;          // search queue [0, L)
    uint64_t *va = RESIDENT ? rr->va + a.Vt : qa + a.L;  // visit queue [Vt, VL)
    int32_t *seen_a = RESIDENT ? rr->seen_a : reinterpret_cast<int32_t *>(va + a.VL);
    int32_t *seen_b = RESIDENT ? rr->seen_b : seen_a + a.E;
    int32_t *exl = RESIDENT ? rr->exl : seen_b + a.E;
    uint8_t *fl = RESIDENT ? rr->fl : reinterpret_cast<uint8_t *>(exl + a.excl_cols);  // per candidate: bit0 wanted, bit1 rest
    __shared__ int wave_cnt[kQueueWaves];
    __shared__ uint64_t red[2 * kQueueWaves];
    int32_t *const newv = g_new_s;
    __shared__ int n_new_s;
    __shared__ int row_changed_s;  // per-query stop: some slot of the search queue's first L changed
    int &n_ex_s = g_n_ex_s;

    BeamCtrl *c = a.ctrl;
    const int t = a.iter;
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1);
    int32_t *qi = a.q_ids + row * a.cap;
    float *qd = a.q_d + row * a.cap;
    int32_t *vi = a.v_ids + row * a.VL;
    float *vd = a.v_d + row * a.VL;
    const int32_t *ci = a.cand_ids + row * a.m;
    const float *cd = a.cand_d + row * a.m;
    const int nva = a.VL - a.Vt;
    int *first_next = &c->first[(t + 1) % 3];

    const int stop = FUSED ? 0 : c->stop;
    const int first_prev = FUSED ? 0 : c->first[(t - 1) % 3];
    const int first = FUSED ? pre.first : c->first[t % 3];
    int cnt = FUSED ? pre.cnt : a.seen_count[row];
    // the ids popped at the start of this iteration (queue.py:87-95), before the row is rewritten
    int32_t popped = VL_MAXINT;
    if constexpr (FUSED) {
        if (threadIdx.x < kWave && (int)threadIdx.x < a.Vt) popped = g_visit_s[threadIdx.x];
        if (threadIdx.x == 0) {
            n_new_s = 0;
            row_changed_s = 0;
        }
    } else {
        // the visited list's fill is at most Vt ids per earlier iteration, so the row can be
        // fetched without first waiting for the exact count
        const int seen_bound = min(a.E, a.Vt * (t - 1));
        for (int i = threadIdx.x; i < a.m; i += blockDim.x) raw[i] = vl_make_key(ci[i], cd[i]);
        for (int i = threadIdx.x; i < a.L; i += blockDim.x) qa[i] = vl_make_key(qi[i], qd[i]);
        for (int i = threadIdx.x; i < nva; i += blockDim.x) va[i] = vl_make_key(vi[a.Vt + i], vd[a.Vt + i]);
        {
            const int32_t *srow = a.seen + row * a.E;
            for (int i = threadIdx.x; i < seen_bound; i += blockDim.x) seen_a[i] = srow[i];
        }
        if (threadIdx.x < kWave && (int)threadIdx.x < a.Vt) popped = vi[threadIdx.x];
        if (threadIdx.x == 0) {
            n_ex_s = a.excl ? a.excl_cols : 0;
            n_new_s = 0;
            row_changed_s = 0;
        }
        __syncthreads();
        if (a.excl) {
            const int32_t *ex = a.excl + row * a.excl_cols;
            for (int i = threadIdx.x; i < a.excl_cols; i += blockDim.x) {
                int32_t e = ex[i];
                exl[i] = e;
                if (e == VL_MAXINT) atomicMin(&n_ex_s, i);
            }
        }
    }
    if (stop) return MergeResult{cnt, false};
    if constexpr (!FUSED) {
        if (!beam_row_state_ok(c, cnt, min(a.E, a.Vt * (t - 1)), threadIdx.x == 0)) return MergeResult{0, false};
    }
    if (!FUSED && t >= 2 && first_prev >= a.E) {
        // the visit queue is no longer fed: every candidate of this iteration is empty
        if (threadIdx.x == 0) raise_running_max(first_next, cnt, min(a.E, a.Vt * t));
        return MergeResult{cnt, false};
    }
    const bool seen_full = first >= a.E;
    const bool checking = (t % a.readahead) == 0;
    __syncthreads();
    const int n_ex = n_ex_s;

    // ---- add_new_to_seen_ : utils.py:61-82 (does not depend on the candidates) ------
    if (!seen_full) {
        const int n_add = min(min(a.E - first, a.Vt), a.E - cnt);  // cnt <= first: rows are packed
        if (threadIdx.x < kWave) {
            const int j = threadIdx.x;
            int32_t x = j < n_add ? popped : VL_MAXINT;
            bool valid = j < n_add && x != VL_MAXINT && !sorted_contains(seen_a, cnt, x);
            for (int i = 0; i < n_add; ++i) {
                int32_t y = __shfl(popped, i);
                if (i < j && y == x) valid = false;
            }
            uint64_t vm = __ballot(valid);
            int rank = 0;
            for (int i = 0; i < n_add; ++i) {
                int32_t y = __shfl(popped, i);
                if (((vm >> i) & 1) && y < x) ++rank;
            }
            if (valid) newv[rank] = x;
            if (j == 0) n_new_s = __popcll(vm);
        }
        __syncthreads();
        const int n_new = n_new_s;
        for (int p = threadIdx.x; p < cnt; p += blockDim.x) {
            int32_t v = seen_a[p];
            int shift = 0;
            for (int i = 0; i < n_new; ++i) shift += newv[i] < v;
            seen_b[p + shift] = v;
        }
        if ((int)threadIdx.x < n_new)
            seen_b[lower_bound(seen_a, cnt, newv[threadIdx.x]) + threadIdx.x] = newv[threadIdx.x];
        __syncthreads();
        cnt += n_new;
        if constexpr (!RESIDENT) {
            if (n_new) {
                int32_t *srow = a.seen + row * a.E;
                for (int i = threadIdx.x; i < cnt; i += blockDim.x) srow[i] = seen_b[i];
            }
            if (threadIdx.x == 0 && n_new) a.seen_count[row] = cnt;
        }
    }
    if constexpr (!RESIDENT) {
        if (threadIdx.x == 0) raise_running_max(first_next, cnt, min(a.E, a.Vt * t));
    }
    if constexpr (FUSED) {
        refine(seen_b, cnt, seen_full, qa[a.L - 1], nva > 0 ? va[nva - 1] : 0ull, fl, red);
        // a thread packs the slots it (or a lane of its own wavefront, before the barrier above or in refine) wrote
        const int32_t *li = reinterpret_cast<const int32_t *>(uk);
        const float *ld = reinterpret_cast<const float *>(li + a.m);
        for (int i = threadIdx.x; i < a.m; i += blockDim.x) raw[i] = vl_make_key(li[i], ld[i]);
    }

    // ---- which candidates can matter at all -------------------------------------------
    // search queue: only keys below its last slot can enter.  visit queue (VL slots, Vt of
    // them just freed): every unvisited key below its last live slot, plus the Vt best
    // distinct unvisited keys above it.  Everything else is dropped before the sort.  What is
    // chosen here may be a superset - the merges below are exact and cut by rank - so the keys
    // above the visit queue's last slot ("rest") are looked up in the visited list only when
    // they come up as one of the smallest.
    const uint64_t ws = qa[a.L - 1];
    const uint64_t wv = nva > 0 ? va[nva - 1] : 0ull;
    for (int i = threadIdx.x; i < a.m; i += blockDim.x) {
        uint64_t k = raw[i];
        int32_t id = vl_key_id(k);
        uint8_t f = 0;
        if (id != VL_MAXINT) {
            if (k < ws) f |= 1;
            if (!seen_full && k != wv) {  // k == wv is the visit queue's own last slot again
                bool unseen = PREFILTERED || !sorted_contains(seen_b, cnt, id);
                if (unseen) f |= (k < wv) ? 1 : 2;
            }
        }
        fl[i] = f;
    }
    // The Vt smallest distinct keys among the "rest" candidates are found by their distances alone (the high
    // word of a key): Vt rounds of a workgroup-wide minimum over 32-bit words give the Vt smallest distinct
    // distances, and every "rest" candidate at or below the last of them is taken - the same candidates, plus
    // others of equal distance when there are ties, which the merges below cut by rank.
    uint32_t sel_max = 0u;  // largest selected distance word among the "rest" candidates
    bool any_rest = false;
    if (!seen_full) {
        uint32_t *red32 = reinterpret_cast<uint32_t *>(red);
        uint32_t last = 0u;
        for (int r = 0; r < a.Vt; ++r) {
            uint32_t mine = 0xFFFFFFFFu;
            for (int i = threadIdx.x; i < a.m; i += blockDim.x) {
                const uint32_t k = (uint32_t)(raw[i] >> 32);
                if ((fl[i] & 2) && (r == 0 || k > last) && k < mine) mine = k;
            }
            const uint32_t mn = block_min_u32(mine, red32, r);
            if (mn == 0xFFFFFFFFu) break;
            last = mn;
            sel_max = mn;
            any_rest = true;
        }
    }
    __syncthreads();
    auto wanted = [&](int i) -> bool {
        uint8_t f = fl[i];
        return (f & 1) || (any_rest && (f & 2) && (uint32_t)(raw[i] >> 32) <= sel_max);
    };
    const int n_u = block_compact(raw, a.m, uk, wanted, wave_cnt);
    int Pu = 2;
    while (Pu < n_u) Pu <<= 1;
    for (int i = n_u + threadIdx.x; i < Pu; i += blockDim.x) uk[i] = kPadKey;
    block_bitonic_sort(uk, Pu);

    // ---- search_queue.insert : ann.py:75-80 -------------------------------------------
    auto keep_search = [&](int i) -> bool {
        uint64_t k = uk[i];
        int32_t id = vl_key_id(k);
        if (i > 0 && id == vl_key_id(uk[i - 1])) return false;   // neighbouring duplicate (kernels.py:314-349)
        if (!(k < ws)) return false;
        for (int e = 0; e < n_ex; ++e)
            if (exl[e] == id) return false;                      // queue.py:52-53
        int p = key_lower_bound(qa, a.L, k);
        return !(p < a.L && qa[p] == k);                         // already queued
    };
    const int n_s = block_compact(uk, n_u, cc, keep_search, wave_cnt);
    bool diff = false;
    if (n_s) {
        for (int i = threadIdx.x; i < a.L; i += blockDim.x) {
            uint64_t k = qa[i];
            int r = i + key_lower_bound(cc, n_s, k);
            if constexpr (RESIDENT) {
                if (r < a.L) rr->qa_out[r] = k;
            } else if (r != i && r < a.L) {
                qi[r] = vl_key_id(k);
                qd[r] = vl_key_dist(k);
            }
        }
        for (int j = threadIdx.x; j < n_s; j += blockDim.x) {
            uint64_t k = cc[j];
            int r = j + key_lower_bound(qa, a.L, k);
            if (r < a.L) {
                if constexpr (RESIDENT) {
                    rr->qa_out[r] = k;
                } else {
                    qi[r] = vl_key_id(k);
                    qd[r] = vl_key_dist(k);
                }
                diff = true;  // a new id inside the first L slots: the row changed (queue.py:57-59)
            }
        }
    }
    int *flag = &c->changed[(t / a.readahead) & 63];  // every writer stores the same 1: no atomic needed
    if (a.row_quiet) {
        // Per-query stop: a row is finished after `readahead` iterations in a row that left its first L
        // slots as they were, or when the visited list has no free column (no pop yields a real id from
        // then on); a row that is not finished at a checking iteration keeps the loop going.
        if (diff) row_changed_s = 1;  // every writer stores the same 1
        __syncthreads();
        if (threadIdx.x == 0) {
            int quiet = row_changed_s ? 0 : (RESIDENT ? *rr->quiet : a.row_quiet[row]) + 1;
            if (seen_full) quiet = a.readahead;
            if constexpr (RESIDENT) *rr->quiet = quiet;
            else a.row_quiet[row] = quiet;
            if (checking && quiet < a.readahead &&
                __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
                __hip_atomic_store(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else if (checking && __ballot(diff) && lane == 0) {
        if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
            __hip_atomic_store(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (seen_full) return MergeResult{cnt, n_s > 0};
    __syncthreads();  // cc is reused below

    // ---- visit_queue.insert(candidates, exclude=seen) : ann.py:85-88 --------------------
    auto keep_visit = [&](int i) -> bool {
        uint64_t k = uk[i];
        int32_t id = vl_key_id(k);
        if (i > 0 && id == vl_key_id(uk[i - 1])) return false;
        if (!PREFILTERED && sorted_contains(seen_b, cnt, id)) return false;      // kernels.py:471-488
        int p = key_lower_bound(va, nva, k);
        return !(p < nva && va[p] == k);
    };
    const int n_v = block_compact(uk, n_u, cc, keep_visit, wave_cnt);
    for (int i = threadIdx.x; i < nva; i += blockDim.x) {
        uint64_t k = va[i];
        int r = i + key_lower_bound(cc, n_v, k);
        if (r < a.VL) {
            if constexpr (RESIDENT) {
                rr->va_out[r] = k;
            } else {
                vi[r] = vl_key_id(k);
                vd[r] = vl_key_dist(k);
            }
        }
    }
    for (int j = threadIdx.x; j < n_v; j += blockDim.x) {
        uint64_t k = cc[j];
        int r = j + key_lower_bound(va, nva, k);
        if (r < a.VL) {
            if constexpr (RESIDENT) {
                rr->va_out[r] = k;
            } else {
                vi[r] = vl_key_id(k);
                vd[r] = vl_key_dist(k);
            }
        }
    }
    for (int r = nva + n_v + threadIdx.x; r < a.VL; r += blockDim.x) {  // the popped slots end up here, empty
        if constexpr (RESIDENT) {
            rr->va_out[r] = vl_make_key(VL_MAXINT, VL_MAXFLOAT);
        } else {
            vi[r] = VL_MAXINT;
            vd[r] = VL_MAXFLOAT;
        }
    }
    return MergeResult{cnt, n_s > 0};
}

template <int THREADS>
__global__ __launch_bounds__(THREADS) void beam_merge2_kernel(MergeArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    merge_row<THREADS, false>(a, smem);
}

// ---- one launch per iteration -------------------------------------------------
// The expand phase (HBM bound) and the merge phase (LDS / latency bound) of one
// row run in the same workgroup, so on every CU some workgroups stream candidate
// rows while others merge: the merge time hides behind the memory traffic, the
// candidate ids and distances never leave LDS, and an iteration is one launch.
struct StepArgs {
    MergeArgs m;
    const float *queries;
    const float *vectors;
    const int32_t *beams;
    int64_t n_vectors;
    int dim, nchunks, width;
    uint32_t width_magic;  // floor(2^32 / width) + 1: slot / width == umulhi(slot, width_magic) for slot * width < 2^32
    uint64_t *memo;
    int memo_shift;
    int32_t *memo_rate;   // per row: share (x 256) of the candidates of iteration kMemoDecide that were cached; bit 16: the row uses the sketch
    int memo_min_rate;    // the cache stays in use only if that share is at least this (x 256)
    int count_evals;
    int l2;  // 0: cosine distance, 1: squared L2
    const uint8_t *sketch;     // 8-bit sketch of `vectors` (sketch_device.h), or null
    const uint8_t *sketch_tails;  // the table's second part: 8 bytes per vector
    int sketch_chunks;         // 16-byte chunks of data in a sketch row
    const uint8_t *rounded_queries;  // the call's query rows rounded for the sketch (sketch_device.h)
    int64_t rounded_query_bytes;
    int window;     // beam_window_kernel: iterations m.iter ... m.iter + window - 1 in this launch
    int lds_slots;  // beam_window_kernel: entries of the row's distance table in LDS (a power of two, or 0)
};

// A probe of the distance cache is a random 8-byte read and every evaluated distance a random 8-byte
// write - a memory sector each, and one more round trip before the candidate rows can be asked for - so
// the cache only pays when enough probes hit; how many depends on the row size (short rows are cheap to
// fetch again).  Each row therefore decides for itself: it uses the cache during its first kMemoDecide - 1
// iterations, measures the share of hits in iteration kMemoDecide, and leaves the cache alone for the rest
// of the call if that share is below the break-even share.  A hit returns the bits that would be computed
// again, so the decision never changes a result.
constexpr int kMemoDecide = 9;

// Elements of a row that one thread brings in at the start of the fused step and keeps in registers until
// the workgroup's other reads have been issued: search queue, visit queue, visited list.  Longer rows load
// their remainder the slow way (read, wait, store) - none of the benchmark shapes has one.
constexpr int kPreQ = 2, kPreV = 2, kPreS = 4;

// SCPL > 0: the kernel can look at candidates through the sketch first (SCPL chunks per lane, SLPR lanes
// per sketch row, SU loads in flight).  A row that does so gets bounds for the candidates the distance cache
// does not know from a quarter of the bytes, then exact distances for the few whose lower bound is not above
// every threshold that decides what the merge phase keeps; it stops doing so when most of them turn out to
// need their exact distance (bit 16 of its word in memo_rate: set at the start of the call, cleared then).
template <int CPL, int LPR, int U, bool GENERIC, int THREADS, int SCPL = 0, int SLPR = 64, int SU = 1>
__device__ __forceinline__ void beam_step_body(const StepArgs &s) {
    extern __shared__ __align__(16) unsigned char smem[];
    const MergeArgs &a = s.m;
    BeamCtrl *c = a.ctrl;
    const int t = a.iter;
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    // ---- every read that depends on nothing else goes out first: loop state, the row's counters, the ids
    // to visit, both queues, the visited list, the exclusions.  A round trip to memory costs more than
    // anything this workgroup computes, so the number of dependent round trips is what it pays for: this
    // one, then the neighbour lists of the visited ids, the cache probes, the candidate rows.
    int32_t *vi = a.v_ids + row * a.VL;
    float *vd = a.v_d + row * a.VL;
    const int32_t *qi = a.q_ids + row * a.cap;
    const float *qd = a.q_d + row * a.cap;
    const int32_t *srow = a.seen + row * a.E;
    const int nva = a.VL - a.Vt;
    const int seen_bound = min(a.E, a.Vt * (t - 1));  // the fill is at most Vt ids per earlier iteration
    const int32_t my_visit = tid < a.Vt ? vi[tid] : VL_MAXINT;
    RowState pre;
    pre.cnt = a.seen_count[row];
    pre.first = c->first[t % 3];
    const int quiet = a.row_quiet ? a.row_quiet[row] : 0;
    const int memo_word = s.memo_rate[row];
    const int memo_rate = memo_word & 0xffff;
    int32_t pq_i[kPreQ], pv_i[kPreV], ps[kPreS];
    float pq_d[kPreQ], pv_d[kPreV];
#pragma unroll
    for (int j = 0; j < kPreQ; ++j) {
        const int i = tid + j * THREADS;
        pq_i[j] = i < a.L ? qi[i] : VL_MAXINT;
        pq_d[j] = i < a.L ? qd[i] : VL_MAXFLOAT;
    }
#pragma unroll
    for (int j = 0; j < kPreV; ++j) {
        const int i = tid + j * THREADS;
        pv_i[j] = i < nva ? vi[a.Vt + i] : VL_MAXINT;
        pv_d[j] = i < nva ? vd[a.Vt + i] : VL_MAXFLOAT;
    }
#pragma unroll
    for (int j = 0; j < kPreS; ++j) {
        const int i = tid + j * THREADS;
        ps[j] = i < seen_bound ? srow[i] : VL_MAXINT;
    }
    int32_t my_excl = VL_MAXINT;
    if (a.excl && tid < a.excl_cols) my_excl = a.excl[row * a.excl_cols + tid];

    const int gate = beam_gate(c, t, a.readahead, a.E, blockIdx.x == 0 && tid == 0);
    if (gate == 2) return;
    if (!beam_row_state_ok(c, pre.cnt, seen_bound, tid == 0)) return;
    if (gate == 1 || (a.row_quiet && quiet >= a.readahead)) {
        // the visit queue is no longer fed (every candidate of this iteration is empty), or this row has
        // stopped on its own: nothing changes, only the running maximum is kept current
        if (tid == 0) raise_running_max(&c->first[(t + 1) % 3], pre.cnt, min(a.E, a.Vt * t));
        return;
    }
    uint64_t *raw = reinterpret_cast<uint64_t *>(smem);
    uint64_t *uk = raw + a.Pc;
    uint64_t *qa = uk + a.Pc;
    uint64_t *va = qa + a.L;
    int32_t *seen_a = reinterpret_cast<int32_t *>(va + a.VL);
    int32_t *exl = seen_a + 2 * a.E;
    int32_t *li = reinterpret_cast<int32_t *>(uk);
    float *ld = reinterpret_cast<float *>(li + a.m);
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const float *q_row = s.queries + row * s.dim;
    uint64_t *memo_row = s.memo ? s.memo + ((uint64_t)row << (32 - s.memo_shift)) : nullptr;
    __shared__ int probe_hits_s, probe_asked_s;
    uint8_t *const lane_order_s = reinterpret_cast<uint8_t *>(g_new_s);  // 64 bytes per wavefront (see g_new_s)
    const bool resample = memo_row && t == kMemoDecide;
    if (memo_row && memo_rate < s.memo_min_rate) memo_row = nullptr;
    bool sketching = false;
    // (not in the first iteration: the visit queue starts with empty slots, so everything unvisited is kept and
    // would be fetched anyway)
    if constexpr (SCPL > 0) sketching = (memo_word >> 16) != 0 && t > 1;
    const bool probing = memo_row != nullptr;
    if (tid < a.Vt) g_visit_s[tid] = my_visit;
    if (tid == 0) {
        g_n_ex_s = a.excl ? a.excl_cols : 0;
        probe_hits_s = 0;
        probe_asked_s = 0;
    }
    // The neighbour lists of the nodes visited in one iteration share ids; only one copy of an id is evaluated.
    // Every candidate claims its id in a hash set in LDS (the second copy of the visited list, which the merge
    // phase fills only later: E slots, each the slot number of the claiming candidate; used when that leaves the
    // set at most two thirds full); a candidate that finds its id claimed becomes the empty pair before anything
    // is asked of memory for it.  The reference evaluates every copy (kernels.py:238-255) and drops all but one
    // when the queues are sorted (kernels.py:314-349): copies carry the same distance, so what the queues receive
    // is the same.
    int32_t *const dset = seen_a + a.E;
    const uint32_t dsize = (uint32_t)a.E;
    const bool dedup = 2 * a.E >= 3 * a.m;
    if (dedup)
        for (int i = tid; i < a.E; i += THREADS) dset[i] = -1;
    __syncthreads();

    // ---- expand: ann.py:69-73 (pop the visit heads, gather their neighbour lists, distances) ----
    // candidate id of slot c0 + lane: the neighbour list of a visited node
    auto resolve = [&](int c0) -> int32_t {
        const int slot = c0 + lane;
        int32_t id = VL_MAXINT;
        if (slot < a.m) {
            int sidx = s.width == 1 ? slot : (int)__umulhi((uint32_t)slot, s.width_magic), k = slot - sidx * s.width;
            int32_t node = g_visit_s[sidx];
            if (node != VL_MAXINT && (uint32_t)node < (uint64_t)s.n_vectors) id = s.beams[(int64_t)node * s.width + k];
        }
        return id;
    };
    int32_t id = resolve(wave * kWave);
    // The row's own state, read at the top, goes to LDS now that the first neighbour lists are on their
    // way.  (Outside the loop below on purpose: inside it, its addresses would be kept in registers across
    // the distance code.)
    {
#pragma unroll
        for (int j = 0; j < kPreQ; ++j) {
            const int i = tid + j * THREADS;
            if (i < a.L) qa[i] = vl_make_key(pq_i[j], pq_d[j]);
        }
#pragma unroll
        for (int j = 0; j < kPreV; ++j) {
            const int i = tid + j * THREADS;
            if (i < nva) va[i] = vl_make_key(pv_i[j], pv_d[j]);
        }
#pragma unroll
        for (int j = 0; j < kPreS; ++j) {
            const int i = tid + j * THREADS;
            if (i < seen_bound) seen_a[i] = ps[j];
        }
        if (a.excl && tid < a.excl_cols) {
            exl[tid] = my_excl;
            if (my_excl == VL_MAXINT) atomicMin(&g_n_ex_s, tid);
        }
        for (int i = tid + kPreQ * THREADS; i < a.L; i += THREADS) qa[i] = vl_make_key(qi[i], qd[i]);
        for (int i = tid + kPreV * THREADS; i < nva; i += THREADS) va[i] = vl_make_key(vi[a.Vt + i], vd[a.Vt + i]);
        for (int i = tid + kPreS * THREADS; i < seen_bound; i += THREADS) seen_a[i] = srow[i];
        for (int i = tid + THREADS; i < a.excl_cols; i += THREADS) {
            int32_t e = a.excl[row * a.excl_cols + i];
            exl[i] = e;
            if (e == VL_MAXINT) atomicMin(&g_n_ex_s, i);
        }
    }
    int n_wanted = 0, n_fetched = 0, n_sketched = 0;  // counts of this wavefront
    float *le = reinterpret_cast<float *>(raw);                     // upper bounds (raw is filled in the merge phase)
    uint8_t *xf = reinterpret_cast<uint8_t *>(exl + a.excl_cols);   // the merge phase's per-candidate flags; 16 = exact
    // A candidate that the visited list holds once this iteration has updated it - an id visited earlier, or one
    // popped now that the list still has room for (utils.py:73-75) - can change neither queue: the visit queue
    // excludes it (ann.py:85-88), and the search queue met it with this very distance when it was first a candidate
    // (every visited id came out of the visit queue, which is fed from the search queue's heads and then with the
    // candidates the search queue is offered in the same iteration, ann.py:75-88), so it either still sits there
    // or lies beyond its last slot, which only ever moves down.  Such candidates become the empty pair here,
    // before a probe or a row is spent on them, and the merge phase knows the others to be unvisited.
    const int n_popped_kept = pre.first >= a.E ? 0 : min(min(a.E - pre.first, a.Vt), a.E - pre.cnt);
    __syncthreads();  // the visited list is in LDS
    // first pass over this wavefront's candidates: ids to LDS, visited ids and later copies of an id out
    for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
        if (c0 != wave * kWave) id = resolve(c0);
        const int slot = c0 + lane;
        const bool has = slot < a.m;
        bool ok = has && id != VL_MAXINT && id >= 0 && (int64_t)id < s.n_vectors;
        if (s.count_evals || resample) n_wanted += __popcll(__ballot(ok));
        if (ok) {
            bool visited = sorted_contains(seen_a, pre.cnt, id);
            for (int j = 0; j < n_popped_kept; ++j) visited |= g_visit_s[j] == id;
            ok = !visited;
        }
        if (has) li[slot] = ok ? id : VL_MAXINT;  // (before the claim: a candidate that meets this one in the set reads it)
        if (ok && dedup) {
            uint32_t h = __umulhi((uint32_t)id * 2654435761u, dsize);
            for (;;) {
                const int owner = atomicCAS(&dset[h], -1, slot);
                if (owner == -1) break;     // first of its id
                if (li[owner] == id) {      // a copy: only the first is evaluated
                    ok = false;
                    break;
                }
                h = h + 1 == dsize ? 0 : h + 1;
            }
            if (!ok) li[slot] = VL_MAXINT;
        }
        if (has && !ok) ld[slot] = VL_MAXFLOAT;
    }
    if constexpr (SCPL > 0) {
        if (sketching) {
            SketchQuery<SCPL> sq;
            sketch_query_load<SCPL, SLPR>(sq, s.rounded_queries + row * s.rounded_query_bytes, s.sketch_chunks);
            for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
                const int slot = c0 + lane;
                const bool has = slot < a.m;
                id = has ? li[slot] : VL_MAXINT;
                bool ok = id != VL_MAXINT;
                if (has) xf[slot] = 0;
                // The cache serves two kinds of repeats: a candidate evaluated exactly before comes back with its
                // distance, one that was only bounded comes back with its bounds (dist_device.h) - either way
                // nothing is fetched for it now.
                if (probing && ok) {
                    const uint64_t e = memo_load(memo_row, s.memo_shift, id);
                    if ((int32_t)((uint32_t)e & ~kMemoBounds) == id) {
                        if ((uint32_t)e & kMemoBounds) {
                            ld[slot] = memo_bound_lo(e);
                            le[slot] = memo_bound_hi(e);
                        } else {
                            const float d = __builtin_bit_cast(float, (uint32_t)(e >> 32));
                            ld[slot] = d;
                            le[slot] = d;
                            xf[slot] = 16;  // exact already
                        }
                        ok = false;
                    }
                }
                if (s.count_evals || resample) n_sketched += __popcll(__ballot(ok));
                wave_sketch<SCPL, SLPR, SU>(sq, s.sketch, s.sketch_tails, s.sketch_chunks, id, ok, ld + c0, le + c0,
                                            lane_order_s + wave * kWave, memo_row, s.memo_shift);
            }
            n_fetched = n_sketched;  // for the share of cache hits: what the cache did not answer
        }
    }
    for (int c0 = wave * kWave; c0 < a.m && !sketching; c0 += THREADS) {
        const int slot = c0 + lane;
        const bool has = slot < a.m;
        id = has ? li[slot] : VL_MAXINT;
        bool ok = id != VL_MAXINT;
        if (probing && ok) {
            uint64_t e = memo_load(memo_row, s.memo_shift, id);
            if ((int32_t)(uint32_t)e == id) {
                ld[slot] = __builtin_bit_cast(float, (uint32_t)(e >> 32));
                ok = false;
            }
        }
        if (s.count_evals || resample) n_fetched += __popcll(__ballot(ok));
        if constexpr (GENERIC)
            wave_distances_generic(q_row, s.vectors, s.dim, s.nchunks, id, ok, ld + c0, memo_row, s.memo_shift, s.l2 != 0);
        else
            wave_distances_lds<CPL, LPR, U>(q_row, s.vectors, s.dim, s.nchunks, id, ok, ld + c0, lane_order_s + wave * kWave,
                                            memo_row, s.memo_shift, s.l2 != 0);
    }
    if (s.count_evals && lane == 0) {
        const int stripe = (int)((blockIdx.x * (THREADS / kWave) + wave) & (kBeamStripes - 1));
        if (n_wanted) atomicAdd(&c->wanted[stripe], (unsigned long long)n_wanted);
        if (n_fetched && !sketching) atomicAdd(&c->evals[stripe], (unsigned long long)n_fetched);
        if (n_sketched) atomicAdd(&c->sketched[stripe], (unsigned long long)n_sketched);
    }
    if (resample && lane == 0) {
        atomicAdd(&probe_asked_s, n_wanted);
        atomicAdd(&probe_hits_s, n_wanted - n_fetched);
    }
    __syncthreads();
    if (resample && tid == 0)
        s.memo_rate[row] = (probe_asked_s > 0 ? (probe_hits_s * 256) / probe_asked_s : 256) | (memo_word & (1 << 16));
    // ---- merge: ann.py:75-88 ----
    if constexpr (SCPL > 0) {
        // A sketched row knows every candidate distance only as lo <= d <= hi (ld holds lo, le holds hi).
        // What the merge phase keeps of the candidates: keys below the search queue's last slot (ws),
        // unvisited keys below the visit queue's last live slot (wv), and the Vt smallest distinct
        // unvisited keys above wv.  Take any Vt distinct unvisited candidates that are certainly above wv
        // (lo > wv) - those with the smallest hi, the likely winners - evaluate them, and let tv be the
        // largest of their distances: Vt candidates are then known to be at most tv, so a candidate with
        // lo > tv is not one of the Vt smallest.  Hence a candidate whose lo is above ws, and which is
        // visited or has lo above both wv and tv, cannot enter either queue and is dropped; all others are
        // evaluated exactly, by the same code and in the same order as an unsketched row's, in two rounds
        // (the second one needs tv).  Comparisons are written so that a NaN bound counts as "evaluate".
        auto refine = [&](const int32_t *seen_b, int cnt, bool seen_full, uint64_t ws, uint64_t wv, uint8_t *flags,
                          uint64_t *red) {
            if (!sketching) return;  // uniform over the workgroup
            const float ws_d = vl_key_dist(ws);
            const float wv_d = nva > 0 ? vl_key_dist(wv) : -1.0f;
            for (int i = tid; i < a.m; i += THREADS) {
                const int32_t cid = li[i];
                uint8_t f = flags[i] & 16;  // set by the expand phase for a distance that came from the cache
                if (cid != VL_MAXINT) {
                    const float lo = ld[i];
                    bool need = !(lo > ws_d);
                    if (!seen_full) {  // (every candidate left is unvisited)
                        if (!(lo > wv_d)) need = true;
                        else f |= 2;  // unvisited and certainly above the visit queue's last live slot
                    }
                    if (need) f |= 4;
                }
                flags[i] = f;
            }
            // The Vt candidates of distinct ids with the smallest upper bounds among those certainly above wv
            // (bit 8), found one block-wide minimum at a time; fewer than Vt of them: every one may be taken.
            // Every copy of a chosen id is marked - copies may carry different bounds (one fresh from the sketch,
            // one decoded from the cache) and must not count twice.
            bool all_rest = false;
            if (!seen_full) {
                for (int r = 0; r < a.Vt; ++r) {
                    uint32_t mine = 0xFFFFFFFFu;
                    for (int i = tid; i < a.m; i += THREADS) {
                        if ((flags[i] & (2 | 8)) != 2) continue;
                        const uint32_t k = bound_slot_key(le[i], i);
                        if (k < mine) mine = k;
                    }
                    const uint32_t mn = block_min_u32(mine, reinterpret_cast<uint32_t *>(red), r);
                    if (mn == 0xFFFFFFFFu) {
                        all_rest = true;
                        break;
                    }
                    const int32_t chosen = li[mn & (kMaxCandidates - 1)];
                    for (int i = tid; i < a.m; i += THREADS)
                        if ((flags[i] & 2) && li[i] == chosen) flags[i] |= 8;
                }
            }
            int n_exact = 0, n_real = 0;
            // first round: everything below a queue's last slot, and those Vt candidates
            for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
                const int slot = c0 + lane;
                const bool has = slot < a.m;
                const int32_t cid = has ? li[slot] : VL_MAXINT;
                const uint8_t f = has ? flags[slot] : 0;
                const bool ok = ((f & (4 | 8)) || (all_rest && (f & 2))) && !(f & 16);
                if (ok) flags[slot] = f | 16;  // its distance is exact from here on
                n_exact += __popcll(__ballot(ok));
                n_real += __popcll(__ballot(cid != VL_MAXINT && !(f & 16)));  // candidates known by bounds only
                wave_distances_lds<CPL, LPR, U>(q_row, s.vectors, s.dim, s.nchunks, cid, ok, ld + c0,
                                                lane_order_s + wave * kWave, memo_row, s.memo_shift, false);
            }
            __syncthreads();
            // tv: the largest exact distance of those Vt candidates.  Vt distinct unvisited candidates above wv
            // are at most tv, so a candidate whose lower bound is above tv is not one of the Vt smallest.
            float tv = -1.0f;
            if (!seen_full && !all_rest) {
                uint32_t mine = 0xFFFFFFFFu;  // (no distance has the key 0)
                for (int i = tid; i < a.m; i += THREADS)
                    if (flags[i] & 8) {
                        const uint32_t k = ~vl_float_key(ld[i]);
                        mine = k < mine ? k : mine;
                    }
                const uint32_t mn = block_min_u32(mine, reinterpret_cast<uint32_t *>(red), a.Vt);
                tv = mn == 0xFFFFFFFFu ? -1.0f : vl_key_float(~mn);
            }
            // second round: the candidates above wv that may still be among the Vt smallest
            for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
                const int slot = c0 + lane;
                const bool has = slot < a.m;
                const int32_t cid = has ? li[slot] : VL_MAXINT;
                const uint8_t f = has ? flags[slot] : 0;
                const bool ok = (f & 2) && !(f & 16) && !(ld[slot] > tv);
                if (has && cid != VL_MAXINT && !ok && !(f & 16)) {
                    li[slot] = VL_MAXINT;
                    ld[slot] = VL_MAXFLOAT;
                }
                n_exact += __popcll(__ballot(ok));
                wave_distances_lds<CPL, LPR, U>(q_row, s.vectors, s.dim, s.nchunks, cid, ok, ld + c0,
                                                lane_order_s + wave * kWave, memo_row, s.memo_shift, false);
            }
            if (s.count_evals && lane == 0 && n_exact)
                atomicAdd(&c->evals[(int)((blockIdx.x * (THREADS / kWave) + wave) & (kBeamStripes - 1))],
                          (unsigned long long)n_exact);
            // A row that has to evaluate more than half of the candidates it knew by bounds exactly after all
            // (they lie within the sketch's error of the queues' last slots: real neighbour lists) gives the
            // sketch up for the rest of the call.  The first iterations fill the visit queue and keep a lot, so
            // until iteration kMemoDecide only a row that evaluates nearly all of them (7 in 8) does.
            if (t > 2 && !resample) {  // (the iteration that measures the cache uses the same two counters)
                if (lane == 0) {
                    atomicAdd(&probe_asked_s, n_real);
                    atomicAdd(&probe_hits_s, n_exact);
                }
                __syncthreads();
                const bool quit = t > kMemoDecide ? 2 * probe_hits_s > probe_asked_s : 8 * probe_hits_s > 7 * probe_asked_s;
                if (tid == 0 && quit) {
                    s.memo_rate[row] = memo_rate;
                    atomicAdd(&c->sketch_rows, -1);
                }
            } else {
                __syncthreads();
            }
        };
        merge_row<THREADS, true, decltype(refine), false, true>(a, smem, pre, refine);
    } else {
        merge_row<THREADS, true, NoRefine, false, true>(a, smem, pre);
    }
}

template <int CPL, int LPR, int U, bool GENERIC, int THREADS>
__global__ __launch_bounds__(THREADS) void beam_step_kernel(StepArgs s) {
    beam_step_body<CPL, LPR, U, GENERIC, THREADS>(s);
}
// The same kernel built to leave room for WPP wavefronts per SIMD.  Its vector registers would allow that anyway;
// what does not is its scalar registers (more than 96 of them mean seven wavefronts instead of eight), which the
// compiler keeps within bounds when asked, at the price of a few moves to and from lanes of a vector register.
template <int CPL, int LPR, int U, int THREADS, int WPP>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WPP)))
void beam_step_kernel_w(StepArgs s) {
    beam_step_body<CPL, LPR, U, false, THREADS>(s);
}

// ---- several iterations per launch ----------------------------------------------
// While parallel_visit_count * t <= E (the visited list's width) no row's visited list can be full at
// iteration t, so every row appends all the ids it pops (utils.py:73-75 with room for them in every row)
// and nothing one row does in iterations t0 ... t0 + W - 1 depends on another row of the batch; the only
// batch-wide facts, the progress flag of the checking iteration (ann.py:90-91) and the largest fill after
// the last of them, are written once.  One workgroup then takes its row through W = speculative_readahead
// iterations in one launch: search queue, visit queue and visited list are read once, stay in LDS (the merge
// phase writes the merged rows to a second set of arrays, which becomes the current one) and go back to
// memory once.  A small direct-mapped table in LDS keeps the (id, distance) or (id, bounds) entries the
// row met in these iterations, so a repeat inside the window costs an LDS read instead of a probe of the
// cache in memory.  Same candidates, same order, same merge code as beam_step_body: the rows are
// bit-identical.  The launch must start right after a progress check (t0 = k * readahead + 1, W = readahead).
template <int CPL, int LPR, int U, int THREADS, int SCPL = 0, int SLPR = 64, int SU = 1>
__device__ __forceinline__ void beam_window_body(const StepArgs &s) {
    extern __shared__ __align__(16) unsigned char smem[];
    MergeArgs a = s.m;
    BeamCtrl *c = a.ctrl;
    const int t0 = a.iter, W = s.window;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int64_t row = blockIdx.x;
    int32_t *vi = a.v_ids + row * a.VL;
    float *vd = a.v_d + row * a.VL;
    int32_t *qi = a.q_ids + row * a.cap;
    float *qd = a.q_d + row * a.cap;
    int32_t *srow = a.seen + row * a.E;
    const int nva = a.VL - a.Vt;
    const int seen_bound = min(a.E, a.Vt * (t0 - 1));  // the fill is at most Vt ids per earlier iteration
    // ---- every read that depends on nothing else goes out first (as in beam_step_body)
    const int32_t my_visit = tid < a.Vt ? vi[tid] : VL_MAXINT;
    int cnt = a.seen_count[row];
    const int quiet0 = a.row_quiet ? a.row_quiet[row] : 0;
    const int memo_word0 = s.memo_rate[row];
    int32_t pq_i[kPreQ], pv_i[kPreV], ps[kPreS];
    float pq_d[kPreQ], pv_d[kPreV];
#pragma unroll
    for (int j = 0; j < kPreQ; ++j) {
        const int i = tid + j * THREADS;
        pq_i[j] = i < a.L ? qi[i] : VL_MAXINT;
        pq_d[j] = i < a.L ? qd[i] : VL_MAXFLOAT;
    }
#pragma unroll
    for (int j = 0; j < kPreV; ++j) {
        const int i = tid + j * THREADS;
        pv_i[j] = i < a.VL ? vi[i] : VL_MAXINT;
        pv_d[j] = i < a.VL ? vd[i] : VL_MAXFLOAT;
    }
#pragma unroll
    for (int j = 0; j < kPreS; ++j) {
        const int i = tid + j * THREADS;
        ps[j] = i < seen_bound ? srow[i] : VL_MAXINT;
    }
    int32_t my_excl = VL_MAXINT;
    if (a.excl && tid < a.excl_cols) my_excl = a.excl[row * a.excl_cols + tid];

    // (the visited lists cannot be full in these iterations; the slots of `first` are not read here, because rows
    // of this very launch that finish early write the one the next launch reads)
    const int gate = beam_gate(c, t0, a.readahead, a.E, blockIdx.x == 0 && tid == 0, false);
    if (gate == 2) return;
    if (!beam_row_state_ok(c, cnt, seen_bound, tid == 0)) return;
    int *first_after = &c->first[(t0 + W) % 3];  // what the launch of iteration t0 + W reads
    const int bound_after = min(a.E, a.Vt * (t0 + W - 1));
    if (a.row_quiet && quiet0 >= a.readahead) {
        // this row has stopped on its own: nothing changes, only the running maximum is kept current
        if (tid == 0) raise_running_max(first_after, cnt, bound_after);
        return;
    }
    const int Pc = a.Pc;
    uint64_t *raw = reinterpret_cast<uint64_t *>(smem);
    uint64_t *uk = raw + Pc;
    // two copies of each queue and of the visited list, the second right behind the first
    uint64_t *const q0 = uk + Pc;
    uint64_t *const v0 = q0 + 2 * a.L;
    auto qbuf = [&](int k) -> uint64_t * { return q0 + k * a.L; };
    auto vbuf = [&](int k) -> uint64_t * { return v0 + k * a.VL; };
    LdsMemo lds;
    lds.tab = s.lds_slots > 0 ? v0 + 2 * a.VL : nullptr;
    lds.shift = 32 - (31 - __builtin_clz(s.lds_slots > 0 ? s.lds_slots : 1));
    int32_t *const s0 = reinterpret_cast<int32_t *>(v0 + 2 * a.VL + s.lds_slots);
    auto sbuf = [&](int k) -> int32_t * { return s0 + k * a.E; };
    int32_t *exl = s0 + 2 * a.E;
    const float *const q_row0 = s.queries + row * s.dim;
    const uint8_t *const rounded_row0 = s.rounded_queries + row * s.rounded_query_bytes;
    uint64_t *const memo_table = s.memo ? s.memo + ((uint64_t)row << (32 - s.memo_shift)) : nullptr;
    __shared__ int probe_hits_s, probe_asked_s, quiet_s, memo_word_s;
    uint8_t *const lane_order_s = reinterpret_cast<uint8_t *>(g_new_s);  // 64 bytes per wavefront (see g_new_s)
    int cur_q = 0, cur_v = 0, cur_s = 0;
    bool queue_dirty = false;

    // candidate id of slot c0 + lane: the neighbour list of a visited node
    auto resolve = [&](int c0) -> int32_t {
        const int slot = c0 + lane;
        int32_t id = VL_MAXINT;
        if (slot < a.m) {
            int sidx = s.width == 1 ? slot : (int)__umulhi((uint32_t)slot, s.width_magic), k = slot - sidx * s.width;
            int32_t node = g_visit_s[sidx];
            if (node != VL_MAXINT && (uint32_t)node < (uint64_t)s.n_vectors) id = s.beams[(int64_t)node * s.width + k];
        }
        return id;
    };
    if (tid < a.Vt) g_visit_s[tid] = my_visit;
    if (tid == 0) {
        g_n_ex_s = a.excl ? a.excl_cols : 0;
        quiet_s = quiet0;
        memo_word_s = memo_word0;
        probe_hits_s = 0;
        probe_asked_s = 0;
    }
    __syncthreads();
    int32_t id = resolve(wave * kWave);
    {
        // the row's state, read at the top, goes to LDS while the first neighbour lists are on their way
#pragma unroll
        for (int j = 0; j < kPreQ; ++j) {
            const int i = tid + j * THREADS;
            if (i < a.L) qbuf(0)[i] = vl_make_key(pq_i[j], pq_d[j]);
        }
#pragma unroll
        for (int j = 0; j < kPreV; ++j) {
            const int i = tid + j * THREADS;
            if (i < a.VL) vbuf(0)[i] = vl_make_key(pv_i[j], pv_d[j]);
        }
#pragma unroll
        for (int j = 0; j < kPreS; ++j) {
            const int i = tid + j * THREADS;
            if (i < seen_bound) sbuf(0)[i] = ps[j];
        }
        if (a.excl && tid < a.excl_cols) {
            exl[tid] = my_excl;
            if (my_excl == VL_MAXINT) atomicMin(&g_n_ex_s, tid);
        }
        for (int i = tid + kPreQ * THREADS; i < a.L; i += THREADS) qbuf(0)[i] = vl_make_key(qi[i], qd[i]);
        for (int i = tid + kPreV * THREADS; i < a.VL; i += THREADS) vbuf(0)[i] = vl_make_key(vi[i], vd[i]);
        for (int i = tid + kPreS * THREADS; i < seen_bound; i += THREADS) sbuf(0)[i] = srow[i];
        for (int i = tid + THREADS; i < a.excl_cols; i += THREADS) {
            int32_t e = a.excl[row * a.excl_cols + i];
            exl[i] = e;
            if (e == VL_MAXINT) atomicMin(&g_n_ex_s, i);
        }
        for (int i = tid; i < s.lds_slots; i += THREADS) lds.tab[i] = (uint64_t)(uint32_t)VL_MAXINT;  // no probe asks for it
        __syncthreads();  // the table is probed below
    }

    for (int w = 0; w < W; ++w) {
        const int t = t0 + w;
        a.iter = t;
        // The LDS addresses of an iteration are formed again from an offset the compiler cannot see through
        // (always 0): hoisted out of this loop, the per-thread addresses of every array below would occupy some
        // thirty registers through all of it, and cost a wavefront per SIMD.
        int z = 0;
        asm volatile("" : "+s"(z));
        unsigned char *const base = smem + z;
        uint64_t *const raw = reinterpret_cast<uint64_t *>(base);
        uint64_t *const uk = raw + Pc;
        uint64_t *const q0 = uk + Pc;
        uint64_t *const v0 = q0 + 2 * a.L;
        auto qbuf = [&](int k) -> uint64_t * { return q0 + k * a.L; };
        auto vbuf = [&](int k) -> uint64_t * { return v0 + k * a.VL; };
        LdsMemo lds;
        lds.tab = s.lds_slots > 0 ? v0 + 2 * a.VL : nullptr;
        lds.shift = 32 - (31 - __builtin_clz(s.lds_slots > 0 ? s.lds_slots : 1));
        int32_t *const s0 = reinterpret_cast<int32_t *>(v0 + 2 * a.VL + s.lds_slots);
        auto sbuf = [&](int k) -> int32_t * { return s0 + k * a.E; };
        int32_t *const exl = s0 + 2 * a.E;
        uint8_t *const xf = reinterpret_cast<uint8_t *>(exl + a.excl_cols);  // the merge phase's per-candidate flags; 16 = exact
        int32_t *const li = reinterpret_cast<int32_t *>(uk);                 // candidate ids, distances behind them
        float *const ld = reinterpret_cast<float *>(li + a.m);
        float *const le = reinterpret_cast<float *>(raw);                    // upper bounds (raw is filled in the merge phase)
        if (w > 0) {
            if (tid < a.Vt) g_visit_s[tid] = vl_key_id(vbuf(cur_v)[tid]);  // queue.py:87-95: the heads are popped
            if (tid == 0) {
                probe_hits_s = 0;
                probe_asked_s = 0;
            }
            __syncthreads();
            id = resolve(wave * kWave);
        }
        // The query row (and its rounded form) is read again in every iteration, as a launch per iteration
        // does: loaded once before the loop it would hold some forty registers through all of it, merge
        // phases included.  The empty asm hides from the compiler that the address is the same each time.
        const float *q_row = q_row0;
        const uint8_t *rounded_row = rounded_row0;
        asm volatile("" : "+s"(q_row), "+s"(rounded_row));
        const int memo_word = memo_word_s;
        const int memo_rate = memo_word & 0xffff;
        uint64_t *memo_row = memo_table;
        const bool resample = memo_row && t == kMemoDecide;
        if (memo_row && memo_rate < s.memo_min_rate) memo_row = nullptr;
        bool sketching = false;
        if constexpr (SCPL > 0) sketching = s.sketch != nullptr && (memo_word >> 16) != 0 && t > 1;
        const bool probing = memo_row != nullptr;

        // ---- expand: ann.py:69-73 ----
        int n_wanted = 0, n_fetched = 0, n_sketched = 0;  // counts of this wavefront
        // A candidate the row met before comes back from the LDS table or, failing that, from the cache in
        // memory: with its distance, or (rows that use the sketch) with its bounds.  Returns the entry or 0.
        auto probe = [&](int32_t cid, bool bounds_too) -> uint64_t {
            uint64_t e = 0;
            bool hit = false;
            if (lds.tab) {
                e = lds_memo_load(lds, cid);
                hit = (int32_t)((uint32_t)e & (bounds_too ? ~kMemoBounds : ~0u)) == cid;
            }
            if (!hit && probing) {
                e = memo_load(memo_row, s.memo_shift, cid);
                hit = (int32_t)((uint32_t)e & (bounds_too ? ~kMemoBounds : ~0u)) == cid;
                if (hit && lds.tab) lds_memo_store(lds, cid, e);
            }
            return hit ? e : 0ull;
        };
        if constexpr (SCPL > 0) {
            if (sketching) {
                SketchQuery<SCPL> sq;
                sketch_query_load<SCPL, SLPR>(sq, rounded_row, s.sketch_chunks);
                for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
                    if (c0 != wave * kWave) id = resolve(c0);
                    const int slot = c0 + lane;
                    const bool has = slot < a.m;
                    bool ok = has && id != VL_MAXINT && id >= 0 && (int64_t)id < s.n_vectors;
                    if (has) {
                        li[slot] = ok ? id : VL_MAXINT;
                        if (!ok) ld[slot] = VL_MAXFLOAT;
                        xf[slot] = 0;
                    }
                    if (s.count_evals || resample) n_wanted += __popcll(__ballot(ok));
                    if (ok) {
                        const uint64_t e = probe(id, true);
                        if (e) {  // (id 0 at distance 0 is the one entry that is all zeros: it reads as a miss and is evaluated again)
                            if ((uint32_t)e & kMemoBounds) {
                                ld[slot] = memo_bound_lo(e);
                                le[slot] = memo_bound_hi(e);
                            } else {
                                const float d = __builtin_bit_cast(float, (uint32_t)(e >> 32));
                                ld[slot] = d;
                                le[slot] = d;
                                xf[slot] = 16;  // exact already
                            }
                            ok = false;
                        }
                    }
                    if (s.count_evals || resample) n_sketched += __popcll(__ballot(ok));
                    wave_sketch<SCPL, SLPR, SU>(sq, s.sketch, s.sketch_tails, s.sketch_chunks, id, ok, ld + c0, le + c0,
                                                lane_order_s + wave * kWave, memo_row, s.memo_shift, lds);
                }
                n_fetched = n_sketched;  // for the share of cache hits: what the cache did not answer
            }
        }
        for (int c0 = wave * kWave; c0 < a.m && !sketching; c0 += THREADS) {
            if (c0 != wave * kWave) id = resolve(c0);
            const int slot = c0 + lane;
            const bool has = slot < a.m;
            bool ok = has && id != VL_MAXINT && id >= 0 && (int64_t)id < s.n_vectors;
            if (has) {
                li[slot] = ok ? id : VL_MAXINT;
                if (!ok) ld[slot] = VL_MAXFLOAT;
            }
            if (s.count_evals || resample) n_wanted += __popcll(__ballot(ok));
            if (ok) {
                const uint64_t e = probe(id, false);
                if (e) {
                    ld[slot] = __builtin_bit_cast(float, (uint32_t)(e >> 32));
                    ok = false;
                }
            }
            if (s.count_evals || resample) n_fetched += __popcll(__ballot(ok));
            wave_distances_lds<CPL, LPR, U>(q_row, s.vectors, s.dim, s.nchunks, id, ok, ld + c0, lane_order_s + wave * kWave,
                                            memo_row, s.memo_shift, s.l2 != 0, lds);
        }
        if (s.count_evals && lane == 0) {
            const int stripe = (int)((blockIdx.x * (THREADS / kWave) + wave) & (kBeamStripes - 1));
            if (n_wanted) atomicAdd(&c->wanted[stripe], (unsigned long long)n_wanted);
            if (n_fetched && !sketching) atomicAdd(&c->evals[stripe], (unsigned long long)n_fetched);
            if (n_sketched) atomicAdd(&c->sketched[stripe], (unsigned long long)n_sketched);
        }
        if (resample && lane == 0) {
            atomicAdd(&probe_asked_s, n_wanted);
            atomicAdd(&probe_hits_s, n_wanted - n_fetched);
        }
        __syncthreads();
        if (resample && tid == 0) {
            const int word = (probe_asked_s > 0 ? (probe_hits_s * 256) / probe_asked_s : 256) | (memo_word & (1 << 16));
            s.memo_rate[row] = word;
            memo_word_s = word;
        }
        // ---- merge: ann.py:75-88 ----
        ResidentRow rr;
        rr.qa = qbuf(cur_q); rr.qa_out = qbuf(cur_q ^ 1);
        rr.va = vbuf(cur_v); rr.va_out = vbuf(cur_v ^ 1);
        rr.seen_a = sbuf(cur_s); rr.seen_b = sbuf(cur_s ^ 1);
        rr.exl = exl; rr.fl = xf; rr.quiet = &quiet_s;
        const RowState pre{cnt, a.Vt * (t - 1)};  // every row has room for the Vt ids it pops (Vt * t <= E)
        MergeResult mr;
        if constexpr (SCPL > 0) {
            // the same rule as beam_step_body's refine (see there), with the row's LDS table kept current
            auto refine = [&](const int32_t *seen_b, int cnt_now, bool seen_full, uint64_t ws, uint64_t wv, uint8_t *flags,
                              uint64_t *red) {
                if (!sketching) return;  // uniform over the workgroup
                const float ws_d = vl_key_dist(ws);
                const float wv_d = nva > 0 ? vl_key_dist(wv) : -1.0f;
                for (int i = tid; i < a.m; i += THREADS) {
                    const int32_t cid = li[i];
                    uint8_t f = flags[i] & 16;
                    if (cid != VL_MAXINT) {
                        const float lo = ld[i];
                        bool need = !(lo > ws_d);
                        if (!seen_full && !sorted_contains(seen_b, cnt_now, cid)) {
                            if (!(lo > wv_d)) need = true;
                            else f |= 2;
                        }
                        if (need) f |= 4;
                    }
                    flags[i] = f;
                }
                bool all_rest = false;
                if (!seen_full) {
                    for (int r = 0; r < a.Vt; ++r) {
                        uint32_t mine = 0xFFFFFFFFu;
                        for (int i = tid; i < a.m; i += THREADS) {
                            if ((flags[i] & (2 | 8)) != 2) continue;
                            const uint32_t k = bound_slot_key(le[i], i);
                            if (k < mine) mine = k;
                        }
                        const uint32_t mn = block_min_u32(mine, reinterpret_cast<uint32_t *>(red), r);
                        if (mn == 0xFFFFFFFFu) {
                            all_rest = true;
                            break;
                        }
                        const int32_t chosen = li[mn & (kMaxCandidates - 1)];
                        for (int i = tid; i < a.m; i += THREADS)
                            if ((flags[i] & 2) && li[i] == chosen) flags[i] |= 8;
                    }
                }
                int n_exact = 0, n_real = 0;
                for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
                    const int slot = c0 + lane;
                    const bool has = slot < a.m;
                    const int32_t cid = has ? li[slot] : VL_MAXINT;
                    const uint8_t f = has ? flags[slot] : 0;
                    const bool ok = ((f & (4 | 8)) || (all_rest && (f & 2))) && !(f & 16);
                    if (ok) flags[slot] = f | 16;
                    n_exact += __popcll(__ballot(ok));
                    n_real += __popcll(__ballot(cid != VL_MAXINT && !(f & 16)));
                    wave_distances_lds<CPL, LPR, U>(q_row, s.vectors, s.dim, s.nchunks, cid, ok, ld + c0,
                                                    lane_order_s + wave * kWave, memo_row, s.memo_shift, false, lds);
                }
                __syncthreads();
                float tv = -1.0f;
                if (!seen_full && !all_rest) {
                    uint32_t mine = 0xFFFFFFFFu;  // (no distance has the key 0)
                    for (int i = tid; i < a.m; i += THREADS)
                        if (flags[i] & 8) {
                            const uint32_t k = ~vl_float_key(ld[i]);
                            mine = k < mine ? k : mine;
                        }
                    const uint32_t mn = block_min_u32(mine, reinterpret_cast<uint32_t *>(red), a.Vt);
                    tv = mn == 0xFFFFFFFFu ? -1.0f : vl_key_float(~mn);
                }
                for (int c0 = wave * kWave; c0 < a.m; c0 += THREADS) {
                    const int slot = c0 + lane;
                    const bool has = slot < a.m;
                    const int32_t cid = has ? li[slot] : VL_MAXINT;
                    const uint8_t f = has ? flags[slot] : 0;
                    const bool ok = (f & 2) && !(f & 16) && !(ld[slot] > tv);
                    if (has && cid != VL_MAXINT && !ok && !(f & 16)) {
                        li[slot] = VL_MAXINT;
                        ld[slot] = VL_MAXFLOAT;
                    }
                    n_exact += __popcll(__ballot(ok));
                    wave_distances_lds<CPL, LPR, U>(q_row, s.vectors, s.dim, s.nchunks, cid, ok, ld + c0,
                                                    lane_order_s + wave * kWave, memo_row, s.memo_shift, false, lds);
                }
                if (s.count_evals && lane == 0 && n_exact)
                    atomicAdd(&c->evals[(int)((blockIdx.x * (THREADS / kWave) + wave) & (kBeamStripes - 1))],
                              (unsigned long long)n_exact);
                if (t > 2 && !resample) {
                    if (lane == 0) {
                        atomicAdd(&probe_asked_s, n_real);
                        atomicAdd(&probe_hits_s, n_exact);
                    }
                    __syncthreads();
                    const bool quit = t > kMemoDecide ? 2 * probe_hits_s > probe_asked_s : 8 * probe_hits_s > 7 * probe_asked_s;
                    if (tid == 0 && quit) {
                        s.memo_rate[row] = memo_rate;
                        memo_word_s = memo_rate;
                        atomicAdd(&c->sketch_rows, -1);
                    }
                } else {
                    __syncthreads();
                }
            };
            mr = merge_row<THREADS, true, decltype(refine), true>(a, base, pre, refine, &rr);
        } else {
            mr = merge_row<THREADS, true, NoRefine, true>(a, base, pre, NoRefine(), &rr);
        }
        cnt = mr.cnt;
        if (mr.queue_moved) {
            cur_q ^= 1;
            queue_dirty = true;
        }
        cur_v ^= 1;
        cur_s ^= 1;
        __syncthreads();  // the merged rows are read below and by the next iteration
        if (a.row_quiet && quiet_s >= a.readahead) break;  // the row has stopped on its own (uniform)
    }
    // ---- the row goes back to memory once ----
    // (addresses formed afresh: kept from the loads at the top they would sit in registers, or in scratch memory,
    // through the whole loop)
    asm volatile("" : "+s"(qi), "+s"(qd), "+s"(vi), "+s"(vd), "+s"(srow));
    if (queue_dirty) {
        const uint64_t *qf = qbuf(cur_q);
        for (int i = tid; i < a.L; i += THREADS) {
            const uint64_t k = qf[i];
            qi[i] = vl_key_id(k);
            qd[i] = vl_key_dist(k);
        }
    }
    {
        const uint64_t *vf = vbuf(cur_v);
        for (int i = tid; i < a.VL; i += THREADS) {
            const uint64_t k = vf[i];
            vi[i] = vl_key_id(k);
            vd[i] = vl_key_dist(k);
        }
        const int32_t *sf = sbuf(cur_s);
        for (int i = tid; i < cnt; i += THREADS) srow[i] = sf[i];
    }
    if (tid == 0) {
        a.seen_count[row] = cnt;
        if (a.row_quiet) a.row_quiet[row] = quiet_s;
        raise_running_max(first_after, cnt, bound_after);
    }
}

// WPE: wavefronts per SIMD asked of the compiler.  The row's phases each wait on memory, so a launch is as fast
// as it has wavefronts to switch to: the registers are capped at what the one-iteration kernel of the same shape
// uses, and what the longer body holds beyond that (addresses for the write-back at the end, mostly) lives in
// scratch memory, stored once and read back rarely.
template <int CPL, int LPR, int U, int THREADS, int WPE>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WPE)))
void beam_window_kernel(StepArgs s) {
    beam_window_body<CPL, LPR, U, THREADS>(s);
}

template <int CPL, int LPR, int U, int THREADS, int SCPL, int SLPR, int SU, int WPE>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WPE)))
void beam_window_sketch_kernel(StepArgs s) {
    beam_window_body<CPL, LPR, U, THREADS, SCPL, SLPR, SU>(s);
}

// The same step for rows that may use the sketch.  WPE: wavefronts per SIMD the compiler is asked to leave room
// for.  The sketch's copy of the query row takes 16 registers per chunk and lane, and a row's phases (sketch
// pass, two rounds of exact rows, merge) each wait on memory, so residency is worth a few spilled registers:
// measured at 768 and 384 columns, five wavefronts per SIMD with two loads in flight beat three wavefronts
// with four (0.84 -> 0.75 ms and 0.61 -> 0.43 ms per launch).  Residency is what a launch that is not bound by
// memory traffic responds to (768 columns, state of the second optimisation loop, workgroups per compute unit
// limited through LDS: 4 / 5 / 6 -> 0.53 / 0.46 / 0.42 ms per launch; 8 with one load in flight and 62 registers:
// 0.415), which is also why the step's LDS arrays are overlaid where their lifetimes allow.
template <int CPL, int LPR, int U, int THREADS, int SCPL, int SLPR, int SU, int WPE>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WPE)))
void beam_step_sketch_kernel(StepArgs s) {
    beam_step_body<CPL, LPR, U, false, THREADS, SCPL, SLPR, SU>(s);
}

template <int CPL, int LPR, int U, bool GENERIC, int SCPL = 0, int SLPR = 64, int SU = 1, int WPE = 4, int UX = U,
          int WPW = WPE, int WPP = 0>
void launch_step(const StepArgs &s, int threads, size_t smem, hipStream_t st) {
    dim3 grid((unsigned)s.m.n_rows);
    if constexpr (SCPL > 0) {
        if (!s.sketch) return launch_step<CPL, LPR, U, GENERIC, 0, 64, 1, WPE, U, WPW, WPP>(s, threads, smem, st);
    }
    if constexpr (!GENERIC) {
        if (s.window > 0) {  // several iterations in this launch (smem is the window kernel's size)
            if constexpr (SCPL > 0) {
                if (threads == 128) {
                    auto kernel = beam_window_sketch_kernel<CPL, LPR, UX, 128, SCPL, SLPR, SU, WPW>;
                    if (vl_allow_lds(kernel, smem) != hipSuccess) return;  // seen by the launch check
                    hipLaunchKernelGGL(kernel, grid, dim3(128), smem, st, s);
                } else {
                    auto kernel = beam_window_sketch_kernel<CPL, LPR, UX, 256, SCPL, SLPR, SU, WPW>;
                    if (vl_allow_lds(kernel, smem) != hipSuccess) return;
                    hipLaunchKernelGGL(kernel, grid, dim3(256), smem, st, s);
                }
            } else if (threads == 128) {
                auto kernel = beam_window_kernel<CPL, LPR, U, 128, WPW>;
                if (vl_allow_lds(kernel, smem) != hipSuccess) return;
                hipLaunchKernelGGL(kernel, grid, dim3(128), smem, st, s);
            } else {
                auto kernel = beam_window_kernel<CPL, LPR, U, 256, WPW>;
                if (vl_allow_lds(kernel, smem) != hipSuccess) return;
                hipLaunchKernelGGL(kernel, grid, dim3(256), smem, st, s);
            }
            return;
        }
    }
    if constexpr (SCPL > 0) {
        if (threads == 128) {
            auto kernel = beam_step_sketch_kernel<CPL, LPR, UX, 128, SCPL, SLPR, SU, WPE>;
            if (vl_allow_lds(kernel, smem) != hipSuccess) return;  // seen by the launch check
            hipLaunchKernelGGL(kernel, grid, dim3(128), smem, st, s);
        } else {
            auto kernel = beam_step_sketch_kernel<CPL, LPR, UX, 256, SCPL, SLPR, SU, WPE>;
            if (vl_allow_lds(kernel, smem) != hipSuccess) return;
            hipLaunchKernelGGL(kernel, grid, dim3(256), smem, st, s);
        }
    } else if constexpr (WPP > 0 && !GENERIC) {
        if (threads == 128) {
            auto kernel = beam_step_kernel_w<CPL, LPR, U, 128, WPP>;
            if (vl_allow_lds(kernel, smem) != hipSuccess) return;
            hipLaunchKernelGGL(kernel, grid, dim3(128), smem, st, s);
        } else {
            auto kernel = beam_step_kernel_w<CPL, LPR, U, 256, WPP>;
            if (vl_allow_lds(kernel, smem) != hipSuccess) return;
            hipLaunchKernelGGL(kernel, grid, dim3(256), smem, st, s);
        }
    } else if (threads == 128) {
        auto kernel = beam_step_kernel<CPL, LPR, U, GENERIC, 128>;
        if (vl_allow_lds(kernel, smem) != hipSuccess) return;
        hipLaunchKernelGGL(kernel, grid, dim3(128), smem, st, s);
    } else {
        auto kernel = beam_step_kernel<CPL, LPR, U, GENERIC, 256>;
        if (vl_allow_lds(kernel, smem) != hipSuccess) return;
        hipLaunchKernelGGL(kernel, grid, dim3(256), smem, st, s);
    }
}

// VL_DIST_VARIANT (experiments only): 1 = two rows per load for rows of up to 512 bytes (32 lanes each) and
// one row per load for rows of up to 1536 bytes, the shapes used before lane groups of 16 / 32 took them over.
int dist_variant() {
    static const int v = [] {
        const char *e = getenv("VL_DIST_VARIANT");
        return e ? atoi(e) : 0;
    }();
    return v;
}

// The numbers after `false` are the sketch's lane shape for rows of that size (chunks per lane, lanes per row,
// loads in flight), the wavefronts per SIMD asked for, the whole rows in flight in the sketch kernel (it fetches
// few of them, so fewer in flight cost nothing and leave registers for another wavefront: 0.40 -> 0.36 ms per
// launch at 384 columns), where given, the wavefronts per SIMD asked for in the kernels that run several
// iterations per launch, and last the wavefronts per SIMD asked for in the kernel without the sketch
// (beam_step_kernel_w; 0 = the compiler's own choice, which is seven at most: the step holds 106 scalar registers).
// Eight wavefronts per SIMD - every workgroup slot a compute unit has - is what the launches that wait on memory
// round trips rather than on bytes want, and the shapes that reach it without spilling a vector register ask for it
// (measured: searches of 1M x 768 1.59 -> 1.69 M queries/s, the 1M x 128 build 4.4 -> 4.1 s; at 384 columns with
// two instead of four whole rows in flight, third-loop launches 0.252 -> 0.217 ms, and the sketch kernel with one
// load in flight 0.317 -> 0.295 ms on the first loop's).  A sketch row has a quarter of the chunks, so a quarter of
// the lanes (or of the chunks per lane) covers it.
int launch_step_by_dim(const StepArgs &s, bool aligned, int threads, size_t smem, hipStream_t st) {
    const int nchunks = s.nchunks;
    const int variant = dist_variant();
    if (!aligned || nchunks > 512) launch_step<1, 64, 1, true>(s, threads, smem, st);
    else if (nchunks <= 16) launch_step<1, 16, 8, false, 1, 8, 4, 5, 8, 6, 8>(s, threads, smem, st);
    else if (nchunks <= 32 && variant == 1) launch_step<1, 32, 8, false>(s, threads, smem, st);
    else if (nchunks <= 32) launch_step<2, 16, 4, false, 1, 8, 4, 5, 4, 6, 8>(s, threads, smem, st);
    else if (nchunks <= 64) launch_step<1, 64, 8, false, 2, 8, 2, 5, 8, 6, 8>(s, threads, smem, st);
    else if (nchunks <= 96 && variant != 1) launch_step<3, 32, 2, false, 3, 8, 1, 8, 1, 6, 8>(s, threads, smem, st);
    else if (nchunks <= 128) launch_step<2, 64, 8, false, 2, 16, 2, 6, 2>(s, threads, smem, st);
    else if (nchunks <= 192) launch_step<3, 64, 2, false, 3, 16, 1, 8, 1, 6, 8>(s, threads, smem, st);
    else if (nchunks <= 256) launch_step<4, 64, 4, false, 4, 16, 2, 5, 2>(s, threads, smem, st);
    else if (nchunks <= 320) launch_step<5, 64, 2, false, 3, 32, 2, 6, 1>(s, threads, smem, st);
    else if (nchunks <= 384) launch_step<6, 64, 2, false, 3, 32, 2, 6, 1>(s, threads, smem, st);
    else if (nchunks <= 448) launch_step<7, 64, 2, false, 4, 32, 2, 5, 1>(s, threads, smem, st);
    else launch_step<8, 64, 2, false, 4, 32, 2, 5, 1>(s, threads, smem, st);
    VL_LAUNCH_CHECK("beam_step_kernel");
    g_step_launches.fetch_add(1, std::memory_order_relaxed);
    return VL_OK;
}

struct BeamLayout {
    int64_t m, VL, Vt, E, head;
    int64_t off_cand_ids, off_cand_d, off_v_ids, off_v_d, off_seen, off_seen_count, off_row_quiet, off_memo_rate, off_ctrl, off_rounded, off_memo, total;
    int memo_slots;
};

inline int64_t align256(int64_t x) { return (x + 255) & ~255ll; }

// lean: the layout of the entry point that allocates nothing - the fused step keeps its candidates in LDS
// and runs without the distance cache, so neither gets room.
int beam_layout(const vl_beam_params *p, BeamLayout *l, bool lean = false) {
    VL_REQUIRE(p, "null params");
    VL_REQUIRE(p->n_rows >= 0 && p->dim > 0 && p->n_vectors > 0 && p->width > 0, "bad sizes");
    VL_REQUIRE(p->beam_size > 0 && p->parallel_visit_count > 0 && p->visit_queue_factor > 0 &&
                   p->exclude_factor > 0 && p->speculative_readahead > 0,
               "configuration values must be positive");
    VL_REQUIRE(p->queue_length > 0 && p->queue_length < p->queue_capacity, "queue length must be below its capacity");
    VL_REQUIRE(p->n_vectors < (1ll << 30), "ids must stay below 2^30");
    VL_REQUIRE(p->metric == VL_METRIC_COSINE || p->metric == VL_METRIC_L2, "unknown metric %lld", (long long)p->metric);
    VL_REQUIRE(p->n_rows <= kMaxBlocks, "a batch of %lld rows is too large for one call (limit %lld)",
               (long long)p->n_rows, (long long)kMaxBlocks);
    l->VL = p->visit_queue_factor * p->beam_size;                                      // ann.py:51
    l->Vt = l->VL < p->parallel_visit_count ? l->VL : p->parallel_visit_count;         // queue.py:89
    l->m = l->Vt * p->width;
    l->E = p->exclude_factor * l->VL;                                                  // ann.py:55
    l->head = p->queue_length < l->VL ? p->queue_length : l->VL;                       // queue.py:31
    VL_REQUIRE(l->Vt <= kMaxVisit, "parallel_visit_count above %d is not supported", kMaxVisit);
    VL_REQUIRE(p->queue_length + l->m <= p->queue_capacity,
               "search queue capacity %lld cannot take %lld candidates after its %lld slots",
               (long long)p->queue_capacity, (long long)l->m, (long long)p->queue_length);
    VL_REQUIRE(p->queue_capacity <= kMaxRowSlots && l->VL + l->m <= kMaxRowSlots && l->E <= kMaxRowSlots,
               "queue rows above %d slots are not supported", kMaxRowSlots);
    VL_REQUIRE(p->excl_cols >= 0 && p->excl_cols <= 1024, "exclusion rows above 1024 ids are not supported here");
    int64_t o = 0;
    l->off_cand_ids = o; o = align256(o + (lean ? 0 : p->n_rows * l->m * 4));
    l->off_cand_d = o; o = align256(o + (lean ? 0 : p->n_rows * l->m * 4));
    l->off_v_ids = o; o = align256(o + p->n_rows * l->VL * 4);
    l->off_v_d = o; o = align256(o + p->n_rows * l->VL * 4);
    l->off_seen = o; o = align256(o + p->n_rows * l->E * 4);
    l->off_seen_count = o; o = align256(o + p->n_rows * 4);
    l->off_row_quiet = o; o = align256(o + p->n_rows * 4);
    l->off_memo_rate = o; o = align256(o + p->n_rows * 4);
    l->off_ctrl = o; o = align256(o + (int64_t)sizeof(BeamCtrl));
    // the query rows rounded for the sketch, for calls that say they bring one
    l->off_rounded = o; o = align256(o + ((p->flags & VL_BEAM_USES_SKETCH) && !lean ? p->n_rows * sketch_query_bytes(p->dim) : 0));
    // per-row cache of evaluated (id, distance) pairs: 128 slots per candidate of one iteration,
    // 1Ki..64Ki per row, the whole table at most 8 GiB (measured at 1M x 768: 16Ki -> 64Ki slots cuts the
    // rows fetched in the second optimisation loop by 30 %, 256Ki adds little)
    static const int memo_env = [] {
        const char *e = getenv("VL_BEAM_MEMO");
        return e ? atoi(e) : -1;
    }();
    // ... and no more than 512 per slot of the search queue: a search with a short queue ends after few
    // iterations, fills little of a large table and would pay for clearing it on every call
    int64_t want = 128 * l->m < 512 * p->queue_length ? 128 * l->m : 512 * p->queue_length;
    int slots = vl_next_pow2(want > 65536 ? 65536 : want);
    if (slots < 1024) slots = 1024;
    if (slots > 65536) slots = 65536;
    while (slots > 1024 && p->n_rows * (int64_t)slots * 8 > (8ll << 30)) slots >>= 1;
    if (memo_env >= 0) slots = memo_env;
    if (lean || (p->flags & VL_BEAM_NO_CACHE)) slots = 0;
    l->memo_slots = slots;
    l->off_memo = o; o = align256(o + p->n_rows * (int64_t)slots * 8);
    l->total = o;
    return VL_OK;
}

}  // namespace

VL_EXPORT int64_t vl_beam_workspace_bytes(const vl_beam_params *p) {
    BeamLayout l;
    int rc = beam_layout(p, &l);
    return rc < 0 ? rc : l.total;
}

namespace {

__global__ void beam_empty_status_kernel(int32_t *status) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        status[0] = 1;
        status[1] = 0;
    }
}

__global__ void beam_status_kernel(const BeamCtrl *c, int iterations, int R, int32_t *status) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    int ended = c->stop, t = c->ended_after;
    if (!ended && iterations % R == 0 && c->changed[(iterations / R) & 63] == 0) {
        ended = 1;  // the last launch was a checking iteration that found every row quiet
        t = iterations;
    }
    status[0] = c->error ? -1 : ended;  // -1: a row's state was impossible (the scratch memory was shared with another call)
    status[1] = ended ? t : iterations;
}

// The loop itself.  fixed_iterations == 0: run until a progress check finds the batch quiet, reading the
// flag on the host every speculative_readahead iterations; returns the iteration count.  fixed_iterations
// > 0: enqueue exactly that many iterations and return 0 without ever waiting for the device - once a
// check finds the batch quiet the remaining launches do nothing (beam_gate) - then one small kernel writes
// status_out[0] = 1 if the loop ended within them (else 0) and status_out[1] = the iteration count.
int64_t beam_loop(const vl_beam_params *p, const BeamLayout &l, const float *queries, const float *vectors,
                  const int32_t *beams, int32_t *q_ids, float *q_dists, const int32_t *exclude, void *workspace,
                  int64_t workspace_bytes, int64_t fixed_iterations, int32_t *status_out, void *stream,
                  const uint8_t *sketch = nullptr) {
    int rc;
    VL_REQUIRE(queries && vectors && beams && q_ids && q_dists && workspace, "null pointer");
    VL_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    if (workspace_bytes < l.total) {
        vl_set_error("workspace of %lld bytes is smaller than the %lld needed", (long long)workspace_bytes,
                     (long long)l.total);
        return VL_ERR_WORKSPACE;
    }
    VL_REQUIRE(p->n_rows * (l.VL > l.m ? l.VL : l.m) < (1ll << 40), "batch too large");
    VL_REQUIRE(p->n_rows * (int64_t)l.VL < (1ll << 31), "batch too large: %lld rows with visit queues of %d slots",
               (long long)p->n_rows, (int)l.VL);
    hipStream_t st = (hipStream_t)stream;
    char *ws = (char *)workspace;
    int32_t *cand_ids = (int32_t *)(ws + l.off_cand_ids);
    float *cand_d = (float *)(ws + l.off_cand_d);
    int32_t *v_ids = (int32_t *)(ws + l.off_v_ids);
    float *v_d = (float *)(ws + l.off_v_d);
    int32_t *seen = (int32_t *)(ws + l.off_seen);
    int32_t *seen_count = (int32_t *)(ws + l.off_seen_count);
    int32_t *row_quiet = (int32_t *)(ws + l.off_row_quiet);
    BeamCtrl *ctrl = (BeamCtrl *)(ws + l.off_ctrl);

    uint64_t *memo = (uint64_t *)(ws + l.off_memo);
    MergeArgs a;
    a.ctrl = ctrl; a.readahead = (int)p->speculative_readahead; a.n_rows = p->n_rows;
    a.cand_ids = cand_ids; a.cand_d = cand_d; a.m = (int)l.m;
    a.q_ids = q_ids; a.q_d = q_dists; a.cap = (int)p->queue_capacity; a.L = (int)p->queue_length;
    a.Ps = vl_next_pow2(a.cap);
    a.excl = p->excl_cols > 0 ? exclude : nullptr; a.excl_cols = a.excl ? (int)p->excl_cols : 0;
    a.v_ids = v_ids; a.v_d = v_d; a.VL = (int)l.VL; a.Vt = (int)l.Vt; a.Pv = vl_next_pow2(l.VL + l.m);
    a.seen = seen; a.seen_count = seen_count; a.E = (int)l.E;
    const bool per_query = (p->flags & VL_BEAM_PER_QUERY_STOP) != 0;
    a.row_quiet = per_query ? row_quiet : nullptr;
    a.Pc = vl_next_pow2(l.m);
    if (a.Pc < 2) a.Pc = 2;
    // VL_BEAM_MERGE=sort selects the full-row-sort form of the merge step (exact for queue rows in any state)
    static const bool sort_merge_env = [] {
        const char *e = getenv("VL_BEAM_MERGE");
        return e && e[0] == 's';
    }();
    const bool use_sort_merge = sort_merge_env || (p->flags & VL_BEAM_SORT_MERGE);
    // threads per row of the merge step: small rows are latency bound and do better with
    // more rows in flight per CU (measured: 128 wins at m=256, E=480 and at m=128, E=960; 256 wins at
    // m=512, E=960)
    static const int merge_threads_env = [] {
        const char *e = getenv("VL_BEAM_MERGE_THREADS");
        return e ? atoi(e) : 0;
    }();
    const int merge_threads = merge_threads_env ? merge_threads_env
                              : ((l.m <= 128 || (l.m + l.E + l.VL + p->queue_length) <= 1024) ? 128 : 256);
    const int Pmax = a.Ps > a.Pv ? a.Ps : a.Pv;
    const size_t smem = use_sort_merge
        ? (size_t)Pmax * 8 + (size_t)a.L * 4 + (size_t)a.E * 8 + (size_t)a.excl_cols * 4
        : (size_t)a.Pc * 16 + (size_t)(a.L + a.VL) * 8 + (size_t)a.E * 8 + (size_t)a.excl_cols * 4 + (size_t)a.m + 16;
    VL_REQUIRE(smem + 2048 <= kLdsPerCu, "queues of this size need %zu bytes of LDS (a compute unit has %zu)", smem,
               kLdsPerCu);

    // VL_BEAM_FUSED=0 runs an iteration as two launches (expand, merge) instead of the fused step
    static const bool fused_env = [] {
        const char *e = getenv("VL_BEAM_FUSED");
        return !(e && e[0] == '0');
    }();
    const bool use_fused = fused_env && !use_sort_merge && merge_threads != 64 && !(p->flags & VL_BEAM_TWO_LAUNCHES);
    VL_REQUIRE(!per_query || use_fused, "the per-query stop is only built into the fused step");
    if (!use_fused) {
        if (use_sort_merge) VL_HIP(vl_allow_lds(beam_merge_kernel, smem));
        else if (merge_threads == 64) VL_HIP(vl_allow_lds(beam_merge2_kernel<64>, smem));
        else if (merge_threads == 128) VL_HIP(vl_allow_lds(beam_merge2_kernel<128>, smem));
        else VL_HIP(vl_allow_lds(beam_merge2_kernel<256>, smem));
    }
    const bool aligned = (p->dim % 4 == 0) && (((uintptr_t)queries | (uintptr_t)vectors) % 16 == 0);
    StepArgs step;
    step.queries = queries; step.vectors = vectors; step.beams = beams; step.n_vectors = p->n_vectors;
    step.dim = (int)p->dim; step.nchunks = (int)((p->dim + 3) / 4); step.width = (int)p->width;
    step.width_magic = (uint32_t)((1ull << 32) / (uint64_t)p->width + 1);  // not used for width 1 (it does not fit)
    step.l2 = p->metric == VL_METRIC_L2;
    step.memo = l.memo_slots > 0 ? memo : nullptr;
    step.memo_rate = (int32_t *)(ws + l.off_memo_rate);  // written in iteration kMemoDecide, read after it
    {
        // break-even share of hits, measured on 512-byte rows at about 0.4 and scaled with the row size
        static const int rate_env = [] {
            const char *e = getenv("VL_BEAM_MEMO_MIN_RATE");
            return e ? atoi(e) : -1;
        }();
        int64_t r = (205ll * 256) / (4 * p->dim);
        step.memo_min_rate = rate_env >= 0 ? rate_env : (int)(r > 255 ? 255 : r);
    }
    // The sketch serves the cosine distance of 16-byte aligned rows in the fused step; other calls ignore it.
    step.sketch = (sketch && !step.l2 && aligned && use_fused && p->dim <= 2048 && l.m <= kMaxCandidates) ? sketch : nullptr;
    VL_REQUIRE(!step.sketch || (p->flags & VL_BEAM_USES_SKETCH),
               "a call with a sketch needs VL_BEAM_USES_SKETCH in flags (and a workspace sized with it)");
    step.rounded_queries = (const uint8_t *)(ws + l.off_rounded);
    step.rounded_query_bytes = sketch_query_bytes(p->dim);
    step.sketch_tails = sketch ? sketch + sketch_tails_offset(p->n_vectors, p->dim) : nullptr;
    step.sketch_chunks = (int)sketch_data_chunks(p->dim);
    step.window = 0;
    step.lds_slots = 0;
    step.memo_shift = 32;
    if (step.memo) {
        int lg = 0;
        while ((1 << lg) < l.memo_slots) ++lg;
        VL_REQUIRE((1 << lg) == l.memo_slots && lg >= 4, "memo slots must be a power of two, 16 or more");
        step.memo_shift = 32 - lg;
    }
    // with a sketch every row starts out using it (and the cache, when there is one)
    const bool sketch_from_start = step.sketch != nullptr;
    if (step.sketch) {
        rc = vl_launch_sketch_queries(queries, p->n_rows, p->dim, (uint8_t *)(ws + l.off_rounded), st);
        if (rc < 0) return rc;
    }
    {
        int64_t n = p->n_rows * l.VL;
        if (n < kBeamStripes) n = kBeamStripes;
        if (n < p->n_rows) n = p->n_rows;
        hipLaunchKernelGGL(beam_init_kernel, dim3((unsigned)((n + kQueueThreads - 1) / kQueueThreads)),
                           dim3(kQueueThreads), 0, st, ctrl, p->n_rows, q_ids, q_dists, (int)p->queue_capacity,
                           (int)l.head, v_ids, v_d, (int)l.VL, seen_count, row_quiet, (int32_t *)(ws + l.off_memo_rate),
                           sketch_from_start ? (256 | (1 << 16)) : 256, sketch_from_start ? (int)p->n_rows : 0);
        VL_LAUNCH_CHECK("beam_init_kernel");
    }
    if (l.memo_slots > 0) {
        hipLaunchKernelGGL(beam_memo_clear_kernel, dim3(4096), dim3(256), 0, st, memo, p->n_rows * (int64_t)l.memo_slots);
        VL_LAUNCH_CHECK("beam_memo_clear_kernel");
    }

    const int R = (int)p->speculative_readahead;
    // Several iterations per launch (beam_window_body; VL_BEAM_WINDOWS in flags, or VL_BEAM_WINDOW=1 in the
    // environment): the R iterations between two progress checks run in one launch while no visited list can fill
    // up in them, i.e. while Vt * (last iteration) <= E; the stretch after that runs one iteration per launch.
    // Off by default: the longer kernel body needs some fifty registers more than the one-iteration kernel, and what
    // it saves (one read and one write of the row's queues per iteration, four launches in five) is less than what
    // the spilled registers or the lost wavefront per SIMD cost (measured at 1M x 768: 0.61 ms per iteration either
    // way on the first optimisation loop's state, 0.48 instead of 0.42 ms on the second's).
    static const bool window_env = [] {
        const char *e = getenv("VL_BEAM_WINDOW");
        return e && e[0] == '1';
    }();
    // entries of the row's distance table in LDS: room for the candidates of one iteration, 256 to 1024
    static const int lds_slots_env = [] {
        const char *e = getenv("VL_BEAM_LDS_SLOTS");
        return e ? atoi(e) : -1;
    }();
    int lds_slots = a.Pc < 256 ? 256 : (a.Pc > 1024 ? 1024 : a.Pc);
    if (lds_slots_env >= 0) lds_slots = lds_slots_env ? vl_next_pow2(lds_slots_env) : 0;
    const size_t smem_window = (size_t)a.Pc * 16 + (size_t)(a.L + a.VL) * 16 + (size_t)lds_slots * 8 + (size_t)a.E * 8 +
                               (size_t)a.excl_cols * 4 + (size_t)a.m + 16;
    const bool use_window = use_fused && (window_env || (p->flags & VL_BEAM_WINDOWS)) && R >= 2 && aligned &&
                            step.nchunks <= 512 && smem_window + 2048 <= kLdsPerCu;
    auto window_fits = [&](int64_t first_iteration) { return use_window && l.Vt * (first_iteration + R - 1) <= l.E; };
    const int step_threads = merge_threads == 128 ? 128 : 256;
    if (fixed_iterations > 0) {
        VL_REQUIRE(use_fused, "a fixed number of iterations is only built for the fused step");
        step.count_evals = 0;
        for (int64_t t = 1; t <= fixed_iterations;) {
            a.iter = (int)t;
            step.m = a;
            const bool windowed = window_fits(t) && (t - 1) % R == 0 && t + R - 1 <= fixed_iterations;
            step.window = windowed ? R : 0;
            step.lds_slots = windowed ? lds_slots : 0;
            rc = launch_step_by_dim(step, aligned, step_threads, windowed ? smem_window : smem, st);
            if (rc < 0) return rc;
            t += windowed ? R : 1;
        }
        hipLaunchKernelGGL(beam_status_kernel, dim3(1), dim3(64), 0, st, ctrl, (int)fixed_iterations, R, status_out);
        VL_LAUNCH_CHECK("beam_status_kernel");
        return 0;
    }
    bool prof;
    {
        std::lock_guard<std::mutex> hold(g_prof_mutex);
        prof = g_prof.enabled != 0;
    }
    step.count_evals = prof ? 1 : 0;
    EventSet events;
    hipEvent_t *ev = events.ev;
    BeamProfile mine;
    if (prof) {
        VL_REQUIRE(R <= 64, "profiling supports speculative_readahead up to 64");
        rc = events.create(3 * R);
        if (rc < 0) return rc;
    }
    // A row expands real nodes in an unbroken run of iterations from the first one, each of
    // which adds at least one id to its visited list of E slots; once no row expands, no
    // queue changes and the next check ends the loop.  More iterations than that mean the
    // control block was overwritten while the loop ran (a workspace shared by two calls).
    const int64_t t_limit = l.E + l.VL + 2 * (int64_t)R + 2;
    // One launch serves the whole batch: the kernel that can read the sketch is launched while most rows of the
    // batch still use it.  A row gives the sketch up when it does not pay (counted on the device, read by the
    // host at its regular progress check); in the other kernel such a row goes on as it would without a sketch.
    const uint8_t *sketch_table = step.sketch;
    int sketch_rows = sketch_from_start ? (int)p->n_rows : 0;
    int64_t t = 0;
    for (;;) {
        int launches = 0;  // of this stretch between two progress checks
        if (window_fits(t + 1)) {
            // the sketch kernel also for the first window: its rows leave the sketch alone in iteration 1
            if (prof) VL_HIP(hipEventRecord(ev[0], st));
            a.iter = (int)(t + 1);
            step.m = a;
            step.sketch = (2 * (int64_t)sketch_rows >= p->n_rows) ? sketch_table : nullptr;
            step.window = R;
            step.lds_slots = lds_slots;
            rc = launch_step_by_dim(step, aligned, step_threads, smem_window, st);
            if (rc < 0) return rc;
            if (prof) VL_HIP(hipEventRecord(ev[1], st));
            step.window = 0;
            step.lds_slots = 0;
            t += R;
            launches = 1;
        }
        for (int r = 0; r < R && !launches; ++r) {
            ++t;
            if (prof) VL_HIP(hipEventRecord(ev[3 * r], st));
            a.iter = (int)t;
            if (use_fused) {
                step.m = a;
                step.sketch = (t > 1 && 2 * (int64_t)sketch_rows >= p->n_rows) ? sketch_table : nullptr;
                rc = launch_step_by_dim(step, aligned, step_threads, smem, st);
                if (rc < 0) return rc;
                if (prof) VL_HIP(hipEventRecord(ev[3 * r + 1], st));
                continue;
            }
            rc = vl_launch_expand(queries, p->n_rows, vectors, p->n_vectors, p->dim, nullptr, v_ids, l.Vt, beams,
                                  p->n_vectors, p->width, l.m, cand_ids, cand_d, ctrl, (int)t, R, (int)l.E, l.VL,
                                  prof ? 1 : 0, memo, l.memo_slots, (int)p->metric, st);
            if (rc < 0) return rc;
            if (prof) VL_HIP(hipEventRecord(ev[3 * r + 1], st));
            if (use_sort_merge)
                hipLaunchKernelGGL(beam_merge_kernel, dim3((unsigned)p->n_rows), dim3(kQueueThreads), smem, st, a);
            else if (merge_threads == 64)
                hipLaunchKernelGGL(beam_merge2_kernel<64>, dim3((unsigned)p->n_rows), dim3(64), smem, st, a);
            else if (merge_threads == 128)
                hipLaunchKernelGGL(beam_merge2_kernel<128>, dim3((unsigned)p->n_rows), dim3(128), smem, st, a);
            else
                hipLaunchKernelGGL(beam_merge2_kernel<256>, dim3((unsigned)p->n_rows), dim3(256), smem, st, a);
            VL_LAUNCH_CHECK("beam merge kernel");
            if (prof) VL_HIP(hipEventRecord(ev[3 * r + 2], st));
        }
        // one copy brings the ring of progress flags and the two words behind it (they are neighbours in the
        // control block): this check's flag, the rows still using the sketch, the error flag
        struct {
            int changed[64];
            int sketch_rows, error;
        } seen_by_host;
        static_assert(offsetof(BeamCtrl, error) - offsetof(BeamCtrl, changed) == 65 * sizeof(int) &&
                          offsetof(BeamCtrl, sketch_rows) - offsetof(BeamCtrl, changed) == 64 * sizeof(int),
                      "changed[64], sketch_rows, error follow each other");
        VL_HIP(hipMemcpyAsync(&seen_by_host, &ctrl->changed[0], sizeof(seen_by_host), hipMemcpyDeviceToHost, st));
        VL_HIP(hipStreamSynchronize(st));
        const int changed = seen_by_host.changed[(t / R) & 63];
        const int state[2] = {seen_by_host.sketch_rows, seen_by_host.error};
        if (sketch_table) sketch_rows = state[0];
        if (state[1]) {
            vl_set_error("a row's visited list holds more ids than %lld iterations can have put there: the workspace "
                         "was overwritten while the loop ran - is it shared with a concurrent call?", (long long)t);
            return VL_ERR_STATE;
        }
        if (prof) {
            const int timed = launches ? launches : R;
            for (int r = 0; r < timed; ++r) {
                float ms = 0;
                VL_HIP(hipEventElapsedTime(&ms, ev[3 * r], ev[3 * r + 1]));
                mine.expand_ms += ms;
                if (!use_fused) {
                    VL_HIP(hipEventElapsedTime(&ms, ev[3 * r + 1], ev[3 * r + 2]));
                    mine.merge_ms += ms;
                }
            }
            mine.expand_launches += timed;
            mine.merge_launches += timed;
        }
        if (!changed) break;  // ann.py:90-91
        if (t > t_limit) {
            vl_set_error("beam search still changing after %lld iterations (bound %lld): its workspace was "
                         "overwritten while it ran - is it shared with a concurrent call?",
                         (long long)t, (long long)t_limit);
            return VL_ERR_STATE;
        }
    }
    if (prof) {
        unsigned long long ev_counts[kBeamStripes];
        VL_HIP(hipMemcpyAsync(ev_counts, ctrl->evals, sizeof(ev_counts), hipMemcpyDeviceToHost, st));
        VL_HIP(hipStreamSynchronize(st));
        for (int i = 0; i < kBeamStripes; ++i) mine.evals += (int64_t)ev_counts[i];
        VL_HIP(hipMemcpyAsync(ev_counts, ctrl->wanted, sizeof(ev_counts), hipMemcpyDeviceToHost, st));
        VL_HIP(hipStreamSynchronize(st));
        for (int i = 0; i < kBeamStripes; ++i) mine.wanted += (int64_t)ev_counts[i];
        VL_HIP(hipMemcpyAsync(ev_counts, ctrl->sketched, sizeof(ev_counts), hipMemcpyDeviceToHost, st));
        VL_HIP(hipStreamSynchronize(st));
        for (int i = 0; i < kBeamStripes; ++i) mine.sketched += (int64_t)ev_counts[i];
        std::lock_guard<std::mutex> hold(g_prof_mutex);
        g_prof.expand_ms += mine.expand_ms; g_prof.merge_ms += mine.merge_ms;
        g_prof.expand_launches += mine.expand_launches; g_prof.merge_launches += mine.merge_launches;
        g_prof.evals += mine.evals; g_prof.wanted += mine.wanted; g_prof.sketched += mine.sketched;
        g_prof.rows += p->n_rows;
        g_prof.iterations += t;
    }
    return t;
}

}  // namespace

VL_EXPORT int64_t vl_closest_vectors(const vl_beam_params *p, const float *queries, const float *vectors,
                                     const int32_t *beams, int32_t *q_ids, float *q_dists,
                                     const int32_t *exclude, void *workspace, int64_t workspace_bytes,
                                     void *stream) {
    BeamLayout l;
    int rc = beam_layout(p, &l);
    if (rc < 0) return rc;
    if (p->n_rows == 0) return 0;
    return beam_loop(p, l, queries, vectors, beams, q_ids, q_dists, exclude, workspace, workspace_bytes, 0, nullptr,
                     stream);
}

VL_EXPORT int64_t vl_closest_vectors_with_sketch(const vl_beam_params *p, const float *queries, const float *vectors,
                                                 const uint8_t *sketch, const int32_t *beams, int32_t *q_ids,
                                                 float *q_dists, const int32_t *exclude, void *workspace,
                                                 int64_t workspace_bytes, void *stream) {
    BeamLayout l;
    int rc = beam_layout(p, &l);
    if (rc < 0) return rc;
    VL_REQUIRE(!sketch || ((uintptr_t)sketch & 15) == 0, "the sketch table must be 16-byte aligned");
    if (p->n_rows == 0) return 0;
    return beam_loop(p, l, queries, vectors, beams, q_ids, q_dists, exclude, workspace, workspace_bytes, 0, nullptr,
                     stream, sketch);
}

// ---- the entry point that allocates nothing -------------------------------------------
// Its scratch memory is this array, part of the loaded code object: every GPU the library runs on holds
// its own copy until the process ends.  In host code the array's name is only a handle; the address the
// kernels are given comes from hipGetSymbolAddress, looked up once per device with that device current.
namespace {

static __device__ __align__(256) unsigned char scratch[VL_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int scratch_of_current_device(void **out) {
    int dev = -1;
    VL_HIP(hipGetDevice(&dev));
    VL_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d is out of range", dev);
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        VL_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        VL_REQUIRE(ptr != nullptr, "no device address for the static scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return VL_OK;
}

}  // namespace

VL_EXPORT int vl_closest_vectors_noalloc(const vl_beam_params *p, const float *queries, const float *vectors,
                                         const int32_t *beams, int32_t *q_ids, float *q_dists,
                                         const int32_t *exclude, int64_t iterations, int32_t *status_out,
                                         void *stream) {
    BeamLayout l;
    int rc = beam_layout(p, &l, true);
    if (rc < 0) return rc;
    VL_REQUIRE(iterations >= 1 && iterations <= 65536, "iterations must be between 1 and 65536");
    VL_REQUIRE(status_out, "null pointer");
    VL_REQUIRE((p->flags & (VL_BEAM_TWO_LAUNCHES | VL_BEAM_SORT_MERGE)) == 0,
               "only the fused step runs without a caller's workspace");
    VL_REQUIRE(l.total <= (int64_t)VL_NOALLOC_SCRATCH_BYTES,
               "this batch needs %lld bytes of scratch memory, the static array holds %lld: use fewer rows per call "
               "(about %lld bytes per row) or vl_closest_vectors with a workspace",
               (long long)l.total, (long long)VL_NOALLOC_SCRATCH_BYTES,
               (long long)(l.VL * 8 + l.E * 4 + 8));
    void *ptr = nullptr;
    rc = scratch_of_current_device(&ptr);
    if (rc < 0) return rc;
    if (p->n_rows == 0) {
        // nothing to search: the loop ended after no iteration
        hipLaunchKernelGGL(beam_empty_status_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, status_out);
        VL_LAUNCH_CHECK("beam_empty_status_kernel");
        return VL_OK;
    }
    return (int)beam_loop(p, l, queries, vectors, beams, q_ids, q_dists, exclude, ptr, VL_NOALLOC_SCRATCH_BYTES,
                          iterations, status_out, stream);
}

// Profiling switch for vl_closest_vectors: when enabled every expand / merge
// launch is bracketed by HIP events on the caller's stream and the fetched
// candidate rows are counted.  out[0..7] = expand ms, merge ms, expand
// launches, merge launches, candidate rows fetched, query rows, iterations,
// candidate distances asked for (fetched + served by the per-row cache),
// out[8] = candidate rows looked at through the sketch, summed since the last
// reset.
VL_EXPORT int64_t vl_beam_launches(void) { return g_step_launches.load(std::memory_order_relaxed); }

VL_EXPORT int vl_beam_profile(int enable, int reset, double *out) {
    std::lock_guard<std::mutex> hold(g_prof_mutex);
    if (out) {
        out[0] = g_prof.expand_ms; out[1] = g_prof.merge_ms;
        out[2] = (double)g_prof.expand_launches; out[3] = (double)g_prof.merge_launches;
        out[4] = (double)g_prof.evals; out[5] = (double)g_prof.rows; out[6] = (double)g_prof.iterations;
        out[7] = (double)g_prof.wanted;
        out[8] = (double)g_prof.sketched;
    }
    if (reset) g_prof = BeamProfile();
    g_prof.enabled = enable;
    return VL_OK;
}
