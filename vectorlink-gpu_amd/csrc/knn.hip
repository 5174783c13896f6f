// Exact k nearest neighbours by cosine or squared Euclidean distance on dense
// fp32 MFMA tiles for gfx950.  The reference has no counterpart (its recall is self-recall@1,
// vectorlink_gpu/ann.py:235-259); this is the ground truth for recall@k and the
// only contraction-shaped step of the path.
//
// One workgroup (4 wavefronts, 2 x 2) owns 128 queries and a strip of the
// vector set; operand tiles go from global memory straight into LDS
// (global_load_lds, double-buffered: the next stage lands while this one is
// multiplied); per step it forms the 128 x 128 tile of dot products with
// v_mfma_f32_32x32x2_f32 (vectors are the M side, queries the N side, so a
// lane's 16 accumulator values all belong to ONE query) and every lane keeps a
// private sorted list of the k best (distance, id) keys for each of its two
// query columns.  The Q x N distance matrix never exists in memory.  A second
// kernel merges the per-lane lists of a query in LDS.
#include <type_traits>

#include "rowsort.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int KMAX = 16;      // longest list kept per lane and query
constexpr int TQ = 128;       // queries per workgroup
constexpr int TV = 128;       // vectors per step
constexpr int KT = 32;        // floats of the reduction dimension per stage
constexpr int CH = KT / 4;    // 16-byte chunks per row and stage
constexpr int TILE = 128 * KT;  // floats of one staged operand tile (16 KB)
constexpr int LISTS_PER_STRIP = 4;  // two half-waves x two wave rows see the same query
// workgroups of the tile kernel resident at once: two per compute unit (64 KB of LDS each), 256 CUs on an MI355X;
// the count is read from the device on first use
int64_t resident_workgroups() {
    static const int64_t n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        return (int64_t)2 * cus;
    }();
    return n;
}

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

__device__ __align__(16) const float kZeroChunk[4] = {0.f, 0.f, 0.f, 0.f};

// A lane's list of the KK best so far: distances ascending with their ids.  A lane meets its
// candidates in ascending id order, so one that ties a kept distance belongs behind it: comparing
// distances alone orders (distance, id) pairs correctly.  The new distance column is a median of
// three per slot; ids follow the same comparisons.
template <int KK>
__device__ __forceinline__ void list_insert(float (&kd)[KK], int32_t (&kid)[KK], float d, int32_t id) {
#pragma unroll
    for (int i = KK - 1; i > 0; --i) {
        const bool before_prev = d < kd[i - 1], before_this = d < kd[i];
        kid[i] = before_prev ? kid[i - 1] : (before_this ? id : kid[i]);
        kd[i] = __builtin_amdgcn_fmed3f(kd[i - 1], d, kd[i]);
    }
    const bool first = d < kd[0];
    kid[0] = first ? id : kid[0];
    kd[0] = first ? d : kd[0];
}

// Chunk c (16 bytes) of tile row r lives in slot r * CH + (c ^ swz(r)): sixteen consecutive
// rows read the same chunk index from sixteen different 16-byte bank groups.
__device__ __forceinline__ int swz(int r) { return (r >> 1) & (CH - 1); }

// Staging: 128 rows x KT floats of an operand go straight from global memory into LDS (no
// registers in between).  A wavefront instruction fills 1 KB = 8 tile rows and lane i writes
// slot i of those rows, so it fetches the chunk that belongs there.  Each lane has four such
// (row, chunk) duties per operand; their source addresses at k = 0 are kept as pointers.
// Rows past `last` repeat row `last` (their results are discarded later).
__device__ __forceinline__ void duty_pointers(const float *__restrict__ src, int64_t first, int64_t last, int dim,
                                              int wave, int lane, const float *(&p)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = 8 * (4 * wave + i) + (lane >> 3);
        const int c = (lane & (CH - 1)) ^ swz(r);
        int64_t row = first + r;
        row = row < last ? row : last;
        p[i] = src + row * dim + 4 * c;
    }
}

// RAGGED: the last stage reaches past `dim`; chunks out there come from a zero chunk.
template <bool RAGGED>
__device__ __forceinline__ void stage_operand(const float *const (&p)[4], int kt, int dim, float *tile, int wave,
                                              int lane) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float *g = p[i] + kt;
        if constexpr (RAGGED) {
            const int r = 8 * (4 * wave + i) + (lane >> 3);
            const int c = (lane & (CH - 1)) ^ swz(r);
            if (kt + 4 * c >= dim) g = kZeroChunk;
        }
        __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(tile + 8 * (4 * wave + i) * KT), 16, 0, 0);
    }
}

// every query's shared bound starts at infinity
__global__ void knn_bound_init_kernel(uint32_t *__restrict__ q_bound, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        q_bound[i] = 0x7F800000u;
}

// squared lengths of rows, one wavefront per row (the L2 tiles add them to -2 q.v)
__global__ __launch_bounds__(256) void row_norms_kernel(const float *__restrict__ rows, int64_t n, int dim,
                                                        float *__restrict__ out) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const int lane = threadIdx.x & 63;
    const float4 *src = reinterpret_cast<const float4 *>(rows + row * dim);
    float s = 0.0f;
    for (int c = lane; c < dim / 4; c += 64) {
        float4 x = src[c];
        s = fmaf(x.x, x.x, s);
        s = fmaf(x.y, x.y, s);
        s = fmaf(x.z, x.z, s);
        s = fmaf(x.w, x.w, s);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (lane == 0) out[row] = s;
}

// L2: distances are |q|^2 + |v|^2 - 2 q.v from the rows' squared lengths (q_norm, v_norm)
template <int KK, bool L2>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void knn_tile_kernel(const float *__restrict__ queries, int64_t n_queries,
                                                      const float *__restrict__ vectors, int64_t n_vectors,
                                                      int dim, int64_t strip_len, int n_strips,
                                                      int n_qblocks, int q_group, uint64_t *__restrict__ cand,
                                                      const float *__restrict__ q_norm,
                                                      const float *__restrict__ v_norm, uint32_t *__restrict__ q_bound) {
    // two buffers per operand as separate arrays: the compiler can then tell that the loads
    // landing in one buffer do not touch the one being read
    __shared__ __align__(16) float sV0[TILE];
    __shared__ __align__(16) float sV1[TILE];
    __shared__ __align__(16) float sQ0[TILE];
    __shared__ __align__(16) float sQ1[TILE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    // Work items (query block, strip) are ordered so that q_group query blocks go through all
    // strips together; workgroups are dealt to the 8 XCDs round-robin and XCD x takes the x-th
    // eighth of that order.  The query rows that are re-read for every vector tile then stay in
    // the XCD's L2, and each vector strip is streamed by q_group workgroups together.
    int q_block, strip;
    {
        const int64_t total = (int64_t)n_qblocks * n_strips;
        const int64_t per_xcd = (total + 7) >> 3;
        const int64_t j = blockIdx.x >> 3;
        const int64_t t = (int64_t)(blockIdx.x & 7) * per_xcd + j;
        if (j >= per_xcd || t >= total) return;
        const int64_t full = (int64_t)(n_qblocks / q_group) * q_group * n_strips;  // items of the complete groups
        if (t < full) {
            const int64_t per_group = (int64_t)q_group * n_strips;
            const int64_t g = t / per_group, w = t - g * per_group;
            strip = (int)(w / q_group);
            q_block = (int)(g * q_group + (w - (int64_t)strip * q_group));
        } else {
            const int rest = n_qblocks % q_group;
            const int64_t w = t - full;
            strip = (int)(w / rest);
            q_block = (n_qblocks / q_group) * q_group + (int)(w - (int64_t)strip * rest);
        }
    }
    const int64_t q0 = (int64_t)q_block * TQ;
    const int64_t v_begin = strip * strip_len;
    const int64_t v_end = min(n_vectors, v_begin + strip_len);

    float kd[2][KK];
    int32_t kid[2][KK];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
        for (int i = 0; i < KK; ++i) {
            kd[cb][i] = __builtin_inff();   // an empty slot
            kid[cb][i] = VL_MAXINT;
        }
    // A value can only matter if it is not above the KK-th best seen so far for its query; the
    // two half-waves hold lists of the same queries, so each uses the tighter of the two bounds.
    float bound[2] = {__builtin_inff(), __builtin_inff()};
    // The KK-th best of ANY list of a query bounds the query's KK-th best overall, so the lists of a query - in
    // this workgroup's other wavefronts and in the workgroups that take the other strips - share the smallest of
    // theirs through q_bound (distances are not negative: their bit patterns order like unsigned integers).  A
    // wavefront publishes its bound when it is below the shared one it last read and picks the shared one up a
    // tile later, so neither access is waited for; a value read late is merely a weaker bound.
    uint32_t shared_bits[2] = {0x7F800000u, 0x7F800000u};

    const int half = lane >> 5;   // which k of an MFMA pair this lane feeds
    const int l32 = lane & 31;

    // Byte offset of this lane's first 16-byte read in a tile for each of its operand rows;
    // the read of step g is that offset with bits 5..6 flipped by g (the chunk swizzle).
    int a_off[2], b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        int ra = 64 * wr + 32 * i + l32, rb = 64 * wc + 32 * i + l32;
        a_off[i] = ra * (KT * 4) | ((half ^ swz(ra)) << 4);
        b_off[i] = rb * (KT * 4) | ((half ^ swz(rb)) << 4);
    }
    const bool ragged = (dim % KT) != 0;
    const float *qp[4], *vp[4];
    duty_pointers(queries, q0, n_queries - 1, dim, wave, lane, qp);
    float qn[2] = {0.0f, 0.0f};
    if constexpr (L2) {
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
            const int64_t q = q0 + 64 * wc + 32 * cb + l32;
            qn[cb] = q_norm[q < n_queries ? q : n_queries - 1];
        }
    }

    if (v_begin < v_end) {
        duty_pointers(vectors, v_begin, v_end - 1, dim, wave, lane, vp);
        if (ragged) {
            stage_operand<true>(vp, 0, dim, sV0, wave, lane);
            stage_operand<true>(qp, 0, dim, sQ0, wave, lane);
        } else {
            stage_operand<false>(vp, 0, dim, sV0, wave, lane);
            stage_operand<false>(qp, 0, dim, sQ0, wave, lane);
        }
    }

    // One stage (tile vt, floats kt .. kt + KT): wait for its operand tiles, start the loads of
    // the next stage into the other buffers, multiply.  The two instances differ only in which
    // buffers they name.
    auto stage = [&](auto which, int64_t vt, int kt, floatx16 (&acc)[2][2]) {
        constexpr int B = decltype(which)::value;
        float *const v_cur = B ? sV1 : sV0, *const q_cur = B ? sQ1 : sQ0;
        float *const v_nxt = B ? sV0 : sV1, *const q_nxt = B ? sQ0 : sQ1;
        // this stage's tiles have landed (own loads, then everybody's) and the other
        // buffers are no longer being read
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        int nkt = kt + KT;
        bool has_next = true;
        if (nkt >= dim) {
            // the first stage of the next tile goes into the first buffers: possible from here
            // only if this stage reads the second ones (an odd stage count ends on the first)
            nkt = 0;
            has_next = B == 1 && vt + TV < v_end;
            if (has_next) duty_pointers(vectors, vt + TV, v_end - 1, dim, wave, lane, vp);
        }
        if (has_next) {
            if (ragged) {
                stage_operand<true>(vp, nkt, dim, v_nxt, wave, lane);
                stage_operand<true>(qp, nkt, dim, q_nxt, wave, lane);
            } else {
                stage_operand<false>(vp, nkt, dim, v_nxt, wave, lane);
                stage_operand<false>(qp, nkt, dim, q_nxt, wave, lane);
            }
        }
        const char *tv = reinterpret_cast<const char *>(v_cur);
        const char *tq = reinterpret_cast<const char *>(q_cur);
        // operands of step g + 1 are read while the products of step g are formed
        float4 a[2][2], b[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) a[0][rb] = *reinterpret_cast<const float4 *>(tv + a_off[rb]);
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) b[0][cb] = *reinterpret_cast<const float4 *>(tq + b_off[cb]);
#pragma unroll
        for (int g = 0; g < KT / 8; ++g) {
            const int cur = g & 1, nxt = cur ^ 1;
            if (g + 1 < KT / 8) {
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
                    a[nxt][rb] = *reinterpret_cast<const float4 *>(tv + (a_off[rb] ^ ((g + 1) << 5)));
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
                    b[nxt][cb] = *reinterpret_cast<const float4 *>(tq + (b_off[cb] ^ ((g + 1) << 5)));
            }
            __builtin_amdgcn_sched_barrier(0);  // keep those reads ahead of this step's products
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) {
                    acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][rb].x, b[cur][cb].x, acc[rb][cb], 0, 0, 0);
                    acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][rb].y, b[cur][cb].y, acc[rb][cb], 0, 0, 0);
                    acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][rb].z, b[cur][cb].z, acc[rb][cb], 0, 0, 0);
                    acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][rb].w, b[cur][cb].w, acc[rb][cb], 0, 0, 0);
                }
        }
    };

    const bool odd_stages = ((dim + KT - 1) / KT) & 1;
    for (int64_t vt = v_begin; vt < v_end; vt += TV) {
        floatx16 acc[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.0f;
        if (odd_stages && vt != v_begin) {
            // nobody could prefetch this tile's first stage: load it now, once the first buffers are free
            __syncthreads();
            duty_pointers(vectors, vt, v_end - 1, dim, wave, lane, vp);
            if (ragged) {
                stage_operand<true>(vp, 0, dim, sV0, wave, lane);
                stage_operand<true>(qp, 0, dim, sQ0, wave, lane);
            } else {
                stage_operand<false>(vp, 0, dim, sV0, wave, lane);
                stage_operand<false>(qp, 0, dim, sQ0, wave, lane);
            }
        }
        for (int kt = 0; kt < dim; kt += 2 * KT) {
            stage(std::integral_constant<int, 0>{}, vt, kt, acc);
            if (kt + KT < dim) stage(std::integral_constant<int, 1>{}, vt, kt + KT, acc);
        }
        // fold the 128 x 128 distances into the lists; accumulator register r of this lane:
        // vector row 8*(r/4) + 4*half + r%4, query column l32 (ids stay below 2^30).
        // Nearly every value is beyond the bound once the lists have warmed up, so a block of 16
        // values is first tested as a whole with one comparison per value, and only a block in
        // which some lane has a candidate goes through the exact test and the insertion.
        const int vbase = (int)vt + 64 * wr + 4 * half;
        const int vlimit = (int)v_end;
        // cosine: distance <= bound exactly when the dot product is at least 1 - 2 bound; the
        // margin covers the rounding of (1 - dot) / 2 for dot products in [-1, 1], and every
        // value passes while the bound is 1 or more (distances are clamped to 1)
        float thr[2];
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
            bound[cb] = fminf(bound[cb], __builtin_bit_cast(float, shared_bits[cb]));  // what the other lists had a tile ago
            thr[cb] = bound[cb] >= 1.0f ? -__builtin_inff() : fmaf(-2.0f, bound[cb], 1.0f) - 4e-7f;
        }
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            float vn[16];
            if constexpr (L2) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int v = vbase + (32 * rb + 8 * (r >> 2) + (r & 3));
                    vn[r] = v_norm[v < vlimit ? v : vlimit - 1];
                }
            }
            auto distance = [&](int cb, int r) {
                if constexpr (L2) return fmaxf(fmaf(-2.0f, acc[rb][cb][r], qn[cb] + vn[r]), 0.0f);
                const float d = (1.0f - acc[rb][cb][r]) * 0.5f;
                return d < 0.0f ? 0.0f : (d > 1.0f ? 1.0f : d);
            };
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                uint64_t hit[16], any = 0;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    bool maybe;
                    if constexpr (L2) maybe = !(distance(cb, r) > bound[cb]);
                    else maybe = acc[rb][cb][r] >= thr[cb];
                    hit[r] = __builtin_amdgcn_ballot_w64(maybe);
                    any |= hit[r];
                }
                if (any == 0) continue;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (hit[r] == 0) continue;
                    const int v = vbase + (32 * rb + 8 * (r >> 2) + (r & 3));
                    const float d = distance(cb, r);
                    if (v < vlimit && !(d > bound[cb]) && d < kd[cb][KK - 1]) list_insert<KK>(kd[cb], kid[cb], d, v);
                }
            }
        }
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
            const float own = kd[cb][KK - 1];
            bound[cb] = fminf(fminf(own, __shfl_xor(own, 32)), bound[cb]);
            const int64_t q = q0 + 64 * wc + 32 * cb + l32;
            if (q < n_queries) {
                if (half == 0 && bound[cb] < __builtin_bit_cast(float, shared_bits[cb]))  // better than what was there
                    __hip_atomic_fetch_min(q_bound + q, __builtin_bit_cast(uint32_t, bound[cb]), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                shared_bits[cb] = __hip_atomic_load(q_bound + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }

    // per query: n_strips * 4 lists of KK keys
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
        int64_t q = q0 + 64 * wc + 32 * cb + l32;
        if (q < n_queries) {
            uint64_t *dst = cand + ((q * n_strips + strip) * LISTS_PER_STRIP + (wr * 2 + half)) * KK;
#pragma unroll
            for (int i = 0; i < KK; ++i) dst[i] = kid[cb][i] == VL_MAXINT ? kPadKey : vl_make_key(kid[cb][i], kd[cb][i]);
        }
    }
}

// A query's candidates are n_lists lists of KK keys, each sorted, and no id is in two of them.  One
// wavefront merges them as a tournament: a lane keeps the heads of its lists (lane, lane + 64, ...)
// and the key behind each head; the smallest head of the wavefront is the next result and the lane
// that held it moves on in that list.  Only the heads and the few keys behind a winner are read.
constexpr int kSelectLists = 4;  // lists per lane: 64 strips x 4 lists at most

__global__ __launch_bounds__(256) void knn_select_kernel(const uint64_t *__restrict__ cand, int n_lists, int KK, int k,
                                                         int32_t *__restrict__ ids_out, float *__restrict__ d_out,
                                                         int64_t n_queries) {
    const int64_t q = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (q >= n_queries) return;  // the whole wavefront leaves
    const int lane = threadIdx.x & 63;
    const uint64_t *base = cand + q * n_lists * KK;
    uint64_t head[kSelectLists], next[kSelectLists];
    int pos[kSelectLists];
#pragma unroll
    for (int j = 0; j < kSelectLists; ++j) {
        const int list = lane + 64 * j;
        head[j] = list < n_lists ? base[(int64_t)list * KK] : kPadKey;
        next[j] = list < n_lists && KK > 1 ? base[(int64_t)list * KK + 1] : kPadKey;
        pos[j] = 0;
    }
    uint64_t result = kPadKey;
    for (int i = 0; i < k; ++i) {
        uint64_t mine = head[0];
        int which = 0;
#pragma unroll
        for (int j = 1; j < kSelectLists; ++j)
            if (head[j] < mine) {
                mine = head[j];
                which = j;
            }
        uint64_t best = mine;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const uint64_t other = __shfl_xor(best, o);
            best = other < best ? other : best;
        }
        if (best == kPadKey) break;  // fewer than k candidates in all
        if (lane == i) result = best;
        if (mine == best) {  // keys are unique: one lane moves on, in one list
#pragma unroll
            for (int j = 0; j < kSelectLists; ++j)
                if (j == which) {
                    ++pos[j];
                    head[j] = next[j];
                    next[j] = pos[j] + 1 < KK ? base[(int64_t)(lane + 64 * j) * KK + pos[j] + 1] : kPadKey;
                }
        }
    }
    if (lane < k) {
        const bool real = result != kPadKey;
        ids_out[q * k + lane] = real ? vl_key_id(result) : VL_MAXINT;
        d_out[q * k + lane] = real ? vl_key_dist(result) : VL_MAXFLOAT;
    }
}

// list lengths the tile kernel is built for: the shortest that holds k is used
__host__ inline int list_length(int64_t k) { return k <= 1 ? 1 : k <= 4 ? 4 : k <= 8 ? 8 : k <= 10 ? 10 : k <= 12 ? 12 : 16; }

struct KnnPlan {
    int list_len;
    int n_strips;
    int64_t strip_len;
    int n_cand;
    int64_t cand_bytes;  // per-lane candidate lists; the queries' shared bounds and the rows' squared lengths (L2) follow
    int64_t bytes;
};

int knn_plan(int64_t n_queries, int64_t n_vectors, int64_t dim, int64_t k, KnnPlan *p) {
    VL_REQUIRE(n_queries >= 0 && n_vectors > 0 && dim > 0, "bad sizes");
    VL_REQUIRE(k >= 1 && k <= KMAX, "k must be between 1 and %d", KMAX);
    VL_REQUIRE(dim % 4 == 0, "exact kNN tiles need a dimension that is a multiple of 4");
    VL_REQUIRE(n_vectors < (1ll << 30), "ids must stay below 2^30");
    int64_t q_blocks = (n_queries + TQ - 1) / TQ;
    if (q_blocks < 1) q_blocks = 1;
    // The vector set is cut into at most 64 strips of whole tiles; q_blocks * strips workgroups
    // share resident_workgroups() slots (two per compute unit), so the run lasts
    // ceil(workgroups / slots) strips' worth of tiles.  Take the strip count with the shortest
    // run; a strip more costs a sixteenth of a tile (wider merge afterwards).
    const int64_t tiles = (n_vectors + TV - 1) / TV;
    int64_t strips = 1, best_cost = -1;
    for (int64_t s = 1; s <= 64 && s <= tiles; ++s) {
        int64_t len_t = (tiles + s - 1) / s;
        int64_t s2 = (tiles + len_t - 1) / len_t;
        if (s2 != s) continue;
        int64_t rounds = (q_blocks * s + resident_workgroups() - 1) / resident_workgroups();
        int64_t cost = rounds * len_t * 16 + s;
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            strips = s;
        }
    }
    int64_t len = (tiles + strips - 1) / strips * TV;
    p->n_strips = (int)strips;
    p->strip_len = len;
    p->list_len = list_length(k);
    p->n_cand = (int)(strips * LISTS_PER_STRIP * p->list_len);
    p->cand_bytes = (n_queries > 0 ? n_queries : 1) * (int64_t)p->n_cand * 8;
    p->bytes = p->cand_bytes + ((2 * n_queries + n_vectors) * 4 + 15) / 16 * 16;
    return VL_OK;
}

}  // namespace

VL_EXPORT int64_t vl_knn_workspace_bytes(int64_t n_queries, int64_t n_vectors, int64_t dim, int64_t k) {
    KnnPlan p;
    int rc = knn_plan(n_queries, n_vectors, dim, k, &p);
    return rc < 0 ? rc : p.bytes;
}

VL_EXPORT int vl_knn_exact(const float *queries, int64_t n_queries, const float *vectors,
                           int64_t n_vectors, int64_t dim, int64_t k, int32_t *ids_out,
                           float *dists_out, void *workspace, int64_t workspace_bytes, void *stream) {
    return vl_knn_exact_metric(queries, n_queries, vectors, n_vectors, dim, k, VL_METRIC_COSINE, ids_out, dists_out,
                               workspace, workspace_bytes, stream);
}

VL_EXPORT int vl_knn_exact_metric(const float *queries, int64_t n_queries, const float *vectors,
                                  int64_t n_vectors, int64_t dim, int64_t k, int32_t metric, int32_t *ids_out,
                                  float *dists_out, void *workspace, int64_t workspace_bytes, void *stream) {
    VL_REQUIRE(metric == VL_METRIC_COSINE || metric == VL_METRIC_L2, "unknown metric %d", (int)metric);
    KnnPlan p;
    int rc = knn_plan(n_queries, n_vectors, dim, k, &p);
    if (rc < 0) return rc;
    if (n_queries == 0) return VL_OK;
    VL_REQUIRE(queries && vectors && ids_out && dists_out && workspace, "null pointer");
    VL_REQUIRE((((uintptr_t)queries | (uintptr_t)vectors | (uintptr_t)workspace) & 15) == 0, "pointers must be 16-byte aligned");
    if (workspace_bytes < p.bytes) {
        vl_set_error("workspace of %lld bytes is smaller than the %lld needed", (long long)workspace_bytes,
                     (long long)p.bytes);
        return VL_ERR_WORKSPACE;
    }
    VL_REQUIRE(n_queries <= kMaxBlocks * TQ, "too many queries for one call (limit %lld)", (long long)(kMaxBlocks * TQ));
    hipStream_t st = (hipStream_t)stream;
    uint64_t *cand = (uint64_t *)workspace;
    const int64_t q_blocks = (n_queries + TQ - 1) / TQ;
    // query blocks kept together: as many as put about 2 MB of query rows into one L2 (1..8)
    int64_t q_group = (2ll << 20) / (TQ * dim * 4);
    q_group = q_group < 1 ? 1 : (q_group > 8 ? 8 : q_group);
    const int64_t blocks = (q_blocks * p.n_strips + 7) / 8 * 8;
    VL_REQUIRE(blocks <= kMaxBlocks * 4, "too many tiles for one call");
    const bool l2 = metric == VL_METRIC_L2;
    uint32_t *q_bound = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(workspace) + p.cand_bytes);
    float *q_norm = reinterpret_cast<float *>(q_bound + n_queries);
    float *v_norm = q_norm + n_queries;
    hipLaunchKernelGGL(knn_bound_init_kernel, dim3(vl_grid_for(n_queries, 256)), dim3(256), 0, st, q_bound, n_queries);
    VL_LAUNCH_CHECK("knn_bound_init_kernel");
    if (l2) {
        VL_REQUIRE((n_vectors + 3) / 4 <= kMaxBlocks * 4, "too many vectors for one call");
        hipLaunchKernelGGL(row_norms_kernel, dim3((unsigned)((n_queries + 3) / 4)), dim3(256), 0, st, queries,
                           n_queries, (int)dim, q_norm);
        hipLaunchKernelGGL(row_norms_kernel, dim3((unsigned)((n_vectors + 3) / 4)), dim3(256), 0, st, vectors,
                           n_vectors, (int)dim, v_norm);
        VL_LAUNCH_CHECK("row_norms_kernel");
    }
#define VL_KNN_LAUNCH(KK)                                                                                     \
    do {                                                                                                      \
        if (l2)                                                                                               \
            hipLaunchKernelGGL((knn_tile_kernel<KK, true>), dim3((unsigned)blocks), dim3(256), 0, st, queries, \
                               n_queries, vectors, n_vectors, (int)dim, p.strip_len, p.n_strips, (int)q_blocks, \
                               (int)q_group, cand, q_norm, v_norm, q_bound);                                  \
        else                                                                                                  \
            hipLaunchKernelGGL((knn_tile_kernel<KK, false>), dim3((unsigned)blocks), dim3(256), 0, st, queries, \
                               n_queries, vectors, n_vectors, (int)dim, p.strip_len, p.n_strips, (int)q_blocks, \
                               (int)q_group, cand, nullptr, nullptr, q_bound);                                \
    } while (0)
    switch (p.list_len) {
        case 1: VL_KNN_LAUNCH(1); break;
        case 4: VL_KNN_LAUNCH(4); break;
        case 8: VL_KNN_LAUNCH(8); break;
        case 10: VL_KNN_LAUNCH(10); break;
        case 12: VL_KNN_LAUNCH(12); break;
        default: VL_KNN_LAUNCH(16); break;
    }
#undef VL_KNN_LAUNCH
    VL_LAUNCH_CHECK("knn_tile_kernel");
    const int n_lists = p.n_strips * LISTS_PER_STRIP;
    VL_REQUIRE(n_lists <= 64 * kSelectLists, "too many candidate lists per query");
    hipLaunchKernelGGL(knn_select_kernel, dim3((unsigned)((n_queries + 3) / 4)), dim3(256), 0, st, cand, n_lists,
                       p.list_len, (int)k, ids_out, dists_out, n_queries);
    VL_LAUNCH_CHECK("knn_select_kernel");
    return VL_OK;
}
