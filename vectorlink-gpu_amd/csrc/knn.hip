// Exact k nearest neighbours by cosine distance on dense fp32 MFMA tiles for
// gfx950.  The reference has no counterpart (its recall is self-recall@1,
// vectorlink_gpu/ann.py:235-259); this is the ground truth for recall@k and the
// only contraction-shaped step of the path.
//
// One workgroup (4 wavefronts, 2 x 2) owns 128 queries and a strip of the
// vector set; per step it forms the 128 x 128 tile of dot products with
// v_mfma_f32_32x32x2_f32 (vectors are the M side, queries the N side, so a
// lane's 16 accumulator values all belong to ONE query) and every lane keeps a
// private sorted list of the k best (distance, id) keys for each of its two
// query columns.  The Q x N distance matrix never exists in memory.  A second
// kernel merges the per-lane lists of a query in LDS.
#include "rowsort.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int KK = 16;        // list length kept per lane and query (k <= KK)
constexpr int TQ = 128;       // queries per workgroup
constexpr int TV = 128;       // vectors per step
constexpr int KT = 32;        // floats of the reduction dimension staged per pass
constexpr int LDS_STRIDE = KT + 4;
constexpr int LISTS_PER_STRIP = 4;  // two half-waves x two wave rows see the same query

__device__ __forceinline__ void list_insert(uint64_t (&key)[KK], uint64_t nk) {
#pragma unroll
    for (int i = KK - 1; i > 0; --i) {
        if (nk < key[i - 1]) key[i] = key[i - 1];
        else if (nk < key[i]) key[i] = nk;
    }
    if (nk < key[0]) key[0] = nk;
}

__global__ __launch_bounds__(256) void knn_tile_kernel(const float *__restrict__ queries, int64_t n_queries,
                                                      const float *__restrict__ vectors, int64_t n_vectors,
                                                      int dim, int64_t strip_len, int n_strips,
                                                      uint64_t *__restrict__ cand) {
    __shared__ __align__(16) float sV[TV * LDS_STRIDE];
    __shared__ __align__(16) float sQ[TQ * LDS_STRIDE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int64_t q0 = (int64_t)blockIdx.x * TQ;
    const int strip = blockIdx.y;
    const int64_t v_begin = strip * strip_len;
    const int64_t v_end = min(n_vectors, v_begin + strip_len);

    uint64_t list[2][KK];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
        for (int i = 0; i < KK; ++i) list[cb][i] = kPadKey;

    const int half = lane >> 5;   // which k of an MFMA pair this lane feeds
    const int l32 = lane & 31;

    for (int64_t vt = v_begin; vt < v_end; vt += TV) {
        floatx16 acc[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.0f;

        for (int kt = 0; kt < dim; kt += KT) {
            // stage 128 x KT of both operands through registers into LDS
            float4 rv[4], rq[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int f = tid + 256 * i;
                int row = f >> 3, c4 = f & 7;
                int k = kt + 4 * c4;
                int64_t v = vt + row, q = q0 + row;
                rv[i] = (v < v_end && k < dim) ? *reinterpret_cast<const float4 *>(vectors + v * dim + k)
                                               : make_float4(0.f, 0.f, 0.f, 0.f);
                rq[i] = (q < n_queries && k < dim) ? *reinterpret_cast<const float4 *>(queries + q * dim + k)
                                                   : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int f = tid + 256 * i;
                int row = f >> 3, c4 = f & 7;
                *reinterpret_cast<float4 *>(&sV[row * LDS_STRIDE + 4 * c4]) = rv[i];
                *reinterpret_cast<float4 *>(&sQ[row * LDS_STRIDE + 4 * c4]) = rq[i];
            }
            __syncthreads();
#pragma unroll
            for (int g = 0; g < KT / 8; ++g) {
                float4 a[2], b[2];
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
                    a[rb] = *reinterpret_cast<const float4 *>(&sV[(64 * wr + 32 * rb + l32) * LDS_STRIDE + 8 * g + 4 * half]);
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
                    b[cb] = *reinterpret_cast<const float4 *>(&sQ[(64 * wc + 32 * cb + l32) * LDS_STRIDE + 8 * g + 4 * half]);
#pragma unroll
                for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb].x, b[cb].x, acc[rb][cb], 0, 0, 0);
                        acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb].y, b[cb].y, acc[rb][cb], 0, 0, 0);
                        acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb].z, b[cb].z, acc[rb][cb], 0, 0, 0);
                        acc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb].w, b[cb].w, acc[rb][cb], 0, 0, 0);
                    }
            }
        }
        // accumulator register r of this lane: vector row 8*(r/4) + 4*half + r%4, query column l32
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    int64_t v = vt + 64 * wr + 32 * rb + 8 * (r >> 2) + 4 * half + (r & 3);
                    float d = (1.0f - acc[rb][cb][r]) * 0.5f;
                    d = d < 0.0f ? 0.0f : (d > 1.0f ? 1.0f : d);
                    uint64_t nk = vl_make_key((int32_t)v, d);
                    if (v < v_end && nk < list[cb][KK - 1]) list_insert(list[cb], nk);
                }
    }

    // per query: n_strips * 4 lists of KK keys
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
        int64_t q = q0 + 64 * wc + 32 * cb + l32;
        if (q < n_queries) {
            uint64_t *dst = cand + ((q * n_strips + strip) * LISTS_PER_STRIP + (wr * 2 + half)) * KK;
#pragma unroll
            for (int i = 0; i < KK; ++i) dst[i] = list[cb][i];
        }
    }
}

__global__ __launch_bounds__(kQueueThreads) void knn_merge_kernel(const uint64_t *__restrict__ cand, int n_cand, int P,
                                                                 int k, int32_t *ids_out, float *d_out, int64_t q0) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint64_t *keys = reinterpret_cast<uint64_t *>(smem);
    const int64_t q = q0 + blockIdx.x;
    for (int i = threadIdx.x; i < P; i += blockDim.x) keys[i] = i < n_cand ? cand[q * n_cand + i] : kPadKey;
    block_bitonic_sort(keys, P);
    for (int i = threadIdx.x; i < k; i += blockDim.x) {
        uint64_t key = keys[i];
        bool real = key != kPadKey;
        ids_out[q * k + i] = real ? vl_key_id(key) : VL_MAXINT;
        d_out[q * k + i] = real ? vl_key_dist(key) : VL_MAXFLOAT;
    }
}

struct KnnPlan {
    int n_strips;
    int64_t strip_len;
    int n_cand;
    int64_t bytes;
};

int knn_plan(int64_t n_queries, int64_t n_vectors, int64_t dim, int64_t k, KnnPlan *p) {
    VL_REQUIRE(n_queries >= 0 && n_vectors > 0 && dim > 0, "bad sizes");
    VL_REQUIRE(k >= 1 && k <= KK, "k must be between 1 and %d", KK);
    VL_REQUIRE(dim % 4 == 0, "exact kNN tiles need a dimension that is a multiple of 4");
    VL_REQUIRE(n_vectors < (1ll << 30), "ids must stay below 2^30");
    int64_t q_blocks = (n_queries + TQ - 1) / TQ;
    if (q_blocks < 1) q_blocks = 1;
    // enough workgroups to fill 256 CUs a few times over, at most 64 strips
    int64_t strips = (2048 + q_blocks - 1) / q_blocks;
    int64_t max_by_len = (n_vectors + TV - 1) / TV;
    if (strips > max_by_len) strips = max_by_len;
    if (strips > 64) strips = 64;
    if (strips < 1) strips = 1;
    int64_t len = (n_vectors + strips - 1) / strips;
    len = (len + TV - 1) / TV * TV;
    strips = (n_vectors + len - 1) / len;
    p->n_strips = (int)strips;
    p->strip_len = len;
    p->n_cand = (int)(strips * LISTS_PER_STRIP * KK);
    p->bytes = (n_queries > 0 ? n_queries : 1) * (int64_t)p->n_cand * 8;
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
    dim3 grid((unsigned)((n_queries + TQ - 1) / TQ), (unsigned)p.n_strips);
    hipLaunchKernelGGL(knn_tile_kernel, grid, dim3(256), 0, st, queries, n_queries, vectors, n_vectors, (int)dim,
                       p.strip_len, p.n_strips, cand);
    VL_LAUNCH_CHECK("knn_tile_kernel");
    int P = vl_next_pow2(p.n_cand);
    for (int64_t q0 = 0; q0 < n_queries; q0 += kMaxBlocks) {
        int64_t rows = n_queries - q0 < kMaxBlocks ? n_queries - q0 : kMaxBlocks;
        hipLaunchKernelGGL(knn_merge_kernel, dim3((unsigned)rows), dim3(kQueueThreads), (size_t)P * 8, st, cand,
                           p.n_cand, P, (int)k, ids_out, dists_out, q0);
    }
    VL_LAUNCH_CHECK("knn_merge_kernel");
    return VL_OK;
}
