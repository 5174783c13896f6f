// Device code shared by the gathered-distance kernel and the fused beam-search
// step: one wavefront evaluates the cosine distances of up to 64 candidate rows
// against a query row held in registers.  See dist.hip for the summation order.
#pragma once
#include "vl_common.h"


__device__ __forceinline__ float clamp_distance(float cos_theta) {
    float r = (1.0f - cos_theta) * 0.5f;  // kernels.py:109
    if (r < 0.0f) r = 0.0f;               // kernels.py:110-113
    else if (r > 1.0f) r = 1.0f;
    return r;
}

// The folded sum as a distance.  Cosine (the reference's only metric, kernels.py:85-114): the sum is
// the dot product.  Squared L2 (an addition): the sum already is sum_j (a_j - b_j)^2, taken in the
// same chunk / lane / fold order with one subtraction and one fused multiply-add per element.
__device__ __forceinline__ float finish_distance(float sum, bool l2) { return l2 ? sum : clamp_distance(sum); }

// Per-row cache of distances already evaluated in this search: slot = hash(id),
// entry = (distance bits << 32) | id.  Several wavefronts read and write a row's
// table concurrently, so an entry is always moved as ONE relaxed 64-bit atomic
// access: a reader sees a whole entry (old or new), never the id of one and the
// distance of another.
// The 16 ids of an aligned group share a 128-byte line of the table (the group is hashed, the id's low four bits
// pick the entry within it): neighbour lists of a graph with local structure, such as the circulant graph a
// build starts from, probe and fill a few lines instead of one per candidate.  Tables have at least 16 slots.
__device__ __forceinline__ uint32_t memo_hash(int32_t id, int shift) {
    const uint32_t group = (((uint32_t)id >> 4) * 2654435761u) >> shift;
    return (group & ~15u) | ((uint32_t)id & 15u);
}
__device__ __forceinline__ uint64_t memo_entry(int32_t id, float d) {
    return ((uint64_t)__builtin_bit_cast(uint32_t, d) << 32) | (uint32_t)id;
}
__device__ __forceinline__ void memo_store(uint64_t *memo_row, int shift, int32_t id, float d) {
    __hip_atomic_store(memo_row + memo_hash(id, shift), memo_entry(id, d), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t memo_load(const uint64_t *memo_row, int shift, int32_t id) {
    return __hip_atomic_load(memo_row + memo_hash(id, shift), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A second kind of entry, for rows that know a candidate only through the 8-bit sketch (cosine distances,
// which lie in [0, 1]): bit 31 of the id word set (ids stay below 2^30), and in place of the distance its
// bounds lo <= d <= hi as 16-bit fixed point, each moved one step outwards so that encoding and decoding
// never narrow them.
constexpr uint32_t kMemoBounds = 0x80000000u;
__device__ __forceinline__ uint64_t memo_bounds_entry(int32_t id, float lo, float hi) {
    int l = lo >= 0.0f ? (int)(lo * 65535.0f) - 1 : 0;   // a NaN bound becomes the widest one
    int h = hi <= 1.0f ? (int)(hi * 65535.0f) + 2 : 65535;
    l = l < 0 ? 0 : l;
    h = h > 65535 ? 65535 : h;
    return ((uint64_t)(((uint32_t)l << 16) | (uint32_t)h) << 32) | ((uint32_t)id | kMemoBounds);
}
__device__ __forceinline__ void memo_store_bounds(uint64_t *memo_row, int shift, int32_t id, float lo, float hi) {
    __hip_atomic_store(memo_row + memo_hash(id, shift), memo_bounds_entry(id, lo, hi), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float memo_bound_lo(uint64_t e) { return (float)(uint32_t)(e >> 48) * (1.0f / 65535.0f); }
__device__ __forceinline__ float memo_bound_hi(uint64_t e) { return (float)((uint32_t)(e >> 32) & 0xffffu) * (1.0f / 65535.0f); }

// The same entries in a small direct-mapped table in LDS (a workgroup that takes a row through several
// iterations keeps one): a repeat inside those iterations never leaves the compute unit.  An entry moves as one
// 8-byte LDS access; shift = 32 - log2(slots); tab == nullptr: no table.
struct LdsMemo {
    uint64_t *tab;
    int shift;
};
__device__ __forceinline__ uint32_t lds_memo_slot(int32_t id, int shift) { return ((uint32_t)id * 2654435761u) >> shift; }
__device__ __forceinline__ uint64_t lds_memo_load(const LdsMemo &t, int32_t id) {
    return __hip_atomic_load(t.tab + lds_memo_slot(id, t.shift), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void lds_memo_store(const LdsMemo &t, int32_t id, uint64_t e) {
    __hip_atomic_store(t.tab + lds_memo_slot(id, t.shift), e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Folds the partial sums of a group of LPR lanes: lane l += lane l + h for h = LPR/2 ... 1, so the
// group's first lane ends with the sum in the fixed order.  Steps of 32 and 16 lanes swap register
// halves / rows (v_permlane32_swap, v_permlane16_swap), steps inside a row of 16 lanes are DPP row
// shifts: no trip through the LDS crossbar.  Other lanes end with values nobody uses.  The swaps
// are written as instructions because the compiler's builtin folds its two results into one when
// both operands hold the same value.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, __builtin_bit_cast(unsigned, x), CTRL, 0xf, 0xf, true));
}
template <int LPR>
__device__ __forceinline__ float fold_group(float acc) {
    static_assert(LPR == 16 || LPR == 32 || LPR == 64, "group sizes of 16, 32 or 64 lanes");
    if constexpr (LPR == 64) {
        float lo = acc, hi = acc;  // after the swap: lo = {acc.lo, acc.lo}, hi = {acc.hi, acc.hi}
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
        acc = lo + hi;
    }
    if constexpr (LPR >= 32) {
        float even = acc, odd = acc;  // after the swap: even = rows {0, 0, 2, 2}, odd = rows {1, 1, 3, 3}
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(even), "+v"(odd));
        acc = even + odd;
    }
    acc = acc + dpp_move<0x108>(acc);  // row_shl:8
    acc = acc + dpp_move<0x104>(acc);  // row_shl:4
    acc = acc + dpp_move<0x102>(acc);  // row_shl:2
    acc = acc + dpp_move<0x101>(acc);  // row_shl:1
    return acc;
}

// One wavefront: lane j holds candidate id `my_id` (valid when `ok`); the
// distance of candidate lane j to the query goes to out_d[j].
template <int CPL, int LPR, int U>
__device__ __forceinline__ void wave_distances(const float *__restrict__ q_row,
                                               const float *__restrict__ vectors, int dim,
                                               int nchunks, int32_t my_id, bool ok,
                                               float *__restrict__ out_d, uint64_t *memo_row,
                                               int memo_shift, bool l2 = false, LdsMemo lds = LdsMemo{nullptr, 0}) {
    constexpr int G = kWave / LPR;
    const int lane = threadIdx.x & (kWave - 1);
    const int grp = lane / LPR;
    const int lig = lane % LPR;

    float4 q[CPL];
    bool cvalid[CPL];
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
        int c = lig + LPR * i;
        cvalid[i] = c < nchunks;
        q[i] = cvalid[i] ? reinterpret_cast<const float4 *>(q_row)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }

    uint64_t mask = __ballot(ok);
    while (mask) {
        int src[U][G];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (mask) {
                    src[u][g] = __builtin_ctzll(mask);
                    mask &= mask - 1;
                } else {
                    src[u][g] = -1;
                }
            }

        float4 r[U][CPL];
        int mysrc[U];
        int32_t ids[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int s = src[u][0];
#pragma unroll
            for (int g = 1; g < G; ++g) s = (grp == g) ? src[u][g] : s;
            mysrc[u] = s;
            int32_t id;
            if constexpr (G == 1) {
                id = (s >= 0) ? __builtin_amdgcn_readlane(my_id, s) : 0;
            } else {
                id = __shfl(my_id, s >= 0 ? s : 0);
            }
            ids[u] = id;
            const float4 *row = reinterpret_cast<const float4 *>(vectors + (int64_t)id * dim);
#pragma unroll
            for (int i = 0; i < CPL; ++i) {
                if (s >= 0 && cvalid[i]) r[u][i] = row[lig + LPR * i];
                else r[u][i] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // Chunk c of a row belongs to partial sum c mod 64.  A lane of an LPR-lane group holds the
            // chunks lig + LPR * i, i.e. the partial sums lig, lig + LPR, ... (V = 64 / LPR of them, the
            // (V + j)-th chunk continuing the j-th sum), and folds them at lane distances 32 and 16 itself
            // before the group's cross-lane folds: the same additions in the same order as 64 lanes with one
            // partial sum each (sums no chunk reaches are +0).
            constexpr int V = kWave / LPR;
            float part[V];
#pragma unroll
            for (int j = 0; j < V; ++j) part[j] = 0.0f;
            if (l2) {  // uniform over the launch
#pragma unroll
                for (int i = 0; i < CPL; ++i) {
                    const float dx = r[u][i].x - q[i].x, dy = r[u][i].y - q[i].y;
                    const float dz = r[u][i].z - q[i].z, dw = r[u][i].w - q[i].w;
                    float a = part[i % V];
                    a = __builtin_fmaf(dx, dx, a);
                    a = __builtin_fmaf(dy, dy, a);
                    a = __builtin_fmaf(dz, dz, a);
                    a = __builtin_fmaf(dw, dw, a);
                    part[i % V] = a;
                }
            } else {
#pragma unroll
                for (int i = 0; i < CPL; ++i) {
                    float a = part[i % V];
                    a = __builtin_fmaf(r[u][i].x, q[i].x, a);
                    a = __builtin_fmaf(r[u][i].y, q[i].y, a);
                    a = __builtin_fmaf(r[u][i].z, q[i].z, a);
                    a = __builtin_fmaf(r[u][i].w, q[i].w, a);
                    part[i % V] = a;
                }
            }
#pragma unroll
            for (int h = V / 2; h >= 1; h >>= 1)
#pragma unroll
                for (int j = 0; j < h; ++j) part[j] = part[j] + part[j + h];
            float acc = part[0];
            acc = fold_group<LPR>(acc);
            if (lig == 0 && mysrc[u] >= 0) {
                float d = finish_distance(acc, l2);
                out_d[mysrc[u]] = d;
                if (memo_row) memo_store(memo_row, memo_shift, ids[u], d);
                if (lds.tab) lds_memo_store(lds, ids[u], memo_entry(ids[u], d));
            }
        }
    }
}

// The same distances for a caller whose out_d is in LDS (the fused beam-search step), with the per-row work cut to
// the sums: the k-th candidate's lane comes from `order` (64 bytes of LDS that belong to this wavefront, filled
// here by rank; with one row per load instruction the lanes are simply taken off the mask), a group slot past the last
// candidate takes the last one again (same addresses, same sum: nothing in the loop depends on a lane having a
// row), and the group's first lane parks the row's sum in out_d of its candidate.  Turning a sum into a distance
// and storing the cache entry is then each lane's own work for its own candidate, once for the wavefront instead
// of once per load.  Same loads, same additions in the same order, same bits as wave_distances.
template <int CPL, int LPR, int U>
__device__ __forceinline__ void wave_distances_lds(const float *__restrict__ q_row,
                                                   const float *__restrict__ vectors, int dim,
                                                   int nchunks, int32_t my_id, bool ok,
                                                   float *out_d, uint8_t *order, uint64_t *memo_row,
                                                   int memo_shift, bool l2 = false, LdsMemo lds = LdsMemo{nullptr, 0}) {
    constexpr int G = kWave / LPR;
    uint64_t mask = __ballot(ok);
    if (!mask) return;  // uniform over the wavefront
    const int lane = threadIdx.x & (kWave - 1);
    const int grp = lane / LPR;
    const int lig = lane % LPR;
    const int n = __popcll(mask);

    float4 q[CPL];
    bool cvalid[CPL];
#pragma unroll
    for (int i = 0; i < CPL; ++i) {
        int c = lig + LPR * i;
        cvalid[i] = c < nchunks;
        q[i] = cvalid[i] ? reinterpret_cast<const float4 *>(q_row)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if constexpr (G > 1) {
        if (ok) order[__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u))] = (uint8_t)lane;
    }
    for (int k0 = 0; k0 < n; k0 += G * U) {
        float4 r[U][CPL];
        int src[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k0 + u * G < n) {  // uniform: a load instruction with no candidate at all is not issued
                int32_t id;
                if constexpr (G == 1) {
                    src[u] = __builtin_ctzll(mask);
                    mask &= mask - 1;
                    id = __builtin_amdgcn_readlane(my_id, src[u]);
                } else {
                    src[u] = order[min(k0 + u * G + grp, n - 1)];
                    id = __shfl(my_id, src[u]);
                }
                const float4 *row = reinterpret_cast<const float4 *>(vectors + (int64_t)id * dim);
#pragma unroll
                for (int i = 0; i < CPL; ++i) {
                    if (cvalid[i]) r[u][i] = row[lig + LPR * i];
                    else r[u][i] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (k0 + u * G < n) {
                // the partial sums of wave_distances, folded in the same order
                constexpr int V = kWave / LPR;
                float part[V];
#pragma unroll
                for (int j = 0; j < V; ++j) part[j] = 0.0f;
                if (l2) {  // uniform over the launch
#pragma unroll
                    for (int i = 0; i < CPL; ++i) {
                        const float dx = r[u][i].x - q[i].x, dy = r[u][i].y - q[i].y;
                        const float dz = r[u][i].z - q[i].z, dw = r[u][i].w - q[i].w;
                        float a = part[i % V];
                        a = __builtin_fmaf(dx, dx, a);
                        a = __builtin_fmaf(dy, dy, a);
                        a = __builtin_fmaf(dz, dz, a);
                        a = __builtin_fmaf(dw, dw, a);
                        part[i % V] = a;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < CPL; ++i) {
                        float a = part[i % V];
                        a = __builtin_fmaf(r[u][i].x, q[i].x, a);
                        a = __builtin_fmaf(r[u][i].y, q[i].y, a);
                        a = __builtin_fmaf(r[u][i].z, q[i].z, a);
                        a = __builtin_fmaf(r[u][i].w, q[i].w, a);
                        part[i % V] = a;
                    }
                }
#pragma unroll
                for (int h = V / 2; h >= 1; h >>= 1)
#pragma unroll
                    for (int j = 0; j < h; ++j) part[j] = part[j] + part[j + h];
                const float acc = fold_group<LPR>(part[0]);
                if (lig == 0) out_d[src[u]] = acc;
            }
        }
    }
    if (ok) {
        const float d = finish_distance(out_d[lane], l2);  // the sum was parked there by the first lane of the row's group
        out_d[lane] = d;
        if (memo_row) memo_store(memo_row, memo_shift, my_id, d);
        if (lds.tab) lds_memo_store(lds, my_id, memo_entry(my_id, d));
    }
}

// Any dimension, any alignment: scalar loads, same summation order.
__device__ __forceinline__ void wave_distances_generic(const float *__restrict__ q_row,
                                                       const float *__restrict__ vectors, int dim,
                                                       int nchunks, int32_t my_id, bool ok,
                                                       float *__restrict__ out_d, uint64_t *memo_row,
                                                       int memo_shift, bool l2 = false) {
    const int lane = threadIdx.x & (kWave - 1);
    uint64_t mask = __ballot(ok);
    while (mask) {
        int s = __builtin_ctzll(mask);
        mask &= mask - 1;
        int32_t id = __builtin_amdgcn_readlane(my_id, s);
        const float *row = vectors + (int64_t)id * dim;
        float acc = 0.0f;
        for (int c = lane; c < nchunks; c += kWave) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int i = 4 * c + j;
                if (i < dim) {
                    const float x = l2 ? row[i] - q_row[i] : row[i];
                    acc = __builtin_fmaf(x, l2 ? x : q_row[i], acc);
                }
            }
        }
        acc = fold_group<kWave>(acc);
        if (lane == 0) {
            float d = finish_distance(acc, l2);
            out_d[s] = d;
            if (memo_row) memo_store(memo_row, memo_shift, id, d);
        }
    }
}
