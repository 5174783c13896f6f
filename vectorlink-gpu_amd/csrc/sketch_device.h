// 8-bit sketch of the vector table, and the distance bounds a wavefront gets from it.
//
// A beam-search iteration asks for hundreds of candidate distances per row and keeps a handful: a
// candidate matters only if its key is below the last slot of the search queue or of the visit queue,
// or is one of the few best beyond that.  The sketch lets a row find out which candidates those are
// for a quarter of the memory traffic.  A sketch row holds the vector rounded to 8 bits per element
// with one scale per row, and how far that rounding moved the vector.  The table of n vectors is one block
// of n * sketch_row_bytes(dim) bytes in two parts, so that the rows of the first part start on 128-byte
// lines whenever 16 * ceil(dim / 16) is a multiple of 128 (a row that straddles lines costs a line more than
// its size: 903 instead of 788 bytes per candidate were measured past L2 at 768 columns with the tail in the row):
//
//   data, n rows of 16 * ceil(dim / 16) bytes:   int8 u_j = round(v_j / scale), scale = max_j |v_j| / 127, then zeros
//   tails, n entries of 8 bytes after the data:  float scale; half resid >= ||v - scale u||_2; half norm >= ||v||_2
//                                                (both rounded up; sixteen neighbouring ids share a line)
//
// The query row is rounded too, to 15 bits per element (Q_j = round(q_j / qscale) = 128 qh_j + ql_j with
// two int8 digits, qscale = max_j |q_j| / 16256), so that the sum is integer work, four elements per
// v_dot4_i32_i8 and exact: s^ = scale * qscale * sum_j Q_j u_j.  It differs from the dot product <q, v> by
//   <q, v - v^> + <q - q^, v^>,   at most ||q|| resid + ||q - q^|| (norm + resid)   (Cauchy-Schwarz),
// with ||q - q^|| <= qscale / 2 * sqrt(dim).  Adding the rounding of the few float operations that turn
// the integer sums into s^, and of the float32 summation the exact kernel performs (at most
// (dim + 16) * 2^-24 times the sum of the absolute values of its terms), gives an eps with
// |s^ - s| <= eps for the very float s the exact kernel computes, and because the map from s to the
// clamped cosine distance is monotone, rounding included,
// lo = distance(s^ + eps) <= exact distance <= hi = distance(s^ - eps).  Nothing that is returned to
// a caller is ever computed from a sketch: the bounds only decide which candidates are evaluated
// exactly (dist_device.h) and which provably cannot enter a queue.
#pragma once
#include "dist_device.h"

__host__ __device__ inline int64_t sketch_data_chunks(int64_t dim) { return (dim + 15) / 16; }
__host__ __device__ inline int64_t sketch_data_bytes(int64_t dim) { return sketch_data_chunks(dim) * 16; }
constexpr int64_t kSketchTailBytes = 8;
__host__ __device__ inline int64_t sketch_row_bytes(int64_t dim) { return sketch_data_bytes(dim) + kSketchTailBytes; }
// where the tails of a table of n vectors start
__host__ __device__ inline int64_t sketch_tails_offset(int64_t n, int64_t dim) { return n * sketch_data_bytes(dim); }

__device__ __forceinline__ float half_bits_as_float(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
// The smallest half that is not below x (x >= 0, or an infinity): bounds are stored rounded up.
__device__ __forceinline__ uint32_t half_bits_not_below(float x) {
    uint16_t h = __builtin_bit_cast(uint16_t, (_Float16)x);   // to nearest; beyond the largest half: infinity
    if (half_bits_as_float(h) < x) ++h;                         // the next half up (from the largest one: infinity)
    return h;
}

// Sum over a group of N neighbouring lanes, left in the group's first lane (other lanes end with
// values nobody uses).  Same moves as fold_group, for groups of 8 lanes as well.
template <int N>
__device__ __forceinline__ float fold_lanes(float acc) {
    static_assert(N == 8 || N == 16 || N == 32 || N == 64, "group sizes of 8, 16, 32 or 64 lanes");
    if constexpr (N >= 16) return fold_group<N>(acc);
    acc = acc + dpp_move<0x104>(acc);  // row_shl:4
    acc = acc + dpp_move<0x102>(acc);  // row_shl:2
    acc = acc + dpp_move<0x101>(acc);  // row_shl:1
    return acc;
}

// The query row as the lanes of a group hold it for the sketch: 16-element chunk c belongs to lane
// c mod SLPR of the group; four elements per word, high and low digit apart.
template <int SCPL>
struct SketchQuery {
    int qh[SCPL][4], ql[SCPL][4];
    float qscale;  // the step of the rounded query
    float norm2;   // ||q||_2
    float qerr;    // >= ||q - q^||_2
    float exactc;  // per unit of ||v||_2: bound on the rounding of the exact kernel's dot product
};

// The rounded query rows of a call are made once, by sketch_query_kernel (sketch.hip), and kept in the call's
// workspace: per row and 16-element chunk 16 high digits then 16 low digits (int8), and after the last chunk
// float qscale, norm2, qerr, exactc.
__host__ __device__ inline int64_t sketch_query_bytes(int64_t dim) { return sketch_data_chunks(dim) * 32 + 16; }

template <int SCPL, int SLPR>
__device__ __forceinline__ void sketch_query_load(SketchQuery<SCPL> &sq, const uint8_t *__restrict__ rounded_row,
                                                  int data_chunks) {
    const int lig = (threadIdx.x & (kWave - 1)) % SLPR;
    const uint4 *words = reinterpret_cast<const uint4 *>(rounded_row);
#pragma unroll
    for (int i = 0; i < SCPL; ++i) {
        const int c = lig + SLPR * i;
        uint4 h = make_uint4(0u, 0u, 0u, 0u), l = h;
        if (c < data_chunks) {
            h = words[2 * c];
            l = words[2 * c + 1];
        }
        sq.qh[i][0] = (int)h.x; sq.qh[i][1] = (int)h.y; sq.qh[i][2] = (int)h.z; sq.qh[i][3] = (int)h.w;
        sq.ql[i][0] = (int)l.x; sq.ql[i][1] = (int)l.y; sq.ql[i][2] = (int)l.z; sq.ql[i][3] = (int)l.w;
    }
    const float4 tail = *reinterpret_cast<const float4 *>(rounded_row + (int64_t)data_chunks * 32);
    sq.qscale = tail.x;
    sq.norm2 = tail.y;
    sq.qerr = tail.z;
    sq.exactc = tail.w;
}

// One wavefront: lane j holds candidate id `my_id` (valid when `ok`); the bounds of its distance to
// the query go to out_lo[j] and out_hi[j].  SLPR lanes share a sketch row (64 / SLPR rows per load
// instruction), a lane holds SCPL of its 16-byte chunks, SU loads of a group are in flight at a time.
// The loop over the rows does the integer sums only: the k-th candidate's lane is looked up in `order`
// (64 bytes of LDS that belong to this wavefront, filled here), a group slot past the last candidate takes
// the last one again (same addresses, same sum, nothing conditional in the loop), and a row's sum goes to
// out_lo of its candidate.  What turns a sum into bounds - the row's tail, asked for before the loop - and
// the cache entry are each lane's own work for its own candidate afterwards, once for the wavefront
// instead of once per load.
template <int SCPL, int SLPR, int SU>
__device__ __forceinline__ void wave_sketch(const SketchQuery<SCPL> &sq, const uint8_t *__restrict__ table,
                                            const uint8_t *__restrict__ tails, int data_chunks, int32_t my_id, bool ok,
                                            float *out_lo, float *out_hi, uint8_t *order,
                                            uint64_t *memo_row = nullptr, int memo_shift = 0,
                                            LdsMemo lds = LdsMemo{nullptr, 0}) {
    constexpr int G = kWave / SLPR;
    const uint64_t mask = __ballot(ok);
    if (!mask) return;  // uniform over the wavefront
    const int lane = threadIdx.x & (kWave - 1);
    const int grp = lane / SLPR;
    const int lig = lane % SLPR;
    const int n = __popcll(mask);
    uint2 tail = make_uint2(0u, 0u);
    if (ok) {
        tail = *reinterpret_cast<const uint2 *>(tails + (int64_t)my_id * kSketchTailBytes);
        order[__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u))] = (uint8_t)lane;
    }
    int chunk_at[SCPL];  // a chunk past the row's last one reads the last one again and meets zeros of the query
#pragma unroll
    for (int i = 0; i < SCPL; ++i) chunk_at[i] = min(lig + SLPR * i, data_chunks - 1);
    for (int k0 = 0; k0 < n; k0 += G * SU) {
        int src[SU];
        uint4 r[SU][SCPL];
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            if (k0 + u * G >= n) continue;  // uniform: a load instruction with no candidate at all is not issued
            src[u] = order[min(k0 + u * G + grp, n - 1)];
            const int32_t id = __shfl(my_id, src[u]);
            const uint4 *row = reinterpret_cast<const uint4 *>(table + (int64_t)id * data_chunks * 16);
#pragma unroll
            for (int i = 0; i < SCPL; ++i) r[u][i] = row[chunk_at[i]];
        }
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            if (k0 + u * G >= n) continue;
            int sh = 0, sl = 0;
#pragma unroll
            for (int i = 0; i < SCPL; ++i) {
                const int w[4] = {(int)r[u][i].x, (int)r[u][i].y, (int)r[u][i].z, (int)r[u][i].w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    sh = __builtin_amdgcn_sdot4(w[k], sq.qh[i][k], sh, false);
                    sl = __builtin_amdgcn_sdot4(w[k], sq.ql[i][k], sl, false);
                }
            }
            // a lane's two sums are below 2^24 (at most 64 elements of 127 * 127 each), so they convert exactly
            const float acc = fold_lanes<SLPR>(__builtin_fmaf(128.0f, (float)sh, (float)sl));
            if (lig == 0) out_lo[src[u]] = acc;
        }
    }
    if (ok) {
        const float acc = out_lo[lane];  // written by the first lane of the group that had this candidate's row
        const float scale = __builtin_bit_cast(float, tail.x);
        const float resid = half_bits_as_float(tail.y & 0xffffu), norm = half_bits_as_float(tail.y >> 16);
        const float s_hat = (scale * sq.qscale) * acc;
        // 4e-6: the integer sums are exact, the float operations that combine them (one fused
        // multiply-add per lane, up to six adds across lanes, two products) each round by 2^-24 of at most
        // ||q^|| ||v^||
        const float eps = (sq.norm2 * resid + (sq.qerr + 4e-6f * sq.norm2) * (norm + resid) + sq.exactc * norm) * 1.0001f + 2e-7f;
        // a row with a bound of infinity (not finite, or longer than a half can say) met by a query of
        // zeros gives 0 x infinity: no NaN leaves here for finite inputs, the widest bounds do
        const bool known = eps == eps;
        const float lo = known ? clamp_distance(s_hat + eps) : 0.0f, hi = known ? clamp_distance(s_hat - eps) : 1.0f;
        out_lo[lane] = lo;
        out_hi[lane] = hi;
        if (memo_row) memo_store_bounds(memo_row, memo_shift, my_id, lo, hi);
        if (lds.tab) lds_memo_store(lds, my_id, memo_bounds_entry(my_id, lo, hi));
    }
}
