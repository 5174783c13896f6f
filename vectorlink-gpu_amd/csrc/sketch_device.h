// 8-bit sketch of the vector table, and the distance bounds a wavefront gets from it.
//
// A beam-search iteration asks for hundreds of candidate distances per row and keeps a handful: a
// candidate matters only if its key is below the last slot of the search queue or of the visit queue,
// or is one of the few best beyond that.  The sketch lets a row find out which candidates those are
// for a quarter of the memory traffic.  A sketch row holds the vector rounded to 8 bits per element
// with one scale per row, and how far that rounding moved the vector:
//
//   bytes [0, dim)            u_j = round(v_j / scale) + 128, scale = max_j |v_j| / 127
//   bytes [dim, pad16(dim))   128 (a zero element)
//   tail, 16 bytes            float scale; float resid >= ||v - scale (u - 128)||_2;
//                             float norm >= ||v||_2; float 0
//
// For a query q, s^ = scale * sum_j q_j (u_j - 128) differs from the dot product <q, v> by at most
// ||q||_2 * resid (Cauchy-Schwarz).  Adding the rounding of the two float32 summations involved (this
// one, and the one the exact kernel performs: at most (dim + 16) * 2^-24 times the sum of the absolute
// values of their terms) gives an eps with |s^ - s| <= eps for the very float s the exact kernel
// computes, and because the map from s to the clamped cosine distance is monotone, rounding included,
// lo = distance(s^ + eps) <= exact distance <= hi = distance(s^ - eps).  Nothing that is returned to
// a caller is ever computed from a sketch: the bounds only decide which candidates are evaluated
// exactly (dist_device.h) and which provably cannot enter a queue.
#pragma once
#include "dist_device.h"

__host__ __device__ inline int64_t sketch_data_chunks(int64_t dim) { return (dim + 15) / 16; }
__host__ __device__ inline int64_t sketch_row_bytes(int64_t dim) { return sketch_data_chunks(dim) * 16 + 16; }

// Byte K of a word as a float (the compiler has one instruction for it: v_cvt_f32_ubyteK).
template <int K>
__device__ __forceinline__ float byte_as_float(unsigned w) {
    return (float)((w >> (8 * K)) & 0xffu);
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
// c mod SLPR of the group, and what the bound needs of the row as a whole.
template <int SCPL>
struct SketchQuery {
    float q[SCPL][16];
    float sum128;  // 128 * sum_j q_j : what the +128 offset of the bytes adds to sum_j q_j u_j
    float norm2;   // ||q||_2
    float roundc;  // per unit of scale: bound on the rounding of sum_j q_j u_j - 128 sum_j q_j
    float exactc;  // per unit of ||v||_2: bound on the rounding of the exact kernel's dot product
};

template <int SCPL, int SLPR>
__device__ __forceinline__ void sketch_query_load(SketchQuery<SCPL> &sq, const float *__restrict__ q_row, int dim) {
    const int lig = (threadIdx.x & (kWave - 1)) % SLPR;
    float s = 0.f, a = 0.f, n = 0.f;
#pragma unroll
    for (int i = 0; i < SCPL; ++i) {
        const int c = lig + SLPR * i;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int j = 16 * c + 4 * w;  // dim is a multiple of 4 on this path
            const float4 x = j < dim ? *reinterpret_cast<const float4 *>(q_row + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            sq.q[i][4 * w + 0] = x.x; sq.q[i][4 * w + 1] = x.y; sq.q[i][4 * w + 2] = x.z; sq.q[i][4 * w + 3] = x.w;
            s += (x.x + x.y) + (x.z + x.w);
            a += (__builtin_fabsf(x.x) + __builtin_fabsf(x.y)) + (__builtin_fabsf(x.z) + __builtin_fabsf(x.w));
            n = __builtin_fmaf(x.x, x.x, n); n = __builtin_fmaf(x.y, x.y, n);
            n = __builtin_fmaf(x.z, x.z, n); n = __builtin_fmaf(x.w, x.w, n);
        }
    }
#pragma unroll
    for (int h = SLPR / 2; h >= 1; h >>= 1) {  // every lane of the group ends with the totals
        s += __shfl_xor(s, h);
        a += __shfl_xor(a, h);
        n += __shfl_xor(n, h);
    }
    const float u = (float)(dim + 16) * 5.9604645e-8f;  // (dim + 16) * 2^-24
    sq.sum128 = 128.0f * s;
    sq.norm2 = __builtin_sqrtf(n);
    sq.roundc = u * 383.0f * a;  // terms |q_j| * u_j <= 255 |q_j| of the one sum, 128 |q_j| of the other
    sq.exactc = u * sq.norm2;    // terms |q_j v_j| sum to at most ||q||_2 ||v||_2
}

// One wavefront: lane j holds candidate id `my_id` (valid when `ok`); the bounds of its distance to
// the query go to out_lo[j] and out_hi[j].  SLPR lanes share a sketch row (64 / SLPR rows per load
// instruction), a lane holds SCPL of its 16-byte chunks, SU loads of a group are in flight at a time.
template <int SCPL, int SLPR, int SU>
__device__ __forceinline__ void wave_sketch(const SketchQuery<SCPL> &sq, const uint8_t *__restrict__ table,
                                            int64_t row_bytes, int data_chunks, int32_t my_id, bool ok,
                                            float *__restrict__ out_lo, float *__restrict__ out_hi) {
    constexpr int G = kWave / SLPR;
    const int lane = threadIdx.x & (kWave - 1);
    const int grp = lane / SLPR;
    const int lig = lane % SLPR;
    uint64_t mask = __ballot(ok);
    while (mask) {
        int mysrc[SU];
        uint4 r[SU][SCPL];
        float4 tail[SU];
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            int s = -1;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                int pick = -1;
                if (mask) {
                    pick = __builtin_ctzll(mask);
                    mask &= mask - 1;
                }
                s = (grp == g) ? pick : s;
            }
            mysrc[u] = s;
            const int32_t id = __shfl(my_id, s >= 0 ? s : 0);
            const uint4 *row = reinterpret_cast<const uint4 *>(table + (int64_t)id * row_bytes);
#pragma unroll
            for (int i = 0; i < SCPL; ++i) {
                const int c = lig + SLPR * i;
                if (s >= 0 && c < data_chunks) r[u][i] = row[c];
                else r[u][i] = make_uint4(0u, 0u, 0u, 0u);  // meets zeros of the query
            }
            if (s >= 0 && lig == 0) tail[u] = *reinterpret_cast<const float4 *>(row + data_chunks);
            else tail[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < SU; ++u) {
            float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
            for (int i = 0; i < SCPL; ++i) {
                const unsigned w[4] = {r[u][i].x, r[u][i].y, r[u][i].z, r[u][i].w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    a0 = __builtin_fmaf(byte_as_float<0>(w[k]), sq.q[i][4 * k + 0], a0);
                    a1 = __builtin_fmaf(byte_as_float<1>(w[k]), sq.q[i][4 * k + 1], a1);
                    a2 = __builtin_fmaf(byte_as_float<2>(w[k]), sq.q[i][4 * k + 2], a2);
                    a3 = __builtin_fmaf(byte_as_float<3>(w[k]), sq.q[i][4 * k + 3], a3);
                }
            }
            float acc = fold_lanes<SLPR>((a0 + a1) + (a2 + a3));
            if (lig == 0 && mysrc[u] >= 0) {
                const float scale = tail[u].x, resid = tail[u].y, norm = tail[u].z;
                const float s_hat = scale * (acc - sq.sum128);
                const float eps = (sq.norm2 * resid + scale * sq.roundc + sq.exactc * norm) * 1.0001f + 2e-7f;
                out_lo[mysrc[u]] = clamp_distance(s_hat + eps);
                out_hi[mysrc[u]] = clamp_distance(s_hat - eps);
            }
        }
    }
}
